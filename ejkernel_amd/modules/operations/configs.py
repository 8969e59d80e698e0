"""Configuration dataclasses of the ragged paged attention ops.

Field names, order and defaults are those of
``ejkernel/modules/operations/configs.py:29-34`` (``BaseOperationConfig``) and
``:242-258`` (``RaggedPageAttentionConfig``), so a config object built for the reference
can be passed here unchanged.  With a single HIP implementation behind the op the fields
mean:

``num_queries_per_block``   query rows of a sequence per tile, a hint for the choice of kernel instantiation, which
                            the library otherwise makes from the (possibly padded) static shapes: 1..16 = the
                            wave-level loop alone (decode steps, short chunks); 17..128 = 128-row workgroup tiles
                            for long chunks; above 128 = 256-row software-pipelined tiles where they exist
                            (head_dim 128, no soft cap, pages of 16 tokens or more).  None = library default
                            (wave-level loop up to 20480 (token, query head) rows, pipelined tiles from 128
                            tokens per ``max_num_seqs`` with block tables for 1024 keys or more, otherwise the
                            device picks them from 512 keys per query row on).  Results stay within the same
                            tolerance either way.
``num_kv_pages_per_block``  the least stretch of a sequence, in pages, one streaming wavefront takes before a small
                            batch is spread over more wavefronts (None = 2 tiles of 32 keys, more for long sequences;
                            and a decode batch of at most 512 (sequence, kv head)s of up to 1024 keys runs one
                            workgroup per (sequence, kv head) with the merge in LDS, which a value here switches off)
``num_warps``               accepted, ignored (workgroups have 4 wavefronts)
``num_stages``              accepted, ignored (2 LDS stages in the 128-row tile, 4 in the pipelined one)
``platform`` / ``backend``  accepted and validated, never used for dispatch
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Literal

_PLATFORMS = ("triton", "pallas", "cuda", "xla", "auto")


@dataclass
class BaseOperationConfig:
    """Base configuration for all operations."""

    platform: Literal["triton", "pallas", "cuda", "xla", "auto"] = "auto"
    backend: str = "any"


@dataclass
class RaggedPageAttentionConfig(BaseOperationConfig):
    """Configuration for the ragged paged attention operation."""

    num_kv_pages_per_block: int | None = None
    num_queries_per_block: int | None = None
    num_warps: int = 4
    num_stages: int = 1

    def validate(self) -> None:
        if self.platform not in _PLATFORMS:
            raise ValueError(f"platform={self.platform!r} must be one of {_PLATFORMS}")
        if self.num_kv_pages_per_block is not None and self.num_kv_pages_per_block <= 0:
            raise ValueError(f"num_kv_pages_per_block={self.num_kv_pages_per_block} must be positive.")
        if self.num_queries_per_block is not None and self.num_queries_per_block <= 0:
            raise ValueError(f"num_queries_per_block={self.num_queries_per_block} must be positive.")


@dataclass
class RaggedPageAttentionv3Config(BaseOperationConfig):
    """Configuration for ragged paged attention v3 (ejkernel/modules/operations/configs.py:262-278)."""

    chunk_prefill_size: int | None = None
    num_kv_pages_per_block: int | None = None
    num_queries_per_block: int | None = None
    num_warps: int = 4
    num_stages: int = 1

    def validate(self) -> None:
        if self.platform not in _PLATFORMS:
            raise ValueError(f"platform={self.platform!r} must be one of {_PLATFORMS}")
        for name in ("chunk_prefill_size", "num_kv_pages_per_block", "num_queries_per_block"):
            v = getattr(self, name)
            if v is not None and v <= 0:
                raise ValueError(f"{name}={v} must be positive.")


@dataclass
class PageAttentionConfig(BaseOperationConfig):
    """Configuration for page attention (ejkernel/modules/operations/configs.py:147-162)."""

    num_splits: int = 0
    pages_per_compute_block: int | None = None
    num_warps: int = 4
    num_stages: int = 1

    def validate(self) -> None:
        if self.platform not in _PLATFORMS:
            raise ValueError(f"platform={self.platform!r} must be one of {_PLATFORMS}")


@dataclass
class FwdParams:
    """Forward block sizes a config may carry (ejkernel/ops/utils/datacarrier.py:58-95); accepted, not used here."""

    blocksize_m: int | None = None
    blocksize_k: int | None = None
    blocksize_n: int | None = None
    q_blocksize: int | None = None
    kv_blocksize: int | None = None
    blocksize_heads: int | None = None
    blocksize_keys: int | None = None
    num_key_splits: int | None = None
    num_warps: int | None = None
    num_stages: int | None = None


@dataclass
class RaggedDecodeAttentionConfig(BaseOperationConfig):
    """Configuration for ragged decode attention (ejkernel/modules/operations/configs.py:224-239)."""

    fwd_params: FwdParams | None = None

    def __post_init__(self):
        if isinstance(self.fwd_params, dict):
            self.fwd_params = FwdParams(**self.fwd_params)

    def validate(self) -> None:
        if self.platform not in _PLATFORMS:
            raise ValueError(f"platform={self.platform!r} must be one of {_PLATFORMS}")
