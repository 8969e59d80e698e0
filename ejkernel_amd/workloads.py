"""Seeded synthetic batches for ragged paged attention.

The layout conventions are those of the reference's own input builder,
``benchmarks/benchmark_ragged_page_attn.py:40-129`` / ``test/test_ragged_page_attn.py:27-115``:
K and V pages are drawn separately and interleaved on the head axis
(``stack([k, v], axis=3).reshape(P, page, 2 * Hkv, D)``), ``context_lens`` counts the
current query tokens, ``num_seqs`` is an int32 array of shape ``[1]``.

Unlike the reference's builder the block tables are a random permutation of the page
pool (physically scattered pages), and ``queries`` carries ``>= 8`` zero slack rows after
the last sequence so that an implementation working in 8-row blocks never has to clamp a
block against the end of the array.

The five named workloads are the benchmark configurations of this repository.  Small
integers are drawn on the host with ``numpy.random.Generator(PCG64(seed))``; bulk data is
drawn on the target device in chunks with a seeded ``torch.Generator``.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch


@dataclass
class Batch:
    queries: torch.Tensor
    kv_pages: torch.Tensor
    context_lens: torch.Tensor
    block_tables: torch.Tensor
    query_start_loc: torch.Tensor
    num_seqs: torch.Tensor
    softmax_scale: float
    sliding_window: int | None = None
    logits_soft_cap: float | None = None
    q_lens: np.ndarray | None = None
    kv_lens: np.ndarray | None = None
    name: str = ""
    meta: dict = field(default_factory=dict)

    @property
    def total_valid_tokens(self) -> int:
        return int(self.q_lens.sum())

    def args(self):
        return (self.queries, self.kv_pages, self.context_lens, self.block_tables, self.query_start_loc,
                self.num_seqs)

    def kwargs(self):
        return dict(softmax_scale=self.softmax_scale, sliding_window=self.sliding_window,
                    logits_soft_cap=self.logits_soft_cap)


@dataclass
class V3Batch:
    """Arguments of ``ragged_page_attention_v3`` built over a :class:`Batch` (same lengths, pages and queries)."""

    queries: torch.Tensor
    keys: torch.Tensor
    values: torch.Tensor
    kv_cache: torch.Tensor
    kv_lens: torch.Tensor
    block_tables: torch.Tensor
    query_start_loc: torch.Tensor
    distribution: torch.Tensor
    base: Batch

    def args(self):
        return (self.queries, self.keys, self.values, self.kv_cache, self.kv_lens, self.block_tables,
                self.query_start_loc, self.distribution)

    def kwargs(self):
        return dict(softmax_scale=self.base.softmax_scale, sliding_window=self.base.sliding_window,
                    logits_soft_cap=self.base.logits_soft_cap)


def to_v3(batch: Batch, seed: int = 0, cache_dtype: torch.dtype | None = None) -> V3Batch:
    """New K/V rows for every query token; the cache shares ``batch.kv_pages``' memory, viewed in five dimensions.

    The positions the new tokens will occupy hold random data beforehand, so a missed write shows in the output.
    A head_dim that is no multiple of 128, or a combined-head count that is no multiple of the packing, gets a cache of
    its own with rows / heads padded to one (random data in the padding).
    With ``cache_dtype`` (an 8-bit float type) the cache is a copy of ``batch.kv_pages`` cast to it, and so are the new rows.
    """
    dev = batch.queries.device
    dtype = batch.queries.dtype
    t_alloc, _, head_dim = batch.queries.shape
    num_pages, page_size, hx2, _ = batch.kv_pages.shape
    cdt = cache_dtype or dtype
    pack = 32 // torch.finfo(cdt).bits
    gen = torch.Generator(device=dev)
    gen.manual_seed(int(seed) + 7919)
    keys = _randn_chunked((t_alloc, hx2 // 2, head_dim), gen, dev, dtype).to(cdt)
    values = _randn_chunked((t_alloc, hx2 // 2, head_dim), gen, dev, dtype).to(cdt)
    S = int(batch.num_seqs.reshape(-1)[0])
    pages = batch.kv_pages if cdt == dtype else batch.kv_pages.to(cdt)
    dalign = -(-head_dim // 128) * 128
    hx2_pad = -(-hx2 // pack) * pack
    if dalign != head_dim or hx2_pad != hx2:  # rows and combined heads padded as merge_kv pads them; the padding
        padded = _randn_chunked((num_pages, page_size, hx2_pad, dalign), gen, dev, dtype).to(cdt)  # holds random data
        padded[:, :, :hx2, :head_dim] = pages
        pages = padded
    return V3Batch(
        queries=batch.queries, keys=keys, values=values,
        kv_cache=pages.view(num_pages, page_size, hx2_pad // pack, pack, dalign),
        kv_lens=batch.context_lens, block_tables=batch.block_tables.reshape(-1).contiguous(),
        query_start_loc=batch.query_start_loc,
        distribution=torch.tensor([0, 0, S], dtype=torch.int32, device=dev), base=batch)


@dataclass
class PageAttnBatch:
    """Arguments of ``page_attention``: one query token per sequence over separate paged K and V caches."""

    query: torch.Tensor
    key_cache: torch.Tensor
    value_cache: torch.Tensor
    context_lens: torch.Tensor
    block_tables: torch.Tensor
    attn_scale: float
    kv_lens: np.ndarray | None = None
    name: str = ""
    meta: dict = field(default_factory=dict)

    def args(self):
        return (self.query, self.key_cache, self.value_cache, self.context_lens, self.block_tables)


def make_page_attention_batch(kv_lens, *, num_q_heads, num_kv_heads, head_dim, block_size, max_blocks, num_blocks=None,
                              seed=0, device="cpu", dtype=torch.bfloat16, name="") -> PageAttnBatch:
    """Random caches of [num_blocks, num_kv_heads, block_size, head_dim]; blocks of different sequences are distinct."""
    kv_lens = np.asarray(kv_lens, dtype=np.int64)
    S = len(kv_lens)
    assert kv_lens.max(initial=0) <= max_blocks * block_size
    num_blocks = num_blocks or S * max_blocks
    assert num_blocks >= S * max_blocks
    rng = np.random.Generator(np.random.PCG64(seed))
    bt = rng.permutation(num_blocks)[: S * max_blocks].reshape(S, max_blocks).astype(np.int32)
    dev = torch.device(device)
    gen = torch.Generator(device=dev)
    gen.manual_seed(int(seed))
    shape = (num_blocks, num_kv_heads, block_size, head_dim)
    return PageAttnBatch(
        query=_randn_chunked((S, num_q_heads, head_dim), gen, dev, dtype),
        key_cache=_randn_chunked(shape, gen, dev, dtype), value_cache=_randn_chunked(shape, gen, dev, dtype),
        context_lens=torch.from_numpy(kv_lens.astype(np.int32)).to(dev), block_tables=torch.from_numpy(bt).to(dev),
        attn_scale=float(head_dim**-0.5), kv_lens=kv_lens, name=name,
        meta=dict(num_q_heads=num_q_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, page_size=block_size,
                  pages_per_seq=max_blocks, num_pages=num_blocks, max_num_seqs=S, seed=seed))


def page_attention_workload(name: str, *, device="cpu", scale: float = 1.0, dtype=torch.bfloat16) -> PageAttnBatch:
    """The decode workloads (one token per sequence) with the cache layout of ``page_attention``."""
    seed = 1003
    rng = np.random.Generator(np.random.PCG64(seed))

    def n(x, lo=1):
        return max(lo, int(round(x * scale)))

    if name == "decode_small":
        kv = rng.integers(64, 513, size=8)
        return make_page_attention_batch(kv, num_q_heads=8, num_kv_heads=2, head_dim=128, block_size=16, max_blocks=32,
                                         num_blocks=512, seed=seed, device=device, dtype=dtype, name=name)
    if name == "decode_llama3_8b":
        S = n(256)
        kv = rng.integers(n(512), n(8192) + 1, size=S)
        mb = -(-n(8192) // 16)
        return make_page_attention_batch(kv, num_q_heads=32, num_kv_heads=8, head_dim=128, block_size=16, max_blocks=mb,
                                         num_blocks=max(S * mb, n(160000)), seed=seed, device=device, dtype=dtype,
                                         name=name)
    raise KeyError(name)


def page_attention_subset(batch: PageAttnBatch, seq_ids) -> PageAttnBatch:
    """Sub-batch of ``seq_ids`` with their blocks renumbered densely, on the CPU (for a host-side checker)."""
    seq_ids = list(seq_ids)
    bs = batch.key_cache.shape[2]
    bt = batch.block_tables.cpu().numpy()
    new_bt = np.zeros((len(seq_ids), bt.shape[1]), np.int32)
    phys = []
    for i, s in enumerate(seq_ids):
        nb = -(-int(batch.kv_lens[s]) // bs)
        new_bt[i, :nb] = np.arange(len(phys), len(phys) + nb)
        phys.extend(bt[s, :nb].tolist())
    phys = phys or [0]
    idx = torch.tensor(phys, dtype=torch.long, device=batch.key_cache.device)
    ids = torch.tensor(seq_ids, dtype=torch.long, device=batch.query.device)
    return PageAttnBatch(query=batch.query[ids].cpu(), key_cache=batch.key_cache[idx].cpu(),
                         value_cache=batch.value_cache[idx].cpu(),
                         context_lens=torch.from_numpy(batch.kv_lens[seq_ids].astype(np.int32)),
                         block_tables=torch.from_numpy(new_bt), attn_scale=batch.attn_scale,
                         kv_lens=batch.kv_lens[seq_ids], name=batch.name + "/sub", meta=dict(batch.meta, rows=ids.cpu()))


@dataclass
class RaggedDecodeBatch:
    """Arguments of ``ragged_decode_attention``: one query token per sequence, contiguous K and V."""

    query: torch.Tensor
    key: torch.Tensor
    value: torch.Tensor
    sequence_start: torch.Tensor
    sequence_end: torch.Tensor
    softmax_scale: float
    starts: np.ndarray | None = None
    ends: np.ndarray | None = None
    name: str = ""
    meta: dict = field(default_factory=dict)

    def args(self):
        return (self.query, self.key, self.value, self.sequence_start, self.sequence_end)


def make_ragged_decode_batch(starts, ends, *, seq_len, num_q_heads, num_kv_heads, head_dim, seed=0, device="cpu",
                             dtype=torch.bfloat16, name="") -> RaggedDecodeBatch:
    starts = np.asarray(starts, dtype=np.int64)
    ends = np.asarray(ends, dtype=np.int64)
    B = len(ends)
    assert ends.max(initial=0) <= seq_len
    dev = torch.device(device)
    gen = torch.Generator(device=dev)
    gen.manual_seed(int(seed))
    shape = (B, seq_len, num_kv_heads, head_dim)
    return RaggedDecodeBatch(
        query=_randn_chunked((B, num_q_heads, head_dim), gen, dev, dtype), key=_randn_chunked(shape, gen, dev, dtype),
        value=_randn_chunked(shape, gen, dev, dtype),
        sequence_start=torch.from_numpy(starts.astype(np.int32)).to(dev),
        sequence_end=torch.from_numpy(ends.astype(np.int32)).to(dev), softmax_scale=float(head_dim**-0.5),
        starts=starts, ends=ends, name=name,
        meta=dict(num_q_heads=num_q_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, seq_len=seq_len, seed=seed))


def ragged_decode_workload(name: str, *, device="cpu", scale: float = 1.0, dtype=torch.bfloat16) -> RaggedDecodeBatch:
    """The decode lengths of the named workloads in the contiguous layout (every sequence owns ``seq_len`` slots)."""
    seed = 1003
    rng = np.random.Generator(np.random.PCG64(seed))

    def n(x, lo=1):
        return max(lo, int(round(x * scale)))

    if name == "decode_small":
        ends = rng.integers(64, 513, size=8)
        return make_ragged_decode_batch(np.zeros(8, int), ends, seq_len=512, num_q_heads=8, num_kv_heads=2,
                                        head_dim=128, seed=seed, device=device, dtype=dtype, name=name)
    if name == "decode_llama3_8b":
        S = n(256)
        ends = rng.integers(n(512), n(8192) + 1, size=S)
        return make_ragged_decode_batch(np.zeros(S, int), ends, seq_len=n(8192), num_q_heads=32, num_kv_heads=8,
                                        head_dim=128, seed=seed, device=device, dtype=dtype, name=name)
    raise KeyError(name)


def _randn_chunked(shape, gen, device, dtype, chunk_elems=1 << 27):
    """N(0,1) in `dtype`, drawn in fp32 chunks so a large pool never needs 2x its size."""
    out = torch.empty(shape, dtype=dtype, device=device)
    flat = out.view(-1)
    n = flat.numel()
    for i in range(0, n, chunk_elems):
        m = min(chunk_elems, n - i)
        flat[i:i + m] = torch.randn(m, generator=gen, device=device, dtype=torch.float32).to(dtype)
    return out


def make_batch(q_lens, kv_lens, *, num_q_heads, num_kv_heads, head_dim, page_size, pages_per_seq, num_pages=None,
               seed=0, device="cpu", dtype=torch.bfloat16, max_num_seqs=None, sliding_window=None,
               logits_soft_cap=None, softmax_scale=None, slack_rows=8, permute_pages=True, name="",
               total_tokens=None, pool_seqs=None) -> Batch:
    """Build one ragged batch. ``q_lens[i] <= kv_lens[i]``; pages of different sequences are distinct.

    ``max_num_seqs`` and ``total_tokens`` pad the static shapes the way a serving caller does (block table, lengths and
    query rows allocated for the largest batch, ``num_seqs`` saying how many sequences are present).  ``pool_seqs``
    sizes the page pool and the permutation for that many block-table rows (default ``max_num_seqs``); rows past it
    point at page 0 and belong to no sequence, so a padded batch can share the pool, the pages and the queries of the
    unpadded one with the same seed."""
    q_lens = np.asarray(q_lens, dtype=np.int64)
    kv_lens = np.asarray(kv_lens, dtype=np.int64)
    S = len(q_lens)
    max_num_seqs = max_num_seqs or S
    assert max_num_seqs >= S and len(kv_lens) == S
    assert (q_lens <= kv_lens).all(), "q_len must not exceed kv_len"
    assert kv_lens.max(initial=0) <= pages_per_seq * page_size, "pages_per_seq too small for kv_lens"
    pool_seqs = pool_seqs or max_num_seqs
    assert S <= pool_seqs <= max_num_seqs
    num_pages = num_pages or pool_seqs * pages_per_seq
    assert num_pages >= pool_seqs * pages_per_seq
    rng = np.random.Generator(np.random.PCG64(seed))
    perm = rng.permutation(num_pages) if permute_pages else np.arange(num_pages)
    block_tables = np.zeros((max_num_seqs, pages_per_seq), np.int32)
    block_tables[:pool_seqs] = perm[: pool_seqs * pages_per_seq].reshape(pool_seqs, pages_per_seq)

    total = int(q_lens.sum())
    t_alloc = ((total + 7) // 8) * 8 + slack_rows if slack_rows else total
    if total_tokens is not None:
        assert total_tokens >= t_alloc, "total_tokens must cover the query rows and their slack"
        t_alloc = int(total_tokens)
    cu = np.zeros(max_num_seqs + 1, dtype=np.int32)
    cu[1:S + 1] = np.cumsum(q_lens)
    cu[S + 1:] = total
    ctx = np.zeros(max_num_seqs, dtype=np.int32)
    ctx[:S] = kv_lens

    dev = torch.device(device)
    gen = torch.Generator(device=dev)
    gen.manual_seed(int(seed))
    queries = torch.zeros((t_alloc, num_q_heads, head_dim), dtype=dtype, device=dev)
    if total:
        queries[:total] = _randn_chunked((total, num_q_heads, head_dim), gen, dev, dtype)
    # k_pages / v_pages drawn separately, then interleaved on the head axis
    kv_pages = torch.empty((num_pages, page_size, 2 * num_kv_heads, head_dim), dtype=dtype, device=dev)
    kv5 = kv_pages.view(num_pages, page_size, num_kv_heads, 2, head_dim)
    pages_per_chunk = max(1, (1 << 26) // (page_size * num_kv_heads * head_dim))
    for which in (0, 1):
        for p0 in range(0, num_pages, pages_per_chunk):
            p1 = min(num_pages, p0 + pages_per_chunk)
            kv5[p0:p1, :, :, which, :] = torch.randn((p1 - p0, page_size, num_kv_heads, head_dim), generator=gen,
                                                      device=dev, dtype=torch.float32).to(dtype)
    return Batch(
        queries=queries,
        kv_pages=kv_pages,
        context_lens=torch.from_numpy(ctx).to(dev),
        block_tables=torch.from_numpy(block_tables).to(dev),
        query_start_loc=torch.from_numpy(cu).to(dev),
        num_seqs=torch.tensor([S], dtype=torch.int32, device=dev),
        softmax_scale=float(head_dim**-0.5 if softmax_scale is None else softmax_scale),
        sliding_window=sliding_window,
        logits_soft_cap=logits_soft_cap,
        q_lens=q_lens,
        kv_lens=kv_lens,
        name=name,
        meta=dict(num_q_heads=num_q_heads, num_kv_heads=num_kv_heads, head_dim=head_dim, page_size=page_size,
                  pages_per_seq=pages_per_seq, num_pages=num_pages, max_num_seqs=max_num_seqs, seed=seed),
    )


# name -> description of the five benchmark configurations
WORKLOADS = {
    "decode_small": "8 seqs x 1 token, kv 64..512, 8q/2kv heads, D=128, page 16, 512 pages",
    "decode_llama3_8b": "256 seqs x 1 token, kv 512..8192, 32q/8kv heads, D=128, page 16, 160k pages",
    "mixed_prefill_decode": "16 prefill chunks x 512 tokens (prior 0..4096) + 240 decode seqs (kv 256..8192), "
                            "32q/8kv heads, D=128, page 32",
    "gemma2_local": "64 seqs x 4 tokens, kv 2048..32768, 16q/8kv heads, D=256, page 16, window 4096, cap 50",
    "decode_long_context": "32 seqs x 1 token, kv 32768..131072, 64q/8kv heads, D=128, page 64, 2^18 pages",
    # the two halves of mixed_prefill_decode on their own (same lengths), to price each against its own roofline
    "mixed_prefill_only": "the 16 prefill chunks of mixed_prefill_decode: 512 tokens each, prior 0..4096",
    "mixed_decode_only": "the 240 decode sequences of mixed_prefill_decode: 1 token each, kv 256..8192",
    # long prompts: every prefill tile walks thousands of keys (the per-tile costs of the 512-token chunks vanish)
    "prefill_long": "2 prompts x 8192 tokens from scratch, 32q/8kv heads, D=128, page 32",
    # head_dim 64 with many query heads per kv head (the attention shape of gpt-oss), chunked prefill
    "prefill_head_dim_64": "32 chunks x 512 tokens after 2048, 64q/8kv heads, D=64, page 32",
    # the decode batch of decode_llama3_8b with half the head_dim: K / V rows of 128 bytes
    "decode_head_dim_64": "256 seqs x 1 token, kv 512..8192, 32q/8kv heads, D=64, page 16",
    # chunked prefill at the attention shape of gemma2_local's global layers (head_dim 256, soft cap, no window): the
    # plain prefill tile's head_dim-256 instantiation
    "prefill_head_dim_256": "16 chunks x 1024 tokens (prior 0..8192), 16q/8kv heads, D=256, page 16, cap 50",
    # a head_dim between the instantiated widths (rows of 192 bytes on the 128-wide kernel): the decode batch of
    # decode_llama3_8b and a mixed batch, 16 chunks x 256 tokens beside 112 decode sequences
    "decode_head_dim_96": "256 seqs x 1 token, kv 512..8192, 32q/8kv heads, D=96, page 16",
    "mixed_head_dim_96": "16 chunks x 256 tokens (prior 0..2048) + 112 decode seqs (kv 256..4096), 32q/8kv heads, D=96, page 32",
    # one request's chunked prefill, alone and beside a few decode steps: few tiles, each with a long key range
    "prefill_chunk_after_8k": "1 chunk x 512 tokens after 8192, 32q/8kv heads, D=128, page 16",
    "chunk_beside_decodes": "1 chunk x 512 tokens after 8192 + 64 decode seqs (kv 256..4096), 32q/8kv heads, D=128, page 16",
    # one long prompt: 512 prefill tiles of 256 rows that walk up to 16384 keys each (per-tile costs vanish)
    "prefill_single_16k": "1 prompt x 16384 tokens from scratch, 32q/8kv heads, D=128, page 32",
    # the static shapes of a serving caller: the same sequences, pages and queries as the unpadded workloads inside
    # arrays allocated for the largest batch (max_num_seqs 512, query rows rounded up), num_seqs as is
    "decode_llama3_8b_padded": "decode_llama3_8b inside max_num_seqs 512 and 8192 query rows",
    "mixed_prefill_decode_padded": "mixed_prefill_decode inside max_num_seqs 512 and 16384 query rows",
    "mixed_prefill_only_padded": "mixed_prefill_only inside max_num_seqs 512 and 16384 query rows",
}

# The reference's own benchmark grid (benchmarks/benchmark_ragged_page_attn.py:148-185): max_num_seqs x page_size at
# 16 pages per sequence, 16 query / 4 kv heads, head_dim 128; "ref_bench_<max_num_seqs>_<page_size>".
REF_BENCH_GRID = [(s, p) for s in (8, 16, 32) for p in (8, 16, 32, 64, 128)]
for _s, _p in REF_BENCH_GRID:
    WORKLOADS[f"ref_bench_{_s}_{_p}"] = (f"the reference benchmark's shape: {_s} seqs, kv 1..{16 * _p}, q 1..kv, 16q/4kv heads, "
                                         f"D=128, page {_p}, 16 pages per sequence, identity block table")


def make_workload(name: str, *, device="cpu", scale: float = 1.0, dtype=torch.bfloat16) -> Batch:
    """Build a named workload. ``scale`` < 1 shrinks sequence counts and lengths for tests."""
    only = None
    padded = None
    if name.endswith("_padded"):  # the unpadded workload's draw inside larger static shapes
        name = name[: -len("_padded")]
        padded = dict(max_num_seqs=512, total_tokens=8192 if name == "decode_llama3_8b" else 16384)
        if scale != 1.0:
            padded = dict(max_num_seqs=max(8, int(512 * scale)), total_tokens=max(64, int(padded["total_tokens"] * scale)))
    if name.startswith("ref_bench_"):
        return _ref_bench_workload(name, device=device, dtype=dtype)
    if name in ("mixed_prefill_only", "mixed_decode_only"):
        only, name = name, "mixed_prefill_decode"
    idx = list(WORKLOADS).index(name) + 1
    seed = 1000 + idx
    rng = np.random.Generator(np.random.PCG64(seed))

    def n(x, lo=1):
        return max(lo, int(round(x * scale)))

    def pages(tokens, page):
        # at 64 pages and above keep a multiple of 64 (block-table windows of 64 entries then never clamp)
        k = -(-tokens // page)
        return k if k < 64 else -(-k // 64) * 64

    if name == "decode_small":
        S = 8
        kv = rng.integers(64, 513, size=S)
        return make_batch(np.ones(S, int), kv, num_q_heads=8, num_kv_heads=2, head_dim=128, page_size=16,
                          pages_per_seq=32, num_pages=512, seed=seed, device=device, dtype=dtype, name=name)
    if name == "decode_llama3_8b":
        S = n(256)
        kv = rng.integers(n(512), n(8192) + 1, size=S)
        pps = pages(n(8192), 16)
        pool = max(S * pps, n(160000))
        pad = {} if padded is None else dict(pool_seqs=S, max_num_seqs=max(S, padded["max_num_seqs"]),
                                             total_tokens=max(S + 16, padded["total_tokens"]))
        return make_batch(np.ones(S, int), kv, num_q_heads=32, num_kv_heads=8, head_dim=128, page_size=16,
                          pages_per_seq=pps, num_pages=pool, seed=seed, device=device, dtype=dtype,
                          name=name + ("_padded" if padded else ""), **pad)
    if name == "mixed_prefill_decode":
        n_pre, n_dec = n(16), n(240)
        chunk = n(512)
        prior = rng.integers(0, n(4096) + 1, size=n_pre)
        kv_dec = rng.integers(n(256), n(8192) + 1, size=n_dec)
        q = np.concatenate([np.full(n_pre, chunk), np.ones(n_dec, int)])
        kv = np.concatenate([prior + chunk, kv_dec])
        order = rng.permutation(n_pre + n_dec)
        if only is not None:
            order = np.array([o for o in order if (o < n_pre) == (only == "mixed_prefill_only")])
        pps = pages(max(n(8192), n(4096) + chunk), 32)
        S = len(order)
        pad = {} if padded is None else dict(pool_seqs=S, max_num_seqs=max(S, padded["max_num_seqs"]),
                                             total_tokens=max(int(q[order].sum()) + 16, padded["total_tokens"]))
        return make_batch(q[order], kv[order], num_q_heads=32, num_kv_heads=8, head_dim=128, page_size=32,
                          pages_per_seq=pps, seed=seed, device=device, dtype=dtype,
                          name=(only or name) + ("_padded" if padded else ""), **pad)
    if name in ("prefill_chunk_after_8k", "chunk_beside_decodes"):
        chunk, prior = n(512), n(8192)
        n_dec = n(64) if name == "chunk_beside_decodes" else 0
        q = np.concatenate([[chunk], np.ones(n_dec, np.int64)])
        kv = np.concatenate([[prior + chunk], rng.integers(n(256), n(4096) + 1, size=n_dec)])
        return make_batch(q, kv, num_q_heads=32, num_kv_heads=8, head_dim=128, page_size=16,
                          pages_per_seq=pages(prior + chunk, 16), seed=seed, device=device, dtype=dtype, name=name)
    if name == "prefill_long":
        L = n(8192)
        return make_batch(np.full(2, L), np.full(2, L), num_q_heads=32, num_kv_heads=8, head_dim=128, page_size=32,
                          pages_per_seq=pages(L, 32), seed=seed, device=device, dtype=dtype, name=name)
    if name == "prefill_single_16k":
        L = n(16384)
        return make_batch(np.full(1, L), np.full(1, L), num_q_heads=32, num_kv_heads=8, head_dim=128, page_size=32,
                          pages_per_seq=pages(L, 32), seed=seed, device=device, dtype=dtype, name=name)
    if name == "prefill_head_dim_64":
        S, chunk, prior = n(32), n(512), n(2048)
        return make_batch(np.full(S, chunk), np.full(S, prior + chunk), num_q_heads=64, num_kv_heads=8, head_dim=64,
                          page_size=32, pages_per_seq=pages(prior + chunk, 32), seed=seed, device=device, dtype=dtype,
                          name=name)
    if name == "decode_head_dim_64":
        S = n(256)
        kv = rng.integers(n(512), n(8192) + 1, size=S)
        return make_batch(np.ones(S, int), kv, num_q_heads=32, num_kv_heads=8, head_dim=64, page_size=16,
                          pages_per_seq=pages(n(8192), 16), seed=seed, device=device, dtype=dtype, name=name)
    if name == "prefill_head_dim_256":
        S, chunk = n(16), n(1024)
        prior = rng.integers(0, n(8192) + 1, size=S)
        return make_batch(np.full(S, chunk), prior + chunk, num_q_heads=16, num_kv_heads=8, head_dim=256, page_size=16,
                          pages_per_seq=pages(n(8192) + chunk, 16), seed=seed, device=device, dtype=dtype, name=name,
                          logits_soft_cap=50.0)
    if name == "decode_head_dim_96":
        S = n(256)
        kv = rng.integers(n(512), n(8192) + 1, size=S)
        return make_batch(np.ones(S, int), kv, num_q_heads=32, num_kv_heads=8, head_dim=96, page_size=16,
                          pages_per_seq=pages(n(8192), 16), seed=seed, device=device, dtype=dtype, name=name)
    if name == "mixed_head_dim_96":
        n_pre, n_dec, chunk = n(16), n(112), n(256)
        prior = rng.integers(0, n(2048) + 1, size=n_pre)
        kv_dec = rng.integers(n(256), n(4096) + 1, size=n_dec)
        q = np.concatenate([np.full(n_pre, chunk), np.ones(n_dec, int)])
        kv = np.concatenate([prior + chunk, kv_dec])
        order = rng.permutation(n_pre + n_dec)
        return make_batch(q[order], kv[order], num_q_heads=32, num_kv_heads=8, head_dim=96, page_size=32,
                          pages_per_seq=pages(max(n(4096), n(2048) + chunk), 32), seed=seed, device=device, dtype=dtype, name=name)
    if name == "gemma2_local":
        S = n(64)
        kv = rng.integers(n(2048), n(32768) + 1, size=S)
        pps = pages(n(32768), 16)
        return make_batch(np.full(S, 4), kv, num_q_heads=16, num_kv_heads=8, head_dim=256, page_size=16,
                          pages_per_seq=pps, seed=seed, device=device, dtype=dtype, name=name,
                          sliding_window=n(4096), logits_soft_cap=50.0)
    if name == "decode_long_context":
        S = n(32)
        kv = rng.integers(n(32768), n(131072) + 1, size=S)
        pps = pages(n(131072), 64)
        pool = max(S * pps, n(1 << 18))
        return make_batch(np.ones(S, int), kv, num_q_heads=64, num_kv_heads=8, head_dim=128, page_size=64,
                          pages_per_seq=pps, num_pages=pool, seed=seed, device=device, dtype=dtype, name=name)
    raise KeyError(name)


def _ref_bench_workload(name: str, *, device="cpu", dtype=torch.bfloat16) -> Batch:
    """One shape of the reference's benchmark grid, drawn the way its input generator draws
    (benchmarks/benchmark_ragged_page_attn.py:40-129): ``num_seqs = max_num_seqs``, ``kv_len ~ U[1, pages_per_seq *
    page_size]``, ``q_len ~ U[1, kv_len]``, identity block table, 16 query / 4 kv heads, head_dim 128, 16 pages per
    sequence, N(0,1) data.  Different here: NumPy's generator instead of jax.random, and the query array carries the
    slack rows that keep the reference program's 8-row query blocks inside the array (its generator allocates exactly
    ``sum(q_len)`` rows, where the program's clamped block windows overwrite rows of earlier sequences)."""
    _, _, s, page = name.split("_")
    S, page = int(s), int(page)
    if (S, page) not in REF_BENCH_GRID:
        raise KeyError(name)
    seed = 3000 + S * 1000 + page
    rng = np.random.Generator(np.random.PCG64(seed))
    kv = rng.integers(1, 16 * page + 1, size=S)
    q = np.array([rng.integers(1, int(k) + 1) for k in kv])
    return make_batch(q, kv, num_q_heads=16, num_kv_heads=4, head_dim=128, page_size=page, pages_per_seq=16, seed=seed,
                      device=device, dtype=dtype, permute_pages=False, name=name)


def compact_for_host(batch: Batch, seq_ids) -> Batch:
    """Sub-batch holding only ``seq_ids`` with their pages renumbered densely, on the CPU.

    Attention of a sequence depends only on its own pages, so the sub-batch yields the
    same rows; it lets a host-side checker handle batches whose pool exceeds host RAM.
    """
    seq_ids = list(seq_ids)
    page_size = batch.kv_pages.shape[1]
    pps = batch.block_tables.shape[1]
    bt = batch.block_tables.cpu().numpy()
    cu = batch.query_start_loc.cpu().numpy()
    q_rows, new_bt, phys = [], np.zeros((len(seq_ids), pps), np.int32), []
    for i, s in enumerate(seq_ids):
        n_pg = -(-int(batch.kv_lens[s]) // page_size)
        new_bt[i, :n_pg] = np.arange(len(phys), len(phys) + n_pg)
        phys.extend(bt[s, :n_pg].tolist())
        q_rows.append(torch.arange(int(cu[s]), int(cu[s + 1])))
    rows = torch.cat(q_rows) if q_rows else torch.zeros(0, dtype=torch.long)
    q_lens = batch.q_lens[seq_ids]
    kv_lens = batch.kv_lens[seq_ids]
    total = int(q_lens.sum())
    t_alloc = ((total + 7) // 8) * 8 + 8
    q = torch.zeros((t_alloc,) + tuple(batch.queries.shape[1:]), dtype=batch.queries.dtype)
    q[:total] = batch.queries[rows.to(batch.queries.device)].cpu()
    pages = batch.kv_pages[torch.tensor(phys, dtype=torch.long, device=batch.kv_pages.device)].cpu()
    ncu = np.zeros(len(seq_ids) + 1, np.int32)
    ncu[1:] = np.cumsum(q_lens)
    sub = Batch(queries=q, kv_pages=pages, context_lens=torch.from_numpy(kv_lens.astype(np.int32)),
                block_tables=torch.from_numpy(new_bt), query_start_loc=torch.from_numpy(ncu),
                num_seqs=torch.tensor([len(seq_ids)], dtype=torch.int32), softmax_scale=batch.softmax_scale,
                sliding_window=batch.sliding_window, logits_soft_cap=batch.logits_soft_cap, q_lens=q_lens,
                kv_lens=kv_lens, name=batch.name + "/sub", meta=dict(batch.meta, rows=rows))
    return sub
