"""Host-side checks that need no GPU: the C-ABI library loads and exports what the header
declares, the Python boundary keeps the reference's signature and config dataclass, and
argument errors are raised the way the reference's validators raise them."""

import ctypes
import dataclasses
import inspect
import re
from pathlib import Path

import numpy as np
import pytest
import torch

from ejkernel_amd import _native
from ejkernel_amd.modules import RaggedPageAttention, RaggedPageAttentionConfig, ragged_page_attention
from ejkernel_amd.workloads import make_batch

ROOT = Path(__file__).resolve().parent.parent


def _declared_functions():
    text = (ROOT / "include" / "rpa_mi355x.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rpa_[a-z0-9_]+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = _native.load()
    declared = _declared_functions()
    assert declared == sorted(_native.EXPORTED_SYMBOLS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.rpa_abi_version() == _native.RPA_ABI_VERSION


def test_struct_layout_matches_header_field_order():
    text = (ROOT / "include" / "rpa_mi355x.h").read_text()
    body = text[text.index("typedef struct RpaParams {"):text.index("} RpaParams;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = re.findall(r"([a-z_]+)\s*;", body)
    assert names == [f[0] for f in _native.RpaParams._fields_]
    assert ctypes.sizeof(_native.RpaParams) % 8 == 0


@pytest.mark.parametrize("name", ["RpaV3Params", "RpaPageAttnParams", "RpaRaggedDecodeParams"])
def test_other_struct_layouts_match_header_field_order(name):
    text = (ROOT / "include" / "rpa_mi355x.h").read_text()
    body = text[text.index(f"typedef struct {name} {{"):text.index(f"}} {name};")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = re.findall(r"([a-z_]+)\s*;", body)
    assert names == [f[0] for f in getattr(_native, name)._fields_]


def test_ragged_decode_sink_arguments_are_checked_before_any_launch():
    lib = _native.load()
    p = _native.RpaRaggedDecodeParams()
    p.batch, p.num_q_heads, p.num_kv_heads, p.head_dim, p.seq_len = 4, 8, 2, 128, 64
    p.softmax_scale, p.window_left = 0.1, -1
    plain = lib.rpa_ragged_decode_workspace_bytes(ctypes.byref(p))
    p.num_sinks, p.aux_rows = 4, 1
    with_sinks = lib.rpa_ragged_decode_workspace_bytes(ctypes.byref(p))
    assert with_sinks >= plain + 4 * 8 * (128 + 2) * 4       # the sink keys' state per (sequence, query head)
    buf = (ctypes.c_char * 192)()
    addr = (ctypes.addressof(buf) + 63) & ~63                 # never dereferenced: every call below fails first
    for f in ("query", "key", "value", "sequence_start", "sequence_end", "out", "workspace"):
        setattr(p, f, addr)
    p.workspace_bytes = with_sinks
    assert lib.rpa_ragged_decode_launch(ctypes.byref(p), None) == -1 and b"softmax_aux is null" in lib.rpa_last_error()
    p.softmax_aux = addr
    p.num_sinks = _native.RPA_MAX_SINK_KEYS + 1
    assert lib.rpa_ragged_decode_launch(ctypes.byref(p), None) == -1 and b"num_sinks" in lib.rpa_last_error()
    p.num_sinks, p.aux_rows = 4, 2                            # 4 query heads per kv head: 1 or 4 rows
    assert lib.rpa_ragged_decode_launch(ctypes.byref(p), None) == -1 and b"aux_rows" in lib.rpa_last_error()
    p.aux_rows, p.workspace_bytes = 4, plain
    assert lib.rpa_ragged_decode_launch(ctypes.byref(p), None) == -3 and b"too small" in lib.rpa_last_error()


def test_python_constants_are_the_header_s():
    """Every RPA_* constant of the ctypes layer has the value the C header defines."""
    import pathlib
    import re
    text = (pathlib.Path(__file__).resolve().parents[1] / "include" / "rpa_mi355x.h").read_text()
    defines = {m.group(1): m.group(2) for m in re.finditer(r"^#define (RPA_[A-Z0-9_]+) \(?(-?\d+)u?\)?", text, re.M)}
    names = [n for n in dir(_native) if n.startswith("RPA_") and isinstance(getattr(_native, n), int)]
    assert len(names) >= 12
    for n in names:
        assert n in defines, f"{n} is not defined in the header"
        assert int(defines[n]) == getattr(_native, n), n


def test_kernel_path_query_names_what_the_mfma_kernels_take():
    """rpa_kernel_path: 1 where the MFMA kernels run, 0 where the scalar kernel does, -1 for dims a launch rejects."""
    lib = _native.load()
    p = _native.RpaParams()
    p.total_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim = 16, 8, 2, 128
    p.page_size, p.num_pages, p.max_num_seqs, p.pages_per_seq = 16, 64, 4, 16
    p.softmax_scale = 0.1
    p.dtype, p.compute = _native.RPA_DTYPE_BF16, _native.RPA_COMPUTE_BF16
    assert lib.rpa_kernel_path(ctypes.byref(p)) == 1
    for field, value in (("head_dim", 48), ("head_dim", 72), ("head_dim", 320), ("page_size", 2), ("page_size", 24),
                         ("flags", _native.RPA_FLAG_FORCE_GENERIC), ("compute", _native.RPA_COMPUTE_F32)):
        keep = getattr(p, field)
        setattr(p, field, value)
        assert lib.rpa_kernel_path(ctypes.byref(p)) == 0, (field, value)
        setattr(p, field, keep)
    for hd in (64, 80, 96, 144, 256):
        p.head_dim = hd
        assert lib.rpa_kernel_path(ctypes.byref(p)) == 1, hd
    p.head_dim, p.num_q_heads = 128, 7   # not a multiple of the kv heads: the launch would reject it
    assert lib.rpa_kernel_path(ctypes.byref(p)) == -1


def test_v3_workspace_counts_the_stored_logits_of_an_8_bit_cache():
    lib = _native.load()
    v = _native.RpaV3Params()
    p = v.attn
    p.total_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim = 16, 8, 2, 128
    p.page_size, p.num_pages, p.max_num_seqs, p.pages_per_seq = 16, 64, 16, 10   # a block-table row holds 160 positions
    p.dtype, p.compute = _native.RPA_DTYPE_BF16, _native.RPA_COMPUTE_BF16
    v.cache_dtype = _native.RPA_DTYPE_FP8_E4M3
    with_logits = lib.rpa_v3_workspace_bytes(ctypes.byref(v))
    p.flags = _native.RPA_FLAG_NO_LOGIT_STASH
    without = lib.rpa_v3_workspace_bytes(ctypes.byref(v))
    assert with_logits - without == 16 * 8 * 192 * 4          # fp32 per (token, query head) and position, pitch 192
    p.flags = 0
    p.total_tokens = 20480 // 8 + 1                            # batches that run on prefill tiles read K twice
    grown = lib.rpa_v3_workspace_bytes(ctypes.byref(v))
    p.flags = _native.RPA_FLAG_NO_LOGIT_STASH
    assert grown == lib.rpa_v3_workspace_bytes(ctypes.byref(v))
    p.flags, p.total_tokens, p.pages_per_seq = 0, 2560, 1 << 16  # 2560 * 8 rows * 2**20 positions * 4 bytes: over the limit
    big = lib.rpa_v3_workspace_bytes(ctypes.byref(v))
    p.flags = _native.RPA_FLAG_NO_LOGIT_STASH
    assert big == lib.rpa_v3_workspace_bytes(ctypes.byref(v))


def test_v3_cache_dtype_arguments_are_checked_before_any_launch():
    lib = _native.load()
    v = _native.RpaV3Params()
    p = v.attn
    p.total_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim = 16, 8, 2, 128
    p.page_size, p.num_pages, p.max_num_seqs, p.pages_per_seq = 16, 64, 4, 16
    p.softmax_scale = 0.1
    p.dtype, p.compute = _native.RPA_DTYPE_BF16, _native.RPA_COMPUTE_BF16
    v.cache_dtype = _native.RPA_DTYPE_BF16
    plain = lib.rpa_v3_workspace_bytes(ctypes.byref(v))
    assert plain == lib.rpa_workspace_bytes(ctypes.byref(p)) > 0
    v.cache_dtype = _native.RPA_DTYPE_FP8_E4M3
    with_stats = lib.rpa_v3_workspace_bytes(ctypes.byref(v))
    assert with_stats >= plain + 16 * 8 * 2 * 4              # row maximum and sum per (token, query head)
    buf = (ctypes.c_char * 192)()
    addr = (ctypes.addressof(buf) + 63) & ~63                 # never dereferenced: every call below fails first
    for f in ("queries", "kv_pages", "context_lens", "block_tables", "query_start_loc", "num_seqs", "out", "workspace"):
        setattr(p, f, addr)
    v.new_keys = v.new_values = addr
    p.workspace_bytes = plain
    assert lib.rpa_v3_launch(ctypes.byref(v), None) == -3 and b"rpa_v3_workspace_bytes" in lib.rpa_last_error()
    p.workspace_bytes = with_stats
    p.flags = _native.RPA_FLAG_FORCE_GENERIC
    assert lib.rpa_v3_launch(ctypes.byref(v), None) == -2 and b"MFMA kernel only" in lib.rpa_last_error()
    p.flags = 0
    p.dtype, p.compute = _native.RPA_DTYPE_F32, _native.RPA_COMPUTE_F32
    assert lib.rpa_v3_launch(ctypes.byref(v), None) == -2 and b"bf16 queries" in lib.rpa_last_error()
    v.cache_dtype = _native.RPA_DTYPE_BF16                    # a float32 call with a bf16 cache: neither rule holds
    assert lib.rpa_v3_launch(ctypes.byref(v), None) == -1 and b"cache_dtype" in lib.rpa_last_error()
    # what the attention step would reject is rejected before the cache update runs: a failed call leaves the cache alone
    p.dtype, p.compute = _native.RPA_DTYPE_BF16, _native.RPA_COMPUTE_BF16
    p.workspace_bytes = plain - 1
    assert lib.rpa_v3_launch(ctypes.byref(v), None) == -3 and b"too small" in lib.rpa_last_error()
    p.workspace_bytes = plain
    p.head_dim = 520                                          # beyond the scalar kernel
    assert lib.rpa_v3_launch(ctypes.byref(v), None) == -2 and b"at most 512" in lib.rpa_last_error()
    p.head_dim = 64
    v.cache_head_dim = 32                                     # shorter than the rows it holds
    assert lib.rpa_v3_launch(ctypes.byref(v), None) == -1 and b"cache_head_dim" in lib.rpa_last_error()
    v.cache_head_dim, v.cache_combined_heads = 128, 2         # fewer than 2 * num_kv_heads = 4
    assert lib.rpa_v3_launch(ctypes.byref(v), None) == -1 and b"cache_combined_heads" in lib.rpa_last_error()


def test_misaligned_pointers_are_rejected_before_any_launch():
    """Rows are fetched in 16-byte pieces wherever a row is a multiple of 16 bytes; rows that are not need the
    element's own alignment (they run on the scalar kernel)."""
    lib = _native.load()
    p = _native.RpaParams()
    p.total_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim = 16, 8, 2, 128
    p.page_size, p.num_pages, p.max_num_seqs, p.pages_per_seq = 16, 64, 4, 16
    p.softmax_scale = 0.1
    p.dtype, p.compute = _native.RPA_DTYPE_BF16, _native.RPA_COMPUTE_BF16
    buf = (ctypes.c_char * 192)()
    addr = (ctypes.addressof(buf) + 63) & ~63                 # never dereferenced: every call below fails first
    fields = ("queries", "kv_pages", "context_lens", "block_tables", "query_start_loc", "num_seqs", "out")
    for bad, off, msg in (("queries", 8, b"16 bytes"), ("kv_pages", 2, b"16 bytes"), ("out", 4, b"16 bytes"),
                          ("block_tables", 2, b"4 bytes"), ("context_lens", 1, b"4 bytes")):
        for f in fields:
            setattr(p, f, addr + (off if f == bad else 0))
        assert lib.rpa_fwd_launch(ctypes.byref(p), None) == -1 and msg in lib.rpa_last_error(), bad
    p.head_dim = 4                                            # rows of 8 bytes: the scalar kernel, element alignment
    for f in fields:
        setattr(p, f, addr)
    p.queries = addr + 8
    p.out = addr + 1
    assert lib.rpa_fwd_launch(ctypes.byref(p), None) == -1 and b"2 bytes" in lib.rpa_last_error()


def test_workspace_bytes_and_errors_without_gpu():
    lib = _native.load()
    p = _native.RpaParams()
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0  # zero dims are invalid
    p.total_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim = 16, 8, 2, 128
    p.page_size, p.num_pages, p.max_num_seqs, p.pages_per_seq = 16, 64, 4, 16
    p.softmax_scale = 0.1
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) >= 256
    assert lib.rpa_fwd_launch(ctypes.byref(p), None) == -1  # null pointers are rejected before any launch
    assert b"null" in lib.rpa_last_error()
    p.num_kv_heads = 3
    assert lib.rpa_workspace_bytes(ctypes.byref(p)) == 0
    assert lib.rpa_fwd_launch(None, None) == -1


def test_signature_matches_reference():
    sig = inspect.signature(ragged_page_attention)
    params = list(sig.parameters.values())
    positional = [p.name for p in params if p.kind is inspect.Parameter.POSITIONAL_ONLY]
    assert positional == ["queries", "kv_pages", "context_lens", "block_tables", "query_start_loc", "num_seqs",
                          "softmax_aux"]
    keyword = [p.name for p in params if p.kind is inspect.Parameter.KEYWORD_ONLY]
    assert keyword == ["softmax_scale", "logits_soft_cap", "compute_dtype", "optimized", "sliding_window",
                       "mask_value", "vmem_limit_bytes", "platform", "cfg", "mesh", "in_specs", "out_specs"]
    assert sig.parameters["softmax_aux"].default is None


def test_config_dataclass_fields_and_defaults():
    fields = [(f.name, f.default) for f in dataclasses.fields(RaggedPageAttentionConfig)]
    assert fields == [("platform", "auto"), ("backend", "any"), ("num_kv_pages_per_block", None),
                      ("num_queries_per_block", None), ("num_warps", 4), ("num_stages", 1)]
    k = RaggedPageAttention()
    assert k.op_id == "ragged_page_attention"
    assert k.heuristic_cfg(None) == RaggedPageAttentionConfig()
    assert k.candidate_cfgs(None) == [RaggedPageAttentionConfig()]


def _b(**kw):
    return make_batch([2, 1], [9, 30], num_q_heads=4, num_kv_heads=2, head_dim=16, page_size=4, pages_per_seq=8,
                      seed=1, **kw)


def test_validation_errors_mirror_reference():
    b = _b()
    a = list(b.args())
    with pytest.raises(ValueError, match="must be positive"):
        ragged_page_attention(*a, sliding_window=0)
    with pytest.raises(ValueError, match="must not be 0.0"):
        ragged_page_attention(*a, logits_soft_cap=0.0)
    with pytest.raises(ValueError, match=r"must be \(1,\)"):
        ragged_page_attention(a[0], a[1], a[2], a[3], a[4], torch.tensor([2, 2], dtype=torch.int32))
    with pytest.raises(ValueError, match="int32"):
        ragged_page_attention(a[0], a[1], a[2].long(), a[3], a[4], a[5])
    with pytest.raises(ValueError, match="context_lens.shape"):
        ragged_page_attention(a[0], a[1], a[2][:1], a[3], a[4], a[5])
    with pytest.raises(ValueError, match="query_start_loc.shape"):
        ragged_page_attention(a[0], a[1], a[2], a[3], a[4][:2], a[5])
    with pytest.raises(ValueError, match="head_dim"):
        ragged_page_attention(a[0][..., :8], a[1], a[2], a[3], a[4], a[5])
    with pytest.raises(ValueError, match="divisible"):
        ragged_page_attention(a[0][:, :3], a[1], a[2], a[3], a[4], a[5])
    with pytest.raises(ValueError, match="num_kv_pages_per_block"):
        ragged_page_attention(*a, cfg=RaggedPageAttentionConfig(num_kv_pages_per_block=9))
    with pytest.raises(ValueError, match="num_queries_per_block"):
        ragged_page_attention(*a, cfg=RaggedPageAttentionConfig(num_queries_per_block=-1))
    with pytest.raises(ValueError, match="platform"):
        ragged_page_attention(*a, platform="tpu")
    with pytest.raises(NotImplementedError):
        ragged_page_attention(*a, mesh=object(), in_specs=(None,) * 7, out_specs=None)


def test_no_cpu_fallback():
    b = _b()
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ragged_page_attention(*b.args())


def test_generated_instruction_stream_is_up_to_date():
    """csrc/rpa_prefill_pipe_asm.inc is what csrc/gen_prefill_pipe_asm.py writes (the key loop of the software-pipelined
    prefill tile is generated; the committed file must not drift from its generator)."""
    import importlib.util
    from pathlib import Path

    csrc = Path(_native.__file__).resolve().parent / "csrc"
    spec = importlib.util.spec_from_file_location("gen_prefill_pipe_asm", csrc / "gen_prefill_pipe_asm.py")
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    assert not gen.PROF, "unset RPA_PPA_PROF for this test"
    assert (csrc / "rpa_prefill_pipe_asm.inc").read_text() == gen.render()


def _regs(tok):
    """Registers an assembler operand names: 'v[4:7]' -> {v4..v7}, 'a12' -> {a12}, anything else -> {}."""
    m = re.fullmatch(r"([vas])\[(\d+):(\d+)\]", tok)
    if m:
        return {f"{m.group(1)}{k}" for k in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.fullmatch(r"([vas])(\d+)", tok)
    return {tok} if m else set()


def test_instruction_stream_writes_only_what_its_constraints_declare():
    """The generated key loop is one asm statement with physical-register operands.  Every register an instruction of
    the stream writes must be an output or a clobber of that statement, none may be an input (the compiler assumes
    inputs survive), and no register is both output and clobber.  m0 is saved and restored by the stream itself."""
    csrc = Path(_native.__file__).resolve().parent / "csrc"
    inc = (csrc / "rpa_prefill_pipe_asm.inc").read_text()
    hdr = (csrc / "rpa_prefill_pipe.h").read_text()
    ops = hdr[hdr.index("#define RPA_PPA_OPERANDS"):hdr.index("if constexpr (kRound) asm volatile")]
    outs_txt, ins_txt = ops.split("\n  : ")[1], ops.split("\n  : ")[2]
    outputs = set().union(*[_regs(t) for t in re.findall(r'"=\{([^}]+)\}"', outs_txt)])
    inputs = set().union(*[_regs(t) for t in re.findall(r'"\{([^}]+)\}"', ins_txt)])
    clob_txt = hdr[hdr.index("#define RPA_PPA_CLOBBERS"):hdr.index("// The key loop of one tile for one wavefront.")]
    clobbers = set(re.findall(r'"([vas]\d+)"', clob_txt))
    assert len(outputs) == 128 + 6 and len(inputs) >= 64 + 8
    assert not (outputs & clobbers), sorted(outputs & clobbers)
    assert not (outputs & inputs) and not (inputs & clobbers), sorted(inputs & clobbers)
    no_dest = ("s_waitcnt", "s_barrier", "s_nop", "s_branch", "s_cbranch", "s_cmp", "buffer_load", "s_setprio", "s_sleep")
    written = set()
    for line in re.findall(r'"([^"\\]+)\\n\\t"', inc):
        line = line.strip()
        if not line or line.endswith(":") or line.startswith(no_dest):
            continue
        mnem, _, rest = line.partition(" ")
        toks = [t.strip() for t in rest.split(",")]
        if mnem.startswith("v_cmp"):
            dst = toks[:1] if toks[0] != "vcc" else []   # a scalar pair or vcc
        elif mnem.startswith("v_permlane32_swap") or mnem.startswith("v_permlane16_swap"):
            dst = toks[:2]
        else:
            dst = toks[:1]
        for t in dst:
            written |= _regs(t)
    assert written, "no instruction parsed"
    undeclared = written - outputs - clobbers
    assert not undeclared, f"written but neither output nor clobber: {sorted(undeclared)}"
    assert not (written & inputs), f"inputs written by the stream: {sorted(written & inputs)}"


def test_hbm_traffic_file_is_well_formed():
    """profiles/hbm_traffic.json (read by bench.py for roofline.traffic): bytes = scaled counters, per workload."""
    import json
    from pathlib import Path

    from ejkernel_amd.workloads import WORKLOADS

    data = json.loads((Path(_native.__file__).resolve().parent.parent / "profiles" / "hbm_traffic.json").read_text())
    for name, e in data.items():
        assert name in WORKLOADS
        want = (e["fetch_size_kib"] * e["fetch_scale"] + e["write_size_kib"] * e["write_scale"]) * 1024.0
        assert abs(e["bytes"] - want) <= 1e-6 * want



def test_xla_ffi_handlers_type_check_against_the_api_stand_in():
    """The XLA FFI handlers need jaxlib's headers, which this image lacks, so they are never built here.  They are at
    least type-checked (host pass only, no code generated) against tests/ffi_stub, a stand-in that declares the part
    of the FFI binding API the file uses: every binding must list what its implementation function takes, in order.
    It says nothing about the real header beyond that; the handlers stay unexercised until a host with JAX runs them."""
    import shutil
    import subprocess

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    root = Path(__file__).resolve().parents[1]
    src = root / "ejkernel_amd" / "csrc" / "rpa_xla_ffi.cc"
    r = subprocess.run([hipcc, "-x", "hip", "--cuda-host-only", "-fsyntax-only", "-std=c++17", "-Wno-unused-command-line-argument",
                        "-I", str(root / "tests" / "ffi_stub"), str(src)], capture_output=True, text=True, cwd="/tmp")
    assert r.returncode == 0, r.stderr[-3000:]
    # the same names are what the Python side registers
    text = src.read_text()
    py = (root / "ejkernel_amd" / "jax_ffi.py").read_text()  # not importable without jax
    symbols = re.findall(r'"(Rpa\w+)"', py[py.index("_TARGETS = {"):py.index("_registered")])
    assert len(symbols) == 4
    for symbol in symbols:
        assert f"XLA_FFI_DEFINE_HANDLER_SYMBOL({symbol}," in text, symbol


def test_bench_long_prompt_parity_leg_detects_damage():
    """bench.py checks prompts too long for the restatement on a prefix (against it) and on sampled deep rows (float64):
    the float64 result passes, a damaged prefix row and a damaged sampled row (the last one is always sampled) fail."""
    import bench
    from ejkernel_amd.workloads import make_workload
    from tests.helpers import run_exact

    b = make_workload("prefill_single_16k", device="cpu", scale=0.03)
    L = int(b.q_lens[0])
    out = torch.from_numpy(np.asarray(run_exact(b), np.float32)).to(torch.bfloat16)
    r = bench.long_prompt_parity(b, out, prefix_tokens=100, sampled_tokens=6)
    assert r["ok"] and r["rows_prefix"] == 100 and 1 <= r["rows_deep"] <= 6
    assert r["prefix_elements_over_2e-2"] >= r["prefix_elements_over_bound"] == 0
    out[L - 1] += 0.25
    assert not bench.long_prompt_parity(b, out, prefix_tokens=100, sampled_tokens=6)["ok"]
    out[L - 1] -= 0.25
    out[7] += 0.5
    assert not bench.long_prompt_parity(b, out, prefix_tokens=100, sampled_tokens=6)["ok"]
    out[7] -= 0.5
    # the widened bound only ever applies to values of magnitude 2 or more: an element below 2 that is off by 0.021
    # fails, and the record counts it against the plain bound and names its magnitude and its row's key count
    ref = np.asarray(run_exact(b), np.float32)
    t, h, d = [(t, h, d) for t in range(40, 60) for h in range(2) for d in range(8) if 0.3 < abs(ref[t, h, d]) < 1.0][0]
    out[t, h, d] = float(out[t, h, d]) + 0.0215 * (1 if ref[t, h, d] > 0 else -1)
    r = bench.long_prompt_parity(b, out, prefix_tokens=100, sampled_tokens=6)
    assert not r["ok"] and r["prefix_elements_over_bound"] >= 1 and r["prefix_elements_over_2e-2"] >= 1
    assert r["over_2e-2_min_abs_value"] < 1.0 and r["over_2e-2_max_visible_keys"] >= t + 1


def test_bench_power_sensor_and_gpu_count_guard():
    """bench.py's board power reader returns watts or None (no GPU here: None, or whatever hwmon file exists), never
    raises; more than one GPU is refused with a message, as this build measures one GPU only."""
    import subprocess
    import sys

    import bench

    now, cap = bench.board_power_watts()
    assert (now is None or now >= 0.0) and (cap is None or cap > 0.0)
    assert bench.SETTLE_S > 0
    root = Path(__file__).resolve().parents[1]
    r = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, cwd=str(root))
    assert r.returncode == 2 and "one GPU" in r.stderr


def test_ffi_attributes_named_alike_in_python_and_in_the_handlers():
    """jax.ffi passes attributes by name: every keyword a wrapper in jax_ffi.py hands to its ffi_call must be an
    Attr of the handler registered under that target, with nothing missing on either side, and the operand counts
    must agree (optional trailing operands arrive through RemainingArgs).  Checked on the source text; neither file
    can run here."""
    import ast

    root = Path(__file__).resolve().parents[1]
    cc = (root / "ejkernel_amd" / "csrc" / "rpa_xla_ffi.cc").read_text()
    py_src = (root / "ejkernel_amd" / "jax_ffi.py").read_text()
    handlers = {}
    for m in re.finditer(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\((\w+),\s*\w+,(.*?)\);\n", cc, flags=re.S):
        body = m.group(2)
        handlers[m.group(1)] = (re.findall(r'\.Attr<\w+>\("(\w+)"\)', body), len(re.findall(r"\.Arg<", body)),
                                ".RemainingArgs()" in body, len(re.findall(r"\.Ret<", body)))
    targets = dict(re.findall(r'"(mi355x_\w+)":\s*"(Rpa\w+)"', py_src))
    targets["mi355x_rpa_fwd" if "mi355x_rpa_fwd" in py_src else "_TARGET"] = "RpaFwd"
    tree = ast.parse(py_src)
    wrappers = {"ragged_page_attention": "RpaFwd", "ragged_page_attention_v3": "RpaV3", "page_attention": "RpaPageAttn",
                "ragged_decode_attention": "RpaRaggedDecode"}
    assert set(wrappers.values()) == set(handlers) and set(targets.values()) >= set(handlers)
    for fn in [n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name in wrappers]:
        attrs, n_args, has_rest, n_rets = handlers[wrappers[fn.name]]
        # the call whose callee is the `call` object made by jax.ffi.ffi_call: its keywords are the attributes
        calls = [c for c in ast.walk(fn) if isinstance(c, ast.Call) and isinstance(c.func, ast.Name) and c.func.id == "call"]
        assert len(calls) == 1, fn.name
        kw = [k.arg for k in calls[0].keywords]
        assert sorted(kw) == sorted(attrs), (fn.name, kw, attrs)
        positional = calls[0].args
        if any(isinstance(a, ast.Starred) for a in positional):
            assert has_rest, fn.name          # a variable operand list needs RemainingArgs in the binding
        else:
            assert len(positional) == n_args and not has_rest, (fn.name, len(positional), n_args)
