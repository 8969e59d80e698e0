"""Generates rpa_prefill_pipe_asm.inc: the key loop of the software-pipelined prefill tile as one instruction stream.

The tile of rpa_prefill_pipe.h runs one wavefront per SIMD, so matrix and vector work only overlap when one
instruction stream interleaves them, and that stream keeps about 400 registers in fixed places (output accumulators
and MFMA operands in accumulation registers, logits and probabilities in ordinary ones).  Left to the compiler, the
same loop moved accumulators between the two register files every half and spilled; here it is written out with
fixed registers.  The C++ side binds its variables to the same registers with physical-register constraints, so the
compiler still sees every value that enters or leaves.  `python gen_prefill_pipe_asm.py` rewrites the .inc file; a
CPU test compares the committed file with this script's output.

Register map (one wavefront; i = lane % 32, g = lane / 32; the 64 rows are two groups of 32, "rg"):
  a[0:127]    O^T accumulators (32x32 MFMA tiles), row group rg, block of 32 output elements blk:
              a[16 (4 rg + blk) : +15]; register 4 q + r of a tile holds element 32 blk + 8 q + 4 g + r of row i    (out)
  a[128:159]  K operands of one half, k-step ks (16 elements of head_dim): a[128 + 4 ks : +3]
  a[160:191]  V^T operands of one half, 16-key step s, block blk: a[160 + 4 (4 s + blk) : +3]
  v[0:31]     logits / exp2 arguments, buffer A: row group rg: v[16 rg : +15]; register 4 q + r holds key 8 q + 4 g + r
  v[32:63]    the same, buffer B (halves alternate between the buffers)
  v[64:127]   Q operands, row group rg, k-step ks: v[64 + 4 (8 rg + ks) : +3]                     (in)
  v[128:143]  P^T operands, row group rg, key step s: v[128 + 4 (2 rg + s) : +3]
  v[144:145]  row sums of the lane's keys per row group (the two lanes of a row add up at the end) (out)
  v146        two bf16 ones (operand of the row-sum dot product)
  v[148:149]  -m log2(e) per row group, the offset of the exp2 argument                           (out)
  v[152:153]  maximum exp2 argument of the half per row group
  v[156:157]  masked halves: first visible key of the lane's rows relative to the lane's first key of the half
  v[160:161]  visible keys of the lane's rows minus one (0 with an unreachable first key: none)   (in)
  v168        LDS address of the V^T operand reads (stage of this tile)
  v169        factor of the exp2 argument: log2(e) times the fp32 logit scale                     (in)
  v170, v195:199  temporaries;  v171  -inf;  v[200:215]  fetch: byte offsets of the lane's pieces
  v[172:173]  threshold of the exp2 arguments per row group: -inf before a row's first key        (out)
  v176        the threshold once a row has a reference point
  v[178:179]  first visible key of the lane's rows minus 4 g (absolute)                           (in)
  v186        LDS address of the V^T operand reads in stage 0                                    (in)
  v[187:189]  fetch: the lane's row in a K block, in a V block, byte offset of its V piece        (in)
  v[190:193]  fetch: byte offset of the lane's 16-byte piece in a K row, per block of four rows   (in)
  v[216:223]  LDS address of the K operand reads per k-step (stage of the next tile)
  v[224:231]  the same in stage 0                                                                (in)
  s[36:43]    halves of this wavefront, tiles, first key of the range, all_lo, all_hi (a half starting at a0 needs no
              mask iff all_lo < a0 <= all_hi), last key of the range, 16 * wavefront, LDS address of the wavefront's
              part of stage 0                                                                     (in)
  s[44:51]    block table row (64 bit), cache base of the kv head's K rows (64 bit), bytes per token, bytes per page,
              log2(page size), pages - 1                                                          (in)
  s[52:75], s[89:92]  temporaries
"""

from __future__ import annotations

import os

NRG, NKS, NBLK = 2, 8, 4   # row groups of 32 rows, k-steps of 16 elements, blocks of 32 output elements
ROWB = 256
STAGE_B = 32768   # K tile + V tile
NSTG = 4
LAZY_LOG2E = 16.0 * 1.4426950408889634

O = lambda rg, blk: f"a[{16 * (4 * rg + blk)}:{16 * (4 * rg + blk) + 15}]"
KOP = lambda ks: f"a[{128 + 4 * ks}:{128 + 4 * ks + 3}]"
VRAW2 = lambda s, blk, t: f"a[{160 + 4 * (4 * s + blk) + 2 * t}:{160 + 4 * (4 * s + blk) + 2 * t + 1}]"
VRAW = lambda s, blk: f"a[{160 + 4 * (4 * s + blk)}:{160 + 4 * (4 * s + blk) + 3}]"
SQ = lambda base, rg: f"v[{base + 16 * rg}:{base + 16 * rg + 15}]"
SE = lambda base, rg, q, r: f"v{base + 16 * rg + 4 * q + r}"
QOP = lambda rg, ks: f"v[{64 + 4 * (8 * rg + ks)}:{64 + 4 * (8 * rg + ks) + 3}]"
PW = lambda rg, s: f"v[{128 + 4 * (2 * rg + s)}:{128 + 4 * (2 * rg + s) + 3}]"
PWE = lambda rg, s, k: f"v{128 + 4 * (2 * rg + s) + k}"
LSUM = lambda rg: f"v{144 + rg}"
ONES2 = "v146"
MNEG = lambda rg: f"v{148 + rg}"
TMAX = lambda rg: f"v{152 + rg}"
MLO = lambda rg: f"v{156 + rg}"
MSPAN = lambda rg: f"v{160 + rg}"
KADDR = lambda ks: f"v{216 + ks}"
VADDR = "v168"
CFAC = "v169"
T0 = "v170"
NINF = "v171"
MTHR = lambda rg: f"v{172 + rg}"
THRC = "v176"
ROWLO = lambda rg: f"v{178 + rg}"
KBASE = lambda ks: f"v{224 + ks}"
VBASE = "v186"
LROW, VROW, VPIECE = "v187", "v188", "v189"
KPIECE = lambda n: f"v{190 + n}"
T1, T2, T3, T4, T5 = "v195", "v196", "v197", "v198", "v199"
MFMA = "v_mfma_f32_32x32x16_bf16"
PROF = os.environ.get("RPA_PPA_PROF", "") != ""   # experiment: cycle counts of the loop's regions in s[76:83]


def stamp(k: int) -> list[str]:
    """Experiment builds: s[84:85] = now; region k (0..7) gets the cycles since the previous stamp."""
    if not PROF:
        return []
    return ["s_memtime s[84:85]", "s_waitcnt lgkmcnt(0)", f"s_sub_u32 s86, s84, s87", f"s_add_u32 s{76 + k}, s{76 + k}, s86", "s_mov_b32 s87, s84"]


# scalar inputs
S_HB, S_NT, S_RLO, S_ALLLO, S_ALLHI, S_TLAST, S_WAVE16, S_LDSW = (f"s{36 + k}" for k in range(8))
S_BTLO, S_BTHI, S_KVLO, S_KVHI, S_STRIDE, S_PAGEB, S_PSHIFT, S_NP1 = (f"s{44 + k}" for k in range(8))
# scalar temporaries
S_HH, S_T, S_A0, S_CUR, S_NXT, S_FBUF = "s52", "s53", "s54", "s55", "s56", "s57"   # loop state; stage byte offsets
S_R = "s[60:63]"                                                                   # buffer resource of a fetch
S_R0, S_R1, S_R2, S_R3 = "s60", "s61", "s62", "s63"
S_X0, S_X1, S_X2, S_X3, S_X4, S_X5 = "s64", "s65", "s66", "s67", "s68", "s69"
S_P = "s[70:71]"
S_PMASK = "s72"
S_TT = "s73"
S_PG, S_TB, S_D, S_LIM = "s89", "s90", "s91", "s92"   # a prepared fetch: page, base key, offset of the group, last row
S_PEND, S_SITE = "s74", "s75"   # fetch of the tile in S_TT pending (this wavefront's site number, or 0); site number


def kload(h: int) -> list[str]:
    """K operands of a half with parity h from the stage that v[216:223] point into: lane (i, g) reads elements
    16 ks + 8 g .. + 7 of key row i."""
    return [f"ds_read_b128 {KOP(ks)}, {KADDR(ks)} offset:{h * 32 * ROWB}" for ks in range(NKS)]


def vload(h: int) -> list[str]:
    """V^T operands of a half with parity h: for key step s and block blk the keys 16 s + 8 t + 4 g .. + 3 (t = 0, 1)
    of output elements 32 blk + i, by two transposing reads (in each group of 16 lanes, lanes 4e..4e+3 address 16
    consecutive elements of key e; lane x receives element x of the four keys)."""
    return [f"ds_read_b64_tr_b16 {VRAW2(s, blk, t)}, {VADDR} offset:{(8 * h + 4 * s + 2 * t) * 1024 + blk * 256}"
            for s in range(2) for blk in range(NBLK) for t in range(2)]


def qk(n: int, nxt: int) -> str:
    """MFMA n (0..15) of S^T = K Q^T: k-step outermost, the two row groups in turn."""
    ks, rg = n >> 1, n & 1
    c = "0" if ks == 0 else SQ(nxt, rg)
    return f"{MFMA} {SQ(nxt, rg)}, {KOP(ks)}, {QOP(rg, ks)}, {c}"


def sm1_pair(cur: int, p: int, mask: bool, rnd: bool) -> list[str]:
    """Pair p (0..15) of the half: elements (rg, q, r), (rg, q, r + 1) with rg = p / 8, q = (p % 8) / 2, r = 2 (p % 2):
    logit -> exp2 argument in place, running maximum of the row group."""
    rg, q, r = p >> 3, (p & 7) >> 1, 2 * (p & 1)
    x0, x1 = SE(cur, rg, q, r), SE(cur, rg, q, r + 1)
    out = []
    if mask:
        for x, cst in ((x0, 8 * q + r), (x1, 8 * q + r + 1)):
            out += [f"v_sub_u32 {T0}, {cst}, {MLO(rg)}", f"v_cmp_le_u32 vcc, {T0}, {MSPAN(rg)}", f"v_cndmask_b32 {x}, {NINF}, {x}, vcc"]
    if rnd:
        out += [f"v_cvt_pk_bf16_f32 {T0}, {x0}, {x1}", f"v_lshlrev_b32 {x0}, 16, {T0}", f"v_and_b32 {x1}, 0xffff0000, {T0}"]
    out += [f"v_fma_f32 {x0}, {x0}, {CFAC}, {MNEG(rg)}", f"v_fma_f32 {x1}, {x1}, {CFAC}, {MNEG(rg)}"]
    out += [f"v_max_f32 {TMAX(rg)}, {x0}, {x1}" if (p & 7) == 0 else f"v_max3_f32 {TMAX(rg)}, {TMAX(rg)}, {x0}, {x1}"]
    return out


def block_a(h: int, mask: bool, rnd: bool) -> list[str]:
    """[QK(next half) | SM1(this half)]: 16 slots of one MFMA (32 cycles of the matrix pipe, about 8 of the issue port)
    and one pair's vector work (six instructions, about 25 cycles)."""
    cur, nxt = (0, 32) if h == 0 else (32, 0)
    out = ["s_waitcnt lgkmcnt(0)"] + vload(h)
    if mask:
        out += [f"v_subrev_u32 {MLO(rg)}, {S_A0}, {ROWLO(rg)}" for rg in range(NRG)]
    for n in range(16):
        out.append(qk(n, nxt))
        out += sm1_pair(cur, n, mask, rnd)
    return out


def sm2_exp(cur: int, rg: int, s: int, k: int) -> list[str]:
    """The exponentials of pair k (0..3) of P(rg, s): elements q = 2 s + k / 2, r = 2 (k % 2), + 1."""
    q, r = 2 * s + (k >> 1), 2 * (k & 1)
    return [f"v_exp_f32 {SE(cur, rg, q, r)}, {SE(cur, rg, q, r)}", f"v_exp_f32 {SE(cur, rg, q, r + 1)}, {SE(cur, rg, q, r + 1)}"]


def sm2_pack(cur: int, rg: int, s: int, k: int) -> list[str]:
    q, r = 2 * s + (k >> 1), 2 * (k & 1)
    return [f"v_cvt_pk_bf16_f32 {PWE(rg, s, k)}, {SE(cur, rg, q, r)}, {SE(cur, rg, q, r + 1)}"]


def rowsum(cur: int, rg: int, s: int, k: int) -> list[str]:
    """Pair k of P(rg, s) joins the lane's row sum: two fp32 additions of the exponentials themselves.  (A
    v_dot2_f32_bf16 of the packed pair against two ones is one instruction instead of two, but it issues at a quarter
    of the rate and, reading an MFMA operand, has to wait for the MFMAs in flight: it cost 3.7 additions' time.)"""
    q, r = 2 * s + (k >> 1), 2 * (k & 1)
    return [f"v_add_f32 {LSUM(rg)}, {LSUM(rg)}, {SE(cur, rg, q, r)}", f"v_add_f32 {LSUM(rg)}, {LSUM(rg)}, {SE(cur, rg, q, r + 1)}"]


def block_b(h: int) -> list[str]:
    """[SM2 | PV]: P^T operand (rg, s) = exp2 of eight arguments per lane, packed to bf16; its four MFMAs (one per
    block of 32 output elements) run while the vector unit prepares the next operand and adds up its row sums.
    Rules the order obeys: the result of a transcendental instruction may not be read by the very next instruction
    (the hardware does not wait); a register written by a vector instruction may not be read by an MFMA within two
    wait states; and a vector instruction that touches a register an MFMA in flight reads waits for that MFMA, so
    the row sums read the exponentials, not the packed operand."""
    cur = 0 if h == 0 else 32
    groups = [(rg, s) for rg in range(NRG) for s in range(2)]
    out = kload(h) + ["s_waitcnt lgkmcnt(8)"]
    rg, s = groups[0]
    out += sm2_exp(cur, rg, s, 0) + sm2_exp(cur, rg, s, 1) + sm2_pack(cur, rg, s, 0) + rowsum(cur, rg, s, 0)
    out += sm2_exp(cur, rg, s, 2) + sm2_pack(cur, rg, s, 1) + rowsum(cur, rg, s, 1)
    out += sm2_exp(cur, rg, s, 3) + sm2_pack(cur, rg, s, 2) + rowsum(cur, rg, s, 2) + sm2_pack(cur, rg, s, 3) + rowsum(cur, rg, s, 3)
    for gi, (rg, s) in enumerate(groups):
        nx = groups[gi + 1] if gi + 1 < len(groups) else None
        for blk in range(NBLK):
            out.append(f"{MFMA} {O(rg, blk)}, {VRAW(s, blk)}, {PW(rg, s)}, {O(rg, blk)}")
            if nx is None:
                continue
            out += sm2_exp(cur, nx[0], nx[1], blk)
            if blk >= 1:
                out += sm2_pack(cur, *nx, blk - 1) + rowsum(cur, *nx, blk - 1)
            if blk == 3:
                out += sm2_pack(cur, *nx, 3) + rowsum(cur, *nx, 3)
    return out


def rescale(h: int, tag: str) -> list[str]:
    """Vote; where some row's exp2 argument exceeds its threshold (or the row sees its first key), move that row's
    reference point up by the row maximum: shift the exp2 arguments, scale row sum and outputs by exp2(-shift)."""
    cur = 0 if h == 0 else 32
    # (a row without a reference point has threshold -inf: the difference is +inf, or NaN when it has no key yet either,
    # which the maximum drops)
    out = [f"v_sub_f32 {T1}, {TMAX(0)}, {MTHR(0)}", f"v_sub_f32 {T2}, {TMAX(1)}, {MTHR(1)}", f"v_max_f32 {T1}, {T1}, {T2}",
           f"v_cmp_lt_f32 vcc, 0, {T1}", f"s_cbranch_vccz .Lpp_noresc_{tag}_%="]
    for rg in range(NRG):
        x = TMAX(rg)
        # maximum over the two lanes that hold one row (lanes l, l ^ 32)
        out += [f"v_mov_b32 {T1}, {x}", f"v_mov_b32 {T2}, {x}", "s_nop 1", f"v_permlane32_swap_b32 {T1}, {T2}", "s_nop 1",
                f"v_max_f32 {T3}, {T1}, {T2}"]
        out += [f"v_cmp_gt_f32 vcc, {T3}, {MTHR(rg)}", f"s_cbranch_vccz .Lpp_skip{rg}_{tag}_%="]
        out += [f"v_cndmask_b32 {T4}, 0, {T3}, vcc",                       # shift: the row maximum where the row moves
                f"v_exp_f32_e64 {T5}, -{T3}",
                f"v_cmp_neq_f32 {S_P}, {MTHR(rg)}, {NINF}",
                f"v_cndmask_b32_e64 {T5}, 0, {T5}, {S_P}",                 # a row without a reference point: outputs are zero
                f"v_cndmask_b32 {T5}, 1.0, {T5}, vcc",                     # alpha
                f"v_cndmask_b32 {MTHR(rg)}, {MTHR(rg)}, {THRC}, vcc"]
        out += [f"v_sub_f32 {SE(cur, rg, q, r)}, {SE(cur, rg, q, r)}, {T4}" for q in range(4) for r in range(4)]
        out += [f"v_sub_f32 {MNEG(rg)}, {MNEG(rg)}, {T4}", f"v_mul_f32 {LSUM(rg)}, {LSUM(rg)}, {T5}"]
        regs = [64 * rg + k for k in range(64)]
        for q in range(0, len(regs), 4):
            grp = regs[q:q + 4]
            tmp = [T1, T2, T3, T4]
            out += [f"v_accvgpr_read_b32 {t}, a{a}" for t, a in zip(tmp, grp)]
            out += [f"v_mul_f32 {t}, {t}, {T5}" for t in tmp]
            out += [f"v_accvgpr_write_b32 a{a}, {t}" for t, a in zip(tmp, grp)]
        out.append(f".Lpp_skip{rg}_{tag}_%=:")
    out.append(f".Lpp_noresc_{tag}_%=:")
    return out


VO = [f"v{200 + k}" for k in range(8)]     # fetch: byte offsets of the lane's pieces in a group of 16 whole rows (4 K, 4 V blocks)
VOX = [f"v{208 + k}" for k in range(8)]    # the same for a group that reaches past the last key


def fetch_setup() -> list[str]:
    """Per-lane byte offsets of a fetch whose 16 rows all exist (every tile but the last of a range)."""
    out = []
    for n in range(4):
        out += [f"v_add_u32 {T3}, {4 * n}, {LROW}", f"v_mad_u32_u24 {VO[n]}, {T3}, {S_STRIDE}, {KPIECE(n)}",
                f"v_add_u32 {T3}, {4 * n}, {VROW}", f"v_mad_u32_u24 {VO[4 + n]}, {T3}, {S_STRIDE}, {VPIECE}"]
    return out


def fetch_prepare() -> list[str]:
    """For the tile whose first key is in S_TT: the group's base key, how far the group lies behind it, the last row
    that exists; requests the page of the base key (the group's 16 keys share it: pages of at least 16 keys)."""
    return [f"s_add_i32 {S_X0}, {S_TT}, {S_WAVE16}",            # first key of the group
            f"s_and_b32 {S_TB}, {S_TLAST}, -16",
            f"s_min_i32 {S_TB}, {S_TB}, {S_X0}",                 # base key: same page as every key fetched
            f"s_sub_i32 {S_D}, {S_X0}, {S_TB}",
            f"s_sub_i32 {S_LIM}, {S_TLAST}, {S_TB}",            # last row that exists, relative to the base
            f"s_lshr_b32 {S_X4}, {S_TB}, {S_PSHIFT}", f"s_lshl_b32 {S_X4}, {S_X4}, 2",
            f"s_add_u32 {S_X4}, {S_BTLO}, {S_X4}", f"s_addc_u32 {S_X5}, {S_BTHI}, 0",
            f"s_load_dword {S_PG}, s[68:69], 0x0"]


def fetch(tag: str) -> list[str]:
    """This wavefront's part (16 K rows, 16 V rows) of the prepared tile into the stage at byte offset S_FBUF.  Keys
    past the range repeat the last one."""
    out = ["s_waitcnt lgkmcnt(0)",
           f"s_max_i32 {S_X0}, {S_PG}, 0", f"s_min_i32 {S_X0}, {S_X0}, {S_NP1}",
           f"s_mul_hi_u32 {S_X5}, {S_X0}, {S_PAGEB}", f"s_mul_i32 {S_X4}, {S_X0}, {S_PAGEB}",
           f"s_and_b32 {S_X1}, {S_TB}, {S_PMASK}", f"s_mul_i32 {S_X1}, {S_X1}, {S_STRIDE}",
           f"s_add_u32 {S_X4}, {S_X4}, {S_X1}", f"s_addc_u32 {S_X5}, {S_X5}, 0",
           f"s_add_u32 {S_R0}, {S_X4}, {S_KVLO}", f"s_addc_u32 {S_R1}, {S_X5}, {S_KVHI}",
           f"s_and_b32 {S_R1}, {S_R1}, 0xffff",
           f"s_add_i32 {S_X0}, {S_LDSW}, {S_FBUF}",
           f"s_cmp_lt_i32 {S_LIM}, 15", f"s_cbranch_scc1 .Lpp_fx_{tag}_%=",
           f"s_cmp_lg_u32 {S_D}, 0", f"s_cbranch_scc1 .Lpp_fx_{tag}_%="]

    def loads(vo):
        o = []
        for n in range(4):
            o += [f"s_add_i32 m0, {S_X0}, {n * 1024}", "s_nop 0", f"buffer_load_dwordx4 {vo[n]}, {S_R}, 0 offen lds",
                  f"s_add_i32 m0, {S_X0}, {16384 + n * 1024}", "s_nop 0", f"buffer_load_dwordx4 {vo[4 + n]}, {S_R}, 0 offen lds"]
        return o

    out += loads(VO) + [f"s_branch .Lpp_fd_{tag}_%=", f".Lpp_fx_{tag}_%=:"]
    out += [f"v_add_u32 {T1}, {S_D}, {LROW}", f"v_add_u32 {T2}, {S_D}, {VROW}"]
    for n in range(4):
        out += [f"v_add_u32 {T3}, {4 * n}, {T1}", f"v_min_i32 {T3}, {S_LIM}, {T3}", f"v_mad_u32_u24 {VOX[n]}, {T3}, {S_STRIDE}, {KPIECE(n)}",
                f"v_add_u32 {T3}, {4 * n}, {T2}", f"v_min_i32 {T3}, {S_LIM}, {T3}", f"v_mad_u32_u24 {VOX[4 + n]}, {T3}, {S_STRIDE}, {VPIECE}"]
    out += loads(VOX) + [f".Lpp_fd_{tag}_%=:"]
    return out


def publish(tag: str, t_reg: str) -> list[str]:
    """Publishes tile t + 1: this wavefront's part of it has landed (its loads complete in order; those of tile
    t + 2 may still be in flight), after the barrier everybody's.  Every wavefront is then past its last read of
    tile t - 1, whose stage (byte offset S_FBUF) takes tile t + NSTG - 1: the fetch is left pending for the wavefront's
    site of the tile, so that the four wavefronts do not issue their loads at the same moment (a compute unit accepts
    one 1-KiB load per 16 cycles or so, and a wavefront is held while its load waits)."""
    return [f"s_add_i32 {S_X0}, {t_reg}, 2", f"s_cmp_ge_i32 {S_X0}, {S_NT}", f"s_cbranch_scc1 .Lpp_w0_{tag}_%=",
            "s_waitcnt vmcnt(8)", f"s_branch .Lpp_w1_{tag}_%=", f".Lpp_w0_{tag}_%=:", "s_waitcnt vmcnt(0)", f".Lpp_w1_{tag}_%=:"] + \
        (stamp(6) if tag == "loop" else []) + ["s_barrier"] + (stamp(7) if tag == "loop" else []) + [
            f"s_add_i32 {S_X0}, {t_reg}, {NSTG - 1}", f"s_cmp_ge_i32 {S_X0}, {S_NT}", f"s_cbranch_scc1 .Lpp_nofetch_{tag}_%=",
            f"s_lshl_b32 {S_TT}, {S_X0}, 6", f"s_add_i32 {S_TT}, {S_TT}, {S_RLO}", f"s_mov_b32 {S_PEND}, {S_SITE}"] + fetch_prepare() + [
            f".Lpp_nofetch_{tag}_%=:"]


def site(k: int, tag: str) -> list[str]:
    """Fetch site k of a tile (0: behind the barrier, 1: end of the first half, 2: middle of the second half, 3: end of
    the tile): the wavefront whose site this is issues its pending fetch.  k < 0: whoever has one pending."""
    test = [f"s_cmp_eq_u32 {S_PEND}, {k + 1}"] if k >= 0 else [f"s_cmp_lg_u32 {S_PEND}, 0"]
    return test + [f"s_cbranch_scc0 .Lpp_nosite_{tag}_%="] + fetch(tag) + [f"s_mov_b32 {S_PEND}, 0", f".Lpp_nosite_{tag}_%=:"]


def half(h: int, rnd: bool) -> tuple[list[str], list[str]]:
    """One half; the second list is its masked block A, kept out of line behind the loop."""
    tag = f"h{h}"
    out = [f"s_cmp_gt_i32 {S_A0}, {S_ALLLO}", f"s_cbranch_scc0 .Lpp_mask_{tag}_%=",
           f"s_cmp_le_i32 {S_A0}, {S_ALLHI}", f"s_cbranch_scc0 .Lpp_mask_{tag}_%="]
    out += stamp(0)
    out += block_a(h, False, rnd) + stamp(1) + [f".Lpp_adone_{tag}_%=:"]
    cold = [f".Lpp_mask_{tag}_%=:"] + block_a(h, True, rnd) + stamp(2) + [f"s_branch .Lpp_adone_{tag}_%="]
    out += rescale(h, tag) + stamp(3)
    if h == 0:
        out += [f"s_add_i32 {S_X0}, {S_T}, 1", f"s_cmp_ge_i32 {S_X0}, {S_NT}", f"s_cbranch_scc1 .Lpp_nopub_%="]
        out += publish("loop", S_T) + [".Lpp_nopub_%=:"] + site(0, "s0") + stamp(4)
    else:
        out += site(2, "s2")
    out += block_b(h) + stamp(5)
    out += site(1 if h == 0 else 3, "s1" if h == 0 else "s3")
    out += [f"s_add_i32 {S_HH}, {S_HH}, 1", f"s_add_i32 {S_A0}, {S_A0}, 32", f"s_cmp_eq_u32 {S_HH}, {S_HB}", "s_cbranch_scc1 .Lpp_done_%="]
    return out, cold


def rotate_stages() -> list[str]:
    """Start of a tile: stage offsets of this tile, the next one and the one to refill; operand addresses."""
    out = [f"s_mov_b32 {S_FBUF}, {S_CUR}",      # after this tile's barrier the previous tile's stage is refilled ...
           f"s_mov_b32 {S_CUR}, {S_NXT}",
           f"s_add_i32 {S_NXT}, {S_NXT}, {STAGE_B}", f"s_cmp_eq_u32 {S_NXT}, {NSTG * STAGE_B}", f"s_cselect_b32 {S_NXT}, 0, {S_NXT}"]
    out += [f"v_add_u32 {VADDR}, {S_CUR}, {VBASE}"] + [f"v_add_u32 {KADDR(ks)}, {S_NXT}, {KBASE(ks)}" for ks in range(NKS)]
    return out


def loop(rnd: bool) -> list[str]:
    out = ["s_mov_b32 s58, m0"]  # the compiler's m0 is restored at the end
    if PROF:
        out += [f"s_mov_b32 s{76 + k}, 0" for k in range(8)] + ["s_memtime s[84:85]", "s_waitcnt lgkmcnt(0)", "s_mov_b32 s87, s84", "s_mov_b32 s88, s84"]
    # ---- set-up
    out += [f"v_accvgpr_write_b32 a{k}, 0" for k in range(128)]
    out += [f"v_mov_b32 {MNEG(rg)}, 0" for rg in range(NRG)] + [f"v_mov_b32 {LSUM(rg)}, 0" for rg in range(NRG)] + [f"v_mov_b32 {NINF}, 0xff800000"]
    out += [f"v_mov_b32 {MTHR(rg)}, {NINF}" for rg in range(NRG)]
    out += [f"v_mov_b32 {THRC}, 0x{float_bits(LAZY_LOG2E):08x}", f"v_mov_b32 {ONES2}, 0x3f803f80"]
    out += [f"s_mov_b32 {S_R2}, 0x7fffffff", f"s_mov_b32 {S_R3}, 0x00020000",
            f"s_lshl_b32 {S_PMASK}, 1, {S_PSHIFT}", f"s_add_i32 {S_PMASK}, {S_PMASK}, -1",
            f"s_mov_b32 {S_HH}, 0", f"s_mov_b32 {S_T}, 0", f"s_mov_b32 {S_A0}, {S_RLO}",
            f"s_mov_b32 {S_PEND}, 0", f"s_lshr_b32 {S_SITE}, {S_WAVE16}, 4", f"s_add_i32 {S_SITE}, {S_SITE}, 1",
            ]
    out += fetch_setup()
    out += [f"s_cmp_eq_u32 {S_HB}, 0", "s_cbranch_scc1 .Lpp_done_%="]
    # stage state as if tile -1 were in progress: the first rotation makes tile 0 current
    out += [f"s_mov_b32 {S_CUR}, {(NSTG - 1) * STAGE_B}", f"s_mov_b32 {S_NXT}, 0"]
    # logits of the first half, K operands of the second (both in tile 0, stage 0)
    out += [f"v_mov_b32 {KADDR(ks)}, {KBASE(ks)}" for ks in range(NKS)]
    out += kload(0) + ["s_waitcnt lgkmcnt(0)"] + [qk(n, 0) for n in range(16)] + ["s_nop 7", "s_nop 7"] + kload(1)
    out.append(".Lpp_tile_%=:")
    out += rotate_stages()
    h0, cold0 = half(0, rnd)
    h1, cold1 = half(1, rnd)
    out += h0 + h1
    out += [f"s_add_i32 {S_T}, {S_T}, 1", "s_branch .Lpp_tile_%="]
    out += cold0 + cold1
    # ---- tiles past this wavefront's last half: it still takes part in their barriers and fetches
    out += [".Lpp_done_%=:"] + site(-1, "sx") + [
            f"s_add_i32 {S_X5}, {S_HH}, 1", f"s_lshr_b32 {S_T}, {S_X5}, 1",
            # the stage to refill at tile t's barrier is that of tile t - 1
            f"s_add_i32 {S_X0}, {S_T}, {NSTG - 1}", f"s_and_b32 {S_X0}, {S_X0}, {NSTG - 1}", f"s_mul_i32 {S_FBUF}, {S_X0}, {STAGE_B}",
            ".Lpp_tail_%=:",
            f"s_add_i32 {S_X0}, {S_T}, 1", f"s_cmp_ge_i32 {S_X0}, {S_NT}", "s_cbranch_scc1 .Lpp_end_%="]
    out += publish("tail", S_T) + site(-1, "st")
    out += [f"s_add_i32 {S_T}, {S_T}, 1",
            f"s_add_i32 {S_FBUF}, {S_FBUF}, {STAGE_B}", f"s_cmp_eq_u32 {S_FBUF}, {NSTG * STAGE_B}", f"s_cselect_b32 {S_FBUF}, 0, {S_FBUF}",
            "s_branch .Lpp_tail_%=", ".Lpp_end_%=:", "s_waitcnt lgkmcnt(0)", "s_mov_b32 m0, s58", "s_nop 7", "s_nop 7", "s_nop 7"]
    if PROF:
        out += []
    return out


def float_bits(x: float) -> int:
    import struct
    return struct.unpack("<I", struct.pack("<f", x))[0]


def macro(name: str, lines: list[str]) -> str:
    body = " \\\n".join(f'  "{ln}\\n\\t"' for ln in lines)
    return f"#define {name} \\\n{body}\n"


def render() -> str:
    parts = ["// Generated by gen_prefill_pipe_asm.py -- do not edit; see that file for the register map.\n#pragma once\n"]
    parts.append(macro("RPA_PPA_LOOP_ROUND", loop(True)))
    parts.append(macro("RPA_PPA_LOOP_PLAIN", loop(False)))
    return "\n".join(parts)


INC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rpa_prefill_pipe_asm.inc")

if __name__ == "__main__":
    with open(INC, "w") as f:
        f.write(render())
    print(f"wrote {INC}")
