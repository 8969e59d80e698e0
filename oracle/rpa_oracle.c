/*
 * C restatement of the reference's XLA ragged paged attention forward, used as the timed
 * CPU baseline and as a second checker.  TEST INFRASTRUCTURE ONLY: nothing shipped links it.
 *
 * It follows ejkernel/kernels/_xla/ragged_page_attention/_xla_impl_fwd.py:39-201 step by step:
 * sequences in order (:195-198), 8-row query blocks (:47,:85-92), KV blocks of
 * min(64, pages_per_seq) pages (:48,:103-114), K at even / V at odd combined head index
 * (:113-114), logits = (q * scale) . k (:49,:119-124), optional cap * tanh(x / cap) (:125-126),
 * mask q_pos >= k_pos, k_pos > q_pos - window, k_pos < kv_len (:128-136), online softmax with the
 * carry (o, l, m) held in the compute dtype (:138-155), denominator clamped at 1e-6 (:174),
 * optional sinks (:161-172).  With bf16 storage every op result is rounded to bf16
 * (round-to-nearest-even), as XLA does for bf16 ops; with fp32 storage nothing is rounded.
 *
 * Two deliberate differences from the reference program, neither visible on rows it defines when
 * `queries` carries >= 8 slack rows and pages_per_seq is < 64 or a multiple of 64:
 *   - a query block stores only the rows that belong to its sequence (the reference also writes
 *     the junk rows of its 8-row window, later overwritten by their owners), which lets blocks run
 *     in parallel;
 *   - block-table windows are not clamped (the reference's clamp misaligns keys when
 *     pages_per_seq >= 64 is not a multiple of 64).
 * The NaN of a row whose first KV block is entirely left of the window IS reproduced.
 *
 * Pinned by tests/test_oracle_pins.py against oracle/rpa_oracle.py (rpa_strict) and the float64
 * evaluation.  Parity unpinned: the exact rounding sequence of XLA:CPU (see rpa_oracle.py).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define QBLK 8
#define CLONES __attribute__((target_clones("default", "avx2", "avx512f")))

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static inline float rb(float f, int bf16) { return bf16 ? bf16_to_f32(f32_to_bf16(f)) : f; }

typedef struct {
  const void* q;
  const void* kv;
  const int32_t* ctx;
  const int32_t* bt;
  const int32_t* cu;
  const float* sinks;
  void* out;
  int T, Hq, Hkv, D, page, P, pps, n_sinks, bf16, window;
  int aux_bf16; /* the sinks' dtype is as narrow as the carry's: the epilogue rounds to bf16 at every op */
  float scale, cap;
} Args;

static inline float load_elem(const void* base, size_t idx, int bf16) {
  return bf16 ? bf16_to_f32(((const uint16_t*)base)[idx]) : ((const float*)base)[idx];
}

CLONES static void scores_block(const float* restrict qs, const float* restrict kb, float* restrict sc, int rows, int keys,
                                int D) {
  for (int r = 0; r < rows; ++r)
    for (int k = 0; k < keys; ++k) {
      float acc = 0.f;
      const float* a = qs + (size_t)r * D;
      const float* b = kb + (size_t)k * D;
      for (int d = 0; d < D; ++d) acc += a[d] * b[d];
      sc[(size_t)r * keys + k] = acc;
    }
}

CLONES static void pv_block(const float* restrict p, const float* restrict vb, float* restrict upd, int rows, int keys,
                            int D) {
  for (int r = 0; r < rows; ++r) {
    float* u = upd + (size_t)r * D;
    for (int d = 0; d < D; ++d) u[d] = 0.f;
    for (int k = 0; k < keys; ++k) {
      const float pk = p[(size_t)r * keys + k];
      if (pk == 0.f) continue;
      const float* v = vb + (size_t)k * D;
      for (int d = 0; d < D; ++d) u[d] += pk * v[d];
    }
  }
}

/* One (sequence, query block, kv head): the body of _process_query_block restricted to one kv head
 * (the reference carries all kv heads at once; they do not interact). */
static void run_item(const Args* a, int s, int qb, int j, float* kb, float* vb, float* sc, float* qs, float* o, float* upd) {
  const int G = a->Hq / a->Hkv, D = a->D, bf = a->bf16, ebf = a->bf16 && a->aux_bf16;
  const int q0 = a->cu[s], q_len = a->cu[s + 1] - q0, kv_len = a->ctx[s];
  const int kvblocks = a->pps >= 64 ? 64 : (a->pps > 1 ? a->pps : 1);
  const int kv_tok = a->page * kvblocks;
  const int n_kvb = (kv_len + kv_tok - 1) / kv_tok;
  const int rows = QBLK * G; /* row r = b * G + g: query row b of the block, group head g */
  const int q_off = qb * QBLK;
  const float scale_q = rb(a->scale, bf);
  float m[QBLK * 64], l[QBLK * 64]; /* G <= 64 */

  for (int b = 0; b < QBLK; ++b)
    for (int g = 0; g < G; ++g) {
      const int row = q0 + q_off + b;
      float* dst = qs + (size_t)(b * G + g) * D;
      if (row < a->T) {
        const size_t base = ((size_t)row * a->Hq + (size_t)j * G + g) * D;
        for (int d = 0; d < D; ++d) dst[d] = rb(load_elem(a->q, base + d, bf) * scale_q, bf); /* :49 */
      } else {
        memset(dst, 0, sizeof(float) * D); /* zero padding rows :51-56 */
      }
    }
  for (int r = 0; r < rows; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
  }
  memset(o, 0, sizeof(float) * rows * D);

  for (int kbi = 0; kbi < n_kvb; ++kbi) {
    /* gather: K rows at combined head 2j, V rows at 2j+1 (:113-114) */
    for (int pg = 0; pg < kvblocks; ++pg) {
      const int slot = kbi * kvblocks + pg;
      int page_id = slot < a->pps ? a->bt[(size_t)s * a->pps + slot] : 0;
      if (page_id < 0) page_id += a->P; /* negative indices wrap, then clamp: what the gather does */
      if (page_id < 0) page_id = 0;
      if (page_id >= a->P) page_id = a->P - 1;
      for (int t = 0; t < a->page; ++t) {
        const size_t src = (((size_t)page_id * a->page + t) * 2 * a->Hkv + 2 * (size_t)j) * D;
        float* kd = kb + ((size_t)pg * a->page + t) * D;
        float* vd = vb + ((size_t)pg * a->page + t) * D;
        for (int d = 0; d < D; ++d) {
          kd[d] = load_elem(a->kv, src + d, bf);
          vd[d] = load_elem(a->kv, src + D + d, bf);
        }
      }
    }
    scores_block(qs, kb, sc, rows, kv_tok, D); /* :119-124 */
    for (int r = 0; r < rows; ++r) {
      const int b = r / G;
      const int q_pos = kv_len - q_len + q_off + b; /* :96-97 */
      float* srow = sc + (size_t)r * kv_tok;
      float cur = -INFINITY;
      for (int k = 0; k < kv_tok; ++k) {
        const int k_pos = kbi * kv_tok + k;
        float x = rb(srow[k], bf);
        if (a->cap != 0.f) { /* :125-126; the Python scalar is weakly typed: it takes the array's dtype first */
          const float capc = rb(a->cap, bf);
          x = rb(rb(tanhf(rb(x / capc, bf)), bf) * capc, bf);
        }
        const int keep = q_pos >= k_pos && k_pos < kv_len && (a->window <= 0 || k_pos > q_pos - a->window);
        x = keep ? x : -INFINITY; /* :138 */
        srow[k] = x;
        if (x > cur) cur = x;
      }
      const float new_m = m[r] > cur ? m[r] : cur; /* :141 */
      float psum = 0.f;
      for (int k = 0; k < kv_tok; ++k) {
        const float x = srow[k];
        /* exp(x - new_m), then where(mask, probs, 0): masked keys are exactly the -inf logits (:143-144) */
        const float pk = x == -INFINITY ? 0.f : rb(expf(rb(x - new_m, bf)), bf);
        srow[k] = pk;
        psum += pk;
      }
      const float resc = rb(expf(rb(m[r] - new_m, bf)), bf); /* :146, NaN when both are -inf */
      l[r] = rb(rb(resc * l[r], bf) + rb(psum, bf), bf);  /* :147 */
      float* orow = o + (size_t)r * D;
      for (int d = 0; d < D; ++d) orow[d] = rb(resc * orow[d], bf);
      m[r] = new_m;
    }
    pv_block(sc, vb, upd, rows, kv_tok, D); /* :148 */
    for (size_t e = 0; e < (size_t)rows * D; ++e) o[e] = rb(o[e] + rb(upd[e], bf), bf); /* :149 */
  }

  for (int b = 0; b < QBLK; ++b) {
    if (q_off + b >= q_len) continue; /* rows of this sequence only */
    const int row = q0 + q_off + b;
    if (row >= a->T) continue;
    for (int g = 0; g < G; ++g) {
      const int r = b * G + g, h = j * G + g;
      const float* orow = o + (size_t)r * D;
      float num = 1.f, den;
      if (a->sinks && a->n_sinks > 0) { /* :161-172 */
        /* float32 sinks promote the epilogue of a bf16 carry to float32 (jnp.maximum at :166 and all after it) */
        const float* sk = a->sinks + (size_t)h * a->n_sinks;
        float smax = -INFINITY, ssum = 0.f;
        for (int k = 0; k < a->n_sinks; ++k) smax = rb(sk[k], ebf) > smax ? rb(sk[k], ebf) : smax;
        const float mt = m[r] > smax ? m[r] : smax;
        for (int k = 0; k < a->n_sinks; ++k) ssum += rb(expf(rb(rb(sk[k], ebf) - mt, ebf)), ebf);
        num = rb(expf(rb(m[r] - mt, ebf)), ebf);
        den = rb(rb(num * l[r], ebf) + rb(ssum, ebf), ebf);
        const float floor_ = rb(1e-6f, ebf);
        den = den > floor_ ? den : floor_;
      } else {
        const float floor_ = rb(1e-6f, bf); /* :174, the weakly typed 1e-6 in the carry's dtype */
        den = l[r] > floor_ ? l[r] : floor_;
        if (l[r] != l[r]) den = l[r];
      }
      const size_t dst = ((size_t)row * a->Hq + h) * D;
      for (int d = 0; d < D; ++d) {
        float v = a->sinks && a->n_sinks > 0 ? rb(rb(rb(num * orow[d], ebf) / den, ebf), bf) : rb(orow[d] / den, bf);
        if (bf) ((uint16_t*)a->out)[dst + d] = f32_to_bf16(v);
        else ((float*)a->out)[dst + d] = v;
      }
    }
  }
}

/* Returns 0, or -1 on bad arguments / allocation failure.  `threads` <= 0 keeps OpenMP's default. */
int rpa_oracle_strict(const void* q, const void* kv, const int32_t* ctx, const int32_t* bt, const int32_t* cu, int num_seqs,
                      int T, int Hq, int Hkv, int D, int page, int P, int pps, float scale, float cap, int window,
                      const float* sinks, int n_sinks, int is_bf16, void* out, int threads, int aux_is_bf16) {
  if (Hq % Hkv || Hq / Hkv > 64 || D <= 0 || page <= 0) return -1;
  Args a = {q, kv, ctx, bt, cu, sinks, out, T, Hq, Hkv, D, page, P, pps, n_sinks, is_bf16, window, aux_is_bf16, scale, cap};
  const int G = Hq / Hkv;
  const int kvblocks = pps >= 64 ? 64 : (pps > 1 ? pps : 1);
  const size_t kv_tok = (size_t)page * kvblocks, rows = (size_t)QBLK * G;
  memset(out, 0, (size_t)T * Hq * D * (is_bf16 ? 2 : 4)); /* zeros_like :58 */

  /* work items in the reference's order: sequence, query block; kv heads are independent */
  size_t n_items = 0;
  for (int s = 0; s < num_seqs; ++s) {
    const int q_len = cu[s + 1] - cu[s];
    if (q_len > 0) n_items += (size_t)((q_len + QBLK - 1) / QBLK) * Hkv;
  }
  int* items = (int*)malloc(sizeof(int) * 3 * (n_items ? n_items : 1));
  if (!items) return -1;
  size_t n = 0;
  for (int s = 0; s < num_seqs; ++s) {
    const int q_len = cu[s + 1] - cu[s];
    if (q_len <= 0) continue; /* :189-193 */
    for (int qb = 0; qb < (q_len + QBLK - 1) / QBLK; ++qb)
      for (int j = 0; j < Hkv; ++j) {
        items[3 * n] = s;
        items[3 * n + 1] = qb;
        items[3 * n + 2] = j;
        ++n;
      }
  }
  int failed = 0;
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#endif
#pragma omp parallel
  {
    float* kb = (float*)malloc(sizeof(float) * kv_tok * D);
    float* vb = (float*)malloc(sizeof(float) * kv_tok * D);
    float* sc = (float*)malloc(sizeof(float) * rows * kv_tok);
    float* qs = (float*)malloc(sizeof(float) * rows * D);
    float* o = (float*)malloc(sizeof(float) * rows * D);
    float* upd = (float*)malloc(sizeof(float) * rows * D);
    if (!kb || !vb || !sc || !qs || !o || !upd) {
#pragma omp atomic write
      failed = 1;
    } else {
#pragma omp for schedule(dynamic, 1)
      for (long it = 0; it < (long)n_items; ++it)
        run_item(&a, items[3 * it], items[3 * it + 1], items[3 * it + 2], kb, vb, sc, qs, o, upd);
    }
    free(kb); free(vb); free(sc); free(qs); free(o); free(upd);
  }
  free(items);
  return failed ? -1 : 0;
}

int rpa_oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
