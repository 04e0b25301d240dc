/*
 * CPU oracle for the block-INT8 fused-MoE path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's
 * `fused_experts_impl_int8(use_int8_w8a8=True, block_shape=[128,128])` path.
 * It is the checker that the HIP kernels are compared with; nothing in the
 * shipped library links, imports or calls it.  Only the tests, the smoke
 * check and the benchmark's cpu-baseline leg may load it.
 *
 * Reference (all paths relative to the reference tree):
 *   routing alignment   python/lightop/_lmslim_native/vllm_compat/moe_align_block_size.py:17-120
 *                       csrc/kernels/moe_align_sum_kernels.cu:1034-1115, :1210-1314
 *                       test/test_moe_align_block_size.py:26-101 (stable ascending order)
 *   1x128 group quant   python/lightop/_lmslim_native/layers/gemm/int8_utils.py:74-195
 *   grouped GEMM        python/lightop/_lmslim_native/layers/fused_moe/int8.py:320-541
 *   SiLU-and-mul        call site int8.py:811; in-repo twin
 *                       csrc/kernels/gated_activation/fuse_silu_mul_quant.cu:893-905
 *   top-k reduce        csrc/kernels/moe_align_sum_kernels.cu:551-637, :860-909
 *   orchestration       int8.py:628-908
 *
 * Arithmetic rules: every fp32 operation is a single IEEE-754 RN operation
 * (compile with -ffp-contract=off, never -ffast-math); bf16 conversion is
 * round-to-nearest-even; float->int8 is truncation toward zero after the
 * clamp; int8 dot products are exact in int32.
 *
 * Pinning status (which independent check fixes each function) is listed in
 * tests/test_oracle.py; a function without one is marked "parity unpinned"
 * there.  Known unpinned points: the intra-expert order of sorted_token_ids
 * (the reference kernels rank with atomics; the stable ascending order of the
 * reference's own Python test is taken as canonical) and the last-ulp
 * behaviour of the third-party expf inside vLLM's silu_and_mul (orc_expf below
 * is checked against libm's expf over every bf16 input instead).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_GROUP 128

/* ------------------------------------------------------- 16-bit floats -- */

/* Element type of the activations: 0 = bf16 (default), 1 = IEEE half (hidden_states.dtype ==
 * torch.float16, int8.py:689-696: compute_type follows it, so every value the path stores between
 * its stages is rounded to that type).  A switch for the test harness, like the activation's. */
static int g_f16 = 0;
void orc_set_dtype(int f16) { g_f16 = f16; }

static inline float raw_bf16_to_f32(uint16_t h) {
  union { uint32_t u; float f; } v;
  v.u = (uint32_t)h << 16;
  return v.f;
}

/* Round-to-nearest-even, the rule of moe_sum_from_float
 * (moe_align_sum_kernels.cu:577-589) and of torch's BFloat16 conversion;
 * NaN is kept quiet. */
static inline uint16_t raw_f32_to_bf16(float f) {
  union { uint32_t u; float f; } v;
  v.f = f;
  if ((v.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((v.u >> 16) | 0x0040u);
  v.u += 0x7fffu + ((v.u >> 16) & 1u);
  return (uint16_t)(v.u >> 16);
}

/* IEEE binary16 <-> binary32, spelled out on the bit patterns: subnormals on both sides, round to
 * nearest even, overflow to infinity, NaN kept quiet.  Pinned in tests/test_oracle.py against
 * torch's conversions on all 65536 halves and on every float that lies next to a rounding boundary
 * of each of them. */
static inline float raw_f16_to_f32(uint16_t h) {
  union { uint32_t u; float f; } v;
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  if (e == 0x1fu) {
    v.u = sign | 0x7f800000u | (m << 13);
  } else if (e != 0) {
    v.u = sign | ((e + 112u) << 23) | (m << 13);
  } else if (m == 0) {
    v.u = sign;
  } else { /* subnormal half: normalise */
    int sh = 0;
    while (!(m & 0x400u)) { m <<= 1; ++sh; }
    v.u = sign | ((uint32_t)(113 - sh) << 23) | ((m & 0x3ffu) << 13);
  }
  return v.f;
}

static inline uint16_t raw_f32_to_f16(float f) {
  union { uint32_t u; float f; } v;
  v.f = f;
  const uint16_t sign = (uint16_t)((v.u >> 16) & 0x8000u);
  const uint32_t a = v.u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu)); /* NaN, quiet */
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);                       /* >= 65536: inf */
  if (a >= 0x38800000u) {                                                        /* normal half */
    uint32_t r = a - 0x38000000u;             /* rebias: exponent 113 -> 1 */
    r += 0xfffu + ((r >> 13) & 1u);           /* round to nearest even on bit 13 */
    return (uint16_t)(sign | (r >> 13));      /* a carry out of the mantissa bumps the exponent, up to inf */
  }
  if (a < 0x33000000u) return sign;           /* below half of the smallest subnormal (2^-25): zero */
  /* subnormal half: value = m * 2^-24 with m = round(|f| * 2^24) */
  {
    const int e = (int)(a >> 23);             /* 102 .. 112 */
    const uint32_t m = (a & 0x7fffffu) | 0x800000u;
    const int shift = 126 - e;                /* m * 2^(e-150) * 2^24 = m >> (126 - e) */
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
  }
}

static inline float bf16_to_f32(uint16_t h) { return g_f16 ? raw_f16_to_f32(h) : raw_bf16_to_f32(h); }
static inline uint16_t f32_to_bf16(float f) { return g_f16 ? raw_f32_to_f16(f) : raw_f32_to_bf16(f); }

uint16_t orc_f32_to_f16(float f) { return raw_f32_to_f16(f); }
float orc_f16_to_f32(uint16_t h) { return raw_f16_to_f32(h); }
uint16_t orc_f32_to_bf16(float f) { return f32_to_bf16(f); }
float orc_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

/* ----------------------------------------------------------- alignment -- */

/*
 * moe_align_block_size.  ids[S] are expert ids in [0, num_experts).
 *
 *   ignore_invalid == 0 (the reference default): count on the given ids;
 *     expert_ids[b] is map[e] when a map is given (moe_align_block_size.py:117-118),
 *     else e.
 *   ignore_invalid != 0: ids with map[id] == -1 are dropped, counting and
 *     expert_ids use the mapped id (moe_align_sum_kernels.cu:83-90).
 *
 * sorted[0:sorted_cap] is filled with S (the pad value) first; within an
 * expert the flat slot ids are ascending.  expert_ids beyond P/bs are set to -1.
 * Returns 0, or -1 if an id is out of range or a buffer is too small.
 */
int orc_moe_align_block_size(const int32_t *ids, int64_t S, int32_t num_experts,
                             int32_t bs, const int32_t *map, int ignore_invalid,
                             int32_t *sorted, int64_t sorted_cap,
                             int32_t *expert_ids, int64_t expert_ids_cap,
                             int32_t *num_tokens_post_pad) {
  int64_t *cnt = (int64_t *)calloc((size_t)num_experts + 1, sizeof(int64_t));
  int64_t *off = (int64_t *)calloc((size_t)num_experts + 1, sizeof(int64_t));
  int rc = 0;
  for (int64_t f = 0; f < S; ++f) {
    int32_t e = ids[f];
    if (e < 0 || e >= num_experts) { rc = -1; goto done; }
    if (ignore_invalid && map) {
      e = map[e];
      if (e < 0) continue;
      if (e >= num_experts) { rc = -1; goto done; }
    }
    cnt[e]++;
  }
  for (int32_t e = 0; e < num_experts; ++e)
    off[e + 1] = off[e] + (cnt[e] + bs - 1) / bs * bs;
  {
    int64_t P = off[num_experts];
    if (P > sorted_cap || P / bs > expert_ids_cap) { rc = -1; goto done; }
    for (int64_t i = 0; i < sorted_cap; ++i) sorted[i] = (int32_t)S;
    for (int64_t b = 0; b < expert_ids_cap; ++b) expert_ids[b] = -1;
    for (int32_t e = 0; e < num_experts; ++e)
      for (int64_t b = off[e] / bs; b < off[e + 1] / bs; ++b)
        expert_ids[b] = (map && !ignore_invalid) ? map[e] : e;
    memset(cnt, 0, ((size_t)num_experts + 1) * sizeof(int64_t));
    for (int64_t f = 0; f < S; ++f) {
      int32_t e = ids[f];
      if (ignore_invalid && map) {
        e = map[e];
        if (e < 0) continue;
      }
      sorted[off[e] + cnt[e]++] = (int32_t)f;
    }
    *num_tokens_post_pad = (int32_t)P;
  }
done:
  free(cnt);
  free(off);
  return rc;
}

/* --------------------------------------------------------- group quant -- */

/*
 * per_token_group_quant_int8 for contiguous bf16 x[R, C], groups of 128 along
 * the last dimension (int8_utils.py:110-116):
 *   amax = max(max|x|, eps);  s = amax / 127;  q = (int8) trunc(clamp(x / s, -128, 127))
 */
void orc_group_quant_int8(const uint16_t *x, int64_t R, int64_t C, float eps,
                          int8_t *q, float *s) {
  int64_t G = C / ORC_GROUP;
#pragma omp parallel for schedule(static)
  for (int64_t g = 0; g < R * G; ++g) {
    const uint16_t *xg = x + g * ORC_GROUP;
    float amax = 0.0f;
    for (int i = 0; i < ORC_GROUP; ++i) {
      float a = fabsf(bf16_to_f32(xg[i]));
      if (a > amax) amax = a;
    }
    if (!(amax > eps)) amax = eps;
    float sc = amax / 127.0f;
    s[g] = sc;
    for (int i = 0; i < ORC_GROUP; ++i) {
      float v = bf16_to_f32(xg[i]) / sc;
      if (v < -128.0f) v = -128.0f;
      if (v > 127.0f) v = 127.0f;
      q[g * ORC_GROUP + i] = (int8_t)(int32_t)v; /* C cast truncates toward zero */
    }
  }
}

/* ------------------------------------------------------- grouped GEMM -- */

/*
 * One stage of the fused-MoE grouped GEMM (Triton fused_moe_kernel,
 * int8.py:320-541) in the block-quantised int8 form.
 *
 *   A   [*, K] int8, row of slot f is f / top_k;   As [*, K/128] f32
 *   W   [E, N, K] int8 (K contiguous);             Ws [E, ceil(N/128), K/128] f32
 *   C   [num_valid, N] bf16, row f
 *
 * For every block b < P/bs with e = expert_ids[b] and every row
 * f = sorted[b*bs + i] < num_valid:
 *   acc = 0;  for kb: d = sum_k A*W (int32, exact);
 *             t = f32(d) * As[row, kb];                               (int8.py:499-508)
 *             acc = fma(t, Ws[e, n/128, kb], acc)    contracted order (the default), or
 *             acc = acc + t * Ws[e, n/128, kb]       separate order (orc_set_scale_order(0))
 *   if mul_routed: acc = acc * topk_w[f]                              (int8.py:521-525)
 *   C[f, n] = bf16(acc);  e == -1 -> C[f, :] = 0                      (int8.py:441-449)
 *
 * acc_dump (optional, [num_valid, N, K/128] int32) receives the exact
 * per-128-block integer dot products, so that the integer part can be checked
 * on its own.
 */
/*
 * Order of the scale arithmetic per 128-wide K block.  The reference line is
 *   accumulator += tl.dot(a, b) * a_scale[:, None] * b_scale[None, :]      (int8.py:499-508)
 * and the kernel is compiled without an enable_fp_fusion override (launch at int8.py:596-626),
 * so Triton's AMD backend, whose default is enable_fp_fusion = True, lets LLVM contract the last
 * multiplication and the addition: acc = fma(f32(d) * a_s, b_s, acc), two roundings per K
 * block.  That contracted order is the default here (g_contract = 1).  The separate order,
 * acc = acc + (f32(d) * a_s) * b_s with three roundings, is what the same line gives with fp
 * fusion off; orc_set_scale_order(0) selects it.  The first multiplication feeds a multiplication,
 * not an addition, so it is never contracted.  A switch for the test harness, like the dtype's.
 */
static int g_contract = 1;
void orc_set_scale_order(int contract) { g_contract = contract; }

/* group_n = rows of W that share a scale: 128 (block-INT8) or 1 (one scale per row and K group) */
static void gemm_core(const int8_t *A, const float *As, const int8_t *W,
                      const float *Ws, const int32_t *sorted,
                      const int32_t *expert_ids,
                      const int32_t *num_tokens_post_pad,
                      const float *topk_w, int mul_routed, int32_t top_k,
                      int64_t num_valid, int64_t N, int64_t K, int32_t bs,
                      uint16_t *C, int32_t *acc_dump, int64_t group_n, float *Cf) {
  /* Cf != NULL: fp32 rows (compute_type tl.float32, int8.py:689-696: the sum is stored unrounded) */
  int64_t KB = K / ORC_GROUP;
  int64_t NB = (N + group_n - 1) / group_n;
  int64_t P = num_tokens_post_pad[0];
  int64_t nblk = P / bs;
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
  for (int64_t b = 0; b < nblk; ++b) {
    for (int32_t i = 0; i < bs; ++i) {
      int64_t f = sorted[b * bs + i];
      if (f >= num_valid) continue;
      int32_t e = expert_ids[b];
      uint16_t *c = Cf ? NULL : C + f * N;
      float *cf = Cf ? Cf + f * N : NULL;
      if (e < 0) {
        for (int64_t n = 0; n < N; ++n) {
          if (cf) cf[n] = 0.0f;
          else c[n] = 0;
        }
        continue;
      }
      int64_t row = f / top_k;
      const int8_t *a = A + row * K;
      const float *as = As + row * KB;
      const int8_t *w = W + (int64_t)e * N * K;
      const float *ws = Ws + (int64_t)e * NB * KB;
      for (int64_t n = 0; n < N; ++n) {
        const int8_t *wn = w + n * K;
        float acc = 0.0f;
        for (int64_t kb = 0; kb < KB; ++kb) {
          int32_t d = 0;
          for (int k = 0; k < ORC_GROUP; ++k)
            d += (int32_t)a[kb * ORC_GROUP + k] * (int32_t)wn[kb * ORC_GROUP + k];
          if (acc_dump) acc_dump[(f * N + n) * KB + kb] = d;
          float t = (float)d * as[kb];
          if (g_contract) {
            acc = fmaf(t, ws[(n / group_n) * KB + kb], acc);
          } else {
            t = t * ws[(n / group_n) * KB + kb];
            acc = acc + t;
          }
        }
        if (mul_routed) acc = acc * topk_w[f];
        if (cf) cf[n] = acc;
        else c[n] = f32_to_bf16(acc);
      }
    }
  }
}

void orc_moe_gemm_block_int8(const int8_t *A, const float *As, const int8_t *W,
                             const float *Ws, const int32_t *sorted,
                             const int32_t *expert_ids,
                             const int32_t *num_tokens_post_pad,
                             const float *topk_w, int mul_routed, int32_t top_k,
                             int64_t num_valid, int64_t N, int64_t K, int32_t bs,
                             uint16_t *C, int32_t *acc_dump) {
  gemm_core(A, As, W, Ws, sorted, expert_ids, num_tokens_post_pad, topk_w, mul_routed, top_k,
            num_valid, N, K, bs, C, acc_dump, ORC_GROUP, NULL);
}

/*
 * W4A8 with K-group scales: weights are signed 4-bit integers in [-8, 7], two per byte
 * along K, with one fp32 scale per output row and 128-wide K group: Ws [E, N, K/128].
 * Nibble order as in the reference's W4A8 kernel: element k of a row sits in byte k/2,
 * even k in the HIGH nibble, odd k in the LOW nibble
 * (python/lightop/_lmslim_native/layers/fused_moe/w4a8.py:341, :375-377).  The reference
 * itself scales per token and per channel in the epilogue only (w4a8.py:395); the K-group
 * form restated here has no reference implementation, so its parity is unpinned beyond the
 * arithmetic it shares with the block-INT8 path (both scale orders, see gemm_core):
 *   acc = fma(f32(sum_k A*w) * As[row, kb], Ws[e, n, kb], acc)
 */
void orc_unpack_int4(const uint8_t *packed, int64_t n_bytes, int8_t *out) {
  for (int64_t i = 0; i < n_bytes; ++i) {
    const int hi = packed[i] >> 4, lo = packed[i] & 15;
    out[2 * i] = (int8_t)(hi >= 8 ? hi - 16 : hi);
    out[2 * i + 1] = (int8_t)(lo >= 8 ? lo - 16 : lo);
  }
}

/* W here is already unpacked to int8 values in [-8, 7] (orc_unpack_int4) */
void orc_moe_gemm_rowscale_int8(const int8_t *A, const float *As, const int8_t *W,
                                const float *Ws, const int32_t *sorted,
                                const int32_t *expert_ids,
                                const int32_t *num_tokens_post_pad,
                                const float *topk_w, int mul_routed, int32_t top_k,
                                int64_t num_valid, int64_t N, int64_t K, int32_t bs,
                                uint16_t *C, int32_t *acc_dump) {
  gemm_core(A, As, W, Ws, sorted, expert_ids, num_tokens_post_pad, topk_w, mul_routed, top_k,
            num_valid, N, K, bs, C, acc_dump, 1, NULL);
}

/* ------------------------------------------------------------ SiLU*mul -- */

/*
 * expf restated with explicit single operations so that the same sequence can
 * be issued on any IEEE machine: n = rint(x*log2e), Cody-Waite reduction with
 * fmaf, degree-7 polynomial, exact scaling by 2^n.  tests/test_oracle.py checks
 * it against libm's expf (<= 1 ulp on the working range) and, exhaustively over
 * all 65536 bf16 inputs, that bf16(silu(x)) built on it equals the one built
 * on libm's expf.
 */
float orc_expf(float x) {
  if (x > 88.72283f) return INFINITY;
  if (x < -87.0f) return 0.0f; /* 1 + e == 1 for every e this small */
  float n = rintf(x * 1.44269504088896341f);
  float r = fmaf(n, -0.693145751953125f, x);
  r = fmaf(n, -1.42860682030941723212e-6f, r);
  float p = 1.9841270114e-4f;
  p = fmaf(p, r, 1.3888889225e-3f);
  p = fmaf(p, r, 8.3333337680e-3f);
  p = fmaf(p, r, 4.1666667908e-2f);
  p = fmaf(p, r, 1.6666667163e-1f);
  p = fmaf(p, r, 5.0000000000e-1f);
  p = fmaf(p, r, 1.0f);
  p = fmaf(p, r, 1.0f);
  /* scale by 2^n in two exact steps so that neither factor leaves the normal range */
  int32_t ni = (int32_t)n;
  int32_t h = ni / 2;
  union { uint32_t u; float f; } a, b;
  a.u = (uint32_t)(h + 127) << 23;
  b.u = (uint32_t)(ni - h + 127) << 23;
  return (p * a.f) * b.f;
}

/*
 * silu_and_mul on bf16 c1[S, 2I] -> act[S, I]:
 *   sg = bf16( g / (1 + expf(-g)) );  act = bf16( f32(sg) * u )
 * gate = first half, up = second half (fuse_silu_mul_quant.cu:893-905).
 */
static inline uint16_t silu_mul_one(uint16_t g16, uint16_t u16) {
  float g = bf16_to_f32(g16);
  float e = orc_expf(-g);
  float sg = bf16_to_f32(f32_to_bf16(g / (1.0f + e)));
  return f32_to_bf16(sg * bf16_to_f32(u16));
}

uint16_t orc_silu_bf16(uint16_t g16) {
  float g = bf16_to_f32(g16);
  return f32_to_bf16(g / (1.0f + orc_expf(-g)));
}

uint16_t orc_silu_bf16_libm(uint16_t g16) {
  float g = bf16_to_f32(g16);
  return f32_to_bf16(g / (1.0f + expf(-g)));
}

void orc_silu_and_mul(const uint16_t *c1, int64_t S, int64_t I, uint16_t *act) {
#pragma omp parallel for schedule(static)
  for (int64_t f = 0; f < S; ++f)
    for (int64_t i = 0; i < I; ++i)
      act[f * I + i] = silu_mul_one(c1[f * 2 * I + i], c1[f * 2 * I + I + i]);
}

/*
 * GELU-and-mul, the activation="gelu" branch (int8.py:825-827, w4a8.py:602-605), which calls
 * torch.ops._C.gelu_and_mul of vLLM (not part of the reference tree); the reference's in-repo
 * twin is gelu_and_mul_opt, csrc/kernels/activation_kernels_opt.cu:234-242 (gelu_kernel) and
 * :159-161 (the product, formed in the tensor's type):
 *   gelu(g) = T((f * 0.5f) * (1.0f + erf(f * ALPHA))),  f = float(g),  ALPHA = float(M_SQRT1_2)
 *   act     = T(float(gelu(g)) * float(u))
 * erf is a library routine there; the canonical choice here is erf correctly rounded to fp32
 * (libm's double-precision erf, rounded once more).  Where the reference's device erf differs
 * from that in its last place, the bf16 result can differ in its last place too: unpinned.
 * Pins (tests/test_oracle.py): closed-form values (gelu(0) = 0, gelu(x) = x for large x, -0 for
 * large negative x), the identity gelu(x) - gelu(-x) = x to rounding, torch's GELU on every
 * finite bf16 input within one bf16 ulp, monotonicity above the minimum.
 */
uint16_t orc_gelu_bf16(uint16_t g16) {
  const float f = bf16_to_f32(g16);
  const float alpha = 0.70710678118654752440f;
  const float e = (float)erf((double)(f * alpha));
  return f32_to_bf16((f * 0.5f) * (1.0f + e));
}

static inline uint16_t gelu_mul_one(uint16_t g16, uint16_t u16) {
  return f32_to_bf16(bf16_to_f32(orc_gelu_bf16(g16)) * bf16_to_f32(u16));
}

void orc_gelu_and_mul(const uint16_t *c1, int64_t S, int64_t I, uint16_t *act) {
#pragma omp parallel for schedule(static)
  for (int64_t f = 0; f < S; ++f)
    for (int64_t i = 0; i < I; ++i)
      act[f * I + i] = gelu_mul_one(c1[f * 2 * I + i], c1[f * 2 * I + I + i]);
}

/* Activation of the whole-path restatements below: 0 = SiLU (default), 1 = GELU.  A switch
 * for the test harness (one thread sets it around a call), not an argument, so that the
 * signatures of the chains stay what the existing callers use. */
static int g_activation = 0;
void orc_set_activation(int activation) { g_activation = activation; }

/* ------------------------------------------------------------ moe_sum -- */

/*
 * out[t, h] from in[M, k, H] bf16.
 *   bias == NULL: bf16( (sum_j f32(in[t,j,h])) * factor ), sequential j in fp32,
 *                 one rounding (moe_align_sum_kernels.cu:619-633).
 *   bias != NULL: x = bf16(sum); x = bf16(f32(x) * factor); x = bf16(f32(x) + f32(bias))
 *                 (moe_align_sum_kernels.cu:886-909).
 */
void orc_moe_sum(const uint16_t *in, int64_t M, int32_t k, int64_t H,
                 const uint16_t *bias, float factor, uint16_t *out) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < M; ++t)
    for (int64_t h = 0; h < H; ++h) {
      float acc = 0.0f;
      for (int32_t j = 0; j < k; ++j) acc = acc + bf16_to_f32(in[(t * k + j) * H + h]);
      if (!bias) {
        out[t * H + h] = f32_to_bf16(acc * factor);
      } else {
        uint16_t x = f32_to_bf16(acc);
        x = f32_to_bf16(bf16_to_f32(x) * factor);
        x = f32_to_bf16(bf16_to_f32(x) + bf16_to_f32(bias[t * H + h]));
        out[t * H + h] = x;
      }
    }
}

/* ------------------------------------------------------- whole path ---- */

/*
 * fused_experts_impl_int8 for one chunk (int8.py:703-888, with the final
 * reduce always performed).  Intermediates are returned when the pointers are
 * non-NULL so that each stage of the HIP path can be compared on its own:
 *   a1q[M,H] a1s[M,H/128]  c1[S,2I]  act[S,I]  a2q[S,I] a2s[S,I/128]  c3[S,H]
 * sorted/expert_ids/ntpp are outputs too (capacities as in
 * moe_align_block_size.py:80-93).  Returns 0 or -1.
 */
static int fused_path(
    const uint16_t *x, int64_t M, int64_t H, int64_t I, int32_t E_local,
    int32_t num_experts_global, int32_t top_k, const int8_t *w1, const float *w1s,
    const int8_t *w2, const float *w2s, const float *topk_w, const int32_t *topk_ids,
    const int32_t *expert_map, int32_t bs, int apply_router_weight_on_input,
    float routed_scaling_factor, const uint16_t *shared_output, uint16_t *out,
    int32_t *sorted, int64_t sorted_cap, int32_t *expert_ids, int64_t expert_ids_cap,
    int32_t *ntpp, int8_t *a1q, float *a1s, uint16_t *c1, uint16_t *act, int8_t *a2q,
    float *a2s, uint16_t *c3, int64_t group_n) {
  (void)E_local;
  int64_t S = M * top_k;
  int own_a1q = !a1q, own_a1s = !a1s, own_c1 = !c1, own_act = !act, own_a2q = !a2q,
      own_a2s = !a2s, own_c3 = !c3;
  if (own_a1q) a1q = (int8_t *)malloc((size_t)(M * H));
  if (own_a1s) a1s = (float *)malloc(sizeof(float) * (size_t)(M * (H / ORC_GROUP)));
  if (own_c1) c1 = (uint16_t *)calloc((size_t)(S * 2 * I), 2);
  if (own_act) act = (uint16_t *)malloc(2 * (size_t)(S * I));
  if (own_a2q) a2q = (int8_t *)malloc((size_t)(S * I));
  if (own_a2s) a2s = (float *)malloc(sizeof(float) * (size_t)(S * (I / ORC_GROUP)));
  if (own_c3) c3 = (uint16_t *)calloc((size_t)(S * H), 2);

  orc_group_quant_int8(x, M, H, 1e-10f, a1q, a1s);
  int rc = orc_moe_align_block_size(topk_ids, S, num_experts_global, bs, expert_map, 0,
                                    sorted, sorted_cap, expert_ids, expert_ids_cap, ntpp);
  if (rc == 0) {
    gemm_core(a1q, a1s, w1, w1s, sorted, expert_ids, ntpp, topk_w,
              apply_router_weight_on_input, top_k, S, 2 * I, H, bs, c1, NULL, group_n, NULL);
    if (g_activation == 1) orc_gelu_and_mul(c1, S, I, act);
    else orc_silu_and_mul(c1, S, I, act);
    orc_group_quant_int8(act, S, I, 1e-10f, a2q, a2s);
    gemm_core(a2q, a2s, w2, w2s, sorted, expert_ids, ntpp, topk_w,
              !apply_router_weight_on_input, 1, S, H, I, bs, c3, NULL, group_n, NULL);
    orc_moe_sum(c3, M, top_k, H, shared_output, routed_scaling_factor, out);
  }
  if (own_a1q) free(a1q);
  if (own_a1s) free(a1s);
  if (own_c1) free(c1);
  if (own_act) free(act);
  if (own_a2q) free(a2q);
  if (own_a2s) free(a2s);
  if (own_c3) free(c3);
  return rc;
}

int orc_fused_experts_block_int8(
    const uint16_t *x, int64_t M, int64_t H, int64_t I, int32_t E_local,
    int32_t num_experts_global, int32_t top_k, const int8_t *w1, const float *w1s,
    const int8_t *w2, const float *w2s, const float *topk_w, const int32_t *topk_ids,
    const int32_t *expert_map, int32_t bs, int apply_router_weight_on_input,
    float routed_scaling_factor, const uint16_t *shared_output, uint16_t *out,
    int32_t *sorted, int64_t sorted_cap, int32_t *expert_ids, int64_t expert_ids_cap,
    int32_t *ntpp, int8_t *a1q, float *a1s, uint16_t *c1, uint16_t *act, int8_t *a2q,
    float *a2s, uint16_t *c3) {
  return fused_path(x, M, H, I, E_local, num_experts_global, top_k, w1, w1s, w2, w2s, topk_w, topk_ids,
                    expert_map, bs, apply_router_weight_on_input, routed_scaling_factor, shared_output,
                    out, sorted, sorted_cap, expert_ids, expert_ids_cap, ntpp, a1q, a1s, c1, act, a2q, a2s,
                    c3, ORC_GROUP);
}

/* The same chain with W4A8 K-group weights: w1, w2 unpacked to int8 in [-8, 7]
 * (orc_unpack_int4), w1s [E, 2I, H/128], w2s [E, H, I/128]. */
int orc_fused_experts_w4a8(
    const uint16_t *x, int64_t M, int64_t H, int64_t I, int32_t E_local,
    int32_t num_experts_global, int32_t top_k, const int8_t *w1, const float *w1s,
    const int8_t *w2, const float *w2s, const float *topk_w, const int32_t *topk_ids,
    const int32_t *expert_map, int32_t bs, int apply_router_weight_on_input,
    float routed_scaling_factor, const uint16_t *shared_output, uint16_t *out,
    int32_t *sorted, int64_t sorted_cap, int32_t *expert_ids, int64_t expert_ids_cap,
    int32_t *ntpp, int8_t *a1q, float *a1s, uint16_t *c1, uint16_t *act, int8_t *a2q,
    float *a2s, uint16_t *c3) {
  return fused_path(x, M, H, I, E_local, num_experts_global, top_k, w1, w1s, w2, w2s, topk_w, topk_ids,
                    expert_map, bs, apply_router_weight_on_input, routed_scaling_factor, shared_output,
                    out, sorted, sorted_cap, expert_ids, expert_ids_cap, ntpp, a1q, a1s, c1, act, a2q, a2s,
                    c3, 1);
}

/* ------------------------------------------------------------------------- *
 * The block form with fp32 activations (hidden_states.dtype == torch.float32: compute_type
 * tl.float32, int8.py:689-696).  Nothing between the stages is rounded to 16 bits:
 *   quant     the same rule on fp32 inputs (int8_utils.py:74-122 widens to fp32 anyway)
 *   GEMM      C[f, n] = acc (the fp32 sum itself; with mul_routed acc * topk_w[f])
 *   SiLU*mul  act = (g / (1 + exp(-g))) * u in fp32 (vLLM's silu_and_mul, called at int8.py:811:
 *             T(float(x) / (1.0f + expf(float(-x)))) * y with T = float); exp is orc_expf, the
 *             fixed sequence of IEEE operations used for the 16-bit tables, so the last place of
 *             the reference's device expf is unpinned
 *   GELU*mul  act = ((g * 0.5f) * (1 + erf(g * ALPHA))) * u, erf correctly rounded (as above)
 *   moe_sum   sequential fp32 sum over the k slots, * factor, + bias
 *             (moe_align_sum_kernels.cu:619-633, :886-909 with T = float)
 * ------------------------------------------------------------------------- */
void orc_group_quant_int8_f32(const float *x, int64_t R, int64_t C, float eps, int8_t *q, float *s) {
  int64_t G = C / ORC_GROUP;
#pragma omp parallel for schedule(static)
  for (int64_t g = 0; g < R * G; ++g) {
    const float *xg = x + g * ORC_GROUP;
    float amax = 0.0f;
    for (int i = 0; i < ORC_GROUP; ++i) {
      float a = fabsf(xg[i]);
      if (a > amax) amax = a;
    }
    if (!(amax > eps)) amax = eps;
    float sc = amax / 127.0f;
    s[g] = sc;
    for (int i = 0; i < ORC_GROUP; ++i) {
      float v = xg[i] / sc;
      if (v < -128.0f) v = -128.0f;
      if (v > 127.0f) v = 127.0f;
      q[g * ORC_GROUP + i] = (int8_t)(int32_t)v;
    }
  }
}

void orc_moe_gemm_block_int8_f32(const int8_t *A, const float *As, const int8_t *W, const float *Ws,
                                 const int32_t *sorted, const int32_t *expert_ids,
                                 const int32_t *num_tokens_post_pad, const float *topk_w, int mul_routed,
                                 int32_t top_k, int64_t num_valid, int64_t N, int64_t K, int32_t bs, float *C,
                                 int32_t *acc_dump) {
  gemm_core(A, As, W, Ws, sorted, expert_ids, num_tokens_post_pad, topk_w, mul_routed, top_k, num_valid, N, K, bs,
            NULL, acc_dump, ORC_GROUP, C);
}

float orc_silu_f32(float g) { return g / (1.0f + orc_expf(-g)); }

float orc_gelu_f32(float g) {
  const float alpha = 0.70710678118654752440f;
  const float e = (float)erf((double)(g * alpha));
  return (g * 0.5f) * (1.0f + e);
}

void orc_act_and_mul_f32(const float *c1, int64_t S, int64_t I, int activation, float *act) {
#pragma omp parallel for schedule(static)
  for (int64_t f = 0; f < S; ++f)
    for (int64_t i = 0; i < I; ++i) {
      const float g = c1[f * 2 * I + i], u = c1[f * 2 * I + I + i];
      act[f * I + i] = (activation == 1 ? orc_gelu_f32(g) : orc_silu_f32(g)) * u;
    }
}

void orc_moe_sum_f32(const float *in, int64_t M, int32_t k, int64_t H, const float *bias, float factor,
                     float *out) {
#pragma omp parallel for schedule(static)
  for (int64_t t = 0; t < M; ++t)
    for (int64_t h = 0; h < H; ++h) {
      float acc = 0.0f;
      for (int32_t j = 0; j < k; ++j) acc = acc + in[(t * k + j) * H + h];
      acc = acc * factor;
      if (bias) acc = acc + bias[t * H + h];
      out[t * H + h] = acc;
    }
}

int orc_fused_experts_block_int8_f32(
    const float *x, int64_t M, int64_t H, int64_t I, int32_t E_local, int32_t num_experts_global, int32_t top_k,
    const int8_t *w1, const float *w1s, const int8_t *w2, const float *w2s, const float *topk_w,
    const int32_t *topk_ids, const int32_t *expert_map, int32_t bs, int apply_router_weight_on_input,
    float routed_scaling_factor, const float *shared_output, float *out, int32_t *sorted, int64_t sorted_cap,
    int32_t *expert_ids, int64_t expert_ids_cap, int32_t *ntpp, int8_t *a1q, float *a1s, float *c1, float *act,
    int8_t *a2q, float *a2s, float *c3) {
  (void)E_local;
  int64_t S = M * top_k;
  int own_a1q = !a1q, own_a1s = !a1s, own_c1 = !c1, own_act = !act, own_a2q = !a2q, own_a2s = !a2s, own_c3 = !c3;
  if (own_a1q) a1q = (int8_t *)malloc((size_t)(M * H));
  if (own_a1s) a1s = (float *)malloc(sizeof(float) * (size_t)(M * (H / ORC_GROUP)));
  if (own_c1) c1 = (float *)calloc((size_t)(S * 2 * I), 4);
  if (own_act) act = (float *)malloc(4 * (size_t)(S * I));
  if (own_a2q) a2q = (int8_t *)malloc((size_t)(S * I));
  if (own_a2s) a2s = (float *)malloc(sizeof(float) * (size_t)(S * (I / ORC_GROUP)));
  if (own_c3) c3 = (float *)calloc((size_t)(S * H), 4);
  orc_group_quant_int8_f32(x, M, H, 1e-10f, a1q, a1s);
  int rc = orc_moe_align_block_size(topk_ids, S, num_experts_global, bs, expert_map, 0, sorted, sorted_cap,
                                    expert_ids, expert_ids_cap, ntpp);
  if (rc == 0) {
    gemm_core(a1q, a1s, w1, w1s, sorted, expert_ids, ntpp, topk_w, apply_router_weight_on_input, top_k, S, 2 * I, H,
              bs, NULL, NULL, ORC_GROUP, c1);
    orc_act_and_mul_f32(c1, S, I, g_activation, act);
    orc_group_quant_int8_f32(act, S, I, 1e-10f, a2q, a2s);
    gemm_core(a2q, a2s, w2, w2s, sorted, expert_ids, ntpp, topk_w, !apply_router_weight_on_input, 1, S, H, I, bs,
              NULL, NULL, ORC_GROUP, c3);
    orc_moe_sum_f32(c3, M, top_k, H, shared_output, routed_scaling_factor, out);
  }
  if (own_a1q) free(a1q);
  if (own_a1s) free(a1s);
  if (own_c1) free(c1);
  if (own_act) free(act);
  if (own_a2q) free(a2q);
  if (own_a2s) free(a2s);
  if (own_c3) free(c3);
  return rc;
}

/* ------------------------------------------------------------------------- *
 * Per-channel W8A8 form of the same entry point (per_channel_quant=True,
 * block_shape=None): one scale per token row and one per weight row, applied
 * once after an exact whole-K int32 sum.
 *
 * Reference:
 *   per-token quant   python/lightop/_lmslim_native/layers/gemm/int8_utils.py:20-44
 *   grouped GEMM      csrc/moe_gemm/w8a8/moe_w8a8.cu:156-166 (first stage),
 *                     :445-470 (second stage, routed weight folded into the token scale);
 *                     call sites int8.py:771-781, :845-855; wrapper gemmopt.py:437-457
 *   SiLU*mul + quant  csrc/kernels/gated_activation/fuse_silu_mul_quant.cu:90-133
 *                     (round to nearest even, :19-35); call site int8.py:811-813
 *
 * Canonical choices: bf16(silu(g)) is the correctly rounded table used for the
 * block path (the reference kernel forms it from the hardware's approximate
 * exp2 and reciprocal, fuse_silu_mul_quant.cu:52-66; where the two differ in the
 * last bf16 ulp is unpinned); nearbyint is round-half-even.
 * ------------------------------------------------------------------------- */

static inline int8_t rne_int8(float v) {
  /* the reference's clamp, fuse_silu_mul_quant.cu:19-35: fminf(127, fmaxf(-128, x)), so a NaN
   * (0 * inf in a row of denormals, whose multiplier overflows) becomes -128 */
  v = fminf(127.0f, fmaxf(-128.0f, v));
  return (int8_t)(int32_t)nearbyintf(v); /* default rounding mode: half to even */
}

/* x[R, C] bf16 -> q[R, C] int8, s[R] f32:
 *   absmax = max(max|x|, 1e-10);  s = absmax / 127;  q = rne(x * (127 / absmax)) */
void orc_per_token_quant_int8(const uint16_t *x, int64_t R, int64_t C, int8_t *q, float *s) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < R; ++r) {
    const uint16_t *xr = x + r * C;
    float amax = 0.0f;
    for (int64_t i = 0; i < C; ++i) {
      float a = fabsf(bf16_to_f32(xr[i]));
      if (a > amax) amax = a;
    }
    if (!(amax > 1e-10f)) amax = 1e-10f;
    s[r] = amax / 127.0f;
    const float inv = 127.0f / amax;
    for (int64_t i = 0; i < C; ++i) q[r * C + i] = rne_int8(bf16_to_f32(xr[i]) * inv);
  }
}

/* c1[S, 2I] bf16 -> q[S, I] int8, s[S] f32 (fuse_silu_mul_quant.cu:90-133):
 *   act = bf16(f32(bf16(silu(g))) * u);  amax = max|act|;  s = amax / 127;
 *   q = rne(clamp(act * (amax == 0 ? 0 : 127 / amax)))
 * act (optional) receives the bf16 products. */
void orc_fuse_silu_mul_quant(const uint16_t *c1, int64_t S, int64_t I, int8_t *q, float *s,
                             uint16_t *act) {
#pragma omp parallel for schedule(static)
  for (int64_t f = 0; f < S; ++f) {
    float amax = 0.0f;
    for (int64_t i = 0; i < I; ++i) {
      float v = fabsf(bf16_to_f32(silu_mul_one(c1[f * 2 * I + i], c1[f * 2 * I + I + i])));
      if (v > amax) amax = v;
    }
    s[f] = amax / 127.0f;
    const float inv = (amax == 0.0f) ? 0.0f : 127.0f / amax;
    for (int64_t i = 0; i < I; ++i) {
      const uint16_t a16 = silu_mul_one(c1[f * 2 * I + i], c1[f * 2 * I + I + i]);
      if (act) act[f * I + i] = a16;
      q[f * I + i] = rne_int8(bf16_to_f32(a16) * inv);
    }
  }
}

/* Between the two stages of the per-channel chains: fuse_silu_mul_quant (int8.py:811-813), or
 * with GELU gelu_and_mul followed by per_token_quant_int8 (int8.py:825-838 through
 * moe_kernel_prepare_input's per-channel branch, int8.py:285-295; w4a8.py:602-605), whose
 * absmax has the 1e-10 floor that the fused SiLU kernel lacks. */
static void channel_act_quant(const uint16_t *c1, int64_t S, int64_t I, int8_t *q, float *s,
                              uint16_t *act) {
  if (g_activation != 1) {
    orc_fuse_silu_mul_quant(c1, S, I, q, s, act);
    return;
  }
  uint16_t *tmp = act ? act : (uint16_t *)malloc(2 * (size_t)(S * I));
  orc_gelu_and_mul(c1, S, I, tmp);
  orc_per_token_quant_int8(tmp, S, I, q, s);
  if (!act) free(tmp);
}

/*
 *   A [*, K] int8, row of slot f is f / top_k;  As [*] f32 (one per row)
 *   W [E, N, K] int8;                           Ws [E, N] f32 (one per weight row)
 *   d = sum_k A*W over the whole K (int32, exact)
 *   C[f, n] = bf16((f32(d) * ts) * Ws[e, n]),  ts = As[row], or topk_w[f] * As[row] with mul_routed
 *   e == -1 -> C[f, :] = 0 (moe_w8a8.cu:96-118)
 * acc_dump (optional, [num_valid, N] int32) receives d.
 */
void orc_moe_gemm_w8a8(const int8_t *A, const float *As, const int8_t *W, const float *Ws,
                       const int32_t *sorted, const int32_t *expert_ids,
                       const int32_t *num_tokens_post_pad, const float *topk_w, int mul_routed,
                       int32_t top_k, int64_t num_valid, int64_t N, int64_t K, int32_t bs,
                       uint16_t *C, int32_t *acc_dump) {
  int64_t P = num_tokens_post_pad[0];
  int64_t nblk = P / bs;
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
  for (int64_t b = 0; b < nblk; ++b) {
    for (int32_t i = 0; i < bs; ++i) {
      int64_t f = sorted[b * bs + i];
      if (f >= num_valid) continue;
      int32_t e = expert_ids[b];
      uint16_t *c = C + f * N;
      if (e < 0) {
        for (int64_t n = 0; n < N; ++n) c[n] = 0;
        continue;
      }
      int64_t row = f / top_k;
      const int8_t *a = A + row * K;
      float ts = As[row];
      if (mul_routed) ts = topk_w[f] * ts;
      for (int64_t n = 0; n < N; ++n) {
        const int8_t *wn = W + ((int64_t)e * N + n) * K;
        int32_t d = 0;
        for (int64_t k = 0; k < K; ++k) d += (int32_t)a[k] * (int32_t)wn[k];
        if (acc_dump) acc_dump[f * N + n] = d;
        float t = (float)d * ts;
        c[n] = f32_to_bf16(t * Ws[(int64_t)e * N + n]);
      }
    }
  }
}

/* The chain of int8.py:703-888 on its per-channel branch, with the final reduce always
 * performed: a1q[M,H] a1s[M]  c1[S,2I]  act[S,I]  a2q[S,I] a2s[S]  c3[S,H]. */
int orc_fused_experts_channel_int8(
    const uint16_t *x, int64_t M, int64_t H, int64_t I, int32_t E_local,
    int32_t num_experts_global, int32_t top_k, const int8_t *w1, const float *w1s,
    const int8_t *w2, const float *w2s, const float *topk_w, const int32_t *topk_ids,
    const int32_t *expert_map, int32_t bs, int apply_router_weight_on_input,
    float routed_scaling_factor, const uint16_t *shared_output, uint16_t *out,
    int32_t *sorted, int64_t sorted_cap, int32_t *expert_ids, int64_t expert_ids_cap,
    int32_t *ntpp, int8_t *a1q, float *a1s, uint16_t *c1, uint16_t *act, int8_t *a2q,
    float *a2s, uint16_t *c3) {
  (void)E_local;
  int64_t S = M * top_k;
  int own_a1q = !a1q, own_a1s = !a1s, own_c1 = !c1, own_a2q = !a2q, own_a2s = !a2s, own_c3 = !c3;
  if (own_a1q) a1q = (int8_t *)malloc((size_t)(M * H));
  if (own_a1s) a1s = (float *)malloc(sizeof(float) * (size_t)M);
  if (own_c1) c1 = (uint16_t *)calloc((size_t)(S * 2 * I), 2);
  if (own_a2q) a2q = (int8_t *)malloc((size_t)(S * I));
  if (own_a2s) a2s = (float *)malloc(sizeof(float) * (size_t)S);
  if (own_c3) c3 = (uint16_t *)calloc((size_t)(S * H), 2);
  orc_per_token_quant_int8(x, M, H, a1q, a1s);
  int rc = orc_moe_align_block_size(topk_ids, S, num_experts_global, bs, expert_map, 0,
                                    sorted, sorted_cap, expert_ids, expert_ids_cap, ntpp);
  if (rc == 0) {
    orc_moe_gemm_w8a8(a1q, a1s, w1, w1s, sorted, expert_ids, ntpp, topk_w,
                      apply_router_weight_on_input, top_k, S, 2 * I, H, bs, c1, NULL);
    channel_act_quant(c1, S, I, a2q, a2s, act);
    orc_moe_gemm_w8a8(a2q, a2s, w2, w2s, sorted, expert_ids, ntpp, topk_w,
                      !apply_router_weight_on_input, 1, S, H, I, bs, c3, NULL);
    orc_moe_sum(c3, M, top_k, H, shared_output, routed_scaling_factor, out);
  }
  if (own_a1q) free(a1q);
  if (own_a1s) free(a1s);
  if (own_c1) free(c1);
  if (own_a2q) free(a2q);
  if (own_a2s) free(a2s);
  if (own_c3) free(c3);
  return rc;
}

/* ------------------------------------------------------------------------- *
 * The reference's own W4A8 form: packed int4 weights, one scale per token row
 * and one per weight row, both applied in the epilogue.
 *
 * Reference: python/lightop/_lmslim_native/layers/fused_moe/w4a8.py
 *   kernel fused_moe_kernel_int4_w4a8 :202-401
 *     weight of element k of row n: byte k/2, shifted left by 4*(k%2) and masked with 0xF0
 *     (:341, :375-377), read as int8: the HIGH nibble for even k, the LOW one for odd k, each
 *     16 times the signed int4 it encodes
 *     accumulator (fp32) += dot(a, b) per K tile (:381)
 *     accumulator *= moe_weight when MUL_ROUTED_WEIGHT (:386-388)
 *     C = compute_type(accumulator * a_scale * b_scale), left to right (:395)
 *     expert -1: zeros (:326-333)
 *   host chain fused_experts_impl_w4a8 :480-658: per_token_quant_int8 -> align -> kernel ->
 *     fuse_silu_mul_quant -> kernel (routed weight, top_k = 1) -> moe_sum
 *
 * Every product is a multiple of 16 and so is every partial sum; below 2^28 in magnitude such
 * a number is exact in fp32, so while K * 128 * 127 < 2^28 (K <= 16512) the reference's fp32
 * running sum equals the exact integer sum whatever its K tile is.  The restatement sums in
 * int32 and converts once; beyond that K the reference's result depends on its tile choice and
 * this one is the exact sum.
 *
 * Parity pins (tests/test_oracle_w4a8.py): the nibble order and the factor 16 on hand-worked
 * bytes; the left-to-right scale order on operands chosen so that every other association
 * rounds differently; the whole stage against an independent numpy restatement that
 * dequantises first (exact in float64) and against orc_moe_gemm_w8a8 on weights pre-multiplied
 * to int8 (identical sums, a different scale order only where the routed weight enters).
 * ------------------------------------------------------------------------- */

/* Wp [E, N, K/2] bytes as the checkpoint packs them.  acc_dump (optional, [num_valid, N] int32)
 * receives the integer sums, factor 16 included. */
void orc_moe_gemm_w4a8_channel(const int8_t *A, const float *As, const uint8_t *Wp, const float *Ws,
                               const int32_t *sorted, const int32_t *expert_ids,
                               const int32_t *num_tokens_post_pad, const float *topk_w,
                               int mul_routed, int32_t top_k, int64_t num_valid, int64_t N,
                               int64_t K, int32_t bs, uint16_t *C, int32_t *acc_dump) {
  int64_t P = num_tokens_post_pad[0];
  int64_t nblk = P / bs;
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
  for (int64_t b = 0; b < nblk; ++b) {
    for (int32_t i = 0; i < bs; ++i) {
      int64_t f = sorted[b * bs + i];
      if (f >= num_valid) continue;
      int32_t e = expert_ids[b];
      uint16_t *c = C + f * N;
      if (e < 0) {
        for (int64_t n = 0; n < N; ++n) c[n] = 0;
        continue;
      }
      int64_t row = f / top_k;
      const int8_t *a = A + row * K;
      for (int64_t n = 0; n < N; ++n) {
        const uint8_t *wn = Wp + ((int64_t)e * N + n) * (K / 2);
        int32_t d = 0;
        for (int64_t k = 0; k < K; ++k) {
          const int8_t w = (int8_t)(uint8_t)((wn[k >> 1] << (4 * (k & 1))) & 0xF0);
          d += (int32_t)a[k] * (int32_t)w;
        }
        if (acc_dump) acc_dump[f * N + n] = d;
        float t = (float)d;
        if (mul_routed) t = t * topk_w[f];
        t = t * As[row];
        c[n] = f32_to_bf16(t * Ws[(int64_t)e * N + n]);
      }
    }
  }
}

/* Chain of w4a8.py:480-658 with the reduce always performed; buffers as in
 * orc_fused_experts_channel_int8, w1 [E, 2I, H/2] and w2 [E, H, I/2] packed bytes. */
int orc_fused_experts_w4a8_channel(
    const uint16_t *x, int64_t M, int64_t H, int64_t I, int32_t E_local,
    int32_t num_experts_global, int32_t top_k, const uint8_t *w1, const float *w1s,
    const uint8_t *w2, const float *w2s, const float *topk_w, const int32_t *topk_ids,
    const int32_t *expert_map, int32_t bs, int apply_router_weight_on_input,
    float routed_scaling_factor, const uint16_t *shared_output, uint16_t *out,
    int32_t *sorted, int64_t sorted_cap, int32_t *expert_ids, int64_t expert_ids_cap,
    int32_t *ntpp, int8_t *a1q, float *a1s, uint16_t *c1, uint16_t *act, int8_t *a2q,
    float *a2s, uint16_t *c3) {
  (void)E_local;
  int64_t S = M * top_k;
  int own_a1q = !a1q, own_a1s = !a1s, own_c1 = !c1, own_a2q = !a2q, own_a2s = !a2s, own_c3 = !c3;
  if (own_a1q) a1q = (int8_t *)malloc((size_t)(M * H));
  if (own_a1s) a1s = (float *)malloc(sizeof(float) * (size_t)M);
  if (own_c1) c1 = (uint16_t *)calloc((size_t)(S * 2 * I), 2);
  if (own_a2q) a2q = (int8_t *)malloc((size_t)(S * I));
  if (own_a2s) a2s = (float *)malloc(sizeof(float) * (size_t)S);
  if (own_c3) c3 = (uint16_t *)calloc((size_t)(S * H), 2);
  orc_per_token_quant_int8(x, M, H, a1q, a1s);
  int rc = orc_moe_align_block_size(topk_ids, S, num_experts_global, bs, expert_map, 0,
                                    sorted, sorted_cap, expert_ids, expert_ids_cap, ntpp);
  if (rc == 0) {
    orc_moe_gemm_w4a8_channel(a1q, a1s, w1, w1s, sorted, expert_ids, ntpp, topk_w,
                              apply_router_weight_on_input, top_k, S, 2 * I, H, bs, c1, NULL);
    channel_act_quant(c1, S, I, a2q, a2s, act);
    orc_moe_gemm_w4a8_channel(a2q, a2s, w2, w2s, sorted, expert_ids, ntpp, topk_w,
                              !apply_router_weight_on_input, 1, S, H, I, bs, c3, NULL);
    orc_moe_sum(c3, M, top_k, H, shared_output, routed_scaling_factor, out);
  }
  if (own_a1q) free(a1q);
  if (own_a1s) free(a1s);
  if (own_c1) free(c1);
  if (own_a2q) free(a2q);
  if (own_a2s) free(a2s);
  if (own_c3) free(c3);
  return rc;
}

/* ------------------------------------------------------------------------- *
 * Routers upstream of the path (they produce topk_ids / topk_weights).
 *
 * Reference: csrc/kernels/softmax/topk_softmax_kernels.cu:1381-1582 (generic
 * kernel; the reference's own test, test/test_softmax_topk.py:28-66, accepts
 * any winner among equal logits and weights within rtol 2e-5 / atol 2e-6) and
 * csrc/kernels/moe_gate/moe_fused_gate.cu:76-312 (grouped sigmoid top-k with
 * correction bias; test/ci_tests/test_fused_moe_gate.py:9-61 is its torch
 * restatement, compared at rtol = atol = 1e-6 after sorting by expert id).
 *
 * Canonical choices where the reference leaves the result open:
 *   - ties are won by the lower index (experts and groups), so the selection
 *     is a stable descending order;
 *   - exp is orc_expf;
 *   - the sum over the selected experts runs in selection order; the full-row
 *     softmax sum (renormalize = 0) is the 64-lane tree spelled out below.
 * Inputs are taken as fp32 (16-bit inputs are widened first, exactly).
 * ------------------------------------------------------------------------- */
#define ORC_NEG (-3.402823466e+38f)

/* Sum of p[0..E) the way 64 lanes do it: lane l adds p[l], p[l+64], ... in that
 * order, then six rounds of s[l] = s[l] + s[l ^ mask], mask = 1, 2, ..., 32. */
static float lane_tree_sum(const float *p, int32_t E) {
  float s[64], t[64];
  for (int l = 0; l < 64; ++l) {
    float a = 0.0f;
    for (int32_t i = l; i < E; i += 64) a = a + p[i];
    s[l] = a;
  }
  for (int mask = 1; mask < 64; mask <<= 1) {
    for (int l = 0; l < 64; ++l) t[l] = s[l] + s[l ^ mask];
    memcpy(s, t, sizeof(s));
  }
  return s[0];
}

/* index of the largest v[i] (lowest index among equals), or -1 if E == 0 */
static int32_t argmax_low(const float *v, int32_t E) {
  int32_t best = -1;
  float bv = 0.0f;
  for (int32_t i = 0; i < E; ++i)
    if (best < 0 || v[i] > bv) { best = i; bv = v[i]; }
  return best;
}

/*
 * gating[T, E] fp32 -> weights[T, k] fp32, indices[T, k] int32,
 * source_rows[T, k] int32 (optional) = j * T + t.
 */
int orc_topk_softmax(const float *gating, int64_t T, int32_t E, int32_t k, int renormalize,
                     float *weights, int32_t *indices, int32_t *source_rows) {
  if (E < 1 || k < 1 || k > E) return -1;
  float *v = (float *)malloc(sizeof(float) * (size_t)E);
  float *p = (float *)malloc(sizeof(float) * (size_t)E);
  if (!v || !p) { free(v); free(p); return -2; }
  for (int64_t t = 0; t < T; ++t) {
    const float *x = gating + t * E;
    float mx = x[0];
    for (int32_t i = 1; i < E; ++i) if (x[i] > mx) mx = x[i];
    float scale = 0.0f;
    if (renormalize) {
      memcpy(v, x, sizeof(float) * (size_t)E);
    } else {
      for (int32_t i = 0; i < E; ++i) p[i] = orc_expf(x[i] - mx);
      scale = 1.0f / (lane_tree_sum(p, E) + 1e-6f);
      memcpy(v, p, sizeof(float) * (size_t)E);
    }
    float sum = 0.0f;
    for (int32_t j = 0; j < k; ++j) {
      const int32_t w = argmax_low(v, E);
      const float val = renormalize ? orc_expf(v[w] - mx) : v[w];
      v[w] = ORC_NEG;
      weights[t * k + j] = val;
      indices[t * k + j] = w;
      sum = sum + val;
      if (source_rows) source_rows[t * k + j] = (int32_t)(j * T + t);
    }
    if (renormalize) scale = 1.0f / (sum + 1e-6f);
    for (int32_t j = 0; j < k; ++j) weights[t * k + j] = weights[t * k + j] * scale;
  }
  free(v);
  free(p);
  return 0;
}

/*
 * input[T, E], bias[E] fp32 -> weights[T, topk] fp32, indices[T, topk] int32.
 * s = 1 / (1 + exp(-x));  c = bias + s;  group score = two largest c of the group added;
 * the topk_group best groups stay; the topk - n_share best c among them are selected;
 * weight = s of the selected / their sum (selection order) * route scale; the shared
 * experts E, E+1, ... follow with weight (sum / rsf) / sum * route scale.
 */
int orc_moe_fused_gate(const float *input, const float *bias, int64_t T, int32_t E,
                       int32_t num_expert_group, int32_t topk_group, int32_t topk,
                       int32_t n_share, double routed_scaling_factor, int apply_on_output,
                       float *weights, int32_t *indices) {
  const int32_t G = num_expert_group;
  if (E < 1 || G < 1 || E % G || topk_group < 1 || topk_group > G || n_share < 0 || topk - n_share < 1)
    return -1;
  const int32_t gs = E / G, kr = topk - n_share;
  if (kr > topk_group * gs) return -1;
  float *s = (float *)malloc(sizeof(float) * (size_t)E);
  float *c = (float *)malloc(sizeof(float) * (size_t)E);
  float *gsc = (float *)malloc(sizeof(float) * (size_t)G);
  char *keep = (char *)malloc((size_t)G);
  if (!s || !c || !gsc || !keep) { free(s); free(c); free(gsc); free(keep); return -2; }
  const float rsf = (float)routed_scaling_factor;
  const float route_scale = (apply_on_output && routed_scaling_factor > 0.0) ? rsf : 1.0f;
  for (int64_t t = 0; t < T; ++t) {
    const float *x = input + t * E;
    for (int32_t i = 0; i < E; ++i) {
      s[i] = 1.0f / (1.0f + orc_expf(-x[i]));
      c[i] = bias[i] + s[i];
    }
    for (int32_t g = 0; g < G; ++g) {
      float t1 = ORC_NEG, t2 = ORC_NEG;
      for (int32_t i = g * gs; i < (g + 1) * gs; ++i) {
        if (c[i] > t1) { t2 = t1; t1 = c[i]; }
        else if (c[i] > t2) t2 = c[i];
      }
      gsc[g] = t1 + t2;
      keep[g] = 0;
    }
    for (int32_t r = 0; r < topk_group; ++r) {
      const int32_t w = argmax_low(gsc, G);
      keep[w] = 1;
      gsc[w] = ORC_NEG;
    }
    for (int32_t i = 0; i < E; ++i) if (!keep[i / gs]) c[i] = ORC_NEG;
    float sum = 0.0f;
    for (int32_t j = 0; j < kr; ++j) {
      const int32_t w = argmax_low(c, E);
      c[w] = ORC_NEG;
      weights[t * topk + j] = s[w];
      indices[t * topk + j] = w;
      sum = sum + s[w];
    }
    for (int32_t j = kr; j < topk; ++j) {
      weights[t * topk + j] = sum / (routed_scaling_factor > 0.0 ? rsf : 1.0f);
      indices[t * topk + j] = E + (j - kr);
    }
    for (int32_t j = 0; j < topk; ++j) weights[t * topk + j] = (weights[t * topk + j] / sum) * route_scale;
  }
  free(s); free(c); free(gsc); free(keep);
  return 0;
}
