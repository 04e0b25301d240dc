// Shared device/host helpers of the gfx950 block-INT8 fused-MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/lightop_mi355.h"

namespace lo {

constexpr int kWave = 64;   // CDNA wavefront
constexpr int kGroup = 128; // quantisation group along K and weight block edge

// Order of the 2 KB blocks (16 rows x 128 K-bytes) of a pre-shuffled expert weight:
// K-block-major, i.e. [K/128][N/16]: the blocks that neighbouring waves read at the same
// step of their K loops are contiguous in memory.  (Row-block-major order puts them
// K*16 bytes apart, which for K = 2048 is a 32 KB stride and piles the concurrent reads
// onto a few memory channels.)
#ifndef LO_SHUF_KB_MAJOR
#define LO_SHUF_KB_MAJOR 1
#endif
// byte offset of block (row block nb, K block kb) inside one expert
__host__ __device__ __forceinline__ int64_t shuf_block_off(int64_t nb, int64_t kb, int64_t NBLK, int64_t KB) {
  return (LO_SHUF_KB_MAJOR ? kb * NBLK + nb : nb * KB + kb) * 2048;
}
// the two strides of that formula, for kernels that advance kb with a scalar offset
__host__ __device__ __forceinline__ int shuf_nb_stride(int KB) { return LO_SHUF_KB_MAJOR ? 2048 : KB * 2048; }
__host__ __device__ __forceinline__ int shuf_kb_stride(int NBLK) { return LO_SHUF_KB_MAJOR ? NBLK * 2048 : 2048; }

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short v4u16 __attribute__((ext_vector_type(4)));
typedef unsigned short v8u16 __attribute__((ext_vector_type(8)));

// ---- error reporting (host) -------------------------------------------------
void set_error(const char *fmt, ...);
int check_launch(const char *what);
// bf16(silu(g)) for all 65536 bf16 patterns g, built on first use (per device).
int silu_table(hipStream_t stream, const uint16_t **table);
// T(act(g)) for all 65536 patterns g of the 16-bit type T (LO_BF16 / LO_F16), act = LO_ACT_SILU / LO_ACT_GELU.
int act_table(hipStream_t stream, int act, int dtype, const uint16_t **table);
// The gated activation of c1 [rows, 2I] from its table, followed by the 1x128 group quantisation
// (q [rows, I], s [rows, I/128]) or by the per-token quantisation (s [rows]; SiLU without a floor
// under the row maximum, as fuse_silu_mul_quant, GELU with per_token_quant_int8's), one launch each.
// row_mask (optional, [rows] bytes): rows whose byte is 0 are skipped.
int launch_act_mul_group_quant(const void *c1, int dtype, int act, int64_t rows, int64_t I, int8_t *q, float *s,
                               const uint8_t *row_mask, hipStream_t stream);
// fp32 rows (elementwise_f32.hip)
int launch_group_quant_f32(const float *x, int64_t groups, float eps, int8_t *q, float *s, hipStream_t stream);
int launch_act_mul_f32(const float *c1, int64_t rows, int64_t I, int act, float *out, hipStream_t stream);
int launch_act_mul_group_quant_f32(const float *c1, int act, int64_t rows, int64_t I, int8_t *q, float *s,
                                   const uint8_t *row_mask, hipStream_t stream);
int launch_moe_sum_f32(const float *in, float *out, const float *bias, const uint8_t *mask, int64_t M, int32_t topk,
                       int64_t H, float factor, const int32_t *num_local_tokens, hipStream_t stream);
int launch_act_mul_row_quant(const void *c1, int dtype, int act, int64_t rows, int64_t I, int8_t *q, float *s,
                             const int32_t *num_local_tokens, int32_t top_k, const int32_t *row_ids,
                             hipStream_t stream);

// Raises a kernel's dynamic-LDS limit once per device instead of on every launch (kernels that use
// more than the default 64 KB).  `done` is the call site's own static flag set, one bit per device.
int reserve_lds_once(const void *kernel, int bytes, unsigned long long *done);

#define LO_REQUIRE(cond, code, ...)  \
  do {                               \
    if (!(cond)) {                   \
      ::lo::set_error(__VA_ARGS__);  \
      return (code);                 \
    }                                \
  } while (0)

// ---- 16-bit float helpers (device) ------------------------------------------
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// Round-to-nearest-even (gfx950 has the conversion in hardware: v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

__device__ __forceinline__ float f16_to_f32(uint16_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, h));
}
// The conversion is kept opaque: written as a cast, the compiler folds a preceding fp32
// multiplication into v_fma_mixlo_f16 (a * b + 0 rounded straight to half), which rounds once where
// the definition rounds twice and turns a -0 product into +0.
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  uint32_t r;
  asm("v_cvt_f16_f32 %0, %1" : "=v"(r) : "v"(f));
  return static_cast<uint16_t>(r);
}

template <int DT> __device__ __forceinline__ float to_f32(uint16_t h) {
  if constexpr (DT == LO_BF16) return bf16_to_f32(h);
  else return f16_to_f32(h);
}
template <int DT> __device__ __forceinline__ uint16_t from_f32(float f) {
  if constexpr (DT == LO_BF16) return f32_to_bf16(f);
  else return f32_to_f16(f);
}

// exp(x) as a fixed sequence of IEEE single operations (Cody-Waite reduction,
// degree-7 polynomial, exact power-of-two scaling), so that the result does not
// depend on a math library.  Used for SiLU: g / (1 + exp(-g)).
__device__ __forceinline__ float det_expf(float x) {
  const float x_in = x;
  x = fminf(fmaxf(x, -87.0f), 88.72283f); // straight-line code: the ends are patched below
  float n = __builtin_rintf(x * 1.44269504088896341f);
  float r = __builtin_fmaf(n, -0.693145751953125f, x);
  r = __builtin_fmaf(n, -1.42860682030941723212e-6f, r);
  float p = 1.9841270114e-4f;
  p = __builtin_fmaf(p, r, 1.3888889225e-3f);
  p = __builtin_fmaf(p, r, 8.3333337680e-3f);
  p = __builtin_fmaf(p, r, 4.1666667908e-2f);
  p = __builtin_fmaf(p, r, 1.6666667163e-1f);
  p = __builtin_fmaf(p, r, 5.0000000000e-1f);
  p = __builtin_fmaf(p, r, 1.0f);
  p = __builtin_fmaf(p, r, 1.0f);
  int ni = static_cast<int>(n);
  int h = ni / 2;
  float a = __uint_as_float(static_cast<uint32_t>(h + 127) << 23);
  float b = __uint_as_float(static_cast<uint32_t>(ni - h + 127) << 23);
  float e = (p * a) * b;
  e = x_in > 88.72283f ? __uint_as_float(0x7f800000u) : e;
  return x_in < -87.0f ? 0.0f : e;
}

// act = T( T(silu(g)) * u ), everything in fp32 between the roundings.
template <int DT> __device__ __forceinline__ uint16_t silu_mul(uint16_t g16, uint16_t u16) {
  float g = to_f32<DT>(g16);
  float e = det_expf(-g);
  float sg = to_f32<DT>(from_f32<DT>(g / (1.0f + e)));
  return from_f32<DT>(sg * to_f32<DT>(u16));
}

// Same with the SiLU taken from the per-device table.
__device__ __forceinline__ uint16_t silu_mul_tab(const uint16_t *__restrict__ table, uint16_t g16, uint16_t u16) {
  const float sg = bf16_to_f32(table[g16]);
  return f32_to_bf16(sg * bf16_to_f32(u16));
}

// Any gated activation whose T(act(g)) sits in a 64K-entry table: act = T(T(act(g)) * u).
template <int DT>
__device__ __forceinline__ uint16_t act_mul_tab(const uint16_t *__restrict__ table, uint16_t g16, uint16_t u16) {
  return from_f32<DT>(to_f32<DT>(table[g16]) * to_f32<DT>(u16));
}

// bf16(silu(g)) has closed forms outside a narrow band of inputs: for |g| <= 0x3bb5 (about
// 0.0055) it is bf16(g / 2), for g >= 0x40bf (about 5.97) it is g, for finite g <= 0xc2b2
// (about -89) it is -0.  The band in between, 1788 patterns per sign, fits in LDS; NaN and
// -inf go to the full table.  (The bounds come from the full table itself; a test drives
// every finite bf16 gate through the kernels that use this.)
constexpr int kSiluBandLo = 0x3bb6, kSiluBandN = 1788; // band = [lo, lo + n) on |g|
// The band travels global -> registers early (kSiluBandPer values per thread of a 256-thread
// workgroup) and registers -> LDS before the workgroup's first barrier.
constexpr int kSiluBandPer = (2 * kSiluBandN + 255) / 256;
__device__ __forceinline__ void silu_band_load(uint16_t (&regs)[kSiluBandPer], const uint16_t *__restrict__ table, int tid) {
#pragma unroll
  for (int j = 0; j < kSiluBandPer; ++j) {
    int i = tid + 256 * j;
    i = i < 2 * kSiluBandN ? i : 2 * kSiluBandN - 1;
    const int sign = i >= kSiluBandN;
    regs[j] = table[(sign ? 0x8000 : 0) + kSiluBandLo + (i - sign * kSiluBandN)];
  }
}
__device__ __forceinline__ void silu_band_store(uint16_t *band, const uint16_t (&regs)[kSiluBandPer], int tid) {
#pragma unroll
  for (int j = 0; j < kSiluBandPer; ++j) {
    const int i = tid + 256 * j;
    if (i < 2 * kSiluBandN) band[i] = regs[j];
  }
}
__device__ __forceinline__ uint16_t silu_mul_band(const uint16_t *band, const uint16_t *__restrict__ table,
                                                  uint16_t g16, uint16_t u16) {
  const uint32_t mag = g16 & 0x7fffu, neg = g16 >> 15;
  const uint32_t bi = mag - kSiluBandLo;
  uint16_t sg16;
  if (bi < static_cast<uint32_t>(kSiluBandN)) {
    sg16 = band[bi + neg * kSiluBandN];
  } else if (mag < static_cast<uint32_t>(kSiluBandLo)) {
    sg16 = f32_to_bf16(bf16_to_f32(g16) * 0.5f);
  } else if (mag > 0x7f80u || g16 == 0xff80u) {
    sg16 = table[g16]; // NaN, -inf
  } else {
    sg16 = neg ? static_cast<uint16_t>(0x8000u) : g16;
  }
  return f32_to_bf16(bf16_to_f32(sg16) * bf16_to_f32(u16));
}

// The same lookup as straight-line code, for epilogues that push dozens of unrelated values per
// lane through it: lanes of a wave never agree on an arm, so per-value branches only add
// exec-mask bookkeeping and keep the LDS reads from being issued back to back.  The three
// common arms are computed and selected; NaN and -inf gates are NOT handled here: the caller
// ORs silu_gate_special() over its values and, if any lane of the wave saw one, redoes the
// values with silu_mul_band().
__device__ __forceinline__ uint16_t silu_mul_band_common(const uint16_t *band, uint16_t g16, uint16_t u16) {
  const uint32_t mag = g16 & 0x7fffu, neg = g16 >> 15;
  const uint32_t bi = mag - kSiluBandLo; // wraps around below the band
  const bool inside = bi < static_cast<uint32_t>(kSiluBandN);
  const uint16_t in_band = band[(inside ? bi : 0u) + neg * kSiluBandN];
  const uint16_t below = f32_to_bf16(bf16_to_f32(g16) * 0.5f);
  const uint16_t above = neg ? static_cast<uint16_t>(0x8000u) : g16;
  const uint16_t sg16 = inside ? in_band : (mag < static_cast<uint32_t>(kSiluBandLo) ? below : above);
  return f32_to_bf16(bf16_to_f32(sg16) * bf16_to_f32(u16));
}
__device__ __forceinline__ bool silu_gate_special(uint16_t g16) {
  return (g16 & 0x7fffu) > 0x7f80u || g16 == 0xff80u; // NaN, -inf
}

// q = (int8) trunc(clamp(v / s, -128, 127))
__device__ __forceinline__ int quant_one(float v, float s) {
  float t = v / s;
  t = fmaxf(t, -128.0f);
  t = fminf(t, 127.0f);
  return static_cast<int>(t);
}

// The same value as quant_one(v, s) from y = 1.0f / s (one IEEE division per row instead of
// one per element): q = RN(v*y) is within an ulp of v/s, the remainder v - q*s is exact in
// a fused multiply-add, and RN(q + rem*y) is then the correctly rounded quotient (Markstein's
// theorem, valid for a correctly rounded reciprocal and no under/overflow).  Quotients
// of denormal magnitude may differ in the last bit; they truncate to 0 either way.  Not
// valid for s = inf (a row that holds an infinity): callers take quant_one then.
__device__ __forceinline__ int quant_one_rcp(float v, float s, float y) {
  const float q = v * y;
  const float rem = __builtin_fmaf(-q, s, v);
  float t = __builtin_fmaf(rem, y, q);
  t = fmaxf(t, -128.0f);
  t = fminf(t, 127.0f);
  return static_cast<int>(t);
}

__device__ __forceinline__ uint32_t pack4_i8(int a, int b, int c, int d) {
  return (static_cast<uint32_t>(a) & 0xffu) | ((static_cast<uint32_t>(b) & 0xffu) << 8) |
         ((static_cast<uint32_t>(c) & 0xffu) << 16) | ((static_cast<uint32_t>(d) & 0xffu) << 24);
}

// four elements of one row -> four packed int8; y = 1.0f / s
__device__ __forceinline__ uint32_t quant4(const float *v, float s, float y) {
  if (s < __builtin_inff()) {
    return pack4_i8(quant_one_rcp(v[0], s, y), quant_one_rcp(v[1], s, y), quant_one_rcp(v[2], s, y),
                    quant_one_rcp(v[3], s, y));
  }
  return pack4_i8(quant_one(v[0], s), quant_one(v[1], s), quant_one(v[2], s), quant_one(v[3], s));
}

// per_token_group_quant_int8 for the groups g = first + i * stride (reference:
// python/lightop/_lmslim_native/layers/gemm/int8_utils.py:74-122).  16 lanes own one group of
// 128 values (8 each); amax is reduced across those 16 lanes; the division is IEEE.
template <int DT>
__device__ __forceinline__ void group_quant_body(const uint16_t *__restrict__ x, int64_t groups, float eps,
                                                 int8_t *__restrict__ q, float *__restrict__ s, int64_t first,
                                                 int64_t stride, int sub) {
  for (int64_t g = first; g < groups; g += stride) {
    const v8u16 raw = *reinterpret_cast<const v8u16 *>(x + g * kGroup + sub * 8);
    float v[8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = to_f32<DT>(raw[i]);
      amax = fmaxf(amax, fabsf(v[i]));
    }
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
    amax = fmaxf(amax, eps);
    const float sc = amax / 127.0f;
    // one IEEE reciprocal per group, then the correctly rounded quotient per value (quant4)
    const float rsc = 1.0f / sc;
    v2i packed;
    packed[0] = static_cast<int>(quant4(&v[0], sc, rsc));
    packed[1] = static_cast<int>(quant4(&v[4], sc, rsc));
    *reinterpret_cast<v2i *>(q + g * kGroup + sub * 8) = packed;
    if (sub == 0) s[g] = sc;
  }
}

// Group quant of x [M, H] and the routing alignment with the quantisation riding in the
// alignment's (first) launch: they are independent, and at decode sizes a launch costs as much
// as either.  scratch: the multi-workgroup alignment's counters (lo_moe_align_scratch_bytes);
// returns LO_ENOTSUP when they are needed and missing - the caller then launches the two stages
// separately.
int launch_quant_align(const void *x, int64_t M, int64_t H, float eps, int8_t *q, float *s,
                       const void *topk_ids, int ids_dtype, int64_t numel, int32_t num_experts,
                       int32_t block_size, const int32_t *expert_map, int32_t *sorted_ids, int64_t sorted_cap,
                       int32_t *expert_ids, int64_t expert_ids_cap, int32_t *num_tokens_post_pad,
                       uint8_t *slot_mask, void *scratch, int64_t scratch_bytes, hipStream_t stream);

} // namespace lo
