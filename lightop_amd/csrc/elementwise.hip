// Streaming stages of the block-INT8 fused-MoE path on gfx950: 1x128 group
// quantisation, SiLU-and-mul, and the top-k reduction.  All are HBM-bound; every
// lane moves 16 bytes per load and a workgroup covers whole 128-element groups.
#include <mutex>

#include "common.h"

namespace lo {

// ---- per_token_group_quant_int8 ----------------------------------------------
// Reference: python/lightop/_lmslim_native/layers/gemm/int8_utils.py:74-122; the body is
// group_quant_body (common.h), shared with the fused quant + alignment launch.
template <int DT>
__global__ __launch_bounds__(256) void group_quant_kernel(const uint16_t *__restrict__ x,
                                                          int64_t groups, float eps,
                                                          int8_t *__restrict__ q,
                                                          float *__restrict__ s) {
  group_quant_body<DT>(x, groups, eps, q, s, static_cast<int64_t>(blockIdx.x) * 16 + (threadIdx.x >> 4),
                       static_cast<int64_t>(gridDim.x) * 16, threadIdx.x & 15);
}

// ---- silu_and_mul --------------------------------------------------------------
// Reference: torch.ops._C.silu_and_mul as called at int8.py:811; in-repo twin
// csrc/kernels/gated_activation/fuse_silu_mul_quant.cu:893-905.
template <int DT>
__global__ __launch_bounds__(256) void silu_mul_kernel(const uint16_t *__restrict__ c1,
                                                       int64_t rows, int64_t I,
                                                       uint16_t *__restrict__ act) {
  const int64_t vec_per_row = I / 8;
  const int64_t total = rows * vec_per_row;
  for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < total;
       v += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = v / vec_per_row, c = (v % vec_per_row) * 8;
    const v8u16 g = *reinterpret_cast<const v8u16 *>(c1 + r * 2 * I + c);
    const v8u16 u = *reinterpret_cast<const v8u16 *>(c1 + r * 2 * I + I + c);
    v8u16 o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = silu_mul<DT>(g[i], u[i]);
    *reinterpret_cast<v8u16 *>(act + r * I + c) = o;
  }
}

// ---- gelu_and_mul ----------------------------------------------------------------
// Reference: torch.ops._C.gelu_and_mul as called at int8.py:826; in-repo twin gelu_and_mul_opt,
// csrc/kernels/activation_kernels_opt.cu:234-242 (erf form) and :159-161 (product in the tensor's
// type): act = T(T(gelu(g)) * u).  T(gelu(g)) comes from a 64K-entry table (act_table below); the
// kernel serves any gated activation that has one.
template <int DT>
__global__ __launch_bounds__(256) void act_mul_tab_kernel(const uint16_t *__restrict__ c1, int64_t rows, int64_t I,
                                                          const uint16_t *__restrict__ table,
                                                          uint16_t *__restrict__ act) {
  const int64_t vec_per_row = I / 8;
  const int64_t total = rows * vec_per_row;
  for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < total;
       v += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t r = v / vec_per_row, c = (v % vec_per_row) * 8;
    const v8u16 g = *reinterpret_cast<const v8u16 *>(c1 + r * 2 * I + c);
    const v8u16 u = *reinterpret_cast<const v8u16 *>(c1 + r * 2 * I + I + c);
    v8u16 o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = act_mul_tab<DT>(table, g[i], u[i]);
    *reinterpret_cast<v8u16 *>(act + r * I + c) = o;
  }
}

// The same followed by the 1x128 group quantisation of per_token_group_quant_int8 (the pair of
// calls at int8.py:826-838 on the block-shape branch) in one pass: c1 [rows, 2I] -> q [rows, I],
// s [rows, I/128].  16 lanes own one group, as in group_quant_body.
template <int DT>
__global__ __launch_bounds__(256) void act_mul_group_quant_kernel(const uint16_t *__restrict__ c1, int64_t rows,
                                                                  int64_t I, const uint16_t *__restrict__ table,
                                                                  float eps, int8_t *__restrict__ q,
                                                                  float *__restrict__ s,
                                                                  const uint8_t *__restrict__ row_mask) {
  const int64_t gpr = I / kGroup, groups = rows * gpr;
  const int sub = threadIdx.x & 15;
  for (int64_t g = static_cast<int64_t>(blockIdx.x) * 16 + (threadIdx.x >> 4); g < groups;
       g += static_cast<int64_t>(gridDim.x) * 16) {
    const int64_t r = g / gpr, c = (g % gpr) * kGroup + sub * 8;
    if (row_mask && !row_mask[r]) continue; // a slot of an expert held elsewhere: nobody reads its row
    const v8u16 ga = *reinterpret_cast<const v8u16 *>(c1 + r * 2 * I + c);
    const v8u16 up = *reinterpret_cast<const v8u16 *>(c1 + r * 2 * I + I + c);
    float v[8];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = to_f32<DT>(act_mul_tab<DT>(table, ga[i], up[i]));
      amax = fmaxf(amax, fabsf(v[i]));
    }
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
    amax = fmaxf(amax, eps);
    const float sc = amax / 127.0f;
    const float rsc = 1.0f / sc;
    v2i packed;
    packed[0] = static_cast<int>(quant4(&v[0], sc, rsc));
    packed[1] = static_cast<int>(quant4(&v[4], sc, rsc));
    *reinterpret_cast<v2i *>(q + r * I + c) = packed;
    if (sub == 0) s[g] = sc;
  }
}

// ---- per-token int8 quantisation, plain and behind SiLU-and-mul ----------------------
// Reference: per_token_quant_int8, python/lightop/_lmslim_native/layers/gemm/int8_utils.py:20-44
// (amax floored at 1e-10, s = amax / 127, q = rne(x * (127 / amax))) and fuse_silu_mul_quant,
// csrc/kernels/gated_activation/fuse_silu_mul_quant.cu:90-133 (act = bf16(bf16(silu(g)) * u),
// no floor: a zero row gets scale 0 and multiplier 0).  One workgroup per row; a thread keeps
// up to CH 8-value pieces of the row in registers between the amax pass and the rounding pass,
// longer rows are read a second time.
// ACT: 0 plain rows; 1 SiLU-and-mul first (the fused kernel above: no floor), bf16 only, through the
// band of the SiLU table; 2 a gated activation from its full table first (`silu` being that table),
// then per_token_quant_int8 with its floor (GELU: the two calls at int8.py:826-838 on the per-channel
// branch); 3 as 2 without the floor (SiLU for fp16 rows, which have no band).
__device__ __forceinline__ int rne_i8(float v) {
  v = fminf(fmaxf(v, -128.0f), 127.0f);
  return static_cast<int>(__builtin_rintf(v)); // v_rndne_f32: ties to even
}

template <int ACT, int CH, int DT>
__global__ __launch_bounds__(256) void row_quant_kernel(const uint16_t *__restrict__ x, int64_t rows, int64_t C,
                                                        const uint16_t *__restrict__ silu, int8_t *__restrict__ q,
                                                        float *__restrict__ s,
                                                        const int32_t *__restrict__ num_local_tokens, int32_t top_k,
                                                        const int32_t *__restrict__ row_ids) {
  static_assert(ACT != 1 || DT == LO_BF16, "the SiLU band is a bf16 table");
  constexpr bool SILU = ACT == 1, GATED = ACT != 0, FLOOR = ACT == 0 || ACT == 2;
  __shared__ float sRed[4];
  __shared__ uint16_t sSilu[SILU ? 2 * kSiluBandN : 2];
  const int tid = threadIdx.x;
  if (num_local_tokens) { // rows of padding tokens are left untouched
    const int64_t n = static_cast<int64_t>(num_local_tokens[0]) * top_k;
    rows = n < 0 ? 0 : (n < rows ? n : rows);
  }
  if (static_cast<int64_t>(blockIdx.x) >= rows) return;
  if constexpr (SILU) {
    uint16_t band_regs[kSiluBandPer];
    silu_band_load(band_regs, silu, tid);
    silu_band_store(sSilu, band_regs, tid);
    __syncthreads();
  }
  const int64_t in_stride = GATED ? 2 * C : C; // C = output columns
  const int pieces = static_cast<int>(C / 8);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    if (row_ids && row_ids[row] == -1) continue; // a row of an expert held elsewhere: left untouched
    const uint16_t *xr = x + row * in_stride;
    auto piece = [&](int p, float (&v)[8]) {
      const v8u16 a = *reinterpret_cast<const v8u16 *>(xr + p * 8);
      if constexpr (GATED) {
        const v8u16 u = *reinterpret_cast<const v8u16 *>(xr + C + p * 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if constexpr (SILU) v[i] = bf16_to_f32(silu_mul_band(sSilu, silu, a[i], u[i]));
          else v[i] = to_f32<DT>(act_mul_tab<DT>(silu, a[i], u[i]));
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = to_f32<DT>(a[i]);
      }
    };
    float keep[CH][8];
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int p = tid + 256 * j;
      if (p < pieces) {
        piece(p, keep[j]);
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(keep[j][i]));
      }
    }
    for (int p = tid + 256 * CH; p < pieces; p += 256) {
      float v[8];
      piece(p, v);
#pragma unroll
      for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
    }
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
    if ((tid & 63) == 0) sRed[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(sRed[0], sRed[1]), fmaxf(sRed[2], sRed[3]));
    __syncthreads(); // sRed is reused by the next row
    float inv;
    if constexpr (!FLOOR) {
      inv = amax == 0.0f ? 0.0f : 127.0f / amax;
    } else {
      amax = fmaxf(amax, 1e-10f);
      inv = 127.0f / amax;
    }
    if (tid == 0) s[row] = amax / 127.0f;
    auto emit = [&](int p, const float (&v)[8]) {
      v2i packed;
      packed[0] = static_cast<int>(pack4_i8(rne_i8(v[0] * inv), rne_i8(v[1] * inv), rne_i8(v[2] * inv), rne_i8(v[3] * inv)));
      packed[1] = static_cast<int>(pack4_i8(rne_i8(v[4] * inv), rne_i8(v[5] * inv), rne_i8(v[6] * inv), rne_i8(v[7] * inv)));
      *reinterpret_cast<v2i *>(q + row * C + p * 8) = packed;
    };
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int p = tid + 256 * j;
      if (p < pieces) emit(p, keep[j]);
    }
    for (int p = tid + 256 * CH; p < pieces; p += 256) {
      float v[8];
      piece(p, v);
      emit(p, v);
    }
  }
}

// The same for rows of at most 512 * CH values: one wavefront per row, four rows per workgroup,
// the row stays in registers and the reduction needs no barrier.
template <int ACT, int CH, int DT>
__global__ __launch_bounds__(256) void row_quant_wave_kernel(const uint16_t *__restrict__ x, int64_t rows, int64_t C,
                                                             const uint16_t *__restrict__ silu,
                                                             int8_t *__restrict__ q, float *__restrict__ s,
                                                             const int32_t *__restrict__ num_local_tokens,
                                                             int32_t top_k, const int32_t *__restrict__ row_ids) {
  static_assert(ACT != 1 || DT == LO_BF16, "the SiLU band is a bf16 table");
  constexpr bool SILU = ACT == 1, GATED = ACT != 0, FLOOR = ACT == 0 || ACT == 2;
  __shared__ uint16_t sSilu[SILU ? 2 * kSiluBandN : 2];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (num_local_tokens) {
    const int64_t n = static_cast<int64_t>(num_local_tokens[0]) * top_k;
    rows = n < 0 ? 0 : (n < rows ? n : rows);
  }
  if (static_cast<int64_t>(blockIdx.x) * 4 >= rows) return;
  if constexpr (SILU) {
    uint16_t band_regs[kSiluBandPer];
    silu_band_load(band_regs, silu, tid);
    silu_band_store(sSilu, band_regs, tid);
    __syncthreads();
  }
  const int64_t in_stride = GATED ? 2 * C : C;
  const int pieces = static_cast<int>(C / 8);
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + wave; row < rows; row += static_cast<int64_t>(gridDim.x) * 4) {
    if (row_ids && row_ids[row] == -1) continue; // a row of an expert held elsewhere: left untouched
    const uint16_t *xr = x + row * in_stride;
    v8u16 ga[CH], up[CH];
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int p = lane + 64 * j;
      const int pc = p < pieces ? p : 0; // lanes past the row re-read its start and are ignored
      ga[j] = *reinterpret_cast<const v8u16 *>(xr + pc * 8);
      if constexpr (GATED) up[j] = *reinterpret_cast<const v8u16 *>(xr + C + pc * 8);
    }
    float v[CH][8];
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const bool live = lane + 64 * j < pieces;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if constexpr (SILU) v[j][i] = bf16_to_f32(silu_mul_band(sSilu, silu, ga[j][i], up[j][i]));
        else if constexpr (GATED) v[j][i] = to_f32<DT>(act_mul_tab<DT>(silu, ga[j][i], up[j][i]));
        else v[j][i] = to_f32<DT>(ga[j][i]);
        amax = fmaxf(amax, live ? fabsf(v[j][i]) : 0.0f);
      }
    }
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
    float inv;
    if constexpr (!FLOOR) {
      inv = amax == 0.0f ? 0.0f : 127.0f / amax;
    } else {
      amax = fmaxf(amax, 1e-10f);
      inv = 127.0f / amax;
    }
    if (lane == 0) s[row] = amax / 127.0f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      const int p = lane + 64 * j;
      if (p >= pieces) continue;
      v2i packed;
      packed[0] = static_cast<int>(pack4_i8(rne_i8(v[j][0] * inv), rne_i8(v[j][1] * inv), rne_i8(v[j][2] * inv), rne_i8(v[j][3] * inv)));
      packed[1] = static_cast<int>(pack4_i8(rne_i8(v[j][4] * inv), rne_i8(v[j][5] * inv), rne_i8(v[j][6] * inv), rne_i8(v[j][7] * inv)));
      *reinterpret_cast<v2i *>(q + row * C + p * 8) = packed;
    }
  }
}

template <int ACT, int DT = LO_BF16>
static void launch_row_quant(const uint16_t *x, int64_t rows, int64_t C, const uint16_t *silu, int8_t *q, float *s,
                             const int32_t *nlt, int32_t top_k, const int32_t *row_ids, hipStream_t st) {
  const int pieces = static_cast<int>(C / 8);
  if (pieces <= 256 && rows >= 4) {
    int64_t grid = (rows + 3) / 4;
    if (grid > 256 * 32) grid = 256 * 32;
    const dim3 g(static_cast<unsigned>(grid)), b(256);
    if (pieces <= 64) hipLaunchKernelGGL((row_quant_wave_kernel<ACT, 1, DT>), g, b, 0, st, x, rows, C, silu, q, s, nlt, top_k, row_ids);
    else if (pieces <= 128) hipLaunchKernelGGL((row_quant_wave_kernel<ACT, 2, DT>), g, b, 0, st, x, rows, C, silu, q, s, nlt, top_k, row_ids);
    else hipLaunchKernelGGL((row_quant_wave_kernel<ACT, 4, DT>), g, b, 0, st, x, rows, C, silu, q, s, nlt, top_k, row_ids);
    return;
  }
  const unsigned grid = static_cast<unsigned>(rows < 65536 ? rows : 65536);
  hipLaunchKernelGGL((row_quant_kernel<ACT, ACT ? 2 : 4, DT>), dim3(grid), dim3(256), 0, st, x, rows, C, silu, q, s, nlt,
                     top_k, row_ids);
}

// ---- moe_sum -------------------------------------------------------------------
// Reference: csrc/kernels/moe_align_sum_kernels.cu:604-637 (fp32 accumulation in slot
// order, one rounding) and :886-909 (with bias: three roundings).
// TOPK > 0: the slot count is a compile-time constant, so the mask bytes and then the rows of
// the unmasked slots are requested back to back and waited for once (with a run-time count every
// mask byte and every row is a round trip of its own).  A masked slot adds
// +0.0f instead of being skipped, which is the same value: the sum starts at +0.0f and can
// never become -0.0f.  TOPK = 0 keeps the run-time loop.
template <int DT, bool HAS_BIAS, int TOPK>
__global__ __launch_bounds__(256) void moe_sum_kernel(const uint16_t *__restrict__ in,
                                                      uint16_t *__restrict__ out,
                                                      const uint16_t *__restrict__ bias,
                                                      const uint8_t *__restrict__ mask,
                                                      int64_t M, int topk, int64_t H,
                                                      float factor,
                                                      const int32_t *__restrict__ num_local_tokens) {
  const int64_t vec_per_row = H / 8;
  // rows of padding tokens (t >= num_local_tokens[0]) are left untouched
  if (num_local_tokens) {
    const int64_t n = num_local_tokens[0];
    M = n < 0 ? 0 : (n < M ? n : M);
  }
  const int64_t total = M * vec_per_row;
  for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < total;
       v += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = v / vec_per_row, c = (v % vec_per_row) * 8;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const uint16_t *p = in + t * topk * H + c;
    if constexpr (TOPK > 0) {
      bool on[TOPK];
#pragma unroll
      for (int j = 0; j < TOPK; ++j) on[j] = !mask || mask[t * TOPK + j] != 0;
      v8u16 r[TOPK];
#pragma unroll
      for (int j = 0; j < TOPK; ++j) {
        r[j] = v8u16{0, 0, 0, 0, 0, 0, 0, 0};
        if (on[j]) r[j] = *reinterpret_cast<const v8u16 *>(p + static_cast<int64_t>(j) * H);
      }
#pragma unroll
      for (int j = 0; j < TOPK; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = acc[i] + to_f32<DT>(r[j][i]);
    } else {
      for (int j = 0; j < topk; ++j) {
        if (mask && !mask[t * topk + j]) continue; // slot of an expert on another rank: adds 0
        const v8u16 r = *reinterpret_cast<const v8u16 *>(p + static_cast<int64_t>(j) * H);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = acc[i] + to_f32<DT>(r[i]);
      }
    }
    v8u16 o;
    if constexpr (HAS_BIAS) {
      const v8u16 b = *reinterpret_cast<const v8u16 *>(bias + t * H + c);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        uint16_t xv = from_f32<DT>(acc[i]);
        xv = from_f32<DT>(to_f32<DT>(xv) * factor);
        o[i] = from_f32<DT>(to_f32<DT>(xv) + to_f32<DT>(b[i]));
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = from_f32<DT>(acc[i] * factor);
    }
    *reinterpret_cast<v8u16 *>(out + t * H + c) = o;
  }
}

// ---- SiLU table ------------------------------------------------------------------
// bf16(silu(g)) for every bf16 pattern g (128 KB, stays in L2).  The GEMM epilogues look
// the activation up instead of spending ~45 vector instructions per element on
// exp / divide / round; the entries are produced by exactly those instructions, once
// per device.
__device__ uint16_t g_silu_bf16_table[65536];

__global__ __launch_bounds__(256) void silu_table_init_kernel(uint16_t *table) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const float g = bf16_to_f32(static_cast<uint16_t>(i));
  table[i] = f32_to_bf16(g / (1.0f + det_expf(-g)));
}

// Tables of the other gated activations: T(act(g)) for every 16-bit pattern g of the activation type T.
//   GELU: (f * 0.5f) * (1.0f + erf(f * ALPHA)) in fp32 with erf correctly rounded to fp32 (taken in
//         double precision and rounded once more), the form of csrc/kernels/activation_kernels_opt.cu:234-242;
//   SiLU for fp16 rows: f / (1 + exp(-f)) with det_expf, as in the bf16 table above.
// Slot = 2 * (T is fp16) + (activation is GELU); slot 0 is g_silu_bf16_table.  Built once per device.
__device__ uint16_t g_act_tables[3][65536];

template <int DT, int ACT>
__global__ __launch_bounds__(256) void act_table_init_kernel(uint16_t *table) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const float f = to_f32<DT>(static_cast<uint16_t>(i));
  if constexpr (ACT == LO_ACT_GELU) {
    const float alpha = 0.70710678118654752440f;
    const float e = static_cast<float>(erf(static_cast<double>(f * alpha)));
    table[i] = from_f32<DT>((f * 0.5f) * (1.0f + e));
  } else {
    table[i] = from_f32<DT>(f / (1.0f + det_expf(-f)));
  }
}

static int grid_for(int64_t work_items, int per_block) {
  int64_t b = (work_items + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > 256 * 16) b = 256 * 16;
  return static_cast<int>(b);
}

static std::mutex g_table_mutex;
static const uint16_t *g_table_ptr[64] = {};
static const uint16_t *g_act_ptr[64][4] = {};

int act_table(hipStream_t stream, int act, int dtype, const uint16_t **out) {
  if (act == LO_ACT_SILU && dtype == LO_BF16) return silu_table(stream, out);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    set_error("activation table: no current HIP device");
    return LO_ELAUNCH;
  }
  if ((act != LO_ACT_SILU && act != LO_ACT_GELU) || (dtype != LO_BF16 && dtype != LO_F16)) {
    set_error("activation table: unknown activation %d or element type %d", act, dtype);
    return LO_EINVAL;
  }
  const int slot = 2 * (dtype == LO_F16) + (act == LO_ACT_GELU);
  std::lock_guard<std::mutex> lock(g_table_mutex);
  if (!g_act_ptr[dev][slot]) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone) {
      set_error("the first call with this activation and element type on a device builds a table and must "
                "not be captured: run the op once before capturing a graph");
      return LO_EINVAL;
    }
    uint16_t *base = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void **>(&base), HIP_SYMBOL(g_act_tables)) != hipSuccess || !base) {
      set_error("activation table: hipGetSymbolAddress failed");
      return LO_ELAUNCH;
    }
    uint16_t *p = base + static_cast<size_t>(slot - 1) * 65536;
    if (slot == 1) hipLaunchKernelGGL((act_table_init_kernel<LO_BF16, LO_ACT_GELU>), dim3(256), dim3(256), 0, stream, p);
    else if (slot == 2) hipLaunchKernelGGL((act_table_init_kernel<LO_F16, LO_ACT_SILU>), dim3(256), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((act_table_init_kernel<LO_F16, LO_ACT_GELU>), dim3(256), dim3(256), 0, stream, p);
    int rc = check_launch("act_table_init");
    if (rc) return rc;
    if (hipStreamSynchronize(stream) != hipSuccess) {
      set_error("activation table: synchronisation failed");
      return LO_ELAUNCH;
    }
    g_act_ptr[dev][slot] = p;
  }
  *out = g_act_ptr[dev][slot];
  return LO_OK;
}

// The launch between the GEMMs where no fused epilogue exists (GELU; fp16 activations): the gated
// activation from its table and the quantisation of the form in one pass over c1 [rows, 2I].
int launch_act_mul_group_quant(const void *c1, int dtype, int act, int64_t rows, int64_t I, int8_t *q, float *s,
                               const uint8_t *row_mask, hipStream_t stream) {
  if (dtype == LO_F32)
    return launch_act_mul_group_quant_f32(static_cast<const float *>(c1), act, rows, I, q, s, row_mask, stream);
  const uint16_t *table = nullptr;
  int rc = act_table(stream, act, dtype, &table);
  if (rc) return rc;
  const int64_t groups = rows * (I / kGroup);
  if (groups == 0) return LO_OK;
  const dim3 g(grid_for(groups, 16)), b(256);
  if (dtype == LO_F16)
    hipLaunchKernelGGL(act_mul_group_quant_kernel<LO_F16>, g, b, 0, stream, static_cast<const uint16_t *>(c1), rows, I,
                       table, 1e-10f, q, s, row_mask);
  else
    hipLaunchKernelGGL(act_mul_group_quant_kernel<LO_BF16>, g, b, 0, stream, static_cast<const uint16_t *>(c1), rows, I,
                       table, 1e-10f, q, s, row_mask);
  return check_launch("act_mul_group_quant");
}

// SiLU: the semantics of fuse_silu_mul_quant (no floor under the row maximum); GELU: gelu_and_mul, then
// per_token_quant_int8 with its floor.
int launch_act_mul_row_quant(const void *c1, int dtype, int act, int64_t rows, int64_t I, int8_t *q, float *s,
                             const int32_t *num_local_tokens, int32_t top_k, const int32_t *row_ids,
                             hipStream_t stream) {
  const uint16_t *table = nullptr;
  int rc = act_table(stream, act, dtype, &table);
  if (rc) return rc;
  if (rows == 0) return LO_OK;
  const uint16_t *x = static_cast<const uint16_t *>(c1);
  if (dtype == LO_F16) {
    if (act == LO_ACT_GELU) launch_row_quant<2, LO_F16>(x, rows, I, table, q, s, num_local_tokens, top_k, row_ids, stream);
    else launch_row_quant<3, LO_F16>(x, rows, I, table, q, s, num_local_tokens, top_k, row_ids, stream);
  } else {
    if (act == LO_ACT_GELU) launch_row_quant<2>(x, rows, I, table, q, s, num_local_tokens, top_k, row_ids, stream);
    else launch_row_quant<1>(x, rows, I, table, q, s, num_local_tokens, top_k, row_ids, stream);
  }
  return check_launch("act_mul_row_quant");
}

int silu_table(hipStream_t stream, const uint16_t **out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    set_error("silu table: no current HIP device");
    return LO_ELAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_table_mutex);
  if (!g_table_ptr[dev]) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone) {
      set_error("the first call on a device builds the SiLU table and must not be captured: "
                "call lo_init() (or run the op once) before capturing a graph");
      return LO_EINVAL;
    }
    uint16_t *p = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(g_silu_bf16_table)) != hipSuccess || !p) {
      set_error("silu table: hipGetSymbolAddress failed");
      return LO_ELAUNCH;
    }
    hipLaunchKernelGGL(silu_table_init_kernel, dim3(256), dim3(256), 0, stream, p);
    int rc = check_launch("silu_table_init");
    if (rc) return rc;
    // one-time only: other streams of this device may use the table right after
    if (hipStreamSynchronize(stream) != hipSuccess) {
      set_error("silu table: synchronisation failed");
      return LO_ELAUNCH;
    }
    g_table_ptr[dev] = p;
  }
  *out = g_table_ptr[dev];
  return LO_OK;
}

} // namespace lo

extern "C" int lo_per_token_group_quant_int8(const void *x, int x_dtype, int64_t rows,
                                             int64_t cols, float eps, int8_t *q, float *s,
                                             lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(x && q && s, LO_EINVAL, "per_token_group_quant_int8: null pointer");
  LO_REQUIRE(x_dtype == LO_BF16 || x_dtype == LO_F16 || x_dtype == LO_F32, LO_ENOTSUP,
             "per_token_group_quant_int8: the input is bf16, fp16 or fp32");
  LO_REQUIRE(rows >= 0 && cols > 0 && cols % kGroup == 0, LO_EINVAL,
             "per_token_group_quant_int8: the last dimension (%lld) must be a multiple of 128",
             (long long)cols);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0,
             LO_EINVAL, "per_token_group_quant_int8: x must be 16-byte and q 8-byte aligned");
  const int64_t groups = rows * (cols / kGroup);
  if (groups == 0) return LO_OK;
  if (x_dtype == LO_F32)
    return launch_group_quant_f32(static_cast<const float *>(x), groups, eps, q, s, static_cast<hipStream_t>(stream));
  if (x_dtype == LO_F16)
    hipLaunchKernelGGL(group_quant_kernel<LO_F16>, dim3(grid_for(groups, 16)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(x), groups, eps, q, s);
  else
    hipLaunchKernelGGL(group_quant_kernel<LO_BF16>, dim3(grid_for(groups, 16)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(x), groups, eps, q, s);
  return check_launch("per_token_group_quant_int8");
}

extern "C" int lo_silu_and_mul(const void *c1, int dtype, int64_t rows, int64_t I, void *act,
                               lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(c1 && act, LO_EINVAL, "silu_and_mul: null pointer");
  LO_REQUIRE(dtype == LO_BF16 || dtype == LO_F16 || dtype == LO_F32, LO_ENOTSUP, "silu_and_mul: bf16, fp16 or fp32");
  LO_REQUIRE(rows >= 0 && I > 0 && I % 8 == 0, LO_EINVAL, "silu_and_mul: I (%lld) must be a multiple of 8",
             (long long)I);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(c1) & 15) == 0 && (reinterpret_cast<uintptr_t>(act) & 15) == 0,
             LO_EINVAL, "silu_and_mul: pointers must be 16-byte aligned");
  if (rows == 0) return LO_OK;
  if (dtype == LO_F32)
    return launch_act_mul_f32(static_cast<const float *>(c1), rows, I, LO_ACT_SILU, static_cast<float *>(act),
                              static_cast<hipStream_t>(stream));
  if (dtype == LO_F16)
    hipLaunchKernelGGL(silu_mul_kernel<LO_F16>, dim3(grid_for(rows * (I / 8), 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(c1), rows, I,
                       static_cast<uint16_t *>(act));
  else
    hipLaunchKernelGGL(silu_mul_kernel<LO_BF16>, dim3(grid_for(rows * (I / 8), 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(c1), rows, I,
                       static_cast<uint16_t *>(act));
  return check_launch("silu_and_mul");
}

extern "C" int lo_gelu_and_mul(const void *c1, int dtype, int64_t rows, int64_t I, void *act,
                               lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(c1 && act, LO_EINVAL, "gelu_and_mul: null pointer");
  LO_REQUIRE(dtype == LO_BF16 || dtype == LO_F16 || dtype == LO_F32, LO_ENOTSUP, "gelu_and_mul: bf16, fp16 or fp32");
  LO_REQUIRE(rows >= 0 && I > 0 && I % 8 == 0, LO_EINVAL, "gelu_and_mul: I (%lld) must be a multiple of 8",
             (long long)I);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(c1) & 15) == 0 && (reinterpret_cast<uintptr_t>(act) & 15) == 0,
             LO_EINVAL, "gelu_and_mul: pointers must be 16-byte aligned");
  if (dtype == LO_F32)
    return launch_act_mul_f32(static_cast<const float *>(c1), rows, I, LO_ACT_GELU, static_cast<float *>(act),
                              static_cast<hipStream_t>(stream));
  const uint16_t *table = nullptr;
  int rc = act_table(static_cast<hipStream_t>(stream), LO_ACT_GELU, dtype, &table);
  if (rc) return rc;
  if (rows == 0) return LO_OK;
  if (dtype == LO_F16)
    hipLaunchKernelGGL(act_mul_tab_kernel<LO_F16>, dim3(grid_for(rows * (I / 8), 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(c1), rows, I, table,
                       static_cast<uint16_t *>(act));
  else
    hipLaunchKernelGGL(act_mul_tab_kernel<LO_BF16>, dim3(grid_for(rows * (I / 8), 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(c1), rows, I, table,
                       static_cast<uint16_t *>(act));
  return check_launch("gelu_and_mul");
}

extern "C" int lo_act_mul_group_quant(const void *c1, int dtype, int activation, int64_t rows, int64_t I, int8_t *q,
                                      float *s, const uint8_t *row_mask, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(c1 && q && s, LO_EINVAL, "act_mul_group_quant: null pointer");
  LO_REQUIRE(dtype == LO_BF16 || dtype == LO_F16 || dtype == LO_F32, LO_ENOTSUP,
             "act_mul_group_quant: bf16, fp16 or fp32");
  LO_REQUIRE(activation == LO_ACT_SILU || activation == LO_ACT_GELU, LO_EINVAL,
             "act_mul_group_quant: unknown activation %d", activation);
  LO_REQUIRE(rows >= 0 && I > 0 && I % kGroup == 0, LO_EINVAL,
             "act_mul_group_quant: the output width (%lld) must be a multiple of 128", (long long)I);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(c1) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0, LO_EINVAL,
             "act_mul_group_quant: input must be 16-byte and q 8-byte aligned");
  return launch_act_mul_group_quant(c1, dtype, activation, rows, I, q, s, row_mask, static_cast<hipStream_t>(stream));
}

extern "C" int lo_activation_table(int activation, int dtype, void *table_out, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(table_out, LO_EINVAL, "activation_table: null pointer");
  const uint16_t *table = nullptr;
  int rc = act_table(static_cast<hipStream_t>(stream), activation, dtype, &table);
  if (rc) return rc;
  if (hipMemcpyAsync(table_out, table, 65536 * 2, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)) != hipSuccess) {
    set_error("activation_table: copy failed");
    return LO_ELAUNCH;
  }
  return LO_OK;
}

extern "C" int lo_moe_sum(const void *in, void *out, const void *bias, const uint8_t *expert_mask,
                          int dtype, int64_t M, int32_t topk, int64_t H, float factor,
                          const int32_t *num_local_tokens, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(in && out, LO_EINVAL, "moe_sum: null pointer");
  LO_REQUIRE(dtype == LO_BF16 || dtype == LO_F16 || dtype == LO_F32, LO_ENOTSUP, "moe_sum: bf16, fp16 or fp32");
  LO_REQUIRE(M >= 0 && topk >= 1 && H > 0 && H % 8 == 0, LO_EINVAL,
             "moe_sum: hidden size (%lld) must be a multiple of 8, topk >= 1", (long long)H);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(in) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(bias) & 15) == 0,
             LO_EINVAL, "moe_sum: pointers must be 16-byte aligned");
  if (M == 0) return LO_OK;
  if (dtype == LO_F32)
    return launch_moe_sum_f32(static_cast<const float *>(in), static_cast<float *>(out),
                              static_cast<const float *>(bias), expert_mask, M, topk, H, factor, num_local_tokens,
                              static_cast<hipStream_t>(stream));
  const int grid = grid_for(M * (H / 8), 256);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define LO_SUM_LAUNCH(DTV, HB, TK)                                                                   \
  hipLaunchKernelGGL((moe_sum_kernel<DTV, HB, TK>), dim3(grid), dim3(256), 0, s,                    \
                     static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out),               \
                     static_cast<const uint16_t *>(bias), expert_mask, M, topk, H, factor, num_local_tokens)
#define LO_SUM_PICK(TK)                                                                              \
  do {                                                                                               \
    if (dtype == LO_F16) { /* fp16 rows: the run-time slot loop serves every width */               \
      if (bias) LO_SUM_LAUNCH(LO_F16, true, 0);                                                      \
      else LO_SUM_LAUNCH(LO_F16, false, 0);                                                          \
    } else if (bias) LO_SUM_LAUNCH(LO_BF16, true, TK);                                               \
    else LO_SUM_LAUNCH(LO_BF16, false, TK);                                                          \
  } while (0)
  switch (topk) { // the usual router widths get the unrolled form
    case 1: LO_SUM_PICK(1); break;
    case 2: LO_SUM_PICK(2); break;
    case 4: LO_SUM_PICK(4); break;
    case 6: LO_SUM_PICK(6); break;
    case 8: LO_SUM_PICK(8); break;
    default: LO_SUM_PICK(0); break;
  }
#undef LO_SUM_PICK
#undef LO_SUM_LAUNCH
  return check_launch("moe_sum");
}

extern "C" int lo_per_token_quant_int8(const void *x, int x_dtype, int64_t rows, int64_t cols, int8_t *q,
                                       float *s, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(x && q && s, LO_EINVAL, "per_token_quant_int8: null pointer");
  LO_REQUIRE(x_dtype == LO_BF16 || x_dtype == LO_F16, LO_ENOTSUP, "per_token_quant_int8: the input is bf16 or fp16");
  LO_REQUIRE(rows >= 0 && cols > 0 && cols % 8 == 0, LO_EINVAL,
             "per_token_quant_int8: the last dimension (%lld) must be a multiple of 8", (long long)cols);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0,
             LO_EINVAL, "per_token_quant_int8: x must be 16-byte and q 8-byte aligned");
  if (rows == 0) return LO_OK;
  if (x_dtype == LO_F16)
    launch_row_quant<0, LO_F16>(static_cast<const uint16_t *>(x), rows, cols, nullptr, q, s, nullptr, 1, nullptr,
                                static_cast<hipStream_t>(stream));
  else
    launch_row_quant<0>(static_cast<const uint16_t *>(x), rows, cols, nullptr, q, s, nullptr, 1, nullptr,
                        static_cast<hipStream_t>(stream));
  return check_launch("per_token_quant_int8");
}

extern "C" int lo_fuse_silu_mul_quant_ids(const void *c1, int dtype, int64_t rows, int64_t I, int8_t *q, float *s,
                                          const int32_t *num_local_tokens, int32_t top_k, const int32_t *row_expert_ids,
                                          lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(c1 && q && s, LO_EINVAL, "fuse_silu_mul_quant: null pointer");
  LO_REQUIRE(dtype == LO_BF16 || dtype == LO_F16, LO_ENOTSUP, "fuse_silu_mul_quant: the input is bf16 or fp16");
  LO_REQUIRE(rows >= 0 && I > 0 && I % 8 == 0 && top_k >= 1, LO_EINVAL,
             "fuse_silu_mul_quant: the output width (%lld) must be a multiple of 8, top_k >= 1", (long long)I);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(c1) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0,
             LO_EINVAL, "fuse_silu_mul_quant: input must be 16-byte and q 8-byte aligned");
  if (rows == 0) return LO_OK;
  return launch_act_mul_row_quant(c1, dtype, LO_ACT_SILU, rows, I, q, s, num_local_tokens, top_k, row_expert_ids,
                                  static_cast<hipStream_t>(stream));
}

extern "C" int lo_fuse_silu_mul_quant(const void *c1, int dtype, int64_t rows, int64_t I, int8_t *q, float *s,
                                      const int32_t *num_local_tokens, int32_t top_k, lo_stream_t stream) {
  return lo_fuse_silu_mul_quant_ids(c1, dtype, rows, I, q, s, num_local_tokens, top_k, nullptr, stream);
}
