// The element-wise stages of the block form on fp32 activations (hidden_states.dtype ==
// torch.float32: compute_type tl.float32, python/lightop/_lmslim_native/layers/fused_moe/
// int8.py:689-696).  Nothing between the stages is rounded to 16 bits, so there are no lookup
// tables here: SiLU is g / (1 + exp(-g)) with the fixed-sequence exp of common.h, GELU
// (g * 0.5f) * (1 + erf(g * ALPHA)) with the double-precision erf rounded once more, the product
// with the up value one fp32 multiplication (vLLM's silu_and_mul / gelu_and_mul with T = float,
// called at int8.py:811 and :826).  The quantisation is the rule of int8_utils.py:74-122; the
// reduce is moe_align_sum_kernels.cu:619-633 / :886-909 with T = float.
//
// This is a completeness path (no benchmark configuration uses fp32 rows): plain grid-stride
// kernels, 16 lanes per 128-wide group as in the 16-bit kernels.
#include "common.h"

namespace lo {

typedef float v4f32 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float act_f32(float g, int act) {
  if (act == LO_ACT_GELU) {
    const float alpha = 0.70710678118654752440f;
    const float e = static_cast<float>(erf(static_cast<double>(g * alpha)));
    return (g * 0.5f) * (1.0f + e);
  }
  return g / (1.0f + det_expf(-g));
}

// eight values of one lane -> amax over the 16 lanes of the group -> scale and packed int8
__device__ __forceinline__ void quant_group_f32(const float (&v)[8], float eps, int8_t *qdst, float *sdst, bool lead) {
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
  for (int d = 1; d < 16; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
  amax = fmaxf(amax, eps);
  const float sc = amax / 127.0f;
  const float rsc = 1.0f / sc;
  v2i packed;
  packed[0] = static_cast<int>(quant4(&v[0], sc, rsc));
  packed[1] = static_cast<int>(quant4(&v[4], sc, rsc));
  *reinterpret_cast<v2i *>(qdst) = packed;
  if (lead) *sdst = sc;
}

__global__ __launch_bounds__(256) void group_quant_f32_kernel(const float *__restrict__ x, int64_t groups, float eps,
                                                              int8_t *__restrict__ q, float *__restrict__ s) {
  const int sub = threadIdx.x & 15;
  for (int64_t g = static_cast<int64_t>(blockIdx.x) * 16 + (threadIdx.x >> 4); g < groups;
       g += static_cast<int64_t>(gridDim.x) * 16) {
    const v4f32 a = *reinterpret_cast<const v4f32 *>(x + g * kGroup + sub * 8);
    const v4f32 b = *reinterpret_cast<const v4f32 *>(x + g * kGroup + sub * 8 + 4);
    const float v[8] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
    quant_group_f32(v, eps, q + g * kGroup + sub * 8, s + g, sub == 0);
  }
}

__global__ __launch_bounds__(256) void act_mul_f32_kernel(const float *__restrict__ c1, int64_t rows, int64_t I, int act,
                                                          float *__restrict__ out) {
  const int64_t per_row = I / 4, total = rows * per_row;
  for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < total;
       v += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = v / per_row, c = (v % per_row) * 4;
    const v4f32 g = *reinterpret_cast<const v4f32 *>(c1 + t * 2 * I + c);
    const v4f32 u = *reinterpret_cast<const v4f32 *>(c1 + t * 2 * I + I + c);
    v4f32 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = act_f32(g[i], act) * u[i];
    *reinterpret_cast<v4f32 *>(out + t * I + c) = o;
  }
}

__global__ __launch_bounds__(256) void act_mul_group_quant_f32_kernel(const float *__restrict__ c1, int64_t rows,
                                                                      int64_t I, int act, float eps,
                                                                      int8_t *__restrict__ q, float *__restrict__ s,
                                                                      const uint8_t *__restrict__ row_mask) {
  const int sub = threadIdx.x & 15;
  const int64_t gpr = I / kGroup, groups = rows * gpr;
  for (int64_t g = static_cast<int64_t>(blockIdx.x) * 16 + (threadIdx.x >> 4); g < groups;
       g += static_cast<int64_t>(gridDim.x) * 16) {
    const int64_t t = g / gpr, c = (g % gpr) * kGroup + sub * 8;
    if (row_mask && !row_mask[t]) continue; // a slot of another rank's expert (uniform over the 16 lanes)
    const float *gp = c1 + t * 2 * I + c, *up = gp + I;
    const v4f32 g0 = *reinterpret_cast<const v4f32 *>(gp), g1 = *reinterpret_cast<const v4f32 *>(gp + 4);
    const v4f32 u0 = *reinterpret_cast<const v4f32 *>(up), u1 = *reinterpret_cast<const v4f32 *>(up + 4);
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = act_f32(g0[i], act) * u0[i];
      v[4 + i] = act_f32(g1[i], act) * u1[i];
    }
    quant_group_f32(v, eps, q + t * I + c, s + g, sub == 0);
  }
}

__global__ __launch_bounds__(256) void moe_sum_f32_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                          const float *__restrict__ bias,
                                                          const uint8_t *__restrict__ mask, int64_t M, int topk,
                                                          int64_t H, float factor,
                                                          const int32_t *__restrict__ num_local_tokens) {
  const int64_t per_row = H / 4;
  if (num_local_tokens) { // rows of padding tokens are left untouched
    const int64_t n = num_local_tokens[0];
    M = n < 0 ? 0 : (n < M ? n : M);
  }
  const int64_t total = M * per_row;
  for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < total;
       v += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t t = v / per_row, c = (v % per_row) * 4;
    v4f32 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int j = 0; j < topk; ++j) {
      if (mask && !mask[t * topk + j]) continue; // slot of an expert on another rank: adds 0
      const v4f32 r = *reinterpret_cast<const v4f32 *>(in + (t * topk + j) * H + c);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = acc[i] + r[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = acc[i] * factor;
    if (bias) {
      const v4f32 b = *reinterpret_cast<const v4f32 *>(bias + t * H + c);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = acc[i] + b[i];
    }
    *reinterpret_cast<v4f32 *>(out + t * H + c) = acc;
  }
}

static int blocks_for(int64_t items, int per_block) {
  int64_t b = (items + per_block - 1) / per_block;
  return static_cast<int>(b < 1 ? 1 : (b > 4096 ? 4096 : b));
}

int launch_group_quant_f32(const float *x, int64_t groups, float eps, int8_t *q, float *s, hipStream_t stream) {
  if (groups == 0) return LO_OK;
  hipLaunchKernelGGL(group_quant_f32_kernel, dim3(blocks_for(groups, 16)), dim3(256), 0, stream, x, groups, eps, q, s);
  return check_launch("per_token_group_quant_int8(fp32)");
}

int launch_act_mul_f32(const float *c1, int64_t rows, int64_t I, int act, float *out, hipStream_t stream) {
  if (rows == 0) return LO_OK;
  hipLaunchKernelGGL(act_mul_f32_kernel, dim3(blocks_for(rows * (I / 4), 256)), dim3(256), 0, stream, c1, rows, I, act,
                     out);
  return check_launch("act_and_mul(fp32)");
}

int launch_act_mul_group_quant_f32(const float *c1, int act, int64_t rows, int64_t I, int8_t *q, float *s,
                                   const uint8_t *row_mask, hipStream_t stream) {
  if (rows == 0) return LO_OK;
  hipLaunchKernelGGL(act_mul_group_quant_f32_kernel, dim3(blocks_for(rows * (I / kGroup), 16)), dim3(256), 0, stream,
                     c1, rows, I, act, 1e-10f, q, s, row_mask);
  return check_launch("act_mul_group_quant(fp32)");
}

int launch_moe_sum_f32(const float *in, float *out, const float *bias, const uint8_t *mask, int64_t M, int32_t topk,
                       int64_t H, float factor, const int32_t *num_local_tokens, hipStream_t stream) {
  if (M == 0) return LO_OK;
  hipLaunchKernelGGL(moe_sum_f32_kernel, dim3(blocks_for(M * (H / 4), 256)), dim3(256), 0, stream, in, out, bias, mask, M,
                     topk, H, factor, num_local_tokens);
  return check_launch("moe_sum(fp32)");
}

} // namespace lo
