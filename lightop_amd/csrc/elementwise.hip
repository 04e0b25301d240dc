// Streaming stages of the block-INT8 fused-MoE path on gfx950: 1x128 group
// quantisation, SiLU-and-mul, and the top-k reduction.  All are HBM-bound; every
// lane moves 16 bytes per load and a workgroup covers whole 128-element groups.
#include <mutex>

#include "common.h"

namespace lo {

// ---- per_token_group_quant_int8 ----------------------------------------------
// Reference: python/lightop/_lmslim_native/layers/gemm/int8_utils.py:74-122.
// 16 lanes own one group of 128 values (8 each); amax is reduced across those 16
// lanes with DPP-free shuffles; the division is IEEE (x / s, never x * (1/s)).
template <int DT>
__global__ __launch_bounds__(256) void group_quant_kernel(const uint16_t *__restrict__ x,
                                                          int64_t groups, float eps,
                                                          int8_t *__restrict__ q,
                                                          float *__restrict__ s) {
  const int sub = threadIdx.x & 15;
  int64_t g = static_cast<int64_t>(blockIdx.x) * 16 + (threadIdx.x >> 4);
  const int64_t gstride = static_cast<int64_t>(gridDim.x) * 16;
  for (; g < groups; g += gstride) {
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
    int qi[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) qi[i] = quant_one(v[i], sc);
    v2i packed;
    packed[0] = static_cast<int>(pack4_i8(qi[0], qi[1], qi[2], qi[3]));
    packed[1] = static_cast<int>(pack4_i8(qi[4], qi[5], qi[6], qi[7]));
    *reinterpret_cast<v2i *>(q + g * kGroup + sub * 8) = packed;
    if (sub == 0) s[g] = sc;
  }
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

// ---- moe_sum -------------------------------------------------------------------
// Reference: csrc/kernels/moe_align_sum_kernels.cu:604-637 (fp32 accumulation in slot
// order, one rounding) and :886-909 (with bias: three roundings).
template <int DT, bool HAS_BIAS>
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
    for (int j = 0; j < topk; ++j) {
      if (mask && !mask[t * topk + j]) continue; // slot of an expert on another rank: adds 0
      const v8u16 r = *reinterpret_cast<const v8u16 *>(p + static_cast<int64_t>(j) * H);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = acc[i] + to_f32<DT>(r[i]);
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

static int grid_for(int64_t work_items, int per_block) {
  int64_t b = (work_items + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > 256 * 16) b = 256 * 16;
  return static_cast<int>(b);
}

static std::mutex g_table_mutex;
static const uint16_t *g_table_ptr[64] = {};

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

extern "C" int lo_init(lo_stream_t stream) {
  const uint16_t *t = nullptr;
  return lo::silu_table(static_cast<hipStream_t>(stream), &t);
}

extern "C" int lo_per_token_group_quant_int8(const void *x, int x_dtype, int64_t rows,
                                             int64_t cols, float eps, int8_t *q, float *s,
                                             lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(x && q && s, LO_EINVAL, "per_token_group_quant_int8: null pointer");
  LO_REQUIRE(x_dtype == LO_BF16, LO_ENOTSUP, "per_token_group_quant_int8: only bf16 input is built");
  LO_REQUIRE(rows >= 0 && cols > 0 && cols % kGroup == 0, LO_EINVAL,
             "per_token_group_quant_int8: the last dimension (%lld) must be a multiple of 128",
             (long long)cols);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0,
             LO_EINVAL, "per_token_group_quant_int8: x must be 16-byte and q 8-byte aligned");
  const int64_t groups = rows * (cols / kGroup);
  if (groups == 0) return LO_OK;
  hipLaunchKernelGGL(group_quant_kernel<LO_BF16>, dim3(grid_for(groups, 16)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(x), groups, eps,
                     q, s);
  return check_launch("per_token_group_quant_int8");
}

extern "C" int lo_silu_and_mul(const void *c1, int dtype, int64_t rows, int64_t I, void *act,
                               lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(c1 && act, LO_EINVAL, "silu_and_mul: null pointer");
  LO_REQUIRE(dtype == LO_BF16, LO_ENOTSUP, "silu_and_mul: only bf16 is built");
  LO_REQUIRE(rows >= 0 && I > 0 && I % 8 == 0, LO_EINVAL, "silu_and_mul: I (%lld) must be a multiple of 8",
             (long long)I);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(c1) & 15) == 0 && (reinterpret_cast<uintptr_t>(act) & 15) == 0,
             LO_EINVAL, "silu_and_mul: pointers must be 16-byte aligned");
  if (rows == 0) return LO_OK;
  hipLaunchKernelGGL(silu_mul_kernel<LO_BF16>, dim3(grid_for(rows * (I / 8), 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t *>(c1), rows, I,
                     static_cast<uint16_t *>(act));
  return check_launch("silu_and_mul");
}

extern "C" int lo_moe_sum(const void *in, void *out, const void *bias, const uint8_t *expert_mask,
                          int dtype, int64_t M, int32_t topk, int64_t H, float factor,
                          const int32_t *num_local_tokens, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(in && out, LO_EINVAL, "moe_sum: null pointer");
  LO_REQUIRE(dtype == LO_BF16, LO_ENOTSUP, "moe_sum: only bf16 is built");
  LO_REQUIRE(M >= 0 && topk >= 1 && H > 0 && H % 8 == 0, LO_EINVAL,
             "moe_sum: hidden size (%lld) must be a multiple of 8, topk >= 1", (long long)H);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(in) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(bias) & 15) == 0,
             LO_EINVAL, "moe_sum: pointers must be 16-byte aligned");
  if (M == 0) return LO_OK;
  const int grid = grid_for(M * (H / 8), 256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (bias)
    hipLaunchKernelGGL((moe_sum_kernel<LO_BF16, true>), dim3(grid), dim3(256), 0, s,
                       static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out),
                       static_cast<const uint16_t *>(bias), expert_mask, M, topk, H, factor, num_local_tokens);
  else
    hipLaunchKernelGGL((moe_sum_kernel<LO_BF16, false>), dim3(grid), dim3(256), 0, s,
                       static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out),
                       static_cast<const uint16_t *>(nullptr), expert_mask, M, topk, H, factor, num_local_tokens);
  return check_launch("moe_sum");
}
