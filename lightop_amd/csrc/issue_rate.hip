// Measurement aid: the rate at which a SIMD of this chip issues int8 MFMAs together with the fp32 vector
// instructions the block-INT8 GEMMs spend on folding each K block's int32 sums into their fp32 accumulators.
//
// The grouped GEMMs run two waves per SIMD; per v_mfma_i32_16x16x64_i8 a wave issues two accumulator
// elements' worth of fold: 4 (fused-scale order), 6 (contracted order) or 8 (separate order) vector
// instructions.  The vector ALU and the matrix pipe of a SIMD share the issue port and, on real operand
// bits, the power budget, so the matrix pipe cannot reach its published peak under that load.  What it can
// reach is measured here with the loop stripped of everything else: groups of eight MFMAs on independent
// accumulators, each followed by `valu_per_mfma` independent v_fma_f32, two waves per SIMD on every compute
// unit, operand registers holding zeros or pseudo-random bytes (the clock this chip sustains depends on how many
// operand bits toggle).  bench.py reports the figure next to the kernel's own rate.
// No counterpart in the reference.
#include <hip/hip_runtime.h>

#include "common.h"

namespace lo {

#define LO_IR_FMA1(i) "v_fma_f32 v" #i ", v" #i ", v8, v9\n\t"
#define LO_IR_FMA2(a, b) LO_IR_FMA1(a) LO_IR_FMA1(b)
#define LO_IR_MFMA(a0, a1) "v_mfma_i32_16x16x64_i8 a[" #a0 ":" #a1 "], v[0:3], v[4:7], a[" #a0 ":" #a1 "]\n\t"
#define LO_IR_CLOBBER                                                                                            \
  "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", "v10", "v11", "v12", "v13", "v14", "v15", "v16",   \
      "v17", "v18", "v19", "v20", "v21", "v22", "v23", "v24", "v25", "a0", "a1", "a2", "a3", "a4", "a5", "a6",   \
      "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15", "a16", "a17", "a18", "a19", "a20", "a21",      \
      "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31"

// V: vector instructions after each MFMA (0, 4, 6 or 8), on registers v10.. (all independent within a group of 8)
template <int V>
__global__ __launch_bounds__(256) void issue_rate_kernel(float *sink, int iters, unsigned mask) {
  // 64 KB of LDS per workgroup: exactly two workgroups fit a compute unit, so a grid of two per compute unit
  // puts two waves on every SIMD
  __shared__ int occupancy_pad[16384 - 256];
  occupancy_pad[threadIdx.x] = iters;
  const unsigned h = (threadIdx.x * 2654435761u) ^ (blockIdx.x * 40503u);
  const unsigned d0 = (h * 747796405u + 1u) & mask, d1 = (h * 2891336453u + 7u) & mask;
  const unsigned d2 = (h * 1664525u + 3u) & mask, d3 = (h * 22695477u + 11u) & mask;
  const unsigned d4 = (h * 69069u + 5u) & mask, d5 = (h * 1103515245u + 9u) & mask;
  const unsigned d6 = (h * 134775813u + 13u) & mask, d7 = (h * 214013u + 17u) & mask;
  const float f8 = mask ? 0.99931f + (h & 255) * 1e-6f : 0.0f, f9 = mask ? 0.37f + (h & 127) * 1e-4f : 0.0f;
  asm volatile("v_mov_b32 v0, %0\n\tv_mov_b32 v1, %1\n\tv_mov_b32 v2, %2\n\tv_mov_b32 v3, %3\n\t"
               "v_mov_b32 v4, %4\n\tv_mov_b32 v5, %5\n\tv_mov_b32 v6, %6\n\tv_mov_b32 v7, %7\n\t"
               "v_mov_b32 v8, %8\n\tv_mov_b32 v9, %9\n\t"
               "v_mov_b32 v10, %8\n\tv_mov_b32 v11, %9\n\tv_mov_b32 v12, %8\n\tv_mov_b32 v13, %9\n\t"
               "v_mov_b32 v14, %8\n\tv_mov_b32 v15, %9\n\tv_mov_b32 v16, %8\n\tv_mov_b32 v17, %9\n\t"
               "v_mov_b32 v18, %8\n\tv_mov_b32 v19, %9\n\tv_mov_b32 v20, %8\n\tv_mov_b32 v21, %9\n\t"
               "v_mov_b32 v22, %8\n\tv_mov_b32 v23, %9\n\tv_mov_b32 v24, %8\n\tv_mov_b32 v25, %9\n\t"
               "v_accvgpr_write_b32 a0, 0\n\tv_accvgpr_write_b32 a1, 0\n\tv_accvgpr_write_b32 a2, 0\n\t"
               "v_accvgpr_write_b32 a3, 0\n\tv_accvgpr_write_b32 a4, 0\n\tv_accvgpr_write_b32 a5, 0\n\t"
               "v_accvgpr_write_b32 a6, 0\n\tv_accvgpr_write_b32 a7, 0\n\tv_accvgpr_write_b32 a8, 0\n\t"
               "v_accvgpr_write_b32 a9, 0\n\tv_accvgpr_write_b32 a10, 0\n\tv_accvgpr_write_b32 a11, 0\n\t"
               "v_accvgpr_write_b32 a12, 0\n\tv_accvgpr_write_b32 a13, 0\n\tv_accvgpr_write_b32 a14, 0\n\t"
               "v_accvgpr_write_b32 a15, 0\n\tv_accvgpr_write_b32 a16, 0\n\tv_accvgpr_write_b32 a17, 0\n\t"
               "v_accvgpr_write_b32 a18, 0\n\tv_accvgpr_write_b32 a19, 0\n\tv_accvgpr_write_b32 a20, 0\n\t"
               "v_accvgpr_write_b32 a21, 0\n\tv_accvgpr_write_b32 a22, 0\n\tv_accvgpr_write_b32 a23, 0\n\t"
               "v_accvgpr_write_b32 a24, 0\n\tv_accvgpr_write_b32 a25, 0\n\tv_accvgpr_write_b32 a26, 0\n\t"
               "v_accvgpr_write_b32 a27, 0\n\tv_accvgpr_write_b32 a28, 0\n\tv_accvgpr_write_b32 a29, 0\n\t"
               "v_accvgpr_write_b32 a30, 0\n\tv_accvgpr_write_b32 a31, 0\n\t" ::"v"(d0),
               "v"(d1), "v"(d2), "v"(d3), "v"(d4), "v"(d5), "v"(d6), "v"(d7), "v"(f8), "v"(f9)
               : LO_IR_CLOBBER);
  for (int it = 0; it < iters; ++it) {
    if constexpr (V == 0) {
      asm volatile(LO_IR_MFMA(0, 3) LO_IR_MFMA(4, 7) LO_IR_MFMA(8, 11) LO_IR_MFMA(12, 15) LO_IR_MFMA(16, 19)
                       LO_IR_MFMA(20, 23) LO_IR_MFMA(24, 27) LO_IR_MFMA(28, 31) ::
                       : LO_IR_CLOBBER);
    } else if constexpr (V == 4) {
      asm volatile(LO_IR_MFMA(0, 3) LO_IR_FMA2(10, 11) LO_IR_FMA2(12, 13) LO_IR_MFMA(4, 7) LO_IR_FMA2(14, 15)
                       LO_IR_FMA2(16, 17) LO_IR_MFMA(8, 11) LO_IR_FMA2(18, 19) LO_IR_FMA2(20, 21) LO_IR_MFMA(12, 15)
                           LO_IR_FMA2(22, 23) LO_IR_FMA2(24, 25) LO_IR_MFMA(16, 19) LO_IR_FMA2(10, 11) LO_IR_FMA2(12, 13)
                               LO_IR_MFMA(20, 23) LO_IR_FMA2(14, 15) LO_IR_FMA2(16, 17) LO_IR_MFMA(24, 27)
                                   LO_IR_FMA2(18, 19) LO_IR_FMA2(20, 21) LO_IR_MFMA(28, 31) LO_IR_FMA2(22, 23)
                                       LO_IR_FMA2(24, 25) ::
                       : LO_IR_CLOBBER);
    } else if constexpr (V == 6) {
      asm volatile(LO_IR_MFMA(0, 3) LO_IR_FMA2(10, 11) LO_IR_FMA2(12, 13) LO_IR_FMA2(14, 15) LO_IR_MFMA(4, 7)
                       LO_IR_FMA2(16, 17) LO_IR_FMA2(18, 19) LO_IR_FMA2(20, 21) LO_IR_MFMA(8, 11) LO_IR_FMA2(22, 23)
                           LO_IR_FMA2(24, 25) LO_IR_FMA2(10, 11) LO_IR_MFMA(12, 15) LO_IR_FMA2(12, 13) LO_IR_FMA2(14, 15)
                               LO_IR_FMA2(16, 17) LO_IR_MFMA(16, 19) LO_IR_FMA2(18, 19) LO_IR_FMA2(20, 21)
                                   LO_IR_FMA2(22, 23) LO_IR_MFMA(20, 23) LO_IR_FMA2(24, 25) LO_IR_FMA2(10, 11)
                                       LO_IR_FMA2(12, 13) LO_IR_MFMA(24, 27) LO_IR_FMA2(14, 15) LO_IR_FMA2(16, 17)
                                           LO_IR_FMA2(18, 19) LO_IR_MFMA(28, 31) LO_IR_FMA2(20, 21) LO_IR_FMA2(22, 23)
                                               LO_IR_FMA2(24, 25) ::
                       : LO_IR_CLOBBER);
    } else {
      static_assert(V == 8, "vector instructions per MFMA: 0, 4, 6 or 8");
      asm volatile(LO_IR_MFMA(0, 3) LO_IR_FMA2(10, 11) LO_IR_FMA2(12, 13) LO_IR_FMA2(14, 15) LO_IR_FMA2(16, 17)
                       LO_IR_MFMA(4, 7) LO_IR_FMA2(18, 19) LO_IR_FMA2(20, 21) LO_IR_FMA2(22, 23) LO_IR_FMA2(24, 25)
                           LO_IR_MFMA(8, 11) LO_IR_FMA2(10, 11) LO_IR_FMA2(12, 13) LO_IR_FMA2(14, 15) LO_IR_FMA2(16, 17)
                               LO_IR_MFMA(12, 15) LO_IR_FMA2(18, 19) LO_IR_FMA2(20, 21) LO_IR_FMA2(22, 23)
                                   LO_IR_FMA2(24, 25) LO_IR_MFMA(16, 19) LO_IR_FMA2(10, 11) LO_IR_FMA2(12, 13)
                                       LO_IR_FMA2(14, 15) LO_IR_FMA2(16, 17) LO_IR_MFMA(20, 23) LO_IR_FMA2(18, 19)
                                           LO_IR_FMA2(20, 21) LO_IR_FMA2(22, 23) LO_IR_FMA2(24, 25) LO_IR_MFMA(24, 27)
                                               LO_IR_FMA2(10, 11) LO_IR_FMA2(12, 13) LO_IR_FMA2(14, 15)
                                                   LO_IR_FMA2(16, 17) LO_IR_MFMA(28, 31) LO_IR_FMA2(18, 19)
                                                       LO_IR_FMA2(20, 21) LO_IR_FMA2(22, 23) LO_IR_FMA2(24, 25) ::
                       : LO_IR_CLOBBER);
    }
  }
  if (sink[0] == 12345.0f) sink[1] = static_cast<float>(occupancy_pad[threadIdx.x ^ 1]); // never true: the buffer holds zeros
}

} // namespace lo

extern "C" int lo_measure_mfma_issue_rate(int valu_per_mfma, int random_operands, int iters, void *stream,
                                          double *int8_ops_per_second) {
  using namespace lo;
  LO_REQUIRE(int8_ops_per_second != nullptr, LO_EINVAL, "lo_measure_mfma_issue_rate: null result pointer");
  LO_REQUIRE(valu_per_mfma == 0 || valu_per_mfma == 4 || valu_per_mfma == 6 || valu_per_mfma == 8, LO_EINVAL,
             "lo_measure_mfma_issue_rate: valu_per_mfma must be 0, 4, 6 or 8 (got %d)", valu_per_mfma);
  LO_REQUIRE(iters >= 1 && iters <= (1 << 22), LO_EINVAL, "lo_measure_mfma_issue_rate: iters out of range");
  hipStream_t s = static_cast<hipStream_t>(stream);
  int dev = 0, cus = 0, rc = LO_OK;
  auto fail = [&](hipError_t err, const char *what) {
    if (err != hipSuccess && rc == LO_OK) {
      set_error("lo_measure_mfma_issue_rate: %s: %s", what, hipGetErrorString(err));
      rc = LO_ELAUNCH;
    }
  };
  float *sink = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  fail(hipGetDevice(&dev), "hipGetDevice");
  fail(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev), "hipDeviceGetAttribute");
  fail(hipMalloc(reinterpret_cast<void **>(&sink), 256), "hipMalloc");
  if (rc != LO_OK) return rc;
  fail(hipMemsetAsync(sink, 0, 256, s), "memset");
  fail(hipEventCreate(&e0), "event");
  fail(hipEventCreate(&e1), "event");
  const unsigned mask = random_operands ? 0xffffffffu : 0u;
  const dim3 grid(static_cast<unsigned>(cus) * 2), block(256); // two four-wave workgroups per compute unit
  auto launch = [&](int n) {
    switch (valu_per_mfma) {
      case 0: hipLaunchKernelGGL(issue_rate_kernel<0>, grid, block, 0, s, sink, n, mask); break;
      case 4: hipLaunchKernelGGL(issue_rate_kernel<4>, grid, block, 0, s, sink, n, mask); break;
      case 6: hipLaunchKernelGGL(issue_rate_kernel<6>, grid, block, 0, s, sink, n, mask); break;
      default: hipLaunchKernelGGL(issue_rate_kernel<8>, grid, block, 0, s, sink, n, mask); break;
    }
  };
  if (rc == LO_OK) {
    launch(iters / 8 + 1); // bring the clock to where the load holds it
    fail(hipEventRecord(e0, s), "record");
    launch(iters);
    fail(hipEventRecord(e1, s), "record");
    fail(hipEventSynchronize(e1), "synchronize");
    fail(hipGetLastError(), "launch");
  }
  if (rc == LO_OK) {
    float ms = 0.0f;
    fail(hipEventElapsedTime(&ms, e0, e1), "elapsed");
    // 8 MFMAs of 16 x 16 x 64 multiply-adds per iteration and wave; 8 waves per compute unit
    const double ops = 2.0 * 16 * 16 * 64 * 8.0 * iters * 8.0 * cus;
    *int8_ops_per_second = ms > 0.0f ? ops / (ms * 1e-3) : 0.0;
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(sink);
  return rc;
}
