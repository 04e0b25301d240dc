// Load-time weight layout for the gfx950 grouped GEMM kernels.
//
// Row-major expert weights [E, N, K] (K contiguous) make every MFMA operand load touch
// 16 or 32 different rows with 16 bytes each.  The pre-shuffled layout stores each block
// of 16 rows x 128 K-bytes as [8 chunks of 16 K-bytes][16 rows][16 bytes] (2 KB), blocks
// ordered [E][K/128][N/16], so that a wavefront's operand load is one contiguous 1 KB
// read and the waves of a workgroup, which hold neighbouring rows and walk K together,
// read one contiguous region per step.
// (The reference keeps a comparable load-time "marlin" shuffle for its native kernels in
// test/moe_w8a8/w8a8_quant.py:66-111; the layout here is specific to the gfx950 kernels.)
#include "common.h"

namespace lo {

__global__ __launch_bounds__(256) void preshuffle_kernel(const int8_t *__restrict__ src,
                                                         int8_t *__restrict__ dst, int64_t N,
                                                         int64_t K, int64_t chunks_total) {
  // one 16-byte chunk per thread; destination-major so that writes are contiguous
  const int64_t KB = K / kGroup;
  for (int64_t d = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; d < chunks_total;
       d += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t blk = d >> 7;       // 128 chunks per 2 KB block
    const int in = static_cast<int>(d & 127);
    const int chunk = in >> 4, r = in & 15;
    const int64_t NBLK = N / 16;
    const int64_t e = blk / (NBLK * KB), rem = blk - e * NBLK * KB;
    const int64_t kb = LO_SHUF_KB_MAJOR ? rem / NBLK : rem % KB;
    const int64_t nb = LO_SHUF_KB_MAJOR ? rem % NBLK : rem / KB;
    const int64_t row = e * N + nb * 16 + r;
    const v4i v = *reinterpret_cast<const v4i *>(src + row * K + kb * kGroup + chunk * 16);
    *reinterpret_cast<v4i *>(dst + d * 16) = v;
  }
}

} // namespace lo

extern "C" int lo_preshuffle_weight_int8(const int8_t *src, int8_t *dst, int32_t E, int64_t N,
                                         int64_t K, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(src && dst && src != dst, LO_EINVAL, "preshuffle_weight_int8: needs distinct non-null buffers");
  LO_REQUIRE(E >= 1 && N > 0 && N % 16 == 0 && K > 0 && K % kGroup == 0, LO_EINVAL,
             "preshuffle_weight_int8: N (%lld) must be a multiple of 16 and K (%lld) of 128",
             (long long)N, (long long)K);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(src) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0,
             LO_EINVAL, "preshuffle_weight_int8: buffers must be 16-byte aligned");
  const int64_t rows = static_cast<int64_t>(E) * N;
  const int64_t chunks = rows * K / 16;
  int64_t grid = (chunks + 255) / 256;
  if (grid > 65536) grid = 65536;
  hipLaunchKernelGGL(preshuffle_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), src, dst, N, K, chunks);
  return check_launch("preshuffle_weight_int8");
}
