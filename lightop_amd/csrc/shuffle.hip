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

// Packed int4 weights (two per byte along K; even k in the high nibble, the reference's
// order, python/lightop/_lmslim_native/layers/fused_moe/w4a8.py:341, :375-377).  A block of
// 16 rows x 128 K is 1 KB: [4 quarters of a 64-wide k-step][16 rows][16 bytes], the 16 bytes
// being k-step 0 (8 bytes) then k-step 1 (8 bytes) of the lane that owns (row, quarter) in the
// 16x16x64 MFMA.  Inside each 32-bit word, byte b holds element b in its low nibble and
// element b + 4 in its high nibble, so that (word << 4) & 0xf0f0f0f0 and word & 0xf0f0f0f0
// are the eight elements, in order, as int8 values 16 times too large.
__global__ __launch_bounds__(256) void preshuffle_int4_kernel(const uint8_t *__restrict__ src,
                                                              uint8_t *__restrict__ dst, int64_t N,
                                                              int64_t K, int64_t words_total) {
  // one 32-bit destination word (8 elements) per thread
  const int64_t KB = K / kGroup, NBLK = N / 16;
  for (int64_t d = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; d < words_total;
       d += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int64_t blk = d >> 8; // 256 words per 1 KB block
    const int in = static_cast<int>(d & 255);
    const int q = in >> 6, r = (in >> 2) & 15, ks = (in >> 1) & 1, w = in & 1;
    const int64_t e = blk / (NBLK * KB), rem = blk - e * NBLK * KB;
    const int64_t kb = LO_SHUF_KB_MAJOR ? rem / NBLK : rem % KB;
    const int64_t nb = LO_SHUF_KB_MAJOR ? rem % NBLK : rem / KB;
    const int64_t row = e * N + nb * 16 + r;
    const int64_t k0 = kb * kGroup + ks * 64 + q * 16 + w * 8; // first of the 8 elements
    const uint32_t p = *reinterpret_cast<const uint32_t *>(src + (row * K + k0) / 2);
    // source byte j holds elements (2j, 2j+1) as (high, low) nibble
    uint32_t out = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int elo = b, ehi = b + 4;
      const uint32_t lo = (p >> (8 * (elo / 2) + ((elo & 1) ? 0 : 4))) & 15u;
      const uint32_t hi = (p >> (8 * (ehi / 2) + ((ehi & 1) ? 0 : 4))) & 15u;
      out |= (lo | (hi << 4)) << (8 * b);
    }
    *reinterpret_cast<uint32_t *>(dst + d * 4) = out;
  }
}

} // namespace lo

extern "C" int lo_preshuffle_weight_int4(const uint8_t *src, uint8_t *dst, int32_t E, int64_t N,
                                         int64_t K, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(src && dst && src != dst, LO_EINVAL, "preshuffle_weight_int4: needs distinct non-null buffers");
  LO_REQUIRE(E >= 1 && N > 0 && N % 16 == 0 && K > 0 && K % kGroup == 0, LO_EINVAL,
             "preshuffle_weight_int4: N (%lld) must be a multiple of 16 and K (%lld) of 128",
             (long long)N, (long long)K);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(src) & 3) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0,
             LO_EINVAL, "preshuffle_weight_int4: source must be 4-byte, destination 16-byte aligned");
  const int64_t words = static_cast<int64_t>(E) * N * K / 8;
  int64_t grid = (words + 255) / 256;
  if (grid > 65536) grid = 65536;
  hipLaunchKernelGGL(preshuffle_int4_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), src, dst, N, K, words);
  return check_launch("preshuffle_weight_int4");
}

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
