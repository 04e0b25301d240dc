// Grouped per-channel W8A8 GEMM for gfx950, LDS-tiled form (reference: moe_gemm_w8a8,
// csrc/moe_gemm/w8a8/moe_w8a8.cu:2389-2536; epilogues :156-166 and :445-470).
//
// One scale per token row and one per weight row, applied once after the whole-K int32 sum, so
// the K loop is loads and MFMAs only and the accumulators never leave the matrix pipe's
// registers.  What bounds such a loop on this chip is the rate at which the compute units can
// pull operands out of L2: every token block re-reads its expert's weights, and the bytes
// requested per multiply-add are 1/tokens + 1/rows of the workgroup tile.  The tile is therefore
// 32*TB tokens x 256 weight rows with TB = 4 where there are enough tokens per expert: four
// wavefronts, each owning 64 weight rows (two 32-row MFMA fragments, global -> registers,
// double buffered) against all 32*TB tokens (gathered through sorted_token_ids into a
// double-buffered, row-padded LDS tile), i.e. 2*TB accumulators of v_mfma_i32_32x32x32_i8.
// Two workgroups share a compute unit (three with 64-token tiles).
//
// STREAM: an expert's weights are read by one token block, by and large, and are loaded with the
// streaming cache policy; with several token blocks per expert the blocks share them through L2
// and the default policy is the faster one.
#include <type_traits>

#include "gemm.h"

namespace lo {

typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kPcRow = 144; // LDS row pitch in bytes: 128 + 16 keeps ds_read_b128 conflict-free

template <bool SHUF, int TB, bool STREAM>
__device__ __forceinline__ void moe_gemm_pc_body(const GemmArgs &a, int m_blocks, int group_m) {
  static_assert(!STREAM || SHUF, "streaming policy: pre-shuffled weights only");
  constexpr int kWAux = STREAM ? kCacheStream : kCacheDefault;
  constexpr int kTileM = 32 * TB;       // tokens per workgroup
  constexpr int kThrPerTok = 256 / kTileM; // threads that gather one token row
  constexpr int kPieces = 8 / kThrPerTok;  // 16-byte pieces per thread and K block
  __shared__ __attribute__((aligned(16))) int8_t sA[2][kTileM * kPcRow];

  int mb, nt;
  if (!tile_of(blockIdx.x, a.n_tiles, m_blocks, group_m, mb, nt)) return;
  if (static_cast<int64_t>(mb) * kTileM >= a.ntpp[0]) return;
  // An expert_map entry outside the weight tensor is treated like an expert of another rank, but its
  // rows are always zero-filled: the slot mask of the alignment counts such a slot as local.
  const int e_raw = a.expert_ids[mb];
  const bool e_oob = e_raw >= a.E;
  const int e = e_oob ? -1 : e_raw;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wr = __builtin_amdgcn_readfirstlane(tid >> 6); // which 64 weight rows of the tile
  const int r = lane & 31, c = lane >> 5;
  const int64_t K = a.K, N = a.N;
  const int KB = static_cast<int>(K / kGroup);

  int64_t f[TB];
  bool valid[TB];
#pragma unroll
  for (int tb = 0; tb < TB; ++tb) {
    f[tb] = a.sorted[static_cast<int64_t>(mb) * kTileM + tb * 32 + r];
    valid[tb] = f[tb] < a.num_valid;
  }
  int64_t nrow[2];
  nrow[0] = static_cast<int64_t>(nt) * 256 + wr * 64;
  nrow[1] = nrow[0] + 32;
  const bool wave_active = nrow[0] < N; // N % 64 == 0 is checked on the host

  if (e < 0) { // expert of another rank: its rows are defined to be zero
    if (wave_active && (!a.skip_nonlocal || e_oob)) {
#pragma unroll
      for (int tb = 0; tb < TB; ++tb)
        if (valid[tb])
#pragma unroll
          for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int q = 0; q < 4; ++q)
              *reinterpret_cast<v2i *>(a.C + f[tb] * N + nrow[rb] + 8 * q + 4 * c) = v2i{0, 0};
    }
    return;
  }

  // cooperative gather role: thread -> (token, run of kPieces 16-byte pieces of the 128-byte K block)
  const int lt = tid / kThrPerTok, lq = tid % kThrPerTok;
  const int64_t lf = a.sorted[static_cast<int64_t>(mb) * kTileM + lt];
  const int64_t lrow = (lf < a.num_valid) ? lf / a.top_k : 0;
  const brsrc rA = make_rsrc(a.A, static_cast<uint32_t>(a.a_rows * K));
  const int aoff = static_cast<int>(lrow * K) + lq * (16 * kPieces);
  int8_t *const sdst0 = &sA[0][lt * kPcRow + lq * (16 * kPieces)];
  int8_t *const sdst1 = &sA[1][lt * kPcRow + lq * (16 * kPieces)];

  const brsrc rW = make_rsrc(a.W + static_cast<int64_t>(e) * N * K, static_cast<uint32_t>(N * K));
  int woff[2];
  const int wkstride = shuf_kb_stride(static_cast<int>(N / 16));
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const int64_t nr = wave_active ? nrow[rb] : 0;
    if constexpr (SHUF) // 2 KB blocks; k-step j of lane half c reads 16-byte chunk 2j+c
      woff[rb] = static_cast<int>(nr / 16 + (r >> 4)) * shuf_nb_stride(KB) + (c * 16 + (r & 15)) * 16;
    else
      woff[rb] = static_cast<int>((nr + r) * K) + c * 64;
  }

  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  v16i acc[TB][2];
#pragma unroll
  for (int tb = 0; tb < TB; ++tb)
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[tb][rb][i] = 0;

  v4i wreg[2][2][4]; // [buffer][row fragment][k-step]
  v4i areg[kPieces]; // token bytes of the next K block on their way to LDS

  // The loop is free of branches: a step past the end of K re-reads the last K block and
  // stores zeros as token bytes, so it adds nothing.
  auto load_act = [&](int kb) {
    const int kc = kb < KB ? kb : KB - 1;
#pragma unroll
    for (int j = 0; j < kPieces; ++j) areg[j] = bld16(rA, aoff, kc * kGroup + j * 16);
  };
  auto store_act = [&](auto ST, bool live) {
    int8_t *d = decltype(ST)::value ? sdst1 : sdst0;
#pragma unroll
    for (int j = 0; j < kPieces; ++j) *reinterpret_cast<v4i *>(d + j * 16) = live ? areg[j] : v4i{0, 0, 0, 0};
  };
  auto load_w = [&](auto BUF, int kb) {
    constexpr int b = decltype(BUF)::value;
    const int kc = kb < KB ? kb : KB - 1;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        wreg[b][rb][ks] = SHUF ? bld16<kWAux>(rW, woff[rb], kc * wkstride + ks * 512)
                               : bld16<kWAux>(rW, woff[rb], kc * kGroup + ks * 16);
  };
  auto compute = [&](auto BUF) {
    constexpr int b = decltype(BUF)::value;
    const int8_t *tile = sA[b];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
      v4i bf[4];
      // the K bytes of k-step ks must be the ones the weight operand holds for it
      const int8_t *src = tile + (tb * 32 + r) * kPcRow + (SHUF ? c * 16 : c * 64);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) bf[ks] = *reinterpret_cast<const v4i *>(src + (SHUF ? ks * 32 : ks * 16));
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
          acc[tb][rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[b][rb][ks], bf[ks], acc[tb][rb], 0, 0, 0);
    }
  };

  load_act(0);
  load_w(B0{}, 0);
  store_act(B0{}, true);
  __syncthreads();
  for (int kb = 0; kb < KB; kb += 2) {
    // even K block: compute from LDS stage 0 / weight buffer 0 while block kb+1 arrives
    load_act(kb + 1);
    load_w(B1{}, kb + 1);
    __builtin_amdgcn_sched_barrier(0); // keep the prefetch ahead of the MFMAs
    compute(B0{});
    store_act(B1{}, kb + 1 < KB);
    __syncthreads();
    // odd K block (a dead step when K/128 is odd)
    load_act(kb + 2);
    load_w(B0{}, kb + 2);
    __builtin_amdgcn_sched_barrier(0);
    compute(B1{});
    store_act(B0{}, kb + 2 < KB);
    __syncthreads();
  }

  if (!wave_active) return;
  const brsrc rWs = make_rsrc(a.Ws + static_cast<int64_t>(e) * N, static_cast<uint32_t>(N * 4));
  v4f bs4[2][4]; // scales of the 16 rows a lane holds per fragment: rows 8q + 4c + i
#pragma unroll
  for (int rb = 0; rb < 2; ++rb)
#pragma unroll
    for (int q = 0; q < 4; ++q)
      bs4[rb][q] = __builtin_bit_cast(v4f, bld16(rWs, static_cast<int>(nrow[rb] + 8 * q + 4 * c) * 4, 0));
  // the K loop ended with a barrier: the token tile's LDS is free and serves as store staging
  int8_t *stg = &sA[0][0] + wr * (32 * kStgPitch);
#pragma unroll
  for (int tb = 0; tb < TB; ++tb) {
    float ts = 0.0f;
    if (valid[tb]) {
      ts = a.As[f[tb] / a.top_k];
      if (a.mul_routed) ts = a.topk_w[f[tb]] * ts;
    }
    v4u16 o[2][4];
    with_out16(a.out_f16, [&](auto cvt) __attribute__((always_inline)) {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float t = static_cast<float>(acc[tb][rb][4 * q + i]) * ts;
            o[rb][q][i] = cvt(t * bs4[rb][q][i]);
          }
    });
    wave_store_32x64_bf16(stg, o, valid[tb] ? static_cast<int>(f[tb]) : -1, a.C, N, nrow[0], lane);
  }
}

// 128 tokens: 246 registers, two waves per SIMD.  64 tokens: 162 registers, so three workgroups
// fit a compute unit and hide each other's barrier and memory waits better than two.
template <bool SHUF, bool STREAM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void moe_gemm_pc_kernel_128(const GemmArgs a, int m_blocks, int group_m) {
  moe_gemm_pc_body<SHUF, 4, STREAM>(a, m_blocks, group_m);
}
template <bool SHUF, bool STREAM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3)))
void moe_gemm_pc_kernel_64(const GemmArgs a, int m_blocks, int group_m) {
  moe_gemm_pc_body<SHUF, 2, STREAM>(a, m_blocks, group_m);
}

bool gemm_pc_supports(const GemmArgs &a, int block_size_m) {
  return a.per_channel && (block_size_m == 64 || block_size_m == 128) && a.N % 64 == 0;
}

int launch_gemm_pc(const GemmArgs &a0, int block_size_m, int64_t m_blocks, hipStream_t s) {
  GemmArgs a = a0;
  a.n_tiles = static_cast<int32_t>((a.N + 255) / 256);
  // every chunk of G token blocks owns G * n_tiles consecutive slots on one XCD
  int64_t G = a.num_valid / (static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) * block_size_m);
  G = G < 2 ? 2 : (G > 16 ? 16 : G);
  const int64_t chunks = (m_blocks + G - 1) / G;
  const int64_t grid = (chunks + 7) / 8 * (G * a.n_tiles) * 8;
  LO_REQUIRE(grid < (1ll << 31), LO_EINVAL, "moe_gemm_w8a8: grid too large");
  const dim3 g(static_cast<unsigned>(grid)), b(256);
  const int mbi = static_cast<int>(m_blocks), gi = static_cast<int>(G);
  // one token block per expert, by and large: up to 48 slots per expert on average with 64-token blocks
  // (as measured for the block form's 64-token kernel), half a block with 128-token blocks
  // (pre-shuffled weights only: a 128-byte line of row-major weights serves several k-steps of a lane,
  // and the hint would have it fetched again for each)
  const bool stream = a.w_shuffled &&
                      a.num_valid <= static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) *
                                         (block_size_m == 64 ? 48 : 64);
#define LO_PC_LAUNCH(KERN)                                                                    \
  do {                                                                                        \
    if (stream) hipLaunchKernelGGL((KERN<true, true>), g, b, 0, s, a, mbi, gi);               \
    else if (a.w_shuffled) hipLaunchKernelGGL((KERN<true, false>), g, b, 0, s, a, mbi, gi);   \
    else hipLaunchKernelGGL((KERN<false, false>), g, b, 0, s, a, mbi, gi);                    \
  } while (0)
  if (block_size_m == 128) LO_PC_LAUNCH(moe_gemm_pc_kernel_128);
  else LO_PC_LAUNCH(moe_gemm_pc_kernel_64);
#undef LO_PC_LAUNCH
  return check_launch("moe_gemm_w8a8(tile)");
}

} // namespace lo
