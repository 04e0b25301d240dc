// Grouped block-INT8 GEMM for gfx950, LDS-tiled form for the compute-bound regime.
//
// Workgroup tile: 64 gathered token rows x 256 weight rows with 4 wavefronts (the default; two
// such workgroups share a compute unit), or 128 x 256 with 8 wavefronts in a 4 (rows) x 2
// (tokens) arrangement.  Each wave owns a 64 x 64 piece as 2 x 2 fragments of
// v_mfma_i32_32x32x32_i8, with the weight fragment as the A operand and the token
// fragment as the B operand; accumulators and the int32 partial sums stay in VGPRs
// (64 + 32 registers), so two waves share a SIMD and one wave's MFMAs overlap the other
// wave's conversion and scaling.  Weight fragments go from global memory (pre-shuffled
// layout: 1 KB contiguous per operand) straight into registers; the token tile of the
// current 128-wide K block is gathered through sorted_token_ids into a double-buffered,
// row-padded LDS tile together with the tokens' group scales.  One barrier per K block.
//
// Per K block every 32x32 fragment is accumulated exactly in int32 (4 MFMAs) and then
// folded into the fp32 accumulator with the token's group scale and the weight block's
// scale (reference: Triton fused_moe_kernel, python/lightop/_lmslim_native/layers/
// fused_moe/int8.py:485-519).  With FUSED_ACT the two fragments of a wave are 32 gate
// rows and the matching 32 up rows, and the epilogue applies bf16 rounding,
// SiLU(gate)*up and the 1x128 re-quantisation (int8.py:811-823) before anything is
// written.
#include <type_traits>

#include "gemm.h"

namespace lo {

typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTileRow = 144;    // LDS row pitch in bytes: 128 + 16 keeps ds_read_b128 conflict-free

// WT = number of 64-token halves per workgroup: 2 -> 128-token tile, 8 waves, one
// workgroup per CU; 1 -> 64-token tile, 4 waves, two workgroups per CU that are not
// synchronised with each other, so one computes while the other waits at its barrier.
//
// STREAM (64-token tiles of pre-shuffled weights): an expert's weights are read by one token block,
// by and large, and are loaded with the streaming cache policy (first GEMM of the Qwen3-30B-A3B
// layer at 512 tokens 132 -> 74 us).  With several token blocks per expert the blocks share the
// weights through L2 and the default policy is the faster one; with row-major weights, where a
// 128-byte line serves several k-steps of a lane, the hint costs 50 %.
template <bool FUSED_ACT, int ORD, bool SHUF, int WT, bool STREAM = false>
__global__ __launch_bounds__(256 * WT) __attribute__((amdgpu_waves_per_eu(2, 2)))
void moe_gemm_tile_kernel(const GemmArgs a, int m_blocks, int group_m) {
  static_assert(!STREAM || (SHUF && WT == 1), "streaming policy: 64-token tiles of pre-shuffled weights");
  constexpr int kWAux = STREAM ? kCacheStream : kCacheDefault;
  constexpr int kTileM = 64 * WT; // tokens per workgroup
  __shared__ __attribute__((aligned(16))) int8_t sA[2][kTileM * kTileRow];
  __shared__ float sS[2][kTileM];
  __shared__ float sRed[WT][2][4][32];
  __shared__ uint16_t sSilu[FUSED_ACT ? 2 * kSiluBandN : 2];

  int mb, nt;
  if (!tile_of(blockIdx.x, a.n_tiles, m_blocks, group_m, mb, nt)) return;
  if (static_cast<int64_t>(mb) * kTileM >= a.ntpp[0]) return;
  // An expert_map entry outside the weight tensor is treated like an expert of another rank, but its
  // rows are always zero-filled: the slot mask of the alignment counts such a slot as local.
  const int e_raw = a.expert_ids[mb];
  const bool e_oob = e_raw >= a.E;
  const int e = e_oob ? -1 : e_raw;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform: scalar address math
  const int wr = wave & 3;  // which 64 weight rows of the tile
  const int wt = wave >> 2; // which 64 tokens of the tile (always 0 when WT == 1)
  const int r = lane & 31, c = lane >> 5;
  const int64_t K = a.K, N = a.N;
  const int KB = static_cast<int>(K / kGroup);
  const int64_t I = N / 2;

  // slots of the two 32-token fragments this lane sees in the accumulator layout
  int64_t f[2];
  bool valid[2];
#pragma unroll
  for (int tb = 0; tb < 2; ++tb) {
    f[tb] = a.sorted[static_cast<int64_t>(mb) * kTileM + wt * 64 + tb * 32 + r];
    valid[tb] = f[tb] < a.num_valid;
  }

  // weight rows of the wave: two 32-row fragments
  int64_t nrow[2];
  if constexpr (FUSED_ACT) {
    nrow[0] = static_cast<int64_t>(nt) * kGroup + wr * 32;
    nrow[1] = I + nrow[0];
  } else {
    nrow[0] = static_cast<int64_t>(nt) * 256 + wr * 64;
    nrow[1] = nrow[0] + 32;
  }
  const bool wave_active = FUSED_ACT || nrow[0] < N; // N % 64 == 0 is checked on the host

  if (e < 0) {
    if constexpr (!FUSED_ACT) {
      if (wave_active && (!a.skip_nonlocal || e_oob)) {
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
          if (valid[tb])
#pragma unroll
            for (int rb = 0; rb < 2; ++rb)
#pragma unroll
              for (int q = 0; q < 4; ++q)
                *reinterpret_cast<v2i *>(a.C + f[tb] * N + nrow[rb] + 8 * q + 4 * c) = v2i{0, 0};
      }
    }
    return;
  }

  // the SiLU band for the epilogue: requested first, so it arrives behind the loads below
  uint16_t band_regs[kSiluBandPer];
  if constexpr (FUSED_ACT) silu_band_load(band_regs, a.silu, tid & 255);

  // cooperative gather role: thread -> (token, 32-byte quarter of the 128-byte K block)
  const int lt = tid >> 2, lq = tid & 3;
  const int64_t lf = a.sorted[static_cast<int64_t>(mb) * kTileM + lt];
  const int64_t lrow = (lf < a.num_valid) ? lf / a.top_k : 0;
  const brsrc rA = make_rsrc(a.A, static_cast<uint32_t>(a.a_rows * K));
  const brsrc rAs = make_rsrc(a.As, static_cast<uint32_t>(a.a_rows * KB * 4));
  const int aoff = static_cast<int>(lrow * K) + lq * 32;
  const int asoff = static_cast<int>(lrow * KB * 4);
  int8_t *const sdst0 = &sA[0][lt * kTileRow + lq * 32];
  int8_t *const sdst1 = &sA[1][lt * kTileRow + lq * 32];

  const int NB = static_cast<int>((N + kGroup - 1) / kGroup);
  const brsrc rW = make_rsrc(a.W + static_cast<int64_t>(e) * N * K, static_cast<uint32_t>(N * K));
  int woff[2];
  const float *wsrow[2];
  const int wkstride = shuf_kb_stride(static_cast<int>(N / 16));
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const int64_t nr = wave_active ? nrow[rb] : 0;
    if constexpr (SHUF) // 2 KB blocks; k-step j of lane half c reads 16-byte chunk 2j+c
      woff[rb] = static_cast<int>(nr / 16 + (r >> 4)) * shuf_nb_stride(KB) + (c * 16 + (r & 15)) * 16;
    else
      woff[rb] = static_cast<int>((nr + r) * K) + c * 64;
    wsrow[rb] = a.Ws + (static_cast<int64_t>(e) * NB + nr / kGroup) * KB;
  }

  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  v16i zero16;
#pragma unroll
  for (int i = 0; i < 16; ++i) zero16[i] = 0;
  float acc[2][2][16]; // [token fragment][row fragment][element]
#pragma unroll
  for (int tb = 0; tb < 2; ++tb)
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[tb][rb][i] = 0.0f;

  v4i wreg[2][2][4]; // [buffer][row fragment][k-step]
  float bsc[2][2];   // [buffer][row fragment] weight-block scales, fetched with the fragments
  v4i areg[2][2]; // [set][16-byte piece]: token bytes in flight for two K blocks
  float sreg[2] = {0.0f, 0.0f};

  // The K loop is free of branches (branches around the loads make the compiler wait for
  // all of them): a step past the end of K re-reads the last K block and stores a token
  // scale of zero, so it adds exactly 0 to every accumulator.
  // The token bytes of K block kb are requested two iterations before they are needed
  // and written to LDS one iteration before: set = kb & 1 in registers, stage = kb & 1
  // in LDS.
  auto load_act = [&](auto SET, int kb) {
    constexpr int st = decltype(SET)::value;
    const int kc = kb < KB ? kb : KB - 1;
#pragma unroll
    for (int j = 0; j < 2; ++j) areg[st][j] = bld16(rA, aoff, kc * kGroup + j * 16);
    sreg[st] = bld_f32(rAs, asoff, kc * 4);
  };
  auto store_act = [&](auto SET, bool live) {
    constexpr int st = decltype(SET)::value;
    int8_t *d = st ? sdst1 : sdst0;
#pragma unroll
    for (int j = 0; j < 2; ++j) *reinterpret_cast<v4i *>(d + j * 16) = areg[st][j];
    if (lq == 0) sS[st][lt] = live ? sreg[st] : 0.0f;
  };
  auto load_w = [&](auto BUF, int kb) {
    constexpr int b = decltype(BUF)::value;
    const int kc = kb < KB ? kb : KB - 1;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        wreg[b][rb][ks] = SHUF ? bld16<kWAux>(rW, woff[rb], kc * wkstride + ks * 512)
                               : bld16(rW, woff[rb], kc * kGroup + ks * 16);
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) bsc[b][rb] = wsrow[rb][kc];
  };
  auto fold = [&](const v16i &d, float as, float bs, float *dst) {
    const float sc = ORD == kOrdFusedScale ? as * bs : 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) dst[i] = fold_elem<ORD>(d[i], sc, as, bs, dst[i]);
    // The accumulators must be final here: an empty asm that "modifies" them stops the
    // optimiser from postponing the fold (and keeping the int32 fragment alive instead).
#pragma unroll
    for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(dst[i]));
  };
  auto compute = [&](auto BUF) {
    constexpr int b = decltype(BUF)::value;
    const int8_t *tile = sA[b];
    // The four 32x32 fragments are software-pipelined: the MFMAs of one fragment are
    // issued, then the previous fragment is folded into the fp32 accumulators while the
    // matrix pipe works.  The scheduling barriers keep the compiler from batching all
    // MFMAs first and all conversions last, which would keep four int32 fragments alive.
    v16i dprev = zero16;
    float as_prev = 0.0f;
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      v4i bf[4];
      // the K bytes of k-step ks must be the ones the weight operand holds for it
      const int8_t *src = tile + (wt * 64 + tb * 32 + r) * kTileRow + (SHUF ? c * 16 : c * 64);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        bf[ks] = *reinterpret_cast<const v4i *>(src + (SHUF ? ks * 32 : ks * 16));
      const float as = sS[b][wt * 64 + tb * 32 + r];
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        v16i d = zero16;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
          d = __builtin_amdgcn_mfma_i32_32x32x32_i8(wreg[b][rb][ks], bf[ks], d, 0, 0, 0);
        if (tb + rb > 0) {
          const int ptb = rb ? tb : tb - 1, prb = rb ? 0 : 1;
          fold(dprev, as_prev, bsc[b][prb], acc[ptb][prb]);
        }
        __builtin_amdgcn_sched_barrier(0);
        dprev = d;
        as_prev = as;
      }
    }
    fold(dprev, as_prev, bsc[b][1], acc[1][1]);
    __builtin_amdgcn_sched_barrier(0);
  };

  load_act(B0{}, 0);
  load_act(B1{}, 1);
  load_w(B0{}, 0);
  store_act(B0{}, true);
  if constexpr (FUSED_ACT)
    if (tid < 256) silu_band_store(sSilu, band_regs, tid);
  __syncthreads();
  for (int kb = 0; kb < KB; kb += 2) {
    // even K block: compute from LDS stage 0 / weight buffer 0
    load_act(B0{}, kb + 2);            // needed in two iterations
    load_w(B1{}, kb + 1);              // needed in the next iteration
    __builtin_amdgcn_sched_barrier(0); // keep the prefetch ahead of the MFMAs
    compute(B0{});
    store_act(B1{}, kb + 1 < KB);      // requested one iteration ago
    __syncthreads();
    // odd K block (a dead step when K/128 is odd: zero token scales)
    load_act(B1{}, kb + 3);
    load_w(B0{}, kb + 2);
    __builtin_amdgcn_sched_barrier(0);
    compute(B1{});
    store_act(B0{}, kb + 2 < KB);
    __syncthreads();
  }

  if constexpr (!FUSED_ACT) {
    if (!wave_active) return;
    // the K loop ended with a barrier: the token tile's LDS is free and serves as store staging
    int8_t *stg = &sA[0][0] + wave * (32 * kStgPitch);
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      float w = 1.0f;
      if (a.mul_routed && valid[tb]) w = a.topk_w[f[tb]];
      v4u16 o[2][4];
      with_out16(a.out_f16, [&](auto cvt) __attribute__((always_inline)) {
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              float v = acc[tb][rb][4 * q + i];
              if (a.mul_routed) v = v * w;
              o[rb][q][i] = cvt(v);
            }
      });
      wave_store_32x64_bf16(stg, o, valid[tb] ? static_cast<int>(f[tb]) : -1, a.C, N, nrow[0], lane);
    }
  } else {
    // acc[.][0] = gate, acc[.][1] = up for activation columns nt*128 + wr*32 + 8q + 4c + i
    float actf[2][16];
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      float w = 1.0f;
      if (a.mul_routed && valid[tb]) w = a.topk_w[f[tb]];
      float amax = 0.0f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float g = acc[tb][0][i], u = acc[tb][1][i];
        if (a.mul_routed) {
          g = g * w;
          u = u * w;
        }
        const uint16_t act16 = silu_mul_band(sSilu, a.silu, f32_to_bf16(g), f32_to_bf16(u));
        actf[tb][i] = bf16_to_f32(act16);
        amax = fmaxf(amax, fabsf(actf[tb][i]));
      }
      amax = fmaxf(amax, __shfl_xor(amax, 32));
      if (c == 0) sRed[wt][tb][wr][r] = amax;
    }
    __syncthreads();
    const int64_t G = I / kGroup;
    // The quantised tile (kTileM tokens x 128 columns of int8) goes through LDS as well, so that
    // it leaves as whole 128-byte rows instead of 4-byte pieces; the token tile's LDS is free.
    constexpr int kQPitch = kGroup + 16;
    int8_t *qst = &sA[0][0];
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      float amax = fmaxf(fmaxf(sRed[wt][tb][0][r], sRed[wt][tb][1][r]),
                         fmaxf(sRed[wt][tb][2][r], sRed[wt][tb][3][r]));
      amax = fmaxf(amax, 1e-10f);
      const float sc = amax / 127.0f;
      const float rsc = 1.0f / sc;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<uint32_t *>(qst + (wt * 64 + tb * 32 + r) * kQPitch + wr * 32 + 8 * q + 4 * c) =
            quant4(&actf[tb][4 * q], sc, rsc);
      if (valid[tb] && wr == 0 && c == 0) a.A2s[f[tb] * G + nt] = sc;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kTileM * 8 / (256 * WT); ++j) {
      const int id = tid + 256 * WT * j, tok = id >> 3, piece = id & 7;
      const int64_t ft = a.sorted[static_cast<int64_t>(mb) * kTileM + tok];
      if (ft < a.num_valid)
        *reinterpret_cast<v4i *>(a.A2q + ft * I + static_cast<int64_t>(nt) * kGroup + piece * 16) =
            *reinterpret_cast<const v4i *>(qst + tok * kQPitch + piece * 16);
    }
  }
}

bool gemm_tile_supports(const GemmArgs &a, bool fused_act, int block_size_m) {
  if (block_size_m != 128 && block_size_m != 64) return false;
  if (!fused_act && a.N % 64 != 0) return false;
  return true;
}

int launch_gemm_tile(const GemmArgs &a0, bool fused_act, int block_size_m, int flags, int64_t m_blocks,
                     hipStream_t s) {
  GemmArgs a = a0;
  a.n_tiles = fused_act ? static_cast<int32_t>(a.N / 2 / kGroup) : static_cast<int32_t>((a.N + 255) / 256);
  // every chunk of G token blocks owns G * n_tiles consecutive slots on one XCD
  int64_t G = a.num_valid / (static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) * block_size_m);
  G = G < 2 ? 2 : (G > 16 ? 16 : G);
  const int64_t chunks = (m_blocks + G - 1) / G;
  const int64_t grid = (chunks + 7) / 8 * (G * a.n_tiles) * 8;
  LO_REQUIRE(grid < (1ll << 31), LO_EINVAL, "moe_gemm: grid too large");
  const int ord = scale_order(flags);
  const int wt = block_size_m / 64;
  const dim3 g(static_cast<unsigned>(grid)), b(256 * wt);
  const int mbi = static_cast<int>(m_blocks);
#define LO_TILE_LAUNCH2(FA, FS, SH)                                                             \
  do {                                                                                          \
    if (wt == 2) hipLaunchKernelGGL((moe_gemm_tile_kernel<FA, FS, SH, 2>), g, b, 0, s, a, mbi, static_cast<int>(G)); \
    else hipLaunchKernelGGL((moe_gemm_tile_kernel<FA, FS, SH, 1>), g, b, 0, s, a, mbi, static_cast<int>(G));         \
  } while (0)
  // one token block per expert, by and large (measured up to 48 slots per expert on average: first GEMM
  // of the Qwen3-30B-A3B layer at 768 tokens 135 -> 88 us; at 64 the second GEMM loses more than
  // the first one gains)
  const bool stream = a.w_shuffled && wt == 1 &&
                      a.num_valid <= static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) * 48;
#define LO_TILE_LAUNCH(FS, FA)                         \
  do {                                                 \
    if (stream)                                        \
      hipLaunchKernelGGL((moe_gemm_tile_kernel<FA, FS, true, 1, true>), g, b, 0, s, a, mbi, static_cast<int>(G)); \
    else if (a.w_shuffled) LO_TILE_LAUNCH2(FA, FS, true);   \
    else LO_TILE_LAUNCH2(FA, FS, false);               \
  } while (0)
  if (fused_act) LO_ORD_DISPATCH(ord, LO_TILE_LAUNCH, true);
  else LO_ORD_DISPATCH(ord, LO_TILE_LAUNCH, false);
#undef LO_TILE_LAUNCH
#undef LO_TILE_LAUNCH2
  return check_launch(fused_act ? "moe_gemm1_silu_quant(tile)" : "moe_gemm(tile)");
}

} // namespace lo
