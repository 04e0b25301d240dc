// Grouped block-INT8 GEMM for gfx950, 128-token LDS-tiled form with both operands in LDS.
//
// What bounds the 64-token LDS-tiled kernel (gemm_tile.hip) is the rate at which the compute
// units pull operands out of L2: every token block re-reads its expert's weights, and the
// bytes requested per multiply-add are 1/tokens + 1/rows of the workgroup tile.  This kernel
// halves the weight part: a workgroup of eight waves owns 128 gathered tokens x 256 weight
// rows, and every operand byte enters the compute unit once, by direct global -> LDS loads
// (buffer_load ... lds, 16 bytes per lane, no staging registers) into a ring of three stages,
// requested two 128-wide K blocks ahead of their use:
//   weights  the 16 pre-shuffled 2 KB blocks of the tile, copied verbatim (32 KB per stage), so a
//            wave's MFMA operand is read back with the same lane offsets it would use in memory;
//   tokens   128 rows x 128 bytes (16 KB per stage); the 16-byte piece a lane fetches is chosen
//            so that piece p of token t lands in slot p ^ (t & 7) of the row, which makes the
//            operand reads conflict-free without padding;
//   scales   the tokens' group scales (512 bytes per stage, through registers).
// Waves form a 4 (row groups) x 2 (token halves) grid; each owns 64 x 64 outputs as 2 x 2
// fragments of v_mfma_i32_32x32x32_i8 and folds every fragment into fp32 per K block exactly as
// the 64-token kernel does (reference arithmetic: Triton fused_moe_kernel,
// python/lightop/_lmslim_native/layers/fused_moe/int8.py:485-519; fused epilogue :811-823).
// One barrier per K block.
//
// Measured on the benchmark layers this form does not beat two decoupled 64-token workgroups
// per compute unit (first GEMM of the Qwen3-30B-A3B layer at 8192 tokens: 420 us against 380 us;
// DeepSeek-V3 share at 4096 tokens: 322 us against 325 us): with a single workgroup per compute
// unit all eight waves are in the same phase of a step, so nothing fills the gaps around the
// barrier.  It is faster than the eight-wave register-fed variant of gemm_tile.hip and serves
// block_size_m = 128 for pre-shuffled weights; the tile table does not choose that size.
#include <type_traits>

#include "gemm.h"

namespace lo {

typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kDmaTokens = 128;
constexpr int kDmaW = 256 * kGroup;          // weight bytes per stage
constexpr int kDmaA = kDmaTokens * kGroup;   // token bytes per stage
constexpr int kDmaS = kDmaTokens * 4;        // token scales per stage
constexpr int kDmaStage = kDmaW + kDmaA + kDmaS;
constexpr int kDmaStages = 3;
constexpr int kDmaRed = 2 * 2 * 4 * 32 * 4;  // amax exchange of the fused epilogue
constexpr int kDmaLds = kDmaStages * kDmaStage + kDmaRed + 2 * kSiluBandN * 2;

// Step barrier of the K loop.  The wave first waits until all but its six most recent
// vector-memory operations are complete (the copies for the K block after this one stay in
// flight; __syncthreads() would drain them too, because the compiler treats a direct-to-LDS load
// as an LDS write that a workgroup fence must make visible) and until its own LDS writes have
// landed, then joins the barrier.  The memory clobber keeps LDS accesses on their side of it.
__device__ __forceinline__ void step_barrier() {
  asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <bool FUSED_ACT, bool FAST_SCALE>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void moe_gemm_dma_kernel(const GemmArgs a, int m_blocks, int group_m) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  float *const sRed = reinterpret_cast<float *>(smem + kDmaStages * kDmaStage); // [wt][tb][wr][32]
  uint16_t *const sSilu = reinterpret_cast<uint16_t *>(smem + kDmaStages * kDmaStage + kDmaRed);

  int mb, nt;
  if (!tile_of(blockIdx.x, a.n_tiles, m_blocks, group_m, mb, nt)) return;
  if (static_cast<int64_t>(mb) * kDmaTokens >= a.ntpp[0]) return;
  const int e = a.expert_ids[mb];
  if (e >= a.E) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform: scalar address math
  const int wr = wave & 3;  // which 64 weight rows of the tile
  const int wt = wave >> 2; // which 64 tokens of the tile
  const int r = lane & 31, c = lane >> 5;
  const int64_t K = a.K, N = a.N;
  const int KB = static_cast<int>(K / kGroup);
  const int64_t I = N / 2;

  // slots of the two 32-token fragments this lane sees in the accumulator layout
  int64_t f[2];
  bool valid[2];
#pragma unroll
  for (int tb = 0; tb < 2; ++tb) {
    f[tb] = a.sorted[static_cast<int64_t>(mb) * kDmaTokens + wt * 64 + tb * 32 + r];
    valid[tb] = f[tb] < a.num_valid;
  }
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
      if (wave_active && !a.skip_nonlocal) {
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

  uint16_t band_regs[kSiluBandPer];
  if constexpr (FUSED_ACT) silu_band_load(band_regs, a.silu, tid & 255);

  // ---- what this wave copies per K block: 4 KB of weights, 2 KB of token rows -----------------
  const int NBLK = static_cast<int>(N / 16);
  const brsrc rW = make_rsrc(a.W + static_cast<int64_t>(e) * N * K, static_cast<uint32_t>(N * K));
  const brsrc rA = make_rsrc(a.A, static_cast<uint32_t>(a.a_rows * K));
  const brsrc rAs = make_rsrc(a.As, static_cast<uint32_t>(a.a_rows * KB * 4));
  const int wkstride = shuf_kb_stride(NBLK);
  int wvoff[4]; // 1 KB pieces wave*4 + j of the stage's 32: 2 KB block (wave*4 + j) / 2, half (wave*4 + j) & 1
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int piece = wave * 4 + j, blk = piece >> 1;
    int64_t nb; // 16-row block of the expert that LDS block `blk` mirrors
    if constexpr (FUSED_ACT) nb = (blk < 8 ? 0 : I / 16) + static_cast<int64_t>(nt) * 8 + (blk & 7);
    else nb = static_cast<int64_t>(nt) * 16 + blk;
    if (nb >= NBLK) nb = 0; // rows past N: computed on block 0, never stored
    wvoff[j] = static_cast<int>(nb) * shuf_nb_stride(KB) + (piece & 1) * 1024 + lane * 16;
  }
  int avoff[2]; // 1 KB pieces wave*2 + j of the stage's 16: eight token rows each
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int t = (wave * 2 + j) * 8 + (lane >> 3);
    const int64_t lf = a.sorted[static_cast<int64_t>(mb) * kDmaTokens + t];
    const int64_t lrow = (lf < a.num_valid) ? lf / a.top_k : 0;
    const int piece = (lane & 7) ^ (t & 7); // slot lane & 7 of row t holds piece slot ^ (t & 7)
    avoff[j] = static_cast<int>(lrow * K) + piece * 16;
  }
  // token scales: thread t < 128 carries the scale of token t
  int asoff = 0;
  if (tid < kDmaTokens) {
    const int64_t lf = a.sorted[static_cast<int64_t>(mb) * kDmaTokens + tid];
    const int64_t lrow = (lf < a.num_valid) ? lf / a.top_k : 0;
    asoff = static_cast<int>(lrow * KB * 4);
  }
  const int NB = static_cast<int>((N + kGroup - 1) / kGroup);
  const float *wsrow[2];
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const int64_t nr = wave_active ? nrow[rb] : 0;
    wsrow[rb] = a.Ws + (static_cast<int64_t>(e) * NB + nr / kGroup) * KB;
  }

  // Six direct global -> LDS loads per wave and K block, the last VMEM operations of a step.
  // All eight waves pass the step barrier together, and the texture path takes 16 bytes per lane
  // at a limited rate, so the copies are issued in three pairs spread over the step's MFMAs
  // rather than in one burst that every wave would wait behind.
  auto copy_pair = [&](int stage, int kb, auto PAIR) {
    constexpr int p = decltype(PAIR)::value;
    const int kc = kb < KB ? kb : KB - 1;
    int8_t *base = smem + stage * kDmaStage;
    if constexpr (p < 2) {
#pragma unroll
      for (int j = 2 * p; j < 2 * p + 2; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rW, base + (wave * 4 + j) * 1024, 16, wvoff[j], kc * wkstride, 0, 0);
    } else {
#pragma unroll
      for (int j = 0; j < 2; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rA, base + kDmaW + (wave * 2 + j) * 1024, 16, avoff[j], kc * kGroup, 0,
                                                 0);
    }
  };
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using P2 = std::integral_constant<int, 2>;
  auto copy_stage = [&](int stage, int kb) {
    copy_pair(stage, kb, P0{});
    copy_pair(stage, kb, P1{});
    copy_pair(stage, kb, P2{});
  };
  auto load_scale = [&](int kb) { return bld_f32(rAs, asoff, (kb < KB ? kb : KB - 1) * 4); };
  auto stage_scales = [&](int stage) { return reinterpret_cast<float *>(smem + stage * kDmaStage + kDmaW + kDmaA); };

  // ---- operand read offsets inside a stage ------------------------------------------------------
  int wlds[2]; // weight fragment rb, k-step 0
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const int blk = FUSED_ACT ? (rb * 8 + wr * 2) : (wr * 4 + rb * 2);
    wlds[rb] = (blk + (r >> 4)) * 2048 + (c * 16 + (r & 15)) * 16;
  }
  int alds[2][4]; // token fragment tb, k-step ks: piece 2*ks + c of token row t sits in slot piece ^ (t & 7)
#pragma unroll
  for (int tb = 0; tb < 2; ++tb)
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int t = wt * 64 + tb * 32 + r;
      alds[tb][ks] = kDmaW + t * kGroup + (((2 * ks + c) ^ (t & 7)) * 16);
    }

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

  auto fold = [&](const v16i &d, float as, float bs, float *dst) {
    if constexpr (FAST_SCALE) {
      const float sc = as * bs;
#pragma unroll
      for (int i = 0; i < 16; ++i) dst[i] = __builtin_fmaf(static_cast<float>(d[i]), sc, dst[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float t = static_cast<float>(d[i]) * as;
        t = t * bs;
        dst[i] = dst[i] + t;
      }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(dst[i])); // keep the fold here
  };
  // The fold of a step's last fragment pair is carried over the step barrier: it needs no LDS, so
  // it runs while the next step's operand reads are in flight instead of leaving the matrix pipe
  // idle at the end of every step (all waves of the workgroup are in the same phase, nobody else
  // would fill that gap).
  v16i dcar[2] = {zero16, zero16};
  float as_car = 0.0f, bs_car[2] = {0.0f, 0.0f};
  auto compute = [&](int stage, const float (&bs)[2], int next_stage, int next_kb) {
    const int8_t *base = smem + stage * kDmaStage;
    const float *sS = reinterpret_cast<const float *>(base + kDmaW + kDmaA);
    v4i wf[2][4];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) wf[rb][ks] = *reinterpret_cast<const v4i *>(base + wlds[rb] + ks * 512);
    v4i bf0[4], bf1[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) bf0[ks] = *reinterpret_cast<const v4i *>(base + alds[0][ks]);
    const float as0 = sS[wt * 64 + r], as1 = sS[wt * 64 + 32 + r];
    copy_pair(next_stage, next_kb, P0{});
    __builtin_amdgcn_sched_barrier(0);
    // previous step's second token fragment
    fold(dcar[0], as_car, bs_car[0], acc[1][0]);
    fold(dcar[1], as_car, bs_car[1], acc[1][1]);
    __builtin_amdgcn_sched_barrier(0);
    // Two fragments (both row groups of one token fragment) run as interleaved MFMA chains, so
    // that consecutive MFMAs of a wave never depend on each other.
    v16i d0[2] = {zero16, zero16};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) d0[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[rb][ks], bf0[ks], d0[rb], 0, 0, 0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) bf1[ks] = *reinterpret_cast<const v4i *>(base + alds[1][ks]);
    copy_pair(next_stage, next_kb, P1{});
    __builtin_amdgcn_sched_barrier(0);
    v16i d1[2] = {zero16, zero16};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) d1[rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[rb][ks], bf1[ks], d1[rb], 0, 0, 0);
    copy_pair(next_stage, next_kb, P2{});
    // first token fragment of this step, while the second one's MFMAs run
    fold(d0[0], as0, bs[0], acc[0][0]);
    fold(d0[1], as0, bs[1], acc[0][1]);
    __builtin_amdgcn_sched_barrier(0);
    dcar[0] = d1[0];
    dcar[1] = d1[1];
    as_car = as1;
    bs_car[0] = bs[0];
    bs_car[1] = bs[1];
  };

  // ---- prologue: K blocks 0 and 1 on their way, scales of block 0 in place ----------------------
  float s_now = 0.0f, s_pending = 0.0f; // thread t < 128: scale of token t for K block 0 / 1
  if (tid < kDmaTokens) {
    s_now = load_scale(0);
    s_pending = load_scale(1);
  }
  float bs_next[2];
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) bs_next[rb] = wsrow[rb][0];
  __builtin_amdgcn_sched_barrier(0);
  copy_stage(0, 0);
  copy_stage(1, 1);
  __builtin_amdgcn_sched_barrier(0);
  if (tid < kDmaTokens) stage_scales(0)[tid] = s_now;
  if constexpr (FUSED_ACT)
    if (tid < 256) silu_band_store(sSilu, band_regs, tid);

  int st = 0; // stage of K block kb
  for (int kb = 0; kb < KB; ++kb) {
    // my copies for K block kb were issued two steps ago: everything but the newest six has landed
    step_barrier(); // so have everyone else's, and nobody still reads the stage refilled below
    const int st1 = st == 2 ? 0 : st + 1, st2 = st1 == 2 ? 0 : st1 + 1;
    float bs[2] = {bs_next[0], bs_next[1]};
    if (tid < kDmaTokens) {
      stage_scales(st1)[tid] = kb + 1 < KB ? s_pending : 0.0f;
      s_pending = load_scale(kb + 2);
    }
    const int kn = kb + 1 < KB ? kb + 1 : KB - 1;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) bs_next[rb] = wsrow[rb][kn];
    __builtin_amdgcn_sched_barrier(0);
    compute(st, bs, st2, kb + 2);
    st = st1;
  }
  fold(dcar[0], as_car, bs_car[0], acc[1][0]);
  fold(dcar[1], as_car, bs_car[1], acc[1][1]);
  __builtin_amdgcn_s_waitcnt(0); // no copy may still be writing LDS when the epilogue reuses it or the wave ends

  if constexpr (!FUSED_ACT) {
    __syncthreads(); // every wave's copies have landed and its operand reads are done: the stages are free
    if (!wave_active) return;
    int8_t *stg = smem + wave * (32 * kStgPitch);
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      float w = 1.0f;
      if (a.mul_routed && valid[tb]) w = a.topk_w[f[tb]];
      v4u16 o[2][4];
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float v = acc[tb][rb][4 * q + i];
            if (a.mul_routed) v = v * w;
            o[rb][q][i] = f32_to_bf16(v);
          }
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
      if (c == 0) sRed[((wt * 2 + tb) * 4 + wr) * 32 + r] = amax;
    }
    __syncthreads(); // also: every wave's copies have landed and its operand reads are done
    const int64_t G = I / kGroup;
    // the quantised tile (128 tokens x 128 columns of int8) leaves through LDS as whole rows
    constexpr int kQPitch = kGroup + 16;
    int8_t *qst = smem;
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      const float *red = sRed + (wt * 2 + tb) * 4 * 32 + r;
      float amax = fmaxf(fmaxf(red[0], red[32]), fmaxf(red[64], red[96]));
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
    for (int j = 0; j < kDmaTokens * 8 / 512; ++j) {
      const int id = tid + 512 * j, tok = id >> 3, piece = id & 7;
      const int64_t ft = a.sorted[static_cast<int64_t>(mb) * kDmaTokens + tok];
      if (ft < a.num_valid)
        *reinterpret_cast<v4i *>(a.A2q + ft * I + static_cast<int64_t>(nt) * kGroup + piece * 16) =
            *reinterpret_cast<const v4i *>(qst + tok * kQPitch + piece * 16);
    }
  }
}

bool gemm_dma_supports(const GemmArgs &a, bool fused_act, int block_size_m) {
  if (block_size_m != 128 || !a.w_shuffled || a.w4 || a.per_channel) return false;
  if (!fused_act && a.N % 64 != 0) return false;
  return true;
}

int launch_gemm_dma(const GemmArgs &a0, bool fused_act, int flags, int64_t m_blocks, hipStream_t s) {
  GemmArgs a = a0;
  a.n_tiles = fused_act ? static_cast<int32_t>(a.N / 2 / kGroup) : static_cast<int32_t>((a.N + 255) / 256);
  int64_t G = a.num_valid / (static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) * kDmaTokens);
  G = G < 2 ? 2 : (G > 16 ? 16 : G);
  const int64_t chunks = (m_blocks + G - 1) / G;
  const int64_t grid = (chunks + 7) / 8 * (G * a.n_tiles) * 8;
  LO_REQUIRE(grid < (1ll << 31), LO_EINVAL, "moe_gemm: grid too large");
  const bool fast = (flags & LO_GEMM_FUSED_SCALE) != 0 || (flags & LO_GEMM_CANONICAL_ORDER) == 0;
  const dim3 g(static_cast<unsigned>(grid)), b(512);
  const int mbi = static_cast<int>(m_blocks), gi = static_cast<int>(G);
#define LO_DMA_LAUNCH(FA, FS)                                                                                   \
  do {                                                                                                          \
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&moe_gemm_dma_kernel<FA, FS>),                       \
                            hipFuncAttributeMaxDynamicSharedMemorySize, kDmaLds) != hipSuccess) {               \
      set_error("moe_gemm(dma): cannot reserve %d bytes of LDS", kDmaLds);                                      \
      return LO_ELAUNCH;                                                                                        \
    }                                                                                                           \
    hipLaunchKernelGGL((moe_gemm_dma_kernel<FA, FS>), g, b, kDmaLds, s, a, mbi, gi);                            \
  } while (0)
  if (fused_act) {
    if (fast) LO_DMA_LAUNCH(true, true);
    else LO_DMA_LAUNCH(true, false);
  } else {
    if (fast) LO_DMA_LAUNCH(false, true);
    else LO_DMA_LAUNCH(false, false);
  }
#undef LO_DMA_LAUNCH
  return check_launch(fused_act ? "moe_gemm1_silu_quant(dma)" : "moe_gemm(dma)");
}

} // namespace lo
