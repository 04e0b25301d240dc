// Grouped block-INT8 GEMM for gfx950, 128-token form with two independent workgroups per
// compute unit.
//
// The LDS-tiled kernels are bound by the rate at which compute units pull operands out of L2:
// bytes requested per multiply-add are 1/tokens + 1/rows of the workgroup tile.  A 128-token
// tile needs 128 fp32 accumulators per lane when four waves share 256 weight rows, which leaves
// no room for weight fragments double-buffered in registers (gemm_tile.hip) at two waves per
// SIMD, and a single eight-wave workgroup per compute unit (gemm_dma.hip) runs phase-locked.
// Here every operand byte enters the compute unit once by direct global -> LDS loads
// (buffer_load ... lds) and costs no staging registers, so four waves hold 128 tokens x 256
// rows in 72 KB of LDS and two such workgroups share a compute unit:
//   weights  each wave copies its own rows: per 128-wide K block four pre-shuffled 2 KB blocks
//            into a private 8 KB stage.  The wave reads the stage into registers at the start of
//            a K block and refills it at once with the next K block, so the stage needs no
//            barrier and no second copy, and is requested a whole K block ahead;
//   tokens   128 rows x 128 bytes per K block into a two-stage ring shared by the workgroup
//            (16-byte pieces XOR-swizzled by row, conflict-free operand reads), requested one K
//            block ahead; one barrier per K block.  Every wave reads each token fragment once per
//            K block and uses it against all 64 of its rows: LDS bandwidth is what this kernel
//            runs out of first;
//   scales   the tokens' group scales, through registers, one K block ahead; the weight-block
//            scales of the tile's rows (two per K block) go to LDS once, before the K loop, so
//            that the loop issues no vector-memory operation whose result it has to wait for
//            (the wait would also drain the copies in flight).
// A wave owns 64 rows x 128 tokens as 4 x 8 fragments of v_mfma_i32_16x16x64_i8 (weights as
// the A operand) and folds each fragment's exact int32 sum over a K block into fp32 as the
// 64-token kernel does (reference arithmetic: Triton fused_moe_kernel,
// python/lightop/_lmslim_native/layers/fused_moe/int8.py:485-519; fused epilogue :811-823).
#include <type_traits>

#include "gemm.h"

namespace lo {

constexpr int kT = 128;                       // tokens per workgroup
constexpr int kTWStage = 8192;                // one wave's weights for one K block
constexpr int kTW = 4 * kTWStage;             // [wave]
constexpr int kTAStage = kT * kGroup;         // token rows of one K block
constexpr int kTA = 2 * kTAStage;
constexpr int kTS = 2 * kT * 4;               // [stage][token] scales
constexpr int kTRed = 4 * kT * 4;             // [wave][token] amax exchange of the fused epilogue
constexpr int kTMaxKB = 128;                  // K blocks whose weight-block scales fit the table below
constexpr int kTBs = 2 * kTMaxKB * 4;         // [fragment][K block] weight-block scales of the tile
constexpr int kTIds = kT * 4;                  // the tile's sorted ids, for the epilogues
constexpr int kTLds = kTW + kTA + kTS + kTRed + kTBs + kTIds + 2 * kSiluBandN * 2;
// NTB = 10: 160 tokens per workgroup (plain epilogue only: no amax exchange, no SiLU band; int8 block
// form, or int4 weights with per-channel scales, whose int32 accumulators need no fold registers), for layers
// whose experts see a few tokens more than 128: a remainder block is a second pass over the expert's
// weights, and at that size the weights are what the stage streams.
constexpr int kT160 = 160;
constexpr int kTLds160 = kTW + 2 * kT160 * kGroup + 2 * kT160 * 4 + kTBs + kT160 * 4;
constexpr int kTPitch = 144;                  // staging pitch of the epilogues: 128 + 16

// Wait until all but the newest `N` vector-memory operations of this wave are complete and its
// LDS operations have landed.  (__syncthreads() would drain every copy in flight: the compiler
// treats a direct-to-LDS load as an LDS write that a workgroup fence must make visible.)
template <int N>
__device__ __forceinline__ void wait_copies() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_copies_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

//
// PC (with W4): the reference's own int4 form (fused_moe_kernel_int4_w4a8,
// python/lightop/_lmslim_native/layers/fused_moe/w4a8.py:341-395): one scale per token row and one
// per weight row, both applied in the epilogue, so the int32 sums run over the whole K inside the
// MFMA accumulators and the K loop has no scale arithmetic at all.
template <bool FUSED_ACT, int ORD, bool STREAM, bool W4, bool PC = false, int NTB = 8>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void moe_gemm_t128_kernel(const GemmArgs a, int m_blocks, int group_m) {
  static_assert(!PC || (!FUSED_ACT && ORD == kOrdSeparate && (W4 || NTB == 10)),
                "per-channel scales: plain GEMM, int4 weights or 160-token tiles of int8 weights");
  static_assert(NTB == 8 || (NTB == 10 && (PC || !W4)),
                "160-token tiles: int8 block form (plain or fused epilogue) or per-channel scales");
  constexpr int T = 16 * NTB;        // tokens per workgroup
  constexpr int AST = T * kGroup;    // token rows of one K block
  constexpr int APW = NTB / 2;       // 1 KB pieces (eight token rows) of a token stage that a wave copies
  constexpr int RED = NTB == 8 ? kTRed : 0;
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  int8_t *const sA = smem + kTW;
  float *const sS = reinterpret_cast<float *>(smem + kTW + 2 * AST);
  // 160-token tiles have no room for the fused epilogue's amax exchange and SiLU band beside the stages
  // (two workgroups per compute unit): there every wave copies the band into its own weight stage once its K
  // loop is done, and its row of the exchange lies behind the band.
  constexpr bool kLateBand = FUSED_ACT && NTB == 10;
  static_assert(!kLateBand || 2 * kSiluBandN * 2 + 160 * 4 <= kTWStage, "band and amax row fit a weight stage");
  auto red_row = [&](int w) __attribute__((always_inline)) { // [token] amax of wave w's 32 columns
    if constexpr (kLateBand) return reinterpret_cast<float *>(smem + w * kTWStage + 2 * kSiluBandN * 2);
    else return reinterpret_cast<float *>(smem + kTW + 2 * AST + 2 * T * 4) + w * T;
  };
  float *const sBs = reinterpret_cast<float *>(smem + kTW + 2 * AST + 2 * T * 4 + RED);
  int32_t *const sIds = reinterpret_cast<int32_t *>(smem + kTW + 2 * AST + 2 * T * 4 + RED + kTBs);
  uint16_t *const sSiluShared = reinterpret_cast<uint16_t *>(smem + kTW + 2 * AST + 2 * T * 4 + RED + kTBs + T * 4);

  int mb, nt;
  if (!tile_of(blockIdx.x, a.n_tiles, m_blocks, group_m, mb, nt)) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // which 64 weight rows of the tile
  const int r = lane & 15, q = lane >> 4;
  const int32_t *const sorted = a.sorted + static_cast<int64_t>(mb) * T;
  // Everything the tile's start-up reads from memory by its block index alone is requested here, in one go:
  // the number of blocks in use, the block's expert and the sorted ids this thread needs (token rows it
  // copies, the last valid token, the token whose scales it carries).  Asked for one after the other, each
  // behind the branch on the one before, they were three round trips in front of the first operand copy.
  // (Not for the fused 160-token form: the values alive across the branches cost it registers it does not have.)
  constexpr bool kEarlyIds = !(FUSED_ACT && NTB == 10);
  const int32_t blocks_end = a.ntpp[0];
  const int e_raw = a.expert_ids[mb];
  int32_t lf_copy[APW];
  int32_t lf_v0 = 0, lf_v1 = 0, lf_v2 = 0, lf_scale = 0;
  auto load_ids = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < APW; ++j) lf_copy[j] = sorted[(wave * APW + j) * 8 + (lane >> 3)];
    lf_v0 = sorted[lane];
    lf_v1 = sorted[lane + 64];
    if constexpr (NTB == 10) lf_v2 = sorted[128 + (lane & 31)];
    lf_scale = sorted[NTB == 8 ? (tid & (T - 1)) : (tid < T ? tid : tid - T)];
  };
  if constexpr (kEarlyIds) load_ids();
  if (static_cast<int64_t>(mb) * T >= blocks_end) return;
  // An expert_map entry outside the weight tensor is treated like an expert of another rank, but its
  // rows are always zero-filled: the slot mask of the alignment counts such a slot as local.
  const bool e_oob = e_raw >= a.E;
  const int e = e_oob ? -1 : e_raw;
  const int64_t K = a.K, N = a.N;
  const int KB = static_cast<int>(K / kGroup);
  const int64_t I = N / 2;

  // first row of the wave's 64 (plain) or of its 32 gate rows (fused)
  const int64_t nrow0 = FUSED_ACT ? static_cast<int64_t>(nt) * kGroup + wave * 32
                                  : static_cast<int64_t>(nt) * 256 + wave * 64;
  const bool wave_active = FUSED_ACT || nrow0 < N; // N % 64 == 0 is checked on the host

  if (e < 0) {
    if constexpr (!FUSED_ACT) {
      if (wave_active && (!a.skip_nonlocal || e_oob)) {
#pragma unroll
        for (int tb = 0; tb < NTB; ++tb) {
          const int64_t ft = sorted[tb * 16 + r];
          if (ft < a.num_valid)
#pragma unroll
            for (int j = 0; j < 4; ++j)
              *reinterpret_cast<v2i *>(a.C + ft * N + nrow0 + j * 16 + 4 * q) = v2i{0, 0};
        }
      }
    }
    return;
  }

  uint16_t band_regs[kSiluBandPer];
  if constexpr (FUSED_ACT && !kLateBand) silu_band_load(band_regs, a.silu, tid);

  // ---- what this wave copies -----------------------------------------------------------------------
  const int NBLK = static_cast<int>(N / 16);
  // W4: packed int4 weights in their load-time layout (1 KB per 16 rows x 128 K, the lane's two
  // k-steps in one 16-byte piece) and one scale per weight row and K block, [E, K/128, N]
  const int64_t wbytes = W4 ? N * K / 2 : N * K; // one expert
  const brsrc rW = make_rsrc(a.W + static_cast<int64_t>(e) * wbytes, static_cast<uint32_t>(wbytes));
  const brsrc rWs = make_rsrc(a.Ws + static_cast<int64_t>(e) * N * (PC ? 1 : KB), static_cast<uint32_t>(N * (PC ? 1 : KB) * 4));
  const brsrc rA = make_rsrc(a.A, static_cast<uint32_t>(a.a_rows * K));
  const brsrc rAs = make_rsrc(a.As, static_cast<uint32_t>(a.a_rows * (PC ? 1 : KB) * 4));
  const int wkstride = W4 ? shuf_kb_stride(NBLK) / 2 : shuf_kb_stride(NBLK);
  int wvoff[2][2]; // [step half][fragment]: the 2 KB block of 16 rows x 128 K, in lane order
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int rf = 0; rf < 2; ++rf) {
      int64_t nb;
      if constexpr (FUSED_ACT) nb = (rf ? I / 16 : 0) + static_cast<int64_t>(nt) * 8 + wave * 2 + h;
      else nb = static_cast<int64_t>(nt) * 16 + wave * 4 + h * 2 + rf;
      if (nb >= NBLK) nb = 0; // rows past N: computed on block 0, never stored
      wvoff[h][rf] = static_cast<int>(nb) * (W4 ? shuf_nb_stride(KB) / 2 : shuf_nb_stride(KB)) + lane * 16;
    }
  // W4: lane l copies the scale of row l of the wave's 64 (fused: 32 gate rows, then the 32 up rows)
  int wsvoff = 0;
  if constexpr (W4) {
    int64_t row;
    if constexpr (FUSED_ACT) row = (lane < 32 ? 0 : I - 32) + static_cast<int64_t>(nt) * kGroup + wave * 32 + lane;
    else row = static_cast<int64_t>(nt) * 256 + wave * 64 + lane;
    if (row >= N) row = 0;
    wsvoff = static_cast<int>(row * 4);
  }
  // STREAM: about one token block per expert, so a weight byte is used by one workgroup only and is
  // requested with the streaming hint (it does not displace the token rows and scales in L2;
  // first GEMM of the DeepSeek-V3 share at 1024 tokens 213 -> 160 us).  With several token blocks
  // per expert the blocks share the weights through L2 and the hint costs 7 %.
  constexpr int kWAux = STREAM ? kCacheStream : kCacheDefault;
  // The first K block's weights depend on the expert only: they are requested before the token
  // ids are read, so that the two dependent round trips of the tile's start-up overlap.
  int8_t *const sWw = smem + wave * kTWStage; // int8: [row half][fragment][k half] x 1 KB; W4: [row half][fragment] x 1 KB, row scales
  if constexpr (W4) {
#pragma unroll
    for (int p = 0; p < 4; ++p)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rW, sWw + p * 1024, 16, wvoff[p >> 1][p & 1], 0, 0, kWAux);
    if constexpr (!PC) __builtin_amdgcn_raw_ptr_buffer_load_lds(rWs, sWw + 4096, 4, wsvoff, 0, 0, kWAux);
  } else {
#pragma unroll
    for (int p = 0; p < 8; ++p)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rW, sWw + p * 1024, 16, wvoff[p >> 2][(p >> 1) & 1], (p & 1) * 1024, 0,
                                               kWAux);
  }
  int avoff[5]; // 1 KB pieces wave*APW + j of a token stage, j < APW: eight token rows each
#pragma unroll
  for (int j = 0; j < APW; ++j) {
    const int t = (wave * APW + j) * 8 + (lane >> 3);
    const int64_t lf = kEarlyIds ? lf_copy[j] : sorted[t];
    const int64_t lrow = (lf < a.num_valid) ? lf / a.top_k : 0;
    const int piece = (lane & 7) ^ (t & 7); // slot lane & 7 of row t holds piece slot ^ (t & 7)
    avoff[j] = static_cast<int>(lrow * K) + piece * 16;
  }
  // The alignment puts a block's valid tokens first, so a block of 128 is on average half a block
  // of padding per expert: token fragments past the last valid token are skipped, in steps of
  // 32 tokens (taken from the position of the last valid token, not from their number, so that
  // a caller's own sorted ids with gaps are still computed in full).
  int nst; // pipeline stages per K block: four per 32 tokens in use
  {
    if constexpr (!kEarlyIds) {
      lf_v0 = sorted[lane];
      lf_v1 = sorted[lane + 64];
      if constexpr (NTB == 10) lf_v2 = sorted[128 + (lane & 31)];
    }
    const uint64_t v0 = __builtin_amdgcn_ballot_w64(lf_v0 < a.num_valid);
    const uint64_t v1 = __builtin_amdgcn_ballot_w64(lf_v1 < a.num_valid);
    int last = v1 ? 127 - __builtin_clzll(v1) : (v0 ? 63 - __builtin_clzll(v0) : 0);
    if constexpr (NTB == 10) {
      const uint64_t v2 = __builtin_amdgcn_ballot_w64(lane < 32 && lf_v2 < a.num_valid);
      if (v2) last = 191 - __builtin_clzll(v2);
    }
    nst = __builtin_amdgcn_readfirstlane(4 * ((last >> 5) + 1)); // the K loop comes in variants of 2, 4, 6, 8 (, 10) fragments
  }
  int asoff; // thread t and thread t + T both carry the scale of token t
  {
    const int64_t lf = kEarlyIds ? lf_scale : sorted[NTB == 8 ? (tid & (T - 1)) : (tid < T ? tid : tid - T)];
    const int64_t lrow = (lf < a.num_valid) ? lf / a.top_k : 0;
    asoff = static_cast<int>(lrow * (PC ? 1 : KB) * 4);
    // The epilogues take the ids from LDS: a global load in each of their exec-masked blocks is a
    // full memory round trip that nothing overlaps.
    if (tid < T) sIds[tid] = static_cast<int32_t>(lf);
  }
  // weight-block scales of the tile: table row 0 / 1 = gate / up block (fused), or the first / second
  // 128 rows of the tile (plain: waves 0, 1 / waves 2, 3).  Thread t fetches entry (t >> 7, t & 127).
  const int NB = static_cast<int>((N + kGroup - 1) / kGroup);
  float bs_mine = 0.0f;
  {
    const int which = tid >> 7, kbi = tid & (kTMaxKB - 1);
    int64_t nblk = FUSED_ACT ? (which ? I / kGroup : 0) + nt : static_cast<int64_t>(nt) * 2 + which;
    if (nblk >= NB) nblk = 0;
    if (!W4 && !PC && kbi < KB) bs_mine = a.Ws[(static_cast<int64_t>(e) * NB + nblk) * KB + kbi];
  }
  const float *const sBs0 = sBs + (FUSED_ACT ? 0 : (wave >> 1) * kTMaxKB);
  const float *const sBs1 = sBs + (FUSED_ACT ? kTMaxKB : (wave >> 1) * kTMaxKB);

  // piece p of the 8 + APW copies a wave issues per K block: 0..7 its weights, then its token rows
  auto copy_piece = [&](int p, int kb) __attribute__((always_inline)) {
    const int kc = kb < KB ? kb : KB - 1;
    if (p < 8) {
      if constexpr (W4) { // four weight pieces, the row scales, three empty slots
        if (p < 4)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rW, sWw + p * 1024, 16, wvoff[p >> 1][p & 1],
                                                   __builtin_amdgcn_readfirstlane(kc * wkstride), 0, kWAux);
        else if (p == 4 && !PC)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rWs, sWw + 4096, 4, wsvoff,
                                                   __builtin_amdgcn_readfirstlane(kc) * static_cast<int>(N) * 4, 0, kWAux);
      } else {
        const int h = p >> 2, rf = (p >> 1) & 1, kh = p & 1;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rW, sWw + p * 1024, 16, wvoff[h][rf],
                                                 __builtin_amdgcn_readfirstlane(kc * wkstride) + kh * 1024, 0, kWAux);
      }
    } else {
      const int j = p - 8;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rA, sA + (kb & 1) * AST + (wave * APW + j) * 1024, 16, avoff[j],
                                               __builtin_amdgcn_readfirstlane(kc) * kGroup, 0, 0);
    }
  };
  auto copy_a = [&](int kb) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 8; p < 8 + APW; ++p) copy_piece(p, kb);
  };
  auto load_scale = [&](int kb) __attribute__((always_inline)) {
    if constexpr (PC) return 0.0f; // one scale per token, read by the epilogue
    return bld_f32(rAs, asoff, (kb < KB ? kb : KB - 1) * 4);
  };

  // ---- operand read offsets -------------------------------------------------------------------------
  // token fragment tb, k-half kh: piece 4*kh + q of row tb*16 + r sits in slot piece ^ (r & 7)
  int alds[2];
#pragma unroll
  for (int kh = 0; kh < 2; ++kh) alds[kh] = r * kGroup + (((4 * kh + q) ^ (r & 7)) * 16);

  float acc[2][NTB][2][4]; // [step half][token fragment][fragment of the half][element]
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int tb = 0; tb < NTB; ++tb)
#pragma unroll
      for (int rf = 0; rf < 2; ++rf)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[h][tb][rf][i] = 0.0f;
  v4i acci[2][NTB][2]; // PC: the whole-K int32 sums
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int tb = 0; tb < NTB; ++tb)
#pragma unroll
      for (int rf = 0; rf < 2; ++rf) acci[h][tb][rf] = v4i{0, 0, 0, 0};

  // W4: every product carries the factor 16 of the unpacked nibbles; it is taken out through the row
  // scale, which read_w() multiplies by 1/16 once per K block (a power of two: (f32(d) * a_s) * (b_s / 16)
  // is bit for bit (f32(d / 16) * a_s) * b_s unless b_s lies below 2^-122 or the product above 2^124).
  // One scale per weight row: bs4[i] for row 4q + i.
  auto fold4 = [&](const v4i &d, float as, const v4f &bs4, float *dst) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) // bs4 already holds scale / 16
      dst[i] = fold_elem<ORD>(d[i], ORD == kOrdFusedScale ? as * bs4[i] : 0.0f, as, bs4[i], dst[i]);
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(dst[i])); // keep the fold here
  };
  auto fold = [&](const v4i &d, float sc, float as, float bs, float *dst) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) dst[i] = fold_elem<ORD>(d[i], sc, as, bs, dst[i]);
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(dst[i])); // keep the fold here
  };

  // One K block: the wave's 64 rows (two halves h of two fragments) against all 128 tokens.
  v4i w[2][2][2]; // the wave's weights of the current K block
  v4f wsc[2][2];  // W4: the scales of the lane's rows 4q .. 4q+3 of each fragment
  auto read_w = [&]() __attribute__((always_inline)) {
    if constexpr (W4) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int rf = 0; rf < 2; ++rf) {
          const v4i pk = *reinterpret_cast<const v4i *>(sWw + (h * 2 + rf) * 1024 + lane * 16);
#pragma unroll
          for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int x = 0; x < 2; ++x) {
              const uint32_t word = static_cast<uint32_t>(pk[2 * ks + x]);
              w[h][rf][ks][2 * x] = static_cast<int>((word << 4) & 0xf0f0f0f0u);
              w[h][rf][ks][2 * x + 1] = static_cast<int>(word & 0xf0f0f0f0u);
            }
          // rows of fragment (h, rf) among the wave's 64: fused 32*rf + 16*h, plain 32*h + 16*rf
          if constexpr (!PC) {
            const int row0 = (FUSED_ACT ? 32 * rf + 16 * h : 32 * h + 16 * rf) + 4 * q;
            wsc[h][rf] = *reinterpret_cast<const v4f *>(sWw + 4096 + row0 * 4);
            wsc[h][rf] = wsc[h][rf] * 0.0625f;
          }
        }
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int rf = 0; rf < 2; ++rf)
#pragma unroll
          for (int kh = 0; kh < 2; ++kh)
            w[h][rf][kh] = *reinterpret_cast<const v4i *>(sWw + ((h * 2 + rf) * 2 + kh) * 1024 + lane * 16);
    }
  };
  // Full tiles meet at the barrier two stages before the end of a K block instead of at its start:
  // by then every copy for the next K block has had eight stages to land and nobody reads this K
  // block's token stage or scales any more, so the next block's first operands are read from LDS
  // under the last two stages and no wave stands waiting for LDS right after a barrier.
  float s_pending;   // token scales on their way from global memory to sS
  v4i bf_first[2];   // first token fragment of the next K block
  float as_first = 0.0f;
  auto kblock = [&](auto NST, int kb) __attribute__((always_inline)) {
    constexpr int nst_c = decltype(NST)::value; // stages of this variant: 4, 8, 12, 16 (or 20)
    constexpr int kFull = 2 * NTB;              // stages of a full tile
    constexpr int kE0 = kFull - 2, kE1 = kFull - 1;
    constexpr bool kEarly = nst_c == kFull && !W4;
    const int8_t *ta = sA + (kb & 1) * AST;
    const float *ts = sS + (kb & 1) * T;
    v4i bf[2][2];
    float as_t[2];
    if constexpr (kEarly) {
      // this wave's reads of the weight stage are complete before copies are aimed at it again
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      bf[0][0] = bf_first[0];
      bf[0][1] = bf_first[1];
      as_t[0] = as_first;
    } else {
#pragma unroll
      for (int kh = 0; kh < 2; ++kh) bf[0][kh] = *reinterpret_cast<const v4i *>(ta + alds[kh]);
      as_t[0] = ts[r];
    }
    const float bs0 = W4 ? 0.0f : sBs0[kb], bs1 = W4 ? 0.0f : sBs1[kb];

    // The weight stage was read into registers before the barrier, so it is free; it and the other
    // token stage are refilled with the next K block, two copies per pipeline stage so that the
    // texture path never sees a burst that this wave (or the other workgroup's) queues behind.
    const v4i cinit = {0, 0, 0, 0};
    v4i dprev[2];
    float as_p = 0.0f;
    float sc0 = 0.0f, sc1 = 0.0f; // scale products of the token fragment being folded (both row halves)
    auto fold_stage = [&](int st) __attribute__((always_inline)) { // fold the fragments of stage st
      const int tb = st >> 1, h = st & 1;
      if constexpr (PC) return;
      if constexpr (W4) {
        fold4(dprev[0], as_p, wsc[h][0], acc[h][tb][0]);
        fold4(dprev[1], as_p, wsc[h][1], acc[h][tb][1]);
        return;
      }
      if (ORD == kOrdFusedScale && h == 0) {
        sc0 = as_p * bs0;
        sc1 = FUSED_ACT ? as_p * bs1 : sc0;
      }
      fold(dprev[0], sc0, as_p, bs0, acc[h][tb][0]);
      fold(dprev[1], sc1, as_p, FUSED_ACT ? bs1 : bs0, acc[h][tb][1]);
    };
    // pipeline stage (tb, h): its MFMAs are issued, then the previous stage's fragments are folded
    // while the matrix pipe works; the operands of token fragment tb + 1 are requested in (tb, 0)
#pragma unroll
    for (int st = 0; st < kFull; ++st) {
      const int tb = st >> 1, h = st & 1;
      const int cur = tb & 1, nxt = cur ^ 1;
      if (nst_c >= 8 && st < 6) {
        copy_piece(2 * st, kb + 1);
        copy_piece(2 * st + 1, kb + 1);
      }
      if (NTB == 10 && nst_c >= 8 && st == 6) copy_piece(12, kb + 1); // the fifth token piece of a 160-token stage
      if (nst_c < 8 && st < 4) {
        copy_piece(3 * st, kb + 1);
        copy_piece(3 * st + 1, kb + 1);
        copy_piece(3 * st + 2, kb + 1);
      }
      if (st < nst_c) {
        if (kEarly && st == kE0) {
          wait_copies_barrier<0>();
          if (tid < T) sS[(kb & 1) * T + tid] = kb + 2 < KB ? s_pending : 0.0f;
          s_pending = load_scale(kb + 3);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (h == 0 && st + 2 < nst_c) {
#pragma unroll
          for (int kh = 0; kh < 2; ++kh)
            bf[nxt][kh] = *reinterpret_cast<const v4i *>(ta + (tb + 1) * 16 * kGroup + alds[kh]);
          as_t[nxt] = ts[(tb + 1) * 16 + r];
        }
        v4i d[2];
#pragma unroll
        for (int rf = 0; rf < 2; ++rf)
          d[rf] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[h][rf][0], bf[cur][0], PC ? acci[h][tb][rf] : cinit, 0, 0, 0);
#pragma unroll
        for (int rf = 0; rf < 2; ++rf)
          d[rf] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[h][rf][1], bf[cur][1], d[rf], 0, 0, 0);
        if constexpr (PC) {
          acci[h][tb][0] = d[0];
          acci[h][tb][1] = d[1];
        }
        if (kEarly && st >= kE0) { // the next K block's operands of this half, over the ones just used
#pragma unroll
          for (int rf = 0; rf < 2; ++rf)
#pragma unroll
            for (int kh = 0; kh < 2; ++kh)
              w[h][rf][kh] = *reinterpret_cast<const v4i *>(sWw + ((h * 2 + rf) * 2 + kh) * 1024 + lane * 16);
          if (st == kE0) {
            const int8_t *tan = sA + ((kb + 1) & 1) * AST;
#pragma unroll
            for (int kh = 0; kh < 2; ++kh) bf_first[kh] = *reinterpret_cast<const v4i *>(tan + alds[kh]);
            as_first = sS[((kb + 1) & 1) * T + r];
          }
        }
        if (st > 0) fold_stage(st - 1);
        if (h == 0 && st + 2 < nst_c) __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (nst_c >= 8 ? ((g < 2 && st < 6) || (NTB == 10 && g == 0 && st == 6)) : (g < 3 && st < 4))
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, W4 ? 7 : 5, 0);
        }
        if (kEarly && st == kE0) __builtin_amdgcn_sched_group_barrier(0x100, 7, 0);
        if (kEarly && st == kE1) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
        __builtin_amdgcn_sched_barrier(0);
        dprev[0] = d[0];
        dprev[1] = d[1];
        as_p = as_t[cur];
      }
    }
    fold_stage(nst_c - 1);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!kEarly) {
      // the next K block's weights have had a whole K block to arrive; reading them here puts the
      // LDS latency under the barrier instead of in front of the first MFMA
      wait_copies<0>();
      read_w();
    }
  };

  // ---- prologue ------------------------------------------------------------------------------------------
  float s_now = load_scale(0);
  s_pending = load_scale(1);
  __builtin_amdgcn_sched_barrier(0);
  copy_a(0);
  __builtin_amdgcn_sched_barrier(0);
  if (tid < T) sS[tid] = s_now;
  sBs[tid] = bs_mine;
  if constexpr (FUSED_ACT && !kLateBand) silu_band_store(sSiluShared, band_regs, tid);
  wait_copies<0>();
  read_w();

  auto k_loop = [&](auto NST) __attribute__((always_inline)) {
    if constexpr (decltype(NST)::value == 2 * NTB && !W4) {
      wait_copies_barrier<0>(); // K block 0 is complete in LDS
      if (tid < T) sS[T + tid] = 1 < KB ? s_pending : 0.0f;
      s_pending = load_scale(2);
#pragma unroll
      for (int kh = 0; kh < 2; ++kh) bf_first[kh] = *reinterpret_cast<const v4i *>(sA + alds[kh]);
      as_first = sS[r];
      __builtin_amdgcn_sched_barrier(0);
      for (int kb = 0; kb < KB; ++kb) kblock(NST, kb);
      return;
    }
    for (int kb = 0; kb < KB; ++kb) {
      // every copy this wave requested a K block ago has landed; after the barrier so have everyone
      // else's token rows, and nobody still reads the token stage and the scales of K block kb-1,
      // which are refilled below
      wait_copies_barrier<0>();
      if (tid < T) sS[((kb + 1) & 1) * T + tid] = kb + 1 < KB ? s_pending : 0.0f;
      s_pending = load_scale(kb + 2);
      __builtin_amdgcn_sched_barrier(0);
      kblock(NST, kb);
    }
  };
  // one K loop per number of token fragments that hold valid tokens (wave-uniform choice)
  if constexpr (NTB == 10) {
    // three variants only (a block this size is chosen where experts fill it; a fourth one made the
    // kernel spill): a tile in between runs the next larger one, whose surplus fragments compute on
    // padding rows and are not stored
    if (nst > 16) k_loop(std::integral_constant<int, 20>{});
    else if (nst > 8) k_loop(std::integral_constant<int, 16>{});
    else k_loop(std::integral_constant<int, 8>{});
  } else {
    if (nst > 12) k_loop(std::integral_constant<int, 16>{});
    else if (nst > 8) k_loop(std::integral_constant<int, 12>{});
    else if (nst > 4) k_loop(std::integral_constant<int, 8>{});
    else k_loop(std::integral_constant<int, 4>{});
  }
  wait_copies<0>(); // no copy may still be writing LDS when the epilogue reuses it or the wave ends
  if constexpr (!FUSED_ACT) {
    if (!wave_active) return;
    // A lane holds 4 consecutive columns of one token per fragment.  Each wave turns a 16-token x
    // 64-column piece around in its own (now idle) weight ring and stores 128-byte row segments.
    int8_t *stg = sWw;
    // PC: the scales of the lane's rows and of its eight tokens, fetched in one batch up front
    v4f pbs[2][2];
    float pas[NTB];
    if constexpr (PC) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int rf = 0; rf < 2; ++rf)
          pbs[h][rf] = __builtin_bit_cast(v4f, bld16(rWs, static_cast<int>((nrow0 + h * 32 + rf * 16 + 4 * q) * 4), 0));
#pragma unroll
      for (int tb = 0; tb < NTB; ++tb) {
        const int64_t ft = sIds[tb * 16 + r];
        pas[tb] = bld_f32(rAs, static_cast<int>((ft < a.num_valid ? ft / a.top_k : 0) * 4), 0);
      }
    }
#pragma unroll
    for (int tb = 0; tb < NTB; ++tb) {
      if (2 * tb >= nst) continue;
      const int64_t ft = sIds[tb * 16 + r];
      const bool valid = ft < a.num_valid;
      float wgt = 1.0f;
      if (a.mul_routed && valid) wgt = a.topk_w[ft];
      with_out16(a.out_f16, [&](auto cvt) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int rf = 0; rf < 2; ++rf) {
            v4u16 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              float v;
              if constexpr (PC && W4) { // left to right: routed weight, token scale, channel scale (w4a8.py:386-395)
                v = static_cast<float>(acci[h][tb][rf][i]);
                if (a.mul_routed) v = v * wgt;
                v = v * pas[tb];
                v = v * pbs[h][rf][i];
              } else if constexpr (PC) { // int8 weights: (f32(d) * ts) * b_s, ts = w * a_s (moe_w8a8.cu:452, :466)
                const float ts = a.mul_routed ? wgt * pas[tb] : pas[tb];
                v = static_cast<float>(acci[h][tb][rf][i]) * ts;
                v = v * pbs[h][rf][i];
              } else {
                v = acc[h][tb][rf][i];
                if (a.mul_routed) v = v * wgt;
              }
              o[i] = cvt(v);
            }
            *reinterpret_cast<v4u16 *>(stg + r * kTPitch + (h * 32 + rf * 16 + 4 * q) * 2) = o;
          }
      });
      __builtin_amdgcn_wave_barrier();
      const int slot = valid ? static_cast<int>(ft) : -1;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int tok = (lane >> 3) + 8 * j;
        const v4i v = *reinterpret_cast<const v4i *>(stg + tok * kTPitch + (lane & 7) * 16);
        const int fs = __shfl(slot, tok);
        if (fs >= 0) *reinterpret_cast<v4i *>(a.C + static_cast<int64_t>(fs) * N + nrow0 + (lane & 7) * 8) = v;
      }
      __builtin_amdgcn_wave_barrier();
    }
  } else {
    const uint16_t *sSilu = sSiluShared;
    if constexpr (kLateBand) {
      // the band of the SiLU table (two runs of kSiluBandN entries, one per sign of the gate) straight into this
      // wave's own weight stage, 256 bytes per copy
      const brsrc rT = make_rsrc(a.silu, 65536 * 2);
      constexpr int kRun = kSiluBandN * 2; // bytes per sign
#pragma unroll
      for (int sgn = 0; sgn < 2; ++sgn)
#pragma unroll
        for (int j = 0; j < (kRun + 255) / 256; ++j) {
          int off = j * 256 + lane * 4;
          off = off < kRun ? off : kRun - 4; // the last copy's surplus lanes repeat the run's last word
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rT, sWw + sgn * kRun + j * 256, 4,
                                                   (sgn * 0x8000 + kSiluBandLo) * 2 + off, 0, 0, 0);
        }
      wait_copies<0>();
      sSilu = reinterpret_cast<const uint16_t *>(sWw);
    }
    // acc[h][tb][0] = gate, acc[h][tb][1] = up for activation columns nt*128 + wave*32 + 16h + 4q + i
    float actf[NTB][2][4];
    if (a.mul_routed) { // router weight on the first GEMM's output: rare, kept out of the main pass
#pragma unroll
      for (int tb = 0; tb < NTB; ++tb) {
        const int64_t ft = sIds[tb * 16 + r];
        const float wgt = ft < a.num_valid ? a.topk_w[ft] : 1.0f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int rf = 0; rf < 2; ++rf)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[h][tb][rf][i] = acc[h][tb][rf][i] * wgt;
      }
    }
    // Token fragments are in use in pairs (nst is a multiple of four stages).  A pair shares one
    // wave-uniform branch, so the LDS lookups of its two fragments are in flight together.
#pragma unroll
    for (int tb = 0; tb < NTB; ++tb) {
      if (2 * (tb & ~1) >= nst) continue; // the same condition for both fragments of a pair
      uint16_t g16[2][4], u16[2][4];
      bool special = false;
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          g16[h][i] = f32_to_bf16(acc[h][tb][0][i]);
          u16[h][i] = f32_to_bf16(acc[h][tb][1][i]);
          special |= silu_gate_special(g16[h][i]);
          actf[tb][h][i] = bf16_to_f32(silu_mul_band_common(sSilu, g16[h][i], u16[h][i]));
        }
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(special) != 0, 0)) { // a NaN or -inf gate in the wave
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            actf[tb][h][i] = bf16_to_f32(silu_mul_band(sSilu, a.silu, g16[h][i], u16[h][i]));
      }
      float amax = 0.0f;
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) amax = fmaxf(amax, fabsf(actf[tb][h][i]));
      amax = fmaxf(amax, __shfl_xor(amax, 16));
      amax = fmaxf(amax, __shfl_xor(amax, 32));
      if (q == 0) red_row(wave)[tb * 16 + r] = amax;
    }
    __syncthreads(); // also: every wave is done with the token stages
    const int64_t G = I / kGroup;
    // the quantised tile (128 tokens x 128 columns of int8) leaves through LDS as whole rows
    int8_t *qst = sA;
    // scales of all eight fragments first, outside the branches on nst: the reads are in bounds
    // either way, and one batch of LDS reads and divisions replaces eight dependent chains
    float sc_all[NTB], rsc_all[NTB];
#pragma unroll
    for (int tb = 0; tb < NTB; ++tb) {
      const int t = tb * 16 + r;
      float amax = fmaxf(fmaxf(red_row(0)[t], red_row(1)[t]), fmaxf(red_row(2)[t], red_row(3)[t]));
      amax = fmaxf(amax, 1e-10f);
      sc_all[tb] = amax / 127.0f;
      rsc_all[tb] = 1.0f / sc_all[tb];
    }
#pragma unroll
    for (int tb = 0; tb < NTB; ++tb) {
      if (2 * (tb & ~1) >= nst) continue;
      const int t = tb * 16 + r;
      const float sc = sc_all[tb], rsc = rsc_all[tb];
#pragma unroll
      for (int h = 0; h < 2; ++h)
        *reinterpret_cast<uint32_t *>(qst + t * kTPitch + wave * 32 + h * 16 + 4 * q) = quant4(actf[tb][h], sc, rsc);
      if (wave == (tb & 3) && q == 0) { // every wave holds every token's scale: the stores are shared out
        const int64_t ft = sIds[t];
        if (ft < a.num_valid) a.A2s[ft * G + nt] = sc;
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < T * 8 / 256; ++j) {
      const int id = tid + 256 * j, tok = id >> 3, piece = id & 7;
      const int64_t ft = sIds[tok];
      if (ft < a.num_valid)
        *reinterpret_cast<v4i *>(a.A2q + ft * I + static_cast<int64_t>(nt) * kGroup + piece * 16) =
            *reinterpret_cast<const v4i *>(qst + tok * kTPitch + piece * 16);
    }
  }
}

bool gemm_t128_supports(const GemmArgs &a, bool fused_act, int block_size_m) {
  if (block_size_m == kT160) { // 160-token tiles: int8 block form (plain or fused epilogue) or per-channel scales
    if (!a.w_shuffled || a.K / kGroup > kTMaxKB) return false;
    if (fused_act) return !a.per_channel && !a.w4;
    return (a.per_channel || !a.w4) && a.N % 64 == 0;
  }
  if (block_size_m != 128 || !a.w_shuffled) return false;
  if (a.per_channel && (!a.w4 || fused_act)) return false; // int8 per-channel weights have gemm_pc.hip
  if (!fused_act && a.N % 64 != 0) return false;
  return a.K / kGroup <= kTMaxKB;
}

int launch_gemm_t128(const GemmArgs &a0, bool fused_act, int block_size_m, int flags, int64_t m_blocks,
                     hipStream_t s) {
  GemmArgs a = a0;
  a.n_tiles = fused_act ? static_cast<int32_t>(a.N / 2 / kGroup) : static_cast<int32_t>((a.N + 255) / 256);
  int64_t G = a.num_valid / (static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) * block_size_m);
  G = G < 2 ? 2 : (G > 16 ? 16 : G);
  const int64_t chunks = (m_blocks + G - 1) / G;
  const int64_t grid = (chunks + 7) / 8 * (G * a.n_tiles) * 8;
  LO_REQUIRE(grid < (1ll << 31), LO_EINVAL, "moe_gemm: grid too large");
  const int ord = scale_order(flags);
  const dim3 g(static_cast<unsigned>(grid)), b(256);
  const int mbi = static_cast<int>(m_blocks), gi = static_cast<int>(G);
#define LO_T128_LAUNCH(FA, FS, ST, W)                                                                           \
  do {                                                                                                          \
    static unsigned long long lds_done = 0; /* per instantiation: one bit per device */                         \
    const int rc_lds = reserve_lds_once(reinterpret_cast<const void *>(&moe_gemm_t128_kernel<FA, FS, ST, W>),    \
                                        kTLds, &lds_done);                                                      \
    if (rc_lds) return rc_lds;                                                                                  \
    hipLaunchKernelGGL((moe_gemm_t128_kernel<FA, FS, ST, W>), g, b, kTLds, s, a, mbi, gi);                      \
  } while (0)
#define LO_T128_LAUNCH_PC(ST)                                                                                   \
  do {                                                                                                          \
    static unsigned long long lds_done = 0;                                                                     \
    const int rc_lds = reserve_lds_once(                                                                        \
        reinterpret_cast<const void *>(&moe_gemm_t128_kernel<false, kOrdSeparate, ST, true, true>), kTLds, &lds_done); \
    if (rc_lds) return rc_lds;                                                                                  \
    hipLaunchKernelGGL((moe_gemm_t128_kernel<false, kOrdSeparate, ST, true, true>), g, b, kTLds, s, a, mbi, gi);       \
  } while (0)
#define LO_T128_PICK(FS, FA)                                                                                    \
  do {                                                                                                          \
    if (a.w4) {                                                                                                 \
      if (stream) LO_T128_LAUNCH(FA, FS, true, true);                                                           \
      else LO_T128_LAUNCH(FA, FS, false, true);                                                                 \
    } else {                                                                                                    \
      if (stream) LO_T128_LAUNCH(FA, FS, true, false);                                                          \
      else LO_T128_LAUNCH(FA, FS, false, false);                                                                \
    }                                                                                                           \
  } while (0)
  if (block_size_m == kT160) {
    // chosen where an expert's tokens fill one block, so a weight byte has one reader: streaming hint
#define LO_T160_LAUNCH(FS, FA)                                                                                  \
  do {                                                                                                          \
    static unsigned long long lds_done = 0;                                                                     \
    const int rc_lds = reserve_lds_once(                                                                        \
        reinterpret_cast<const void *>(&moe_gemm_t128_kernel<FA, FS, true, false, false, 10>), kTLds160,        \
        &lds_done);                                                                                             \
    if (rc_lds) return rc_lds;                                                                                  \
    hipLaunchKernelGGL((moe_gemm_t128_kernel<FA, FS, true, false, false, 10>), g, b, kTLds160, s, a, mbi, gi);  \
  } while (0)
    if (a.per_channel && a.w4) {
      static unsigned long long lds_done = 0;
      const int rc_lds = reserve_lds_once(
          reinterpret_cast<const void *>(&moe_gemm_t128_kernel<false, kOrdSeparate, true, true, true, 10>), kTLds160, &lds_done);
      if (rc_lds) return rc_lds;
      hipLaunchKernelGGL((moe_gemm_t128_kernel<false, kOrdSeparate, true, true, true, 10>), g, b, kTLds160, s, a, mbi, gi);
    } else if (a.per_channel) {
      static unsigned long long lds_done = 0;
      const int rc_lds = reserve_lds_once(
          reinterpret_cast<const void *>(&moe_gemm_t128_kernel<false, kOrdSeparate, true, false, true, 10>), kTLds160, &lds_done);
      if (rc_lds) return rc_lds;
      hipLaunchKernelGGL((moe_gemm_t128_kernel<false, kOrdSeparate, true, false, true, 10>), g, b, kTLds160, s, a, mbi, gi);
    } else if (fused_act) {
      LO_ORD_DISPATCH(ord, LO_T160_LAUNCH, true);
    } else {
      LO_ORD_DISPATCH(ord, LO_T160_LAUNCH, false);
    }
#undef LO_T160_LAUNCH
    return check_launch(fused_act ? "moe_gemm1_silu_quant(t160)" : "moe_gemm(t160)");
  }
  // one token block per expert, by and large: the slots spread over the routed experts fill half a block
  const bool stream = a.num_valid <= static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) * (kT / 2);
  if (a.per_channel) {
    if (stream) LO_T128_LAUNCH_PC(true);
    else LO_T128_LAUNCH_PC(false);
  } else if (fused_act) {
    LO_ORD_DISPATCH(ord, LO_T128_PICK, true);
  } else {
    LO_ORD_DISPATCH(ord, LO_T128_PICK, false);
  }
#undef LO_T128_PICK
#undef LO_T128_LAUNCH_PC
#undef LO_T128_LAUNCH
  return check_launch(fused_act ? "moe_gemm1_silu_quant(t128)" : "moe_gemm(t128)");
}

} // namespace lo
