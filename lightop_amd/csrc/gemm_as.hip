// Grouped block-INT8 GEMM for gfx950, activation-stationary form for a short K (the
// second GEMM of a layer with a small intermediate size).
//
// With K of a few hundred bytes the 64 gathered token rows of a token block fit in LDS
// whole (64 x K bytes plus their group scales).  A workgroup loads them once and then
// walks several 256-row weight tiles with them: the K loop needs no barrier, no LDS
// write and no token reload, the weight prefetch (two K blocks deep) runs on across tile boundaries, and the
// gather of sorted_token_ids is paid once per token block instead of once per tile.
// Wave tile, MFMA layout, scaling order and output are those of the LDS-tiled kernel
// (gemm_tile.hip); reference: Triton fused_moe_kernel, python/lightop/_lmslim_native/
// layers/fused_moe/int8.py:485-541.
#include <type_traits>

#include "gemm.h"

namespace lo {

typedef int v16i __attribute__((ext_vector_type(16)));

// KBT: K / 128 as a compile-time constant (a multiple of three, so that a tile starts on ring buffer 0),
// or 0 for any K.  With it a tile's steps and its stores are straight-line code: the compiler then
// knows how many memory operations follow each weight load and waits for exactly those; in the
// general form the stores sit in a branch, the wait counts assume they did not happen, and after
// every tile the wave waits for loads it has only just issued.
template <int ORD, bool SHUF, int KBT = 0>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void moe_gemm_as_kernel(const GemmArgs a, int m_blocks, int group_m,
                                                          int n_groups, int n_cnt, int sub_shift) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  constexpr int kTileM = 64;
  const int K = static_cast<int>(a.K);
  const int KB = K / kGroup;
  const int pitch = K + 16; // = 16 mod 128: ds_read_b128 of 32 consecutive rows is conflict-free
  int8_t *const sA = smem;
  float *const sS = reinterpret_cast<float *>(smem + kTileM * pitch); // [KB][64]
  // per-wave staging of 32 output rows x 64 columns (bf16), for row-contiguous stores
  int8_t *const sStage = smem + kTileM * pitch + KB * kTileM * 4;

  int mb, ng;
  if (!tile_of(blockIdx.x, n_groups, m_blocks, group_m, mb, ng)) return;
  if (static_cast<int64_t>(mb) * kTileM >= a.ntpp[0]) return;
  // mb counts 64-token pieces; an alignment block of 128 tokens is two of them (sub_shift = 1), and
  // a piece that holds padding only is skipped
  // An expert_map entry outside the weight tensor is treated like an expert of another rank, but its
  // rows are always zero-filled: the slot mask of the alignment counts such a slot as local.
  const int e_raw = a.expert_ids[mb >> sub_shift];
  const bool e_oob = e_raw >= a.E;
  const int e = e_oob ? -1 : e_raw;
  const int tid = threadIdx.x, lane = tid & 63;
  if (sub_shift &&
      __builtin_amdgcn_ballot_w64(a.sorted[static_cast<int64_t>(mb) * kTileM + lane] < a.num_valid) == 0)
    return;
  const int wr = __builtin_amdgcn_readfirstlane(tid >> 6); // which 64 weight rows of a tile
  const int r = lane & 31, c = lane >> 5;
  const int64_t N = a.N;
  const int n_tiles = static_cast<int>((N + 255) / 256);
  const int nt0 = ng * n_cnt;
  int nt_end = nt0 + n_cnt < n_tiles ? nt0 + n_cnt : n_tiles;
  // N % 64 == 0 is checked on the host; in the last tile the waves past N have no rows
  if (static_cast<int64_t>(nt_end - 1) * 256 + wr * 64 >= N) --nt_end;

  int64_t f[2];
  bool valid[2];
#pragma unroll
  for (int tb = 0; tb < 2; ++tb) {
    f[tb] = a.sorted[static_cast<int64_t>(mb) * kTileM + tb * 32 + r];
    valid[tb] = f[tb] < a.num_valid;
  }

  if (e < 0) {
    if ((!a.skip_nonlocal || e_oob)) {
      for (int nt = nt0; nt < nt_end; ++nt)
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
          if (valid[tb])
#pragma unroll
            for (int rb = 0; rb < 2; ++rb)
#pragma unroll
              for (int q = 0; q < 4; ++q)
                *reinterpret_cast<v2i *>(a.C + f[tb] * N + static_cast<int64_t>(nt) * 256 + wr * 64 + rb * 32 +
                                         8 * q + 4 * c) = v2i{0, 0};
    }
    return;
  }

  // ---- the token block into LDS, once ------------------------------------------------
  {
    const int lt = tid >> 2, lq = tid & 3; // thread -> (token, every fourth 16-byte piece)
    const int64_t lf = a.sorted[static_cast<int64_t>(mb) * kTileM + lt];
    const int64_t lrow = (lf < a.num_valid) ? lf / a.top_k : 0;
    const brsrc rA = make_rsrc(a.A, static_cast<uint32_t>(a.a_rows * K));
    const int aoff = static_cast<int>(lrow * K) + lq * 16;
    int8_t *dst = sA + lt * pitch + lq * 16;
    const int pieces = K / 64; // per thread
    for (int j0 = 0; j0 < pieces; j0 += 4) {
      v4i t[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) t[j] = bld16(rA, aoff, (j0 + j < pieces ? j0 + j : pieces - 1) * 64);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (j0 + j < pieces) *reinterpret_cast<v4i *>(dst + (j0 + j) * 64) = t[j];
    }
    const int st = tid & 63;
    const int64_t sf = a.sorted[static_cast<int64_t>(mb) * kTileM + st];
    const int64_t srow = (sf < a.num_valid) ? sf / a.top_k : 0;
    for (int kb = tid >> 6; kb < KB; kb += 4) sS[kb * kTileM + st] = a.As[srow * KB + kb];
  }

  const int NB = static_cast<int>((N + kGroup - 1) / kGroup);
  const brsrc rW = make_rsrc(a.W + static_cast<int64_t>(e) * N * K, static_cast<uint32_t>(N * K));
  // the offset in 32 bits: a 64-bit multiply is a vector instruction, and a descriptor that has
  // been through vector registers costs a readfirstlane loop at every load
  const brsrc rWs = make_rsrc(a.Ws + e * NB * KB, static_cast<uint32_t>(NB * KB * 4));
  // lane offsets inside tile nt0; a later tile and the K block go into the scalar offset
  int woff[2], wsoff[2];
  const int wkstride = SHUF ? shuf_kb_stride(static_cast<int>(N / 16)) : kGroup;
  const int wtstride = SHUF ? 16 * shuf_nb_stride(KB) : 256 * K; // 256 rows further
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const int nr = nt0 * 256 + wr * 64 + rb * 32;
    if constexpr (SHUF) // 2 KB blocks; k-step j of lane half c reads 16-byte chunk 2j+c
      woff[rb] = (nr / 16 + (r >> 4)) * shuf_nb_stride(KB) + (c * 16 + (r & 15)) * 16;
    else
      woff[rb] = (nr + r) * K + c * 64;
    wsoff[rb] = (nr / kGroup) * KB * 4;
  }

  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  using B2 = std::integral_constant<int, 2>;
  v16i zero16;
#pragma unroll
  for (int i = 0; i < 16; ++i) zero16[i] = 0;
  float acc[2][2][16]; // [token fragment][row fragment][element]
  // Ring of three weight buffers: a K block is short work (16 MFMAs per wave), an L2 round trip
  // under load is not, so fragments are requested two K blocks ahead.
  v4i wreg[3][2][4];   // [buffer][row fragment][k-step]
  float bsc[3][2];     // [buffer][row fragment] weight-block scales, fetched with the fragments

  auto load_w = [&](auto BUF, int nt, int kb) __attribute__((always_inline)) {
    constexpr int b = decltype(BUF)::value;
    const int so = (nt - nt0) * wtstride + kb * wkstride;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) wreg[b][rb][ks] = bld16(rW, woff[rb], so + (SHUF ? ks * 512 : ks * 16));
    const int ss = ((nt - nt0) * 2 * KB + kb) * 4;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) bsc[b][rb] = bld_f32(rWs, wsoff[rb], ss);
  };
  auto fold = [&](const v16i &d, float as, float bs, float *dst) __attribute__((always_inline)) {
    const float sc = ORD == kOrdFusedScale ? as * bs : 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) dst[i] = fold_elem<ORD>(d[i], sc, as, bs, dst[i]);
    // The accumulators must be final here: an empty asm that "modifies" them stops the
    // optimiser from postponing the fold (and keeping the int32 fragment alive instead).
#pragma unroll
    for (int i = 0; i < 16; ++i) asm volatile("" : "+v"(dst[i]));
  };
  auto compute = [&](auto BUF, int kb, bool live) __attribute__((always_inline)) {
    constexpr int b = decltype(BUF)::value;
    // The four 32x32 fragments are software-pipelined: the MFMAs of one fragment are
    // issued, then the previous fragment is folded into the fp32 accumulators while the
    // matrix pipe works.
    v16i dprev = zero16;
    float as_prev = 0.0f;
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      v4i bf[4];
      // the K bytes of k-step ks must be the ones the weight operand holds for it
      const int8_t *src = sA + (tb * 32 + r) * pitch + kb * kGroup + (SHUF ? c * 16 : c * 64);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) bf[ks] = *reinterpret_cast<const v4i *>(src + (SHUF ? ks * 32 : ks * 16));
      const float as = live ? sS[kb * kTileM + tb * 32 + r] : 0.0f; // a step past the end adds 0
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

  // The (tile, K block) pairs form one flat sequence of steps; step s uses buffer s % 3.
  // Positions in that sequence are kept as (tile, K block) counters: a division by KB per step
  // is a long scalar dependency chain in front of the loads.
  const int total = (nt_end - nt0) * KB;
  int l_nt = nt0, l_kb = 0; // the next step to load
  int c_nt = nt0, c_kb = 0; // the next step to compute
  auto load_step = [&](auto BUF) __attribute__((always_inline)) { // a step past the end re-reads the last one
    const bool past = l_nt >= nt_end;
    load_w(BUF, past ? nt_end - 1 : l_nt, past ? KB - 1 : l_kb);
    if (++l_kb == KB) {
      l_kb = 0;
      ++l_nt;
    }
  };
  auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int tb = 0; tb < 2; ++tb)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[tb][rb][i] = 0.0f;
  };
  auto store_tile = [&](int nt) __attribute__((always_inline)) {
    const int64_t nrow0 = static_cast<int64_t>(nt) * 256 + wr * 64;
    int8_t *stg = sStage + wr * (32 * kStgPitch);
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
            for (int i = 0; i < 4; ++i) o[rb][q][i] = cvt(acc[tb][rb][4 * q + i] * w); // w = 1 leaves every value as it is
      });
      wave_store_32x64_bf16(stg, o, valid[tb] ? static_cast<int>(f[tb]) : -1, a.C, N, nrow0, lane);
    }
  };
  auto step = [&](auto BUF, auto NEXT) __attribute__((always_inline)) {
    load_step(NEXT);
    __builtin_amdgcn_sched_barrier(0); // keep the prefetch ahead of the MFMAs
    const bool live = c_nt < nt_end;
    compute(BUF, c_kb, live);
    if (live && c_kb == KB - 1) { // a tile is complete
      store_tile(c_nt);
      zero_acc();
    }
    if (++c_kb == KB) {
      c_kb = 0;
      ++c_nt;
    }
  };

  if (total > 0) { // before the barrier: in flight while the tokens land
    load_step(B0{});
    load_step(B1{});
  }
  __syncthreads(); // the only barrier: the token block is complete
  zero_acc();
  if constexpr (KBT > 0) {
    static_assert(KBT % 3 == 0, "a tile must start on ring buffer 0");
    for (int nt = nt0; nt < nt_end; ++nt) {
#pragma unroll
      for (int kb = 0; kb < KBT; ++kb) {
        // the step two ahead: this tile's, or the next tile's first two (the last tile re-reads its end)
        const bool wrap = kb + 2 >= KBT;
        const bool past = wrap && nt + 1 >= nt_end;
        const int lnt = past ? nt : (wrap ? nt + 1 : nt), lkb = past ? KBT - 1 : (wrap ? kb + 2 - KBT : kb + 2);
        if (kb % 3 == 0) load_w(B2{}, lnt, lkb);
        else if (kb % 3 == 1) load_w(B0{}, lnt, lkb);
        else load_w(B1{}, lnt, lkb);
        __builtin_amdgcn_sched_barrier(0); // keep the prefetch ahead of the MFMAs
        if (kb % 3 == 0) compute(B0{}, kb, true);
        else if (kb % 3 == 1) compute(B1{}, kb, true);
        else compute(B2{}, kb, true);
      }
      store_tile(nt);
      zero_acc();
    }
  } else {
    for (int s = 0; s < total; s += 3) {
      step(B0{}, B2{});
      step(B1{}, B0{});
      step(B2{}, B1{});
    }
  }
}

static int64_t as_lds_bytes(int64_t K) { return 64 * (K + 16) + (K / kGroup) * 64 * 4 + 4 * 32 * kStgPitch; }

bool gemm_as_supports(const GemmArgs &a, bool fused_act, int block_size_m) {
  if (fused_act || (block_size_m != 64 && block_size_m != 128)) return false;
  if (a.N % 64 != 0 || (reinterpret_cast<uintptr_t>(a.C) & 15) != 0) return false;
  if (as_lds_bytes(a.K) > 80 * 1024) return false; // two workgroups per CU
  // Pays off only when the launch is several rounds of workgroups deep even with half a
  // token block's weight tiles per workgroup; below that the per-tile kernel balances better.
  return a.num_valid / 64 + (a.experts_routed + 1) / 2 >= 1024;
}

int launch_gemm_as(const GemmArgs &a0, int flags, int block_size_m, int64_t m_blocks_bs, hipStream_t s) {
  const int sub_shift = block_size_m == 128 ? 1 : 0;
  const int64_t m_blocks = m_blocks_bs << sub_shift; // in 64-token pieces
  GemmArgs a = a0;
  const int n_tiles = static_cast<int>((a.N + 255) / 256);
  // Weight tiles per workgroup: half of them.  Fewer workgroups than that leave the
  // launch unbalanced, more pay the token gather more often (measured on 128 experts,
  // N = 2048, K = 768: 250 us with two groups, 269 with one, 296 with eight at 8192 tokens).
  int n_groups = n_tiles >= 2 ? 2 : 1;
  const int n_cnt = (n_tiles + n_groups - 1) / n_groups;
  n_groups = (n_tiles + n_cnt - 1) / n_cnt;
  a.n_tiles = n_groups;
  int64_t G = a.num_valid / (static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) * 64);
  G = G < 2 ? 2 : (G > 16 ? 16 : G);
  const int64_t chunks = (m_blocks + G - 1) / G;
  const int64_t grid = (chunks + 7) / 8 * (G * n_groups) * 8;
  LO_REQUIRE(grid < (1ll << 31), LO_EINVAL, "moe_gemm: grid too large");
  const int ord = scale_order(flags);
  const size_t lds = static_cast<size_t>(as_lds_bytes(a.K));
  const dim3 g(static_cast<unsigned>(grid)), b(256);
  const int mbi = static_cast<int>(m_blocks), Gi = static_cast<int>(G);
#define LO_AS_LAUNCH(FS, SH)                                                                          \
  do {                                                                                                \
    if (a.K == 6 * kGroup) LO_AS_LAUNCH_K(FS, SH, 6);                                                 \
    else LO_AS_LAUNCH_K(FS, SH, 0);                                                                   \
  } while (0)
#define LO_AS_LAUNCH_K(FS, SH, KBT)                                                                   \
  do {                                                                                                \
    auto kern = moe_gemm_as_kernel<FS, SH, KBT>;                                                      \
    static unsigned long long lds_done = 0; /* per instantiation: one bit per device */               \
    const int rc_lds = reserve_lds_once(reinterpret_cast<const void *>(kern), 80 * 1024, &lds_done);  \
    if (rc_lds) return rc_lds;                                                                        \
    hipLaunchKernelGGL(kern, g, b, lds, s, a, mbi, Gi, n_groups, n_cnt, sub_shift);                   \
  } while (0)
  if (a.w_shuffled) LO_ORD_DISPATCH(ord, LO_AS_LAUNCH, true);
  else LO_ORD_DISPATCH(ord, LO_AS_LAUNCH, false);
#undef LO_AS_LAUNCH
#undef LO_AS_LAUNCH_K
  return check_launch("moe_gemm(activation-stationary)");
}

} // namespace lo
