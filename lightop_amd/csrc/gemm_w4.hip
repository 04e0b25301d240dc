// Grouped W4A8 GEMM with K-group scales for gfx950, LDS-tiled form for many tokens per expert.
//
// Same arithmetic as the W4 instantiations of the weight-streaming kernel (gemm_ws.hip):
// packed int4 weights in the load-time layout of preshuffle_int4_kernel, unpacked in registers
// to int8 values 16 times too large, v_mfma_i32_16x16x64_i8 with the weight fragment as the A
// operand, an exact arithmetic shift of the int32 sum, then per 128-wide K block
//   acc = acc + (f32(d) * As[token, kb]) * Ws[e, kb, row]          (one scale per weight row)
// (nibble order: python/lightop/_lmslim_native/layers/fused_moe/w4a8.py:341, :375-377; the
// K-group scaling itself has no counterpart in the reference, whose kernel scales once in the
// epilogue, w4a8.py:395).
//
// What differs is where the tokens come from.  The streaming kernel lets every wave read its
// token rows from global memory, which is right while a token block is 16 or 32 rows; at 64
// tokens those reads outweigh the (half-size) weights four to one.  Here a workgroup of four
// waves gathers the 64 token rows of the current K block once into a double-buffered,
// row-padded LDS tile (with their group scales) and every wave multiplies its 64 weight rows
// (four 16-row fragments, global -> registers, double buffered; the row scales of the
// workgroup's 256 rows for every K block are copied to LDS before the K loop, already divided by
// 16, and read from there: fetched per K block they were as many 16-byte loads as the weights)
// against all of them: 16 accumulators of 16x16 per wave.  With FUSED_ACT the four fragments
// are 32 gate rows and the matching 32 up rows, and the epilogue is the SiLU(gate)*up +
// 1x128 re-quantisation of the block-INT8 path.
#include <type_traits>

#include "gemm.h"

namespace lo {

constexpr int kW4Row = 144; // LDS row pitch in bytes: 128 + 16 keeps ds_read_b128 conflict-free

//
// STREAM: an expert's weights and row scales are read by one token block, by and large: they are
// loaded with the streaming cache policy (first GEMM of a 4096 x 1536 layer with 16 or 32 slots per
// expert: 227 -> 180 us).  With several token blocks per expert the blocks share the weights through
// L2 and the default policy is the faster one.
template <bool FUSED_ACT, int ORD, bool STREAM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void moe_gemm_w4_tile_kernel(const GemmArgs a, int m_blocks, int group_m) {
  constexpr int kTileM = 64;
  constexpr int kWAux = STREAM ? kCacheStream : kCacheDefault;
  __shared__ __attribute__((aligned(16))) int8_t sA[2][kTileM * kW4Row];
  __shared__ float sS[2][kTileM];
  __shared__ float sRed[4][kTileM];
  __shared__ uint16_t sSilu[FUSED_ACT ? 2 * kSiluBandN : 2];
  extern __shared__ __attribute__((aligned(16))) float sRowScale[]; // [K block][256 rows], already / 16

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
  const int r = lane & 15, q = lane >> 4;
  const int64_t K = a.K, N = a.N;
  const int KB = static_cast<int>(K / kGroup);
  const int64_t I = N / 2;

  // slots of the four 16-token fragments this lane sees in the accumulator layout
  int64_t f[4];
  bool valid[4];
#pragma unroll
  for (int tf = 0; tf < 4; ++tf) {
    f[tf] = a.sorted[static_cast<int64_t>(mb) * kTileM + tf * 16 + r];
    valid[tf] = f[tf] < a.num_valid;
  }

  // weight rows of the wave: four 16-row fragments
  int64_t nrow[4];
#pragma unroll
  for (int rf = 0; rf < 4; ++rf) {
    if constexpr (FUSED_ACT) nrow[rf] = (rf >= 2 ? I : 0) + static_cast<int64_t>(nt) * kGroup + wr * 32 + (rf & 1) * 16;
    else nrow[rf] = static_cast<int64_t>(nt) * 256 + wr * 64 + rf * 16;
  }

  if (e < 0) {
    if constexpr (!FUSED_ACT) {
      if ((!a.skip_nonlocal || e_oob)) {
#pragma unroll
        for (int tf = 0; tf < 4; ++tf)
          if (valid[tf])
#pragma unroll
            for (int rf = 0; rf < 4; ++rf)
              if (nrow[rf] < N) *reinterpret_cast<v2i *>(a.C + f[tf] * N + nrow[rf] + 4 * q) = v2i{0, 0};
      }
    }
    return;
  }

  uint16_t band_regs[kSiluBandPer];
  if constexpr (FUSED_ACT) silu_band_load(band_regs, a.silu, tid);

  // cooperative gather role: thread -> (token, 32-byte quarter of the 128-byte K block)
  const int lt = tid >> 2, lq = tid & 3;
  const int64_t lf = a.sorted[static_cast<int64_t>(mb) * kTileM + lt];
  const int64_t lrow = (lf < a.num_valid) ? lf / a.top_k : 0;
  const brsrc rA = make_rsrc(a.A, static_cast<uint32_t>(a.a_rows * K));
  const brsrc rAs = make_rsrc(a.As, static_cast<uint32_t>(a.a_rows * KB * 4));
  const int aoff = static_cast<int>(lrow * K) + lq * 32;
  const int asoff = static_cast<int>(lrow * KB * 4);
  int8_t *const sdst0 = &sA[0][lt * kW4Row + lq * 32];
  int8_t *const sdst1 = &sA[1][lt * kW4Row + lq * 32];

  const int64_t wbytes = N * K / 2; // one expert
  const brsrc rW = make_rsrc(a.W + static_cast<int64_t>(e) * wbytes, static_cast<uint32_t>(wbytes));
  const brsrc rWs = make_rsrc(a.Ws + static_cast<int64_t>(e) * N * KB, static_cast<uint32_t>(N * KB * 4));
  const int wkstride = shuf_kb_stride(static_cast<int>(N / 16)) / 2;
  int woff[4], wsoff[4];
#pragma unroll
  for (int rf = 0; rf < 4; ++rf) {
    const int64_t nr = nrow[rf] < N ? nrow[rf] : 0; // fragments past N: computed on row 0, never stored
    woff[rf] = static_cast<int>(nr / 16) * (shuf_nb_stride(KB) / 2) + lane * 16; // 1 KB blocks, lane order
    // the lane's rows 4q .. 4q+3 inside the LDS copy of the row scales
    wsoff[rf] = ((FUSED_ACT ? (rf >= 2 ? 128 : 0) + wr * 32 + (rf & 1) * 16 : wr * 64 + rf * 16) + 4 * q) * 4;
  }
  // scales are stored [E][K/128][N]: per K block the workgroup's rows are one run of 256 floats (plain)
  // or two of 128 (gate rows, up rows), copied in pieces of four rows; rows past N
  // read zeros (an offset outside the buffer) and belong to fragments that are never stored.  Eight
  // pieces per thread and pass: 32 K blocks are one memory round trip.
  auto copy_row_scales = [&]() {
    const int sc_total = KB * 64;
    for (int base = 0; base < sc_total; base += 8 * 256) {
      v4i raw[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int p = base + u * 256 + tid;
        const int kb = p >> 6, w4 = p & 63;
        int64_t grow;
        if constexpr (FUSED_ACT) grow = (w4 < 32 ? 0 : I - kGroup) + static_cast<int64_t>(nt) * kGroup + 4 * w4;
        else grow = static_cast<int64_t>(nt) * 256 + 4 * w4;
        const bool in = p < sc_total && grow < N;
        raw[u] = bld16<kWAux>(rWs, in ? static_cast<int>((static_cast<int64_t>(kb) * N + grow) * 4) : 0x7ffffff0, 0);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int p = base + u * 256 + tid;
        if (p < sc_total) {
          v4f sc = __builtin_bit_cast(v4f, raw[u]);
          // every product carries the factor 16 of the unpacked nibbles: 1/16 goes into the row scale (a
          // power of two: (f32(d) * a_s) * (b_s / 16) is bit for bit (f32(d / 16) * a_s) * b_s unless b_s
          // lies below 2^-122 or the product above 2^124)
#pragma unroll
          for (int i = 0; i < 4; ++i) sc[i] = sc[i] * 0.0625f;
          *reinterpret_cast<v4f *>(sRowScale + static_cast<int64_t>(p) * 4) = sc;
        }
      }
    }
  };

  using B0 = std::integral_constant<int, 0>;
  using B1 = std::integral_constant<int, 1>;
  v4f acc[4][4]; // [row fragment][token fragment]
#pragma unroll
  for (int rf = 0; rf < 4; ++rf)
#pragma unroll
    for (int tf = 0; tf < 4; ++tf) acc[rf][tf] = v4f{0.f, 0.f, 0.f, 0.f};

  v4i wreg[2][4]; // [buffer][row fragment]: both k-steps of a K block, packed
  v4i areg[2][2];  // [set][16-byte piece]: token bytes in flight for two K blocks
  float sreg[2] = {0.0f, 0.0f};

  // The K loop is free of branches: a step past the end of K re-reads the last K block and
  // stores a token scale of zero, so it adds exactly 0 to every accumulator.
  // The token bytes of K block kb are requested two iterations before they are needed and
  // written to LDS one iteration before: set = kb & 1 in registers, stage = kb & 1 in LDS.
  auto load_act = [&](auto ST, int kb) {
    constexpr int st = decltype(ST)::value;
    const int kc = kb < KB ? kb : KB - 1;
#pragma unroll
    for (int j = 0; j < 2; ++j) areg[st][j] = bld16(rA, aoff, kc * kGroup + j * 16);
    sreg[st] = bld_f32(rAs, asoff, kc * 4);
  };
  auto store_act = [&](auto ST, bool live) {
    constexpr int st = decltype(ST)::value;
    int8_t *d = st ? sdst1 : sdst0;
#pragma unroll
    for (int j = 0; j < 2; ++j) *reinterpret_cast<v4i *>(d + j * 16) = areg[st][j];
    if (lq == 0) sS[st][lt] = live ? sreg[st] : 0.0f;
  };
  auto load_w = [&](auto BUF, int kb) {
    constexpr int b = decltype(BUF)::value;
    const int kc = kb < KB ? kb : KB - 1;
#pragma unroll
    for (int rf = 0; rf < 4; ++rf) wreg[b][rf] = bld16<kWAux>(rW, woff[rf], kc * wkstride);
  };
  auto fold = [&](const v4i (&d)[4], const v4f &bs16, const float (&as)[4], v4f (&dst)[4]) {
#pragma unroll
    for (int tf = 0; tf < 4; ++tf)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        dst[tf][i] = fold_elem<ORD>(d[tf][i], ORD == kOrdFusedScale ? as[tf] * bs16[i] : 0.0f, as[tf], bs16[i], dst[tf][i]);
#pragma unroll
    for (int tf = 0; tf < 4; ++tf)
#pragma unroll
      for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(dst[tf][i])); // keep the fold here
  };
  auto compute = [&](auto BUF, int kb) {
    constexpr int b = decltype(BUF)::value;
    const int8_t *tile = sA[b];
    v4i bf[4][2];
    float as[4];
    // a step past the end of K reads the last K block's scales (finite: its token scales are zero)
    const char *const srow = reinterpret_cast<const char *>(sRowScale) + (kb < KB ? kb : KB - 1) * 1024;
    v4f bsv[4];
#pragma unroll
    for (int rf = 0; rf < 4; ++rf) bsv[rf] = *reinterpret_cast<const v4f *>(srow + wsoff[rf]);
#pragma unroll
    for (int tf = 0; tf < 4; ++tf) {
      const int8_t *src = tile + (tf * 16 + r) * kW4Row + q * 16;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) bf[tf][ks] = *reinterpret_cast<const v4i *>(src + ks * 64);
      as[tf] = sS[b][tf * 16 + r];
    }
    // software pipeline over the row fragments: the MFMAs of fragment rf are issued, then
    // fragment rf-1 is folded into the fp32 accumulators while the matrix pipe works
    v4i dprev[4];
#pragma unroll
    for (int rf = 0; rf < 4; ++rf) {
      v4i wop[2];
      const v4i pk = wreg[b][rf];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          const uint32_t word = static_cast<uint32_t>(pk[2 * ks + w]);
          wop[ks][2 * w] = static_cast<int>((word << 4) & 0xf0f0f0f0u);
          wop[ks][2 * w + 1] = static_cast<int>(word & 0xf0f0f0f0u);
        }
      v4i d[4];
#pragma unroll
      for (int tf = 0; tf < 4; ++tf) {
        d[tf] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
          d[tf] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wop[ks], bf[tf][ks], d[tf], 0, 0, 0);
      }
      if (rf > 0) fold(dprev, bsv[rf - 1], as, acc[rf - 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int tf = 0; tf < 4; ++tf) dprev[tf] = d[tf];
    }
    fold(dprev, bsv[3], as, acc[3]);
    __builtin_amdgcn_sched_barrier(0);
  };

  load_act(B0{}, 0);
  load_act(B1{}, 1);
  load_w(B0{}, 0);
  __builtin_amdgcn_sched_barrier(0); // the first K block's requests go out ahead of the scales'
  copy_row_scales();
  store_act(B0{}, true);
  if constexpr (FUSED_ACT) silu_band_store(sSilu, band_regs, tid);
  __syncthreads();
  for (int kb = 0; kb < KB; kb += 2) {
    load_act(B0{}, kb + 2);            // needed in two iterations
    load_w(B1{}, kb + 1);              // needed in the next iteration
    __builtin_amdgcn_sched_barrier(0); // keep the prefetch ahead of the MFMAs
    compute(B0{}, kb);
    store_act(B1{}, kb + 1 < KB);      // requested one iteration ago
    __syncthreads();
    load_act(B1{}, kb + 3);
    load_w(B0{}, kb + 2);
    __builtin_amdgcn_sched_barrier(0);
    compute(B1{}, kb + 1);
    store_act(B0{}, kb + 2 < KB);
    __syncthreads();
  }

  if constexpr (!FUSED_ACT) {
    // A lane holds 4 consecutive columns of one token per fragment; stored directly that is
    // 8 bytes to each of 64 rows per instruction.  Each wave turns a 16-token x 64-column piece
    // around in LDS (in order within a wave: no barrier; the token tile's LDS is free after the K
    // loop's last barrier) and stores 128-byte row segments instead.
    int8_t *stg = &sA[0][0] + wr * (16 * kW4Row);
#pragma unroll
    for (int tf = 0; tf < 4; ++tf) {
      float w = 1.0f;
      if (a.mul_routed && valid[tf]) w = a.topk_w[f[tf]];
      with_out16(a.out_f16, [&](auto cvt) __attribute__((always_inline)) {
#pragma unroll
        for (int rf = 0; rf < 4; ++rf) {
          v4u16 o;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float v = acc[rf][tf][i];
            if (a.mul_routed) v = v * w;
            o[i] = cvt(v);
          }
          *reinterpret_cast<v4u16 *>(stg + r * kW4Row + (rf * 16 + 4 * q) * 2) = o;
        }
      });
      __builtin_amdgcn_wave_barrier();
      const int slot = valid[tf] ? static_cast<int>(f[tf]) : -1;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int tok = (lane >> 3) + 8 * j;
        const v4i v = *reinterpret_cast<const v4i *>(stg + tok * kW4Row + (lane & 7) * 16);
        const int ft = __shfl(slot, tok);
        // columns past N (a last tile narrower than 256) are never stored: N % 64 == 0 on this path
        if (ft >= 0 && nrow[0] < N)
          *reinterpret_cast<v4i *>(a.C + static_cast<int64_t>(ft) * N + nrow[0] + (lane & 7) * 8) = v;
      }
      __builtin_amdgcn_wave_barrier();
    }
  } else {
    // acc[0..1] = gate, acc[2..3] = up for activation columns nt*128 + wr*32 + 16*g + 4q + i
    float actf[4][2][4];
#pragma unroll
    for (int tf = 0; tf < 4; ++tf) {
      float w = 1.0f;
      if (a.mul_routed && valid[tf]) w = a.topk_w[f[tf]];
      float amax = 0.0f;
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float gv = acc[g][tf][i], uv = acc[2 + g][tf][i];
          if (a.mul_routed) {
            gv = gv * w;
            uv = uv * w;
          }
          const uint16_t act16 = silu_mul_band(sSilu, a.silu, f32_to_bf16(gv), f32_to_bf16(uv));
          actf[tf][g][i] = bf16_to_f32(act16);
          amax = fmaxf(amax, fabsf(actf[tf][g][i]));
        }
      amax = fmaxf(amax, __shfl_xor(amax, 16));
      amax = fmaxf(amax, __shfl_xor(amax, 32));
      if (q == 0) sRed[wr][tf * 16 + r] = amax;
    }
    __syncthreads();
    const int64_t G = I / kGroup;
    // the quantised tile (64 tokens x 128 columns of int8) leaves through LDS as whole rows
    int8_t *qst = &sA[0][0];
#pragma unroll
    for (int tf = 0; tf < 4; ++tf) {
      const int t = tf * 16 + r;
      float amax = fmaxf(fmaxf(sRed[0][t], sRed[1][t]), fmaxf(sRed[2][t], sRed[3][t]));
      amax = fmaxf(amax, 1e-10f);
      const float sc = amax / 127.0f;
      const float rsc = 1.0f / sc;
#pragma unroll
      for (int g = 0; g < 2; ++g)
        *reinterpret_cast<uint32_t *>(qst + t * kW4Row + wr * 32 + g * 16 + 4 * q) = quant4(actf[tf][g], sc, rsc);
      if (valid[tf] && wr == 0 && q == 0) a.A2s[f[tf] * G + nt] = sc;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kTileM * 8 / 256; ++j) {
      const int id = tid + 256 * j, tok = id >> 3, piece = id & 7;
      const int64_t ft = a.sorted[static_cast<int64_t>(mb) * kTileM + tok];
      if (ft < a.num_valid)
        *reinterpret_cast<v4i *>(a.A2q + ft * I + static_cast<int64_t>(nt) * kGroup + piece * 16) =
            *reinterpret_cast<const v4i *>(qst + tok * kW4Row + piece * 16);
    }
  }
}

bool gemm_w4_tile_supports(const GemmArgs &a, bool fused_act, int block_size_m) {
  if (!fused_act && a.N % 64 != 0) return false; // a wave stores its 64 columns as one piece
  return a.w4 && a.w_shuffled && block_size_m == 64;
}

int launch_gemm_w4_tile(const GemmArgs &a0, bool fused_act, int flags, int64_t m_blocks, hipStream_t s) {
  GemmArgs a = a0;
  a.n_tiles = fused_act ? static_cast<int32_t>(a.N / 2 / kGroup) : static_cast<int32_t>((a.N + 255) / 256);
  int64_t G = a.num_valid / (static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) * 64);
  G = G < 2 ? 2 : (G > 16 ? 16 : G);
  const int64_t chunks = (m_blocks + G - 1) / G;
  const int64_t grid = (chunks + 7) / 8 * (G * a.n_tiles) * 8;
  LO_REQUIRE(grid < (1ll << 31), LO_EINVAL, "moe_gemm(w4): grid too large");
  const int ord = scale_order(flags);
  const dim3 g(static_cast<unsigned>(grid)), b(256);
  const int mbi = static_cast<int>(m_blocks), gi = static_cast<int>(G);
  // the row scales of the workgroup's 256 rows, every K block, sit in LDS next to 28 KB of static arrays
  const int64_t lds = a.K / kGroup * 1024;
  LO_REQUIRE(lds <= 128 * 1024, LO_ENOTSUP, "moe_gemm(w4 tile): K = %lld is more than 128 K groups",
             static_cast<long long>(a.K));
  // one token block per expert, by and large (measured up to 47 slots per expert on average, where the
  // 128-token kernel takes over: whole path at 640 tokens of a 4096 x 1536 layer 0.384 -> 0.359 ms)
  const bool stream = a.num_valid <= static_cast<int64_t>(a.experts_routed > 0 ? a.experts_routed : 1) * 48;
#define LO_W4_TILE_LAUNCH(FA, FS, ST)                                                                          \
  do {                                                                                                         \
    if (lds > 32 * 1024) {                                                                                     \
      static unsigned long long lds_done = 0; /* per instantiation: one bit per device */                      \
      const int rc_lds = reserve_lds_once(reinterpret_cast<const void *>(&moe_gemm_w4_tile_kernel<FA, FS, ST>), \
                                          128 * 1024, &lds_done);                                              \
      if (rc_lds) return rc_lds;                                                                               \
    }                                                                                                          \
    hipLaunchKernelGGL((moe_gemm_w4_tile_kernel<FA, FS, ST>), g, b, static_cast<size_t>(lds), s, a, mbi, gi);  \
  } while (0)
#define LO_W4_TILE_PICK(FS, FA)              \
  do {                                       \
    if (stream) LO_W4_TILE_LAUNCH(FA, FS, true); \
    else LO_W4_TILE_LAUNCH(FA, FS, false);   \
  } while (0)
  if (fused_act) LO_ORD_DISPATCH(ord, LO_W4_TILE_PICK, true);
  else LO_ORD_DISPATCH(ord, LO_W4_TILE_PICK, false);
#undef LO_W4_TILE_PICK
#undef LO_W4_TILE_LAUNCH
  return check_launch(fused_act ? "moe_gemm1_silu_quant(w4 tile)" : "moe_gemm(w4 tile)");
}

} // namespace lo
