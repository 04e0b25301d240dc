// Decode-size whole path of the block-INT8 fused MoE in two launches.
//
// With a handful of tokens the path is a stream of weights (2 * tokens op/B against a ridge of
// 629) and every launch costs about as much as the bytes it moves, so the stages of the
// reference (quant, align, GEMM1, activation + quant, GEMM2, reduce:
// python/lightop/_lmslim_native/layers/fused_moe/int8.py:752-888) are folded into two kernels
// that need no alignment buffers, no quantised copy of x and no per-slot output rows, and whose
// workgroups never wait for one another:
//
//   dec_gemm1_kernel   one workgroup per (routed slot, 16 activation columns).  The workgroup
//                      of the first slot routed to an expert serves all slots of that expert
//                      (it finds them straight from topk_ids; the others leave at once), so an
//                      expert's weights are read once.  Its waves split K: each streams its own
//                      K blocks of the 16 gate rows and the matching 16 up rows from HBM, all
//                      loads in flight at once, quantises its K range of the token rows
//                      (1x128 groups, layers/gemm/int8_utils.py:74-122) into LDS while they
//                      fly, and leaves one product f32(d) * a_s per K block in LDS.  The sum over
//                      K runs in K order (acc = fma(product, b_s, acc), or acc + product * b_s
//                      with LO_GEMM_SEPARATE_ORDER), so after one barrier the last wave walks
//                      the products; it ends with SiLU * mul (int8.py:811-813) and writes the
//                      bf16 activations [S, I].
//   dec_gemm2_kernel   one workgroup per (token, 16 output columns), one wave per routed slot
//                      of the token: the wave re-quantises its slot's activation row
//                      (int8.py:813-823) into LDS while its expert's 16 weight rows are on
//                      their way, multiplies (int8.py:857-880), and the workgroup then reduces
//                      the token's slots in slot order (csrc/kernels/moe_align_sum_kernels.cu:
//                      619-633, :886-909) and writes the output row.  No per-slot rows in HBM
//                      and no separate reduction launch.
//
// The second kernel reads an expert's weights once per slot routed to it, which is why the path
// is taken only while slots rarely share an expert.
#include <cstdlib>
#include <type_traits>

#include "gemm.h"

namespace lo {

constexpr int kDecTP = 4;     // token rows the first kernel multiplies per pass
constexpr int kDecMaxKBw = 7; // K blocks per wave of the first kernel (all held in registers)
constexpr int kDecMaxSlots = 512;
constexpr int kDecMaxKB2 = 32;  // K blocks of the second kernel (I <= 4096): its activation row is held in registers

struct DecArgs {
  const uint16_t *x;         // [M, H] bf16
  const void *ids;           // [S] int32 / int64
  const int32_t *expert_map; // [Eg] or null
  const float *topk_w;       // [S]
  const int8_t *w1, *w2;     // load-time layout
  const float *w1s, *w2s;
  const uint16_t *shared;    // [M, H] or null
  uint16_t *act;             // [S, I] bf16: SiLU(gate) * up of every local slot
  uint16_t *out;             // [M, H]
  float factor;
  int32_t ids64, M, S, top_k, E, Eg, H, I, kbw, mul_on_input;
  int32_t contract;          // acc = fma(f32(d) * a_s, b_s, acc) (the default order); 0: acc + (f32(d) * a_s) * b_s
};

// Global expert id of flat slot s (returned through g) and the local expert that serves it, or -1.
__device__ __forceinline__ int dec_expert(const DecArgs &a, int s, int64_t &g) {
  g = a.ids64 ? static_cast<const int64_t *>(a.ids)[s] : static_cast<const int32_t *>(a.ids)[s];
  int le = -1;
  if (g >= 0 && g < a.Eg) le = a.expert_map ? a.expert_map[g] : static_cast<int>(g);
  return le >= a.E ? -1 : le; // a map entry outside the weight tensor: served by nobody, adds zero
}

// Quantise one 128-value group (8 values per lane of a 16-lane group) and return the packed bytes.
__device__ __forceinline__ v2i dec_quant8(const v8u16 raw, float &scale) {
  float v[8];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    v[i] = bf16_to_f32(raw[i]);
    amax = fmaxf(amax, fabsf(v[i]));
  }
#pragma unroll
  for (int d = 1; d < 16; d <<= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
  amax = fmaxf(amax, 1e-10f);
  const float sc = amax / 127.0f, rsc = 1.0f / sc;
  scale = sc;
  v2i packed;
  packed[0] = static_cast<int>(quant4(&v[0], sc, rsc));
  packed[1] = static_cast<int>(quant4(&v[4], sc, rsc));
  return packed;
}

// The two MFMA operands (k-steps) of a K block from a lane's 16 bytes of packed int4 in the load-time
// layout: int8 values 16 times too large (reference nibble order: layers/fused_moe/w4a8.py:341, :375-377).
__device__ __forceinline__ void unpack_int4(const v4i pk, v4i &w0, v4i &w1) {
#pragma unroll
  for (int x = 0; x < 2; ++x) {
    const uint32_t a0 = static_cast<uint32_t>(pk[x]), a1 = static_cast<uint32_t>(pk[2 + x]);
    w0[2 * x] = static_cast<int>((a0 << 4) & 0xf0f0f0f0u);
    w0[2 * x + 1] = static_cast<int>(a0 & 0xf0f0f0f0u);
    w1[2 * x] = static_cast<int>((a1 << 4) & 0xf0f0f0f0u);
    w1[2 * x + 1] = static_cast<int>(a1 & 0xf0f0f0f0u);
  }
}

__device__ __forceinline__ float lane_value(float v, int l) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}

// Both kernels are chains of dependent memory round trips (ids -> expert -> weights), each about as
// long as the streaming itself at these sizes, so everything whose address does not depend on the
// routing is requested before the routing is looked at, and everything that depends on the expert
// only is requested the moment the expert is known.
// KBW: K blocks a wave holds in registers at most (4, or kDecMaxKBw).  W4: packed int4 weights in their
// load-time layout (one 16-byte piece per lane holds both k-steps of a K block) with one scale per weight
// row and K block, [E, K/128, N]; the factor 16 of the unpacked nibbles leaves through the scales.
template <int KBW, bool W4>
__device__ __forceinline__ void dec_gemm1_body(const DecArgs &a) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int W = blockDim.x >> 6;
  const int n = lane & 15, c = lane >> 4;
  const int rb = blockIdx.x, s0 = blockIdx.y;
  const int KB = a.H / kGroup, KBw = a.kbw, kb0 = wave * KBw;
  const int I = a.I, N = 2 * I;
  const int pitch = KBw * kGroup + 16;

  // LDS: slot list, counter, the products of every K block and their weight scales, per-wave token tiles
  int32_t *const sSlots = reinterpret_cast<int32_t *>(smem);                    // [S rounded up to 4]
  int32_t *const sMeta = sSlots + ((a.S + 3) & ~3);                             // [4]
  float *const sT = reinterpret_cast<float *>(sMeta + 4);                       // [KB][8 values][4 c][TP tokens]
  constexpr int SB = W4 ? 32 : 2; // weight scales per K block: one per row (W4: [8 values][4 c]), else gate block, up block
  float *const sB = sT + KB * 128;                                              // [KB][SB]
  float *const sAs = sB + KB * SB + wave * (kDecTP * KBW);                      // [TP][KBw] of this wave
  int8_t *const sA = reinterpret_cast<int8_t *>(sB + KB * SB + W * (kDecTP * KBW)) + wave * (kDecTP * pitch);

  // ---- requests that do not wait for the routing: the slot's own token row ----------------------
  const int sub = lane & 15, gq = lane >> 4;
  v8u16 raw_own[2];
  {
    const int64_t t = s0 / a.top_k;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int g = gq + 4 * q;
      raw_own[q] = v8u16{0, 0, 0, 0, 0, 0, 0, 0};
      if (g < KBw) raw_own[q] = *reinterpret_cast<const v8u16 *>(a.x + t * a.H + (kb0 + g) * kGroup + sub * 8);
    }
  }
  // (wave 0) the expert ids of the first 128 slots, for the search below (further slots, which only a
  // forced call has, are fetched when the search gets there)
  auto slot_gid = [&](int i) __attribute__((always_inline)) -> int32_t {
    // (expert ids fit 32 bits: anything else is no expert at all)
    if (i >= a.S) return -1;
    const int64_t g = a.ids64 ? static_cast<const int64_t *>(a.ids)[i] : static_cast<const int32_t *>(a.ids)[i];
    return g >= 0 && g < a.Eg ? static_cast<int32_t>(g) : -1;
  };
  int32_t gid[2] = {-1, -1};
  if (wave == 0) {
    gid[0] = slot_gid(lane);
    gid[1] = slot_gid(64 + lane);
  }

  int64_t g0;
  const int e = dec_expert(a, s0, g0);
  if (e < 0) return;

  // ---- the wave's weights: its K blocks of 16 gate rows and of the matching 16 up rows.  Requested
  //      before it is known whether this workgroup is the one that serves the expert: the path is
  //      meant for batches in which two slots rarely meet on an expert. -----------------------------
  const int64_t wbytes = W4 ? static_cast<int64_t>(N) * a.H / 2 : static_cast<int64_t>(N) * a.H;
  const brsrc rW = make_rsrc(a.w1 + static_cast<int64_t>(e) * wbytes, static_cast<uint32_t>(wbytes));
  const brsrc rWs = make_rsrc(a.w1s + static_cast<int64_t>(e) * KB * N, static_cast<uint32_t>(W4 ? static_cast<int64_t>(KB) * N * 4 : 0));
  const int wkstride = W4 ? shuf_kb_stride(N / 16) / 2 : shuf_kb_stride(N / 16);
  const int wnstride = W4 ? shuf_nb_stride(KB) / 2 : shuf_nb_stride(KB);
  int woff[2], wsoff[2];
  woff[0] = rb * wnstride + lane * 16;
  woff[1] = (I / 16 + rb) * wnstride + lane * 16;
  wsoff[0] = (rb * 16 + 4 * c) * 4; // W4: the scales of the lane's four gate rows, then of its four up rows
  wsoff[1] = (I + rb * 16 + 4 * c) * 4;
  v4i wbuf[KBW][2][W4 ? 1 : 2];
  v4f wsc[W4 ? KBW : 1][2];
  auto issue_all = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < KBW; ++p)
      if (p < KBw) {
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          if constexpr (W4) {
            wbuf[p][g][0] = bld16<kCacheStream>(rW, woff[g], (kb0 + p) * wkstride);
            wsc[p][g] = __builtin_bit_cast(v4f, bld16<kCacheStream>(rWs, wsoff[g], (kb0 + p) * N * 4)); // the weights' policy: mixed policies cost time
          } else {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
              wbuf[p][g][ks] = bld16<kCacheStream>(rW, woff[g], (kb0 + p) * wkstride + ks * 1024);
          }
        }
      }
  };
  issue_all();
  // block scales of the wave's K range: lanes 0..7 the gate rows', lanes 8..15 the up rows'
  float bs_l = 0.0f;
  if constexpr (!W4) {
    if (lane < 16 && (lane & 7) < KBw)
      bs_l = a.w1s[(static_cast<int64_t>(e) * (N / kGroup) + (lane >> 3) * (I / kGroup) + rb / 8) * KB + kb0 + (lane & 7)];
  }

  // ---- slots routed to the same expert, ascending; the workgroup of the first one serves them ---
  if (wave == 0) {
    int cnt = 0;
    for (int b = 0; b * 64 < a.S; ++b) {
      const int32_t gb = b == 0 ? gid[0] : (b == 1 ? gid[1] : slot_gid(b * 64 + lane));
      const bool mine = gb == static_cast<int32_t>(g0); // (slots past S hold -1, 0 <= g0 < Eg)
      const uint64_t bal = __builtin_amdgcn_ballot_w64(mine);
      if (mine) sSlots[cnt + __builtin_popcountll(bal & ((1ull << lane) - 1))] = b * 64 + lane;
      cnt += __builtin_popcountll(bal);
    }
    if (lane == 0) sMeta[0] = cnt;
  }
  __syncthreads();
  const int cnt = sMeta[0];
  if (sSlots[0] != s0) return;

  for (int chunk0 = 0; chunk0 < cnt; chunk0 += kDecTP) {
    const int nc = cnt - chunk0 < kDecTP ? cnt - chunk0 : kDecTP;
    if (chunk0 > 0) issue_all(); // an expert with many slots: its weights again for every pass
    // ---- quantise this pass's token rows (the wave's K range only) into the wave's LDS tile -----
    if (cnt == 1) { // the usual case: the row requested at the start
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int g = gq + 4 * q;
        if (g < KBw) {
          float sc;
          const v2i packed = dec_quant8(raw_own[q], sc);
          *reinterpret_cast<v2i *>(sA + g * kGroup + sub * 8) = packed;
          if (sub == 0) sAs[g] = sc;
        }
      }
    } else {
      for (int g = gq; g < nc * KBw; g += 4) {
        const int tokl = g / KBw, kbl = g - tokl * KBw;
        const int64_t t = sSlots[chunk0 + tokl] / a.top_k;
        const v8u16 raw = *reinterpret_cast<const v8u16 *>(a.x + t * a.H + (kb0 + kbl) * kGroup + sub * 8);
        float sc;
        const v2i packed = dec_quant8(raw, sc);
        *reinterpret_cast<v2i *>(sA + tokl * pitch + kbl * kGroup + sub * 8) = packed;
        if (sub == 0) sAs[tokl * KBW + kbl] = sc;
      }
    }
    __builtin_amdgcn_wave_barrier();

    // ---- one product f32(d) * a_s per K block: weights from registers, tokens from LDS; the products
    //      of the pass's tokens and the weight scales they meet go to LDS, K block by K block --------
#pragma unroll
    for (int p = 0; p < KBW; ++p) {
      if (p < KBw) {
        v4i b0 = v4i{0, 0, 0, 0}, b1 = v4i{0, 0, 0, 0};
        float as = 0.0f;
        if (n < nc) {
          b0 = *reinterpret_cast<const v4i *>(sA + n * pitch + p * kGroup + c * 16);
          b1 = *reinterpret_cast<const v4i *>(sA + n * pitch + p * kGroup + 64 + c * 16);
          as = sAs[n * KBW + p];
        }
        const float bs[2] = {lane_value(bs_l, p), lane_value(bs_l, 8 + p)};
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          v4i w0, w1;
          if constexpr (W4) {
            unpack_int4(wbuf[p][g][0], w0, w1);
          } else {
            w0 = wbuf[p][g][0];
            w1 = wbuf[p][g][W4 ? 0 : 1];
          }
          v4i d = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, b0, v4i{0, 0, 0, 0}, 0, 0, 0);
          d = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, b1, d, 0, 0, 0);
          if (n < nc) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              sT[((kb0 + p) * 8 + g * 4 + i) * 16 + c * kDecTP + n] = static_cast<float>(d[i]) * as;
            if constexpr (W4) { // the scales of the lane's four rows, as loaded ([c][i]; the factor 1/16 is applied by the reader)
              if (n == 0) *reinterpret_cast<v4f *>(sB + ((kb0 + p) * 2 + g) * 16 + c * 4) = wsc[W4 ? p : 0][g];
            } else {
              if (lane == 0) sB[(kb0 + p) * 2 + g] = bs[g];
            }
          }
        }
      }
    }
    __syncthreads();

    // ---- the sum over K in K order, SiLU * mul (computed, not looked up: a table entry would be
    //      one more dependent round trip).  Lane (i, c, token) of the last wave adds the gate terms
    //      and the up terms of activation column 4c + i. ---------------------------------------------
    if (wave == W - 1) {
      float accg = 0.0f, accu = 0.0f;
      auto sum_k = [&](auto CONTRACT) __attribute__((always_inline)) {
        auto add = [](float acc, float t, float b) __attribute__((always_inline)) {
          if constexpr (W4) b = b * 0.0625f; // int4 nibbles are unpacked 16 times too large
          if constexpr (decltype(CONTRACT)::value) return __builtin_fmaf(t, b, acc);
          const float tb = t * b;
          return acc + tb;
        };
        // lane (i, c, token): row 4c + i of the fragment
        const int brow = ((lane >> 2) & 3) * 4 + (lane >> 4);
        const float *const bg = sB + (W4 ? brow : 0), *const bu = sB + (W4 ? 16 + brow : 1);
        int kb = 0;
        for (; kb + 4 <= KB; kb += 4) {
          float tg[4], tu[4], sg[4], su[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            tg[j] = sT[(kb + j) * 128 + lane];
            tu[j] = sT[(kb + j) * 128 + 64 + lane];
            sg[j] = bg[(kb + j) * SB];
            su[j] = bu[(kb + j) * SB];
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            accg = add(accg, tg[j], sg[j]);
            accu = add(accu, tu[j], su[j]);
          }
        }
        for (; kb < KB; ++kb) {
          accg = add(accg, sT[kb * 128 + lane], bg[kb * SB]);
          accu = add(accu, sT[kb * 128 + 64 + lane], bu[kb * SB]);
        }
      };
      if (a.contract) sum_k(std::true_type{});
      else sum_k(std::false_type{});
      const int i = lane >> 4, cc = (lane >> 2) & 3, tok = lane & 3;
      if (tok < nc) {
        const int64_t fslot = sSlots[chunk0 + tok];
        if (a.mul_on_input) {
          const float wgt = a.topk_w[fslot];
          accg = accg * wgt;
          accu = accu * wgt;
        }
        a.act[fslot * I + rb * 16 + 4 * cc + i] = silu_mul<LO_BF16>(f32_to_bf16(accg), f32_to_bf16(accu));
      }
    }
    if (chunk0 + kDecTP < cnt) __syncthreads(); // the terms' LDS is free again
  }
}

// Up to four K blocks per wave: half the registers, so four waves per SIMD (twice the workgroups in
// flight per compute unit) instead of two.
template <bool W4>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void dec_gemm1_small_kernel(const DecArgs a) {
  dec_gemm1_body<4, W4>(a);
}
template <bool W4>
__global__ __launch_bounds__(512) void dec_gemm1_kernel(const DecArgs a) { dec_gemm1_body<kDecMaxKBw, W4>(a); }

template <int PD, int RAWN, bool W4> // weight K blocks in flight per wave; 16-byte pieces of the activation row per lane
__global__ __launch_bounds__(512) void dec_gemm2_kernel(const DecArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int W = blockDim.x >> 6;
  const int n = lane & 15, c = lane >> 4;
  const int rb = blockIdx.x, t = blockIdx.y;
  const int H = a.H, I = a.I, KB = I / kGroup, k = a.top_k;

  uint16_t *const sC = reinterpret_cast<uint16_t *>(smem);                     // [k][16] per-slot output values
  uint8_t *const sLoc = reinterpret_cast<uint8_t *>(sC + k * 16);              // [k] slot served by this rank
  const int head = (k * 16 * 2 + k + 15) & ~15;
  float *const sAs = reinterpret_cast<float *>(smem + head) + wave * KB;       // [KB] of this wave
  int8_t *const sA = smem + head + ((W * KB * 4 + 15) & ~15) + wave * I;       // [I] of this wave

  const int sub = lane & 15, gq = lane >> 4;
  for (int j = wave; j < k; j += W) {
    const int s = t * k + j;
    // the slot's activation row and routed weight do not wait for the routing
    v8u16 raw[RAWN];
#pragma unroll
    for (int q = 0; q < RAWN; ++q) {
      raw[q] = v8u16{0, 0, 0, 0, 0, 0, 0, 0};
      if (gq + 4 * q < KB)
        raw[q] = *reinterpret_cast<const v8u16 *>(a.act + static_cast<int64_t>(s) * I + (gq + 4 * q) * kGroup + sub * 8);
    }
    const float wgt = a.mul_on_input ? 1.0f : a.topk_w[s];
    int64_t g;
    const int e = dec_expert(a, s, g);
    if (lane == 0) sLoc[j] = e >= 0 ? 1 : 0;
    if (e < 0) continue; // (its activation row was never written: nothing of it is used)

    const int64_t wbytes = W4 ? static_cast<int64_t>(H) * I / 2 : static_cast<int64_t>(H) * I;
    const brsrc rW = make_rsrc(a.w2 + static_cast<int64_t>(e) * wbytes, static_cast<uint32_t>(wbytes));
    const brsrc rWs = make_rsrc(a.w2s + static_cast<int64_t>(e) * KB * H, static_cast<uint32_t>(W4 ? static_cast<int64_t>(KB) * H * 4 : 0));
    const int wkstride = W4 ? shuf_kb_stride(H / 16) / 2 : shuf_kb_stride(H / 16);
    const int woff = rb * (W4 ? shuf_nb_stride(KB) / 2 : shuf_nb_stride(KB)) + lane * 16;
    const int wsoff = (rb * 16 + 4 * c) * 4; // W4: the scales of the lane's four rows
    v4i wbuf[PD][W4 ? 1 : 2];
    v4f wsc[W4 ? PD : 1];
    auto issue = [&](int p, int kb) __attribute__((always_inline)) {
      if constexpr (W4) {
        wbuf[p][0] = bld16<kCacheStream>(rW, woff, kb * wkstride);
        wsc[p] = __builtin_bit_cast(v4f, bld16<kCacheStream>(rWs, wsoff, kb * H * 4));
      } else {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) wbuf[p][ks] = bld16<kCacheStream>(rW, woff, kb * wkstride + ks * 1024);
      }
    };
#pragma unroll
    for (int p = 0; p < PD; ++p)
      if (p < KB) issue(p, p);
    float bs_l = 0.0f; // lane l: the block scale of K block l
    if constexpr (!W4) {
      if (lane < KB) bs_l = a.w2s[(static_cast<int64_t>(e) * (H / kGroup) + rb / 8) * KB + lane];
    }

    // the activation row, re-quantised in 1x128 groups, into the wave's LDS row
#pragma unroll
    for (int q = 0; q < RAWN; ++q) {
      const int gi = gq + 4 * q;
      if (gi < KB) {
        float sc;
        const v2i packed = dec_quant8(raw[q], sc);
        *reinterpret_cast<v2i *>(sA + gi * kGroup + sub * 8) = packed;
        if (sub == 0) sAs[gi] = sc;
      }
    }
    __builtin_amdgcn_wave_barrier();

    v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
    for (int kb0 = 0; kb0 < KB; kb0 += PD) {
#pragma unroll
      for (int p = 0; p < PD; ++p) {
        const int kb = kb0 + p;
        if (kb < KB) {
          // every column of the token operand is the same row: all lanes end up with valid sums
          const v4i b0 = *reinterpret_cast<const v4i *>(sA + kb * kGroup + c * 16);
          const v4i b1 = *reinterpret_cast<const v4i *>(sA + kb * kGroup + 64 + c * 16);
          v4i w0, w1;
          v4f bs4 = v4f{0.f, 0.f, 0.f, 0.f};
          if constexpr (W4) {
            unpack_int4(wbuf[p][0], w0, w1);
            bs4 = wsc[W4 ? p : 0] * 0.0625f;
          } else {
            w0 = wbuf[p][0];
            w1 = wbuf[p][W4 ? 0 : 1];
          }
          v4i d = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, b0, v4i{0, 0, 0, 0}, 0, 0, 0);
          d = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, b1, d, 0, 0, 0);
          if (kb + PD < KB) issue(p, kb + PD);
          const float as = sAs[kb], bs = lane_value(bs_l, kb);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float tt = static_cast<float>(d[i]) * as;
            if (a.contract) {
              acc[i] = __builtin_fmaf(tt, W4 ? bs4[i] : bs, acc[i]);
            } else {
              tt = tt * (W4 ? bs4[i] : bs);
              acc[i] = acc[i] + tt;
            }
          }
        }
      }
    }
    if (n == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = acc[i];
        if (!a.mul_on_input) v = v * wgt;
        sC[j * 16 + 4 * c + i] = f32_to_bf16(v);
      }
    }
    __builtin_amdgcn_wave_barrier(); // the next slot of this wave reuses the LDS row
  }
  __syncthreads();

  // ---- the token's slots in slot order, the slots of other ranks left out ------------------------
  if (tid < 16) {
    float acc = 0.0f;
    for (int j = 0; j < k; ++j)
      if (sLoc[j]) acc = acc + bf16_to_f32(sC[j * 16 + tid]);
    const int64_t o = static_cast<int64_t>(t) * H + rb * 16 + tid;
    uint16_t r;
    if (a.shared) {
      uint16_t xv = f32_to_bf16(acc);
      xv = f32_to_bf16(bf16_to_f32(xv) * a.factor);
      r = f32_to_bf16(bf16_to_f32(xv) + bf16_to_f32(a.shared[o]));
    } else {
      r = f32_to_bf16(acc * a.factor);
    }
    a.out[o] = r;
  }
}


// K split of the first kernel: waves per workgroup such that each holds at most kDecMaxKBw K
// blocks, preferring four or more blocks per wave.  0: no admissible split.
static int pick_waves(int KB) {
  int fallback = 0;
  for (int w = 8; w >= 1; w >>= 1) {
    if (KB % w || KB / w > kDecMaxKBw) continue;
    if (KB / w >= 4) return w;
    fallback = w; // fewer than four blocks per wave: take the smallest such split
  }
  return fallback;
}

// Largest number of routed slots the two-launch path is taken for.  Its second kernel reads an
// expert's weights once per slot, so it pays while slots rarely share an expert.
static int decode_max_slots() {
  static const int v = [] {
    const char *s = std::getenv("LIGHTOP_AMD_DECODE_MAX_SLOTS");
    if (!s || !*s) return -1;
    const long x = std::strtol(s, nullptr, 10);
    return static_cast<int>(x < 0 ? 0 : (x > kDecMaxSlots ? kDecMaxSlots : x));
  }();
  return v;
}

bool decode_path_applies(int64_t M, int32_t top_k, int64_t H, int64_t I, int32_t num_experts, bool force, bool w4) {
  const int64_t S = M * top_k;
  if (S > kDecMaxSlots || top_k > 64) return false;
  if (H % kGroup || I % kGroup || 2 * I * H >= (1ll << 31)) return false;
  if (I > H || I / kGroup > kDecMaxKB2) return false; // the bf16 activations [S, I] live in the caller's [S, H] buffer
  if (pick_waves(static_cast<int>(H / kGroup)) == 0) return false;
  if (force) return true;
  const int forced = decode_max_slots();
  if (forced >= 0) return S <= forced;
  // measured on both benchmark layers (top-8 routing): well ahead of the five-stage path at one and
  // two tokens, ahead at four; at eight only where a wave holds at most four K blocks (the first
  // kernel then fits four waves per SIMD: Qwen3 layer 62 against 67 us, DeepSeek share 114 against
  // 78 us); behind from sixteen on: its workgroups hold their whole share of the weights in
  // registers and live too briefly to overlap one another
  (void)num_experts;
  const int KB = static_cast<int>(H / kGroup);
  // packed int4 (Qwen3-235B-A22B-shaped layer): 33 against 41 us at one token, level at two, behind at four
  if (w4) return S <= 16;
  return S <= 32 || (S <= 64 && KB / pick_waves(KB) <= 4);
}

void decode_path_waves(int32_t top_k, int64_t H, int *gemm1_waves, int *gemm2_waves) {
  *gemm1_waves = pick_waves(static_cast<int>(H / kGroup));
  *gemm2_waves = top_k < 8 ? top_k : 8;
}

// Whole path in two launches; LO_ENOTSUP when the problem is not a decode-size one this file serves.
// act: room for [S, I] bf16 (the caller's cache13 has it).
int launch_decode_path(const void *x, int64_t M, int64_t H, int64_t I, int32_t E, int32_t num_experts, int32_t top_k,
                       const int8_t *w1, const float *w1s, const int8_t *w2, const float *w2s, const float *topk_w,
                       const void *topk_ids, int ids_dtype, const int32_t *expert_map, int apply_router_weight_on_input,
                       float factor, const void *shared_output, void *act, void *out, bool force, bool w4, int flags,
                       hipStream_t stream) {
  if (!decode_path_applies(M, top_k, H, I, num_experts, force, w4)) return LO_ENOTSUP;
  const int64_t S = M * top_k;
  const int KB1 = static_cast<int>(H / kGroup), KB2 = static_cast<int>(I / kGroup);
  int W1, W2;
  decode_path_waves(top_k, H, &W1, &W2);

  DecArgs a{};
  a.x = static_cast<const uint16_t *>(x);
  a.ids = topk_ids; a.ids64 = ids_dtype == LO_I64; a.expert_map = expert_map; a.topk_w = topk_w;
  a.w1 = w1; a.w2 = w2; a.w1s = w1s; a.w2s = w2s;
  a.shared = static_cast<const uint16_t *>(shared_output);
  a.act = static_cast<uint16_t *>(act); a.out = static_cast<uint16_t *>(out);
  a.factor = factor;
  a.M = static_cast<int>(M); a.S = static_cast<int>(S); a.top_k = top_k; a.E = E; a.Eg = num_experts;
  a.H = static_cast<int>(H); a.I = static_cast<int>(I); a.kbw = KB1 / W1;
  a.mul_on_input = apply_router_weight_on_input ? 1 : 0;
  // two orders only: LO_GEMM_FUSED_SCALE buys nothing at this size and gets the default order
  a.contract = scale_order(flags) == kOrdSeparate ? 0 : 1;

  const size_t l1 = static_cast<size_t>((S + 3) & ~int64_t(3)) * 4 + 16 + static_cast<size_t>(KB1) * (128 + (w4 ? 32 : 2)) * 4 +
                    static_cast<size_t>(W1) * kDecTP * kDecMaxKBw * 4 +
                    static_cast<size_t>(W1) * kDecTP * (a.kbw * kGroup + 16);
  const size_t l2 = ((static_cast<size_t>(top_k) * 33 + 15) & ~size_t(15)) + ((static_cast<size_t>(W2) * KB2 * 4 + 15) & ~size_t(15)) +
                    static_cast<size_t>(W2) * I;
  if (l1 > 64 * 1024 || l2 > 64 * 1024) return LO_ENOTSUP;
  const dim3 g1(static_cast<unsigned>(I / 16), static_cast<unsigned>(S)), g2(static_cast<unsigned>(H / 16), static_cast<unsigned>(M));
  // fewer registers where the shape allows it: more workgroups in flight per compute unit
#define LO_DEC_LAUNCH(W4)                                                                                        \
  do {                                                                                                           \
    if (a.kbw <= 4) hipLaunchKernelGGL(dec_gemm1_small_kernel<W4>, g1, dim3(64 * W1), l1, stream, a);            \
    else hipLaunchKernelGGL(dec_gemm1_kernel<W4>, g1, dim3(64 * W1), l1, stream, a);                             \
    const int rc = check_launch("fused_experts(decode, gemm1)");                                                 \
    if (rc) return rc;                                                                                           \
    if (KB2 <= 6) hipLaunchKernelGGL((dec_gemm2_kernel<6, 2, W4>), g2, dim3(64 * W2), l2, stream, a);            \
    else if (KB2 <= 8) hipLaunchKernelGGL((dec_gemm2_kernel<8, 2, W4>), g2, dim3(64 * W2), l2, stream, a);       \
    else if (KB2 <= 16) hipLaunchKernelGGL((dec_gemm2_kernel<8, 4, W4>), g2, dim3(64 * W2), l2, stream, a);      \
    else hipLaunchKernelGGL((dec_gemm2_kernel<8, 8, W4>), g2, dim3(64 * W2), l2, stream, a);                     \
  } while (0)
  if (w4) LO_DEC_LAUNCH(true);
  else LO_DEC_LAUNCH(false);
#undef LO_DEC_LAUNCH
  return check_launch("fused_experts(decode, gemm2)");
}

} // namespace lo
