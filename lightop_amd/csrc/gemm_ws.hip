// Grouped block-INT8 GEMM for gfx950, weight-streaming form.
//
// Each wavefront keeps 16 weight rows "stationary": it streams them from HBM
// straight into registers (16 bytes per lane, no LDS hop, every byte read once by
// one wave) and multiplies them with up to BM = 16*TM gathered token rows using
// v_mfma_i32_16x16x64_i8, with the weight tile as the A operand and the token tile
// as the B operand, so that a lane ends up with 4 consecutive output columns of one
// token.  The int32 partial sum of each 128-wide K block is exact; it is converted
// to fp32 and scaled by the token's group scale and the weight block's scale before
// it is added to the fp32 accumulator (Triton fused_moe_kernel, reference
// python/lightop/_lmslim_native/layers/fused_moe/int8.py:485-519).
//
// With FUSED_ACT the workgroup (8 waves) owns one 128-wide group of activation
// columns: each wave computes 16 gate rows and the matching 16 up rows, and the
// epilogue rounds both to bf16, applies SiLU(gate)*up, reduces the group's amax
// through LDS and writes the int8 re-quantised activations and their scales
// (int8.py:811-823), so that the first GEMM's output never reaches HBM.
//
// This form is meant for the HBM-bound regime (few tokens per expert); it needs no
// barrier in the main loop and keeps PD K-blocks of loads in flight per wave.
#include "gemm.h"

#ifndef LO_WS_STREAM_TM
#define LO_WS_STREAM_TM 2
#endif
#ifndef LO_WS_PD_SMALL
#define LO_WS_PD_SMALL 4
#endif
#ifndef LO_WS_PD_PLAIN
#define LO_WS_PD_PLAIN 2
#endif

namespace lo {

//
// W4: the weights are packed signed int4 in the load-time layout of preshuffle_int4_kernel
// (one 16-byte load per lane holds both k-steps of a 128-wide K block; two vector
// instructions per 8 elements turn them into int8 values 16 times too large, which the
// row scales take out again as a factor 1/16) and every weight row has its own scale per K
// block, stored K-group-major, Ws [E, K/128, N].  The workgroup copies the scales of its rows for
// every K block into LDS before the K loop (6 % of its weight bytes, requested together with
// the first weight blocks), already divided by 16; a lane then reads the scales of its four rows
// as one 16-byte LDS read per fragment and K block (fetched inside the loop, one 4-byte load per
// lane, fragment and K block and the other three rows by DPP from the quad, they were as many
// memory instructions as the weights themselves).
//
// PC (per-channel W8A8, reference csrc/moe_gemm/w8a8/moe_w8a8.cu:156-166, :445-470): one scale
// per token row, As [a_rows], and one per weight row, Ws [E, N]; the int32 sum runs over the
// whole K inside the MFMA accumulator and the scales are applied once, in the epilogue:
// C = bf16((f32(d) * ts) * Ws[e, n]) with ts = As[row], or topk_w[f] * As[row].
//
// W4 and PC together are the reference's own int4 form (fused_moe_kernel_int4_w4a8,
// python/lightop/_lmslim_native/layers/fused_moe/w4a8.py:341-395): the nibbles enter the sum as
// int8(nibble << 4), the factor 16 stays in it, and C = bf16(((f32(d) [* topk_w[f]]) * As[row])
// * Ws[e, n]).
template <int TM, bool FUSED_ACT, int ORD, bool SHUF, int NWAVES, int PD, int RPW, bool W4 = false,
          bool PC = false>
__global__ __launch_bounds__(NWAVES * 64) void moe_gemm_ws_kernel(const GemmArgs a) {
  static_assert(!W4 || SHUF, "int4 weights exist in the load-time layout only");
  static_assert(!PC || !FUSED_ACT, "the per-channel form is a plain GEMM");
  constexpr int BM = 16 * TM;
  constexpr int NS = W4 ? 4 : 1; // weight scales per 16-row fragment and lane
  // 16-row weight fragments per wave: (gate, up) when fused, else RPW consecutive ones
  constexpr int NW = FUSED_ACT ? 2 : RPW;
  // With at most 32 tokens per block an expert's weights are read by one pass only:
  // mark those loads as streaming so that they do not displace the activations in L2.
  constexpr int WAUX = (TM <= LO_WS_STREAM_TM) ? kCacheStream : kCacheDefault;
  const int bid = blockIdx.x;
  const int mb = bid / a.n_tiles, nt = bid - mb * a.n_tiles;
  if (static_cast<int64_t>(mb) * BM >= a.ntpp[0]) return;
  // An expert_map entry outside the weight tensor is treated like an expert of another rank, but its
  // rows are always zero-filled: the slot mask of the alignment counts such a slot as local.
  const int e_raw = a.expert_ids[mb];
  const bool e_oob = e_raw >= a.E;
  const int e = e_oob ? -1 : e_raw;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // wave-uniform: scalar address math
  const int r = lane & 15, c = lane >> 4;
  const int64_t K = a.K, N = a.N;
  const int KB = static_cast<int>(K / kGroup);

  // tokens of this block, one per (sub-tile, r)
  int64_t f[TM];
  bool valid[TM];
  int aoff[TM], asoff[TM]; // byte offsets of the token's row in A and As
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    f[j] = a.sorted[static_cast<int64_t>(mb) * BM + j * 16 + r];
    valid[j] = f[j] < a.num_valid;
    const int64_t row = valid[j] ? f[j] / a.top_k : 0;
    aoff[j] = static_cast<int>(row * K) + c * 16;
    asoff[j] = static_cast<int>(row * (PC ? 1 : KB) * 4);
  }
  const brsrc rA = make_rsrc(a.A, static_cast<uint32_t>(a.a_rows * K));
  const brsrc rAs = make_rsrc(a.As, static_cast<uint32_t>(a.a_rows * (PC ? 1 : KB) * 4));

  constexpr bool kScalesInLds = W4 && !PC;
  constexpr int ROWS = FUSED_ACT ? 256 : 16 * NWAVES * RPW; // weight rows of the workgroup
  bool wave_dead = false; // no rows left for this wave (it still helps with the scale copy)
  if constexpr (!FUSED_ACT) {
    const int64_t n0 = static_cast<int64_t>(nt) * (16 * NWAVES * RPW) + wave * (16 * RPW);
    wave_dead = n0 >= N;
    if (wave_dead && (!kScalesInLds || e < 0)) return;
    if (e < 0) { // expert not held by this rank: the rows are defined to be zero
      if (a.skip_nonlocal && !e_oob) return;
#pragma unroll
      for (int j = 0; j < TM; ++j)
        if (valid[j])
#pragma unroll
          for (int g = 0; g < NW; ++g)
            if (n0 + g * 16 < N) {
              if (a.out_f32)
                *reinterpret_cast<v4i *>(reinterpret_cast<float *>(a.C) + f[j] * N + n0 + g * 16 + 4 * c) = v4i{0, 0, 0, 0};
              else
                *reinterpret_cast<v2i *>(a.C + f[j] * N + n0 + g * 16 + 4 * c) = v2i{0, 0};
            }
      return;
    }
  } else {
    if (e < 0) return;
  }

  // weight rows of this wave
  const int64_t I = N / 2; // fused only
  int64_t nrow[NW];
  if constexpr (FUSED_ACT) {
    nrow[0] = static_cast<int64_t>(nt) * kGroup + wave * 16;
    nrow[NW - 1] = I + nrow[0];
  } else {
#pragma unroll
    for (int g = 0; g < NW; ++g)
      nrow[g] = static_cast<int64_t>(nt) * (16 * NWAVES * RPW) + wave * (16 * RPW) + g * 16;
  }
  const int NB = static_cast<int>((N + kGroup - 1) / kGroup);
  const int64_t wbytes = W4 ? N * K / 2 : N * K; // one expert
  const brsrc rW = make_rsrc(a.W + static_cast<int64_t>(e) * wbytes, static_cast<uint32_t>(wbytes));
  const brsrc rWs = PC ? make_rsrc(a.Ws + static_cast<int64_t>(e) * N, static_cast<uint32_t>(N * 4))
                       : make_rsrc(a.Ws + static_cast<int64_t>(e) * N * KB, static_cast<uint32_t>(W4 ? N * KB * 4 : 0));
  int woff[NW];
  const float *wsrow[NW];
  int wsoff[NW]; // W4 with PC: byte offset of the lane's first scale row; W4: the same inside the LDS copy
  const int wkstride = W4 ? shuf_kb_stride(static_cast<int>(N / 16)) / 2 : shuf_kb_stride(static_cast<int>(N / 16));
#pragma unroll
  for (int g = 0; g < NW; ++g) {
    if constexpr (W4) // 1 KB blocks; both k-steps of a lane in one 16-byte piece
      woff[g] = static_cast<int>(nrow[g] / 16) * (shuf_nb_stride(KB) / 2) + lane * 16;
    else if constexpr (SHUF) // 2 KB blocks; one MFMA operand = 1 KB in lane order
      woff[g] = static_cast<int>(nrow[g] / 16) * shuf_nb_stride(KB) + lane * 16;
    else
      woff[g] = static_cast<int>((nrow[g] + r) * K) + c * 16;
    const int64_t nclamp = nrow[g] < N ? nrow[g] : 0; // fragments past N: loads return 0, nothing is stored
    wsrow[g] = a.Ws + (static_cast<int64_t>(e) * NB + nclamp / kGroup) * KB;
    // accumulator rows of this lane: 4c .. 4c+3
    if constexpr (kScalesInLds)
      wsoff[g] = ((FUSED_ACT ? g * 128 + wave * 16 : wave * (16 * RPW) + g * 16) + 4 * c) * 4;
    else
      wsoff[g] = static_cast<int>((nclamp + 4 * c) * 4);
  }

  v4f acc[NW][TM];
  v4i acci[NW][TM]; // PC: the whole-K int32 sums
#pragma unroll
  for (int g = 0; g < NW; ++g)
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      acc[g][j] = v4f{0.f, 0.f, 0.f, 0.f};
      acci[g][j] = v4i{0, 0, 0, 0};
    }

  // register ring: PD K-blocks (128 bytes of K per row each) in flight, together with
  // the scales that belong to them.  The scales travel in the same ring because the
  // vector-memory counter retires in order: a scale load issued after a prefetch could
  // only be waited for by draining the prefetch as well.
  v4i wbuf[PD][NW][W4 ? 1 : 2];
  v4i abuf[PD][TM][2];
  float asbuf[PD][TM];
  float bsbuf[PD][NW][1]; // (int4 weights: the row scales come from LDS)
  // The loop body is kept free of branches: a slot past the end of K re-reads the last
  // K block and gets a token scale of zero, so it adds exactly 0 to every accumulator.
  // (Branches around the loads make the compiler fall back to waiting for all of them.)
  auto issue = [&](int slot, int kb) {
    const int kc = kb < KB ? kb : KB - 1;
    if constexpr (W4) {
#pragma unroll
      for (int g = 0; g < NW; ++g) wbuf[slot][g][0] = bld16<WAUX>(rW, woff[g], kc * wkstride);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      if constexpr (!W4) {
#pragma unroll
        for (int g = 0; g < NW; ++g)
          wbuf[slot][g][ks] = SHUF ? bld16<WAUX>(rW, woff[g], kc * wkstride + ks * 1024)
                                   : bld16<WAUX>(rW, woff[g], kc * kGroup + ks * 64);
      }
#pragma unroll
      for (int j = 0; j < TM; ++j) abuf[slot][j][ks] = bld16(rA, aoff[j], kc * kGroup + ks * 64);
    }
    if constexpr (PC) return; // no scales inside the K loop
#pragma unroll
    for (int g = 0; g < NW; ++g) {
      if constexpr (!W4) bsbuf[slot][g][0] = wsrow[g][kc];
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) asbuf[slot][j] = bld_f32(rAs, asoff[j], kc * 4);
  };
  extern __shared__ __attribute__((aligned(16))) float sRowScale[]; // [K block][ROWS], already / 16
  // scales are stored [E][K/128][N]: per K block the workgroup's rows are one run of ROWS floats
  // (plain) or two of 128 (gate rows, up rows).  Four pieces of four rows per thread and pass, so
  // that a pass is one memory round trip; rows past N and pieces past the last K block read zeros
  // (an offset outside the buffer) and belong to fragments that are never stored.
  constexpr int kPieces = ROWS / 4, kThreads = NWAVES * 64;
  const int sc_total = KB * kPieces;
  auto scale_load = [&](int base, v4i (&raw)[4]) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = base + u * kThreads + static_cast<int>(threadIdx.x);
      const int kb = p / kPieces, w4 = p - kb * kPieces;
      int64_t grow;
      if constexpr (FUSED_ACT) grow = (w4 < 32 ? 0 : I - kGroup) + static_cast<int64_t>(nt) * kGroup + 4 * w4;
      else grow = static_cast<int64_t>(nt) * ROWS + 4 * w4;
      const bool in = p < sc_total && grow < N;
      // with the weights' cache policy: next to streaming weight loads, scale loads with the default policy
      // cost 15 % of the launch (measured at 32 tokens of a 4096 x 1536 layer: 162 -> 138 us)
      raw[u] = bld16<WAUX>(rWs, in ? static_cast<int>((static_cast<int64_t>(kb) * N + grow) * 4) : 0x7ffffff0, 0);
    }
  };
  auto scale_store = [&](int base, const v4i (&raw)[4]) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = base + u * kThreads + static_cast<int>(threadIdx.x);
      if (p < sc_total) {
        v4f sc = __builtin_bit_cast(v4f, raw[u]);
        // every product carries the factor 16 of the unpacked nibbles: 1/16 goes into the row scales (a
        // power of two: (f32(d) * a_s) * (b_s / 16) is bit for bit (f32(d / 16) * a_s) * b_s unless b_s
        // lies below 2^-122 or the product above 2^124)
#pragma unroll
        for (int i = 0; i < 4; ++i) sc[i] = sc[i] * 0.0625f;
        *reinterpret_cast<v4f *>(sRowScale + static_cast<int64_t>(p) * 4) = sc;
      }
    }
  };
  // the first pass of scale loads goes out ahead of the weight ring and lands first (loads return in
  // order), so that it is in LDS while the first weight blocks are still on their way
  v4i sc_raw[4];
  if constexpr (kScalesInLds) {
    scale_load(0, sc_raw);
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int p = 0; p < PD; ++p) {
    issue(p, p);
    __builtin_amdgcn_sched_barrier(0); // keep the slots in issue order: the waits count on it
  }
  if constexpr (kScalesInLds) {
    scale_store(0, sc_raw);
    for (int base = 4 * kThreads; base < sc_total; base += 4 * kThreads) { // more than 32 K blocks
      scale_load(base, sc_raw);
      scale_store(base, sc_raw);
    }
    __syncthreads();
    if (wave_dead) return;
  }

  for (int kb0 = 0; kb0 < KB; kb0 += PD) {
#pragma unroll
    for (int p = 0; p < PD; ++p) {
      const int kb = kb0 + p;
      v4i d[NW][TM];
#pragma unroll
      for (int g = 0; g < NW; ++g) {
        v4i wop[2]; // the two k-steps of the weight fragment as MFMA operands
        if constexpr (W4) {
          const v4i pk = wbuf[p][g][0];
#pragma unroll
          for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int w = 0; w < 2; ++w) {
              const uint32_t word = static_cast<uint32_t>(pk[2 * ks + w]);
              wop[ks][2 * w] = static_cast<int>((word << 4) & 0xf0f0f0f0u);
              wop[ks][2 * w + 1] = static_cast<int>(word & 0xf0f0f0f0u);
            }
        } else {
          wop[0] = wbuf[p][g][0];
          wop[1] = wbuf[p][g][W4 ? 0 : 1];
        }
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          if constexpr (PC) {
            // a slot past the end of K holds a copy of the last K block: feed zeros instead
            const v4i z = v4i{0, 0, 0, 0};
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
              acci[g][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wop[ks], kb < KB ? abuf[p][j][ks] : z, acci[g][j], 0, 0, 0);
            continue;
          }
          d[g][j] = v4i{0, 0, 0, 0};
#pragma unroll
          for (int ks = 0; ks < 2; ++ks)
            d[g][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wop[ks], abuf[p][j][ks], d[g][j], 0, 0, 0);
        }
      }
      float bs[NW][NS], as[TM];
      if constexpr (!PC) {
#pragma unroll
        for (int g = 0; g < NW; ++g) {
          if constexpr (W4) { // a dead slot reads the last K block's scales (finite: its token scale is zero)
            const int kc = kb < KB ? kb : KB - 1;
            const v4f sc = *reinterpret_cast<const v4f *>(reinterpret_cast<const char *>(sRowScale) + kc * (ROWS * 4) + wsoff[g]);
#pragma unroll
            for (int i = 0; i < NS; ++i) bs[g][i] = sc[i];
          } else {
            bs[g][0] = bsbuf[p][g][0];
          }
        }
#pragma unroll
        for (int j = 0; j < TM; ++j) as[j] = kb < KB ? asbuf[p][j] : 0.0f; // dead slot: adds 0
      }
      // pin the refill of this slot here: the scheduler would otherwise sink the loads
      // next to their use (to save registers) and lose the prefetch distance
      __builtin_amdgcn_sched_barrier(0);
      issue(p, kb + PD);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (PC) continue;
#pragma unroll
      for (int j = 0; j < TM; ++j) {
#pragma unroll
        for (int g = 0; g < NW; ++g) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float b = bs[g][W4 ? i : 0];
            acc[g][j][i] = fold_elem<ORD>(d[g][j][i], ORD == kOrdFusedScale ? as[j] * b : 0.0f, as[j], b, acc[g][j][i]);
          }
        }
      }
    }
  }

  if constexpr (PC) {
    v4f bs4[NW];
#pragma unroll
    for (int g = 0; g < NW; ++g) bs4[g] = __builtin_bit_cast(v4f, bld16(rWs, wsoff[g], 0));
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      if (!valid[j]) continue;
      const float as = bld_f32(rAs, asoff[j], 0);
      const float w = a.mul_routed ? a.topk_w[f[j]] : 1.0f;
      const float ts = a.mul_routed ? w * as : as;
#pragma unroll
      for (int g = 0; g < NW; ++g) {
        if (nrow[g] >= N) continue;
        v4u16 o;
        with_out16(a.out_f16, [&](auto cvt) __attribute__((always_inline)) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float t;
            if constexpr (W4) {
              // the reference's int4 kernel keeps the factor 16 of its unpacked nibbles in the sum
              // (a multiple of 16 below 2^28, exact in fp32) and scales left to right: routed
              // weight, token scale, channel scale (w4a8.py:386-395)
              t = static_cast<float>(acci[g][j][i]);
              if (a.mul_routed) t = t * w;
              t = t * as;
            } else {
              t = static_cast<float>(acci[g][j][i]) * ts;
            }
            o[i] = cvt(t * bs4[g][i]);
          }
        });
        *reinterpret_cast<v4u16 *>(a.C + f[j] * N + nrow[g] + 4 * c) = o;
      }
    }
  } else if constexpr (!FUSED_ACT) {
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      if (!valid[j]) continue;
      float w = 1.0f;
      if (a.mul_routed) w = a.topk_w[f[j]];
#pragma unroll
      for (int g = 0; g < NW; ++g) {
        if (nrow[g] >= N) continue;
        if (__builtin_expect(a.out_f32 != 0, 0)) { // fp32 rows: the sum itself, unrounded (compute_type tl.float32)
          v4f o32;
#pragma unroll
          for (int i = 0; i < 4; ++i) o32[i] = a.mul_routed ? acc[g][j][i] * w : acc[g][j][i];
          *reinterpret_cast<v4f *>(reinterpret_cast<float *>(a.C) + f[j] * N + nrow[g] + 4 * c) = o32;
          continue;
        }
        v4u16 o;
        with_out16(a.out_f16, [&](auto cvt) __attribute__((always_inline)) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float v = acc[g][j][i];
            if (a.mul_routed) v = v * w;
            o[i] = cvt(v);
          }
        });
        *reinterpret_cast<v4u16 *>(a.C + f[j] * N + nrow[g] + 4 * c) = o;
      }
    }
  } else {
    __shared__ float red[TM][NWAVES][16];
    float actf[TM][4];
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      float w = 1.0f;
      if (a.mul_routed && valid[j]) w = a.topk_w[f[j]];
      float amax = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float g = acc[0][j][i], u = acc[NW - 1][j][i];
        if (a.mul_routed) {
          g = g * w;
          u = u * w;
        }
        const uint16_t act16 = silu_mul_tab(a.silu, f32_to_bf16(g), f32_to_bf16(u));
        actf[j][i] = bf16_to_f32(act16);
        amax = fmaxf(amax, fabsf(actf[j][i]));
      }
      amax = fmaxf(amax, __shfl_xor(amax, 16));
      amax = fmaxf(amax, __shfl_xor(amax, 32));
      if (c == 0) red[j][wave][r] = amax;
    }
    __syncthreads();
    const int64_t G = I / kGroup;
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      if (!valid[j]) continue;
      float amax = 0.0f;
#pragma unroll
      for (int w2 = 0; w2 < NWAVES; ++w2) amax = fmaxf(amax, red[j][w2][r]);
      amax = fmaxf(amax, 1e-10f);
      const float sc = amax / 127.0f;
      const uint32_t packed = quant4(actf[j], sc, 1.0f / sc);
      *reinterpret_cast<uint32_t *>(a.A2q + f[j] * I + nrow[0] + 4 * c) = packed;
      if (wave == 0 && c == 0) a.A2s[f[j] * G + nt] = sc;
    }
  }
}

template <int TM, bool FUSED_ACT, int ORD>
static int launch_ws(const GemmArgs &a0, int64_t m_blocks, hipStream_t s) {
  constexpr int NWAVES = FUSED_ACT ? 8 : LO_WS_PLAIN_WAVES;
  // A plain-GEMM wave takes RPW consecutive 16-row fragments so that it streams a few
  // hundred KB even when K is short; the ring depth shrinks as the fragments multiply.
  constexpr int RPW = FUSED_ACT ? 2 : (TM <= 2 ? LO_WS_RPW : (TM == 4 ? 2 : 1));
  constexpr int PD = FUSED_ACT ? ((TM <= 2) ? LO_WS_PD_SMALL : (TM == 4 ? 2 : 1))
                               : ((TM <= 2) ? LO_WS_PD_PLAIN : (TM == 4 ? 2 : 1));
  GemmArgs a = a0;
  if (!FUSED_ACT) a.n_tiles = static_cast<int32_t>((a.N + 16 * NWAVES * RPW - 1) / (16 * NWAVES * RPW));
  const dim3 grid(static_cast<unsigned>(m_blocks * a.n_tiles)), block(NWAVES * 64);
  if constexpr (!FUSED_ACT && ORD == kOrdSeparate) {
    if (a.per_channel) {
      if (a.w4)
        hipLaunchKernelGGL((moe_gemm_ws_kernel<TM, false, kOrdSeparate, true, NWAVES, PD, RPW, true, true>), grid, block, 0, s, a);
      else if (a.w_shuffled)
        hipLaunchKernelGGL((moe_gemm_ws_kernel<TM, false, kOrdSeparate, true, NWAVES, PD, RPW, false, true>), grid, block, 0, s, a);
      else
        hipLaunchKernelGGL((moe_gemm_ws_kernel<TM, false, kOrdSeparate, false, NWAVES, PD, RPW, false, true>), grid, block, 0, s, a);
      return LO_OK;
    }
  }
  if (a.w4) {
    // the row scales of the workgroup's rows, every K block, sit in LDS
    constexpr int ROWS = FUSED_ACT ? 256 : 16 * NWAVES * RPW;
    const int64_t lds = a.K / kGroup * ROWS * 4;
    LO_REQUIRE(lds <= 128 * 1024, LO_ENOTSUP, "moe_gemm(int4): K = %lld is more than this kernel's %d K groups",
               static_cast<long long>(a.K), 128 * 1024 / (ROWS * 4));
    const auto kern = &moe_gemm_ws_kernel<TM, FUSED_ACT, ORD, true, NWAVES, PD, RPW, true>;
    if (lds > 48 * 1024) {
      static unsigned long long lds_done = 0; // per instantiation: one bit per device
      const int rc_lds = reserve_lds_once(reinterpret_cast<const void *>(kern), 128 * 1024, &lds_done);
      if (rc_lds) return rc_lds;
    }
    hipLaunchKernelGGL(kern, grid, block, static_cast<size_t>(lds), s, a);
  } else if (a.w_shuffled)
    hipLaunchKernelGGL((moe_gemm_ws_kernel<TM, FUSED_ACT, ORD, true, NWAVES, PD, RPW>), grid, block, 0, s, a);
  else
    hipLaunchKernelGGL((moe_gemm_ws_kernel<TM, FUSED_ACT, ORD, false, NWAVES, PD, RPW>), grid, block, 0, s, a);
  return LO_OK;
}

template <bool FUSED_ACT>
static int dispatch_ws(const GemmArgs &a, int bs, int flags, int64_t m_blocks, hipStream_t s) {
  // per-channel scales are applied once, in the epilogue: one instantiation (tagged kOrdSeparate)
  const int ord = a.per_channel ? kOrdSeparate : scale_order(flags);
  int rc = LO_OK;
#define LO_WS_CASE(TMV)                                               \
  case 16 * TMV:                                                      \
    rc = ord == kOrdContract   ? launch_ws<TMV, FUSED_ACT, kOrdContract>(a, m_blocks, s)     \
         : ord == kOrdSeparate ? launch_ws<TMV, FUSED_ACT, kOrdSeparate>(a, m_blocks, s)     \
                               : launch_ws<TMV, FUSED_ACT, kOrdFusedScale>(a, m_blocks, s);  \
    break;
  switch (bs) {
    LO_WS_CASE(1)
    LO_WS_CASE(2)
    LO_WS_CASE(4)
    LO_WS_CASE(8)
  default:
    set_error("moe_gemm: block_size_m %d is not one of 16, 32, 64, 128", bs);
    return LO_EINVAL;
  }
#undef LO_WS_CASE
  if (rc) return rc;
  return check_launch(FUSED_ACT ? "moe_gemm1_silu_quant" : "moe_gemm");
}

int launch_gemm_ws(const GemmArgs &a, bool fused_act, int block_size_m, int flags, int64_t m_blocks,
                   hipStream_t s) {
  return fused_act ? dispatch_ws<true>(a, block_size_m, flags, m_blocks, s)
                   : dispatch_ws<false>(a, block_size_m, flags, m_blocks, s);
}

} // namespace lo
