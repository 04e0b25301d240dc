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
#include "common.h"

namespace lo {

struct GemmArgs {
  const int8_t *A;       // [a_rows, K]
  const float *As;       // [a_rows, K/128]
  const int8_t *W;       // [E, N, K]
  const float *Ws;       // [E, NB, K/128]
  uint16_t *C;           // plain: [num_valid, N]
  int8_t *A2q;           // fused: [num_valid, I]
  float *A2s;            // fused: [num_valid, I/128]
  const float *topk_w;   // [num_valid]
  const int32_t *sorted; // [>= m_blocks*BM]
  const int32_t *expert_ids;
  const int32_t *ntpp;
  int64_t num_valid;
  int64_t N;             // weight rows per expert (2I for the fused first GEMM)
  int64_t K;
  int32_t top_k;
  int32_t n_tiles;       // workgroups along N
  int32_t E;             // experts held by W
  int32_t mul_routed;
};

__device__ __forceinline__ v4i ld16(const int8_t *p) { return *reinterpret_cast<const v4i *>(p); }

template <int TM, bool FUSED_ACT, bool FAST_SCALE, int NWAVES, int PD>
__global__ __launch_bounds__(NWAVES * 64) void moe_gemm_ws_kernel(const GemmArgs a) {
  constexpr int BM = 16 * TM;
  constexpr int NW = FUSED_ACT ? 2 : 1; // weight fragments per wave (gate, up)
  const int bid = blockIdx.x;
  const int mb = bid / a.n_tiles, nt = bid - mb * a.n_tiles;
  if (static_cast<int64_t>(mb) * BM >= a.ntpp[0]) return;
  const int e = a.expert_ids[mb];
  if (e >= a.E) return; // an expert_map entry outside the weight tensor: nothing to read
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int64_t K = a.K, N = a.N;
  const int KB = static_cast<int>(K / kGroup);

  // tokens of this block, one per (sub-tile, r)
  int64_t f[TM];
  bool valid[TM];
  const int8_t *arow[TM];
  const float *asrow[TM];
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    f[j] = a.sorted[static_cast<int64_t>(mb) * BM + j * 16 + r];
    valid[j] = f[j] < a.num_valid;
    const int64_t row = valid[j] ? f[j] / a.top_k : 0;
    arow[j] = a.A + row * K + c * 16;
    asrow[j] = a.As + row * KB;
  }

  if constexpr (!FUSED_ACT) {
    const int64_t n0 = static_cast<int64_t>(nt) * (16 * NWAVES) + wave * 16;
    if (n0 >= N) return;
    if (e < 0) { // expert not held by this rank: the rows are defined to be zero
#pragma unroll
      for (int j = 0; j < TM; ++j)
        if (valid[j]) *reinterpret_cast<v2i *>(a.C + f[j] * N + n0 + 4 * c) = v2i{0, 0};
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
    nrow[0] = static_cast<int64_t>(nt) * (16 * NWAVES) + wave * 16;
  }
  const int NB = static_cast<int>((N + kGroup - 1) / kGroup);
  const int8_t *wrow[NW];
  const float *wsrow[NW];
#pragma unroll
  for (int g = 0; g < NW; ++g) {
    wrow[g] = a.W + (static_cast<int64_t>(e) * N + nrow[g] + r) * K + c * 16;
    wsrow[g] = a.Ws + (static_cast<int64_t>(e) * NB + nrow[g] / kGroup) * KB;
  }

  v4f acc[NW][TM];
#pragma unroll
  for (int g = 0; g < NW; ++g)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[g][j] = v4f{0.f, 0.f, 0.f, 0.f};

  // register ring: PD K-blocks (128 bytes of K per row each) in flight
  v4i wbuf[PD][NW][2];
  v4i abuf[PD][TM][2];
  auto issue = [&](int slot, int kb) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int g = 0; g < NW; ++g) wbuf[slot][g][ks] = ld16(wrow[g] + kb * kGroup + ks * 64);
#pragma unroll
      for (int j = 0; j < TM; ++j) abuf[slot][j][ks] = ld16(arow[j] + kb * kGroup + ks * 64);
    }
  };
#pragma unroll
  for (int p = 0; p < PD; ++p)
    if (p < KB) issue(p, p);

  for (int kb0 = 0; kb0 < KB; kb0 += PD) {
#pragma unroll
    for (int p = 0; p < PD; ++p) {
      const int kb = kb0 + p;
      if (kb < KB) {
        v4i d[NW][TM];
#pragma unroll
        for (int g = 0; g < NW; ++g)
#pragma unroll
          for (int j = 0; j < TM; ++j) {
            d[g][j] = v4i{0, 0, 0, 0};
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
              d[g][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wbuf[p][g][ks], abuf[p][j][ks],
                                                              d[g][j], 0, 0, 0);
          }
        if (kb + PD < KB) issue(p, kb + PD);
        float bs[NW];
#pragma unroll
        for (int g = 0; g < NW; ++g) bs[g] = wsrow[g][kb];
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          const float as = asrow[j][kb];
#pragma unroll
          for (int g = 0; g < NW; ++g) {
            if constexpr (FAST_SCALE) {
              const float s = as * bs[g];
#pragma unroll
              for (int i = 0; i < 4; ++i)
                acc[g][j][i] = __builtin_fmaf(static_cast<float>(d[g][j][i]), s, acc[g][j][i]);
            } else {
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                float t = static_cast<float>(d[g][j][i]) * as;
                t = t * bs[g];
                acc[g][j][i] = acc[g][j][i] + t;
              }
            }
          }
        }
      }
    }
  }

  if constexpr (!FUSED_ACT) {
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      if (!valid[j]) continue;
      float w = 1.0f;
      if (a.mul_routed) w = a.topk_w[f[j]];
      v4u16 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = acc[0][j][i];
        if (a.mul_routed) v = v * w;
        o[i] = f32_to_bf16(v);
      }
      *reinterpret_cast<v4u16 *>(a.C + f[j] * N + nrow[0] + 4 * c) = o;
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
        const uint16_t act16 = silu_mul<LO_BF16>(f32_to_bf16(g), f32_to_bf16(u));
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
      const uint32_t packed = pack4_i8(quant_one(actf[j][0], sc), quant_one(actf[j][1], sc),
                                       quant_one(actf[j][2], sc), quant_one(actf[j][3], sc));
      *reinterpret_cast<uint32_t *>(a.A2q + f[j] * I + nrow[0] + 4 * c) = packed;
      if (wave == 0 && c == 0) a.A2s[f[j] * G + nt] = sc;
    }
  }
}

template <int TM, bool FUSED_ACT, bool FAST_SCALE>
static void launch_ws(const GemmArgs &a, int64_t m_blocks, hipStream_t s) {
  constexpr int NWAVES = FUSED_ACT ? 8 : 4;
  constexpr int PD = (TM <= 2) ? 4 : (TM == 4 ? 2 : 1);
  const int64_t grid = m_blocks * a.n_tiles;
  hipLaunchKernelGGL((moe_gemm_ws_kernel<TM, FUSED_ACT, FAST_SCALE, NWAVES, PD>),
                     dim3(static_cast<unsigned>(grid)), dim3(NWAVES * 64), 0, s, a);
}

template <bool FUSED_ACT>
static int dispatch_ws(const GemmArgs &a, int bs, int flags, int64_t m_blocks, hipStream_t s) {
  const bool fast = (flags & LO_GEMM_FUSED_SCALE) != 0;
#define LO_WS_CASE(TMV)                                               \
  case 16 * TMV:                                                      \
    if (fast) launch_ws<TMV, FUSED_ACT, true>(a, m_blocks, s);        \
    else launch_ws<TMV, FUSED_ACT, false>(a, m_blocks, s);            \
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
  return check_launch(FUSED_ACT ? "moe_gemm1_silu_quant" : "moe_gemm");
}

static int64_t grid_m_blocks(int64_t sorted_cap, int64_t num_valid, int bs) {
  // The sorted list can hold at most one partially filled block per slot, so when
  // there are fewer slots than blocks the tail can never be reached (the bound of
  // invoke_fused_moe_kernel_int8, int8.py:572-580).
  int64_t blocks = sorted_cap / bs;
  if (num_valid < blocks) blocks = num_valid;
  return blocks;
}

static int validate_common(const char *who, const void *A, const void *As, const void *W,
                           const void *Ws, const void *sorted, const void *eids, const void *ntpp,
                           int64_t K, int32_t top_k, int32_t E, int64_t a_rows) {
  LO_REQUIRE(A && As && W && Ws && sorted && eids && ntpp, LO_EINVAL, "%s: null pointer", who);
  LO_REQUIRE(K > 0 && K % kGroup == 0, LO_EINVAL, "%s: K (%lld) must be a multiple of 128", who,
             (long long)K);
  LO_REQUIRE(top_k >= 1 && E >= 1 && a_rows >= 1, LO_EINVAL, "%s: bad top_k / E / a_rows", who);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(A) & 15) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0,
             LO_EINVAL, "%s: A and W must be 16-byte aligned", who);
  return LO_OK;
}

} // namespace lo

extern "C" int lo_moe_gemm_block_int8(const int8_t *A, const float *As, const int8_t *W,
                                      const float *Ws, void *C, int c_dtype, const float *topk_w,
                                      const int32_t *sorted_ids, const int32_t *expert_ids,
                                      const int32_t *num_tokens_post_pad, int64_t sorted_cap,
                                      int64_t num_valid, int64_t a_rows, int32_t E, int64_t N,
                                      int64_t K, int32_t top_k, int32_t block_size_m,
                                      int mul_routed, int flags, lo_stream_t stream) {
  using namespace lo;
  int rc = validate_common("moe_gemm", A, As, W, Ws, sorted_ids, expert_ids, num_tokens_post_pad, K,
                           top_k, E, a_rows);
  if (rc) return rc;
  LO_REQUIRE(C, LO_EINVAL, "moe_gemm: null output");
  LO_REQUIRE(c_dtype == LO_BF16, LO_ENOTSUP, "moe_gemm: only bf16 output is built");
  LO_REQUIRE(N > 0 && N % 16 == 0, LO_EINVAL, "moe_gemm: N (%lld) must be a multiple of 16", (long long)N);
  LO_REQUIRE(!mul_routed || topk_w, LO_EINVAL, "moe_gemm: mul_routed needs topk_weights");
  LO_REQUIRE((reinterpret_cast<uintptr_t>(C) & 7) == 0, LO_EINVAL, "moe_gemm: C must be 8-byte aligned");
  LO_REQUIRE((num_valid + top_k - 1) / top_k <= a_rows, LO_EINVAL,
             "moe_gemm: %lld slots / top_k %d exceed the %lld rows of A", (long long)num_valid, top_k,
             (long long)a_rows);
  if (num_valid == 0) return LO_OK;
  GemmArgs a{};
  a.A = A; a.As = As; a.W = W; a.Ws = Ws; a.C = static_cast<uint16_t *>(C);
  a.topk_w = topk_w; a.sorted = sorted_ids; a.expert_ids = expert_ids; a.ntpp = num_tokens_post_pad;
  a.E = E; a.num_valid = num_valid; a.N = N; a.K = K; a.top_k = top_k; a.mul_routed = mul_routed ? 1 : 0;
  a.n_tiles = static_cast<int32_t>((N + 63) / 64);
  const int64_t mblocks = grid_m_blocks(sorted_cap, num_valid, block_size_m);
  LO_REQUIRE(mblocks * a.n_tiles < (1ll << 31), LO_EINVAL, "moe_gemm: grid too large");
  if (mblocks == 0) return LO_OK;
  return dispatch_ws<false>(a, block_size_m, flags, mblocks, static_cast<hipStream_t>(stream));
}

extern "C" int lo_moe_gemm1_silu_quant_block_int8(
    const int8_t *A, const float *As, const int8_t *W, const float *Ws, int8_t *A2q, float *A2s,
    int c_dtype, const float *topk_w, const int32_t *sorted_ids, const int32_t *expert_ids,
    const int32_t *num_tokens_post_pad, int64_t sorted_cap, int64_t num_valid, int64_t a_rows,
    int32_t E, int64_t I, int64_t K, int32_t top_k, int32_t block_size_m, int mul_routed, int flags,
    lo_stream_t stream) {
  using namespace lo;
  int rc = validate_common("moe_gemm1_silu_quant", A, As, W, Ws, sorted_ids, expert_ids,
                           num_tokens_post_pad, K, top_k, E, a_rows);
  if (rc) return rc;
  LO_REQUIRE(A2q && A2s, LO_EINVAL, "moe_gemm1_silu_quant: null output");
  LO_REQUIRE(c_dtype == LO_BF16, LO_ENOTSUP, "moe_gemm1_silu_quant: only bf16 rounding is built");
  LO_REQUIRE(I > 0 && I % kGroup == 0, LO_EINVAL,
             "moe_gemm1_silu_quant: intermediate size (%lld) must be a multiple of 128", (long long)I);
  LO_REQUIRE(!mul_routed || topk_w, LO_EINVAL, "moe_gemm1_silu_quant: mul_routed needs topk_weights");
  LO_REQUIRE((reinterpret_cast<uintptr_t>(A2q) & 3) == 0, LO_EINVAL,
             "moe_gemm1_silu_quant: A2q must be 4-byte aligned");
  LO_REQUIRE((num_valid + top_k - 1) / top_k <= a_rows, LO_EINVAL,
             "moe_gemm1_silu_quant: %lld slots / top_k %d exceed the %lld rows of A",
             (long long)num_valid, top_k, (long long)a_rows);
  if (num_valid == 0) return LO_OK;
  GemmArgs a{};
  a.A = A; a.As = As; a.W = W; a.Ws = Ws; a.A2q = A2q; a.A2s = A2s;
  a.topk_w = topk_w; a.sorted = sorted_ids; a.expert_ids = expert_ids; a.ntpp = num_tokens_post_pad;
  a.E = E; a.num_valid = num_valid; a.N = 2 * I; a.K = K; a.top_k = top_k; a.mul_routed = mul_routed ? 1 : 0;
  a.n_tiles = static_cast<int32_t>(I / kGroup);
  const int64_t mblocks = grid_m_blocks(sorted_cap, num_valid, block_size_m);
  LO_REQUIRE(mblocks * a.n_tiles < (1ll << 31), LO_EINVAL, "moe_gemm1_silu_quant: grid too large");
  if (mblocks == 0) return LO_OK;
  return dispatch_ws<true>(a, block_size_m, flags, mblocks, static_cast<hipStream_t>(stream));
}
