// Routers upstream of the fused-MoE path: softmax top-k and grouped sigmoid top-k with a
// correction bias.  One wavefront per token row: lane l holds experts l, l+64, l+128, ...
// in registers, the k winners are found by k rounds of (local best, 64-lane arg-max), and
// lane j keeps winner j, so the outputs of a row leave as one coalesced store.
//
// Reference: csrc/kernels/softmax/topk_softmax_kernels.cu:1381-1582 (topk_softmax) and
// csrc/kernels/moe_gate/moe_fused_gate.cu:76-312 (moe_fused_gate).  Where the reference
// leaves the result open (which of several equal scores wins, the order of the fp32 sums)
// the choice is fixed: the lower index wins, the selected weights are summed in selection
// order, the full-row softmax sum is per-lane sequential followed by a butterfly.
#include "common.h"

namespace lo {

constexpr float kNeg = -3.402823466e+38f; // the reference's "minus infinity" (-FLT_MAX)

template <int DT> __device__ __forceinline__ float load_as_f32(const void *p, int64_t i) {
  if constexpr (DT == LO_F32) return static_cast<const float *>(p)[i];
  else return to_f32<DT>(static_cast<const uint16_t *>(p)[i]);
}

// Lane exchange inside a row of 16 lanes by DPP (no LDS round trip): partner = lane ^ 1,
// lane ^ 2, then the mirror images inside 8 and inside 16 lanes.  At the step where a mirror
// is used all lanes of the smaller unit already hold the same value, so it acts like
// lane ^ 4 and lane ^ 8.
template <int CTRL> __device__ __forceinline__ int dpp_i(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, dpp_i<CTRL>(__builtin_bit_cast(int, v)));
}
constexpr int kXor1 = 0xB1, kXor2 = 0x4E, kMirror8 = 0x141, kMirror16 = 0x140;
__device__ __forceinline__ float lane_f(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// (value, index) of the best lane; ties go to the lower index, so every lane agrees
template <int CTRL> __device__ __forceinline__ void argmax_step(float &v, int &idx) {
  const float ov = dpp_f<CTRL>(v);
  const int oi = dpp_i<CTRL>(idx);
  const bool take = ov > v || (ov == v && oi < idx);
  v = take ? ov : v;
  idx = take ? oi : idx;
}
__device__ __forceinline__ void wave_argmax(float &v, int &idx) {
  argmax_step<kXor1>(v, idx);
  argmax_step<kXor2>(v, idx);
  argmax_step<kMirror8>(v, idx);
  argmax_step<kMirror16>(v, idx);
  // the four rows, through scalar registers
  float bv = lane_f(v, 0);
  int bi = __builtin_amdgcn_readlane(idx, 0);
#pragma unroll
  for (int r = 1; r < 4; ++r) {
    const float ov = lane_f(v, 16 * r);
    const int oi = __builtin_amdgcn_readlane(idx, 16 * r);
    const bool take = ov > bv || (ov == bv && oi < bi);
    bv = take ? ov : bv;
    bi = take ? oi : bi;
  }
  v = bv;
  idx = bi;
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f<kXor1>(v));
  v = fmaxf(v, dpp_f<kXor2>(v));
  v = fmaxf(v, dpp_f<kMirror8>(v));
  v = fmaxf(v, dpp_f<kMirror16>(v));
  return fmaxf(fmaxf(lane_f(v, 0), lane_f(v, 16)), fmaxf(lane_f(v, 32), lane_f(v, 48)));
}
// s[l] = s[l] + s[l ^ m] for m = 1, 2, 4, 8, 16, 32: the same bits in every lane
__device__ __forceinline__ float wave_sum_tree(float v) {
  v = v + dpp_f<kXor1>(v);
  v = v + dpp_f<kXor2>(v);
  v = v + dpp_f<kMirror8>(v);
  v = v + dpp_f<kMirror16>(v);
  return (lane_f(v, 0) + lane_f(v, 16)) + (lane_f(v, 32) + lane_f(v, 48));
}

// One round: the best remaining entry of the row (value, expert); the winner erases it.
template <int VPT> __device__ __forceinline__ void pick_best(float (&v)[VPT], int lane, float &best, int &bidx) {
  best = kNeg;
  bidx = lane; // an index this lane owns, so an all-erased row still yields distinct lanes
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    if (v[j] > best) {
      best = v[j];
      bidx = lane + 64 * j;
    }
  wave_argmax(best, bidx);
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    if (bidx == lane + 64 * j) v[j] = kNeg;
}

template <int VPT, int DT, typename IdxT>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const void *__restrict__ gating, int64_t T, int E, int k,
                                                           int renormalize, float *__restrict__ weights,
                                                           IdxT *__restrict__ indices, int32_t *__restrict__ source_rows) {
  const int lane = threadIdx.x & 63;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  float x[VPT], v[VPT];
  float mx = kNeg;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int e = lane + 64 * j;
    x[j] = e < E ? load_as_f32<DT>(gating, t * E + e) : kNeg;
    mx = fmaxf(mx, x[j]);
  }
  mx = wave_max(mx);
  float scale = 0.0f;
  if (renormalize) {
#pragma unroll
    for (int j = 0; j < VPT; ++j) v[j] = x[j];
  } else {
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const bool in = lane + 64 * j < E;
      const float p = in ? det_expf(x[j] - mx) : 0.0f;
      v[j] = in ? p : kNeg;
      s = s + p;
    }
    scale = 1.0f / (wave_sum_tree(s) + 1e-6f);
  }
  float sum = 0.0f, mine = 0.0f;
  int mine_idx = 0;
  for (int j = 0; j < k; ++j) { // k <= 64 (host check): lane j keeps winner j
    float best;
    int bidx;
    pick_best<VPT>(v, lane, best, bidx);
    const float val = renormalize ? det_expf(best - mx) : best;
    sum = sum + val;
    if (lane == j) {
      mine = val;
      mine_idx = bidx;
    }
  }
  if (renormalize) scale = 1.0f / (sum + 1e-6f);
  if (lane < k) {
    weights[t * k + lane] = mine * scale;
    indices[t * k + lane] = static_cast<IdxT>(mine_idx);
    if (source_rows) source_rows[t * k + lane] = static_cast<int32_t>(lane * T + t);
  }
}

template <int VPT, int DT, int BT, typename IdxT>
__global__ __launch_bounds__(256) void moe_fused_gate_kernel(const void *__restrict__ input, const void *__restrict__ bias,
                                                             int64_t T, int E, int G, int topk_group, int topk,
                                                             int n_share, float rsf, float route_scale,
                                                             float *__restrict__ weights, IdxT *__restrict__ indices) {
  __shared__ float sC[4][64 * VPT];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * 4 + wv;
  if (t >= T) return;
  const int gs = E / G, kr = topk - n_share;
  float s[VPT], c[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int e = lane + 64 * j;
    if (e < E) {
      const float xv = load_as_f32<DT>(input, t * E + e);
      s[j] = 1.0f / (1.0f + det_expf(-xv));
      c[j] = load_as_f32<BT>(bias, e) + s[j];
      sC[wv][e] = c[j];
    } else {
      s[j] = 0.0f;
      c[j] = kNeg;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  uint64_t keep = ~0ull;
  if (G > 1) {
    // lpg lanes (a power of two, at most one DPP row) share a group: each scans every lpg-th
    // score of it, then the two largest are merged across the lpg lanes (values only, so the
    // order of the merges does not matter)
    int lpg = 16;
    while (lpg * G > 64) lpg >>= 1;
    const int g = lane / lpg, sub = lane % lpg;
    float t1 = kNeg, t2 = kNeg;
    if (g < G)
      for (int i = g * gs + sub; i < (g + 1) * gs; i += lpg) {
        const float cv = sC[wv][i];
        if (cv > t1) {
          t2 = t1;
          t1 = cv;
        } else if (cv > t2) {
          t2 = cv;
        }
      }
#define LO_TOP2_MERGE(CTRL)                                  \
  do {                                                       \
    const float o1 = dpp_f<CTRL>(t1), o2 = dpp_f<CTRL>(t2);  \
    const float n1 = fmaxf(t1, o1);                          \
    t2 = fmaxf(fminf(t1, o1), fmaxf(t2, o2));                \
    t1 = n1;                                                 \
  } while (0)
    if (lpg > 1) LO_TOP2_MERGE(kXor1);
    if (lpg > 2) LO_TOP2_MERGE(kXor2);
    if (lpg > 4) LO_TOP2_MERGE(kMirror8);
    if (lpg > 8) LO_TOP2_MERGE(kMirror16);
#undef LO_TOP2_MERGE
    float gscore = (g < G && sub == 0) ? t1 + t2 : kNeg;
    keep = 0;
    for (int r = 0; r < topk_group; ++r) {
      float bv = gscore;
      int bi = g;
      wave_argmax(bv, bi);
      keep |= 1ull << bi;
      if (g == bi) gscore = kNeg;
    }
  }
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int e = lane + 64 * j;
    if (e < E && !((keep >> (e / gs)) & 1)) c[j] = kNeg;
  }
  float sum = 0.0f, mine = 0.0f;
  int mine_idx = 0;
  for (int j = 0; j < kr; ++j) {
    float best;
    int bidx;
    pick_best<VPT>(c, lane, best, bidx);
    // the winner's sigmoid (without the bias), from the lane and register that hold it
    float sv = 0.0f;
#pragma unroll
    for (int q = 0; q < VPT; ++q)
      if (bidx == lane + 64 * q) sv = s[q];
    sv = lane_f(sv, __builtin_amdgcn_readfirstlane(bidx) & 63);
    sum = sum + sv;
    if (lane == j) {
      mine = sv;
      mine_idx = bidx;
    }
  }
  if (lane >= kr && lane < topk) {
    mine = sum / (rsf > 0.0f ? rsf : 1.0f);
    mine_idx = E + (lane - kr);
  }
  if (lane < topk) {
    weights[t * topk + lane] = (mine / sum) * route_scale;
    indices[t * topk + lane] = static_cast<IdxT>(mine_idx);
  }
}

// ---- sixteen lanes per token row ------------------------------------------------------------------
// With thousands of rows the kernels above are bound by instruction issue: a wavefront spends the
// same few hundred instructions on one row whether the row fills its lanes or not.  Up to 256
// experts a row fits 16 lanes (one DPP row: the arg-max needs no scalar step across rows), so a
// wavefront serves four token rows at once.  Lane l of a row holds experts l, l + 16, ...; every
// result is bit for bit the one of the 64-lane kernels (the full-row softmax sum keeps their order:
// four partial sums per lane, one per 64-lane row that the expert would have sat in).
__device__ __forceinline__ void row_argmax(float &v, int &idx) {
  argmax_step<kXor1>(v, idx);
  argmax_step<kXor2>(v, idx);
  argmax_step<kMirror8>(v, idx);
  argmax_step<kMirror16>(v, idx);
}
__device__ __forceinline__ float row_max(float v) {
  v = fmaxf(v, dpp_f<kXor1>(v));
  v = fmaxf(v, dpp_f<kXor2>(v));
  v = fmaxf(v, dpp_f<kMirror8>(v));
  return fmaxf(v, dpp_f<kMirror16>(v));
}
__device__ __forceinline__ float row_sum_tree(float v) {
  v = v + dpp_f<kXor1>(v);
  v = v + dpp_f<kXor2>(v);
  v = v + dpp_f<kMirror8>(v);
  return v + dpp_f<kMirror16>(v);
}
template <int VPT> __device__ __forceinline__ void pick_best16(float (&v)[VPT], int sub, float &best, int &bidx) {
  best = kNeg;
  bidx = sub;
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    if (v[j] > best) {
      best = v[j];
      bidx = sub + 16 * j;
    }
  row_argmax(best, bidx);
#pragma unroll
  for (int j = 0; j < VPT; ++j)
    if (bidx == sub + 16 * j) v[j] = kNeg;
}

template <int VPT, int DT, typename IdxT>
__global__ __launch_bounds__(256) void topk_softmax16_kernel(const void *__restrict__ gating, int64_t T, int E, int k,
                                                             int renormalize, float *__restrict__ weights,
                                                             IdxT *__restrict__ indices, int32_t *__restrict__ source_rows) {
  const int sub = threadIdx.x & 15;
  const int64_t t_raw = static_cast<int64_t>(blockIdx.x) * 16 + (threadIdx.x >> 4);
  const bool active = t_raw < T;
  const int64_t t = active ? t_raw : T - 1; // rows past the end compute the last row again and store nothing
  float x[VPT], v[VPT];
  float mx = kNeg;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int e = sub + 16 * j;
    x[j] = e < E ? load_as_f32<DT>(gating, t * E + e) : kNeg;
    mx = fmaxf(mx, x[j]);
  }
  mx = row_max(mx);
  float scale = 0.0f;
  if (renormalize) {
#pragma unroll
    for (int j = 0; j < VPT; ++j) v[j] = x[j];
  } else {
    float s4[4] = {0.0f, 0.0f, 0.0f, 0.0f}; // expert e sat in 64-lane row (e / 16) % 4
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const bool in = sub + 16 * j < E;
      const float p = in ? det_expf(x[j] - mx) : 0.0f;
      v[j] = in ? p : kNeg;
      s4[j & 3] = s4[j & 3] + p;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) s4[r] = row_sum_tree(s4[r]);
    scale = 1.0f / (((s4[0] + s4[1]) + (s4[2] + s4[3])) + 1e-6f);
  }
  float mine = 0.0f;
  int mine_idx = 0;
  for (int j = 0; j < k; ++j) { // k <= 16 (host check): lane j of the row keeps winner j
    float best;
    int bidx;
    pick_best16<VPT>(v, sub, best, bidx);
    if (sub == j) {
      mine = best;
      mine_idx = bidx;
    }
  }
  // one exponential per winner, in the lane that keeps it; then the sum in selection order
  if (renormalize) mine = det_expf(mine - mx);
  float sum = 0.0f;
  const int row_base = threadIdx.x & 48;
  for (int j = 0; j < k; ++j) sum = sum + __shfl(mine, row_base | j);
  if (renormalize) scale = 1.0f / (sum + 1e-6f);
  if (active && sub < k) {
    weights[t * k + sub] = mine * scale;
    indices[t * k + sub] = static_cast<IdxT>(mine_idx);
    if (source_rows) source_rows[t * k + sub] = static_cast<int32_t>(sub * T + t);
  }
}

template <int VPT, int DT, int BT, typename IdxT>
__global__ __launch_bounds__(256) void moe_fused_gate16_kernel(const void *__restrict__ input, const void *__restrict__ bias,
                                                               int64_t T, int E, int G, int topk_group, int topk,
                                                               int n_share, float rsf, float route_scale,
                                                               float *__restrict__ weights, IdxT *__restrict__ indices) {
  __shared__ float sC[16][16 * VPT]; // biased scores of the row, for the group ranking
  __shared__ float sS[16][16 * VPT]; // its sigmoids, for the winners
  const int lane = threadIdx.x & 63, sub = threadIdx.x & 15, row = threadIdx.x >> 4;
  const int64_t t_raw = static_cast<int64_t>(blockIdx.x) * 16 + row;
  const bool active = t_raw < T;
  const int64_t t = active ? t_raw : T - 1;
  const int gs = E / G, kr = topk - n_share;
  float s[VPT], c[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int e = sub + 16 * j;
    if (e < E) {
      const float xv = load_as_f32<DT>(input, t * E + e);
      s[j] = 1.0f / (1.0f + det_expf(-xv));
      c[j] = load_as_f32<BT>(bias, e) + s[j];
      if (G > 1) sC[row][e] = c[j];
      sS[row][e] = s[j];
    } else {
      s[j] = 0.0f;
      c[j] = kNeg;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  uint32_t keep = ~0u;
  if (G > 1) { // G <= 16 (host check)
    int lpg = 16;
    while (lpg * G > 16) lpg >>= 1;
    const int g = sub / lpg, lsub = sub % lpg;
    float t1 = kNeg, t2 = kNeg;
    if (g < G)
      for (int i = g * gs + lsub; i < (g + 1) * gs; i += lpg) {
        const float cv = sC[row][i];
        if (cv > t1) {
          t2 = t1;
          t1 = cv;
        } else if (cv > t2) {
          t2 = cv;
        }
      }
#define LO_TOP2_MERGE(CTRL)                                  \
  do {                                                       \
    const float o1 = dpp_f<CTRL>(t1), o2 = dpp_f<CTRL>(t2);  \
    const float n1 = fmaxf(t1, o1);                          \
    t2 = fmaxf(fminf(t1, o1), fmaxf(t2, o2));                \
    t1 = n1;                                                 \
  } while (0)
    if (lpg > 1) LO_TOP2_MERGE(kXor1);
    if (lpg > 2) LO_TOP2_MERGE(kXor2);
    if (lpg > 4) LO_TOP2_MERGE(kMirror8);
    if (lpg > 8) LO_TOP2_MERGE(kMirror16);
#undef LO_TOP2_MERGE
    float gscore = (g < G && lsub == 0) ? t1 + t2 : kNeg;
    keep = 0;
    for (int r = 0; r < topk_group; ++r) {
      float bv = gscore;
      int bi = g;
      row_argmax(bv, bi);
      keep |= 1u << bi;
      if (g == bi) gscore = kNeg;
    }
  }
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int e = sub + 16 * j;
    if (e < E && !((keep >> (e / gs)) & 1)) c[j] = kNeg;
  }
  float mine = 0.0f;
  int mine_idx = 0;
  for (int j = 0; j < kr; ++j) {
    float best;
    int bidx;
    pick_best16<VPT>(c, sub, best, bidx);
    if (sub == j) mine_idx = bidx;
  }
  // the winners' sigmoids (without the bias), then their sum in selection order
  if (sub < kr) mine = sS[row][mine_idx];
  float sum = 0.0f;
  for (int j = 0; j < kr; ++j) sum = sum + __shfl(mine, (lane & 48) | j);
  if (sub >= kr && sub < topk) {
    mine = sum / (rsf > 0.0f ? rsf : 1.0f);
    mine_idx = E + (sub - kr);
  }
  if (active && sub < topk) {
    weights[t * topk + sub] = (mine / sum) * route_scale;
    indices[t * topk + sub] = static_cast<IdxT>(mine_idx);
  }
}

// Rows from which the 16-lane kernels are used: below, a row per wavefront finishes sooner (a
// quarter of the per-lane work) and there are compute units to spare.
constexpr int64_t kRows16From = 65;

template <int VPT, int DT> static void launch_topk_softmax(const void *g, int64_t T, int E, int k, int renorm,
                                                           float *w, void *idx, int idx_dtype, int32_t *src,
                                                           hipStream_t s) {
  if constexpr (VPT <= 4) { // up to 256 experts
    if (T >= kRows16From && k <= 16) {
      const dim3 grid16(static_cast<unsigned>((T + 15) / 16)), block16(256);
      if (idx_dtype == LO_I64)
        hipLaunchKernelGGL((topk_softmax16_kernel<4 * VPT, DT, int64_t>), grid16, block16, 0, s, g, T, E, k, renorm, w,
                           static_cast<int64_t *>(idx), src);
      else
        hipLaunchKernelGGL((topk_softmax16_kernel<4 * VPT, DT, int32_t>), grid16, block16, 0, s, g, T, E, k, renorm, w,
                           static_cast<int32_t *>(idx), src);
      return;
    }
  }
  const dim3 grid(static_cast<unsigned>((T + 3) / 4)), block(256);
  if (idx_dtype == LO_I64)
    hipLaunchKernelGGL((topk_softmax_kernel<VPT, DT, int64_t>), grid, block, 0, s, g, T, E, k, renorm, w,
                       static_cast<int64_t *>(idx), src);
  else
    hipLaunchKernelGGL((topk_softmax_kernel<VPT, DT, int32_t>), grid, block, 0, s, g, T, E, k, renorm, w,
                       static_cast<int32_t *>(idx), src);
}

template <int VPT, int DT, int BT>
static void launch_gate(const void *x, const void *b, int64_t T, int E, int G, int tg, int topk, int ns, float rsf,
                        float scale, float *w, void *idx, int idx_dtype, hipStream_t s) {
  if constexpr (VPT <= 4) { // up to 256 experts
    // (256 experts: 16 scores per lane make every selection round longer than the 64-lane kernel's)
    if (T >= kRows16From && topk <= 16 && G <= 16 && VPT <= 2) {
      const dim3 grid16(static_cast<unsigned>((T + 15) / 16)), block16(256);
      if (idx_dtype == LO_I64)
        hipLaunchKernelGGL((moe_fused_gate16_kernel<4 * VPT, DT, BT, int64_t>), grid16, block16, 0, s, x, b, T, E, G, tg,
                           topk, ns, rsf, scale, w, static_cast<int64_t *>(idx));
      else
        hipLaunchKernelGGL((moe_fused_gate16_kernel<4 * VPT, DT, BT, int32_t>), grid16, block16, 0, s, x, b, T, E, G, tg,
                           topk, ns, rsf, scale, w, static_cast<int32_t *>(idx));
      return;
    }
  }
  const dim3 grid(static_cast<unsigned>((T + 3) / 4)), block(256);
  if (idx_dtype == LO_I64)
    hipLaunchKernelGGL((moe_fused_gate_kernel<VPT, DT, BT, int64_t>), grid, block, 0, s, x, b, T, E, G, tg, topk, ns,
                       rsf, scale, w, static_cast<int64_t *>(idx));
  else
    hipLaunchKernelGGL((moe_fused_gate_kernel<VPT, DT, BT, int32_t>), grid, block, 0, s, x, b, T, E, G, tg, topk, ns,
                       rsf, scale, w, static_cast<int32_t *>(idx));
}

static bool float_dtype_ok(int dt) { return dt == LO_BF16 || dt == LO_F16 || dt == LO_F32; }

} // namespace lo

#define LO_BY_VPT(E, CALL)           \
  do {                               \
    if ((E) <= 64) { CALL(1); }      \
    else if ((E) <= 128) { CALL(2); } \
    else if ((E) <= 256) { CALL(4); } \
    else if ((E) <= 512) { CALL(8); } \
    else { CALL(16); }               \
  } while (0)

extern "C" int lo_topk_softmax(const void *gating, int dtype, int64_t num_tokens, int32_t num_experts, int32_t topk,
                               int renormalize, float *topk_weights, void *topk_indices, int idx_dtype,
                               int32_t *token_expert_indices, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(gating && topk_weights && topk_indices, LO_EINVAL, "topk_softmax: null pointer");
  LO_REQUIRE(float_dtype_ok(dtype), LO_ENOTSUP, "topk_softmax: gating must be fp32, fp16 or bf16");
  LO_REQUIRE(idx_dtype == LO_I32 || idx_dtype == LO_I64, LO_EINVAL, "topk_softmax: indices must be int32 or int64");
  LO_REQUIRE(num_tokens >= 0 && num_experts >= 1 && num_experts <= 1024, LO_EINVAL,
             "topk_softmax: num_experts (%d) must be in 1..1024", num_experts);
  LO_REQUIRE(topk >= 1 && topk <= num_experts && topk <= 64, LO_EINVAL,
             "topk_softmax: topk (%d) must be in 1..min(num_experts, 64)", topk);
  LO_REQUIRE(!token_expert_indices || num_tokens * topk < (1ll << 31), LO_EINVAL,
             "topk_softmax: token_expert_indices would overflow int32");
  if (num_tokens == 0) return LO_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define LO_TS(V)                                                                                              \
  do {                                                                                                        \
    if (dtype == LO_F32) launch_topk_softmax<V, LO_F32>(gating, num_tokens, num_experts, topk, renormalize,   \
                                                        topk_weights, topk_indices, idx_dtype, token_expert_indices, s); \
    else if (dtype == LO_F16) launch_topk_softmax<V, LO_F16>(gating, num_tokens, num_experts, topk, renormalize, \
                                                        topk_weights, topk_indices, idx_dtype, token_expert_indices, s); \
    else launch_topk_softmax<V, LO_BF16>(gating, num_tokens, num_experts, topk, renormalize, topk_weights,    \
                                         topk_indices, idx_dtype, token_expert_indices, s);                   \
  } while (0)
  LO_BY_VPT(num_experts, LO_TS);
#undef LO_TS
  return check_launch("topk_softmax");
}

extern "C" int lo_moe_fused_gate(const void *input, int dtype, const void *bias, int bias_dtype, int64_t num_tokens,
                                 int32_t num_experts, int32_t num_expert_group, int32_t topk_group, int32_t topk,
                                 int32_t n_share_experts_fusion, double routed_scaling_factor,
                                 int apply_routed_scaling_factor_on_output, float *topk_weights, void *topk_indices,
                                 int idx_dtype, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(input && bias && topk_weights && topk_indices, LO_EINVAL, "moe_fused_gate: null pointer");
  LO_REQUIRE(float_dtype_ok(dtype) && float_dtype_ok(bias_dtype), LO_ENOTSUP,
             "moe_fused_gate: input and bias must be fp32, fp16 or bf16");
  LO_REQUIRE(idx_dtype == LO_I32 || idx_dtype == LO_I64, LO_EINVAL, "moe_fused_gate: indices must be int32 or int64");
  LO_REQUIRE(num_tokens >= 0 && num_experts >= 1 && num_experts <= 1024, LO_EINVAL,
             "moe_fused_gate: num_experts (%d) must be in 1..1024", num_experts);
  LO_REQUIRE(num_expert_group >= 1 && num_expert_group <= 64 && num_experts % num_expert_group == 0, LO_EINVAL,
             "moe_fused_gate: num_expert_group (%d) must divide num_experts (%d) and be at most 64",
             num_expert_group, num_experts);
  LO_REQUIRE(topk_group >= 1 && topk_group <= num_expert_group, LO_EINVAL,
             "moe_fused_gate: topk_group (%d) must be in 1..num_expert_group", topk_group);
  const int kr = topk - n_share_experts_fusion;
  LO_REQUIRE(n_share_experts_fusion >= 0 && kr >= 1 && topk <= 64, LO_EINVAL,
             "moe_fused_gate: topk (%d) must exceed the shared experts (%d) and be at most 64", topk,
             n_share_experts_fusion);
  LO_REQUIRE(kr <= topk_group * (num_experts / num_expert_group), LO_EINVAL,
             "moe_fused_gate: %d routed experts cannot come from %d groups of %d", kr, topk_group,
             num_experts / num_expert_group);
  LO_REQUIRE(routed_scaling_factor == routed_scaling_factor && routed_scaling_factor - routed_scaling_factor == 0.0,
             LO_EINVAL, "moe_fused_gate: routed_scaling_factor must be finite");
  if (num_tokens == 0) return LO_OK;
  const float rsf = static_cast<float>(routed_scaling_factor);
  const float scale = (apply_routed_scaling_factor_on_output && routed_scaling_factor > 0.0) ? rsf : 1.0f;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define LO_G2(V, DT)                                                                                             \
  do {                                                                                                           \
    if (bias_dtype == LO_F32) launch_gate<V, DT, LO_F32>(input, bias, num_tokens, num_experts, num_expert_group,  \
        topk_group, topk, n_share_experts_fusion, rsf, scale, topk_weights, topk_indices, idx_dtype, s);          \
    else if (bias_dtype == LO_F16) launch_gate<V, DT, LO_F16>(input, bias, num_tokens, num_experts, num_expert_group, \
        topk_group, topk, n_share_experts_fusion, rsf, scale, topk_weights, topk_indices, idx_dtype, s);          \
    else launch_gate<V, DT, LO_BF16>(input, bias, num_tokens, num_experts, num_expert_group, topk_group, topk,    \
        n_share_experts_fusion, rsf, scale, topk_weights, topk_indices, idx_dtype, s);                            \
  } while (0)
#define LO_G1(V)                               \
  do {                                         \
    if (dtype == LO_F32) LO_G2(V, LO_F32);     \
    else if (dtype == LO_F16) LO_G2(V, LO_F16); \
    else LO_G2(V, LO_BF16);                    \
  } while (0)
  LO_BY_VPT(num_experts, LO_G1);
#undef LO_G1
#undef LO_G2
  return check_launch("moe_fused_gate");
}
