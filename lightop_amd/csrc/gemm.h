// Argument block and launchers shared by the grouped block-INT8 GEMM kernels.
#pragma once
#include "common.h"

// Shape of the plain (not fused) weight-streaming workgroup: waves, and 16-row fragments per wave
// at token blocks of 16 or 32 (gemm_ws.hip; the tile query reports the same numbers).
#ifndef LO_WS_PLAIN_WAVES
#define LO_WS_PLAIN_WAVES 4
#endif
#ifndef LO_WS_RPW
#define LO_WS_RPW 4
#endif

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
  const uint16_t *silu;  // fused: bf16(silu(g)) table indexed by the bf16 pattern of g
  const int32_t *sorted; // [>= m_blocks*BM]
  const int32_t *expert_ids;
  const int32_t *ntpp;
  int64_t num_valid;
  int64_t a_rows;        // rows of A / As
  int64_t N;             // weight rows per expert (2I for the fused first GEMM)
  int64_t K;
  int32_t top_k;
  int32_t n_tiles;       // workgroups along N
  int32_t E;             // experts held by W
  int32_t experts_routed; // experts the routing spreads the slots over (estimate, for tile order)
  int32_t mul_routed;
  int32_t w_shuffled;    // W is in the pre-shuffled layout (shuffle.hip)
  int32_t skip_nonlocal; // blocks of expert -1: leave the output rows untouched
  int32_t w4;            // W is packed int4 (load-time layout), Ws is [E, K/128, N]
  int32_t per_channel;   // As is [a_rows], Ws is [E, N]: scales applied once, after the whole-K int32 sum
  int32_t out_f16;       // C holds IEEE half instead of bf16 (plain epilogues only)
  int32_t out_f32;       // C holds the fp32 sums themselves (block form, weight-streaming kernel only)
};

// The 16-bit form a plain epilogue stores: bf16, or IEEE half when the caller's activations are fp16.
// `body(cvt)` is run with the conversion of the output type; the choice is one wave-uniform branch
// around the caller's loops, so the bf16 path pays nothing per value (a per-value select cost the
// activation-stationary second GEMM 10 %).
template <typename Body>
__device__ __forceinline__ void with_out16(int f16, Body body) {
  if (__builtin_expect(f16 != 0, 0)) body([](float v) { return f32_to_f16(v); });
  else body([](float v) { return f32_to_bf16(v); });
}

// Order of the scale arithmetic per 128-wide K block (d = the block's exact int32 sum):
//   kOrdContract   acc = fma(f32(d) * a_s, b_s, acc)    the default: what the reference's Triton line
//                  `accumulator += tl.dot(a, b) * a_scale * b_scale` (int8.py:499-508) compiles to with
//                  the AMD backend's default enable_fp_fusion; three vector instructions per element
//   kOrdSeparate   acc = acc + (f32(d) * a_s) * b_s     the same line without fp fusion; four instructions
//                  (LO_GEMM_SEPARATE_ORDER)
//   kOrdFusedScale acc = fma(f32(d), a_s * b_s, acc)    two instructions, last-ulp differences in fp32
//                  (LO_GEMM_FUSED_SCALE)
// The CPU checker restates the first two bit for bit.
constexpr int kOrdSeparate = 0, kOrdFusedScale = 1, kOrdContract = 2;
inline int scale_order(int flags) {
  if (flags & LO_GEMM_SEPARATE_ORDER) return kOrdSeparate;
  return (flags & LO_GEMM_FUSED_SCALE) ? kOrdFusedScale : kOrdContract;
}
// One accumulator element.  sc = a_s * b_s is read by kOrdFusedScale only, as and bs by the other two.
template <int ORD>
__device__ __forceinline__ float fold_elem(int d, float sc, float as, float bs, float acc) {
  if constexpr (ORD == kOrdFusedScale) {
    return __builtin_fmaf(static_cast<float>(d), sc, acc);
  } else if constexpr (ORD == kOrdContract) {
    return __builtin_fmaf(static_cast<float>(d) * as, bs, acc);
  } else {
    float t = static_cast<float>(d) * as;
    t = t * bs;
    return acc + t;
  }
}
// Three-way dispatch of a launcher macro on the order: LO_ORD_DISPATCH(ord, MACRO, args...) expands to
// MACRO(order constant, args...).
#define LO_ORD_DISPATCH(ord, MACRO, ...)                                   \
  do {                                                                     \
    if ((ord) == ::lo::kOrdContract) MACRO(::lo::kOrdContract, __VA_ARGS__);      \
    else if ((ord) == ::lo::kOrdSeparate) MACRO(::lo::kOrdSeparate, __VA_ARGS__); \
    else MACRO(::lo::kOrdFusedScale, __VA_ARGS__);                         \
  } while (0)

__device__ __forceinline__ v4i ld16(const int8_t *p) { return *reinterpret_cast<const v4i *>(p); }

// Buffer addressing: a wave-uniform 128-bit resource (base, extent) + one 32-bit lane
// offset + one scalar offset.  The K loop then advances a scalar only, no per-lane 64-bit
// address arithmetic, and a read past the extent returns zero instead of faulting.
typedef __amdgpu_buffer_rsrc_t brsrc;
__device__ __forceinline__ brsrc make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, static_cast<int>(bytes), 0x00020000);
}
constexpr int kCacheDefault = 0;
constexpr int kCacheStream = 2; // "nt": data that is read once (weights in the streaming regime)
template <int AUX = kCacheDefault>
__device__ __forceinline__ v4i bld16(brsrc r, int voff, int soff) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, AUX);
}
__device__ __forceinline__ float bld_f32(brsrc r, int voff, int soff) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}

// Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
// The logical tile list is cut into chunks of (G token blocks x all weight tiles): the
// tiles of a chunk share token rows, and neighbouring token blocks mostly share an
// expert's weights; G is about one expert's worth of token blocks, so that an expert's
// weights are fetched into one L2 only.  Chunks are dealt round-robin to the XCDs, and the workgroups that
// an XCD receives one after the other walk through one chunk, so what is shared is
// fetched into that XCD's L2 once; blocks of experts that are not on this rank (which
// cluster by expert id) still spread evenly over all XCDs.
__device__ __forceinline__ bool tile_of(int bid, int n_tiles, int m_blocks, int G, int &mb, int &nt) {
  constexpr int XCD = 8;
  const int xcd = bid % XCD, slot = bid / XCD;
  const int span = G * n_tiles;                      // tiles per chunk
  const int chunk = (slot / span) * XCD + xcd, in = slot % span;
  const int first = chunk * G;
  if (first >= m_blocks) return false;
  const int gsz = (m_blocks - first < G) ? (m_blocks - first) : G;
  nt = in / G;
  const int off = in - nt * G;
  if (off >= gsz) return false;
  mb = first + off;
  return true;
}

// Output of the 32x32-MFMA kernels.  In the accumulator layout a lane (r = lane & 31, c = lane >> 5)
// holds, of one 32-token x 64-column piece, token r and columns rb*32 + 8q + 4c + i: four
// consecutive bf16 per (rb, q).  Stored directly that is 8 bytes to each of 64 different token
// rows per instruction, and the texture path, which also carries the operand loads these
// kernels are bound by, spends a cycle per row touched.  Each wave therefore turns its piece
// around in LDS (LDS operations of one wave execute in order: no barrier) and stores whole
// 128-byte row segments, eight rows per instruction.
//   stg   32 * kStgPitch bytes of LDS owned by this wave
//   o     the lane's 2 x 4 packed column quadruples
//   slot  output row of token r, or -1 (lanes r and r + 32 agree)
//   C     + slot * N + col0: first of the piece's 64 columns; 16-byte aligned
constexpr int kStgPitch = 64 * 2 + 16; // bytes per staged token row: 16 mod 128 keeps both passes conflict-free
__device__ __forceinline__ void wave_store_32x64_bf16(int8_t *stg, const v4u16 (&o)[2][4], int slot, uint16_t *C,
                                                      int64_t N, int64_t col0, int lane) {
  const int r = lane & 31, c = lane >> 5;
#pragma unroll
  for (int rb = 0; rb < 2; ++rb)
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<v4u16 *>(stg + r * kStgPitch + (rb * 32 + 8 * q + 4 * c) * 2) = o[rb][q];
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int tok = (lane >> 3) + 8 * j;
    const v4i v = *reinterpret_cast<const v4i *>(stg + tok * kStgPitch + (lane & 7) * 16);
    const int ft = __shfl(slot, tok);
    if (ft >= 0) *reinterpret_cast<v4i *>(C + static_cast<int64_t>(ft) * N + col0 + (lane & 7) * 8) = v;
  }
  __builtin_amdgcn_wave_barrier();
}

// Kernel a stage is served by, and its workgroup shape (gemm_api.hip).
int pick_gemm_kernel(const GemmArgs &a, bool fused_act, int block_size_m, int flags);
void describe_gemm_kernel(int kernel, bool fused_act, int block_size_m, lo_moe_tile *t);

// Decode-size whole path in two launches (gemm_dec.hip): LO_ENOTSUP when it does not apply.
// act: room for [M * top_k, I] bf16.  w4: packed int4 weights with K-group scales [E, K/128, N].
bool decode_path_applies(int64_t M, int32_t top_k, int64_t H, int64_t I, int32_t num_experts, bool force, bool w4);
void decode_path_waves(int32_t top_k, int64_t H, int *gemm1_waves, int *gemm2_waves);
int launch_decode_path(const void *x, int64_t M, int64_t H, int64_t I, int32_t E, int32_t num_experts, int32_t top_k,
                       const int8_t *w1, const float *w1s, const int8_t *w2, const float *w2s, const float *topk_w,
                       const void *topk_ids, int ids_dtype, const int32_t *expert_map, int apply_router_weight_on_input,
                       float factor, const void *shared_output, void *act, void *out, bool force, bool w4, int flags,
                       hipStream_t stream);

// Weight-streaming kernels (gemm_ws.hip): block_size_m in {16, 32, 64, 128}.
int launch_gemm_ws(const GemmArgs &a, bool fused_act, int block_size_m, int flags, int64_t m_blocks,
                   hipStream_t s);
// LDS-tiled kernels (gemm_tile.hip): block_size_m 64 or 128, compute-bound regime.
int launch_gemm_tile(const GemmArgs &a, bool fused_act, int block_size_m, int flags, int64_t m_blocks,
                     hipStream_t s);
bool gemm_tile_supports(const GemmArgs &a, bool fused_act, int block_size_m);
// Activation-stationary kernel (gemm_as.hip): plain epilogue, block_size_m 64 or 128, short K.
int launch_gemm_as(const GemmArgs &a, int flags, int block_size_m, int64_t m_blocks, hipStream_t s);
bool gemm_as_supports(const GemmArgs &a, bool fused_act, int block_size_m);

// 128-token kernel, two four-wave workgroups per compute unit (gemm_t128.hip): pre-shuffled int8 weights.
int launch_gemm_t128(const GemmArgs &a, bool fused_act, int block_size_m, int flags, int64_t m_blocks, hipStream_t s);
bool gemm_t128_supports(const GemmArgs &a, bool fused_act, int block_size_m);
// W4A8 LDS-tiled kernel (gemm_w4.hip): block_size_m 64.
int launch_gemm_w4_tile(const GemmArgs &a, bool fused_act, int flags, int64_t m_blocks, hipStream_t s);
bool gemm_w4_tile_supports(const GemmArgs &a, bool fused_act, int block_size_m);
// Per-channel LDS-tiled kernel (gemm_pc.hip): block_size_m 64 or 128.
int launch_gemm_pc(const GemmArgs &a, int block_size_m, int64_t m_blocks, hipStream_t s);
bool gemm_pc_supports(const GemmArgs &a, int block_size_m);

} // namespace lo
