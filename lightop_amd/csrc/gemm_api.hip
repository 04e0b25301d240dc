// C ABI of the grouped block-INT8 GEMM stages: validation and kernel choice.
#include "gemm.h"

namespace lo {

static int64_t grid_m_blocks(int64_t sorted_cap, int64_t num_valid, int bs) {
  // The sorted list can hold at most one partially filled block per slot, so when
  // there are fewer slots than blocks the tail can never be reached (the bound of
  // invoke_fused_moe_kernel_int8, int8.py:572-580).
  int64_t blocks = sorted_cap / bs;
  if (num_valid < blocks) blocks = num_valid;
  return blocks;
}

static bool valid_block_m(int bs) { return bs == 16 || bs == 32 || bs == 64 || bs == 128; }

static int validate_common(const char *who, const void *A, const void *As, const void *W,
                           const void *Ws, const void *sorted, const void *eids, const void *ntpp,
                           int64_t K, int32_t top_k, int32_t E, int64_t a_rows) {
  LO_REQUIRE(A && As && W && Ws && sorted && eids && ntpp, LO_EINVAL, "%s: null pointer", who);
  LO_REQUIRE(K > 0 && K % kGroup == 0, LO_EINVAL, "%s: K (%lld) must be a multiple of 128", who,
             (long long)K);
  LO_REQUIRE(top_k >= 1 && E >= 1 && a_rows >= 1, LO_EINVAL, "%s: bad top_k / E / a_rows", who);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(A) & 15) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0,
             LO_EINVAL, "%s: A and W must be 16-byte aligned", who);
  // the kernels address A and one expert's weights with 32-bit byte offsets
  LO_REQUIRE(a_rows * K < (1ll << 31), LO_ENOTSUP, "%s: A (%lld x %lld bytes) exceeds 2 GiB", who,
             (long long)a_rows, (long long)K);
  return LO_OK;
}

// Which kernel serves a stage.  Token blocks of 64 or 128 rows go to the LDS-tiled kernels (tokens
// per expert large enough for operand reuse to matter); smaller ones stream weights.  The tile
// query (lo_moe_tile_query_form) reports this very choice.
int pick_gemm_kernel(const GemmArgs &a, bool fused_act, int bs, int flags) {
  if (a.out_f32) return LO_KERNEL_WS; // fp32 rows: the weight-streaming kernel's plain epilogue only
  if (bs == 160) return LO_KERNEL_T128; // 160-token blocks exist for that kernel only (the entry point checks)
  const bool tiled = !(flags & LO_GEMM_FORCE_STREAMING);
  if (a.w4 && a.per_channel) // the reference's own int4 form: 128-token LDS tiles, else streaming
    return tiled && gemm_t128_supports(a, fused_act, bs) ? LO_KERNEL_T128 : LO_KERNEL_WS;
  if (a.w4) { // int4 weights: 128- or 64-token LDS tiles, else streaming
    if (tiled && gemm_t128_supports(a, fused_act, bs)) return LO_KERNEL_T128;
    if (tiled && gemm_w4_tile_supports(a, fused_act, bs)) return LO_KERNEL_W4_TILE;
    return LO_KERNEL_WS;
  }
  if (tiled) {
    if (gemm_pc_supports(a, bs)) return LO_KERNEL_PC;
    if (a.per_channel) return LO_KERNEL_WS;
    if (gemm_as_supports(a, fused_act, bs)) return LO_KERNEL_AS;
    if (gemm_t128_supports(a, fused_act, bs)) return LO_KERNEL_T128;
    if (gemm_tile_supports(a, fused_act, bs)) return LO_KERNEL_TILE;
  }
  return LO_KERNEL_WS;
}

// Workgroup shape of that kernel: wavefronts and weight rows per workgroup.
void describe_gemm_kernel(int kernel, bool fused_act, int bs, lo_moe_tile *t) {
  t->block_size_m = bs;
  t->kernel = kernel;
  switch (kernel) {
  case LO_KERNEL_WS: { // gemm_ws.hip: launch_ws
    const int tm = bs / 16;
    const int rpw = tm <= 2 ? LO_WS_RPW : (tm == 4 ? 2 : 1);
    t->waves = fused_act ? 8 : LO_WS_PLAIN_WAVES;
    t->block_n = fused_act ? 256 : 16 * LO_WS_PLAIN_WAVES * rpw;
    break;
  }
  case LO_KERNEL_TILE:
    t->waves = bs == 128 ? 8 : 4;
    t->block_n = 256;
    break;
  default: // t128, activation-stationary, per-channel and int4 tiles: four waves x 64 rows
    t->waves = 4;
    t->block_n = 256;
    break;
  }
}

static int launch_gemm(const GemmArgs &a, bool fused_act, int bs, int flags, int64_t m_blocks,
                       hipStream_t s) {
  switch (pick_gemm_kernel(a, fused_act, bs, flags)) {
  case LO_KERNEL_T128: return launch_gemm_t128(a, fused_act, bs, flags, m_blocks, s);
  case LO_KERNEL_W4_TILE: return launch_gemm_w4_tile(a, fused_act, flags, m_blocks, s);
  case LO_KERNEL_PC: return launch_gemm_pc(a, bs, m_blocks, s);
  case LO_KERNEL_AS: return launch_gemm_as(a, flags, bs, m_blocks, s);
  case LO_KERNEL_TILE: return launch_gemm_tile(a, fused_act, bs, flags, m_blocks, s);
  default: return launch_gemm_ws(a, fused_act, bs, flags, m_blocks, s);
  }
}

} // namespace lo

extern "C" int lo_moe_gemm_block_int8(const int8_t *A, const float *As, const int8_t *W,
                                      const float *Ws, void *C, int c_dtype, const float *topk_w,
                                      const int32_t *sorted_ids, const int32_t *expert_ids,
                                      const int32_t *num_tokens_post_pad, int64_t sorted_cap,
                                      int64_t num_valid, int64_t a_rows, int32_t E, int32_t num_experts,
                                      int64_t N, int64_t K, int32_t top_k, int32_t block_size_m,
                                      int mul_routed, int flags, lo_stream_t stream) {
  using namespace lo;
  int rc = validate_common("moe_gemm", A, As, W, Ws, sorted_ids, expert_ids, num_tokens_post_pad, K,
                           top_k, E, a_rows);
  if (rc) return rc;
  LO_REQUIRE(valid_block_m(block_size_m) || block_size_m == 160, LO_EINVAL,
             "moe_gemm: block_size_m %d is not one of 16, 32, 64, 128 (or 160)", block_size_m);
  LO_REQUIRE(C, LO_EINVAL, "moe_gemm: null output");
  LO_REQUIRE(c_dtype == LO_BF16 || c_dtype == LO_F16 || c_dtype == LO_F32, LO_ENOTSUP,
             "moe_gemm: the output is bf16, fp16 or fp32");
  LO_REQUIRE(c_dtype != LO_F32 || block_size_m != 160, LO_ENOTSUP, "moe_gemm: fp32 rows have no 160-token blocks");
  LO_REQUIRE(N > 0 && N % 16 == 0, LO_EINVAL, "moe_gemm: N (%lld) must be a multiple of 16", (long long)N);
  LO_REQUIRE(N * K < (1ll << 31), LO_ENOTSUP, "moe_gemm: one expert's weights exceed 2 GiB");
  LO_REQUIRE(!mul_routed || topk_w, LO_EINVAL, "moe_gemm: mul_routed needs topk_weights");
  LO_REQUIRE((reinterpret_cast<uintptr_t>(C) & 15) == 0, LO_EINVAL, "moe_gemm: C must be 16-byte aligned");
  LO_REQUIRE((num_valid + top_k - 1) / top_k <= a_rows, LO_EINVAL,
             "moe_gemm: %lld slots / top_k %d exceed the %lld rows of A", (long long)num_valid, top_k,
             (long long)a_rows);
  if (num_valid == 0) return LO_OK;
  GemmArgs a{};
  a.A = A; a.As = As; a.W = W; a.Ws = Ws; a.C = static_cast<uint16_t *>(C);
  a.topk_w = topk_w; a.sorted = sorted_ids; a.expert_ids = expert_ids; a.ntpp = num_tokens_post_pad;
  a.E = E; a.experts_routed = num_experts > E ? num_experts : E; a.a_rows = a_rows; a.num_valid = num_valid; a.N = N; a.K = K; a.top_k = top_k; a.mul_routed = mul_routed ? 1 : 0;
  a.w_shuffled = (flags & LO_GEMM_W_PRESHUFFLED) ? 1 : 0;
  a.skip_nonlocal = (flags & LO_GEMM_SKIP_NONLOCAL) ? 1 : 0;
  a.w4 = (flags & LO_GEMM_W4) ? 1 : 0;
  a.out_f16 = c_dtype == LO_F16 ? 1 : 0;
  a.out_f32 = c_dtype == LO_F32 ? 1 : 0;
  LO_REQUIRE(!a.w4 || a.w_shuffled, LO_ENOTSUP,
             "moe_gemm: int4 weights must be in the layout of lo_preshuffle_weight_int4 (LO_GEMM_W_PRESHUFFLED)");
  a.n_tiles = static_cast<int32_t>((N + 63) / 64);
  LO_REQUIRE(block_size_m != 160 || gemm_t128_supports(a, false, 160), LO_ENOTSUP,
             "moe_gemm: 160-token blocks need int8 weights in the load-time layout (LO_GEMM_W_PRESHUFFLED), "
             "N a multiple of 64 and K <= %d", kGroup * 128);
  const int64_t mblocks = grid_m_blocks(sorted_cap, num_valid, block_size_m);
  LO_REQUIRE(mblocks * a.n_tiles < (1ll << 30), LO_EINVAL, "moe_gemm: grid too large");
  if (mblocks == 0) return LO_OK;
  return launch_gemm(a, false, block_size_m, flags, mblocks, static_cast<hipStream_t>(stream));
}

extern "C" int lo_moe_gemm1_silu_quant_block_int8(
    const int8_t *A, const float *As, const int8_t *W, const float *Ws, int8_t *A2q, float *A2s,
    int c_dtype, const float *topk_w, const int32_t *sorted_ids, const int32_t *expert_ids,
    const int32_t *num_tokens_post_pad, int64_t sorted_cap, int64_t num_valid, int64_t a_rows,
    int32_t E, int32_t num_experts, int64_t I, int64_t K, int32_t top_k, int32_t block_size_m, int mul_routed,
    int flags, lo_stream_t stream) {
  using namespace lo;
  int rc = validate_common("moe_gemm1_silu_quant", A, As, W, Ws, sorted_ids, expert_ids,
                           num_tokens_post_pad, K, top_k, E, a_rows);
  if (rc) return rc;
  LO_REQUIRE(valid_block_m(block_size_m) || block_size_m == 160, LO_EINVAL,
             "moe_gemm1_silu_quant: block_size_m %d is not one of 16, 32, 64, 128 (or 160)", block_size_m);
  LO_REQUIRE(A2q && A2s, LO_EINVAL, "moe_gemm1_silu_quant: null output");
  LO_REQUIRE(c_dtype == LO_BF16, LO_ENOTSUP, "moe_gemm1_silu_quant: only bf16 rounding is built");
  LO_REQUIRE(I > 0 && I % kGroup == 0, LO_EINVAL,
             "moe_gemm1_silu_quant: intermediate size (%lld) must be a multiple of 128", (long long)I);
  LO_REQUIRE(2 * I * K < (1ll << 31), LO_ENOTSUP, "moe_gemm1_silu_quant: one expert's weights exceed 2 GiB");
  LO_REQUIRE(!mul_routed || topk_w, LO_EINVAL, "moe_gemm1_silu_quant: mul_routed needs topk_weights");
  LO_REQUIRE((reinterpret_cast<uintptr_t>(A2q) & 15) == 0, LO_EINVAL,
             "moe_gemm1_silu_quant: A2q must be 16-byte aligned");
  LO_REQUIRE((num_valid + top_k - 1) / top_k <= a_rows, LO_EINVAL,
             "moe_gemm1_silu_quant: %lld slots / top_k %d exceed the %lld rows of A",
             (long long)num_valid, top_k, (long long)a_rows);
  if (num_valid == 0) return LO_OK;
  GemmArgs a{};
  a.A = A; a.As = As; a.W = W; a.Ws = Ws; a.A2q = A2q; a.A2s = A2s;
  a.topk_w = topk_w; a.sorted = sorted_ids; a.expert_ids = expert_ids; a.ntpp = num_tokens_post_pad;
  a.E = E; a.experts_routed = num_experts > E ? num_experts : E; a.a_rows = a_rows; a.num_valid = num_valid; a.N = 2 * I; a.K = K; a.top_k = top_k; a.mul_routed = mul_routed ? 1 : 0;
  a.w_shuffled = (flags & LO_GEMM_W_PRESHUFFLED) ? 1 : 0;
  a.skip_nonlocal = (flags & LO_GEMM_SKIP_NONLOCAL) ? 1 : 0;
  a.w4 = (flags & LO_GEMM_W4) ? 1 : 0;
  LO_REQUIRE(!a.w4 || a.w_shuffled, LO_ENOTSUP,
             "moe_gemm1_silu_quant: int4 weights must be in the layout of lo_preshuffle_weight_int4 "
             "(LO_GEMM_W_PRESHUFFLED)");
  a.n_tiles = static_cast<int32_t>(I / kGroup);
  LO_REQUIRE(block_size_m != 160 || gemm_t128_supports(a, true, 160), LO_ENOTSUP,
             "moe_gemm1_silu_quant: 160-token blocks need int8 weights in the load-time layout "
             "(LO_GEMM_W_PRESHUFFLED) and K <= %d", kGroup * 128);
  rc = silu_table(static_cast<hipStream_t>(stream), &a.silu);
  if (rc) return rc;
  const int64_t mblocks = grid_m_blocks(sorted_cap, num_valid, block_size_m);
  LO_REQUIRE(mblocks * a.n_tiles < (1ll << 31), LO_EINVAL, "moe_gemm1_silu_quant: grid too large");
  if (mblocks == 0) return LO_OK;
  return launch_gemm(a, true, block_size_m, flags, mblocks, static_cast<hipStream_t>(stream));
}

extern "C" int lo_moe_gemm_w8a8(const int8_t *A, const float *As, const int8_t *W, const float *Ws,
                                void *C, int c_dtype, const float *topk_w, const int32_t *sorted_ids,
                                const int32_t *expert_ids, const int32_t *num_tokens_post_pad,
                                int64_t sorted_cap, int64_t num_valid, int64_t a_rows, int32_t E,
                                int32_t num_experts, int64_t N, int64_t K, int32_t top_k,
                                int32_t block_size_m, int mul_routed, int flags, lo_stream_t stream) {
  using namespace lo;
  int rc = validate_common("moe_gemm_w8a8", A, As, W, Ws, sorted_ids, expert_ids, num_tokens_post_pad, K,
                           top_k, E, a_rows);
  if (rc) return rc;
  LO_REQUIRE(valid_block_m(block_size_m) || (block_size_m == 160 && (flags & LO_GEMM_W_PRESHUFFLED)), LO_EINVAL,
             "moe_gemm_w8a8: block_size_m %d is not one of 16, 32, 64, 128 (160: weights in the load-time layout)",
             block_size_m);
  LO_REQUIRE(C, LO_EINVAL, "moe_gemm_w8a8: null output");
  LO_REQUIRE(c_dtype == LO_BF16 || c_dtype == LO_F16, LO_ENOTSUP, "moe_gemm_w8a8: the output is bf16 or fp16");
  LO_REQUIRE(N > 0 && N % 16 == 0, LO_EINVAL, "moe_gemm_w8a8: N (%lld) must be a multiple of 16", (long long)N);
  LO_REQUIRE(N * K < (1ll << 31), LO_ENOTSUP, "moe_gemm_w8a8: one expert's weights exceed 2 GiB");
  LO_REQUIRE(K <= 131072, LO_ENOTSUP, "moe_gemm_w8a8: K (%lld) could overflow the int32 sum", (long long)K);
  LO_REQUIRE(!mul_routed || topk_w, LO_EINVAL, "moe_gemm_w8a8: mul_routed needs topk_weights");
  LO_REQUIRE(!(flags & LO_GEMM_W4) || (flags & LO_GEMM_W_PRESHUFFLED), LO_ENOTSUP,
             "moe_gemm_w8a8: int4 weights exist in the load-time layout only (lo_preshuffle_weight_int4)");
  LO_REQUIRE((reinterpret_cast<uintptr_t>(C) & 15) == 0 && (reinterpret_cast<uintptr_t>(Ws) & 15) == 0, LO_EINVAL,
             "moe_gemm_w8a8: C and the weight scales must be 16-byte aligned");
  LO_REQUIRE((num_valid + top_k - 1) / top_k <= a_rows, LO_EINVAL,
             "moe_gemm_w8a8: %lld slots / top_k %d exceed the %lld rows of A", (long long)num_valid, top_k,
             (long long)a_rows);
  if (num_valid == 0) return LO_OK;
  GemmArgs a{};
  a.A = A; a.As = As; a.W = W; a.Ws = Ws; a.C = static_cast<uint16_t *>(C);
  a.topk_w = topk_w; a.sorted = sorted_ids; a.expert_ids = expert_ids; a.ntpp = num_tokens_post_pad;
  a.E = E; a.experts_routed = num_experts > E ? num_experts : E; a.a_rows = a_rows;
  a.num_valid = num_valid; a.N = N; a.K = K; a.top_k = top_k; a.mul_routed = mul_routed ? 1 : 0;
  a.w_shuffled = (flags & LO_GEMM_W_PRESHUFFLED) ? 1 : 0;
  a.skip_nonlocal = (flags & LO_GEMM_SKIP_NONLOCAL) ? 1 : 0;
  a.per_channel = 1;
  a.out_f16 = c_dtype == LO_F16 ? 1 : 0;
  a.w4 = (flags & LO_GEMM_W4) ? 1 : 0;
  a.n_tiles = static_cast<int32_t>((N + 63) / 64);
  LO_REQUIRE(block_size_m != 160 || gemm_t128_supports(a, false, 160), LO_ENOTSUP,
             "moe_gemm_w8a8: 160-token blocks need N a multiple of 64 and K <= %d", kGroup * 128);
  const int64_t mblocks = grid_m_blocks(sorted_cap, num_valid, block_size_m);
  LO_REQUIRE(mblocks * a.n_tiles < (1ll << 30), LO_EINVAL, "moe_gemm_w8a8: grid too large");
  if (mblocks == 0) return LO_OK;
  return launch_gemm(a, false, block_size_m, flags & ~(LO_GEMM_FUSED_SCALE | LO_GEMM_SEPARATE_ORDER), mblocks,
                     static_cast<hipStream_t>(stream));
}
