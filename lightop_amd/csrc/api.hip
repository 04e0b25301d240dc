// Host side of the C ABI: error reporting, the gfx950 tile table and the whole-path
// entry point that chains the stage kernels on one stream.
#include <cstdarg>
#include <cstdio>
#include <mutex>

#include "gemm.h"

namespace lo {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return LO_ELAUNCH;
  }
  return LO_OK;
}

int reserve_lds_once(const void *kernel, int bytes, unsigned long long *done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    set_error("no current HIP device");
    return LO_ELAUNCH;
  }
  const unsigned long long bit = 1ull << dev;
  if (__atomic_load_n(done, __ATOMIC_ACQUIRE) & bit) return LO_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
    (void)hipGetLastError();
    set_error("cannot reserve %d bytes of LDS for a kernel", bytes);
    return LO_ELAUNCH;
  }
  __atomic_fetch_or(done, bit, __ATOMIC_RELEASE);
  return LO_OK;
}

static int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// Extents of the alignment buffers (moe_align_block_size.py:80-93 of the reference).
static void align_caps(int64_t numel, int32_t num_experts, int32_t bs, int64_t *sorted_cap,
                       int64_t *blocks_cap) {
  int64_t cap = numel + static_cast<int64_t>(num_experts) * (bs - 1);
  if (numel < num_experts && numel * bs < cap) cap = numel * bs;
  *sorted_cap = cap;
  *blocks_cap = (cap + bs - 1) / bs;
}

struct WsLayout {
  int64_t off[9];
  int64_t align_scratch;
  int64_t total;
  int64_t sorted_cap, blocks_cap;
};

static WsLayout ws_layout(int64_t M, int32_t top_k, int64_t H, int64_t I, int32_t num_experts,
                          int32_t bs) {
  WsLayout L{};
  const int64_t S = M * top_k;
  align_caps(S, num_experts, bs, &L.sorted_cap, &L.blocks_cap);
  L.align_scratch = lo_moe_align_scratch_bytes(S, num_experts);
  const int64_t sizes[9] = {M * H,                 // a1q
                            M * (H / kGroup) * 4,  // a1s
                            L.sorted_cap * 4,      // sorted_ids
                            L.blocks_cap * 4,      // expert_ids
                            4,                     // num_tokens_post_pad
                            S * I,                 // a2q
                            S * (I / kGroup) * 4,  // a2s
                            S,                     // slot mask
                            L.align_scratch};      // per-chunk expert counters of the alignment
  int64_t o = 0;
  for (int i = 0; i < 9; ++i) {
    L.off[i] = o;
    o += align_up(sizes[i] > 0 ? sizes[i] : 1, 256);
  }
  L.total = o;
  return L;
}

// 160-token blocks: both K extents have to fit the kernel's scale table (128 K blocks); where the first GEMM
// is not fused with the activation (fp16 rows, GELU) its 16-bit output [S, 2I] has to fit the caller's [S, H]
// buffer as well.
static bool blocks_of_160_fit(int64_t H, int64_t I, bool fused) {
  return (fused || 2 * I <= H) && H / kGroup <= 128 && I / kGroup <= 128;
}

// gfx950 tile table.  The token tile (= alignment block) follows the expected number
// of slots per expert: small tiles waste no MFMA columns on padding while the layer
// is weight-streaming bound, larger ones amortise each pass over an expert's weights.
//
// The key is (form, weight layout, shape class, expected slots per expert).  The shape class is the size of one
// expert's weights, 3 * H * I bytes of int8: a handful of megabytes (Qwen3-30B-A3B: H 2048, I 768, 4.7 MB),
// around twenty (Qwen3-235B-A22B: 4096 x 1536, 18.9 MB), forty and more (DeepSeek-V3: 7168 x 2048, 44 MB); the
// thresholds below were measured on one layer of each class with `python -m lightop_amd.tune`.
static int32_t pick_block_m(int64_t M, int32_t num_experts, int32_t top_k, int64_t H, int64_t I,
                            int form = LO_FORM_BLOCK, bool preshuffled = true, bool int4_channel = false,
                            bool allow160 = false) {
  const double per_expert = static_cast<double>(M) * top_k / (num_experts > 0 ? num_experts : 1);
  // Packed int4 weights with per-channel scales: the 128-token kernel has no scale arithmetic in
  // its K loop and skips the padded part of a block, so it takes over as soon as an expert sees more
  // than a dozen tokens (measured on the Qwen3-235B-A22B-shaped layer, whole path in us, 16 / 32 /
  // 64 / 128: at 128 tokens 247 / 254 / 401 / 267, at 256: 365 / 294 / 433 / 285, at 1024: 953 / 727 /
  // 842 / 382, at 2048: 1610 / 1224 / 1455 / 596).
  // Around 128 slots per expert the 160-token form of that kernel holds an expert's tokens in one block
  // (a remainder block is a second pass over the expert's weights): same layer, 128 / 160: at 1024
  // tokens 345 / 358, at 1280: 394 / 386, at 1792: 488 / 422, at 2048: 541 / 444, at 2304: 629 / 517, at
  // 2560: 658 / 620, at 3072: 686 / 754.  The same happens around 256 slots per expert, where two 160-token
  // blocks hold what would spill into a third 128-token block (at 3840 tokens 779 / 796, at 4096: 869 / 797,
  // at 4352: 938 / 830, at 4608: 964 / 868, at 4864: 997 / 924, at 5120: 1012 / 1030); the int8 forms,
  // whose tiles are bound by arithmetic at that size, gain nothing there.
  if (form == LO_FORM_CHANNEL && int4_channel) {
    if (per_expert <= 12.0) return 16;
    const bool one_block = per_expert >= 76.0 && per_expert < 170.0;
    const bool two_blocks = per_expert >= 248.0 && per_expert < 312.0;
    return (allow160 && (one_block || two_blocks)) ? 160 : 128;
  }
  // W4A8: the streaming kernel re-reads the token rows per wave, which outweighs the half-size
  // weights early; the LDS-tiled kernel (64 tokens) wins above about 8 slots per expert.
  // From 48 slots per expert on the 128-token kernel takes over (measured, 64 / 128: 475 / 394 us at
  // 1024 tokens of the Qwen3-235B-A22B-shaped layer, 720 / 660 at 2048, 1227 / 1074 at 4096; equal
  // or 3 % behind up to 512 tokens, where a K block of half-size weights is shorter than the memory
  // round trip it would have to hide).
  if (form == LO_FORM_W4) return per_expert <= 8.0 ? 16 : (per_expert < 48.0 ? 64 : 128);
  // Block form with pre-shuffled weights: the kernel that copies both operands straight into LDS
  // (gemm_t128.hip, 128-token blocks, padded parts of a block skipped in steps of 32 tokens) takes
  // over from the weight-streaming kernels as soon as an expert sees a handful of tokens - with
  // about one token block per expert it streams the weights with the non-temporal hint and keeps
  // far more bytes in flight per compute unit than the register-fed kernels - and stays ahead of
  // the 64-token LDS tiles except around 128 slots per expert on a short K, where its longer
  // epilogue weighs most.  Measured (us, whole path, 16 / 32 / 64 / 128): Qwen3-30B-A3B layer at
  // 128 tokens 133 / 139 / 186 / 139, at 256: 190 / 160 / 190 / 146, at 1024: 505 / 414 / 224 /
  // 191, at 2048: 878 / 690 / 267 / 285, at 8192: - / - / 682 / 645; DeepSeek-V3 share of 32
  // experts at 128 tokens 248 / 262 / 315 / 241, at 2048: 1034 / 810 / 427 / 336, at 8192:
  // - / - / 928 / 776.
  // Around 128 slots per expert a 128-token block spills a few tokens into a second block on half of
  // the experts, and that remainder block is a second pass over the expert's weights - the bytes the
  // stage is bound by at that size.  160-token blocks (the same kernel with ten token fragments, plain
  // epilogues, the activation in a launch of its own) hold such an expert in one block.  Measured,
  // whole path in us, table before / 160: Qwen3-30B-A3B layer at 1280 tokens (80 slots per expert)
  // 239 / 229, 1536: 264 / 230, 1792: 275 / 239, 2048: 302 / 265, 2304: 351 / 301, 2560: 348 / 355;
  // DeepSeek-V3 share at 3072 (96 per expert): 435 / 451, 3584: 544 / 468, 4096: 581 / 495, 4352:
  // 610 / 616, 4608: 620 / 660.
  if (form == LO_FORM_BLOCK && preshuffled && allow160) {
    // With the first stage's fused epilogue in the 160-token form as well (no activation launch, no [S, 2I] round
    // trip) the window widens; whole path in us, 128 / 160: Qwen3-30B-A3B layer at 1024 tokens (64 slots per
    // expert) 184 / 193, at 1152: 230 / 197, at 2048: 279 / 221, at 2432: 306 / 276, at 2560: 298 / 307;
    // DeepSeek-V3 share at 2560 (80 per expert): 380 / 367, at 3072: 381 / 373, at 4096: 541 / 428, at 4352:
    // 561 / 570.
    // Medium experts (Qwen3-235B-A22B-shaped layer, int8): at 1280 tokens (80 per expert) 573 / 580, at 1536: 606 /
    // 596, at 2048: 775 / 659, at 2304: 889 / 742, at 2560: 911 / 934.
    const bool medium = H >= 4096 && 3 * H * I < (32ll << 20);
    if (medium ? (per_expert >= 88.0 && per_expert < 152.0)
               : H >= 4096 ? (per_expert >= 76.0 && per_expert < 134.0) : (per_expert >= 68.0 && per_expert < 156.0))
      return 160;
    // Small experts again around 256 slots per expert, where two 160-token blocks hold what would spill into a
    // third block of 128 (Qwen3-30B-A3B layer, 128 / 160: at 3840 tokens 365 / 381, at 4096: 391 / 376, at 4352:
    // 415 / 382, at 4608: 429 / 427, at 5120: 445 / 491); the larger experts, whose tiles are bound by arithmetic
    // at that size, gain nothing there (DeepSeek-V3 share at 8192 tokens 795 / 801).
    if (H < 4096 && per_expert >= 248.0 && per_expert < 284.0) return 160;
  }
  // With about one token block per expert the 64-token kernel with register-fed weights
  // (gemm_tile.hip) streams them with the non-temporal hint as well, and its shorter start-up and
  // epilogue put it ahead on a short K.  Measured (us, whole path, 16 / 64 / 128): Qwen3-30B-A3B layer
  // at 64 tokens 117 / 117 / 130, at 128: 126 / 119 / 133, at 256: 184 / 126 / 140, at 512: 289 / 135 /
  // 157, at 768: - / 162 / 176, at 1024: - / 218 / 194; DeepSeek-V3 share at 512 tokens 356 / 251 / 251,
  // at 768: 508 / 264 / 264, at 1024: 638 / 276 / 283, at 1536: 847 / 292 / 303, at 2048: - / 428 / 333.
  if (form == LO_FORM_BLOCK && preshuffled) {
    if (H < 4096) {
      if (per_expert < 6.0) return 16;
      // 96 to 152 (where 160-token blocks cannot be used): the remainder blocks' second pass costs the
      // 64-token tiles less; from 160 slots per expert on the 128-token kernel is ahead again (at 2560
      // tokens 313 / 303, at 2816: 325 / 306)
      if (per_expert <= 48.0 || (per_expert >= 96.0 && per_expert < 152.0)) return 64;
      return 128;
    }
    if (3 * H * I < (32ll << 20)) {
      // Medium experts, measured on the Qwen3-235B-A22B-shaped layer with int8 weights (us, whole path, 16 /
      // 64 / 128): at 16 tokens 253 / 246 / 256, at 64: 416 / 376 / 391, at 128: 450 / 391 / 407, at 256: 631 /
      // 414 / 427, at 512: 1022 / 444 / 461, at 768: - / 504 / 488, at 1024: - / 618 / 522, at 4096: - / 1392 /
      // 1200.
      if (per_expert < 1.0) return 16;
      return per_expert <= 40.0 ? 64 : 128;
    }
    if (per_expert < 4.0) return 16;
    return (per_expert >= 28.0 && per_expert <= 48.0) ? 64 : 128; // equal within 0.2 % from 16 to 24
  }
  // Per-channel form: no scale arithmetic in the K loop, so the accumulators of 128 tokens fit
  // and the larger tile halves the weight bytes requested from L2 per multiply-add; with about one
  // token block per expert the LDS-tiled kernels stream the weights with the non-temporal hint and
  // take over from the weight-streaming kernel at half a dozen slots per expert.  Measured (us, whole
  // path, 16 / 32 / 64 / 128): Qwen3-30B-A3B-shaped layer at 64 tokens 122 / 122 / 121 / 126, at 128:
  // 130 / 132 / 127 / 130, at 256: 188 / 147 / 135 / 138, at 512: 296 / 223 / 152 / 153, at 1024:
  // 489 / 361 / 223 / 173; DeepSeek-V3 share of 32 experts at 128 tokens 252 / 251 / 253 / 253, at
  // 256: 268 / 268 / 270 / 262, at 512: 365 / 296 / 297 / 285, at 1024: 627 / 476 / 336 / 319.
  // Around 128 slots per expert the 160-token form of the direct-to-LDS kernel (int32 sums over the whole K
  // in its accumulators) holds an expert's tokens in one block, where a 128-token block spills into a
  // second pass over the expert's weights.  Measured, 128 / 160: DeepSeek-V3 share at 2048 tokens 378 / 384,
  // at 2560: 476 / 418, at 3584: 616 / 475, at 4096: 629 / 514, at 4608: 659 / 686; Qwen3-shaped layer at
  // 1024 tokens 173 / 192, at 1280: 222 / 201, at 2048: 259 / 226, at 2304: 285 / 250, at 2560: 273 / 306.
  if (form == LO_FORM_CHANNEL) {
    if (per_expert <= 6.0) return 16;
    if (allow160 && per_expert >= 72.0 && per_expert < (H >= 4096 ? 140.0 : 152.0)) return 160;
    return (H >= 4096 || per_expert >= 48.0) ? 128 : 64;
  }
  if (per_expert <= 12.0) return 16;
  if (per_expert <= 24.0) return 32;
  // Row-major block-form weights: 64-token LDS tiles, two workgroups per CU; their 128-token
  // kernel is one phase-locked workgroup per CU and measured slower on every layer shape tried.
  return 64;
}

// What the block-form whole-path call (int8 weights, or int4 weights with K-group scales) does with a
// problem: the token-block size and which launches follow.  One function for the call itself, for its
// no-allocation variant's space check and for the tile query, so that the three cannot drift apart.
struct BlockPlan {
  int flags;            // the caller's flags, LO_GEMM_W4 implying LO_GEMM_W_PRESHUFFLED
  int32_t block_size_m; // the caller's, or the table's pick when the caller passed 0
  bool bs160;           // 160-token blocks of the direct-to-LDS kernel
  bool unfused;         // the first GEMM writes [S, 2I] and one launch applies the activation and quantises
  bool try_decode;      // the two-launch path is attempted first (it may still decline by size)
};
static int plan_block_path(int dtype, int flags, int64_t M, int32_t num_experts, int32_t top_k, int64_t H, int64_t I,
                           int32_t block_size_m, BlockPlan *plan) {
  if (flags & LO_GEMM_W4) flags |= LO_GEMM_W_PRESHUFFLED; // packed int4 exists in the load-time layout only
  const bool w4 = (flags & LO_GEMM_W4) != 0, pre = (flags & LO_GEMM_W_PRESHUFFLED) != 0;
  const bool gelu = (flags & LO_FUSED_ACT_GELU) != 0;
  const bool block_size_m_auto = block_size_m == 0;
  if (block_size_m == 0 && dtype == LO_F32) // fp32 rows go through the weight-streaming kernel at every size
    block_size_m = pick_block_m(M, num_experts, top_k, H, I, LO_FORM_BLOCK, false);
  if (block_size_m == 0)
    block_size_m = pick_block_m(M, num_experts, top_k, H, I, w4 ? LO_FORM_W4 : LO_FORM_BLOCK, pre, false,
                                !w4 && dtype == LO_BF16 && !gelu && blocks_of_160_fit(H, I, true));
  // 160: the 160-token form of the direct-to-LDS kernel (int8 block form, load-time layout) for both GEMMs; bf16
  // rows with SiLU take its fused first stage, fp16 rows and GELU the plain one and the activation launch
  const bool fused_ok = dtype == LO_BF16 && !gelu;
  const bool bs160 = block_size_m == 160 && pre && !w4 && dtype != LO_F32 && blocks_of_160_fit(H, I, fused_ok);
  LO_REQUIRE(block_size_m == 16 || block_size_m == 32 || block_size_m == 64 || block_size_m == 128 || bs160,
             LO_EINVAL,
             "fused_experts: block_size_m %d is not one of 16, 32, 64, 128 (160: int8 weights in the load-time "
             "layout and 16-bit rows; with fp16 rows or GELU 2I <= H as well)", block_size_m);
  plan->flags = flags;
  plan->block_size_m = block_size_m;
  plan->bs160 = bs160;
  // GELU and fp16 / fp32 activations have no fused epilogue
  plan->unfused = !fused_ok;
  plan->try_decode = block_size_m_auto && pre && !plan->unfused && !(flags & LO_FUSED_NO_DECODE_PATH);
  return LO_OK;
}

} // namespace lo

extern "C" int lo_version(void) { return 101; }

extern "C" const char *lo_last_error(void) { return lo::g_err; }

extern "C" int lo_moe_tile_query_path(int form, int flags, int dtype, int32_t block_size_m, int64_t M, int32_t E_local,
                                      int32_t num_experts, int32_t top_k, int64_t H, int64_t I, lo_moe_tile *gemm1,
                                      lo_moe_tile *gemm2) {
  using namespace lo;
  LO_REQUIRE(form == LO_FORM_BLOCK || form == LO_FORM_CHANNEL || form == LO_FORM_W4, LO_EINVAL,
             "moe_tile_query: unknown form %d", form);
  LO_REQUIRE(M >= 0 && num_experts >= 1 && top_k >= 1 && H > 0 && I > 0, LO_EINVAL,
             "moe_tile_query: bad problem size");
  LO_REQUIRE(dtype == LO_BF16 || dtype == LO_F16 || dtype == LO_F32, LO_EINVAL, "moe_tile_query: unknown dtype %d", dtype);
  if (form == LO_FORM_W4) flags |= LO_GEMM_W4 | LO_GEMM_W_PRESHUFFLED;
  int32_t bm = block_size_m;
  bool fused = false, decode = false;
  if (form == LO_FORM_CHANNEL) {
    const bool pre = (flags & (LO_GEMM_W4 | LO_GEMM_W_PRESHUFFLED)) != 0;
    if (bm == 0)
      bm = pick_block_m(M, num_experts, top_k, H, I, form, true, (flags & LO_GEMM_W4) != 0,
                        pre && H / kGroup <= 128 && I / kGroup <= 128);
  } else {
    BlockPlan plan;
    const int rc = plan_block_path(dtype, flags, M, num_experts, top_k, H, I, block_size_m, &plan);
    if (rc) return rc;
    flags = plan.flags;
    bm = plan.block_size_m;
    fused = !plan.unfused;
    decode = plan.try_decode && M > 0 &&
             decode_path_applies(M, top_k, H, I, num_experts, (flags & LO_FUSED_FORCE_DECODE_PATH) != 0,
                                 (flags & LO_GEMM_W4) != 0);
  }
  const bool pre = (flags & LO_GEMM_W_PRESHUFFLED) != 0;
  // the argument blocks the stage entry points would build for this problem
  GemmArgs a{};
  a.num_valid = M * top_k;
  a.E = E_local > 0 ? E_local : num_experts;
  a.experts_routed = num_experts;
  a.top_k = top_k;
  a.w_shuffled = pre ? 1 : 0;
  a.w4 = (flags & LO_GEMM_W4) ? 1 : 0;
  a.per_channel = form == LO_FORM_CHANNEL ? 1 : 0;
  a.out_f16 = dtype == LO_F16 ? 1 : 0;
  a.out_f32 = dtype == LO_F32 ? 1 : 0;
  const int gflags = flags & ~(LO_FUSED_ACT_GELU | LO_FUSED_NO_DECODE_PATH | LO_FUSED_FORCE_DECODE_PATH);
  if (gemm1) {
    a.N = 2 * I; a.K = H; a.a_rows = M;
    describe_gemm_kernel(pick_gemm_kernel(a, fused, bm, gflags), fused, bm, gemm1);
  }
  if (gemm2) {
    a.N = H; a.K = I; a.a_rows = M * top_k;
    describe_gemm_kernel(pick_gemm_kernel(a, false, bm, gflags), false, bm, gemm2);
  }
  // a few tokens: the whole-path call serves the block form with its two-launch path
  if (decode) {
    int w1 = 0, w2 = 0;
    decode_path_waves(top_k, H, &w1, &w2);
    if (gemm1) { gemm1->kernel = LO_KERNEL_DEC; gemm1->waves = w1; gemm1->block_n = 16; }
    if (gemm2) { gemm2->kernel = LO_KERNEL_DEC; gemm2->waves = w2; gemm2->block_n = 16; }
  }
  return LO_OK;
}

extern "C" int lo_moe_tile_query_form(int form, int flags, int64_t M, int32_t E_local, int32_t num_experts,
                                      int32_t top_k, int64_t H, int64_t I, lo_moe_tile *gemm1, lo_moe_tile *gemm2) {
  return lo_moe_tile_query_path(form, flags, LO_BF16, 0, M, E_local, num_experts, top_k, H, I, gemm1, gemm2);
}

extern "C" int lo_moe_tile_query(int64_t M, int32_t E_local, int32_t num_experts, int32_t top_k,
                                 int64_t H, int64_t I, lo_moe_tile *gemm1, lo_moe_tile *gemm2) {
  return lo_moe_tile_query_form(LO_FORM_BLOCK, LO_GEMM_W_PRESHUFFLED, M, E_local, num_experts, top_k, H, I, gemm1,
                                gemm2);
}

extern "C" int64_t lo_fused_experts_workspace_bytes(int64_t M, int32_t top_k, int64_t H, int64_t I,
                                                    int32_t num_experts, int32_t block_size_m) {
  using namespace lo;
  if (M < 0 || top_k < 1 || H < kGroup || I < kGroup || num_experts < 1) return LO_EINVAL;
  if (block_size_m != 0) return ws_layout(M, top_k, H, I, num_experts, block_size_m).total + 256;
  // 0: whatever the table (or a later explicit choice) picks.  The sorted ids grow with the block
  // size, the per-block expert ids shrink with it: take the largest layout of the four.
  int64_t most = 0;
  for (int32_t bs : {16, 32, 64, 128, 160}) {
    const int64_t t = ws_layout(M, top_k, H, I, num_experts, bs).total;
    most = t > most ? t : most;
  }
  return most + 256;
}

extern "C" int64_t lo_fused_experts_workspace_offset(int which, int64_t M, int32_t top_k, int64_t H,
                                                     int64_t I, int32_t num_experts,
                                                     int32_t block_size_m) {
  using namespace lo;
  if (which < 0 || which > 7 || block_size_m <= 0) return LO_EINVAL;
  return ws_layout(M, top_k, H, I, num_experts, block_size_m).off[which];
}

extern "C" int lo_fused_experts_block_int8(
    const void *x, int dtype, int64_t M, int64_t H, int64_t I, int32_t E, int32_t num_experts,
    int32_t top_k, const int8_t *w1, const float *w1s, const int8_t *w2, const float *w2s,
    const float *topk_w, const void *topk_ids, int ids_dtype, const int32_t *expert_map,
    int apply_router_weight_on_input, float routed_scaling_factor, const void *shared_output,
    void *cache3, void *out, void *workspace, int64_t workspace_bytes, int32_t block_size_m,
    int flags, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(x && w1 && w1s && w2 && w2s && topk_w && topk_ids && cache3 && out && workspace,
             LO_EINVAL, "fused_experts: null pointer");
  LO_REQUIRE(dtype == LO_BF16 || dtype == LO_F16 || (dtype == LO_F32 && !(flags & LO_GEMM_W4)), LO_ENOTSUP,
             "fused_experts: activations are bf16, fp16 or (int8 weights) fp32");
  LO_REQUIRE(M >= 0 && H >= kGroup && H % kGroup == 0 && I >= kGroup && I % kGroup == 0, LO_EINVAL,
             "fused_experts: hidden (%lld) and intermediate (%lld) sizes must be multiples of 128",
             (long long)H, (long long)I);
  LO_REQUIRE(E >= 1 && num_experts >= E && top_k >= 1, LO_EINVAL, "fused_experts: bad expert counts");
  LO_REQUIRE(num_experts == E || expert_map, LO_EINVAL,
             "fused_experts: global_num_experts (%d) != local experts (%d) needs an expert_map",
             num_experts, E);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, LO_EINVAL,
             "fused_experts: workspace must be 256-byte aligned");
  if (M == 0) return LO_OK;
  BlockPlan plan;
  const int rc_plan = plan_block_path(dtype, flags, M, num_experts, top_k, H, I, block_size_m, &plan);
  if (rc_plan) return rc_plan;
  flags = plan.flags;
  block_size_m = plan.block_size_m;
  const WsLayout L = ws_layout(M, top_k, H, I, num_experts, block_size_m);
  LO_REQUIRE(workspace_bytes >= L.total, LO_ENOSPC, "fused_experts: workspace holds %lld bytes, needs %lld",
             (long long)workspace_bytes, (long long)L.total);
  char *ws = static_cast<char *>(workspace);
  int8_t *a1q = reinterpret_cast<int8_t *>(ws + L.off[0]);
  float *a1s = reinterpret_cast<float *>(ws + L.off[1]);
  int32_t *sorted = reinterpret_cast<int32_t *>(ws + L.off[2]);
  int32_t *eids = reinterpret_cast<int32_t *>(ws + L.off[3]);
  int32_t *ntpp = reinterpret_cast<int32_t *>(ws + L.off[4]);
  int8_t *a2q = reinterpret_cast<int8_t *>(ws + L.off[5]);
  float *a2s = reinterpret_cast<float *>(ws + L.off[6]);
  // With an expert_map most slots may belong to other ranks: their rows of cache3 are
  // neither zero-filled by the second GEMM nor read by the reduction.
  uint8_t *mask = expert_map ? reinterpret_cast<uint8_t *>(ws + L.off[7]) : nullptr;
  const int64_t S = M * top_k;

  // Decode sizes: routing, quantisation, both GEMMs and the reduction in two launches (in the default scale
  // order, or the one of LO_GEMM_SEPARATE_ORDER; LO_GEMM_FUSED_SCALE buys nothing there and gets the default).
  const bool gelu = (flags & LO_FUSED_ACT_GELU) != 0;
  const bool unfused = plan.unfused;
  if (plan.try_decode) {
    // (cache3 is the front of the caller's cache13: the path keeps its bf16 activations [S, I] there)
    const int rc2 = launch_decode_path(x, M, H, I, E, num_experts, top_k, w1, w1s, w2, w2s, topk_w, topk_ids, ids_dtype,
                                       expert_map, apply_router_weight_on_input, routed_scaling_factor, shared_output,
                                       cache3, out, (flags & LO_FUSED_FORCE_DECODE_PATH) != 0, (flags & LO_GEMM_W4) != 0,
                                       flags, static_cast<hipStream_t>(stream));
    if (rc2 != LO_ENOTSUP) return rc2;
  }

  // the quantisation rides in the alignment's launch (bf16 rows)
  int rc = dtype != LO_BF16 ? LO_ENOTSUP
                            : launch_quant_align(x, M, H, 1e-10f, a1q, a1s, topk_ids, ids_dtype, S, num_experts,
                                                 block_size_m, expert_map, sorted, L.sorted_cap, eids, L.blocks_cap,
                                                 ntpp, mask, ws + L.off[8], L.align_scratch,
                                                 static_cast<hipStream_t>(stream));
  if (rc == LO_ENOTSUP) {
    rc = lo_per_token_group_quant_int8(x, dtype, M, H, 1e-10f, a1q, a1s, stream);
    if (rc) return rc;
    rc = lo_moe_align_block_size_ws(topk_ids, ids_dtype, S, num_experts, block_size_m, expert_map, 0,
                                    sorted, L.sorted_cap, eids, L.blocks_cap, ntpp, mask, ws + L.off[8],
                                    L.align_scratch, stream);
  }
  if (rc) return rc;
  if (unfused) {
    // rows of slots whose expert another rank holds are neither written by the first GEMM nor read by
    // the activation launch (the slot mask of the alignment says which)
    rc = lo_moe_gemm_block_int8(a1q, a1s, w1, w1s, cache3, dtype, topk_w, sorted, eids, ntpp, L.sorted_cap, S, M, E,
                                num_experts, 2 * I, H, top_k, block_size_m, apply_router_weight_on_input,
                                (flags & ~LO_FUSED_ACT_GELU) | (mask ? LO_GEMM_SKIP_NONLOCAL : 0), stream);
    if (rc) return rc;
    rc = launch_act_mul_group_quant(cache3, dtype, gelu ? LO_ACT_GELU : LO_ACT_SILU, S, I, a2q, a2s, mask,
                                    static_cast<hipStream_t>(stream));
  } else {
    rc = lo_moe_gemm1_silu_quant_block_int8(a1q, a1s, w1, w1s, a2q, a2s, dtype, topk_w, sorted, eids,
                                            ntpp, L.sorted_cap, S, M, E, num_experts, I, H, top_k, block_size_m,
                                            apply_router_weight_on_input, flags, stream);
  }
  if (rc) return rc;
  rc = lo_moe_gemm_block_int8(a2q, a2s, w2, w2s, cache3, dtype, topk_w, sorted, eids, ntpp,
                              L.sorted_cap, S, S, E, num_experts, H, I, 1, block_size_m,
                              !apply_router_weight_on_input,
                              (flags & ~LO_FUSED_ACT_GELU) | (mask ? LO_GEMM_SKIP_NONLOCAL : 0), stream);
  if (rc) return rc;
  return lo_moe_sum(cache3, out, shared_output, mask, dtype, M, top_k, H, routed_scaling_factor,
                    nullptr, stream);
}

// The per-channel form of the same chain (int8.py:703-888 with per_channel_quant=True,
// block_shape=None): per-token quant -> align -> moe_gemm_w8a8 -> fuse_silu_mul_quant ->
// moe_gemm_w8a8 (routed weight in its epilogue) -> moe_sum.  cache13 holds the first GEMM's
// output [S, 2I] and then the second's [S, H], as in the reference (int8.py:681-682).
// x_q / x_s: the activations already quantised per token by the caller (the i_q / i_s of int8.py:291-293,
// LMSLIM_USE_FUSED_RMS_QUANT); then x is not read and the quantisation launch is left out.
static int fused_experts_channel(
    const void *x, const int8_t *x_q, const float *x_s, int dtype, int64_t M, int64_t H, int64_t I, int32_t E,
    int32_t num_experts, int32_t top_k, const int8_t *w1, const float *w1s, const int8_t *w2, const float *w2s,
    const float *topk_w, const void *topk_ids, int ids_dtype, const int32_t *expert_map,
    int apply_router_weight_on_input, float routed_scaling_factor, const void *shared_output,
    void *cache13, void *out, void *workspace, int64_t workspace_bytes, int32_t block_size_m,
    int flags, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE((x || (x_q && x_s)) && w1 && w1s && w2 && w2s && topk_w && topk_ids && cache13 && out && workspace,
             LO_EINVAL, "fused_experts(channel): null pointer");
  LO_REQUIRE(dtype == LO_BF16 || dtype == LO_F16, LO_ENOTSUP, "fused_experts(channel): activations are bf16 or fp16");
  LO_REQUIRE(M >= 0 && H >= kGroup && H % kGroup == 0 && I >= kGroup && I % kGroup == 0, LO_EINVAL,
             "fused_experts(channel): hidden (%lld) and intermediate (%lld) sizes must be multiples of 128",
             (long long)H, (long long)I);
  LO_REQUIRE(E >= 1 && num_experts >= E && top_k >= 1, LO_EINVAL, "fused_experts(channel): bad expert counts");
  LO_REQUIRE(num_experts == E || expert_map, LO_EINVAL,
             "fused_experts(channel): global_num_experts (%d) != local experts (%d) needs an expert_map",
             num_experts, E);
  LO_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, LO_EINVAL,
             "fused_experts(channel): workspace must be 256-byte aligned");
  if (M == 0) return LO_OK;
  if (block_size_m == 0)
    block_size_m = pick_block_m(M, num_experts, top_k, H, I, LO_FORM_CHANNEL, true, (flags & LO_GEMM_W4) != 0,
                                (flags & (LO_GEMM_W4 | LO_GEMM_W_PRESHUFFLED)) && H / kGroup <= 128 &&
                                    I / kGroup <= 128);
  // 160: the 160-token form of the direct-to-LDS kernel (weights in the load-time layout)
  const bool bs160 = block_size_m == 160 && (flags & (LO_GEMM_W4 | LO_GEMM_W_PRESHUFFLED)) && H / kGroup <= 128 &&
                     I / kGroup <= 128;
  LO_REQUIRE(block_size_m == 16 || block_size_m == 32 || block_size_m == 64 || block_size_m == 128 || bs160,
             LO_EINVAL,
             "fused_experts(channel): block_size_m %d is not one of 16, 32, 64, 128 (160: weights in the load-time "
             "layout)", block_size_m);
  // the block layout is roomy enough: its scale segments hold one float per 128 values
  const WsLayout L = ws_layout(M, top_k, H, I, num_experts, block_size_m);
  LO_REQUIRE(workspace_bytes >= L.total, LO_ENOSPC,
             "fused_experts(channel): workspace holds %lld bytes, needs %lld", (long long)workspace_bytes,
             (long long)L.total);
  char *ws = static_cast<char *>(workspace);
  const int8_t *a1q = x_q ? x_q : reinterpret_cast<int8_t *>(ws + L.off[0]);
  const float *a1s = x_q ? x_s : reinterpret_cast<float *>(ws + L.off[1]);
  int32_t *sorted = reinterpret_cast<int32_t *>(ws + L.off[2]);
  int32_t *eids = reinterpret_cast<int32_t *>(ws + L.off[3]);
  int32_t *ntpp = reinterpret_cast<int32_t *>(ws + L.off[4]);
  int8_t *a2q = reinterpret_cast<int8_t *>(ws + L.off[5]);
  float *a2s = reinterpret_cast<float *>(ws + L.off[6]);
  uint8_t *mask = expert_map ? reinterpret_cast<uint8_t *>(ws + L.off[7]) : nullptr;
  const int64_t S = M * top_k;

  int rc = LO_OK;
  if (!x_q)
    rc = lo_per_token_quant_int8(x, dtype, M, H, reinterpret_cast<int8_t *>(ws + L.off[0]),
                                 reinterpret_cast<float *>(ws + L.off[1]), stream);
  if (rc) return rc;
  rc = lo_moe_align_block_size_ws(topk_ids, ids_dtype, S, num_experts, block_size_m, expert_map, 0,
                                  sorted, L.sorted_cap, eids, L.blocks_cap, ntpp, mask, ws + L.off[8],
                                  L.align_scratch, stream);
  if (rc) return rc;
  // rows of experts on other ranks are zero-filled here: the activation kernel reads every row
  const int gflags = flags & ~LO_FUSED_ACT_GELU;
  rc = lo_moe_gemm_w8a8(a1q, a1s, w1, w1s, cache13, dtype, topk_w, sorted, eids, ntpp, L.sorted_cap, S, M, E,
                        num_experts, 2 * I, H, top_k, block_size_m, apply_router_weight_on_input, gflags, stream);
  if (rc) return rc;
  if (flags & LO_FUSED_ACT_GELU) // gelu_and_mul, then per_token_quant_int8 with its floor (int8.py:826-838)
    rc = launch_act_mul_row_quant(cache13, dtype, LO_ACT_GELU, S, I, a2q, a2s, nullptr, 1, nullptr,
                                  static_cast<hipStream_t>(stream));
  else
    rc = lo_fuse_silu_mul_quant(cache13, dtype, S, I, a2q, a2s, nullptr, 1, stream);
  if (rc) return rc;
  rc = lo_moe_gemm_w8a8(a2q, a2s, w2, w2s, cache13, dtype, topk_w, sorted, eids, ntpp, L.sorted_cap, S, S, E,
                        num_experts, H, I, 1, block_size_m, !apply_router_weight_on_input,
                        gflags | (mask ? LO_GEMM_SKIP_NONLOCAL : 0), stream);
  if (rc) return rc;
  return lo_moe_sum(cache13, out, shared_output, mask, dtype, M, top_k, H, routed_scaling_factor, nullptr,
                    stream);
}

extern "C" int lo_fused_experts_channel_int8(
    const void *x, int dtype, int64_t M, int64_t H, int64_t I, int32_t E, int32_t num_experts,
    int32_t top_k, const int8_t *w1, const float *w1s, const int8_t *w2, const float *w2s,
    const float *topk_w, const void *topk_ids, int ids_dtype, const int32_t *expert_map,
    int apply_router_weight_on_input, float routed_scaling_factor, const void *shared_output,
    void *cache13, void *out, void *workspace, int64_t workspace_bytes, int32_t block_size_m,
    int flags, lo_stream_t stream) {
  LO_REQUIRE(x, LO_EINVAL, "fused_experts(channel): null pointer");
  return fused_experts_channel(x, nullptr, nullptr, dtype, M, H, I, E, num_experts, top_k, w1, w1s, w2, w2s, topk_w,
                               topk_ids, ids_dtype, expert_map, apply_router_weight_on_input, routed_scaling_factor,
                               shared_output, cache13, out, workspace, workspace_bytes, block_size_m, flags, stream);
}

extern "C" int lo_fused_experts_channel_int8_prequant(
    const int8_t *x_q, const float *x_s, int dtype, int64_t M, int64_t H, int64_t I, int32_t E, int32_t num_experts,
    int32_t top_k, const int8_t *w1, const float *w1s, const int8_t *w2, const float *w2s,
    const float *topk_w, const void *topk_ids, int ids_dtype, const int32_t *expert_map,
    int apply_router_weight_on_input, float routed_scaling_factor, const void *shared_output,
    void *cache13, void *out, void *workspace, int64_t workspace_bytes, int32_t block_size_m,
    int flags, lo_stream_t stream) {
  LO_REQUIRE(x_q && x_s, LO_EINVAL, "fused_experts(channel, quantised input): null pointer");
  return fused_experts_channel(nullptr, x_q, x_s, dtype, M, H, I, E, num_experts, top_k, w1, w1s, w2, w2s, topk_w,
                               topk_ids, ids_dtype, expert_map, apply_router_weight_on_input, routed_scaling_factor,
                               shared_output, cache13, out, workspace, workspace_bytes, block_size_m, flags, stream);
}

// ---- whole path for callers that cannot allocate -------------------------------------------
// The scratch of the whole-path call (quantised activations, alignment buffers, slot mask) in a
// device array that is part of the library's image instead of a caller workspace.  Every GPU the
// library runs on holds its own copy at its own address for the life of the process; the address
// is looked up once per device and only that pointer is ever handed to kernels.
namespace lo {

constexpr int64_t kScratchBytes = LO_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

static std::mutex g_scratch_mutex;
static void *g_scratch_ptr[64] = {};

// Device address of `scratch` on the current device.
static int static_scratch(void **out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    set_error("static scratch: no current HIP device");
    return LO_ELAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      set_error("static scratch: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
      return LO_ELAUNCH;
    }
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return LO_OK;
}

} // namespace lo

extern "C" int lo_init(lo_stream_t stream) {
  const uint16_t *t = nullptr;
  int rc = lo::silu_table(static_cast<hipStream_t>(stream), &t);
  if (rc) return rc;
  void *p = nullptr;
  return lo::static_scratch(&p);
}

extern "C" int lo_fused_experts_block_int8_noalloc(
    const void *x, int dtype, int64_t M, int64_t H, int64_t I, int32_t E, int32_t num_experts,
    int32_t top_k, const int8_t *w1, const float *w1s, const int8_t *w2, const float *w2s,
    const float *topk_w, const void *topk_ids, int ids_dtype, const int32_t *expert_map,
    int apply_router_weight_on_input, float routed_scaling_factor, const void *shared_output,
    void *cache3, void *out, int32_t block_size_m, int flags, lo_stream_t stream) {
  using namespace lo;
  LO_REQUIRE(M >= 0 && top_k >= 1 && H >= kGroup && I >= kGroup && num_experts >= 1, LO_EINVAL,
             "fused_experts(noalloc): bad problem size");
  LO_REQUIRE(dtype == LO_BF16 || dtype == LO_F16 || (dtype == LO_F32 && !(flags & LO_GEMM_W4)), LO_ENOTSUP,
             "fused_experts(noalloc): activations are bf16, fp16 or (int8 weights) fp32");
  // the block size the workspace form will resolve to (same function, same arguments), for the space check
  BlockPlan plan;
  const int rc_plan = plan_block_path(dtype, flags, M, num_experts, top_k, H, I, block_size_m, &plan);
  if (rc_plan) return rc_plan;
  const int32_t block_size_m_arg = block_size_m;
  block_size_m = plan.block_size_m;
  const int64_t need = ws_layout(M, top_k, H, I, num_experts, block_size_m).total;
  LO_REQUIRE(need <= kScratchBytes, LO_ENOSPC,
             "fused_experts(noalloc): this problem needs %lld bytes of scratch, the built-in scratch holds %lld; "
             "use lo_fused_experts_block_int8 with a caller workspace",
             (long long)need, (long long)kScratchBytes);
  void *ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc) return rc;
  // Nothing in the scratch has to start at zero: every segment is written before it is read
  // (padding values, expert ids past the last block and the alignment's counters included).
  return lo_fused_experts_block_int8(x, dtype, M, H, I, E, num_experts, top_k, w1, w1s, w2, w2s, topk_w, topk_ids,
                                     ids_dtype, expert_map, apply_router_weight_on_input, routed_scaling_factor,
                                     shared_output, cache3, out, ws, kScratchBytes, block_size_m_arg, flags, stream);
}
