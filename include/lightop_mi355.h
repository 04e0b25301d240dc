/*
 * lightop_mi355 - C ABI of the block-INT8 fused-MoE path for AMD Instinct MI355X (gfx950).
 *
 * Every entry point takes raw device pointers, extents and a HIP stream, launches
 * on that stream, never synchronises, never reads device results on the host and
 * never allocates.  Return value: 0 on success, a negative LO_E* code otherwise;
 * lo_last_error() returns a thread-local description of the last failure.
 *
 * Each function names the reference interface it replaces (paths relative to the
 * HYGON-AI/lightop tree).
 */
#ifndef LIGHTOP_MI355_H
#define LIGHTOP_MI355_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *lo_stream_t; /* hipStream_t */

enum {
  LO_OK = 0,
  LO_EINVAL = -1,   /* bad shape, alignment, dtype or null pointer */
  LO_ENOSPC = -2,   /* caller buffer / workspace too small */
  LO_ELAUNCH = -3,  /* hipGetLastError() after a launch */
  LO_ENOTSUP = -4   /* valid request that this build has no kernel for */
};

/* activation element types.  fp16 rows go the same way as bf16 ones except that no kernel fuses the gated
 * activation for them: the first GEMM writes [S, 2I] in fp16 and one launch applies the activation and
 * quantises (as with LO_FUSED_ACT_GELU), and the two-launch path is not taken.  LO_F32 (besides router
 * inputs): the block form with int8 weights and its stages (lo_per_token_group_quant_int8,
 * lo_moe_gemm_block_int8, lo_silu_and_mul, lo_gelu_and_mul, lo_act_mul_group_quant, lo_moe_sum); nothing
 * between the stages is rounded to 16 bits then (compute_type tl.float32, int8.py:689-696), and the GEMMs
 * are the weight-streaming kernel at every size. */
enum { LO_BF16 = 0, LO_F16 = 1, LO_F32 = 2 };
/* gated activations */
enum { LO_ACT_SILU = 0, LO_ACT_GELU = 1 };
/* index element types of topk_ids */
enum { LO_I32 = 0, LO_I64 = 1 };

/* flags of lo_moe_gemm_block_int8 / lo_fused_experts_block_int8 */
enum {
  /* Per 128-wide K block every kernel accumulates acc = fma(f32(d) * a_s, b_s, acc) (d: the block's
   * exact int32 sum): the order the reference's Triton line
   *   accumulator += tl.dot(a, b) * a_scale[:, None] * b_scale[None, :]
   * (python/lightop/_lmslim_native/layers/fused_moe/int8.py:499-508) compiles to under the AMD
   * backend's default enable_fp_fusion. */
  LO_GEMM_DEFAULT = 0,
  /* accumulate acc = fma(f32(d), a_s * b_s, acc) instead.  The int32 partial sums are identical; the
   * fp32 rounding differs in the last ulp, so outputs (and the re-quantised int8 activations
   * between the GEMMs) are no longer bit-identical to the default ones, only within the path's
   * tolerance.  Two vector instructions per accumulator element and K block instead of three. */
  LO_GEMM_FUSED_SCALE = 1,
  /* always use the weight-streaming kernels, also where the LDS-tiled kernel applies */
  LO_GEMM_FORCE_STREAMING = 2,
  /* accumulate acc = acc + (f32(d) * a_s) * b_s, every operation rounded on its own: the same
   * reference line compiled without fp fusion (four vector instructions).  Wins over
   * LO_GEMM_FUSED_SCALE. */
  LO_GEMM_SEPARATE_ORDER = 4,
  /* W (for the whole path: w1 and w2) is in the layout of lo_preshuffle_weight_int8 */
  LO_GEMM_W_PRESHUFFLED = 8,
  /* leave the output rows of blocks whose expert id is -1 untouched instead of zeroing
   * them (the caller then reduces with an expert_mask, see lo_moe_sum) */
  LO_GEMM_SKIP_NONLOCAL = 16,
  /* W4A8 with K-group scales (the benchmark's int4 variant): W (w1 and w2 for the whole path) is
   * packed signed int4 in the layout of lo_preshuffle_weight_int4 (LO_GEMM_W_PRESHUFFLED must
   * be set too) and the weight scales are one per output row and 128-wide K group, stored
   * K-group-major (transposed once at load time), Ws [E, K/128, N] instead of
   * [E, N/128, K/128]; N % 4 == 0:
   *   acc = acc + (f32(sum_k A*w) * As[row, kb]) * Ws[e, kb, n],  w in [-8, 7].
   * The reference's W4A8 (python/lightop/_lmslim_native/layers/fused_moe/w4a8.py:211-401)
   * scales per token and per channel in the epilogue instead; its nibble order (even k in
   * the high nibble, :341, :375-377) is the one lo_preshuffle_weight_int4 reads.  Served by
   * an LDS-tiled kernel at block_size_m 64 and by the weight-streaming kernels otherwise. */
  LO_GEMM_W4 = 32,
  /* whole-path calls only.  With block_size_m = 0 and weights in the load-time layout the block
   * form serves small batches (few routed slots per expert) with a two-launch path that needs no
   * alignment, no quantised copy of x and no per-slot output rows; same results bit for bit.
   * NO_DECODE_PATH: never take it.  FORCE_DECODE_PATH: take it whenever it can serve the problem
   * (at most 512 routed slots), whatever the size heuristic says. */
  LO_FUSED_NO_DECODE_PATH = 64,
  LO_FUSED_FORCE_DECODE_PATH = 128,
  /* whole-path calls only: activation="gelu" (int8.py:825-838, w4a8.py:602-605) instead of SiLU.
   * No fused epilogue exists for it: the first GEMM writes bf16 [S, 2I], one launch applies
   * GELU-and-mul and quantises, so cache3 / cache13 must hold S * max(2I, H) elements. */
  LO_FUSED_ACT_GELU = 256
};

int lo_version(void);
const char *lo_last_error(void);

/*
 * Optional one-time set-up for the current device: builds the 128 KB bf16 SiLU table
 * that the fused GEMM epilogue looks activations up in and looks up the address of the
 * built-in scratch of lo_fused_experts_block_int8_noalloc.  The first fused-GEMM call on a
 * device does this by itself (and synchronises the stream once); call lo_init() first
 * when that first call would fall inside a HIP graph capture.  No counterpart in the
 * reference.
 */
int lo_init(lo_stream_t stream);

/*
 * Routing alignment.
 * Replaces op.moe_align_block_size (csrc/pybind/export.cpp:1593-1605,
 * csrc/kernels/moe_align_sum_kernels.cu:1210-1314) together with the
 * expert_map post-mapping of python/lightop/_lmslim_native/vllm_compat/
 * moe_align_block_size.py:117-118.
 *
 *   topk_ids      [numel] int32 or int64 (ids_dtype = LO_I32 / LO_I64), values in [0, num_experts)
 *   expert_map    [num_experts] int32 or NULL
 *   ignore_invalid 0: count on the given ids, expert_ids[b] = expert_map[e] (or e)
 *                  1: drop ids whose expert_map entry is -1, count on mapped ids
 *   sorted_ids    [sorted_cap] int32  - slot ids grouped by expert, ascending inside an
 *                                       expert, every other entry = numel
 *   expert_ids    [expert_ids_cap] int32 - expert of each block, -1 past the last block
 *   num_tokens_post_pad [1] int32
 * sorted_cap must be >= numel + num_experts*(block_size-1) or numel*block_size,
 * whichever is smaller; expert_ids_cap >= ceil(sorted_cap / block_size).
 */
int lo_moe_align_block_size(const void *topk_ids, int ids_dtype, int64_t numel,
                            int32_t num_experts, int32_t block_size,
                            const int32_t *expert_map, int ignore_invalid,
                            int32_t *sorted_ids, int64_t sorted_cap,
                            int32_t *expert_ids, int64_t expert_ids_cap,
                            int32_t *num_tokens_post_pad, lo_stream_t stream);

/*
 * Same, and additionally writes slot_mask[numel] (one byte per slot): 1 if the slot's
 * expert is held by this rank (expert_map[id] >= 0, or no map), else 0 - the
 * expert_mask that lo_moe_sum takes.
 */
int lo_moe_align_block_size_mask(const void *topk_ids, int ids_dtype, int64_t numel,
                                 int32_t num_experts, int32_t block_size,
                                 const int32_t *expert_map, int ignore_invalid,
                                 int32_t *sorted_ids, int64_t sorted_cap,
                                 int32_t *expert_ids, int64_t expert_ids_cap,
                                 int32_t *num_tokens_post_pad, uint8_t *slot_mask,
                                 lo_stream_t stream);

/*
 * Same again with a scratch buffer that lets large inputs (numel >= 8192) be aligned by
 * many workgroups instead of one: lo_moe_align_scratch_bytes(numel, num_experts) bytes of
 * device memory, 4-byte aligned, contents irrelevant (0 = no scratch needed).  Without
 * scratch the single-workgroup kernel runs; the result is identical.  The reference's
 * large-input kernels allocate a zeroed tensor themselves
 * (csrc/kernels/moe_align_sum_kernels.cu:1175).
 */
int64_t lo_moe_align_scratch_bytes(int64_t numel, int32_t num_experts);
int lo_moe_align_block_size_ws(const void *topk_ids, int ids_dtype, int64_t numel,
                               int32_t num_experts, int32_t block_size,
                               const int32_t *expert_map, int ignore_invalid,
                               int32_t *sorted_ids, int64_t sorted_cap,
                               int32_t *expert_ids, int64_t expert_ids_cap,
                               int32_t *num_tokens_post_pad, uint8_t *slot_mask,
                               void *scratch, int64_t scratch_bytes, lo_stream_t stream);

/*
 * Same again for batches padded to a fixed size: num_local_tokens is a device int32[1] (or
 * NULL) and only the slots of the first num_local_tokens[0] tokens (top_k slots each) are
 * counted and sorted; the pad value stays numel, slot_mask is 0 for the padding tokens'
 * slots (the num_local_tokens argument of op.moe_align_block_size,
 * csrc/pybind/export.cpp:1593-1605, csrc/kernels/moe_align_sum_kernels.cu:32-45).  With a
 * count of 0 the reference returns without writing anything; here num_tokens_post_pad is
 * written as 0 and the buffers are filled with their pad values, so that the GEMMs skip
 * every block.
 */
int lo_moe_align_block_size_local(const void *topk_ids, int ids_dtype, int64_t numel,
                                  int32_t num_experts, int32_t block_size,
                                  const int32_t *expert_map, int ignore_invalid,
                                  int32_t *sorted_ids, int64_t sorted_cap,
                                  int32_t *expert_ids, int64_t expert_ids_cap,
                                  int32_t *num_tokens_post_pad, uint8_t *slot_mask,
                                  void *scratch, int64_t scratch_bytes,
                                  const int32_t *num_local_tokens, int32_t top_k,
                                  lo_stream_t stream);

/*
 * 1x128 group quantisation of activations to int8 with fp32 scales.
 * Replaces per_token_group_quant_int8 (python/lightop/_lmslim_native/layers/gemm/
 * int8_utils.py:125-195, Triton kernel :74-122).
 *   x [rows, cols] contiguous, cols % 128 == 0;  q [rows, cols] int8;  s [rows, cols/128] f32
 *   amax = max(max|x|, eps); s = amax / 127; q = trunc(clamp(x / s, -128, 127))
 */
int lo_per_token_group_quant_int8(const void *x, int x_dtype, int64_t rows, int64_t cols,
                                  float eps, int8_t *q, float *s, lo_stream_t stream);

/*
 * One grouped GEMM stage over the aligned routing.
 * Replaces invoke_fused_moe_kernel_int8 / Triton fused_moe_kernel
 * (python/lightop/_lmslim_native/layers/fused_moe/int8.py:543-626, :320-541) for
 * use_int8_w8a8=True, block_shape=[128,128].
 *
 *   A  [a_rows, K] int8;  As [a_rows, K/128] f32;  the row of slot f is f / top_k
 *   W  [E, N, K] int8 (K contiguous);  Ws [E, ceil(N/128), K/128] f32
 *   C  [num_valid, N] c_dtype, row f;  rows of blocks whose expert id is -1 are zeroed
 *   topk_w [num_valid] f32, used when mul_routed != 0
 *   sorted_ids / expert_ids / num_tokens_post_pad as produced by lo_moe_align_block_size
 *   with block_size == block_size_m (16, 32, 64 or 128; also 160 with int8 weights in the load-time
 *   layout, N % 64 == 0 and K <= 16384); sorted_cap is the extent of sorted_ids
 *   (any extent >= the alignment's own works, e.g. one rounded up by the caller), and expert_ids
 *   holds at least sorted_cap / block_size_m entries: a kernel may read the entry and the sorted ids of
 *   any block below that bound before it knows num_tokens_post_pad (it uses them only for blocks in use).
 *   E: experts held by W.  num_experts: experts the routing spreads the slots over (the
 *   num_experts given to the alignment; 0 = E).  It only steers scheduling choices (tile order,
 *   cache hints), never the result.
 * K % 128 == 0, N % 16 == 0; A, W and C 16-byte aligned.
 */
int lo_moe_gemm_block_int8(const int8_t *A, const float *As, const int8_t *W, const float *Ws,
                           void *C, int c_dtype, const float *topk_w, const int32_t *sorted_ids,
                           const int32_t *expert_ids, const int32_t *num_tokens_post_pad,
                           int64_t sorted_cap, int64_t num_valid, int64_t a_rows, int32_t E,
                           int32_t num_experts, int64_t N, int64_t K, int32_t top_k,
                           int32_t block_size_m, int mul_routed, int flags, lo_stream_t stream);

/*
 * First grouped GEMM with the activation fused into its epilogue:
 * GEMM1 -> bf16 round -> SiLU(gate) * up -> 1x128 group quant, i.e. the sequence
 * int8.py:784-823 without materialising intermediate_cache1 / intermediate_cache2.
 *   W [E, 2I, K] (gate rows first, then up rows), Ws [E, 2I/128, K/128]
 *   A2q [num_valid, I] int8, A2s [num_valid, I/128] f32 (rows of -1 blocks untouched)
 * I % 128 == 0, K % 128 == 0; A, W and A2q 16-byte aligned.  block_size_m: 16, 32, 64, 128, or 160 with
 * int8 weights in the load-time layout and K <= 16384.
 */
int lo_moe_gemm1_silu_quant_block_int8(const int8_t *A, const float *As, const int8_t *W,
                                       const float *Ws, int8_t *A2q, float *A2s, int c_dtype,
                                       const float *topk_w, const int32_t *sorted_ids,
                                       const int32_t *expert_ids,
                                       const int32_t *num_tokens_post_pad, int64_t sorted_cap,
                                       int64_t num_valid, int64_t a_rows, int32_t E,
                                       int32_t num_experts, int64_t I, int64_t K, int32_t top_k,
                                       int32_t block_size_m, int mul_routed, int flags,
                                       lo_stream_t stream);

/*
 * SiLU-and-mul: act[f, i] = T( T(silu(c1[f, i])) * c1[f, I + i] ).
 * Replaces torch.ops._C.silu_and_mul at int8.py:811 (in-repo twin:
 * csrc/kernels/gated_activation/fuse_silu_mul_quant.cu:893-905).
 */
int lo_silu_and_mul(const void *c1, int dtype, int64_t rows, int64_t I, void *act,
                    lo_stream_t stream);

/*
 * GELU-and-mul, erf form: act[f, i] = T( T(gelu(c1[f, i])) * c1[f, I + i] ),
 * gelu(x) = (x * 0.5f) * (1.0f + erf(x * float(M_SQRT1_2))) in fp32 with erf correctly rounded.
 * Replaces torch.ops._C.gelu_and_mul at int8.py:826 (in-repo twin: gelu_and_mul_opt,
 * csrc/kernels/activation_kernels_opt.cu:234-242, :159-161, :319-323).
 */
int lo_gelu_and_mul(const void *c1, int dtype, int64_t rows, int64_t I, void *act,
                    lo_stream_t stream);
/*
 * The gated activation followed by the 1x128 group quantisation in one pass: c1 [rows, 2I] ->
 * q [rows, I] int8, s [rows, I/128] f32.  Replaces the pair of calls between the two GEMMs where the
 * first GEMM's epilogue does not do it: silu_and_mul + per_token_group_quant_int8 (int8.py:811-823) or
 * gelu_and_mul + per_token_group_quant_int8 (int8.py:826-838).  activation: LO_ACT_SILU / LO_ACT_GELU.
 * row_mask (may be NULL): one byte per row as lo_moe_align_block_size_mask writes it; rows whose byte
 * is 0 (slots of experts on other ranks) are neither read nor written.
 */
int lo_act_mul_group_quant(const void *c1, int dtype, int activation, int64_t rows, int64_t I, int8_t *q,
                           float *s, const uint8_t *row_mask, lo_stream_t stream);
/* The 65536 values T(act(g)), indexed by the bit pattern of g, that the kernels look up for activation
 * LO_ACT_SILU / LO_ACT_GELU and element type LO_BF16 / LO_F16, copied to table_out (device memory,
 * 128 KB).  For tests; no counterpart in the reference. */
int lo_activation_table(int activation, int dtype, void *table_out, lo_stream_t stream);

/*
 * Top-k reduction back to token order: out[t, :] = factor * sum_j in[t, j, :] (+ bias[t, :]).
 * Replaces op.moe_sum (csrc/pybind/export.cpp:1584-1592,
 * csrc/kernels/moe_align_sum_kernels.cu:1315-2092).  fp32 accumulation in slot
 * order; without bias one rounding (:619-633), with bias the three roundings of :886-909.
 * expert_mask [M*topk] bytes or NULL: slots whose byte is 0 are not read and add nothing
 * (the expert_mask argument of the reference op, :661-672).
 * num_local_tokens: device int32[1] or NULL; rows t >= num_local_tokens[0] (padding tokens of
 * a fixed-size batch) are left untouched (:644-649, :735-741; one of the reference's
 * variants tests t > n and so also writes row n).
 */
int lo_moe_sum(const void *in, void *out, const void *bias, const uint8_t *expert_mask, int dtype,
               int64_t M, int32_t topk, int64_t H, float factor, const int32_t *num_local_tokens,
               lo_stream_t stream);

/*
 * Load-time layout of packed int4 weights for LO_GEMM_W4: src [E, N, K/2] bytes, element k of
 * a row in byte k/2, even k in the high nibble; dst the same number of bytes, blocks of
 * 16 rows x 128 K (1 KB) ordered [E][K/128][N/16].  N % 16 == 0, K % 128 == 0; src != dst.
 * No counterpart in the reference (its Triton kernel reads the row-major packed tensor).
 */
int lo_preshuffle_weight_int4(const uint8_t *src, uint8_t *dst, int32_t E, int64_t N, int64_t K,
                              lo_stream_t stream);

/*
 * Load-time weight layout for the GEMM kernels: every block of 16 rows x 128 K-bytes of
 * W [E, N, K] is stored as [8 chunks of 16 K-bytes][16 rows][16 bytes], blocks ordered
 * [E][K/128][N/16].  Same size as the source; N % 16 == 0, K % 128 == 0; src != dst.
 * No counterpart on the reference's block-INT8 path (its Triton kernel reads row-major
 * weights); comparable to the load-time shuffle of its native kernels,
 * test/moe_w8a8/w8a8_quant.py:66-111.
 */
int lo_preshuffle_weight_int8(const int8_t *src, int8_t *dst, int32_t E, int64_t N, int64_t K,
                              lo_stream_t stream);

/*
 * Tile table: block_size_m (the alignment block and GEMM token tile) chosen for a
 * problem.  Replaces get_w8a8moe_json / W8a8GetCacheJSON (int8.py:220-256,
 * vllm_compat/w8a8_get_cache_json.py:12-174) and the per-device JSON files
 * configs/w8a8/MOE_BLOCKINT8[128,128]_*.json.
 */
typedef struct lo_moe_tile {
  int32_t block_size_m; /* 16, 32, 64, 128 or 160 (160: int8 weights in the load-time layout; bf16 rows with
                         * SiLU keep the fused first stage, fp16 rows and GELU take the plain stage
                         * followed by lo_act_mul_group_quant, as they do with every block size) */
  int32_t kernel;       /* LO_KERNEL_*: the kernel the stage entry points launch for this problem */
  int32_t waves;        /* wavefronts per workgroup of that kernel */
  int32_t block_n;      /* weight rows per workgroup of that kernel */
} lo_moe_tile;

/* kernel families (lo_moe_tile.kernel) */
enum {
  LO_KERNEL_WS = 0,      /* weight-streaming, no LDS in the K loop (token blocks of 16 / 32) */
  LO_KERNEL_TILE = 1,    /* LDS-tiled, weights register-fed (row-major weights, 64 / 128 tokens) */
  LO_KERNEL_PC = 2,      /* per-channel LDS-tiled */
  LO_KERNEL_AS = 3,      /* activation-stationary second GEMM (short K) */
  LO_KERNEL_T128 = 4,    /* 128 tokens, both operands copied global -> LDS (pre-shuffled weights) */
  LO_KERNEL_W4_TILE = 5, /* packed-int4 LDS-tiled, 64 tokens */
  LO_KERNEL_DEC = 6      /* the whole-path call's two-launch path for a few tokens (weights in the load-time
                          * layout, block_size_m = 0): 16 weight rows per workgroup, the waves of the first
                          * kernel split K, those of the second take one routed slot each.  The stage entry
                          * points have no such kernel: given the reported block_size_m they launch
                          * LO_KERNEL_WS. */
};

/* Block form with weights in the load-time layout (flags = LO_GEMM_W_PRESHUFFLED). */
int lo_moe_tile_query(int64_t M, int32_t E_local, int32_t num_experts, int32_t top_k, int64_t H,
                      int64_t I, lo_moe_tile *gemm1, lo_moe_tile *gemm2);
/* The same for every form of the path: block, per-channel (replaces get_moe_cuda_config,
 * int8.py:735-741, and its MODE / DELTA tables) and W4A8 with K-group scales.  flags: the
 * LO_GEMM_* flags the call will carry (LO_GEMM_W_PRESHUFFLED decides between the row-major
 * and the load-time weight layout, LO_GEMM_FORCE_STREAMING is honoured; LO_GEMM_W4 is implied
 * by the form).  The answer is what lo_fused_experts_* picks with block_size_m = 0 and what the
 * stage entry points launch when given that block_size_m. */
enum { LO_FORM_BLOCK = 0, LO_FORM_CHANNEL = 1, LO_FORM_W4 = 2 };
int lo_moe_tile_query_form(int form, int flags, int64_t M, int32_t E_local, int32_t num_experts,
                           int32_t top_k, int64_t H, int64_t I, lo_moe_tile *gemm1,
                           lo_moe_tile *gemm2);
/* The same for a given element type of the activations (LO_BF16 / LO_F16 / LO_F32: 16-bit rows other than
 * bf16 and fp32 rows take other kernels) and a given block_size_m (0: the table's pick; otherwise the
 * size a caller passes to lo_fused_experts_*, e.g. one read from a tuning file as get_w8a8moe_json does,
 * vllm_compat/w8a8_get_cache_json.py:133-174).  flags may carry LO_FUSED_ACT_GELU and the decode-path
 * flags as well.  The whole-path calls resolve block size, fused / plain first stage and the two-launch
 * path through the very function this query reports from.  lo_moe_tile_query_form is this call with
 * LO_BF16 and block_size_m = 0. */
int lo_moe_tile_query_path(int form, int flags, int dtype, int32_t block_size_m, int64_t M, int32_t E_local,
                           int32_t num_experts, int32_t top_k, int64_t H, int64_t I, lo_moe_tile *gemm1,
                           lo_moe_tile *gemm2);

/*
 * Measurement aid; no counterpart in the reference.  The block-INT8 GEMMs fold each 128-wide K block's int32
 * sums into fp32 accumulators with 2, 3 or 4 vector instructions per element (LO_GEMM_FUSED_SCALE, the default
 * contracted order, LO_GEMM_SEPARATE_ORDER): 4, 6 or 8 per v_mfma_i32_16x16x64_i8, issued by the wave that
 * issues the MFMA.  This call times a loop of nothing but such MFMAs, each followed by valu_per_mfma (0, 4, 6
 * or 8) independent v_fma_f32, two waves per SIMD on every compute unit, for `iters` groups of eight MFMAs per
 * wave, on operand registers holding pseudo-random bytes (random_operands != 0) or zeros, and returns the
 * int8 operations per second (multiply and add counted separately) the device sustained: the ceiling the
 * chip's issue logic and clock management put on a K loop with that much scale arithmetic.  It allocates
 * 256 bytes for the duration of the call and waits for its own kernel.  bench.py reports the result beside
 * the dominant kernel's rate.
 */
int lo_measure_mfma_issue_rate(int valu_per_mfma, int random_operands, int iters, void *stream,
                               double *int8_ops_per_second);

/*
 * Whole path for one chunk of tokens: quant -> align -> GEMM1(+SiLU*mul+quant) -> GEMM2
 * -> weighted top-k reduce.  Replaces the body of fused_experts_impl_int8
 * (int8.py:703-888); the reduce is always performed.
 *
 *   x [M, H] bf16 or fp16 (dtype; compute_type of int8.py:689-696: every value stored between the
 *   stages, cache3 and out have that type);  w1 [E, 2I, H], w2 [E, H, I] int8;
 *   w1s [E, 2I/128, H/128], w2s [E, H/128, I/128]
 *   topk_w [M, top_k] f32;  topk_ids [M, top_k] int32/int64;  expert_map [num_experts] or NULL
 *   cache3 [M*top_k, H] act dtype: the caller's cache13 workspace (second GEMM's output); with fp16
 *   rows or LO_FUSED_ACT_GELU it also receives the first GEMM's output: [M*top_k, max(2I, H)]
 *   shared_output [M, H] or NULL;  out [M, H]
 *   workspace: lo_fused_experts_workspace_bytes(...) bytes of device memory, 256-byte aligned
 *   block_size_m: 0 = take it from the tile table (lo_fused_experts_workspace_bytes(.., 0) is
 *   large enough for whatever the table picks and for every explicit block size); 16, 32, 64, 128,
 *   or 160 (int8 weights in the load-time layout: 160-token blocks of the direct-to-LDS kernel - what
 *   the table picks around 128 slots per expert, where a 128-token block would spill into a second
 *   pass over the expert's weights; with fp16 rows or GELU the first GEMM is not fused with the
 *   activation, cache3 also receives its output [M*top_k, 2I], and 2I <= H is required)
 */
int64_t lo_fused_experts_workspace_bytes(int64_t M, int32_t top_k, int64_t H, int64_t I,
                                         int32_t num_experts, int32_t block_size_m);

int lo_fused_experts_block_int8(const void *x, int dtype, int64_t M, int64_t H, int64_t I,
                                int32_t E, int32_t num_experts, int32_t top_k, const int8_t *w1,
                                const float *w1s, const int8_t *w2, const float *w2s,
                                const float *topk_w, const void *topk_ids, int ids_dtype,
                                const int32_t *expert_map, int apply_router_weight_on_input,
                                float routed_scaling_factor, const void *shared_output,
                                void *cache3, void *out, void *workspace, int64_t workspace_bytes,
                                int32_t block_size_m, int flags, lo_stream_t stream);

/*
 * The same call for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): no workspace argument, the scratch is a
 * device array inside the library, LO_NOALLOC_SCRATCH_BYTES (32 MiB) per GPU, held until the
 * process ends.  No counterpart in the reference, whose path allocates four
 * tensors per call (int8.py:685-701, moe_align_block_size.py:87-95).  Problems whose scratch
 * (lo_fused_experts_workspace_bytes(..., block_size_m)) exceeds that size are refused with
 * LO_ENOSPC.  The function calls no allocator; lo_init() looks the array's address up
 * beforehand (otherwise the first call on a device does), and must have run before a graph
 * capture, as for every fused call.  All calls on one GPU share that GPU's array: calls that
 * overlap there (two streams, two threads) race; serialise them or use the workspace form.
 */
#define LO_NOALLOC_SCRATCH_BYTES (32ll << 20)
int lo_fused_experts_block_int8_noalloc(const void *x, int dtype, int64_t M, int64_t H, int64_t I,
                                        int32_t E, int32_t num_experts, int32_t top_k,
                                        const int8_t *w1, const float *w1s, const int8_t *w2,
                                        const float *w2s, const float *topk_w, const void *topk_ids,
                                        int ids_dtype, const int32_t *expert_map,
                                        int apply_router_weight_on_input, float routed_scaling_factor,
                                        const void *shared_output, void *cache3, void *out,
                                        int32_t block_size_m, int flags, lo_stream_t stream);

/*
 * Views into the workspace of the last layout computed for the same arguments, so
 * that tests can read every intermediate of lo_fused_experts_block_int8:
 * which = 0 a1q, 1 a1s, 2 sorted_ids, 3 expert_ids, 4 num_tokens_post_pad, 5 a2q, 6 a2s,
 * 7 slot mask.
 * Returns the byte offset inside the workspace or a negative error.
 */
int64_t lo_fused_experts_workspace_offset(int which, int64_t M, int32_t top_k, int64_t H, int64_t I,
                                          int32_t num_experts, int32_t block_size_m);

/* ---- per-channel W8A8 form of the same entry point ----------------------------------
 * fused_experts_impl_int8(per_channel_quant=True, block_shape=None): one scale per token row
 * and one per weight row, applied once after a whole-K int32 sum.
 */

/*
 * q [rows, cols] int8, s [rows] f32: amax = max(max|x|, 1e-10), s = amax / 127,
 * q = round-half-even(x * (127 / amax)).  Replaces per_token_quant_int8
 * (python/lightop/_lmslim_native/layers/gemm/int8_utils.py:20-71).  cols % 8 == 0.
 */
int lo_per_token_quant_int8(const void *x, int x_dtype, int64_t rows, int64_t cols, int8_t *q,
                            float *s, lo_stream_t stream);

/*
 * c1 [rows, 2I] -> q [rows, I] int8, s [rows] f32: act = T(T(silu(gate)) * up), amax = max|act|,
 * s = amax / 127, q = round-half-even(clamp(act * (amax == 0 ? 0 : 127 / amax))).  Replaces
 * op.fuse_silu_mul_quant(input, output, scales, num_local_tokens_tensor, topk, ...)
 * (python/lightop/fuse_silu_mul_quant.py:45-62;
 * csrc/kernels/gated_activation/fuse_silu_mul_quant.cu:90-133, :135-199).
 * num_local_tokens (device int32[1] or NULL): only the first num_local_tokens[0] * top_k rows
 * are processed.  I % 8 == 0.
 */
int lo_fuse_silu_mul_quant(const void *c1, int dtype, int64_t rows, int64_t I, int8_t *q, float *s,
                           const int32_t *num_local_tokens, int32_t top_k, lo_stream_t stream);
/* The same with the reference's expert_ids argument (fuse_silu_mul_quant.py:45-62, kernel
 * act_and_mul_quant_kernel_opt1_new, fuse_silu_mul_quant.cu:269-283, dispatch :649-705):
 * row_expert_ids [rows] int32 or NULL; a row whose entry is -1 (its expert is held by another
 * rank) is skipped, q and s of that row are left untouched. */
int lo_fuse_silu_mul_quant_ids(const void *c1, int dtype, int64_t rows, int64_t I, int8_t *q, float *s,
                               const int32_t *num_local_tokens, int32_t top_k,
                               const int32_t *row_expert_ids, lo_stream_t stream);

/*
 * One grouped-GEMM stage in the per-channel form.  Replaces
 * op.moe_gemm_w8a8(input, b_qweight, output, a_scale, b_scale, topk_weights, sorted_token_ids,
 * experts_ids, num_tokens_post_pad, top_k, mode, delta) (python/lightop/gemmopt.py:437-457;
 * csrc/moe_gemm/w8a8/moe_w8a8.cu:2389-2536; epilogues :156-166 and :445-470).
 *
 *   As [a_rows] f32, Ws [E, N] f32 (16-byte aligned, like C); everything else as lo_moe_gemm_block_int8.
 *   C[f, n] = T((f32(sum_k A*W) * ts) * Ws[e, n]),  ts = As[f / top_k], or
 *   topk_w[f] * As[f / top_k] with mul_routed;  rows of expert -1 are zero.
 *   flags: LO_GEMM_W_PRESHUFFLED, LO_GEMM_SKIP_NONLOCAL, LO_GEMM_FORCE_STREAMING, LO_GEMM_W4.
 * The reference picks a kernel by `mode`/`delta` from its tuning tables; here block_size_m
 * selects it.
 *
 * With LO_GEMM_W4 (and LO_GEMM_W_PRESHUFFLED) the stage is the reference's own int4 kernel,
 * fused_moe_kernel_int4_w4a8 (python/lightop/_lmslim_native/layers/fused_moe/w4a8.py:341-395):
 * W is the load-time layout of lo_preshuffle_weight_int4, K counts unpacked elements, every
 * nibble enters the sum as int8(nibble << 4), i.e. 16 times the signed int4, and
 *   C[f, n] = T(((f32(sum_k A*w16) [* topk_w[f]]) * As[f / top_k]) * Ws[e, n]).
 * With weights in the load-time layout (LO_GEMM_W_PRESHUFFLED; int8 or int4) block_size_m may also
 * be 160 (N % 64 == 0, K <= 16384): 160-token blocks of the direct-to-LDS kernel with the int32 sums
 * of the whole K in its accumulators, for layers whose experts see a few tokens more than 128.
 */
int lo_moe_gemm_w8a8(const int8_t *A, const float *As, const int8_t *W, const float *Ws, void *C,
                     int c_dtype, const float *topk_w, const int32_t *sorted_ids,
                     const int32_t *expert_ids, const int32_t *num_tokens_post_pad,
                     int64_t sorted_cap, int64_t num_valid, int64_t a_rows, int32_t E,
                     int32_t num_experts, int64_t N, int64_t K, int32_t top_k, int32_t block_size_m,
                     int mul_routed, int flags, lo_stream_t stream);

/*
 * Whole path in the per-channel form: per-token quant -> align -> GEMM1 -> SiLU*mul + per-token
 * quant -> GEMM2 -> weighted top-k reduce (the per-channel branch of int8.py:703-888; the reduce
 * is always performed).  Arguments as lo_fused_experts_block_int8 except:
 *   w1s [E, 2I], w2s [E, H] f32;
 *   cache13 [M*top_k, max(2I, H)] act dtype: holds the first GEMM's output, then the second's
 *   (the reference shares the buffer the same way, int8.py:681-682).
 * The workspace is the one of lo_fused_experts_workspace_bytes.
 * flags LO_GEMM_W4 | LO_GEMM_W_PRESHUFFLED: both stages are the int4 kernel described at
 * lo_moe_gemm_w8a8, which makes the call the reference's fused_experts_impl_w4a8 (w4a8.py:480-658)
 * with w1 [E, 2I, H/2] and w2 [E, H, I/2] in the layout of lo_preshuffle_weight_int4.
 * With weights in the load-time layout (either kind) block_size_m may also be 160 (H, I <= 16384),
 * which the tile table picks around 128 slots per expert.
 */
int lo_fused_experts_channel_int8(const void *x, int dtype, int64_t M, int64_t H, int64_t I,
                                  int32_t E, int32_t num_experts, int32_t top_k, const int8_t *w1,
                                  const float *w1s, const int8_t *w2, const float *w2s,
                                  const float *topk_w, const void *topk_ids, int ids_dtype,
                                  const int32_t *expert_map, int apply_router_weight_on_input,
                                  float routed_scaling_factor, const void *shared_output,
                                  void *cache13, void *out, void *workspace, int64_t workspace_bytes,
                                  int32_t block_size_m, int flags, lo_stream_t stream);

/*
 * The same with the activations already quantised per token by the caller: the i_q / i_s arguments of
 * fused_experts_impl_int8 (int8.py:652-653), which moe_kernel_prepare_input takes in place of
 * per_token_quant_int8(hidden_states) when LMSLIM_USE_FUSED_RMS_QUANT is set (int8.py:291-293; the
 * producer is the fused RMS-norm + quant upstream of the layer).
 *   x_q [M, H] int8, x_s [M] f32: neither is written; the quantisation launch is left out.
 *   dtype: the type of cache13, shared_output and out (LO_BF16 / LO_F16).
 * Everything else as lo_fused_experts_channel_int8.
 */
int lo_fused_experts_channel_int8_prequant(const int8_t *x_q, const float *x_s, int dtype, int64_t M, int64_t H,
                                           int64_t I, int32_t E, int32_t num_experts, int32_t top_k,
                                           const int8_t *w1, const float *w1s, const int8_t *w2,
                                           const float *w2s, const float *topk_w, const void *topk_ids,
                                           int ids_dtype, const int32_t *expert_map,
                                           int apply_router_weight_on_input, float routed_scaling_factor,
                                           const void *shared_output, void *cache13, void *out, void *workspace,
                                           int64_t workspace_bytes, int32_t block_size_m, int flags,
                                           lo_stream_t stream);

/* ---- routers upstream of the path (they produce topk_ids / topk_weights) ---------- */

/*
 * Softmax over all experts, the topk largest, their probabilities.
 * Replaces op.topk_softmax(topk_weights, topk_indices, token_expert_indices, gating_output,
 * Is_renormalize) (csrc/pybind/export.cpp:546, :1437;
 * csrc/kernels/softmax/topk_softmax_kernels.cu:1716-1790, kernel :1381-1582).
 *
 *   gating [num_tokens, num_experts] fp32 / fp16 / bf16 (dtype = LO_F32 / LO_F16 / LO_BF16)
 *   topk_weights [num_tokens, topk] fp32;  topk_indices [num_tokens, topk] int32 / int64
 *   token_expert_indices [num_tokens, topk] int32 or NULL: entry (t, j) = j * num_tokens + t
 *   renormalize = 0: exp(x - max) / (sum over all experts + 1e-6)
 *   renormalize = 1: exp(x - max) / (sum over the selected + 1e-6)
 * Winners in descending order; equal scores are won by the lower expert id (the reference
 * leaves that open).  num_experts <= 1024, topk <= 64.
 */
int lo_topk_softmax(const void *gating, int dtype, int64_t num_tokens, int32_t num_experts,
                    int32_t topk, int renormalize, float *topk_weights, void *topk_indices,
                    int idx_dtype, int32_t *token_expert_indices, lo_stream_t stream);

/*
 * Grouped sigmoid top-k with a correction bias (DeepSeek-V3 style).  Replaces
 * op.moe_fused_gate(input, bias, num_expert_group, topk_group, topk, n_share_experts_fusion,
 * routed_scaling_factor, apply_routed_scaling_factor_on_output, output_indices_int64)
 * (csrc/pybind/export.cpp:566, :1508; csrc/kernels/moe_gate/moe_fused_gate.cu:76-312, :1331-1530).
 *
 *   s = sigmoid(input);  c = bias + s;  group score = sum of the two largest c of the group;
 *   the topk_group best groups stay; the topk - n_share best c among them are selected
 *   (descending, ties to the lower id); weight = s / (sum of the selected s) * scale with
 *   scale = routed_scaling_factor if apply_... and the factor is positive, else 1.
 *   The n_share shared experts follow with ids num_experts, num_experts + 1, ... and weight
 *   (sum / routed_scaling_factor) / sum * scale.
 *   input [num_tokens, num_experts], bias [num_experts]: fp32 / fp16 / bf16 each.
 * Unlike the reference, every (num_experts <= 1024, groups <= 64, topk <= 64) combination
 * that divides evenly is served by one kernel.
 */
int lo_moe_fused_gate(const void *input, int dtype, const void *bias, int bias_dtype,
                      int64_t num_tokens, int32_t num_experts, int32_t num_expert_group,
                      int32_t topk_group, int32_t topk, int32_t n_share_experts_fusion,
                      double routed_scaling_factor, int apply_routed_scaling_factor_on_output,
                      float *topk_weights, void *topk_indices, int idx_dtype, lo_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LIGHTOP_MI355_H */
