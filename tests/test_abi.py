"""The C-ABI library loads without a GPU and exports exactly what include/lightop_mi355.h
declares; argument validation that happens before any HIP call is exercised too."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lightop_mi355.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lo_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from lightop_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from lightop_amd import build

        build.build_library()
    return _lib.lib()


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("lo_moe_align_block_size", "lo_per_token_group_quant_int8", "lo_moe_gemm_block_int8",
                 "lo_moe_gemm1_silu_quant_block_int8", "lo_silu_and_mul", "lo_moe_sum",
                 "lo_fused_experts_block_int8", "lo_fused_experts_workspace_bytes",
                 "lo_preshuffle_weight_int8", "lo_moe_tile_query", "lo_last_error", "lo_version"):
        assert must in names


def test_every_declared_symbol_is_exported_and_bound(lib):
    from lightop_amd import _lib

    names = declared_functions()
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature in lightop_amd/_lib.py"
    assert sorted(_lib.SIGNATURES) == names, "ctypes table and header disagree"


def test_header_cites_the_reference_for_every_entry_point():
    text = open(HEADER).read()
    for cite in ("export.cpp:1593-1605", "int8_utils.py:125-195", "int8.py:543-626", "int8.py:811",
                 "export.cpp:1584-1592", "int8.py:220-256", "int8.py:703-888", "int8_utils.py:20-71",
                 "gemmopt.py:437-457", "fuse_silu_mul_quant.cu:90-133", "w4a8.py:211-401"):
        assert cite in text


def test_version_and_tile_table(lib):
    from lightop_amd import _lib

    assert lib.lo_version() >= 100
    t1, t2 = _lib.LoMoeTile(), _lib.LoMoeTile()
    # DeepSeek-V3 EP share: 256 global experts, top-8
    sizes = {}
    for M in (1, 16, 64, 256, 1024, 4096, 8192):
        assert lib.lo_moe_tile_query(M, 32, 256, 8, 7168, 2048, t1, t2) == 0
        assert t1.block_size_m == t2.block_size_m and t1.block_size_m in (16, 32, 64, 128, 160)
        sizes[M] = t1.block_size_m
    assert sizes[1] == 16 and sizes[64] == 16 and sizes[4096] == 160 and sizes[8192] == 128
    assert lib.lo_moe_tile_query(-1, 32, 256, 8, 7168, 2048, t1, t2) < 0
    assert b"moe_tile_query" in lib.lo_last_error()
    # the block-form table as the tuning harness last derived it (pre-shuffled weights): LDS-tiled
    # kernels from a handful of slots per expert on (64-token tiles while there is about one token block
    # per expert, on a short K up to 48 slots per expert), 160-token blocks around 128 slots per expert
    # (where a 128-token block would spill a few tokens into a second pass over the expert's weights)
    for M, want in ((64, 16), (128, 128), (256, 128), (512, 128), (1024, 64), (1280, 64), (1536, 64), (2048, 128), (2304, 128),
                    (2560, 160), (3072, 160), (3584, 160), (4096, 160), (4352, 128)):
        assert lib.lo_moe_tile_query(M, 32, 256, 8, 7168, 2048, t1, t2) == 0 and t1.block_size_m == want
    for M, want in ((64, 16), (128, 64), (512, 64), (768, 64), (1024, 128), (1152, 160), (1280, 160), (1536, 160),
                    (2048, 160), (2304, 160), (2432, 160), (2560, 128), (3072, 128), (4096, 160), (4352, 160), (4608, 128),
                    (8192, 128)):
        assert lib.lo_moe_tile_query(M, 128, 128, 8, 2048, 768, t1, t2) == 0 and t1.block_size_m == want
    assert lib.lo_moe_tile_query(512, 128, 128, 8, 2048, 768, t1, t2) == 0
    assert t1.kernel == _lib.LO_KERNEL_TILE == t2.kernel
    # a third shape class by the size of an expert's weights (3 * H * I bytes: 4096 x 1536 lies between the two
    # layers above): 64-token tiles up to 40 slots per expert, 160-token blocks from 88 to 152
    for M, want in ((8, 16), (16, 64), (512, 64), (768, 128), (1280, 128), (1536, 160), (2304, 160), (2560, 128)):
        assert lib.lo_moe_tile_query(M, 128, 128, 8, 4096, 1536, t1, t2) == 0 and t1.block_size_m == want
    # 160-token blocks: the same direct-to-LDS kernel for both GEMMs
    assert lib.lo_moe_tile_query(4096, 32, 256, 8, 7168, 2048, t1, t2) == 0
    assert t1.kernel == _lib.LO_KERNEL_T128 == t2.kernel and (t1.waves, t1.block_n) == (4, 256)
    # not with row-major weights; the fused first stage needs no [S, 2I] buffer, so 2I > H is no obstacle
    assert lib.lo_moe_tile_query_form(_lib.LO_FORM_BLOCK, 0, 2048, 128, 128, 8, 2048, 768, t1, t2) == 0
    assert t1.block_size_m == 64
    assert lib.lo_moe_tile_query(2048, 128, 128, 8, 2048, 1536, t1, t2) == 0 and t1.block_size_m == 160
    # per-channel form: streaming tiles up to half a dozen slots per expert, then the LDS-tiled kernels
    # (128 tokens on a long K; on a short K 64 tokens until an expert sees 48)
    for M, want in ((1, 16), (64, 16), (192, 16), (256, 128), (1024, 128), (8192, 128)):
        assert lib.lo_moe_tile_query_form(_lib.LO_FORM_CHANNEL, 0, M, 32, 256, 8, 7168, 2048, t1, t2) == 0
        assert t1.block_size_m == want and t2.block_size_m == want
    for M, want in ((64, 16), (128, 64), (512, 64), (1024, 128)):
        assert lib.lo_moe_tile_query_form(_lib.LO_FORM_CHANNEL, 0, M, 128, 128, 8, 2048, 768, t1, t2) == 0
        assert t1.block_size_m == want and t2.block_size_m == want
    # W4A8: streaming for a handful of slots per expert, the 64-token LDS tile from 8 on, 128 tokens from 48 on
    for M, want in ((1, 16), (128, 16), (256, 16), (512, 64), (1024, 64), (2048, 128), (8192, 128)):
        assert lib.lo_moe_tile_query_form(_lib.LO_FORM_W4, 0, M, 32, 256, 8, 7168, 2048, t1, t2) == 0
        assert t1.block_size_m == want
    assert lib.lo_moe_tile_query_form(7, 0, 1, 32, 256, 8, 7168, 2048, t1, t2) < 0


def test_tile_query_names_the_kernel_that_is_launched(lib):
    """kernel / waves / block_n are those of the kernel the stage entry points pick for the block size,
    for both weight layouts (they share one selection function with the launcher)."""
    from lightop_amd import _lib

    t1, t2 = _lib.LoMoeTile(), _lib.LoMoeTile()
    pre = _lib.LO_GEMM_W_PRESHUFFLED
    q = lambda form, flags, M, *shape: lib.lo_moe_tile_query_form(form, flags, M, *shape, t1, t2)
    qwen, dsv3 = (128, 128, 8, 2048, 768), (32, 256, 8, 7168, 2048)
    # decode sizes: weight streaming, eight waves own one 128-column activation group in the fused GEMM
    assert q(_lib.LO_FORM_BLOCK, pre, 16, *dsv3) == 0
    assert (t1.block_size_m, t1.kernel, t1.waves, t1.block_n) == (16, _lib.LO_KERNEL_WS, 8, 256)
    assert (t2.kernel, t2.waves, t2.block_n) == (_lib.LO_KERNEL_WS, 4, 256)
    # a few tokens: the whole-path call's two-launch path (four waves split K = 2048, eight K = 7168)
    assert q(_lib.LO_FORM_BLOCK, pre, 1, *qwen) == 0
    assert (t1.block_size_m, t1.kernel, t1.waves, t1.block_n) == (16, _lib.LO_KERNEL_DEC, 4, 16)
    assert (t2.kernel, t2.waves, t2.block_n) == (_lib.LO_KERNEL_DEC, 8, 16)
    assert q(_lib.LO_FORM_BLOCK, pre, 4, *dsv3) == 0 and (t1.kernel, t1.waves) == (_lib.LO_KERNEL_DEC, 8)
    assert q(_lib.LO_FORM_BLOCK, pre | _lib.LO_FUSED_NO_DECODE_PATH, 1, *qwen) == 0 and t1.kernel == _lib.LO_KERNEL_WS
    assert q(_lib.LO_FORM_BLOCK, 0, 1, *qwen) == 0 and t1.kernel == _lib.LO_KERNEL_WS  # row-major weights
    assert q(_lib.LO_FORM_BLOCK, pre, 8, *qwen) == 0 and t1.kernel == _lib.LO_KERNEL_DEC  # four K blocks per wave
    assert q(_lib.LO_FORM_BLOCK, pre, 8, *dsv3) == 0 and t1.kernel == _lib.LO_KERNEL_WS   # seven: up to four tokens
    assert q(_lib.LO_FORM_BLOCK, pre, 16, *qwen) == 0 and t1.kernel == _lib.LO_KERNEL_WS
    assert q(_lib.LO_FORM_BLOCK, pre | _lib.LO_FUSED_FORCE_DECODE_PATH, 16, *qwen) == 0 and t1.kernel == _lib.LO_KERNEL_DEC
    # prefill, load-time layout: 128-token direct-to-LDS kernel for GEMM1, activation-stationary GEMM2 on a short K
    assert q(_lib.LO_FORM_BLOCK, pre, 8192, *qwen) == 0
    assert (t1.block_size_m, t1.kernel, t1.waves, t1.block_n) == (128, _lib.LO_KERNEL_T128, 4, 256)
    assert t2.kernel == _lib.LO_KERNEL_AS
    assert q(_lib.LO_FORM_BLOCK, pre, 4096, *dsv3) == 0
    assert t1.kernel == _lib.LO_KERNEL_T128 and t2.kernel == _lib.LO_KERNEL_T128  # K = 2048: too long to stay in LDS
    # row-major weights: 64-token register-fed tiles, and a different block size than the load-time layout
    assert q(_lib.LO_FORM_BLOCK, 0, 8192, *qwen) == 0
    assert (t1.block_size_m, t1.kernel, t1.waves) == (64, _lib.LO_KERNEL_TILE, 4)
    assert q(_lib.LO_FORM_BLOCK, 0, 256, *qwen) == 0 and t1.block_size_m == 32 and t1.kernel == _lib.LO_KERNEL_WS
    assert q(_lib.LO_FORM_BLOCK, pre, 256, *qwen) == 0 and (t1.block_size_m, t1.kernel) == (64, _lib.LO_KERNEL_TILE)
    assert q(_lib.LO_FORM_BLOCK, pre, 256, *dsv3) == 0 and (t1.block_size_m, t1.kernel) == (128, _lib.LO_KERNEL_T128)
    # forced streaming is honoured
    assert q(_lib.LO_FORM_BLOCK, pre | _lib.LO_GEMM_FORCE_STREAMING, 8192, *qwen) == 0 and t1.kernel == _lib.LO_KERNEL_WS
    # per-channel and int4 forms
    assert q(_lib.LO_FORM_CHANNEL, pre, 8192, *qwen) == 0 and t1.kernel == _lib.LO_KERNEL_PC == t2.kernel
    # the reference's own int4 form (per-channel scales on packed int4 weights): 128-token tiles or streaming
    assert q(_lib.LO_FORM_CHANNEL, pre | _lib.LO_GEMM_W4, 8192, *qwen) == 0
    assert t1.kernel == _lib.LO_KERNEL_T128 == t2.kernel and t1.block_size_m == 128
    assert q(_lib.LO_FORM_CHANNEL, pre | _lib.LO_GEMM_W4, 16, *qwen) == 0 and t1.kernel == _lib.LO_KERNEL_WS == t2.kernel
    # ... and its 160-token form around 128 slots per expert
    assert q(_lib.LO_FORM_CHANNEL, pre | _lib.LO_GEMM_W4, 2048, *qwen) == 0
    assert t1.kernel == _lib.LO_KERNEL_T128 == t2.kernel and t1.block_size_m == 160 == t2.block_size_m
    assert q(_lib.LO_FORM_CHANNEL, pre | _lib.LO_GEMM_W4, 1024, *qwen) == 0 and t1.block_size_m == 128
    # ... and again around 256, where two such blocks hold what would need a third of 128 tokens
    for M, want in ((3072, 128), (3840, 128), (4096, 160), (4608, 160), (5120, 128)):
        assert q(_lib.LO_FORM_CHANNEL, pre | _lib.LO_GEMM_W4, M, *qwen) == 0 and t1.block_size_m == want, M
    assert q(_lib.LO_FORM_CHANNEL, pre, 4096, *qwen) == 0 and t1.block_size_m == 128  # int8 weights: no second window
    assert q(_lib.LO_FORM_CHANNEL, pre, 2048, *qwen) == 0 and (t1.block_size_m, t1.kernel) == (160, _lib.LO_KERNEL_T128)
    assert q(_lib.LO_FORM_CHANNEL, 0, 2048, *qwen) == 0 and t1.block_size_m == 128  # row-major weights: no such form
    assert q(_lib.LO_FORM_W4, 0, 2, *dsv3) == 0 and t1.kernel == _lib.LO_KERNEL_DEC  # int4: up to 16 slots
    assert q(_lib.LO_FORM_W4, 0, 4, *dsv3) == 0 and t1.kernel == _lib.LO_KERNEL_WS
    assert q(_lib.LO_FORM_W4, 0, 512, *dsv3) == 0 and t1.kernel == _lib.LO_KERNEL_W4_TILE
    assert q(_lib.LO_FORM_W4, 0, 8192, *dsv3) == 0 and t1.kernel == _lib.LO_KERNEL_T128
    # the convenience query is the block form with the load-time layout
    t3 = _lib.LoMoeTile()
    assert lib.lo_moe_tile_query(8192, *qwen, t3, None) == 0 and q(_lib.LO_FORM_BLOCK, pre, 8192, *qwen) == 0
    assert (t1.block_size_m, t1.kernel, t1.waves, t1.block_n) == (t3.block_size_m, t3.kernel, t3.waves, t3.block_n)


def test_workspace_sizing(lib):
    n16 = lib.lo_fused_experts_workspace_bytes(64, 8, 7168, 2048, 256, 16)
    n0 = lib.lo_fused_experts_workspace_bytes(64, 8, 7168, 2048, 256, 0)
    assert 0 < n16 <= n0
    # a1q + a2q alone
    assert n16 >= 64 * 7168 + 64 * 8 * 2048
    assert lib.lo_fused_experts_workspace_bytes(64, 8, 100, 2048, 256, 16) < 0
    offs = [lib.lo_fused_experts_workspace_offset(i, 64, 8, 7168, 2048, 256, 16) for i in range(8)]
    assert offs == sorted(offs) and all(o % 256 == 0 for o in offs)
    assert lib.lo_fused_experts_workspace_offset(8, 64, 8, 7168, 2048, 256, 16) < 0
    # block_size_m = 0 must cover every block size the call may end up with: few experts and many
    # tokens make the per-block expert ids of small blocks the larger segment
    for (M, k, H, I, E) in ((16384, 2, 1024, 512, 2), (16384, 2, 1024, 512, 8), (64, 8, 7168, 2048, 256),
                            (1, 8, 2048, 768, 128), (8192, 8, 2048, 768, 128)):
        n0 = lib.lo_fused_experts_workspace_bytes(M, k, H, I, E, 0)
        for bs in (16, 32, 64, 128):
            assert n0 >= lib.lo_fused_experts_workspace_bytes(M, k, H, I, E, bs), (M, E, bs)


def test_validation_happens_before_any_launch(lib):
    """Null pointers and bad shapes are rejected on the host (no GPU needed)."""
    null = ctypes.c_void_p(0)
    assert lib.lo_moe_align_block_size(null, 0, 8, 8, 16, null, 0, null, 128, null, 8, null, null) == -1
    assert b"null pointer" in lib.lo_last_error()
    buf = (ctypes.c_int32 * 64)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.lo_moe_align_block_size(p, 7, 8, 8, 16, null, 0, p, 128, p, 8, p, null) == -1     # bad id dtype
    assert lib.lo_moe_align_block_size(p, 0, 8, 8, 16, null, 0, p, 10, p, 8, p, null) == -2      # buffer too small
    assert b"sorted_ids holds 10" in lib.lo_last_error()
    assert lib.lo_per_token_group_quant_int8(p, 0, 1, 100, 1e-10, p, p, null) == -1              # cols % 128
    assert lib.lo_per_token_group_quant_int8(p, 3, 1, 128, 1e-10, p, p, null) == -4              # no such element type
    assert lib.lo_per_token_quant_int8(p, 2, 1, 128, p, p, null) == -4                           # per-channel form: no fp32 rows
    assert lib.lo_moe_sum(p, p, null, null, 0, 1, 8, 100, 1.0, null, null) == -1                       # H % 8
    assert lib.lo_preshuffle_weight_int8(p, p, 1, 16, 128, null) == -1                           # src == dst


def test_stage_entry_points_reject_a_bad_block_size(lib):
    """block_size_m divides the sorted-id extent: 0 (the whole-path call's "ask the table") and sizes
    that are not 16 / 32 / 64 / 128 are an error here, not a division by zero."""
    null = ctypes.c_void_p(0)
    buf = (ctypes.c_int32 * 1024)()
    p = ctypes.c_void_p((ctypes.addressof(buf) + 15) // 16 * 16)
    for bad in (0, 48, -16, 256):
        rc = lib.lo_moe_gemm_block_int8(p, p, p, p, p, 0, null, p, p, p, 128, 8, 8, 1, 1, 16, 128, 1, bad, 0, 0, null)
        assert rc == -1 and b"block_size_m" in lib.lo_last_error(), bad
        rc = lib.lo_moe_gemm1_silu_quant_block_int8(p, p, p, p, p, p, 0, null, p, p, p, 128, 8, 8, 1, 1, 128, 128,
                                                    1, bad, 0, 0, null)
        assert rc == -1 and b"block_size_m" in lib.lo_last_error(), bad
        rc = lib.lo_moe_gemm_w8a8(p, p, p, p, p, 0, null, p, p, p, 128, 8, 8, 1, 1, 16, 128, 1, bad, 0, 0, null)
        assert rc == -1 and b"block_size_m" in lib.lo_last_error(), bad


def test_tile_query_path_follows_element_type_activation_and_block_size(lib):
    """The whole-path call resolves its block size, fused / plain first stage and the two-launch path in one
    function; lo_moe_tile_query_path reports from that function for any element type, activation and
    caller-chosen block size, so what it says is what the call launches."""
    from lightop_amd import _lib

    t1, t2 = _lib.LoMoeTile(), _lib.LoMoeTile()
    pre = _lib.LO_GEMM_W_PRESHUFFLED
    qwen, dsv3 = (128, 128, 8, 2048, 768), (32, 256, 8, 7168, 2048)

    def q(form, flags, dtype, bs, M, shape):
        assert lib.lo_moe_tile_query_path(form, flags, dtype, bs, M, *shape, t1, t2) == 0
        return (t1.block_size_m, t1.kernel), (t2.block_size_m, t2.kernel)

    # bf16 + SiLU: exactly lo_moe_tile_query_form
    for M in (1, 8, 64, 512, 2048, 8192):
        for shape in (qwen, dsv3):
            want = q(_lib.LO_FORM_BLOCK, pre, _lib.LO_BF16, 0, M, shape)
            assert lib.lo_moe_tile_query_form(_lib.LO_FORM_BLOCK, pre, M, *shape, t1, t2) == 0
            assert ((t1.block_size_m, t1.kernel), (t2.block_size_m, t2.kernel)) == want
    # one token: bf16 + SiLU takes the two-launch path; GELU and fp16 rows have no fused epilogue and never do
    assert q(_lib.LO_FORM_BLOCK, pre, _lib.LO_BF16, 0, 1, qwen)[0][1] == _lib.LO_KERNEL_DEC
    assert q(_lib.LO_FORM_BLOCK, pre | _lib.LO_FUSED_ACT_GELU, _lib.LO_BF16, 0, 1, qwen)[0][1] == _lib.LO_KERNEL_WS
    assert q(_lib.LO_FORM_BLOCK, pre, _lib.LO_F16, 0, 1, qwen)[0][1] == _lib.LO_KERNEL_WS
    # the plain first GEMM of those paths has the plain workgroup shape (four waves), not the fused one (eight)
    q(_lib.LO_FORM_BLOCK, pre, _lib.LO_F16, 0, 16, dsv3)
    assert (t1.kernel, t1.waves) == (_lib.LO_KERNEL_WS, 4)
    q(_lib.LO_FORM_BLOCK, pre, _lib.LO_BF16, 0, 16, dsv3)
    assert (t1.kernel, t1.waves) == (_lib.LO_KERNEL_WS, 8)
    # 160-token blocks are the table's pick for bf16 + SiLU only; fp16 rows and GELU get 64 / 128 there
    assert q(_lib.LO_FORM_BLOCK, pre, _lib.LO_BF16, 0, 2048, qwen)[0][0] == 160
    assert q(_lib.LO_FORM_BLOCK, pre, _lib.LO_F16, 0, 2048, qwen)[0][0] == 64
    assert q(_lib.LO_FORM_BLOCK, pre | _lib.LO_FUSED_ACT_GELU, _lib.LO_BF16, 0, 2048, qwen)[0][0] == 64
    assert q(_lib.LO_FORM_BLOCK, pre, _lib.LO_F16, 160, 2048, qwen)[0] == (160, _lib.LO_KERNEL_T128)  # on request
    # fp32 rows: the row-major table and the weight-streaming kernel at every size, whatever the layout
    for M in (1, 512, 8192):
        a, b = q(_lib.LO_FORM_BLOCK, pre, _lib.LO_F32, 0, M, qwen)
        assert a[1] == _lib.LO_KERNEL_WS == b[1]
        assert a[0] == q(_lib.LO_FORM_BLOCK, 0, _lib.LO_BF16, 0, M, qwen)[0][0]
    assert lib.lo_moe_tile_query_path(_lib.LO_FORM_BLOCK, pre, _lib.LO_F32, 160, 2048, *qwen, t1, t2) < 0  # refused, as the call does
    # a caller's block size (for instance from a tuning file) is described as it would be launched, and
    # switches the two-launch path off, as it does in the call
    assert q(_lib.LO_FORM_BLOCK, pre, _lib.LO_BF16, 64, 8192, qwen)[0] == (64, _lib.LO_KERNEL_TILE)
    assert q(_lib.LO_FORM_BLOCK, pre, _lib.LO_BF16, 16, 1, qwen)[0] == (16, _lib.LO_KERNEL_WS)
    assert lib.lo_moe_tile_query_path(_lib.LO_FORM_BLOCK, pre, _lib.LO_BF16, 48, 64, *qwen, t1, t2) < 0
    assert lib.lo_moe_tile_query_path(_lib.LO_FORM_BLOCK, pre, 9, 0, 64, *qwen, t1, t2) < 0
    # int4 weights imply the load-time layout in the whole-path call, at every size
    assert q(_lib.LO_FORM_W4, 0, _lib.LO_BF16, 0, 2, dsv3)[0][1] == _lib.LO_KERNEL_DEC
    assert q(_lib.LO_FORM_BLOCK, _lib.LO_GEMM_W4, _lib.LO_BF16, 0, 2048, dsv3) == \
        q(_lib.LO_FORM_W4, 0, _lib.LO_BF16, 0, 2048, dsv3)
