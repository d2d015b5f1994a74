"""The C-ABI library: it loads without a GPU, exports every symbol that
include/neox_hotpath.h declares, and its argument validation (which happens
before anything touches the device) returns the documented status codes."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "neox_hotpath.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nhp_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("nhp_causal_softmax_fwd", "nhp_causal_softmax_bwd", "nhp_masked_softmax_fwd",
                 "nhp_masked_softmax_bwd", "nhp_softmax_batch_per_block", "nhp_rope_cached_fwd",
                 "nhp_rope_cached_bwd", "nhp_rope_freqs_fwd", "nhp_rope_freqs_bwd"):
        assert must in names


def test_library_exports_every_declared_symbol(hotpath):
    lib = ctypes.CDLL(hotpath.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    # and the Python binding declares exactly the header's functions
    hotpath.lib()
    assert sorted(hotpath.EXPORTS) == declared_functions()


def test_every_header_comment_cites_the_reference():
    text = open(HEADER).read()
    for name in declared_functions():
        if name in ("nhp_abi_version", "nhp_status_string", "nhp_softmax_max_resident_row", "nhp_softmax_geometry"):
            continue
        if name.endswith("_workspace_bytes"):  # size query, documented with the function it serves
            continue
        if name == "nhp_layernorm_bwd_noalloc":
            # the one entry point without a counterpart in the reference: its comment must say so
            before = text[: text.index(name + "(")]
            assert "No counterpart in the reference" in before[before.rindex("/*"):]
            continue
        before = text[: text.index(name + "(")]
        comment = before[before.rindex("/*") :]
        # the backward/forward pairs of the rotary functions share one comment
        assert "megatron/fused_kernels/" in comment or "megatron/model/" in comment or name.startswith("nhp_rope_"), name
    assert text.count("Replaces ") >= 7


def test_status_strings_and_version(hotpath):
    lib = hotpath.lib()
    assert lib.nhp_abi_version() == hotpath.ABI_VERSION
    assert lib.nhp_status_string(0) == b"ok"
    seen = set()
    for code in range(-7, 0):
        s = lib.nhp_status_string(code)
        assert s and s != b"unknown status"
        seen.add(s)
    assert len(seen) == 7
    assert lib.nhp_status_string(-99) == b"unknown status"
    assert lib.nhp_softmax_max_resident_row() == 65536
    L, K, W = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    for kind in range(5):
        assert lib.nhp_softmax_geometry(2048, kind, ctypes.byref(L), ctypes.byref(K), ctypes.byref(W)) == 0
        assert L.value == 64 and L.value * K.value * W.value * 8 >= 2048
    assert lib.nhp_softmax_geometry(2047, 0, ctypes.byref(L), ctypes.byref(K), ctypes.byref(W)) == -2  # scalar kernel
    assert lib.nhp_softmax_geometry(2048, 9, ctypes.byref(L), ctypes.byref(K), ctypes.byref(W)) == -2


def test_batch_per_block_matches_reference_formula(hotpath):
    import oracle

    lib = hotpath.lib()
    for sk in (1, 2, 8, 16, 17, 32, 33, 64, 65, 128, 129, 256, 1000, 2048, 4096, 8192):
        assert lib.nhp_softmax_batch_per_block(1024, sk, 4, 8) == oracle.batch_per_block(sk, 64), sk
    assert lib.nhp_softmax_batch_per_block(4, 0, 1, 1) == -2  # NHP_ERR_SHAPE


def test_argument_validation_needs_no_gpu(hotpath):
    lib = hotpath.lib()
    F16, BF16, F32 = hotpath.F16, hotpath.BF16, hotpath.F32
    p = ctypes.c_void_p(0x1000)  # never dereferenced: every call below fails validation or is empty
    o = ctypes.c_void_p(0x9000)
    null = ctypes.c_void_p(0)
    st = (ctypes.c_int64 * 4)(8, 8, 8, 1)
    # dtype
    assert lib.nhp_causal_softmax_fwd(p, p, 1.0, 1, 8, F32, None) == -1
    assert lib.nhp_causal_softmax_bwd(p, p, p, 1.0, 1, 8, 7, None) == -1
    assert lib.nhp_masked_softmax_fwd(p, p, p, 1.0, 1, 1, 2, 8, 1, F32, None) == -1
    assert lib.nhp_masked_softmax_bwd(p, p, p, 1.0, 2, 8, -1, None) == -1
    assert lib.nhp_rope_cached_fwd(p, p, p, p, 1, 1, 1, 8, 8, st, st, 5, F32, None) == -1
    assert lib.nhp_rope_cached_fwd(p, p, p, p, 1, 1, 1, 8, 8, st, st, BF16, F16, None) == -1  # tables neither fp32 nor same
    assert lib.nhp_rope_freqs_bwd(p, p, p, 1, 1, 1, 8, 8, st, st, 9, None) == -1
    # shape
    assert lib.nhp_causal_softmax_fwd(p, p, 1.0, -1, 8, BF16, None) == -2
    assert lib.nhp_causal_softmax_fwd(p, p, 1.0, 1 << 40, 1 << 20, BF16, None) == -2
    assert lib.nhp_masked_softmax_fwd(p, p, p, 1.0, 1, 1, -2, 8, 1, F16, None) == -2
    assert lib.nhp_rope_cached_fwd(p, p, p, p, 1, 1, 1, 8, 16, st, st, BF16, BF16, None) == -2  # d2 > d
    # empty tensors are fine and launch nothing, even with null pointers
    assert lib.nhp_causal_softmax_fwd(null, null, 1.0, 0, 8, BF16, None) == 0
    assert lib.nhp_causal_softmax_bwd(null, null, null, 1.0, 4, 0, BF16, None) == 0
    assert lib.nhp_masked_softmax_fwd(null, null, null, 1.0, 2, 0, 4, 8, 2, F16, None) == 0
    assert lib.nhp_masked_softmax_bwd(null, null, null, 1.0, 0, 8, F16, None) == 0
    assert lib.nhp_rope_cached_bwd(null, null, null, null, 0, 1, 1, 8, 8, st, st, F32, F32, None) == 0
    assert lib.nhp_rope_freqs_fwd(null, null, null, 4, 0, 1, 8, 8, st, st, F16, None) == 0
    # null pointers for non-empty tensors
    assert lib.nhp_causal_softmax_fwd(null, p, 1.0, 1, 8, BF16, None) == -3
    assert lib.nhp_masked_softmax_fwd(p, p, null, 1.0, 1, 1, 2, 8, 1, F16, None) == -3
    assert lib.nhp_rope_cached_fwd(o, p, null, p, 1, 1, 1, 8, 8, st, st, BF16, BF16, None) == -3
    assert lib.nhp_rope_freqs_fwd(o, p, null, 1, 1, 1, 8, 8, st, st, BF16, None) == -3
    assert lib.nhp_rope_freqs_fwd(o, p, p, 1, 1, 1, 8, 8, None, st, BF16, None) == -3
    assert lib.nhp_rope_freqs_qk_fwd(o, ctypes.c_void_p(0xa000), p, p, null, 1, 1, 1, 1, 8, 8, st, st, st, st, BF16, None) == -3
    assert lib.nhp_rope_freqs_qk_fwd(o, o, p, p, p, 1, 1, 1, 1, 8, 8, st, st, st, st, BF16, None) == -6
    assert lib.nhp_rope_freqs_qk_bwd(null, null, null, null, null, 0, 1, 1, 1, 8, 8, st, st, st, st, F16, None) == 0
    assert lib.nhp_rope_freqs_qk_bwd(o, ctypes.c_void_p(0xa000), p, p, p, 1, 1, 1, 1, 8, 16, st, st, st, st, F16, None) == -2
    # mask batch dimension
    assert lib.nhp_masked_softmax_fwd(p, p, p, 1.0, 4, 1, 2, 8, 3, F16, None) == -4
    # aliasing that is not allowed: dx over y, rotary in place
    assert lib.nhp_causal_softmax_bwd(p, ctypes.c_void_p(0x2000), p, 1.0, 1, 8, BF16, None) == -6
    assert lib.nhp_masked_softmax_bwd(p, ctypes.c_void_p(0x2000), p, 1.0, 2, 8, BF16, None) == -6
    assert lib.nhp_rope_cached_fwd(p, p, p, p, 1, 1, 1, 8, 8, st, st, BF16, BF16, None) == -6


def test_argument_validation_of_the_layer_entry_points(hotpath):
    lib = hotpath.lib()
    F16, BF16, F32 = hotpath.F16, hotpath.BF16, hotpath.F32
    p = ctypes.c_void_p(0x1000)  # never dereferenced
    q = ctypes.c_void_p(0x2000)
    q2 = ctypes.c_void_p(0x3000)
    null = ctypes.c_void_p(0)
    # causal softmax variants: heads must divide attn_batches when a per-head operand is given
    assert lib.nhp_causal_softmax_ex_fwd(q, p, 1.0, 6, 8, -1, p, null, null, 4, BF16, None) == -2
    assert lib.nhp_causal_softmax_ex_fwd(q, p, 1.0, 6, 8, -1, null, p, null, 0, BF16, None) == -2
    assert lib.nhp_causal_softmax_ex_fwd(q, p, 1.0, 6, 8, -1, null, null, p, 5, BF16, None) == -2
    assert lib.nhp_causal_softmax_ex_fwd(q, p, 1.0, 6, 8, -1, null, q, null, 3, BF16, None) == -6   # bias over the output
    assert lib.nhp_causal_softmax_ex_bwd(q, p, p, 1.0, 6, 8, -1, p, 4, BF16, None) == -2
    assert lib.nhp_causal_softmax_ex_fwd(null, null, 1.0, 0, 8, 3, null, null, null, 1, F16, None) == 0
    # the same extras with dropout, and on the padding-mask softmax
    assert lib.nhp_causal_softmax_ex_dropout_fwd(q, q2, p, 1.0, 6, 8, -1, 0, p, null, null, 4, 0.1, 1, 0, BF16, None) == -2
    assert lib.nhp_causal_softmax_ex_dropout_fwd(q, q2, p, 1.0, 6, 8, -1, 0, null, q2, null, 3, 0.1, 1, 0, BF16, None) == -6
    assert lib.nhp_causal_softmax_ex_dropout_fwd(q, q2, p, 1.0, 6, 8, -1, 0, null, q, null, 3, 0.1, 1, 0, BF16, None) == -6
    assert lib.nhp_causal_softmax_ex_dropout_fwd(q, q2, p, 1.0, 6, 8, -1, 0, null, null, null, 1, 1.0, 1, 0, BF16, None) == -2
    assert lib.nhp_causal_softmax_ex_dropout_bwd(q, p, p, 1.0, 6, 8, -1, 0, p, 4, 0.1, 1, 0, BF16, None) == -2
    assert lib.nhp_causal_softmax_ex_dropout_bwd(null, null, null, 1.0, 0, 8, -1, 0, null, 1, 0.1, 1, 0, BF16, None) == 0
    assert lib.nhp_masked_softmax_ex_fwd(q, p, p, 1.0, 2, 2, 8, 16, 1, p, null, null, BF16, None) == -2   # AliBi needs sq == sk
    assert lib.nhp_masked_softmax_ex_fwd(q, p, p, 1.0, 2, 2, 8, 16, 1, null, q, null, BF16, None) == -6   # bias over the output
    assert lib.nhp_masked_softmax_ex_fwd(q, p, p, 1.0, 2, 2, 8, 16, 3, null, null, p, BF16, None) == -4
    assert lib.nhp_masked_softmax_ex_fwd(q, p, p, 1.0, 2, 2, 8, 16, 1, null, null, null, F32, None) == -1
    assert lib.nhp_masked_softmax_ex_fwd(null, null, null, 1.0, 2, 0, 8, 16, 1, null, null, null, F16, None) == 0
    assert lib.nhp_masked_softmax_ex_dropout_fwd(q2, q, p, p, 1.0, 2, 2, 8, 16, 1, null, q2, null, 0.1, 1, 0, BF16, None) == -6
    assert lib.nhp_masked_softmax_ex_dropout_fwd(q, q, p, p, 1.0, 2, 2, 8, 16, 1, null, null, null, 0.1, 1, 0, BF16, None) == -6
    assert lib.nhp_masked_softmax_ex_dropout_fwd(null, q, p, p, 1.0, 2, 2, 8, 16, 1, null, null, null, 0.1, 1, 0, BF16, None) == -3
    assert lib.nhp_masked_softmax_ex_dropout_fwd(q2, q, p, p, 1.0, 2, 2, 8, 16, 1, null, null, null, -0.5, 1, 0, BF16, None) == -2
    # block-limited variants: the block size must be 0 or a power of two of at least 8
    for bad in (4, 12, 100, -8):
        assert lib.nhp_causal_softmax_blocks_fwd(q, p, 1.0, 6, 64, -1, bad, null, null, null, 1, BF16, None) == -2
        assert lib.nhp_causal_softmax_blocks_bwd(q, p, p, 1.0, 6, 64, -1, bad, null, 1, BF16, None) == -2
        assert lib.nhp_causal_softmax_dropout_blocks_fwd(q, q2, p, 1.0, 6, 64, -1, bad, 0.1, 1, 0, BF16, None) == -2
        assert lib.nhp_causal_softmax_dropout_blocks_bwd(q, p, p, 1.0, 6, 64, -1, bad, 0.1, 1, 0, BF16, None) == -2
    assert lib.nhp_causal_softmax_blocks_fwd(q, p, 1.0, 6, 64, -1, 16, null, null, null, 1, 5, None) == -1
    assert lib.nhp_causal_softmax_blocks_fwd(null, p, 1.0, 6, 64, -1, 16, null, null, null, 1, BF16, None) == -3
    assert lib.nhp_causal_softmax_blocks_fwd(null, null, 1.0, 0, 64, -1, 16, null, null, null, 1, BF16, None) == 0
    assert lib.nhp_causal_softmax_blocks_bwd(q, p, q, 1.0, 6, 64, -1, 16, null, 1, BF16, None) == -6
    # bias + GeLU, bias + residual
    assert lib.nhp_bias_gelu_fwd(q, p, p, 4, 8, 9, None) == -1
    assert lib.nhp_bias_gelu_fwd(q, p, p, -1, 8, BF16, None) == -2
    assert lib.nhp_bias_gelu_fwd(null, null, null, 0, 8, BF16, None) == 0
    assert lib.nhp_bias_gelu_fwd(null, p, p, 4, 8, BF16, None) == -3
    assert lib.nhp_bias_gelu_bwd(q, p, null, p, null, null, 4, 8, F32, None) == -3
    assert lib.nhp_bias_gelu_bwd(q, p, p, p, q, p, 4, 8, BF16, None) == -6        # dbias over dx
    assert lib.nhp_bias_gelu_bwd(q, p, p, p, ctypes.c_void_p(0x3000), null, 4, 8, BF16, None) == -3  # workspace missing
    assert lib.nhp_bias_gelu_bwd_workspace_bytes(4, 8, BF16) > 0
    assert lib.nhp_bias_gelu_bwd_workspace_bytes(4, 7, BF16) == 0                 # scalar path needs none
    assert lib.nhp_bias_gelu_bwd_workspace_bytes(0, 8, BF16) == 0
    big = lib.nhp_bias_gelu_bwd_workspace_bytes(1 << 20, 8192, BF16)
    assert 0 < big <= 512 * 8192 * 4                                               # bounded, whatever the row count
    # softmax + dropout: probability range, missing or aliased second output, mask layout
    assert lib.nhp_causal_softmax_dropout_fwd(q, p, p, 1.0, 2, 8, -1, 1.0, 1, 0, BF16, None) == -2
    assert lib.nhp_causal_softmax_dropout_fwd(null, p, p, 1.0, 2, 8, -1, 0.1, 1, 0, BF16, None) == -3
    assert lib.nhp_causal_softmax_dropout_fwd(p, p, q, 1.0, 2, 8, -1, 0.1, 1, 0, BF16, None) == -6
    assert lib.nhp_masked_softmax_dropout_fwd(q, p, p, p, 1.0, 2, 2, 4, 8, 2, -0.5, 1, 0, BF16, None) == -2
    assert lib.nhp_masked_softmax_dropout_fwd(q, p, p, p, 1.0, 2, 2, 4, 8, 3, 0.1, 1, 0, BF16, None) == -4   # pad_batches
    assert lib.nhp_masked_softmax_dropout_fwd(q, p, p, null, 1.0, 2, 2, 4, 8, 2, 0.1, 1, 0, BF16, None) == -3
    assert lib.nhp_masked_softmax_dropout_fwd(p, p, q, p, 1.0, 2, 2, 4, 8, 2, 0.1, 1, 0, BF16, None) == -6
    assert lib.nhp_masked_softmax_dropout_fwd(q, p, p, p, 1.0, 2, 2, 4, 8, 2, 0.1, 1, 0, F32, None) == -1
    assert lib.nhp_masked_softmax_dropout_bwd(p, q, p, 1.0, 16, 8, 0.1, 1, 0, BF16, None) == -6              # dx == y
    assert lib.nhp_masked_softmax_dropout_bwd(q, q, p, 1.0, 16, 8, 1.5, 1, 0, BF16, None) == -2
    assert lib.nhp_masked_softmax_dropout_bwd(null, null, null, 1.0, 0, 8, 0.1, 1, 0, BF16, None) == 0
    assert lib.nhp_column_sum(null, p, p, 4, 8, BF16, None) == -3
    assert lib.nhp_column_sum(q, p, null, 4, 8, BF16, None) == -3                  # workspace missing
    assert lib.nhp_column_sum(p, p, q, 4, 8, BF16, None) == -6                     # sums over their own input
    assert lib.nhp_column_sum(q, p, p, 4, 8, 7, None) == -1
    assert lib.nhp_column_sum(null, null, null, 0, 8, BF16, None) == 0
    assert lib.nhp_column_sum_workspace_bytes(4, 8, BF16) == lib.nhp_bias_gelu_bwd_workspace_bytes(4, 8, BF16) > 0
    assert lib.nhp_column_sum_workspace_bytes(4, 7, BF16) == 0
    assert lib.nhp_bias_add_residual(q, null, p, p, 4, 8, F16, None) == -3
    assert lib.nhp_bias_add_residual(q, p, null, null, 4, 8, 3, None) == -1
    # norms: parameter dtype is the data dtype or fp32
    assert lib.nhp_layernorm_fwd(q, null, null, p, p, p, 1e-5, 4, 8, BF16, F16, None) == -1
    assert lib.nhp_layernorm_fwd(q, null, null, p, p, p, 1e-5, 4, 8, 4, F32, None) == -1
    assert lib.nhp_layernorm_fwd(q, null, null, p, p, p, 1e-5, -4, 8, BF16, F32, None) == -2
    assert lib.nhp_layernorm_fwd(q, null, null, null, p, p, 1e-5, 4, 8, BF16, F32, None) == -3
    assert lib.nhp_layernorm_fwd(null, null, null, null, null, null, 1e-5, 4, 0, BF16, BF16, None) == 0
    assert lib.nhp_layernorm_bwd(q, null, null, p, p, null, p, p, null, 4, 8, BF16, BF16, None) == -3   # mean missing
    assert lib.nhp_layernorm_bwd(q, p, null, p, p, p, p, p, null, 4, 8, BF16, BF16, None) == -3          # workspace missing
    # attention branch + MLP branch + residual in one pass
    assert lib.nhp_bias_add_residual_pair(q, p, p, p, p, p, 4, 8, 9, None) == -1
    assert lib.nhp_bias_add_residual_pair(q, p, p, p, p, p, -4, 8, BF16, None) == -2
    assert lib.nhp_bias_add_residual_pair(q, p, null, null, null, p, 4, 8, BF16, None) == -3   # x2 missing
    assert lib.nhp_bias_add_residual_pair(q, p, null, p, null, null, 4, 8, BF16, None) == -3   # residual missing
    assert lib.nhp_bias_add_residual_pair(null, null, null, null, null, null, 0, 8, BF16, None) == 0
    # two LayerNorms of one input
    assert lib.nhp_layernorm_pair_fwd(q, q2, null, null, p, p, p, p, p, 1e-5, 4, 8, 4, F32, None) == -1
    assert lib.nhp_layernorm_pair_fwd(q, q2, null, null, p, p, p, p, p, 1e-5, 4, 8, BF16, F16, None) == -1
    assert lib.nhp_layernorm_pair_fwd(q, q2, null, null, p, p, p, p, p, 1e-5, 4, -8, BF16, F32, None) == -2
    assert lib.nhp_layernorm_pair_fwd(q, null, null, null, p, p, p, p, p, 1e-5, 4, 8, BF16, F32, None) == -3   # y2 missing
    assert lib.nhp_layernorm_pair_fwd(q, q, null, null, p, p, p, p, p, 1e-5, 4, 8, BF16, F32, None) == -6      # y1 is y2
    assert lib.nhp_layernorm_pair_fwd(null, null, null, null, null, null, null, null, null, 1e-5, 0, 8, BF16, BF16, None) == 0
    assert lib.nhp_layernorm_pair_bwd(q, null, null, null, null, p, null, p, p, p, p, p, null, 4, 8, BF16, BF16, None) == -3
    assert lib.nhp_layernorm_pair_bwd(q, null, null, p, null, p, p, p, p, p, p, p, null, 4, 8, BF16, BF16, None) == -3  # workspace
    assert lib.nhp_layernorm_pair_bwd(q, null, null, null, null, p, p, p, p, p, p, p, null, 4, 8, 7, BF16, None) == -1
    assert lib.nhp_layernorm_pair_bwd_workspace_bytes(4096, 2048, BF16) == 2 * lib.nhp_norm_bwd_workspace_bytes(4096, 2048, BF16)
    assert lib.nhp_layernorm_pair_bwd_workspace_bytes(4096, 2048, 9) == 0
    assert lib.nhp_rmsnorm_fwd(q, null, p, p, null, 1e-5, 3, 4, 8, BF16, BF16, None) == -2               # eps_mode
    assert lib.nhp_rmsnorm_partial_fwd(q, null, p, p, null, 1e-5, 1, 4, 8, 0, BF16, BF16, None) == -2    # no statistic columns
    assert lib.nhp_rmsnorm_partial_fwd(q, null, p, p, null, 1e-5, 1, 4, 8, 9, BF16, BF16, None) == -2    # more than the row has
    assert lib.nhp_rmsnorm_partial_fwd(q, null, null, p, null, 1e-5, 1, 4, 8, 3, BF16, BF16, None) == -3
    assert lib.nhp_rmsnorm_partial_bwd(q, null, null, p, p, p, p, null, 1e-5, 1, 4, 8, 9, BF16, BF16, None) == -2
    assert lib.nhp_rmsnorm_bwd(q, null, null, p, p, null, p, null, 1e-5, 1, 4, 8, BF16, BF16, None) == -3  # inv missing
    assert lib.nhp_rmsnorm_bwd(q, null, null, p, p, p, p, null, 1e-5, 3, 4, 8, BF16, BF16, None) == -2
    assert lib.nhp_norm_bwd_workspace_bytes(4, 8, BF16) > 0
    assert lib.nhp_norm_bwd_workspace_bytes(4, 7, BF16) == 0
    assert lib.nhp_norm_bwd_workspace_bytes(4, 8, 11) == 0
    assert 0 < lib.nhp_norm_bwd_workspace_bytes(1 << 22, 2048, BF16) <= 2 * 4096 * 2048 * 4


def test_missing_library_fails_loudly(hotpath, monkeypatch, tmp_path):
    """No fallback: without the built library the binding raises ImportError."""
    monkeypatch.setattr(hotpath, "_lib", None)
    monkeypatch.setattr(hotpath, "LIB_PATH", str(tmp_path / "libneox_hotpath.so"))
    with pytest.raises(ImportError):
        hotpath.lib()


def test_probe_library_exports_and_validates():
    """bench.py's data-movement probes (bench_probes/libneox_probe.so, measurement equipment, not part of the
    product library): every entry point bench.py binds exists, and bad arguments are refused before any launch."""
    import ctypes
    import subprocess

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    path = os.path.join(root, "bench_probes", "libneox_probe.so")
    if not os.path.exists(path):
        subprocess.run(["make", "-C", os.path.dirname(path)], check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    lib = ctypes.CDLL(path)
    vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    sigs = {
        "nhp_probe_copy": [vp, vp, i64, ci, vp],
        "nhp_probe_streams": [vp, vp, vp, vp, i64, ci, ci, vp],
        "nhp_probe_causal_pattern": [vp, vp, i64, i64, vp],
        "nhp_probe_causal_bwd_pattern": [vp, vp, i64, i64, vp],
        "nhp_probe_masked_pattern": [vp, vp, vp, i64, i64, i64, vp],
        "nhp_probe_strided_runs": [vp, vp, vp, i64, ci, i64, ci, vp],
        "nhp_probe_seq_major_pattern": [vp, vp, i64, i64, vp],
    }
    for name, args in sigs.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = ci
    p = ctypes.c_void_p(0x1000)  # never dereferenced: every call below is refused
    shape, null = -2, -3
    assert lib.nhp_probe_copy(p, p, 24, 256, None) == shape          # not a multiple of 16 bytes
    assert lib.nhp_probe_copy(None, p, 32, 256, None) == null
    assert lib.nhp_probe_streams(p, p, p, p, 32, 4, 1, None) == shape
    assert lib.nhp_probe_causal_pattern(p, p, 1, 1000, None) == shape
    assert lib.nhp_probe_causal_bwd_pattern(p, None, 1, 2048, None) == null
    assert lib.nhp_probe_masked_pattern(p, p, p, 1, 3, 8, None) == shape  # odd number of heads
    assert lib.nhp_probe_strided_runs(p, None, p, 8, 24, 48, 0, None) == shape
    assert lib.nhp_probe_strided_runs(p, None, p, 8, 32, 48, 1, None) == null
    assert lib.nhp_probe_seq_major_pattern(p, p, 4, 100, None) == shape
