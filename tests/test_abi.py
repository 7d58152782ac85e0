"""The C-ABI library builds, loads without a GPU, and exports every symbol the header declares."""
import ctypes
import json
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "bamboo_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bb_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported():
    from bamboo_amd import hip
    lib = ctypes.CDLL(hip.library_path())
    syms = declared_symbols()
    assert len(syms) >= 15
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in include/bamboo_hip.h but not exported"
    assert sorted(hip.EXPORTS) == syms


def test_version_and_error_string():
    from bamboo_amd import hip
    L = hip.lib()
    assert L.bb_version() == 1
    # argument validation happens on the host before any HIP call: no GPU needed
    assert L.bb_gemm(None, None) == -1
    assert b"null descriptor" in L.bb_last_error()
    d = hip.GemmDesc()
    d.layout, d.dtype, d.c_dtype = 7, 0, 0
    assert L.bb_gemm(ctypes.byref(d), None) == -1
    assert b"bad layout" in L.bb_last_error()
    assert L.bb_residual_add(1, 12, 1, 1, 1, None) == -1      # bf16 needs n % 8 == 0
    assert L.bb_adam_multi(1, None, None, None, None, None, None, 1e-3, 0.9, 0.999, 1e-8, 0, 1, 1, 0.0, 0, None) == -1
    # the allocation-free LayerNorm backward refuses rows wider than its built-in scratch array
    one = ctypes.c_void_p(16)
    assert L.bb_layernorm_bwd_static(1, 0, 8, 4096, 1e-5, one, one, one, one, one, None, one, one, one, None) == -1
    assert b"beyond the built-in scratch" in L.bb_last_error()


def test_convolution_entry_points_validate_on_the_host():
    """What the implicit-GEMM convolution entry points take and refuse is decided on the host, before any HIP call."""
    from bamboo_amd import hip
    L = hip.lib()
    BF16, F32, FWD, DGRAD = hip.BF16, hip.F32, hip.CONV_FWD, hip.CONV_DGRAD
    ok = L.bb_conv3x3_supported
    assert ok(BF16, FWD, 32, 14, 14, 256, 256) == 1 and ok(BF16, DGRAD, 32, 14, 14, 256, 256) == 1
    assert ok(BF16, FWD, 4, 6, 6, 64, 72) == 1            # gathered channels % 64, produced % 8
    assert ok(BF16, FWD, 4, 6, 6, 96, 64) == 0            # 96 gathered channels: a k-tile would straddle two taps
    assert ok(BF16, DGRAD, 4, 6, 6, 64, 96) == 0          # the input gradient gathers the output channels
    assert ok(F32, FWD, 4, 6, 6, 64, 64) == 0 and ok(BF16, 2, 4, 6, 6, 64, 64) == 0
    assert ok(BF16, FWD, 3, 6, 6, 64, 64) == 0            # 108 pixels: fewer than one 128-row tile
    assert L.bb_conv3x3(BF16, FWD, 4, 6, 6, 96, 64, 16, 16, 16, None, None) == -1
    assert b"unsupported problem" in L.bb_last_error()
    assert L.bb_conv3x3(BF16, FWD, 4, 6, 6, 64, 64, None, None, None, None, None) == -1
    assert b"null operand" in L.bb_last_error()
    assert L.bb_strip_stats_workspace(6272, 256) == 196 * 3 * 256 and L.bb_strip_stats_workspace(33, 8) == 2 * 3 * 8
    # a patch-matrix B (weight gradient of the 3x3 convolution) is a BB_TN, bf16, unbatched affair
    d = hip.GemmDesc()
    d.layout, d.dtype, d.c_dtype = hip.TN, BF16, F32
    d.M, d.N, d.K, d.nb1, d.nb2 = 256, 9 * 128, 288, 1, 1
    d.A, d.B, d.C, d.lda, d.ldb, d.ldc = 4096, 8192, 12288, 256, 128, 9 * 128
    d.alpha, d.accumulate = 1.0, 1
    d.conv_h, d.conv_w, d.conv_c = 6, 6, 96
    assert L.bb_gemm(ctypes.byref(d), None) == -1 and b"multiple of 128" in L.bb_last_error()
    d.conv_c, d.N = 128, 9 * 128 + 8
    assert L.bb_gemm(ctypes.byref(d), None) == -1 and b"9 * conv_c" in L.bb_last_error()
    d.N, d.layout = 9 * 128, hip.NN
    assert L.bb_gemm(ctypes.byref(d), None) == -1 and b"BB_TN" in L.bb_last_error()
    d.layout, d.conv_h, d.conv_w = hip.TN, 2, 8          # 32 consecutive pixels span two whole images
    assert L.bb_gemm(ctypes.byref(d), None) == -1 and b"image boundary" in L.bb_last_error()
    # strip statistics: only where the kernels that carry them run
    s = hip.GemmDesc()
    s.layout, s.dtype, s.c_dtype, s.M, s.N, s.K, s.nb1, s.nb2, s.alpha = hip.NT, BF16, BF16, 6272, 256, 1024, 1, 1, 1.0
    assert L.bb_gemm_strip_stats_supported(ctypes.byref(s)) == 1
    s.K = 96
    assert L.bb_gemm_strip_stats_supported(ctypes.byref(s)) == 0
    s.K, s.layout = 1024, hip.NN
    assert L.bb_gemm_strip_stats_supported(ctypes.byref(s)) == 0


def test_gemm_desc_layout_matches_header():
    """Field order of the ctypes mirror follows the struct in the header."""
    from bamboo_amd import hip
    text = open(os.path.join(ROOT, "include", "bamboo_hip.h")).read()
    body = text[text.index("typedef struct bb_gemm_desc {"): text.index("} bb_gemm_desc;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.replace("typedef struct bb_gemm_desc {", "").strip()
        if not decl:
            continue
        parts = decl.split(",")
        first = parts[0].split()[-1].lstrip("*")
        names.append(first)
        names += [p.strip().lstrip("*") for p in parts[1:]]
    assert names == [f[0] for f in hip.GemmDesc._fields_]


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")


def test_partition_known_answers():
    """The partitioning known answers of the reference's unit tests (tests/unit/test_partition.py:95-193),
    kept as data in tests/golden/."""
    from bamboo_amd.utils import partition_balanced, partition_uniform
    kat = json.load(open(GOLDEN))
    for c in kat["partition_uniform"]["cases"]:
        assert partition_uniform(c["num_items"], c["num_parts"]) == c["parts"]
    assert partition_uniform(2, 4) == [0, 1, 2, 2, 2]
    for c in kat["partition_balanced"]["cases"]:
        assert partition_balanced(c["weights"], c["num_parts"]) == c["parts"]
    for c in kat["partition_balanced_valid_only"]["cases"]:
        w, parts = c["weights"], partition_balanced(c["weights"], c["num_parts"])
        # assert_valid_partition of the reference: P+1 non-decreasing bounds from 0 to N
        assert len(parts) == c["num_parts"] + 1 and parts[0] == 0 and parts[-1] == len(w)
        assert all(a <= b for a, b in zip(parts, parts[1:]))
    w = kat["partition_balanced_valid_only"]["cases"][1]["weights"]
    parts = partition_balanced(w, 8)
    heaviest = max(sum(w[a:b]) for a, b in zip(parts, parts[1:]))
    assert heaviest <= 52559872 + 12596224        # optimum: one end layer plus at most one transformer layer


def test_layer_parameter_count_matches_reference_figure():
    """12h^2 + 13h parameters per encoder layer at f = 4h: the figure the reference's partition test uses."""
    kat = json.load(open(GOLDEN))["transformer_layer_parameters"]
    h, f = kat["hidden"], kat["ffn"]
    assert 4 * (h * h + h) + 2 * h * f + f + h + 4 * h == kat["params"]
    from bamboo_amd.layers import TransformerLayer
    assert TransformerLayer(h, 16, f).num_params() == kat["params"]


def test_config_batch_triad():
    from bamboo_amd.config import BambooConfig
    c = BambooConfig({"train_batch_size": 128, "train_micro_batch_size_per_gpu": 8})
    assert c.gradient_accumulation_steps == 16
    c = BambooConfig({"train_micro_batch_size_per_gpu": 4, "gradient_accumulation_steps": 8, "bf16": {"enabled": True}})
    assert c.train_batch_size == 32 and c.bf16
    with pytest.raises(ValueError):
        BambooConfig({"train_batch_size": 10, "train_micro_batch_size_per_gpu": 4, "gradient_accumulation_steps": 2})
    assert (c.lr, c.betas, c.eps, c.weight_decay, c.adam_w_mode) == (1e-3, (0.9, 0.999), 1e-8, 0.0, True)


def test_engine_flag_errors_without_gpu():
    """eager_recovery without redundancy, and level > 1, are rejected as in the reference
    (engine.py:173-181); checked through the flag logic only (no device work)."""
    from bamboo_amd.utils import get_redundant_stage_ids
    assert get_redundant_stage_ids(1, 1, 4) == [2]
    assert get_redundant_stage_ids(0, 1, 4) == []


def test_wrappers_refuse_operands_that_do_not_fit_before_any_launch():
    """The C ABI takes raw pointers; the ctypes layer checks what a kernel and its grid assume about its operands
    (shapes, dtypes, contiguity) and raises before anything is launched -- here on CPU tensors, without a GPU."""
    import pytest
    import torch

    from bamboo_amd import hip
    bf, f32 = torch.bfloat16, torch.float32
    batch, heads, seq = 2, 2, 64
    h = heads * 64
    qkv, out = torch.zeros(batch * seq, 3 * h, dtype=bf), torch.zeros(batch * seq, h, dtype=bf)
    lse = torch.zeros(batch, heads, seq)
    with pytest.raises(hip.HipKernelError, match="qkv must be"):
        hip.attention_fwd(qkv, out, lse, batch + 1, heads, seq, 0)              # more samples than the tensor holds
    with pytest.raises(hip.HipKernelError, match="lse"):
        hip.attention_fwd(qkv, out, lse[:, :1], batch, heads, seq, 0)
    with pytest.raises(hip.HipKernelError, match="key_len"):
        hip.attention_fwd(qkv, out, lse, batch, heads, seq, 2, key_len=torch.zeros(batch + 1, dtype=torch.int32))
    with pytest.raises(hip.HipKernelError, match="d_qkv"):
        hip.attention_bwd(qkv, out, out.clone(), lse, lse.clone(), qkv[:-1], batch, heads, seq, 0)
    x = torch.zeros(16, 32, dtype=bf)
    with pytest.raises(hip.HipKernelError, match="mean"):
        hip.layernorm_fwd(x, torch.zeros(32, dtype=bf), torch.zeros(32, dtype=bf), torch.zeros_like(x), torch.zeros(15), torch.zeros(16), 0, 1e-5)
    with pytest.raises(hip.HipKernelError, match="gain"):
        hip.layernorm_fwd(x, torch.zeros(32), torch.zeros(32, dtype=bf), torch.zeros_like(x), torch.zeros(16), torch.zeros(16), 0, 1e-5)
    with pytest.raises(hip.HipKernelError, match="contiguous"):
        hip.layernorm_fwd(x.t(), torch.zeros(16, dtype=bf), torch.zeros(16, dtype=bf), torch.zeros(32, 16, dtype=bf), torch.zeros(32), torch.zeros(32), 0, 1e-5)
    with pytest.raises(hip.HipKernelError, match="dy"):
        hip.batchnorm_bwd(x, torch.zeros(32, dtype=bf), torch.zeros(32), torch.zeros(32), x[:8], None, torch.zeros_like(x), None,
                          torch.zeros(32), torch.zeros(32), torch.zeros(1))
    with pytest.raises(hip.HipKernelError, match="out"):
        hip.residual_add(x, x, torch.zeros(16, 32))
    with pytest.raises(hip.HipKernelError, match="target"):
        hip.mse_fwd_bwd(x, x[:8], torch.zeros_like(x), 1.0, torch.zeros(1), False, torch.zeros(4096))
    with pytest.raises(hip.HipKernelError, match="cast"):
        hip.cast(x, torch.zeros(8, 32))


def test_batchnorm_backward_sums_and_head_pairs_validate_on_the_host():
    """The entry points of the BatchNorm backward sums and the fused attention's head widths: refused on the host,
    before any HIP call, when the problem is not one the kernels take."""
    from bamboo_amd import hip
    L = hip.lib()
    BF16, F32 = hip.BF16, hip.F32
    one = ctypes.c_void_p(16)
    assert L.bb_bn_bwd_strips_workspace(6272, 256) == 196 * 2 * 256 and L.bb_bn_bwd_strips_workspace(33, 8) == 2 * 2 * 8
    # fp32 has no strip-sum kernels
    assert L.bb_batchnorm_bwd_strip_sums(F32, 64, 64, one, one, one, one, None, None, one, None) == -1
    assert b"bf16 only" in L.bb_last_error()
    # a ReLU needs a place for the masked gradient
    assert L.bb_batchnorm_bwd_strip_sums(BF16, 64, 64, one, one, one, one, one, None, one, None) == -1
    assert b"masked gradient" in L.bb_last_error()
    assert L.bb_batchnorm_bwd_strips(BF16, 64, 64, one, one, one, one, one, None, one, one, one, None) == -1
    assert b"null pointer" in L.bb_last_error()
    # the GEMM with the sums: an NN product whose C is contiguous, no bias, no accumulation
    d = hip.GemmDesc()
    d.layout, d.dtype, d.c_dtype, d.M, d.N, d.K = hip.NN, BF16, BF16, 6272, 256, 1024
    d.A, d.B, d.C, d.lda, d.ldb, d.ldc, d.alpha = 16, 16, 16, 1024, 256, 256, 1.0
    assert L.bb_gemm_bn_bwd_supported(ctypes.byref(d)) == 1
    d.ldc = 512
    assert L.bb_gemm_bn_bwd_supported(ctypes.byref(d)) == 0
    d.ldc, d.layout = 256, hip.NT
    assert L.bb_gemm_bn_bwd_supported(ctypes.byref(d)) == 0
    d.layout, d.K = hip.NN, 96
    assert L.bb_gemm_bn_bwd_supported(ctypes.byref(d)) == 0
    assert L.bb_gemm_bn_bwd(ctypes.byref(d), None, None) == -1 and b"bb_gemm_bn_bwd: needs" in L.bb_last_error()
    d.K = 1024
    bn = hip.BnBwdStats(16, 16, 16, None)
    assert L.bb_gemm_bn_bwd(ctypes.byref(d), ctypes.byref(bn), None) == -1 and b"null pointer in bb_bn_bwd_stats" in L.bb_last_error()
    # attention: 64-wide heads, or an even number of 32-wide ones
    args = lambda heads, dim: (BF16, 0, 1, heads, 64, dim, one, one, one, 3 * heads * dim, one, heads * dim, one, None, 0.0, 0, 0, None)
    assert L.bb_attention_fwd(*args(3, 32)) == -1 and b"even number of heads" in L.bb_last_error()
    assert L.bb_attention_fwd(*args(2, 96)) == -1 and b"head dimension" in L.bb_last_error()
