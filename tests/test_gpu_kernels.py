"""Kernel parity on the GPU, called through the C ABI: every kernel against the oracle / a plain
torch fp32 statement of the same operation on the same seeded inputs.

Tolerances: fp32 relative 1e-5 of the tensor's scale (accumulation order differs from the
CPU's), bf16 relative 2e-2; Adam is compared bit for bit with the oracle formula."""
import math

import numpy as np
import pytest
import torch

from oracle import adam as oadam
from oracle import layers as ol

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return 1e-5 if dtype == torch.float32 else 2e-2


def rel_err(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def randn(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


GEMM_SHAPES = [(256, 256, 64), (512, 384, 128), (304, 200, 96), (64, 1024, 256), (1024, 64, 512),
               (136, 72, 40), (2048, 768, 768), (8, 8, 8),
               # ragged edges under the 256x128 tiles with 64-wide k-tiles (two and three stages)
               (4000, 1496, 1024), (2104, 2000, 2048), (4000, 1496, 128),
               # NT: 256x192 tiles (three accumulator tiles across a wave: the epilogue's single-tile tail)
               (4000, 4792, 192)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layout", [0, 1, 2])
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gemm_layouts(hiplib, dtype, layout, M, N, K):
    a_shape = (K, M) if layout == hiplib.TN else (M, K)
    b_shape = (N, K) if layout == hiplib.NT else (K, N)
    A, B = randn(*a_shape, dtype=dtype, seed=1), randn(*b_shape, dtype=dtype, seed=2)
    C = torch.full((M, N), float("nan"), dtype=dtype, device=DEV)
    hiplib.gemm(layout, A, B, C)
    Af, Bf = A.double().cpu(), B.double().cpu()
    ref = (Af.t() if layout == hiplib.TN else Af) @ (Bf.t() if layout == hiplib.NT else Bf)
    assert rel_err(C, ref) < tol(dtype)
    # determinism: a second run is bit-identical
    C2 = torch.empty_like(C)
    hiplib.gemm(layout, A, B, C2)
    assert torch.equal(C, C2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_epilogues(hiplib, dtype):
    M, N, K = 384, 512, 256
    A, W = randn(M, K, dtype=dtype, seed=3), randn(N, K, dtype=dtype, seed=4, scale=0.1)
    bias, R = randn(N, dtype=dtype, seed=5), randn(M, N, dtype=dtype, seed=6)
    Af, Wf, bf_, Rf = A.double().cpu(), W.double().cpu(), bias.double().cpu(), R.double().cpu()
    lin = Af @ Wf.t() + bf_
    C = torch.empty(M, N, dtype=dtype, device=DEV)
    hiplib.gemm(hiplib.NT, A, W, C, bias=bias)
    assert rel_err(C, lin) < tol(dtype)
    hiplib.gemm(hiplib.NT, A, W, C, bias=bias, epilogue=hiplib.EPI_RESIDUAL, resid=R)
    assert rel_err(C, lin + Rf) < tol(dtype)
    for act, name in ((hiplib.ACT_RELU, "relu"), (hiplib.ACT_GELU_TANH, "gelu_tanh")):
        U = torch.empty_like(C)
        hiplib.gemm(hiplib.NT, A, W, C, bias=bias, epilogue=hiplib.EPI_ACT, act=act, aux_out=U)
        assert rel_err(U, lin) < tol(dtype)
        assert rel_err(C, ol.activation(lin, name)) < tol(dtype)
        # dact: C = (A W^T) * act'(U)
        Uf = U.double().cpu().requires_grad_(True)
        ol.activation(Uf, name).sum().backward()
        hiplib.gemm(hiplib.NT, A, W, C, epilogue=hiplib.EPI_DACT, act=act, aux_in=U)
        assert rel_err(C, (Af @ Wf.t()) * Uf.grad) < tol(dtype)
        # act and act' from one epilogue: C = act(v), aux_out = act'(v) (from the unrounded v)
        D = torch.empty_like(C)
        hiplib.gemm(hiplib.NT, A, W, C, bias=bias, epilogue=hiplib.EPI_ACT_DACT, act=act, aux_out=D)
        lf = lin.clone().requires_grad_(True)
        ol.activation(lf, name).sum().backward()
        assert rel_err(C, ol.activation(lin, name)) < tol(dtype)
        if name == "relu":   # a step function: compare away from the step
            far = lin.abs() > 1e-2
            assert torch.equal(D.double().cpu()[far], lf.grad[far])
        else:
            assert rel_err(D, lf.grad) < tol(dtype)
        # a redundant forward writes act alone and the backward after a failover runs ACT_DACT over the
        # same operands: both must give the same act, bit for bit
        C1 = torch.empty_like(C)
        hiplib.gemm(hiplib.NT, A, W, C1, bias=bias, epilogue=hiplib.EPI_ACT, act=act)
        assert torch.equal(C1, C)
    # mul: C = (A W^T) * R
    hiplib.gemm(hiplib.NT, A, W, C, epilogue=hiplib.EPI_MUL, aux_in=R)
    assert rel_err(C, (Af @ Wf.t()) * Rf) < tol(dtype)
    # mul_pos: C = alpha (A W^T) where R > 0, else 0 -- the gradient through a ReLU whose output R was kept; exactly
    # the alpha-product where it passes, exactly zero elsewhere, and equal to MUL with the 0 / 1 mask
    Rz = torch.where(R.abs() < 0.3, torch.zeros_like(R), R)     # zeros of its own, like a ReLU output
    hiplib.gemm(hiplib.NT, A, W, C, epilogue=hiplib.EPI_MUL_POS, aux_in=Rz, alpha=1.25)
    pos = (Rz > 0)
    assert rel_err(C, 1.25 * (Af @ Wf.t()) * pos.double().cpu()) < tol(dtype)
    assert not C[~pos].any()
    Cm = torch.empty_like(C)
    hiplib.gemm(hiplib.NT, A, W, Cm, epilogue=hiplib.EPI_MUL, aux_in=pos.to(dtype), alpha=1.25)
    assert torch.equal(C, Cm)
    # fp32 accumulate (weight-gradient form): G += A^T B
    G0 = randn(K, N, dtype=torch.float32, seed=7)
    G = G0.clone()
    Bm = randn(M, N, dtype=dtype, seed=8)
    hiplib.gemm(hiplib.TN, A, Bm, G, accumulate=True)
    assert rel_err(G, G0.double().cpu() + Af.t() @ Bm.double().cpu()) < tol(dtype)
    # alpha
    hiplib.gemm(hiplib.NT, A, W, C, alpha=0.125)
    assert rel_err(C, 0.125 * (Af @ Wf.t())) < tol(dtype)


@pytest.mark.parametrize("layout,M,N,K", [(lay, *shape) for shape in [(7168, 4096, 576), (7100, 4104, 640), (8192, 4096, 1024)]
                                          for lay in ("nt", "nn")] + [("nn", 7168, 4096, 128)])
def test_gemm_persistent_blocks(hiplib, layout, M, N, K):
    """More than one round of 256x256 tiles: the blocks of the persistent kernel walk several tiles each with the
    k-tile stream running through the tile boundaries.  Every epilogue kind against fp64 (ragged edges included), and
    bit for bit against the same product cut into row slabs small enough for the one-tile-per-block kernels: the
    order of the contraction is the same in all of them."""
    dtype = torch.bfloat16
    lay = hiplib.NT if layout == "nt" else hiplib.NN
    A = randn(M, K, dtype=dtype, seed=11)
    W = randn(N, K, dtype=dtype, seed=12, scale=0.1) if layout == "nt" else randn(K, N, dtype=dtype, seed=12, scale=0.1)
    bias, X = randn(N, dtype=dtype, seed=13), randn(M, N, dtype=dtype, seed=14)
    C, D = torch.empty(M, N, dtype=dtype, device=DEV), torch.empty(M, N, dtype=dtype, device=DEV)
    assert hiplib.gemm_variant(hiplib.gemm_desc(lay, A, W, C)).endswith("dma256x256p")
    Af, Wf = A.double().cpu(), (W.double().cpu().t() if layout == "nt" else W.double().cpu())
    lin = Af @ Wf
    cases = {
        "plain": (dict(), lambda: lin),
        "bias": (dict(bias=bias), lambda: lin + bias.double().cpu()),
        "residual": (dict(bias=bias, epilogue=hiplib.EPI_RESIDUAL, resid=X), lambda: lin + bias.double().cpu() + X.double().cpu()),
        "mul": (dict(epilogue=hiplib.EPI_MUL, aux_in=X), lambda: lin * X.double().cpu()),
        "act_dact": (dict(bias=bias, epilogue=hiplib.EPI_ACT_DACT, act=hiplib.ACT_GELU_TANH, aux_out=D),
                     lambda: ol.activation(lin + bias.double().cpu(), "gelu_tanh")),
    }
    slab = 1024
    for name, (kw, ref) in cases.items():
        C.fill_(float("nan"))
        hiplib.gemm(lay, A, W, C, **kw)
        assert rel_err(C, ref()) < tol(dtype), name
        if name == "plain":     # a second run gives the same bits (no atomics, fixed tile walk)
            C2 = torch.empty_like(C)
            hiplib.gemm(lay, A, W, C2, **kw)
            assert torch.equal(C, C2)
        if name == "act_dact":
            u = (lin + bias.double().cpu()).requires_grad_(True)
            ol.activation(u, "gelu_tanh").sum().backward()
            assert rel_err(D, u.grad) < tol(dtype)
        # row slabs: at most 4 x 17 tiles, far below a round, so another kernel runs them
        Cs, Ds = torch.empty_like(C), torch.empty_like(D)
        for r0 in range(0, M, slab):
            r1 = min(M, r0 + slab)
            kws = {k: (v[r0:r1] if k in ("resid", "aux_in") else v) for k, v in kw.items()}
            if "aux_out" in kws:
                kws["aux_out"] = Ds[r0:r1]
            assert not hiplib.gemm_variant(hiplib.gemm_desc(lay, A[r0:r1], W, Cs[r0:r1])).endswith("p")
            hiplib.gemm(lay, A[r0:r1], W, Cs[r0:r1], **kws)
        assert torch.equal(C, Cs), name
        if name == "act_dact":
            assert torch.equal(D, Ds)
    # fp32 output, accumulated into
    G0 = randn(M, N, dtype=torch.float32, seed=15)
    G = G0.clone()
    hiplib.gemm(lay, A, W, G, accumulate=True)
    assert rel_err(G, G0.double().cpu() + lin) < tol(dtype)


@pytest.mark.parametrize("layout", ["tn", "nt"])
def test_gemm_grouped_splitk(hiplib, layout):
    """Few output tiles, long contraction: chunks of the contraction into fp32 partials, added to C
    in chunk order.  Against fp64, against the unsplit grouped call, twice in a row (accumulate),
    and with a C that is a strided view."""
    torch.manual_seed(0)
    dtype = torch.bfloat16
    K = 6272
    shapes = [(1024, 256), (256, 2304), (256, 1024)]
    As, Bs, Cs, refs = [], [], [], []
    for i, (M, N) in enumerate(shapes):
        if layout == "tn":
            A, B = randn(K, M, dtype=dtype, seed=50 + i, scale=0.1), randn(K, N, dtype=dtype, seed=60 + i, scale=0.1)
            ref = A.double().cpu().t() @ B.double().cpu()
        else:
            A, B = randn(M, K, dtype=dtype, seed=50 + i, scale=0.1), randn(N, K, dtype=dtype, seed=60 + i, scale=0.1)
            ref = A.double().cpu() @ B.double().cpu().t()
        As.append(A); Bs.append(B); refs.append(ref)
    C0 = [randn(M, N, dtype=torch.float32, seed=70 + i) for i, (M, N) in enumerate(shapes)]
    lay = hiplib.TN if layout == "tn" else hiplib.NT
    # last C is a view with a larger leading dimension
    big = torch.zeros(shapes[2][0], shapes[2][1] + 64, device=DEV)
    Cs = [C0[0].clone(), C0[1].clone(), big[:, :shapes[2][1]]]
    Cs[2].copy_(C0[2])
    descs = [hiplib.gemm_desc(lay, A, B, C, accumulate=True) for A, B, C in zip(As, Bs, Cs)]
    ws = torch.empty(hiplib.gemm_splitk_workspace(descs) // 4, device=DEV)
    hiplib.gemm_grouped(descs, splitk_ws=ws)
    plain = [c.clone() for c in C0]
    hiplib.gemm_grouped([hiplib.gemm_desc(lay, A, B, C, accumulate=True) for A, B, C in zip(As, Bs, plain)])
    for C, c0, ref, pl in zip(Cs, C0, refs, plain):
        assert rel_err(C, c0.double().cpu() + ref) < tol(dtype)
        assert rel_err(C, pl) < 1e-5                     # same products, different fp32 summation order
    assert float(big[:, shapes[2][1]:].abs().max()) == 0.0   # nothing written past the view
    hiplib.gemm_grouped(descs, splitk_ws=ws)            # accumulates once more, reproducibly
    again = [c.clone() for c in Cs]
    for C, c0, ref in zip(Cs, C0, refs):
        assert rel_err(C, c0.double().cpu() + 2 * ref) < tol(dtype)
    Cs2 = [C0[0].clone(), C0[1].clone(), C0[2].clone()]
    d2 = [hiplib.gemm_desc(lay, A, B, C, accumulate=True) for A, B, C in zip(As, Bs, Cs2)]
    hiplib.gemm_grouped(d2, splitk_ws=ws); hiplib.gemm_grouped(d2, splitk_ws=ws)
    for a, b in zip(again, Cs2):
        assert torch.equal(a.contiguous(), b)
    # too small a workspace is an error, not a silent fallback
    with pytest.raises(hiplib.HipKernelError):
        hiplib.gemm_grouped(descs, splitk_ws=ws[:1024])
    # large groups are not cut: same call, same result as the plain grouped entry
    M, N = 1024, 4096
    A, B = randn(8192, M, dtype=dtype, seed=80, scale=0.1), randn(8192, N, dtype=dtype, seed=81, scale=0.1)
    c1, c2 = torch.zeros(M, N, device=DEV), torch.zeros(M, N, device=DEV)
    d_big = [hiplib.gemm_desc(hiplib.TN, A, B, c1, accumulate=True), hiplib.gemm_desc(hiplib.TN, A, B, c2, accumulate=True)]
    hiplib.gemm_grouped(d_big, splitk_ws=ws)
    ref_big = torch.zeros(M, N, device=DEV)
    hiplib.gemm(hiplib.TN, A, B, ref_big, accumulate=True)
    assert torch.equal(c1, ref_big) and torch.equal(c2, ref_big)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_batched_heads(hiplib, dtype):
    """Q K^T and P V over (batch, head) strides inside a [rows, 3h] buffer."""
    b, a, s, d = 2, 3, 128, 64
    h = a * d
    qkv = randn(b * s, 3 * h, dtype=dtype, seed=9, scale=0.5)
    P = torch.empty(b, a, s, s, dtype=dtype, device=DEV)
    es = qkv.element_size()
    hiplib.gemm_batched(hiplib.NT, hiplib.dtype_code(dtype), s, s, d, qkv.data_ptr(), 3 * h, (s * 3 * h, d),
                        qkv.data_ptr() + h * es, 3 * h, (s * 3 * h, d), P.data_ptr(), s, (a * s * s, s * s), b, a,
                        alpha=0.125)
    q = qkv[:, :h].double().cpu().view(b, s, a, d).transpose(1, 2)
    k = qkv[:, h:2 * h].double().cpu().view(b, s, a, d).transpose(1, 2)
    v = qkv[:, 2 * h:].double().cpu().view(b, s, a, d).transpose(1, 2)
    assert rel_err(P, 0.125 * q @ k.transpose(-1, -2)) < tol(dtype)
    ctx = torch.empty(b * s, h, dtype=dtype, device=DEV)
    hiplib.gemm_batched(hiplib.NN, hiplib.dtype_code(dtype), s, d, s, P.data_ptr(), s, (a * s * s, s * s),
                        qkv.data_ptr() + 2 * h * es, 3 * h, (s * 3 * h, d), ctx.data_ptr(), h, (s * h, d), b, a)
    ref = (P.double().cpu() @ v).transpose(1, 2).reshape(b * s, h)
    assert rel_err(ctx, ref) < tol(dtype)
    dV = torch.empty(b * s, h, dtype=dtype, device=DEV)
    hiplib.gemm_batched(hiplib.TN, hiplib.dtype_code(dtype), s, d, s, P.data_ptr(), s, (a * s * s, s * s),
                        ctx.data_ptr(), h, (s * h, d), dV.data_ptr(), h, (s * h, d), b, a)
    c4 = ctx.double().cpu().view(b, s, a, d).transpose(1, 2)
    ref = (P.double().cpu().transpose(-1, -2) @ c4).transpose(1, 2).reshape(b * s, h)
    assert rel_err(dV, ref) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_grouped_weight_gradients(hiplib, dtype):
    """Four dW += dy^T x products in one launch equal the four separate calls."""
    rows = 512
    shapes = [(256, 1024), (1024, 256), (256, 256), (768, 256)]      # (out_features, in_features)
    dys = [randn(rows, o, dtype=dtype, seed=40 + i) for i, (o, _) in enumerate(shapes)]
    xs = [randn(rows, k, dtype=dtype, seed=50 + i) for i, (_, k) in enumerate(shapes)]
    g0 = [randn(o, k, seed=60 + i) for i, (o, k) in enumerate(shapes)]
    one = [g.clone() for g in g0]
    for dy, x, g in zip(dys, xs, one):
        hiplib.gemm(hiplib.TN, dy, x, g, accumulate=True)
    grp = [g.clone() for g in g0]
    hiplib.gemm_grouped([hiplib.gemm_desc(hiplib.TN, dy, x, g, accumulate=True) for dy, x, g in zip(dys, xs, grp)])
    for a, b, dy, x, g in zip(one, grp, dys, xs, g0):
        ref = g.double().cpu() + dy.double().cpu().t() @ x.double().cpu()
        assert rel_err(b, ref) < tol(dtype)
        assert rel_err(a, b.double().cpu()) < 1e-6


@pytest.mark.parametrize("layout", ["nt", "nn"])
@pytest.mark.parametrize("M,N,K", [(256, 192, 520),     # 33 k-tiles: the second wave group's share is one shorter
                                   (2048, 768, 768),    # C1's attention output projection
                                   (100, 72, 1036)])    # ragged rows, columns and contraction
def test_gemm_fp32_contraction_shared_by_wave_groups(hiplib, layout, M, N, K):
    """fp32 problems with fewer than two 64x64 tiles per CU and a long contraction take 64x32 tiles and deal the k-tiles
    of a tile to two groups of waves (partial tiles added in group order): against fp64 with bias, residual and accumulation, the same
    bits on a second call, and problems outside the rule keep the plain kernel."""
    lay = {"nt": hiplib.NT, "nn": hiplib.NN}[layout]
    A = randn(M, K, seed=120)
    B = randn(N, K, seed=121) if layout == "nt" else randn(K, N, seed=121)
    bias, resid, C0 = randn(N, seed=122), randn(M, N, seed=123), randn(M, N, seed=124)
    prod = A.double().cpu() @ (B.double().cpu().t() if layout == "nt" else B.double().cpu())
    C = torch.empty(M, N, device=DEV)
    assert hiplib.gemm_variant(hiplib.gemm_desc(lay, A, B, C)).endswith("64x32k2")
    hiplib.gemm(lay, A, B, C, bias=bias, epilogue=hiplib.EPI_RESIDUAL, resid=resid)
    assert rel_err(C, prod + bias.double().cpu() + resid.double().cpu()) < 1e-5
    C2 = torch.zeros_like(C)
    hiplib.gemm(lay, A, B, C2, bias=bias, epilogue=hiplib.EPI_RESIDUAL, resid=resid)
    assert torch.equal(C, C2)
    Ca = C0.clone()
    hiplib.gemm(lay, A, B, Ca, accumulate=True, alpha=0.5)
    assert rel_err(Ca, C0.double().cpu() + 0.5 * prod) < 1e-5
    # a short contraction, many tiles, or the weight-gradient layout: the plain kernels
    assert hiplib.gemm_variant(hiplib.gemm_desc(lay, A[:, :256], B[:, :256] if layout == "nt" else B[:256], C)).endswith("64x64")
    big = torch.empty(2048, 3072, device=DEV)
    Bb = torch.empty(3072, K, device=DEV) if layout == "nt" else torch.empty(K, 3072, device=DEV)
    assert hiplib.gemm_variant(hiplib.gemm_desc(lay, torch.empty(2048, K, device=DEV), Bb, big)).endswith("64x64")
    assert hiplib.gemm_variant(hiplib.gemm_desc(hiplib.TN, torch.empty(K, M, device=DEV), torch.empty(K, N, device=DEV), C)).endswith("64x64")


@pytest.mark.parametrize("layout", ["tn", "nt", "nn"])
def test_gemm_grouped_fp32_shares_a_launch_bit_equal(hiplib, layout):
    """fp32 problems that take the small tile share one launch: ragged shapes (rows, columns and contraction that are
    no multiples of the tile or the k-step), bias-gradient column sums on the weight-gradient layout, an accumulating
    and a plain problem side by side -- every output bit-equal to the calls made one by one."""
    K = 200
    shapes = [(100, 72), (260, 132), (64, 64), (36, 300)]
    lay = {"tn": hiplib.TN, "nt": hiplib.NT, "nn": hiplib.NN}[layout]
    mk = lambda *sh, seed: randn(*sh, seed=seed)
    ops = []
    for i, (M, N) in enumerate(shapes):
        A = mk(K, M, seed=80 + i) if layout == "tn" else mk(M, K, seed=80 + i)
        B = mk(N, K, seed=90 + i) if layout == "nt" else mk(K, N, seed=90 + i)
        ops.append((A, B, mk(M, N, seed=100 + i), mk(M, seed=110 + i)))
    ws = torch.empty(hiplib.colsum_workspace(max(m for m, _ in shapes)), device=DEV)
    def run(grouped):
        Cs, sums, descs = [c.clone() for _, _, c, _ in ops], [b.clone() for _, _, _, b in ops], []
        for i, ((A, B, _, _), C, bsum) in enumerate(zip(ops, Cs, sums)):
            kw = dict(accumulate=i % 2 == 0)
            if layout == "tn":
                kw.update(colsum_out=bsum, colsum_ws=ws)
            descs.append(hiplib.gemm_desc(lay, A, B, C, **kw))
        if grouped:
            hiplib.gemm_grouped(descs)
        else:
            for d in descs:
                hiplib.gemm_grouped([d])
        torch.cuda.synchronize()
        return Cs, sums
    c1, s1 = run(False)
    c2, s2 = run(True)
    for i, ((A, B, C0, b0), a, b) in enumerate(zip(ops, c1, c2)):
        assert torch.equal(a, b), i
        Ad, Bd = A.double().cpu(), B.double().cpu()
        ref = (Ad.t() if layout == "tn" else Ad) @ (Bd.t() if layout == "nt" else Bd) + (C0.double().cpu() if i % 2 == 0 else 0)
        assert rel_err(b, ref) < 1e-5, i
    if layout == "tn":
        for i, ((A, _, _, b0), x, y) in enumerate(zip(ops, s1, s2)):
            assert torch.equal(x, y) and rel_err(y, b0.double().cpu() + A.double().cpu().sum(0)) < 1e-5, i


def test_gemm_rejects_bad_arguments(hiplib):
    A = torch.zeros(16, 12, dtype=torch.bfloat16, device=DEV)   # K = 12 is not a multiple of 8
    B = torch.zeros(16, 12, dtype=torch.bfloat16, device=DEV)
    C = torch.zeros(16, 16, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(hiplib.HipKernelError):
        hiplib.gemm(hiplib.NT, A, B, C)
    A8 = torch.zeros(16, 8, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(hiplib.HipKernelError):
        hiplib.gemm(hiplib.NT, A8, A8, C, accumulate=True)  # accumulate needs fp32 C
    # empty problem is a no-op
    hiplib.gemm(hiplib.NT, A8[:0], A8, C[:0])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["standard", "annotated"])
@pytest.mark.parametrize("rows,cols", [(64, 768), (37, 1024), (16, 1600), (5, 64), (3, 4096),
                                       (2100, 1600),   # every wave of every block owns rows, some two (8 waves in bf16)
                                       (300, 2048),    # fp32: 8 waves, bf16: 8 waves at their widest row
                                       (130, 6144)])   # bf16 only: 4 waves, sums through the three LDS slots
def test_layernorm_fwd_bwd(hiplib, dtype, kind, rows, cols):
    if cols > 4096 and dtype == torch.float32:
        pytest.skip("fp32 rows hold at most 4096 columns")
    eps = 1e-6 if kind == "annotated" else 1e-5
    x, dy, dres = randn(rows, cols, dtype=dtype, seed=10), randn(rows, cols, dtype=dtype, seed=11), randn(rows, cols, dtype=dtype, seed=12)
    g = (1 + 0.1 * randn(cols, seed=13)).to(dtype)
    b = (0.1 * randn(cols, seed=14)).to(dtype)
    y = torch.empty_like(x)
    mean, rinv = torch.empty(rows, device=DEV), torch.empty(rows, device=DEV)
    hiplib.layernorm_fwd(x, g, b, y, mean, rinv, hiplib.LN_CODES[kind], eps)
    xr = x.double().cpu().requires_grad_(True)
    gr, br = g.double().cpu().requires_grad_(True), b.double().cpu().requires_grad_(True)
    yr = ol.layer_norm(xr, gr, br, kind, eps)
    assert rel_err(y, yr.detach()) < tol(dtype)
    yr.backward(dy.double().cpu())
    dx = torch.empty_like(x)
    dg0, db0 = randn(cols, seed=15), randn(cols, seed=16)
    dg, db = dg0.clone(), db0.clone()
    ws = torch.empty(hiplib.layernorm_bwd_workspace(cols), device=DEV)
    hiplib.layernorm_bwd(x, g, mean, rinv, dy, dres, dx, dg, db, ws, hiplib.LN_CODES[kind], eps)
    assert rel_err(dx, xr.grad + dres.double().cpu()) < tol(dtype)
    assert rel_err(dg - dg0, gr.grad) < tol(dtype) * 2
    assert rel_err(db - db0, br.grad) < tol(dtype) * 2
    hiplib.layernorm_bwd(x, g, mean, rinv, dy, None, dx, dg, db, ws, hiplib.LN_CODES[kind], eps)
    assert rel_err(dx, xr.grad) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mask", ["none", "causal", "key_padding"])
def test_softmax(hiplib, dtype, mask):
    b, a, s = 3, 2, 256
    sc = randn(b, a, s, s, dtype=dtype, seed=17, scale=2.0)
    lens = torch.tensor([256, 1, 100], dtype=torch.int32, device=DEV) if mask == "key_padding" else None
    ref_in = sc.double().cpu()
    cfg = ol.TransformerCfg(hidden=8, heads=a, ffn=8, mask=mask)
    m = ol.build_mask(cfg, b, s, None if lens is None else lens.cpu())
    if m is not None:
        ref_in = ref_in.masked_fill(~m, -1e9)
    ref = torch.softmax(ref_in, -1)
    p = sc.clone()
    hiplib.softmax_fwd(p, hiplib.MASK_CODES[mask], lens)
    assert float((p.double().cpu() - ref).abs().max()) < (1e-6 if dtype == torch.float32 else 4e-3)
    if mask == "causal":
        assert float(p[:, :, 0, 1:].abs().max()) == 0.0
    dp = randn(b, a, s, s, dtype=dtype, seed=18)
    pr = p.double().cpu()
    dref = pr * (dp.double().cpu() - (dp.double().cpu() * pr).sum(-1, keepdim=True))
    hiplib.softmax_bwd(p, dp)
    assert rel_err(dp, dref) < tol(dtype)


@pytest.mark.parametrize("mask", ["none", "causal", "key_padding"])
@pytest.mark.parametrize("b,a,s,d", [(2, 3, 128, 64), (1, 2, 64, 64), (2, 2, 96, 64), (1, 4, 384, 64), (3, 1, 32, 64), (1, 16, 1024, 64),
                                     (2, 6, 128, 32), (1, 2, 64, 32), (2, 4, 96, 32), (3, 2, 32, 32), (1, 16, 1024, 32),
                                     (2, 3, 128, 128), (1, 2, 64, 128), (2, 1, 96, 128), (3, 1, 32, 128), (1, 8, 1024, 128)])
def test_fused_attention_fwd_bwd(hiplib, mask, b, a, s, d):
    """Fused attention (bf16, d = 64, d = 32 with the heads taken in pairs, d = 128 as two 64-wide column panels) against
    softmax(QK^T/sqrt(d), mask) V and its autograd gradients, computed in fp64 from the same bf16 inputs."""
    h = a * d
    qkv = randn(b * s, 3 * h, dtype=torch.bfloat16, seed=70, scale=1.0)
    d_out = randn(b * s, h, dtype=torch.bfloat16, seed=71)
    lens = None
    if mask == "key_padding":
        g = torch.Generator().manual_seed(3)
        lens = torch.randint(max(1, s // 4), s + 1, (b,), generator=g, dtype=torch.int32)
        lens[0] = s
    out = torch.full((b * s, h), float("nan"), dtype=torch.bfloat16, device=DEV)
    lse = torch.empty(b, a, s, device=DEV)
    kl = None if lens is None else lens.to(DEV)
    hiplib.attention_fwd(qkv, out, lse, b, a, s, hiplib.MASK_CODES[mask], kl)
    x = qkv.double().cpu().requires_grad_(True)
    q, k, v = [x[:, i * h:(i + 1) * h].view(b, s, a, d).transpose(1, 2) for i in range(3)]
    sc = q @ k.transpose(-1, -2) / math.sqrt(d)
    m = ol.build_mask(ol.TransformerCfg(hidden=h, heads=a, ffn=8, mask=mask), b, s, lens)
    if m is not None:
        sc = sc.masked_fill(~m, -1e9)
    ref = (torch.softmax(sc, -1) @ v).transpose(1, 2).reshape(b * s, h)
    l2 = lambda t, r: float((t.double().cpu() - r).norm() / r.norm())
    assert l2(out, ref.detach()) < 1e-2
    ref_lse = torch.logsumexp(sc, -1) / math.log(2.0)
    assert float((lse.double().cpu() - ref_lse.detach()).abs().max()) < 2e-2
    ref.backward(d_out.double().cpu())
    d_qkv = torch.full((b * s, 3 * h), float("nan"), dtype=torch.bfloat16, device=DEV)
    delta = torch.empty(b, a, s, device=DEV)
    hiplib.attention_bwd(qkv, out, d_out, lse, delta, d_qkv, b, a, s, hiplib.MASK_CODES[mask], kl)
    for i, name in enumerate("qkv"):
        got, want = d_qkv[:, i * h:(i + 1) * h], x.grad[:, i * h:(i + 1) * h]
        assert torch.isfinite(got.float()).all(), name
        assert l2(got, want) < 2e-2, (name, l2(got, want))
    # determinism
    out2, d2 = torch.empty_like(out), torch.empty_like(d_qkv)
    hiplib.attention_fwd(qkv, out2, lse, b, a, s, hiplib.MASK_CODES[mask], kl)
    hiplib.attention_bwd(qkv, out2, d_out, lse, delta, d2, b, a, s, hiplib.MASK_CODES[mask], kl)
    assert torch.equal(out, out2) and torch.equal(d_qkv, d2)


def test_fused_attention_rejects(hiplib):
    qkv = torch.zeros(64, 3 * 64, device=DEV)
    with pytest.raises(hiplib.HipKernelError):
        hiplib.attention_fwd(qkv, torch.zeros(64, 64, device=DEV), torch.zeros(1, 1, 64, device=DEV), 1, 1, 64, 0)  # fp32
    # 32-wide heads go in pairs: an odd number of them is refused (by the wrapper, and by the library itself)
    q3 = torch.zeros(64, 3 * 96, dtype=torch.bfloat16, device=DEV)
    o3, l3 = torch.zeros(64, 96, dtype=torch.bfloat16, device=DEV), torch.zeros(1, 3, 64, device=DEV)
    with pytest.raises(hiplib.HipKernelError):
        hiplib.attention_fwd(q3, o3, l3, 1, 3, 64, 0)
    L = hiplib.lib()
    rc = L.bb_attention_fwd(hiplib.BF16, 0, 1, 3, 64, 32, q3.data_ptr(), q3.data_ptr() + 192, q3.data_ptr() + 384, 288, o3.data_ptr(), 96,
                            l3.data_ptr(), None, 0.0, 0, 0, None)
    assert rc != 0 and b"even number of heads" in L.bb_last_error()
    rc = L.bb_attention_fwd(hiplib.BF16, 0, 1, 1, 64, 96, q3.data_ptr(), q3.data_ptr(), q3.data_ptr(), 288, o3.data_ptr(), 96,
                            l3.data_ptr(), None, 0.0, 0, 0, None)
    assert rc != 0 and b"head dimension" in L.bb_last_error()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,cols", [(1000, 768), (8192, 3072), (7, 64), (513, 1600)])
def test_colsum(hiplib, dtype, rows, cols):
    x = randn(rows, cols, dtype=dtype, seed=19)
    out0 = randn(cols, seed=20)
    out = out0.clone()
    ws = torch.empty(hiplib.colsum_workspace(cols), device=DEV)
    hiplib.colsum_acc(x, out, ws)
    ref = out0.double().cpu() + x.double().cpu().sum(0)
    assert rel_err(out, ref) < 1e-5
    out2 = out0.clone()
    hiplib.colsum_acc(x, out2, ws)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_residual_add_cast_fill(hiplib, dtype):
    a, b = randn(1000, 64, dtype=dtype, seed=21), randn(1000, 64, dtype=dtype, seed=22)
    out = torch.empty_like(a)
    hiplib.residual_add(a, b, out)
    assert torch.equal(out, (a.float() + b.float()).to(dtype))
    src = randn(12345, seed=23)
    dst = torch.empty(12345, dtype=torch.bfloat16, device=DEV)
    hiplib.cast(src, dst)
    assert torch.equal(dst, src.to(torch.bfloat16))             # round-to-nearest-even both sides
    back = torch.empty(12345, device=DEV)
    hiplib.cast(dst, back)
    assert torch.equal(back, dst.float())
    f = torch.empty(777, device=DEV)
    hiplib.fill_f32(f, 3.5)
    assert float(f.min()) == float(f.max()) == 3.5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["relu", "gelu_tanh"])
def test_act_fwd(hiplib, dtype, name):
    x = randn(4096, 96, dtype=dtype, seed=26, scale=3.0)
    out = torch.empty_like(x)
    hiplib.act_fwd(x, out, hiplib.ACT_CODES[name])
    ref = ol.activation(x.double().cpu(), name)
    assert rel_err(out, ref) < tol(dtype)
    # with the derivative, written over the input
    xf = x.double().cpu().requires_grad_(True)
    ol.activation(xf, name).sum().backward()
    out2, x2 = torch.empty_like(x), x.clone()
    hiplib.act_fwd(x2, out2, hiplib.ACT_CODES[name], dact=x2)
    assert torch.equal(out2, out)
    assert rel_err(x2, xf.grad) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_fused_bias_gradient(hiplib, dtype):
    """dW += dy^T x with db += colsum(dy) riding in the same call, fused (bf16, large) or not."""
    for rows, out_f, in_f in [(512, 256, 384), (96, 40, 72)]:
        dy, x = randn(rows, out_f, dtype=dtype, seed=27), randn(rows, in_f, dtype=dtype, seed=28)
        g0, b0 = randn(out_f, in_f, seed=29), randn(out_f, seed=30)
        g, bgrad = g0.clone(), b0.clone()
        ws = torch.empty(hiplib.colsum_workspace(out_f), device=DEV)
        d = hiplib.gemm_desc(hiplib.TN, dy, x, g, accumulate=True, colsum_out=bgrad, colsum_ws=ws)
        hiplib.gemm_grouped([d])
        assert rel_err(g, g0.double().cpu() + dy.double().cpu().t() @ x.double().cpu()) < tol(dtype)
        assert rel_err(bgrad, b0.double().cpu() + dy.double().cpu().sum(0)) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,cols,relu,with_resid", [(144, 16, True, False), (6272, 256, True, False), (500, 64, True, True), (144, 64, False, False)])
def test_batchnorm_fwd_bwd(hiplib, dtype, rows, cols, relu, with_resid):
    x = randn(rows, cols, dtype=dtype, seed=31, scale=2.0) + 0.5
    gamma = (1 + 0.1 * randn(cols, seed=32)).to(dtype)
    beta = (0.1 * randn(cols, seed=33)).to(dtype)
    resid = randn(rows, cols, dtype=dtype, seed=34) if with_resid else None
    dy = randn(rows, cols, dtype=dtype, seed=35)
    y = torch.empty_like(x)
    mean, rstd = torch.empty(cols, device=DEV), torch.empty(cols, device=DEV)
    rm, rv = torch.zeros(cols, device=DEV), torch.ones(cols, device=DEV)
    ws = torch.empty(hiplib.bn_workspace(cols), device=DEV)
    hiplib.batchnorm_fwd(x, gamma, beta, resid, y, mean, rstd, rm, rv, ws, 1e-5, 0.1, relu)
    xr = x.double().cpu().requires_grad_(True)
    gr, br = gamma.double().cpu().requires_grad_(True), beta.double().cpu().requires_grad_(True)
    rm_ref, rv_ref = torch.zeros(cols, dtype=torch.float64), torch.ones(cols, dtype=torch.float64)
    z = torch.nn.functional.batch_norm(xr, rm_ref, rv_ref, gr, br, training=True, momentum=0.1, eps=1e-5)
    if with_resid:
        z = z + resid.double().cpu()
    yr = torch.relu(z) if relu else z
    assert rel_err(y, yr.detach()) < tol(dtype)
    assert rel_err(rm, rm_ref) < 1e-5 and rel_err(rv, rv_ref) < 1e-4
    yr.backward(dy.double().cpu())
    dx, g_out = torch.empty_like(x), torch.empty_like(x)
    dg0, db0 = randn(cols, seed=36), randn(cols, seed=37)
    dg, db = dg0.clone(), db0.clone()
    hiplib.batchnorm_bwd(x, gamma, mean, rstd, dy, y if relu else None, dx, g_out, dg, db, ws)
    t = tol(dtype) * (1 if dtype == torch.float32 else 1.5)
    assert rel_err(dx, xr.grad) < max(t, 1e-4)
    assert rel_err(dg - dg0, gr.grad) < max(t, 1e-4) and rel_err(db - db0, br.grad) < max(t, 1e-4)
    mask = (yr.detach() > 0) if relu else torch.ones_like(yr, dtype=torch.bool)
    assert rel_err(g_out, dy.double().cpu() * mask) < tol(dtype)
    # a redundant forward (no running buffers) leaves the statistics untouched and gives the same output
    y2 = torch.empty_like(y)
    rm2 = rm.clone()
    hiplib.batchnorm_fwd(x, gamma, beta, resid, y2, mean, rstd, None, None, ws, 1e-5, 0.1, relu)
    assert torch.equal(y, y2) and torch.equal(rm, rm2)


@pytest.mark.parametrize("kind", ["conv1x1", "conv1x1+skip", "conv3x3"])
@pytest.mark.parametrize("n,h,w,cm,co,relu", [(32, 14, 14, 256, 1024, True), (32, 14, 14, 1024, 256, True), (3, 10, 10, 128, 256, True),
                                              (5, 9, 7, 192, 128, False)])
def test_bn_bwd_sums_from_the_input_gradient(hiplib, kind, n, h, w, cm, co, relu):
    """The backward pass of BatchNorm -> ReLU -> convolution with the normalisation's sums taken from the epilogue of
    the convolution's input gradient: against the separate kernels (input gradient, then ``batchnorm_bwd`` with its own
    reduction pass), and against fp64.  The ResNet-152 conv4_x shape (6272 rows: 196 strips over 98 row tiles) and two
    with a ragged last strip, one of them with a column count that leaves half a pair of accumulator tiles."""
    dt, R = torch.bfloat16, n * h * w
    x = randn(R, cm, dtype=dt, seed=71, scale=2.0) + 0.5             # the normalisation's input
    gamma = (1 + 0.1 * randn(cm, seed=72)).to(dt)
    beta = (0.1 * randn(cm, seed=73)).to(dt)
    a = torch.empty_like(x)                                          # its (ReLU'd) output
    mean, rstd = torch.empty(cm, device=DEV), torch.empty(cm, device=DEV)
    ws = torch.empty(hiplib.bn_workspace(max(cm, co)), device=DEV)
    hiplib.batchnorm_fwd(x, gamma, beta, None, a, mean, rstd, None, None, ws, 1e-5, 0.1, relu)
    relu_out = a if relu else None
    if kind.startswith("conv1x1"):
        # "+skip": the gradient of a skip connection joins the product before the ReLU (what a bottleneck hands to
        # the block in front of it)
        skip = randn(R, cm, dtype=dt, seed=78) if kind.endswith("skip") else None
        dy_next = randn(R, co, dtype=dt, seed=74)
        wt = randn(co, cm, dtype=dt, seed=75, scale=co ** -0.5)
        plain = lambda dst: hiplib.gemm(hiplib.NN, dy_next, wt, dst, **(dict(epilogue=hiplib.EPI_RESIDUAL, resid=skip) if skip is not None else {}))
        fused = lambda dst, strips: hiplib.gemm_bn_bwd(dy_next, wt, dst, relu_out, x, mean, rstd, strips, resid=skip)
        assert hiplib.gemm_bn_bwd_supported(dy_next, wt, torch.empty_like(x), relu_out, skip)
        full = dy_next.double().cpu() @ wt.double().cpu() + (skip.double().cpu() if skip is not None else 0)
    else:
        dy_next = randn(R, co, dtype=dt, seed=74)
        if not hiplib.conv3x3_supported(dt, hiplib.CONV_DGRAD, n, h, w, cm, co):
            pytest.skip("the implicit input gradient does not take this shape")
        wt = randn(co, 3, 3, cm, dtype=dt, seed=75, scale=(9 * co) ** -0.5)
        plain = lambda dst: hiplib.conv3x3(hiplib.CONV_DGRAD, dy_next, wt, dst, n, h, w, cm, co)
        fused = lambda dst, strips: hiplib.conv3x3_dgrad_bn(dy_next, wt, dst, n, h, w, cm, co, relu_out, x, mean, rstd, strips)
        F = torch.nn.functional
        dn = dy_next.double().cpu().view(n, h, w, co).permute(0, 3, 1, 2)
        full = F.conv_transpose2d(dn, wt.double().cpu().permute(0, 3, 1, 2), padding=1).permute(0, 2, 3, 1).reshape(R, cm)
    # separate kernels
    d_a, dx0, g0 = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    dg_init, db_init = randn(cm, seed=76), randn(cm, seed=77)
    dg0, db0 = dg_init.clone(), db_init.clone()
    plain(d_a)
    hiplib.batchnorm_bwd(x, gamma, mean, rstd, d_a, relu_out, dx0, g0, dg0, db0, ws)
    # sums from the epilogue
    g1 = torch.full_like(x, 3.0)
    dx1 = torch.full_like(x, 5.0)
    strips = torch.full((hiplib.bn_bwd_strips_workspace(R, cm) + 8,), float("nan"), device=DEV)
    dg1, db1 = dg_init.clone(), db_init.clone()
    fused(g1, strips)
    hiplib.batchnorm_bwd_strips(x, gamma, mean, rstd, g1, strips, dx1, dg1, db1)
    torch.cuda.synchronize()
    assert torch.equal(g1, g0)                                  # the masked gradient: same products, same rounding
    assert bool(torch.isnan(strips[-8:]).all()) and not bool(torch.isnan(strips[:-8]).any())
    # fp64 from the stored gradient
    gd, xd = g1.double().cpu(), x.double().cpu()
    mask = (a.double().cpu() > 0) if relu else torch.ones_like(gd, dtype=torch.bool)
    assert rel_err(g1, full * mask) < 1e-2
    xhat = (xd - mean.double().cpu()) * rstd.double().cpu()
    sg, sgx = gd.sum(0), (gd * xhat).sum(0)
    scale_g, scale_gx = gd.abs().sum(0).max(), (gd * xhat).abs().sum(0).max()
    assert float(((db1 - db_init).double().cpu() - sg).abs().max() / scale_g) < 1e-5
    assert float(((dg1 - dg_init).double().cpu() - sgx).abs().max() / scale_gx) < 1e-5
    dx_ref = gamma.double().cpu() * rstd.double().cpu() * (gd - sg / R - xhat * sgx / R)
    assert rel_err(dx1, dx_ref) < 1e-2
    # and against the separate kernels: sums equal up to the fp32 order of addition, dx up to an ulp of bf16
    assert float((db1 - db0).abs().max() / scale_g) < 1e-5 and float((dg1 - dg0).abs().max() / scale_gx) < 1e-5
    assert float((dx1.float() - dx0.float()).abs().max() / dx0.float().abs().max()) < 2 ** -7
    # The pass that makes the strip sums where no epilogue left them adds up in the epilogues' order: from the
    # unmasked gradient of the plain kernel it gives the same strips, hence the same dx, dgamma and dbeta, bit for bit
    # (masked gradient in place).
    d_a2 = torch.empty_like(x)
    plain(d_a2)
    strips2 = torch.full_like(strips, float("nan"))
    dx2, dg2, db2 = torch.full_like(x, 7.0), dg_init.clone(), db_init.clone()
    hiplib.batchnorm_bwd_strip_sums(x, mean, rstd, d_a2, relu_out, d_a2 if relu else None, strips2)
    hiplib.batchnorm_bwd_strips(x, gamma, mean, rstd, d_a2, strips2, dx2, dg2, db2)
    torch.cuda.synchronize()
    assert torch.equal(d_a2, g1) and torch.equal(strips2[:-8], strips[:-8])
    assert torch.equal(dx2, dx1) and torch.equal(dg2, dg1) and torch.equal(db2, db1)
    # what does not fit is refused before anything is launched
    with pytest.raises(hiplib.HipKernelError):
        fused(g1, strips[: hiplib.bn_bwd_strips_workspace(R, cm) - 1])
    with pytest.raises(hiplib.HipKernelError):
        hiplib.batchnorm_bwd_strips(x, gamma, mean[:-1], rstd, g1, strips, dx1, dg1, db1)


@pytest.mark.parametrize("stride", [1, 2, 3])
@pytest.mark.parametrize("dtype", DTYPES)
def test_patch3x3_and_adjoint(hiplib, dtype, stride):
    """Patch matrix of nn.Conv2d(k=3, stride, padding=1) against torch's unfold, the product with the weight against
    conv2d, the adjoint against fold; odd image sides, so the last strided pixel's patch leaves the image."""
    F = torch.nn.functional
    n, h, w, c = 3, 5, 7, 16
    ho, wo = (h - 1) // stride + 1, (w - 1) // stride + 1
    x = randn(n * h * w, c, dtype=dtype, seed=38)
    col = torch.empty(n * ho * wo, 9 * c, dtype=dtype, device=DEV)
    hiplib.patch3x3(x, col, n, h, w, c, stride=stride)
    xn = x.float().cpu().view(n, h, w, c).permute(0, 3, 1, 2)
    ref = F.unfold(xn, 3, padding=1, stride=stride)                         # [n, c*9, ho*wo], (c, tap) order
    assert ref.shape[2] == ho * wo
    ref = ref.view(n, c, 9, ho * wo).permute(0, 3, 2, 1).reshape(n * ho * wo, 9 * c)
    assert torch.equal(col.float().cpu(), ref)
    # conv3x3 == patches @ W^T with W in [out, tap, in] order
    wt = randn(8, c, 3, 3, seed=39).cpu()
    conv = F.conv2d(xn, wt, padding=1, stride=stride).permute(0, 2, 3, 1).reshape(n * ho * wo, 8)
    assert rel_err(col.float().cpu() @ wt.permute(0, 2, 3, 1).reshape(8, 9 * c).t(), conv) < 1e-5
    # adjoint: <patch(x), d> == <x, adjoint(d)>
    d = randn(n * ho * wo, 9 * c, dtype=dtype, seed=40)
    back = torch.full_like(x, 7.0)      # every input pixel is written, also those no patch reads
    hiplib.patch3x3(d, back, n, h, w, c, adjoint=True, stride=stride)
    dn = d.float().cpu().view(n, ho * wo, 9, c).permute(0, 3, 2, 1).reshape(n, c * 9, ho * wo)
    fold = F.fold(dn, (h, w), 3, padding=1, stride=stride).permute(0, 2, 3, 1).reshape(n * h * w, c)
    assert rel_err(back, fold) < (1e-6 if dtype == torch.float32 else 1e-2)
    with pytest.raises(hiplib.HipKernelError):
        hiplib.patch3x3(x, col[:-1], n, h, w, c, stride=stride)


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("dtype", DTYPES)
def test_subsample_and_adjoint(hiplib, dtype, stride):
    """Rows a strided 1x1 convolution reads (bit-exact against slicing), and the adjoint added in place."""
    n, h, w, c = 2, 7, 6, 24
    ho, wo = (h - 1) // stride + 1, (w - 1) // stride + 1
    x = randn(n * h * w, c, dtype=dtype, seed=41)
    xs = torch.empty(n * ho * wo, c, dtype=dtype, device=DEV)
    hiplib.subsample(x, xs, n, h, w, c, stride)
    ref = x.view(n, h, w, c)[:, ::stride, ::stride].reshape(n * ho * wo, c)
    assert torch.equal(xs, ref)
    base = randn(n * h * w, c, dtype=dtype, seed=42)
    d = randn(n * ho * wo, c, dtype=dtype, seed=43)
    got = base.clone()
    hiplib.subsample(d, got, n, h, w, c, stride, adjoint=True)
    want = base.float().view(n, h, w, c).clone()
    want[:, ::stride, ::stride] += d.float().view(n, ho, wo, c)
    assert torch.equal(got, want.to(dtype).view(n * h * w, c))
    with pytest.raises(hiplib.HipKernelError):
        hiplib.subsample(x, xs[:-1], n, h, w, c, stride)


CONV_SHAPES = [(4, 5, 7, 64, 64),        # 140 pixels: one ragged row tile, one k-tile per tap
               (4, 6, 6, 64, 128),        # 144 pixels, as many output as a dgrad column tile
               (3, 9, 8, 128, 192),       # cin != cout, two k-tiles per tap forward and three backward
               (32, 14, 14, 256, 256),    # a ResNet-152 conv4_x block at micro-batch 32 (6272 pixels)
               (2, 1, 70, 64, 128), (2, 70, 1, 128, 128)]   # degenerate images: whole rows / columns of taps fall outside


@pytest.mark.parametrize("n,h,w,cin,cout", CONV_SHAPES)
def test_conv3x3_implicit_gemm(hiplib, n, h, w, cin, cout):
    """nn.Conv2d(cin, cout, 3, padding=1, bias=False) (reference resnet.py:58) and its input gradient as implicit
    GEMMs, against torch's conv2d and its autograd in fp64 on the same bf16 values; the forward is also
    bit-equal to the patch matrix followed by the GEMM kernel of the same tile shape, which multiplies the
    same numbers in the same order."""
    dt = torch.bfloat16
    rows = n * h * w
    assert hiplib.conv3x3_supported(dt, hiplib.CONV_FWD, n, h, w, cin, cout)
    assert hiplib.conv3x3_supported(dt, hiplib.CONV_DGRAD, n, h, w, cin, cout)
    x = randn(rows, cin, dtype=dt, seed=60)
    wt = randn(cout, 3, 3, cin, dtype=dt, seed=61, scale=math.sqrt(2.0 / (9 * cin)))   # [out, tap, in]
    dy = randn(rows, cout, dtype=dt, seed=62)
    y = torch.full((rows, cout), float("nan"), dtype=dt, device=DEV)
    dx = torch.full((rows, cin), float("nan"), dtype=dt, device=DEV)
    hiplib.conv3x3(hiplib.CONV_FWD, x, wt, y, n, h, w, cin, cout)
    hiplib.conv3x3(hiplib.CONV_DGRAD, dy, wt, dx, n, h, w, cin, cout)
    xr = x.double().cpu().view(n, h, w, cin).permute(0, 3, 1, 2).requires_grad_(True)
    wr = wt.double().cpu().permute(0, 3, 1, 2)                                            # the reference's [O, I, kh, kw]
    yr = torch.nn.functional.conv2d(xr, wr, padding=1)
    yr.backward(dy.double().cpu().view(n, h, w, cout).permute(0, 3, 1, 2))
    assert rel_err(y, yr.detach().permute(0, 2, 3, 1).reshape(rows, cout)) < tol(dt)
    assert rel_err(dx, xr.grad.permute(0, 2, 3, 1).reshape(rows, cin)) < tol(dt)
    # deterministic
    y2, dx2 = torch.empty_like(y), torch.empty_like(dx)
    hiplib.conv3x3(hiplib.CONV_FWD, x, wt, y2, n, h, w, cin, cout)
    hiplib.conv3x3(hiplib.CONV_DGRAD, dy, wt, dx2, n, h, w, cin, cout)
    assert torch.equal(y, y2) and torch.equal(dx, dx2)
    # the explicit route: patch matrix, then the GEMM
    col = torch.empty(rows, 9 * cin, dtype=dt, device=DEV)
    hiplib.patch3x3(x, col, n, h, w, cin)
    y3 = torch.empty_like(y)
    hiplib.gemm(hiplib.NT, col, wt.view(cout, 9 * cin), y3)
    if hiplib.gemm_variant(hiplib.gemm_desc(hiplib.NT, col, wt.view(cout, 9 * cin), y3)).endswith("dma128x64k64s3"):
        assert torch.equal(y, y3)
    else:
        assert rel_err(y, y3.double()) < 1e-2


@pytest.mark.parametrize("n,h,w,c,cout", [(4, 6, 6, 128, 128),      # 144 pixels... rounded to 128 below; 32-pixel k-tiles cross image borders
                                          (8, 4, 9, 128, 256),      # 288 pixels, images of 36 pixels: a k-tile nearly spans one
                                          (32, 14, 14, 256, 256)])  # the ResNet-152 conv4_x block (6272 pixels)
def test_conv3x3_weight_gradient_implicit_gemm(hiplib, n, h, w, c, cout):
    """dW[o, tap, i] += sum_p dy[p, o] * x[p + shift(tap), i] with the patch matrix gathered inside the GEMM
    (``conv=``): bit-equal to the same GEMM over the explicit patch matrix (same tiles, same order), alone,
    in a group, and cut along the pixels; and equal to torch's conv2d weight gradient."""
    dt = torch.bfloat16
    rows = n * h * w // 32 * 32                                      # K must be a multiple of 32: drop the tail pixels
    x_full = randn(n * h * w, c, dtype=dt, seed=70)
    dy_full = randn(n * h * w, cout, dtype=dt, seed=71)
    if rows != n * h * w:
        dy_full[rows:] = 0                                           # ... by giving them no gradient
    x, dy = x_full, dy_full[:rows]
    col = torch.empty(n * h * w, 9 * c, dtype=dt, device=DEV)
    hiplib.patch3x3(x_full, col, n, h, w, c)
    base = randn(cout, 9 * c, seed=72)
    want, got = base.clone(), base.clone()
    hiplib.gemm_grouped([hiplib.gemm_desc(hiplib.TN, dy, col[:rows], want, accumulate=True)])
    hiplib.gemm(hiplib.TN, dy, x[:rows], got, accumulate=True, conv=(h, w))
    assert torch.equal(got, want)
    xr = x_full.double().cpu().view(n, h, w, c).permute(0, 3, 1, 2)
    wr = torch.zeros(cout, c, 3, 3, dtype=torch.float64, requires_grad=True)
    torch.nn.functional.conv2d(xr, wr, padding=1).backward(dy_full.double().cpu().view(n, h, w, cout).permute(0, 3, 1, 2))
    ref = wr.grad.permute(0, 2, 3, 1).reshape(cout, 9 * c)
    assert rel_err(got.double().cpu() - base.double().cpu(), ref) < tol(dt)
    # in a group with an ordinary problem, whole and cut along the contraction
    a2, w2 = randn(rows, 256, dtype=dt, seed=73), randn(256, 128, seed=74)
    for splitk in (False, True):
        outs = []
        for implicit in (False, True):
            g1, g2 = base.clone(), w2.clone()
            descs = [hiplib.gemm_desc(hiplib.TN, a2, dy[:, :128].contiguous(), g2, accumulate=True),
                     hiplib.gemm_desc(hiplib.TN, dy, x[:rows], g1, accumulate=True, conv=(h, w)) if implicit
                     else hiplib.gemm_desc(hiplib.TN, dy, col[:rows], g1, accumulate=True)]
            ws = torch.empty(hiplib.gemm_splitk_workspace(descs) // 4, dtype=torch.float32, device=DEV) if splitk else None
            hiplib.gemm_grouped(descs, splitk_ws=ws)
            outs.append((g1, g2))
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
        assert rel_err(outs[1][0].double().cpu() - base.double().cpu(), ref) < tol(dt)


def _strip_reference(y, rows, cols):
    """(pivot, sum (y - pivot), sum (y - pivot)^2) per 32-row strip and column, in fp64, from the stored tensor."""
    return ol.strip_triples(y.double().cpu())                           # [strips, 3, cols]


@pytest.mark.parametrize("M,N,K", [(6272, 256, 1024),     # conv1 of the ResNet block: 128x64 tiles
                                   (6272, 1024, 256),     # conv3: short contraction, 128x64 tiles
                                   (6272, 1024, 1024),    # the 256x128 tile (two strips per wave)
                                   (300, 72, 128)])       # ragged: 12 rows in the last strip, 8 columns in the last group
def test_gemm_strip_statistics_feed_batchnorm(hiplib, M, N, K):
    """The GEMM epilogue's per-strip column statistics: the product is bit-equal to the plain call, the triples
    equal an fp64 restatement on the stored values, and BatchNorm fed from them equals BatchNorm reading the tensor."""
    dt = torch.bfloat16
    A, B = randn(M, K, dtype=dt, seed=80), randn(N, K, dtype=dt, seed=81, scale=0.05)
    A += 3.0                                                              # a mean far from zero: what the pivot is for
    y0 = torch.empty(M, N, dtype=dt, device=DEV)
    y1 = torch.empty_like(y0)
    assert hiplib.gemm_strip_stats_supported(hiplib.NT, A, B, y0)
    strips = torch.full((hiplib.strip_stats_workspace(M, N),), float("nan"), device=DEV)
    hiplib.gemm(hiplib.NT, A, B, y1, strip_stats=strips)
    if (M, N, K) == (6272, 1024, 1024):
        assert hiplib.gemm_variant(hiplib.gemm_desc(hiplib.NT, A, B, y1)).endswith("dma256x128k64s3")
    ref_prod = A.double().cpu() @ B.double().cpu().t()
    assert rel_err(y1, ref_prod) < tol(dt)
    ns = (M + 31) // 32
    got = strips[: ns * 3 * N].view(ns, 3, N).double().cpu()
    want = _strip_reference(y1, M, N)
    assert torch.equal(got[:, 0], want[:, 0])
    assert rel_err(got[:, 1], want[:, 1]) < 1e-5 and rel_err(got[:, 2], want[:, 2]) < 1e-5
    _check_batchnorm_from_strips(hiplib, y1, strips, M, N)


def _check_batchnorm_from_strips(hiplib, y, strips, M, N):
    dt = torch.bfloat16
    gamma, beta = randn(N, dtype=dt, seed=82) * 0.1 + 1.0, randn(N, dtype=dt, seed=83) * 0.1
    ws = torch.empty(hiplib.bn_workspace(N), device=DEV)
    outs = []
    for st in (None, strips):
        o = torch.empty_like(y)
        mean, rstd = torch.empty(N, device=DEV), torch.empty(N, device=DEV)
        rm, rv = torch.zeros(N, device=DEV), torch.ones(N, device=DEV)
        hiplib.batchnorm_fwd(y, gamma, beta, None, o, mean, rstd, rm, rv, ws, 1e-5, 0.1, True, strip_stats=st)
        outs.append((o, mean, rstd, rm, rv))
    yd = y.double().cpu()
    mu, var = yd.mean(0), yd.var(0, unbiased=False)
    mu_s, var_s = ol.batch_stats_from_strips(strips[: ((M + 31) // 32) * 3 * N].view(-1, 3, N).double().cpu(), M)
    assert rel_err(mu_s, mu) < 1e-6 and rel_err(var_s, var) < 1e-5     # the GPU's triples through the oracle's finish
    for o, mean, rstd, rm, rv in outs:
        assert rel_err(mean, mu) < 1e-5
        assert float(((rstd.double().cpu() - 1 / torch.sqrt(var + 1e-5)).abs() * torch.sqrt(var + 1e-5)).max()) < 1e-5
        assert rel_err(rv, 0.9 + 0.1 * yd.var(0, unbiased=True)) < 1e-5
    assert rel_err(outs[1][0], outs[0][0].double()) < 1e-2               # bf16 outputs: a rounding step apart at most


def test_conv3x3_strip_statistics(hiplib):
    n, h, w, cin, cout = 8, 6, 6, 128, 192
    dt = torch.bfloat16
    rows = n * h * w
    x = randn(rows, cin, dtype=dt, seed=84)
    wt = randn(cout, 3, 3, cin, dtype=dt, seed=85, scale=0.03)
    y0, y1 = torch.empty(rows, cout, dtype=dt, device=DEV), torch.empty(rows, cout, dtype=dt, device=DEV)
    strips = torch.full((hiplib.strip_stats_workspace(rows, cout),), float("nan"), device=DEV)
    hiplib.conv3x3(hiplib.CONV_FWD, x, wt, y0, n, h, w, cin, cout)
    hiplib.conv3x3(hiplib.CONV_FWD, x, wt, y1, n, h, w, cin, cout, strip_stats=strips)
    assert torch.equal(y0, y1)
    got = strips.view(rows // 32, 3, cout).double().cpu()
    want = _strip_reference(y1, rows, cout)
    assert torch.equal(got[:, 0], want[:, 0])
    assert rel_err(got[:, 1], want[:, 1]) < 1e-5 and rel_err(got[:, 2], want[:, 2]) < 1e-5
    _check_batchnorm_from_strips(hiplib, y1, strips, rows, cout)


def test_conv3x3_refuses_what_it_does_not_take(hiplib):
    dt = torch.bfloat16
    assert not hiplib.conv3x3_supported(dt, hiplib.CONV_FWD, 4, 6, 6, 16, 64)            # 16 gathered channels
    assert not hiplib.conv3x3_supported(torch.float32, hiplib.CONV_FWD, 4, 6, 6, 64, 64)
    assert not hiplib.conv3x3_supported(dt, hiplib.CONV_FWD, 1, 6, 6, 64, 64)            # 36 pixels
    x, wt, y = randn(144, 16, dtype=dt), randn(64, 3, 3, 16, dtype=dt), torch.empty(144, 64, dtype=dt, device=DEV)
    with pytest.raises(hiplib.HipKernelError):
        hiplib.conv3x3(hiplib.CONV_FWD, x, wt, y, 4, 6, 6, 16, 64)


@pytest.mark.parametrize("dtype", DTYPES)
def test_mse(hiplib, dtype):
    n = 4 * 128 * 768
    y, t = randn(n, dtype=dtype, seed=24), randn(n, dtype=dtype, seed=25)
    dy = torch.empty_like(y)
    loss = torch.full((1,), 5.0, device=DEV)
    ws = torch.empty(hiplib.mse_workspace(), device=DEV)
    hiplib.mse_fwd_bwd(y, t, dy, 0.125, loss, True, ws)
    yr = y.double().cpu().requires_grad_(True)
    lr = torch.nn.functional.mse_loss(yr, t.double().cpu())
    (lr * 0.125).backward()
    assert abs(float(loss) - 5.0 - float(lr)) < 1e-5 * float(lr)
    assert rel_err(dy, yr.grad) < tol(dtype)
    hiplib.mse_fwd_bwd(y, t, dy, 0.125, loss, False, ws)
    assert abs(float(loss) - float(lr)) < 1e-5 * float(lr)


@pytest.mark.parametrize("adam_w,wd", [(True, 0.0), (True, 0.01), (False, 0.01)])
def test_adam_bit_exact_with_oracle(hiplib, adam_w, wd):
    """Sizes of the reference's own Adam test (tests/unit/test_cpu_adam.py:25-27) plus ragged
    ones; 10 steps; fp32 state compared bit for bit with the oracle formula, bf16 copy with
    the rounded parameter."""
    sizes = [22, 55, 64, 127, 1024, 1048576, 4097, 8192 + 3]
    sizes = [(n + 3) // 4 * 4 for n in sizes]          # 16-byte aligned tensor starts
    total = sum(sizes)
    flat = lambda seed: randn(total, seed=seed)
    P, M_, V = flat(30), torch.zeros(total, device=DEV), torch.zeros(total, device=DEV)
    LP = torch.zeros(total, dtype=torch.bfloat16, device=DEV)
    offs = np.cumsum([0] + sizes)
    split = lambda t: [t[offs[i]: offs[i + 1]] for i in range(len(sizes))]
    p_ref = P.cpu().numpy().copy()
    m_ref, v_ref = np.zeros(total, np.float32), np.zeros(total, np.float32)
    for step in range(1, 11):
        G = flat(100 + step)
        g_ref = G.cpu().numpy().copy()
        hiplib.adam_multi(split(G), split(P), split(M_), split(V), split(LP), lr=1e-3, beta1=0.9, beta2=0.999,
                          eps=1e-8, step=step, adam_w_mode=adam_w, weight_decay=wd, zero_grad=(step % 2 == 0))
        oadam.adam_step(p_ref, g_ref, m_ref, v_ref, step, weight_decay=wd, adam_w_mode=adam_w)
        assert np.array_equal(P.cpu().numpy(), p_ref), f"step {step}: parameters differ"
        assert np.array_equal(M_.cpu().numpy(), m_ref) and np.array_equal(V.cpu().numpy(), v_ref)
        assert torch.equal(LP, P.to(torch.bfloat16))
        assert (float(G.abs().max()) == 0.0) == (step % 2 == 0)
    # agreement with torch.optim (the reference's own check, atol 1e-2) follows from the oracle test


@pytest.mark.parametrize("max_norm", [1.0, 1e9])
def test_gradient_clipping_coefficient_and_scaled_adam(hiplib, max_norm):
    """Global gradient norm over several tensors (ragged sizes, more tensors than one launch's table holds) and the
    clipping coefficient against the oracle's restatement of clip_grad_norm_; the Adam step that reads the
    coefficient from device memory equals, bit for bit, the oracle's Adam step on gradients multiplied by that
    coefficient in fp32; a bound above the norm changes nothing."""
    sizes = [(n + 3) // 4 * 4 for n in [22, 4097, 1048576, 8192 + 3, 64] + [128] * 24]
    total = sum(sizes)
    offs = np.cumsum([0] + sizes)
    split = lambda t: [t[offs[i]: offs[i + 1]] for i in range(len(sizes))]
    G, P = randn(total, seed=61), randn(total, seed=62)
    M_, V = torch.zeros(total, device=DEV), torch.zeros(total, device=DEV)
    out = torch.full((2,), -1.0, device=DEV)
    ws = torch.full((hiplib.grad_clip_workspace(split(G)),), float("nan"), device=DEV)
    hiplib.grad_clip_coef(split(G), max_norm, out, ws)
    hiplib.grad_clip_coef(split(G), max_norm, out, ws)       # the carried sum starts over with every call
    g_ref = [g.cpu().numpy().copy() for g in split(G)]
    norm, coef = oadam.clip_grad_norm(g_ref, max_norm)
    assert abs(float(out[0]) - norm) < 2e-6 * norm
    assert abs(float(out[1]) - min(coef, 1.0)) < 2e-6 * min(coef, 1.0)
    assert (float(out[1]) == 1.0) == (max_norm > 1e6)
    # the reference multiplies by the coefficient in fp32 (p.grad.data.mul_), then steps
    c = np.float32(float(out[1]))
    g_clipped = np.concatenate([g.cpu().numpy() for g in split(G)])
    if c < 1:
        g_clipped = g_clipped * c
    p_ref, m_ref, v_ref = P.cpu().numpy().copy(), np.zeros(total, np.float32), np.zeros(total, np.float32)
    oadam.adam_step(p_ref, g_clipped, m_ref, v_ref, 1)
    hiplib.adam_multi(split(G), split(P), split(M_), split(V), None, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=1,
                      grad_scale=out[1:])
    assert np.array_equal(P.cpu().numpy(), p_ref) and np.array_equal(M_.cpu().numpy(), m_ref) and np.array_equal(V.cpu().numpy(), v_ref)
    # no tensors at all: norm 0, coefficient 1
    hiplib.grad_clip_coef([], 1.0, out, ws)
    assert out.tolist() == [0.0, 1.0]


def test_adam_rejects_bad_arguments(hiplib):
    t = torch.zeros(16, device=DEV)
    with pytest.raises(hiplib.HipKernelError):
        hiplib.adam_multi([t], [t], [t], [t], None, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=0)
    hiplib.adam_multi([], [], [], [], None, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=1)  # empty list is fine

def test_same_type_copy(hiplib):
    """cast with equal types is a copy: 16 bytes per lane when both pointers allow it, with a scalar tail,
    element by element otherwise; the bytes beyond the range stay untouched."""
    for n, off in ((8 * 1000 + 3, 0), (8 * 1000 + 3, 1), (5, 0), (1 << 20, 0)):
        src = randn(n + 16, dtype=torch.bfloat16, seed=91)
        dst = torch.full((n + 16,), 7.0, dtype=torch.bfloat16, device=DEV)
        hiplib.cast(src[off:off + n], dst[off:off + n])
        assert torch.equal(dst[off:off + n], src[off:off + n])
        assert torch.all(dst[off + n:] == 7.0) and torch.all(dst[:off] == 7.0)
