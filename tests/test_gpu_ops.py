"""GPU parity of the three stand-alone products ns_line_1 / ns_line_2 / ns_line_3 (reference
muon.py:420-457, 547-588, 705-745) against their CPU restatements in the oracle and against the
exact (float64) value of each expression.

Bound against the exact value E of an element: one bf16 rounding, |E| * 2^-8, plus what fp32
accumulation in another order and the 16-bit intermediate of the fused epilogue may add, 2^-13 of the
sum of the absolute values of the terms.  Against the oracle's bf16 result (fp32 sums in another
order, then the same single rounding): no element more than one bf16 step away, few differing at all.
"""
import pytest
import torch

from oracle import muon_oracle as O

pytestmark = pytest.mark.gpu

A_, B_, C_ = O.NS_COEFFS


@pytest.fixture(scope="module")
def M():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need an MI355X; torch.cuda.is_available() is False")
    import muon_amd
    from muon_amd import _lib
    _lib.load()
    return muon_amd


def _check(got, exact, terms, oracle, what):
    assert got.dtype == torch.bfloat16 and got.shape == oracle.shape, what
    g = got.double().cpu()
    err = (g - exact).abs()
    bound = 2.0 ** -8 * 1.001 * exact.abs() + 2.0 ** -13 * terms
    assert (err <= bound).all(), (what, float((err - bound).max()))
    o = oracle.double()
    step = 2.0 ** -7 * o.abs() + 2.0 ** -13 * terms          # one bf16 step at the value, plus the slack above
    assert ((g - o).abs() <= step).all(), (what, float(((g - o).abs() - step).max()))
    assert (g != o).double().mean() < 0.03, (what, float((g != o).double().mean()))


def _rand(shape, scale, seed):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale).bfloat16()


def _sym(shape, seed):
    """A symmetric bf16 matrix (batch) with entries of the size a Gram matrix of a normalised iterate has."""
    R = torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) / shape[-1] ** 0.5
    return ((R + R.mT) / 2).bfloat16()


LINE1_SHAPES = [(128, 64), (100, 200), (5, 3), (768, 3072), (1024, 4096), (1300, 520), (3, 200, 136), (2, 1024, 1024),
                (128, 16384), (3, 200, 8200), (512, 4608)]      # short and very wide: split reductions


@pytest.mark.parametrize("shape", LINE1_SHAPES)
def test_ns_line_1_matches_the_oracle(M, shape):
    A = _rand(shape, 0.05, 31)
    got = M.ns_line_1(A.cuda())
    Ad = A.double()
    _check(got, Ad @ Ad.mT, Ad.abs() @ Ad.abs().mT, O.ns_line_1(A), f"ns_line_1 {shape}")
    assert torch.equal(got, got.mT)                        # the mirrored store


@pytest.mark.parametrize("shape", [(256, 256), (300, 300), (40, 40), (1024, 1024), (1100, 1100), (3, 200, 200)])
def test_ns_line_2_matches_the_oracle(M, shape):
    A = _sym(shape, 32)
    for alpha, beta in ((C_, B_), (1.0, 0.0), (0.0, 1.5)):
        got = M.ns_line_2(A.cuda(), alpha, beta)
        Ad = A.double()
        exact = alpha * (Ad @ Ad.mT) + beta * Ad
        terms = abs(alpha) * (Ad.abs() @ Ad.abs().mT) + abs(beta) * Ad.abs()
        _check(got, exact, terms, O.ns_line_2(A, alpha, beta), f"ns_line_2 {shape} {alpha} {beta}")
        assert torch.equal(got, got.mT)


@pytest.mark.parametrize("shape", [(128, 256), (100, 300), (40, 8), (768, 2304), (1024, 4096), (1100, 1500),
                                   (3, 200, 136), (2, 1024, 1280),
                                   (22, 768, 1024)])       # short matrices, enough of them for 256 x 256 tiles
def test_ns_line_3_matches_the_oracle(M, shape):
    X = _rand(shape, 0.05, 33)
    m = shape[-2]
    B = _sym((*shape[:-2], m, m), 34)
    for a in (A_, 0.0):
        got = M.ns_line_3(B.cuda(), X.cuda(), a)
        Bd, Xd = B.double(), X.double()
        _check(got, a * Xd + Bd @ Xd, abs(a) * Xd.abs() + Bd.abs() @ Xd.abs(), O.ns_line_3(B, X, a),
               f"ns_line_3 {shape} {a}")
    # B need not be symmetric: the product is B X, not B^T X
    R = _rand((m, m), 0.05, 35)
    X2 = X[0] if X.ndim == 3 else X
    got = M.ns_line_3(R.cuda(), X2.cuda(), 0.0)
    _check(got, R.double() @ X2.double(), R.double().abs() @ X2.double().abs(), O.ns_line_3(R, X2, 0.0),
           f"ns_line_3 {shape} non-symmetric B")


def test_out_arguments_strides_and_broadcast(M):
    A = _rand((200, 136), 0.05, 36)
    want = O.ns_line_1(A)
    Ag = A.cuda()
    # an `out` that the kernel can write in place (tile-sized, contiguous), one it cannot, and a view
    for rows in (200, 256):
        Ap = _rand((rows, 128), 0.05, 37)
        out = torch.full((rows, rows), 7.0, dtype=torch.bfloat16, device="cuda")
        res = M.ns_line_1(Ap.cuda(), out=out)
        assert res is out
        _check(out, Ap.double() @ Ap.double().mT, Ap.double().abs() @ Ap.double().abs().mT, O.ns_line_1(Ap), f"out {rows}")
    big = torch.zeros(300, 400, dtype=torch.bfloat16, device="cuda")
    view = big[50:250, 100:300]
    M.ns_line_1(Ag, out=view)
    assert torch.equal(view.cpu(), M.ns_line_1(Ag).cpu())
    assert float(big[:50].abs().sum()) == 0 and float(big[:, 300:].abs().sum()) == 0
    # a transposed view as input
    At = Ag.mT.contiguous().mT
    assert not At.is_contiguous()
    assert torch.equal(M.ns_line_1(At).cpu(), M.ns_line_1(Ag).cpu())
    assert (M.ns_line_1(Ag).cpu().double() - want.double()).abs().max() <= 2.0 ** -7 * want.double().abs().max()
    # ns_line_3: a 2-D B with a batch of X (muon.py:727: b_stride_b = 0), and the result written over X
    X = _rand((3, 256, 384), 0.05, 38)
    B = _sym((256, 256), 39)
    got = M.ns_line_3(B.cuda(), X.cuda(), A_)
    for k in range(3):
        assert torch.equal(got[k].cpu(), M.ns_line_3(B.cuda(), X[k].cuda(), A_).cpu())
    Xg = X.cuda()
    res = M.ns_line_3(B.cuda(), Xg, A_, out=Xg)
    assert res is Xg and torch.equal(Xg.cpu(), got.cpu())
    # ns_line_2 over its own input
    S = _sym((256, 256), 40).cuda()
    want2 = M.ns_line_2(S, C_, B_).cpu()
    M.ns_line_2(S, C_, B_, out=S)
    assert torch.equal(S.cpu(), want2)


def test_shape_errors_are_the_reference_s(M):
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError, match="must be 2D or 3D"):          # muon.py:424-425
        M.ns_line_1(z(2, 2, 4, 4))
    with pytest.raises(ValueError, match="must be 2D or 3D"):          # muon.py:551-552
        M.ns_line_2(z(8), 1.0, 1.0)
    with pytest.raises(ValueError, match="symmetric square matrix"):   # muon.py:555-558
        M.ns_line_2(z(4, 6), 1.0, 1.0)
    with pytest.raises(ValueError, match="B must be square"):          # muon.py:710-711
        M.ns_line_3(z(4, 6), z(4, 6), 1.0)
    with pytest.raises(ValueError, match="same number of rows"):       # muon.py:713-714
        M.ns_line_3(z(4, 4), z(6, 6), 1.0)
    with pytest.raises(AssertionError, match="incorrect shape"):       # muon.py:431-432
        M.ns_line_1(z(4, 6), out=z(6, 6))
    with pytest.raises(TypeError):
        M.ns_line_1(torch.zeros(4, 4, device="cuda"))
    with pytest.raises(M.MuonAmdError):
        M.ns_line_1(torch.zeros(4, 4, dtype=torch.bfloat16))
    assert M.ns_line_1(z(0, 5)).shape == (0, 0)
    assert float(M.ns_line_1(z(5, 0)).abs().sum()) == 0 and M.ns_line_1(z(5, 0)).shape == (5, 5)
    assert M.ns_line_3(z(4, 4), z(4, 0), 1.0).shape == (4, 0)


def test_newton_schulz_built_from_the_operators(M):
    """The iteration muon.py:285-287 written with the three operators, as the reference's live loop
    does (muon.py:789-794), orthogonalises like the specification: within the bf16 bound of the
    float64 closed form, for a small, a GPT-2-sized and a batched input."""
    for shape, seed in (((256, 512), 41), ((768, 3072), 42), ((2, 384, 640), 43)):
        G = torch.randn(*shape, generator=torch.Generator().manual_seed(seed))
        X = (G / (G.norm(dim=(-2, -1), keepdim=True) + 1e-7)).bfloat16().cuda()
        for _ in range(5):
            A = M.ns_line_1(X)
            B = M.ns_line_2(A, alpha=C_, beta=B_)
            X = M.ns_line_3(B, X, A_)
        if G.ndim == 2:
            assert O.rel_fro(X.float().cpu(), O.ns5_fp64_closed_form(G.double().numpy())) < 2e-2, shape
        else:
            for k in range(shape[0]):
                assert O.rel_fro(X[k].float().cpu(), O.ns5_fp64_closed_form(G[k].double().numpy())) < 2e-2, (shape, k)


def test_operators_against_the_golden_fixture(M, golden_dir):
    """The committed vectors (tests/golden/ops_golden.npz, written by tests/golden/make_golden.py from
    the oracle): each operator on the fixture's own bf16 inputs, within one bf16 step of the stored
    result and within one rounding of the stored exact value."""
    import os
    import numpy as np
    z = np.load(os.path.join(golden_dir, "ops_golden.npz"))
    bf = lambda a: torch.from_numpy(a.astype(np.int16)).view(torch.bfloat16)
    for name in sorted({k.split("/")[0] for k in z.files}):
        X, A, B = bf(z[name + "/X"]), bf(z[name + "/line1"]), bf(z[name + "/line2"])
        Xd, Ad, Bd = X.double().abs(), A.double().abs(), B.double().abs()
        cases = (("line1", M.ns_line_1(X.cuda()), Xd @ Xd.mT),
                 ("line2", M.ns_line_2(A.cuda(), 2.0315, -4.7750), 2.0315 * (Ad @ Ad.mT) + 4.7750 * Ad),
                 ("line3", M.ns_line_3(B.cuda(), X.cuda(), 3.4445), 3.4445 * Xd + Bd @ Xd))
        for key, got, terms in cases:
            _check(got, torch.from_numpy(z[f"{name}/{key}_exact"]).double(), terms, bf(z[f"{name}/{key}"]), f"{name} {key}")
