"""Pins the CPU oracle (oracle/muon_oracle.py) without the reference being importable: closed
forms, brute force, invariants and library special cases chosen so that a dropped term, a wrong
sign/index or a transposed operand fails at least one of them."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import muon_oracle as O

A_, B_, C_ = O.NS_COEFFS


# ------------------------------------------------------------------------------------------
# scalar map
# ------------------------------------------------------------------------------------------
def test_coefficients_and_scalar_map_facts():
    assert O.NS_COEFFS == (3.4445, -4.7750, 2.0315)          # muon.py:276
    p1 = A_ + B_ + C_
    assert abs(p1 - 0.7010) < 1e-12
    assert abs(O.ns_poly(1.0, 1) - p1) < 1e-12
    assert abs(O.ns_poly(1.0, 5) - 0.69644) < 1e-4
    x = np.linspace(0.005, 1.0, 20001)
    y = O.ns_poly(x, 5)
    assert 0.68 < y.min() < 0.69 and 1.15 < y.max() < 1.16
    # slope at zero after five steps is a^5
    assert abs(O.ns_poly(1e-9, 5) / 1e-9 - A_ ** 5) < 1e-3
    assert abs(A_ ** 5 - 484.876) < 1e-2


# ------------------------------------------------------------------------------------------
# Newton-Schulz: closed form, brute force, invariants
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(8, 8), (6, 17), (17, 6), (32, 96), (96, 32), (3, 4)])
def test_ns_fp32_matches_fp64_svd_closed_form(shape):
    torch.manual_seed(hash(shape) % 1000)
    G = torch.randn(*shape, dtype=torch.float64)
    got = O._ns5(G, 5, 1e-7, torch.float64).numpy()
    want = O.ns5_fp64_closed_form(G)
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-9)
    assert O.rel_fro(O.ns5_fp32(G.float()), want) < 2e-4


@pytest.mark.parametrize("shape", [(3, 5), (5, 3), (4, 4), (2, 7)])
def test_ns_matches_triple_loop_brute_force(shape):
    torch.manual_seed(7)
    G = torch.randn(*shape, dtype=torch.float64)
    brute = np.array(O.ns5_brute_force(G.tolist()))
    np.testing.assert_allclose(O._ns5(G, 5, 1e-7, torch.float64).numpy(), brute, atol=1e-10)
    np.testing.assert_allclose(O.ns5_fp64_closed_form(G), brute, atol=1e-9)


@pytest.mark.parametrize("steps", [0, 1, 2, 5])
def test_ns_step_count(steps):
    torch.manual_seed(3)
    G = torch.randn(5, 9, dtype=torch.float64)
    np.testing.assert_allclose(O._ns5(G, steps, 1e-7, torch.float64).numpy(),
                               O.ns5_fp64_closed_form(G, steps), atol=1e-10)
    if steps == 0:   # just the Frobenius normalisation
        np.testing.assert_allclose(O._ns5(G, 0, 1e-7, torch.float64).numpy(),
                                   (G / (G.norm() + 1e-7)).numpy(), atol=1e-15)


def test_ns_transpose_rule():
    # muon.py:278-279, 289-290: a tall input is iterated as its transpose, so NS(G^T) == NS(G)^T
    # up to the summation order of the matrix products (strided vs contiguous operands).
    torch.manual_seed(11)
    G = torch.randn(40, 24, dtype=torch.float64)
    a, b = O._ns5(G.mT.contiguous(), 5, 1e-7, torch.float64), O._ns5(G, 5, 1e-7, torch.float64).mT
    assert O.rel_fro(a, b) < 1e-12
    assert O.rel_fro(O.ns5_fp32(G.float().mT.contiguous()), O.ns5_fp32(G.float()).mT) < 1e-4
    assert O.rel_fro(O.ns5_bf16(G.float().mT.contiguous()), O.ns5_bf16(G.float()).mT) < 2e-2
    sq = torch.randn(16, 16, dtype=torch.float64)   # square is not transposed (strict >) but the map commutes
    assert O.rel_fro(O._ns5(sq.mT.contiguous(), 5, 0.0, torch.float64), O._ns5(sq, 5, 0.0, torch.float64).mT) < 1e-10


def test_ns_scale_and_orthogonal_invariance():
    torch.manual_seed(5)
    G = torch.randn(12, 30, dtype=torch.float64)
    base = O._ns5(G, 5, 0.0, torch.float64)
    assert O.rel_fro(O._ns5(G * 37.5, 5, 0.0, torch.float64), base) < 1e-12
    Q1, _ = torch.linalg.qr(torch.randn(12, 12, dtype=torch.float64))
    Q2, _ = torch.linalg.qr(torch.randn(30, 30, dtype=torch.float64))
    assert O.rel_fro(O._ns5(Q1 @ G @ Q2, 5, 0.0, torch.float64), Q1 @ base @ Q2) < 1e-10


def test_ns_special_inputs():
    assert torch.equal(O.ns5_fp32(torch.zeros(4, 6)), torch.zeros(4, 6))        # eps keeps 0/0 finite
    assert torch.equal(O.ns5_bf16(torch.zeros(6, 4)).float(), torch.zeros(6, 4))
    d = torch.tensor([3.0, 1.0, 0.5, 0.25], dtype=torch.float64)
    got = O._ns5(torch.diag(d), 5, 0.0, torch.float64)
    np.testing.assert_allclose(got.numpy(), np.diag(O.ns_poly((d / d.norm()).numpy(), 5)), atol=1e-12)
    Q, _ = torch.linalg.qr(torch.randn(9, 9, dtype=torch.float64))
    np.testing.assert_allclose(O._ns5(Q, 5, 0.0, torch.float64).numpy(),
                               (O.ns_poly(1 / 3.0, 5) * Q).numpy(), atol=1e-10)


def test_ns_batched_equals_per_matrix():
    torch.manual_seed(2)
    G = torch.randn(3, 10, 14)
    out = O.ns5_bf16(G)
    for b in range(3):
        assert torch.equal(out[b], O.ns5_bf16(G[b]))
    assert out.dtype == torch.bfloat16 and out.shape == G.shape          # muon.py:277


def test_ns_bf16_tracks_fp32_and_singular_values_land_in_band():
    torch.manual_seed(9)
    G = torch.randn(128, 384) * 1e-3
    rb, rf = O.ns5_bf16(G).float(), O.ns5_fp32(G)
    assert O.rel_fro(rb, rf) < 4e-2
    s = torch.linalg.svdvals(rf.double())
    assert s.min() > 0.66 and s.max() < 1.17


# ------------------------------------------------------------------------------------------
# muon_update
# ------------------------------------------------------------------------------------------
def test_muon_update_first_step_closed_form():
    torch.manual_seed(4)
    g = torch.randn(20, 30) * 1e-3
    g0 = g.clone()
    mom = torch.zeros_like(g)
    upd = O.muon_update(g, mom, beta=0.95)
    # zero momentum: m = (1-b) g, blend = (1-b) g + b (1-b) g = (1-b^2) g; NS is scale invariant
    np.testing.assert_allclose(mom.numpy(), (0.05 * g0.double()).float().numpy(), rtol=1e-6)
    np.testing.assert_allclose(g.numpy(), ((1 - 0.95 ** 2) * g0.double()).float().numpy(), rtol=2e-6)
    assert upd.dtype == torch.bfloat16
    assert O.rel_fro(upd, O.ns5_fp64_closed_form(g0)) < 4e-2


def test_muon_update_fp64_recurrence_and_no_nesterov():
    torch.manual_seed(6)
    mom = torch.zeros(8, 12)
    m64 = np.zeros((8, 12))
    for _ in range(4):
        g = torch.randn(8, 12)
        g64 = g.double().numpy()
        m64 = m64 + 0.05 * (g64 - m64)
        u64 = 0.05 * g64 + 0.95 * m64
        upd = O.muon_update(g, mom, beta=0.95, nesterov=True)
        np.testing.assert_allclose(mom.numpy(), m64, rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(g.numpy(), u64, rtol=1e-5, atol=1e-7)
        assert O.rel_fro(upd, O.ns5_fp64_closed_form(u64)) < 8e-2   # bf16 noise on a tiny matrix
    g = torch.randn(8, 12)
    g_before = g.clone()
    upd = O.muon_update(g, mom, beta=0.9, nesterov=False)
    assert torch.equal(g, g_before)                       # only the nesterov branch writes grad
    assert O.rel_fro(upd, O.ns5_fp64_closed_form(mom)) < 8e-2


@pytest.mark.parametrize("shape,scale", [((30, 10), math.sqrt(3.0)), ((10, 30), 1.0),
                                          ((16, 4, 3, 3), 1.0), ((8, 2, 4, 2), math.sqrt(2.0))])
def test_muon_update_aspect_scale_uses_unflattened_sizes(shape, scale):
    torch.manual_seed(8)
    g = torch.randn(*shape)
    flat = g.reshape(shape[0], -1).clone()
    upd = O.muon_update(g, torch.zeros_like(g), beta=0.0, nesterov=False)   # beta=0: momentum == grad
    want = O.ns5_bf16(flat)
    want = (want.float() * scale).bfloat16() if scale != 1.0 else want
    assert upd.shape == flat.shape                       # conv filters come back 2-D (muon.py:11-12)
    assert torch.equal(upd, want)


# ------------------------------------------------------------------------------------------
# adam_update
# ------------------------------------------------------------------------------------------
def test_adam_update_first_step_closed_form():
    g = torch.tensor([1e-3, -2.0, 0.5, 0.0])
    m, v = torch.zeros(4), torch.zeros(4)
    upd = O.adam_update(g, m, v, 1, (0.9, 0.95), 1e-10)
    np.testing.assert_allclose(upd.numpy(), (g / (g.abs() + 1e-10)).numpy(), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(m.numpy(), 0.1 * g.numpy(), rtol=1e-6)
    np.testing.assert_allclose(v.numpy(), 0.05 * g.numpy() ** 2, rtol=1e-6)


def test_adam_branch_equals_torch_adamw():
    torch.manual_seed(10)
    p1 = torch.nn.Parameter(torch.randn(7, 5))
    p2 = torch.nn.Parameter(p1.detach().clone())
    o1 = O.OracleSingleDeviceMuonWithAuxAdam([dict(params=[p1], use_muon=False, lr=1e-2, betas=(0.9, 0.95),
                                                   eps=1e-10, weight_decay=0.1)])
    o2 = torch.optim.AdamW([p2], lr=1e-2, betas=(0.9, 0.95), eps=1e-10, weight_decay=0.1)
    for _ in range(10):
        g = torch.randn(7, 5)
        p1.grad, p2.grad = g.clone(), g.clone()
        o1.step()
        o2.step()
    np.testing.assert_allclose(p1.detach().numpy(), p2.detach().numpy(), rtol=1e-5, atol=1e-7)


# ------------------------------------------------------------------------------------------
# step classes
# ------------------------------------------------------------------------------------------
def test_single_device_muon_config1_shape_collapses_to_ns_of_grad():
    torch.manual_seed(1)
    p = torch.nn.Parameter(torch.randn(48, 192) * 0.02)
    p0 = p.detach().clone()
    g = torch.randn(48, 192) * 1e-3
    p.grad = g.clone()
    opt = O.OracleSingleDeviceMuon([p], lr=0.02, weight_decay=0.01, momentum=0.95)
    opt.step()
    want = p0.double() * (1 - 0.02 * 0.01) - 0.02 * torch.from_numpy(O.ns5_fp64_closed_form(g))
    assert O.rel_fro(p.detach(), want) < 5e-3    # bf16 NS noise (3e-2) on an update of ~7% of |p|
    assert set(opt.state[p].keys()) == {"momentum_buffer"}


def test_step_classes_behaviour():
    p = torch.nn.Parameter(torch.ones(4, 6))
    q = torch.nn.Parameter(torch.ones(5))
    opt = O.OracleSingleDeviceMuonWithAuxAdam([dict(params=[p], use_muon=True, weight_decay=0.5),
                                               dict(params=[q], use_muon=False, weight_decay=0.5)])
    assert opt.param_groups[0]["lr"] == 0.02 and opt.param_groups[0]["momentum"] == 0.95
    assert opt.param_groups[1]["lr"] == 3e-4 and opt.param_groups[1]["betas"] == (0.9, 0.95)
    assert opt.param_groups[1]["eps"] == 1e-10
    calls = []
    loss = opt.step(lambda: calls.append(1) or torch.tensor(3.0))
    assert loss.item() == 3.0 and calls == [1]
    # grad None -> zeros, parameter still decayed (muon.py:91-93, 98)
    assert p.grad is not None and torch.count_nonzero(p.grad) == 0
    np.testing.assert_allclose(p.detach().numpy(), np.full((4, 6), 1 - 0.02 * 0.5), rtol=1e-6)
    np.testing.assert_allclose(q.detach().numpy(), np.full(5, 1 - 3e-4 * 0.5), rtol=1e-6)
    assert set(opt.state[q].keys()) == {"exp_avg", "exp_avg_sq", "step"} and opt.state[q]["step"] == 1
    with pytest.raises(AssertionError):
        O.OracleSingleDeviceMuonWithAuxAdam([dict(params=[p], use_muon=True, betas=(0.9, 0.9))])
    with pytest.raises(AssertionError):
        O.OracleSingleDeviceMuonWithAuxAdam([dict(params=[p])])


# ------------------------------------------------------------------------------------------
# golden fixtures are what the oracle produces (guards against silent drift of either)
# ------------------------------------------------------------------------------------------
def test_oracle_reproduces_golden_fixtures(golden_dir):
    z = np.load(os.path.join(golden_dir, "ns_golden.npz"))
    names = sorted({k.split("/")[0] for k in z.files})
    assert len(names) >= 6
    for n in names:
        G = torch.from_numpy(z[n + "/in"])
        got = O.ns5_bf16(G).contiguous().view(torch.int16).numpy().astype(np.uint16)
        assert np.array_equal(got, z[n + "/bf16"]), n
        np.testing.assert_allclose(O.ns5_fp32(G).numpy(), z[n + "/fp32"], rtol=1e-6, atol=1e-7)
        if G.ndim == 2:
            assert O.rel_fro(z[n + "/fp32"], z[n + "/fp64_closed_form"]) < 2e-4


# ------------------------------------------------------------------------------------------
# The 4-iteration AOL-rescaled variant (muon.py:748-799)
# ------------------------------------------------------------------------------------------
def _uneven_rows(shape, seed):
    g = torch.Generator().manual_seed(seed)
    G = torch.randn(*shape, dtype=torch.float64, generator=g)
    return G * (torch.rand(*shape[:-1], 1, dtype=torch.float64, generator=g) * 3 + 0.05)


@pytest.mark.parametrize("shape", [(64, 96), (96, 64), (128, 128), (30, 200), (3, 40, 24)])
def test_aol4_matches_its_svd_closed_form(shape):
    G = _uneven_rows(shape, 77)
    want = O.ns_aol4_closed_form(G.numpy())
    assert O.rel_fro(O.ns_aol4(G, work_dtype=torch.float64), want) < 1e-12
    assert O.rel_fro(O.ns_aol4(G.float(), work_dtype=torch.float32).double(), want) < 1e-5
    assert O.rel_fro(O.ns_aol4(G.float()).double(), want) < 2e-2          # bf16 storage
    # transpose rule (muon.py:761-762, 797-798; a square matrix is never transposed, and the row
    # rescaling is not symmetric in rows and columns) and batching
    if shape[-2] != shape[-1]:
        assert O.rel_fro(O.ns_aol4(G.mT.contiguous(), work_dtype=torch.float64).mT, want) < 1e-12
    if G.ndim == 3:
        per = torch.stack([O.ns_aol4(g, work_dtype=torch.float64) for g in G])
        assert O.rel_fro(per, want) < 1e-12


def test_aol4_special_inputs_reduce_to_the_scalar_chain():
    chain1 = float(O.aol_poly_chain(1.0))
    assert abs(chain1 - (-0.9935212261846591)) < 1e-12      # the first quintic is negative above 0.884
    Q, _ = torch.linalg.qr(torch.randn(48, 48, dtype=torch.float64, generator=torch.Generator().manual_seed(5)))
    # orthogonal input: A = I, s = 1, every singular value is 1
    assert (O.ns_aol4(Q, work_dtype=torch.float64) - chain1 * Q).abs().max() < 1e-12
    # diagonal input: A = diag(d^2), s = d^2, the rescaled matrix is diag(sign d)
    d = torch.tensor([0.5, -2.0, 3.0, 0.1], dtype=torch.float64)
    got = O.ns_aol4(torch.diag(d), work_dtype=torch.float64)
    assert (got - torch.diag(chain1 * torch.sign(d))).abs().max() < 1e-12
    assert torch.count_nonzero(O.ns_aol4(torch.zeros(8, 12))) == 0


def test_aol_rescaling_bounds_the_spectral_norm_and_the_band():
    for seed, shape in enumerate([(64, 96), (200, 30), (128, 128)]):
        G = _uneven_rows(shape, 100 + seed)
        X = G.mT if shape[0] > shape[1] else G
        s = (X @ X.mT).abs().sum(-1, keepdim=True)
        assert torch.linalg.svdvals(X * torch.rsqrt(s)).max() <= 1 + 1e-12      # AOL bound
        sv = torch.linalg.svdvals(O.ns_aol4(G, work_dtype=torch.float64))
        assert sv.max() < 1.25                                                   # stays in the attracting band
    # the scalar chain maps [0.03, 0.86] into a tight band around 1 (the first quintic has a root
    # at 0.884: larger singular values change sign)
    y = O.aol_poly_chain(np.linspace(0.03, 0.86, 400))
    assert y.min() > 0.98 and y.max() < 1.02
    assert O.aol_poly_chain(0.92) < -0.9


def test_row_only_rescaling_of_the_gram_matrix_is_not_a_contraction():
    """Why ns_aol4 rescales the Gram matrix on both sides: `A / s` (muon.py:785) divides rows
    only; with the mirrored store of the polynomial kernel (muon.py:538-552, either triangle,
    muon.py:493-495) the iteration leaves the attracting band for matrices with uneven row norms."""
    def rows_only(G, upper):
        X = G.clone()
        A = X @ X.mT
        s = A.abs().sum(-1, keepdim=True).clamp_min(1e-7)
        X = X * torch.rsqrt(s)
        A = A / s
        for it, (a, b, c) in enumerate(O.AOL_CONSTS):
            if it > 0:
                A = X @ X.mT
            F = c * (A @ A.mT) + b * A
            B = torch.triu(F) + torch.triu(F, 1).mT if upper else torch.tril(F) + torch.tril(F, -1).mT
            X = a * X + B @ X
        return torch.linalg.svdvals(X).max().item()

    G = _uneven_rows((30, 200), 3)
    assert rows_only(G, True) > 10 and rows_only(G, False) > 10
    assert torch.linalg.svdvals(O.ns_aol4(G, work_dtype=torch.float64)).max() < 1.25


def test_aol4_rows_only_restatement():
    """ns_aol4_rows (muon.py:785 as written: the rows of the Gram matrix divided, its columns not):
    against a python-loop float64 restatement on tiny matrices with mildly uneven rows, where it
    differs from the two-sided rescaling; equal to it when every row sum s_i is the same."""
    for seed in range(4):
        g = torch.Generator().manual_seed(seed)
        Q, _ = torch.linalg.qr(torch.randn(8, 5, dtype=torch.float64, generator=g))
        scale = torch.tensor([1.0, 1.1, 0.9, 1.05, 0.95], dtype=torch.float64)[:, None]
        G = (Q.mT + 0.05 * torch.randn(5, 8, dtype=torch.float64, generator=g)) * scale
        got = O.ns_aol4_rows(G, work_dtype=torch.float64)
        want = torch.tensor(O.ns_aol4_rows_brute_force(G.tolist()), dtype=torch.float64)
        assert (got - want).abs().max() < 1e-12
        assert (got - O.ns_aol4(G, work_dtype=torch.float64)).abs().max() > 1e-2       # not the same map
        tall = O.ns_aol4_rows(G.mT.contiguous(), work_dtype=torch.float64)             # transpose rule, muon.py:761-762, 797-798
        assert (tall.mT - got).abs().max() < 1e-12
    Q, _ = torch.linalg.qr(torch.randn(24, 24, dtype=torch.float64, generator=torch.Generator().manual_seed(9)))
    for G in (Q, 3.0 * Q, torch.diag(torch.tensor([0.5, -2.0, 3.0], dtype=torch.float64))):
        # equal row sums (orthogonal input), and a diagonal input (A and A / s are diagonal: symmetric)
        assert (O.ns_aol4_rows(G, work_dtype=torch.float64) - O.ns_aol4(G, work_dtype=torch.float64)).abs().max() < 1e-12
    G = torch.randn(64, 96, generator=torch.Generator().manual_seed(10))
    assert O.rel_fro(O.ns_aol4_rows(G).float(), O.ns_aol4_rows(G.double(), work_dtype=torch.float64)) < 2e-2   # bf16 storage
    assert torch.count_nonzero(O.ns_aol4_rows(torch.zeros(8, 12))) == 0


def test_aol4_golden_fixture_is_what_the_oracle_computes(golden_dir):
    z = np.load(os.path.join(golden_dir, "aol4_golden.npz"))
    for name in sorted({k.split("/")[0] for k in z.files}):
        G = torch.from_numpy(z[name + "/in"])
        got = O.ns_aol4(G)
        want = torch.from_numpy(z[name + "/bf16"].astype(np.int16)).view(torch.bfloat16)
        assert O.rel_fro(got.float(), want.float()) < 1e-6, name        # bf16 CPU matmuls are deterministic here
        assert O.rel_fro(got.double(), z[name + "/fp64_closed_form"]) < 2e-2, name


# ------------------------------------------------------------------------------------------
# the three products as operators of their own (muon.py:420-457, 547-588, 705-745)
# ------------------------------------------------------------------------------------------
def test_product_operators_against_brute_force_and_the_cases_that_single_out_each_term():
    g = torch.Generator().manual_seed(21)
    A = torch.randn(5, 7, dtype=torch.float64, generator=g)
    S = torch.randn(6, 6, dtype=torch.float64, generator=g)
    S = S + S.mT
    X = torch.randn(6, 4, dtype=torch.float64, generator=g)
    T = lambda M: [list(col) for col in zip(*M)]
    mm = lambda P, Q: torch.tensor(O.matmul_brute_force(P.tolist(), Q.tolist()), dtype=torch.float64)
    # float64 in, float64 arithmetic: the formulas themselves (a transposed operand, a swapped pair of
    # scalars or a dropped term fails one of these)
    assert (O.ns_line_1(A) - mm(A, A.mT)).abs().max() < 1e-12                     # 5 x 5, not A^T A (7 x 7)
    assert O.ns_line_1(A).shape == (5, 5)
    assert (O.ns_line_2(S, 2.0, -3.0) - (2.0 * mm(S, S) - 3.0 * S)).abs().max() < 1e-12
    assert (O.ns_line_2(S, 0.0, 1.5) - 1.5 * S).abs().max() < 1e-12               # beta goes with A
    assert (O.ns_line_2(S, 1.0, 0.0) - O.ns_line_1(S)).abs().max() < 1e-12        # alpha with the product
    assert (O.ns_line_3(S, X, 0.5) - (0.5 * X + mm(S, X))).abs().max() < 1e-12    # B X, not X B or B^T... (S symmetric)
    R = torch.randn(6, 6, dtype=torch.float64, generator=g)                       # a non-symmetric B tells B X from B^T X
    assert (O.ns_line_3(R, X, 0.0) - mm(R, X)).abs().max() < 1e-12
    assert (O.ns_line_3(torch.zeros(6, 6, dtype=torch.float64), X, -2.0) + 2.0 * X).abs().max() < 1e-12
    assert (O.ns_line_3(torch.eye(6, dtype=torch.float64), X, 3.0) - 4.0 * X).abs().max() < 1e-12
    # the mirrored store (muon.py:402-413, 538-552): what is below the diagonal is the image of what
    # is above it, also for an input whose two triangles differ
    N = S * torch.tensor([1.0, 1.2, 0.8, 1.1, 0.9, 1.0], dtype=torch.float64)[:, None]
    got = O.ns_line_2(N, 1.0, 1.0)
    full = mm(N, N.mT) + N
    assert (torch.triu(got) - torch.triu(full)).abs().max() < 1e-12
    assert (got - got.mT).abs().max() == 0 and (full - full.mT).abs().max() > 1e-2
    # a batch is its matrices one by one
    Ab = torch.randn(3, 4, 9, dtype=torch.float64, generator=g)
    for k in range(3):
        assert (O.ns_line_1(Ab)[k] - O.ns_line_1(Ab[k])).abs().max() < 1e-12
    # bf16 storage: fp32 accumulation and one rounding -> within half a bf16 step of the exact value
    Ah = torch.randn(40, 72, generator=g).bfloat16()
    exact = Ah.double() @ Ah.double().mT
    got = O.ns_line_1(Ah)
    assert got.dtype == torch.bfloat16
    assert ((got.double() - exact).abs() <= 2.0 ** -8 * exact.abs() * 1.001 + 1e-5).all()
    Sh = O.ns_line_1((torch.randn(48, 48, generator=g) / 7).bfloat16())            # symmetric bf16 input
    exact = -4.775 * Sh.double() + 2.0315 * Sh.double() @ Sh.double()
    got = O.ns_line_2(Sh, 2.0315, -4.775)
    assert ((got.double() - exact).abs() <= 2.0 ** -8 * exact.abs() * 1.001 + 1e-4).all()
    Xh = torch.randn(48, 80, generator=g).bfloat16()
    exact = 3.4445 * Xh.double() + Sh.double() @ Xh.double()
    got = O.ns_line_3(Sh, Xh, 3.4445)
    assert ((got.double() - exact).abs() <= 2.0 ** -8 * exact.abs() * 1.001 + 1e-4).all()


def test_newton_schulz_iteration_built_from_the_product_operators():
    """muon.py:285-287 written with the three operators (as muon.py:789-794 does) is the iteration
    of the specification: in float64 the two agree to rounding."""
    G = torch.randn(12, 20, dtype=torch.float64, generator=torch.Generator().manual_seed(22))
    X = G / (G.norm() + 1e-7)
    for _ in range(5):
        A = O.ns_line_1(X)
        B = O.ns_line_2(A, alpha=C_, beta=B_)
        X = O.ns_line_3(B, X, A_)
    assert (X - O._ns5(G, 5, 1e-7, torch.float64)).abs().max() < 1e-12


def test_product_operator_golden_fixture_is_what_the_oracle_computes(golden_dir):
    z = np.load(os.path.join(golden_dir, "ops_golden.npz"))
    bf = lambda a: torch.from_numpy(a.astype(np.int16)).view(torch.bfloat16)
    for name in sorted({k.split("/")[0] for k in z.files}):
        X = bf(z[name + "/X"])
        A = O.ns_line_1(X)
        B = O.ns_line_2(A, 2.0315, -4.7750)
        C = O.ns_line_3(B, X, 3.4445)
        for got, key in ((A, "line1"), (B, "line2"), (C, "line3")):
            want = bf(z[f"{name}/{key}"])
            # the CPU's fp32 sums may come in another order on another host: at most one bf16 step, rarely
            d = (got.double() - want.double()).abs()
            assert (d <= 2.0 ** -7 * want.double().abs() + 1e-6).all(), (name, key)
            assert (d != 0).double().mean() < 0.01, (name, key)
            exact = torch.from_numpy(z[f"{name}/{key}_exact"]).double()
            # one rounding of the exact value, plus what fp32 sums of these terms may be off by
            Xd, Ad, Bd = X.double().abs(), bf(z[name + "/line1"]).double().abs(), bf(z[name + "/line2"]).double().abs()
            terms = {"line1": Xd @ Xd.mT, "line2": 2.0315 * (Ad @ Ad.mT) + 4.7750 * Ad, "line3": 3.4445 * Xd + Bd @ Xd}[key]
            assert ((want.double() - exact).abs() <= 2.0 ** -8 * 1.001 * exact.abs() + 2.0 ** -18 * terms).all(), (name, key)
