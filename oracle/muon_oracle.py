"""CPU oracle for the Muon optimizer step.  TEST INFRASTRUCTURE -- not product code.

Only the test-suite, the smoke check and the benchmark's CPU-baseline leg may import this
module; the shipped package never does.  Everything here runs on the CPU with plain
torch / numpy operations and restates, line by line, the algorithm of the reference
implementation (all citations are into /root/reference/muon.py):

  ns5_bf16 / ns5_fp32        muon.py:265-291  (the Newton-Schulz specification: Frobenius
                             pre-scale, `steps` quintic iterations with a, b, c =
                             3.4445, -4.7750, 2.0315, transpose-if-tall, bf16 storage)
  ns5_fp64_closed_form       the same map written through the SVD in float64:
                             U diag(p^steps(sigma / ||G||_F)) V^T, p(x) = a x + b x^3 + c x^5
  ns_aol4                    muon.py:748-799  (the live 4-iteration variant with AOL rescaling,
                             built on the Triton kernels muon.py:349-746; see its docstring
                             for what of it can and cannot be pinned)
  ns_aol4_rows               the same with muon.py:785 (`A / s`, rows only) taken as written
  ns_line_1 / _2 / _3        muon.py:420-457, 547-588, 705-745  (the three products as operators of
                             their own: A A^T, alpha A A^T + beta A, a X + B X)
  muon_update                muon.py:8-15
  adam_update                muon.py:104-109
  OracleSingleDeviceMuon     muon.py:73-101
  OracleSingleDeviceMuonWithAuxAdam   muon.py:202-260

What pins each function (the reference ships no tests, golden vectors or fixtures):
  * ns5_fp32      -- against ns5_fp64_closed_form (independent derivation through the SVD),
                     a triple-loop float64 brute force on tiny matrices, and the invariants
                     NS(G^T)=NS(G)^T, NS(alpha G)=NS(G), NS(Q1 G Q2)=Q1 NS(G) Q2, NS(0)=0,
                     NS(diag d)=diag(p^5(d/||d||)), NS(Q)=p^5(1/sqrt(m)) Q.
  * ns5_bf16      -- same code path as ns5_fp32 with the bf16 casts of muon.py:277; pinned to
                     ns5_fp32 within bf16 rounding noise and to the same invariants.
  * muon_update   -- first-step closed form (zero momentum => update = NS(g) because the
                     Nesterov blend is (1-beta^2) g and NS is scale invariant), float64
                     recurrences for several steps, the conv-shape aspect-ratio rule.
  * adam_update   -- equals torch.optim.AdamW step for step; first-step closed form g/(|g|+eps).
  * step classes  -- behavioural unit tests written from the cited lines.
  * ns_aol4       -- PARITY UNPINNED against the reference's live code: that variant only
                     runs through Triton kernels under torch.compile on a GPU (neither can
                     run where this oracle is written), its rounding points are chosen by the
                     compiler's fusion, and its `A / s` (muon.py:785) divides the rows of the
                     Gram matrix only, which is not symmetric: stored through the mirroring
                     kernel (muon.py:538-552) the result depends on the autotuned tile and
                     triangle, and in float64 the iteration then diverges for matrices with
                     uneven row norms (tests/test_oracle.py shows it).  ns_aol4 restates the
                     variant with the Gram matrix rescaled on both sides, diag(r) A diag(r) --
                     the Gram matrix of the rescaled X, which is what the derivation of the
                     iteration assumes.  That map is pinned by an independent closed form
                     (ns_aol4_closed_form: the SVD of diag(r) X with the chain of the four
                     quintics applied to its singular values), by orthogonal and diagonal
                     inputs (both reduce to the scalar chain at 1), the AOL bound
                     sigma_max(diag(r) X) <= 1, the transpose rule and batched == per-matrix.
  * ns_aol4_rows  -- the literal reading of muon.py:785.  Pinned by a python-loop float64
                     restatement on tiny matrices, by inputs whose row sums s_i are all equal
                     (then it is ns_aol4: orthogonal and scaled-orthogonal inputs), and by the
                     diagonal case.  PARITY UNPINNED against the reference's live code for the
                     same reasons as ns_aol4; in addition the reference's mirrored store makes
                     its own output depend on the autotuned block size, which is not restated.
  * ns_line_1/2/3 -- what each computes is pinned by float64 matrix products and by the special
                     cases that single out each term and each scalar (alpha = 0, beta = 0, a = 0,
                     B = 0, B = I, a row-scaled A whose two triangles differ); ns_aol4, built from
                     them, is pinned as above.  Their rounding against the reference's live
                     kernels (which run only under Triton on a GPU) is PARITY UNPINNED: fp32
                     accumulation and one cast at the store are what the kernels' source states
                     (muon.py:388-400, 512-536, 694-696); the order of the fp32 sums and, for
                     ns_line_3, the type in which the kernel forms `X * alpha` (muon.py:679-685) are
                     the compiler's.
No other function here is "parity unpinned".
"""
from __future__ import annotations

import numpy as np
import torch

NS_COEFFS = (3.4445, -4.7750, 2.0315)  # muon.py:276


# --------------------------------------------------------------------------------------
# Newton-Schulz (muon.py:265-291)
# --------------------------------------------------------------------------------------
def _ns5(G: torch.Tensor, steps: int, eps: float, work_dtype: torch.dtype) -> torch.Tensor:
    assert G.ndim >= 2                                    # muon.py:275
    a, b, c = NS_COEFFS                                   # muon.py:276
    X = G.to(work_dtype)                                  # muon.py:277 (bf16 in the reference)
    tall = G.size(-2) > G.size(-1)
    if tall:                                              # muon.py:278-279
        X = X.mT
    X = X / (X.norm(dim=(-2, -1), keepdim=True) + eps)    # muon.py:282
    for _ in range(steps):                                # muon.py:284
        A = X @ X.mT                                      # muon.py:285
        B = b * A + c * A @ A                             # muon.py:286  ((c*A) @ A)
        X = a * X + B @ X                                 # muon.py:287
    if tall:                                              # muon.py:289-290
        X = X.mT
    return X


# muon.py:754-759
AOL_CONSTS = ((4.0098, -7.0585, 2.4635), (3.4585, -5.5479, 2.5959),
              (2.7573, -3.2939, 1.4254), (2.7215, -3.0494, 1.3169))


def _upper_mirrored(F: torch.Tensor) -> torch.Tensor:
    """What a kernel that computes the blocks on or above the diagonal and stores each block and
    its transpose leaves in memory (muon.py:414-423, 538-552), taken to the limit of 1 x 1 blocks."""
    return torch.triu(F) + torch.triu(F, 1).mT


def _acc_dtype(t: torch.Tensor) -> torch.dtype:
    return torch.float64 if t.dtype == torch.float64 else torch.float32


def ns_line_1(A: torch.Tensor) -> torch.Tensor:
    """C = A @ A.T, muon.py:420-457: the kernel accumulates in fp32 and casts once to the tensor's
    dtype (muon.py:388-400), and stores every block on or above the diagonal together with its
    mirror image (muon.py:374-378, 402-413).  A is (M, K) or (batch, M, K)."""
    acc = _acc_dtype(A)
    return _upper_mirrored((A.to(acc) @ A.to(acc).mT).to(A.dtype))


def ns_line_2(A: torch.Tensor, alpha: float, beta: float) -> torch.Tensor:
    """C = alpha * A @ A.T + beta * A for a symmetric square A, muon.py:547-588: fp32 accumulation of
    the product, alpha and beta applied in fp32, one cast (muon.py:512-536), mirrored store
    (muon.py:538-552)."""
    acc = _acc_dtype(A)
    Af = A.to(acc)
    return _upper_mirrored((alpha * (Af @ Af.mT) + beta * Af).to(A.dtype))


def ns_line_3(B: torch.Tensor, X: torch.Tensor, a: float) -> torch.Tensor:
    """C = a * X + B @ X, muon.py:705-745, by the formula of its docstring (muon.py:707) in fp32 with
    one cast at the store (muon.py:694-696).  (The kernel seeds its accumulator with `X * alpha`
    evaluated by Triton's scalar promotion before the fp32 cast, muon.py:679-685: in which type that
    product is taken is the compiler's rule, not restated; PARITY UNPINNED against the live kernel.)"""
    acc = _acc_dtype(X)
    return (a * X.to(acc) + B.to(acc) @ X.to(acc)).to(X.dtype)


def ns_aol4(G: torch.Tensor, epsilon: float = 1e-7, work_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """The 4-iteration AOL-rescaled variant, muon.py:748-799, with the Gram matrix rescaled on
    both sides (see the module docstring).  Every Triton kernel of the reference accumulates in
    fp32 and rounds once at its store (muon.py:411-412, 531-536, 701-702); the pointwise torch
    expressions between them are taken in fp32 with one rounding at each stored tensor, as the
    compiler the reference runs them through fuses them.  With work_dtype=float64 nothing rounds."""
    assert G.ndim >= 2
    acc = torch.float64 if work_dtype == torch.float64 else torch.float32
    X = G.to(work_dtype)                                           # muon.py:760
    tall = G.size(-2) > G.size(-1)
    if tall:                                                       # muon.py:761-762
        X = X.mT
    A = ns_line_1(X)                                               # muon.py:778
    s = torch.clamp_min(A.to(acc).abs().sum(dim=-1, keepdim=True).to(work_dtype).to(acc), epsilon)  # muon.py:779-781
    r = torch.rsqrt(s)
    X = (X.to(acc) * r).to(work_dtype)                             # muon.py:782
    A = (A.to(acc) * (r * r.mT)).to(work_dtype)                    # muon.py:785, on both sides
    for it, (a, b, c) in enumerate(AOL_CONSTS):
        if it > 0:
            A = ns_line_1(X)                                       # muon.py:792
        B = ns_line_2(A, alpha=c, beta=b)                          # muon.py:786, 793
        X = ns_line_3(B, X, a)                                     # muon.py:787, 794
    if tall:                                                       # muon.py:797-798
        X = X.mT
    return X


def ns_aol4_rows(G: torch.Tensor, epsilon: float = 1e-7, work_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """muon.py:748-799 with `A = A / s` taken as written (muon.py:785: the rows of the Gram matrix
    are divided, its columns are not), at the level of the tensor expressions and of what the
    docstrings of the three kernels state (ns_line_1: X X^T, muon.py:364; ns_line_2:
    alpha A A^T + beta A, muon.py:485; ns_line_3: a X + B X).  The reference's polynomial kernel
    stores every block it computes and its transpose (muon.py:538-552), so on this non-symmetric A
    its own result depends on the block size its autotuner picked; that artefact is not restated
    here: B is the full, unmirrored alpha A A^T + beta A.  Roundings as in ns_aol4."""
    assert G.ndim >= 2
    acc = torch.float64 if work_dtype == torch.float64 else torch.float32
    X = G.to(work_dtype)
    tall = G.size(-2) > G.size(-1)
    if tall:
        X = X.mT
    gram = lambda Y: _upper_mirrored((Y.to(acc) @ Y.to(acc).mT).to(work_dtype))
    A = gram(X)                                                    # muon.py:778
    s = torch.clamp_min(A.to(acc).abs().sum(dim=-1, keepdim=True).to(work_dtype).to(acc), epsilon)  # muon.py:779-781
    r = torch.rsqrt(s)
    X = (X.to(acc) * r).to(work_dtype)                             # muon.py:782
    A = (A.to(acc) * (r * r)).to(work_dtype)                       # muon.py:785: A / s, rows only
    for it, (a, b, c) in enumerate(AOL_CONSTS):
        if it > 0:
            A = gram(X)
        Af = A.to(acc)
        F = (c * (Af @ Af.mT) + b * Af).to(work_dtype)             # ns_line_2
        B = F if it == 0 else _upper_mirrored(F)                   # symmetric from the second iteration on
        X = (a * X.to(acc) + B.to(acc) @ X.to(acc)).to(work_dtype)
    if tall:
        X = X.mT
    return X


def ns_aol4_rows_brute_force(G_rows, epsilon: float = 1e-7):
    """ns_aol4_rows in float64 with python loops only (lists of lists; wide or square input): an
    independent restatement for tiny matrices."""
    X = [[float(v) for v in row] for row in G_rows]
    m, n = len(X), len(X[0])
    assert m <= n
    mm = lambda P, Q: [[sum(P[i][k] * Q[k][j] for k in range(len(Q))) for j in range(len(Q[0]))] for i in range(len(P))]
    tr = lambda P: [list(col) for col in zip(*P)]
    A = mm(X, tr(X))
    s = [max(sum(abs(v) for v in row), epsilon) for row in A]
    X = [[X[i][j] / s[i] ** 0.5 for j in range(n)] for i in range(m)]
    A = [[A[i][j] / s[i] for j in range(m)] for i in range(m)]
    for it, (a, b, c) in enumerate(AOL_CONSTS):
        if it > 0:
            A = mm(X, tr(X))
        AAt = mm(A, tr(A))
        B = [[c * AAt[i][j] + b * A[i][j] for j in range(m)] for i in range(m)]
        BX = mm(B, X)
        X = [[a * X[i][j] + BX[i][j] for j in range(n)] for i in range(m)]
    return X


def ns_aol4_closed_form(G, epsilon: float = 1e-7) -> np.ndarray:
    """The same map through the SVD, in float64: with Y = diag(r) X = U diag(sigma) V^T every
    iteration acts on the singular values only, so the result is U diag(q3(q2(q1(q0(sigma))))) V^T."""
    G = np.asarray(G, dtype=np.float64)
    tall = G.shape[-2] > G.shape[-1]
    X = np.swapaxes(G, -1, -2) if tall else G
    A = X @ np.swapaxes(X, -1, -2)
    s = np.maximum(np.abs(A).sum(axis=-1, keepdims=True), epsilon)
    U, sig, Vt = np.linalg.svd(X / np.sqrt(s), full_matrices=False)
    out = (U * aol_poly_chain(sig)[..., None, :]) @ Vt
    return np.swapaxes(out, -1, -2) if tall else out


def aol_poly_chain(x):
    """q3(q2(q1(q0(x)))) for the four quintics of muon.py:754-759, elementwise in float64."""
    x = np.asarray(x, dtype=np.float64)
    for a, b, c in AOL_CONSTS:
        x = a * x + b * x ** 3 + c * x ** 5
    return x


def ns5_bf16(G: torch.Tensor, steps: int = 5, eps: float = 1e-7) -> torch.Tensor:
    """The reference bf16 result: muon.py:265-291 run with torch CPU bf16 arithmetic."""
    return _ns5(G, steps, eps, torch.bfloat16)


def ns5_fp32(G: torch.Tensor, steps: int = 5, eps: float = 1e-7) -> torch.Tensor:
    """The fp32 oracle: same sequence without the bf16 cast."""
    return _ns5(G.float(), steps, eps, torch.float32)


def ns_poly(x, steps: int = 5):
    """p^steps(x) with p(x) = a x + b x^3 + c x^5, the scalar map NS applies to singular values."""
    a, b, c = NS_COEFFS
    x = np.asarray(x, dtype=np.float64)
    for _ in range(steps):
        x2 = x * x
        x = x * (a + x2 * (b + c * x2))
    return x


def ns5_fp64_closed_form(G, steps: int = 5, eps: float = 1e-7) -> np.ndarray:
    """U diag(p^steps(sigma/(||G||_F+eps))) V^T in float64; 2-D input only."""
    G = np.asarray(G.detach().double().cpu().numpy() if isinstance(G, torch.Tensor) else G,
                   dtype=np.float64)
    assert G.ndim == 2
    U, s, Vt = np.linalg.svd(G, full_matrices=False)
    fro = np.sqrt((s * s).sum())
    return (U * ns_poly(s / (fro + eps), steps)) @ Vt


# --------------------------------------------------------------------------------------
# Update rules
# --------------------------------------------------------------------------------------
def muon_update(grad: torch.Tensor, momentum: torch.Tensor, beta: float = 0.95,
                nesterov: bool = True, ns_steps: int = 5, ns=None) -> torch.Tensor:
    """muon.py:8-15.  Mutates `momentum` and (with nesterov) `grad` exactly as the reference.
    `ns` replaces the orthogonalisation (muon.py:13 calls whichever zeropower_via_newtonschulz5
    the module defines: the specification by default here, ns_aol4 for the live variant)."""
    momentum.lerp_(grad, 1 - beta)                                        # muon.py:9
    update = grad.lerp_(momentum, beta) if nesterov else momentum         # muon.py:10
    if update.ndim == 4:                                                  # muon.py:11-12
        update = update.view(len(update), -1)
    update = ns5_bf16(update, ns_steps) if ns is None else ns(update)     # muon.py:13
    update *= max(1, grad.size(-2) / grad.size(-1)) ** 0.5                # muon.py:14
    return update


def adam_update(grad, buf1, buf2, step, betas, eps):
    """muon.py:104-109."""
    buf1.lerp_(grad, 1 - betas[0])                       # muon.py:105
    buf2.lerp_(grad.square(), 1 - betas[1])              # muon.py:106
    buf1c = buf1 / (1 - betas[0] ** step)                # muon.py:107
    buf2c = buf2 / (1 - betas[1] ** step)                # muon.py:108
    return buf1c / (buf2c.sqrt() + eps)                  # muon.py:109


# --------------------------------------------------------------------------------------
# Optimizer classes (single-device semantics)
# --------------------------------------------------------------------------------------
class OracleSingleDeviceMuon(torch.optim.Optimizer):
    """muon.py:73-101."""

    def __init__(self, params, lr=0.02, weight_decay=0, momentum=0.95, ns=None):
        defaults = dict(lr=lr, weight_decay=weight_decay, momentum=momentum)
        super().__init__(params, defaults)
        self.ns = ns

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            for p in group["params"]:
                _muon_param_step(self, p, group)
        return loss


def _muon_param_step(opt, p, group):
    if p.grad is None:                                                     # muon.py:91-93
        p.grad = torch.zeros_like(p)
    state = opt.state[p]
    if len(state) == 0:                                                    # muon.py:95-96
        state["momentum_buffer"] = torch.zeros_like(p)
    update = muon_update(p.grad, state["momentum_buffer"], beta=group["momentum"],
                         ns=getattr(opt, "ns", None))                      # muon.py:97
    p.mul_(1 - group["lr"] * group["weight_decay"])                        # muon.py:98
    p.add_(update.reshape(p.shape), alpha=-group["lr"])                    # muon.py:99


def _adam_param_step(opt, p, group):
    if p.grad is None:                                                     # muon.py:246-248
        p.grad = torch.zeros_like(p)
    state = opt.state[p]
    if len(state) == 0:                                                    # muon.py:250-253
        state["exp_avg"] = torch.zeros_like(p)
        state["exp_avg_sq"] = torch.zeros_like(p)
        state["step"] = 0
    state["step"] += 1                                                     # muon.py:254
    update = adam_update(p.grad, state["exp_avg"], state["exp_avg_sq"],
                         state["step"], group["betas"], group["eps"])      # muon.py:255-256
    p.mul_(1 - group["lr"] * group["weight_decay"])                        # muon.py:257
    p.add_(update, alpha=-group["lr"])                                     # muon.py:258


class OracleSingleDeviceMuonWithAuxAdam(torch.optim.Optimizer):
    """muon.py:202-260."""

    def __init__(self, param_groups, ns=None):
        self.ns = ns
        for group in param_groups:
            assert "use_muon" in group
            if group["use_muon"]:
                group["lr"] = group.get("lr", 0.02)
                group["momentum"] = group.get("momentum", 0.95)
                group["weight_decay"] = group.get("weight_decay", 0)
                assert set(group.keys()) == {"params", "lr", "momentum", "weight_decay", "use_muon"}
            else:
                group["lr"] = group.get("lr", 3e-4)
                group["betas"] = group.get("betas", (0.9, 0.95))
                group["eps"] = group.get("eps", 1e-10)
                group["weight_decay"] = group.get("weight_decay", 0)
                assert set(group.keys()) == {"params", "lr", "betas", "eps", "weight_decay", "use_muon"}
        super().__init__(param_groups, dict())

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            if group["use_muon"]:
                for p in group["params"]:
                    _muon_param_step(self, p, group)
            else:
                for p in group["params"]:
                    _adam_param_step(self, p, group)
        return loss


# --------------------------------------------------------------------------------------
# Helpers used by tests
# --------------------------------------------------------------------------------------
def rel_fro(x, ref) -> float:
    """Relative Frobenius error ||x - ref||_F / ||ref||_F computed in float64."""
    x = x.detach().double().cpu() if isinstance(x, torch.Tensor) else torch.as_tensor(np.asarray(x)).double()
    ref = ref.detach().double().cpu() if isinstance(ref, torch.Tensor) else torch.as_tensor(np.asarray(ref)).double()
    den = ref.norm().item()
    num = (x - ref).norm().item()
    return num / den if den > 0 else num


def matmul_brute_force(A, B):
    """Textbook triple loop in Python floats (float64); tiny matrices only."""
    n, k = len(A), len(A[0])
    k2, m = len(B), len(B[0])
    assert k == k2
    C = [[0.0] * m for _ in range(n)]
    for i in range(n):
        for j in range(m):
            s = 0.0
            for t in range(k):
                s += A[i][t] * B[t][j]
            C[i][j] = s
    return C


def ns5_brute_force(G_rows, steps: int = 5, eps: float = 1e-7):
    """muon.py:278-290 with every product a triple loop; G_rows: list of lists (2-D)."""
    a, b, c = NS_COEFFS
    r, cc = len(G_rows), len(G_rows[0])
    X = [list(map(float, row)) for row in G_rows]
    tall = r > cc
    T = lambda M: [list(col) for col in zip(*M)]
    if tall:
        X = T(X)
    fro = sum(v * v for row in X for v in row) ** 0.5
    X = [[v / (fro + eps) for v in row] for row in X]
    for _ in range(steps):
        A = matmul_brute_force(X, T(X))
        AA = matmul_brute_force(A, A)
        B = [[b * A[i][j] + c * AA[i][j] for j in range(len(A))] for i in range(len(A))]
        BX = matmul_brute_force(B, X)
        X = [[a * X[i][j] + BX[i][j] for j in range(len(X[0]))] for i in range(len(X))]
    if tall:
        X = T(X)
    return X
