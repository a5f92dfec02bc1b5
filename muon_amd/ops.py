"""The three products of a Newton-Schulz iteration as operators of their own, under the reference's
names with its argument order, defaults and shape errors (reference muon.py:420-457, 547-588,
705-745), executed by the grouped GEMM kernel of libmuon_amd.so.

    ns_line_1(A)               C = A A^T
    ns_line_2(A, alpha, beta)  C = alpha * A A^T + beta * A      (A square and symmetric)
    ns_line_3(B, X, a)         C = a * X + B X                   (B square)

Arithmetic: bf16 operands, fp32 accumulation, one rounding to bf16 of the finished expression, as
the reference's kernels do (muon.py:399-400, 531-536, 675-696).  The two symmetric products compute
the tiles on and above the diagonal and store each with its mirror image (muon.py:402-413): for a
symmetric A, which ns_line_2 asks for, that is the whole result; otherwise what lands below the
diagonal tiles is the image of what is above them, and depends on the tile size here (128 or 256)
as it does on the autotuned block in the reference.  bf16 CUDA tensors only; any strides; 2-D or
3-D (a batch).

The optimizer classes do not come through here: they run the same kernel over whole parameter
groups with its fused epilogues.  These entry points serve callers that used the reference's
operators directly.
"""
from __future__ import annotations

import numpy as np
import torch

from . import _lib, plan as _plan
from .engine import _Staging, _stream_ptr, _upload, require_gpu_tensor
from .functional import _PRODUCT_CACHE, _PRODUCT_CACHE_MAX, _cached, _exclusive


def _product_jobs(tile_class: int, batch: int, rows_p: int, cols_p: int, kdim: int, sym: bool,
                  nsplit: int = 1) -> np.ndarray:
    """One job per output tile and matrix (for a mirrored product: per tile on or above the
    diagonal), in super-block order dealt to the XCDs.  nsplit > 1: the reduction of every tile is
    shared by nsplit jobs that meet in a group of fp32 slots (tile t of the launch: slots
    t * nsplit ..), as the optimizer does for the X X^T of short, very wide matrices."""
    TR, TC = _plan.TILE_DIMS[tile_class]
    si, sj = _plan.SUPER_DIMS[tile_class]
    ti, tj = _plan._tile_order(rows_p // TR, cols_p // TC, sym, TR // TC, si, sj)
    one = np.zeros(len(ti) * nsplit, dtype=_lib.TILE_JOB)
    one["i0"], one["j0"] = np.repeat(ti * TR, nsplit), np.repeat(tj * TC, nsplit)
    if sym:
        one["diag"] = np.repeat((ti == tj // (TR // TC)).astype(np.int32), nsplit)
    if nsplit == 1:
        one["k1"] = kdim
    else:
        edges = (np.arange(nsplit + 1) * (kdim // _plan.GEMM_BK) // nsplit) * _plan.GEMM_BK
        idx = np.tile(np.arange(nsplit), len(ti))
        one["k0"], one["k1"] = edges[idx], edges[idx + 1]
        one["part_base"] = np.repeat(np.arange(len(ti)) * nsplit, nsplit)
        one["split"] = idx | (nsplit << 16)
    jobs = np.tile(one, batch)
    jobs["desc"] = np.repeat(np.arange(batch, dtype=np.int32), len(one))
    if nsplit > 1:
        jobs["part_base"] += np.repeat(np.arange(batch) * len(ti) * nsplit, len(one))
    return np.ascontiguousarray(jobs[_plan.xcd_permutation(len(jobs), si * sj)])


class _Product:
    """Job list (uploaded once), descriptor buffer and, for split reductions, the fp32 slots and
    their counters, of one product shape on one device."""

    def __init__(self, device, tile_class: int, batch: int, rows_p: int, cols_p: int, kdim: int, sym: bool,
                 nsplit: int = 1):
        self.jobs = _product_jobs(tile_class, batch, rows_p, cols_p, kdim, sym, nsplit)
        self.device = device
        self.tile_class = tile_class
        self.batch = batch
        self.jobs_dev = _upload(self.jobs, device)
        self.desc_dev = torch.empty(batch * _lib.GEMM_DESC.itemsize, dtype=torch.uint8, device=device)
        self.staging = _Staging(device)
        self.desc_key = None
        self.split_slots = len(self.jobs) if nsplit > 1 else 0
        if self.split_slots:
            TR, TC = _plan.TILE_DIMS[tile_class]
            self.partials = torch.empty(self.split_slots * TR * TC, dtype=torch.float32, device=device)
            self.counters = torch.zeros(self.split_slots, dtype=torch.int32, device=device)

    def launch(self, descs: np.ndarray, alpha: float, beta: float, flags: int) -> None:
        lib = _lib.load()
        key = descs.tobytes()
        if key != self.desc_key:          # the same tensors as last time (a loop over fixed buffers): nothing to redo
            _lib.check(lib.muon_amd_validate_gemm(_lib.host_ptr(descs), self.batch, _lib.host_ptr(self.jobs),
                                                  len(self.jobs), self.tile_class, self.split_slots), "validate_gemm")
            self.staging.upload(descs, self.desc_dev)
            self.desc_key = key
        partials = counters = None
        if self.split_slots:
            self.counters.zero_()         # every launch leaves them zero; a launch that died must not poison the next
            partials, counters = self.partials.data_ptr(), self.counters.data_ptr()
        _lib.check(lib.muon_amd_ns_gemm(self.desc_dev.data_ptr(), self.jobs_dev.data_ptr(), len(self.jobs),
                                        self.tile_class, alpha, beta, 0.0, flags, partials, counters,
                                        _stream_ptr(self.device)), "ns_gemm")


def _check_input(t: torch.Tensor, name: str) -> None:
    require_gpu_tensor(t, name)
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name} is {t.dtype}: the products run on bf16 tensors")


def _as_batch(t: torch.Tensor) -> torch.Tensor:
    return t if t.ndim == 3 else t.unsqueeze(0)


def _padded(t3: torch.Tensor, rows_p: int, cols_p: int) -> torch.Tensor:
    """`t3` (batch, r, c) as row-major memory of rows_p x cols_p per matrix, zero beyond r x c: the
    tensor itself when it already is that, else a copy."""
    b, r, c = t3.shape
    if r == rows_p and c == cols_p and t3.is_contiguous() and t3.data_ptr() % 16 == 0:
        return t3
    buf = torch.zeros((b, rows_p, cols_p), dtype=torch.bfloat16, device=t3.device)
    buf[:, :r, :c] = t3
    return buf


def _overlaps(a: torch.Tensor, b: torch.Tensor) -> bool:
    return a.untyped_storage().data_ptr() == b.untyped_storage().data_ptr()


def _result(out3: torch.Tensor, rows_p: int, cols_p: int, *inputs) -> torch.Tensor:
    """Where the kernel writes: `out3` itself when it is padded row-major memory apart from the
    inputs (tiles of one launch read operands while others store), else a buffer copied out after."""
    b, r, c = out3.shape
    if (r == rows_p and c == cols_p and out3.is_contiguous() and out3.data_ptr() % 16 == 0 and
            not any(_overlaps(out3, t) for t in inputs)):
        return out3
    return torch.empty((b, rows_p, cols_p), dtype=torch.bfloat16, device=out3.device)


def _addresses(t3: torch.Tensor, batch: int):
    step = t3.stride(0) * 2 if t3.size(0) > 1 else 0
    return [t3.data_ptr() + k * step for k in range(batch)]


def _symmetric_product(A: torch.Tensor, out, alpha: float, beta: float, addend: bool) -> torch.Tensor:
    M, K = A.shape[-2:]
    if out is None:
        out = torch.empty((*A.shape[:-1], M), device=A.device, dtype=A.dtype)
    assert out.size(-2) == M, "Output matrix has incorrect shape"
    assert out.size(-1) == M, "Output matrix has incorrect shape"
    _check_input(out, "out")
    assert out.ndim == A.ndim and out.device == A.device and out.shape[:-2] == A.shape[:-2]
    if M == 0 or A.numel() == 0:
        if out.numel():
            out.zero_()
        return out
    A3, out3 = _as_batch(A), _as_batch(out)
    batch = A3.size(0)
    tile_class = _plan.tile_class_for(M)
    unit = _plan.pad_unit(tile_class)
    mp = _plan._round_up(M, unit)
    kp = mp if addend else _plan._round_up(K, _plan.GEMM_BK)
    with torch.cuda.device(A.device):
        # X X^T of a short, very wide matrix: a few tiles with very long reductions, which are split
        nsplit = 1 if addend or tile_class != 0 else _plan.split_factor(mp, kp)
        prod = _cached(("sym_product", A.device, tile_class, batch, mp, kp, nsplit),
                       lambda: _Product(A.device, tile_class, batch, mp, mp, kp, True, nsplit),
                       _PRODUCT_CACHE, _PRODUCT_CACHE_MAX)
        with _exclusive(prod, A.device):
            src = _padded(A3, mp, kp)
            dst = _result(out3, mp, mp, A3)
            d = np.zeros(batch, dtype=_lib.GEMM_DESC)
            d["P"] = d["Q"] = _addresses(src, batch)
            if addend:
                d["D"] = d["P"]
                d["ldd"] = kp
            d["C"] = d["CT"] = _addresses(dst, batch)
            d["ldp"] = d["ldq"] = kp
            d["ldc"] = d["ldct"] = mp
            d["K"], d["rows"], d["colsn"] = kp, mp, mp
            # one rounding of the finished expression; without an addend the product's own rounding
            # is that one rounding in either mode, and the reference-mode path takes it exactly
            prod.launch(d, float(alpha), float(beta), _lib.ROUND_FUSED if addend else _lib.ROUND_REFERENCE)
            if dst is not out3:
                out3.copy_(dst[:, :M, :M])
    return out


def ns_line_1(A: torch.Tensor, *, out: torch.Tensor = None) -> torch.Tensor:
    """C = A @ A.T (reference muon.py:420-457); A is (M, K) or (batch, M, K)."""
    if A.ndim > 3 or A.ndim < 2:
        raise ValueError(f"Input tensor must be 2D or 3D, but got {A.ndim}D tensor.")
    _check_input(A, "A")
    return _symmetric_product(A, out, 1.0, 0.0, False)


def ns_line_2(A: torch.Tensor, alpha: float, beta: float, *, out: torch.Tensor = None) -> torch.Tensor:
    """C = alpha * A @ A.T + beta * A (reference muon.py:547-588); A square and symmetric."""
    if A.ndim > 3 or A.ndim < 2:
        raise ValueError(f"Input tensor must be 2D or 3D, but got {A.ndim}D tensor.")
    M, K = A.shape[-2:]
    if M != K:
        raise ValueError(f"Input must be symmetric square matrix, but got shape {A.shape}")
    _check_input(A, "A")
    return _symmetric_product(A, out, alpha, beta, True)


def ns_line_3(B: torch.Tensor, X: torch.Tensor, a: float, *, out: torch.Tensor = None) -> torch.Tensor:
    """C = a * X + B @ X (reference muon.py:705-745); B is (M, M) or (batch, M, M), X (M, N) or
    (batch, M, N); a 2-D B goes with every matrix of a 3-D X."""
    if B.shape[-2] != B.shape[-1]:
        raise ValueError("B must be square")
    if B.shape[-2] != X.shape[-2]:
        raise ValueError("B and X must have the same number of rows")
    if X.ndim > 3 or X.ndim < 2 or B.ndim > 3 or B.ndim < 2:
        raise ValueError(f"Input tensors must be 2D or 3D, but got {B.ndim}D and {X.ndim}D tensors.")
    _check_input(B, "B")
    _check_input(X, "X")
    assert B.device == X.device
    M, N = X.shape[-2:]
    if out is None:
        out = torch.empty_like(X)
    _check_input(out, "out")
    assert out.shape == X.shape and out.device == X.device
    if X.numel() == 0:
        return out
    X3, B3, out3 = _as_batch(X), _as_batch(B), _as_batch(out)
    batch = X3.size(0)
    assert B3.size(0) in (1, batch), "B and X must have the same batch size"
    tile_class = _plan.tile_class_for(min(M, N))
    unit = _plan.pad_unit(tile_class)
    mp, np_ = _plan._round_up(M, unit), _plan._round_up(N, unit)
    # as in the optimizer's update launches: 256 x 256 tiles also for shorter matrices when their
    # padded sizes allow it and there are enough of them to give every CU one
    if (tile_class == 0 and mp % 256 == 0 and np_ % 256 == 0 and
            batch * (mp // 256) * (np_ // 256) >= _plan.RESIDENT_BIG_TILE_WORKGROUPS):
        tile_class = 1
    with torch.cuda.device(X.device):
        prod = _cached(("update_product", X.device, tile_class, batch, mp, np_),
                       lambda: _Product(X.device, tile_class, batch, mp, np_, mp, False),
                       _PRODUCT_CACHE, _PRODUCT_CACHE_MAX)
        with _exclusive(prod, X.device):
            bsrc, xsrc = _padded(B3, mp, mp), _padded(X3, mp, np_)
            dst = _result(out3, mp, np_, X3, B3)
            d = np.zeros(batch, dtype=_lib.GEMM_DESC)
            d["P"] = _addresses(bsrc, batch)
            # X itself is the second operand, read k-major (its rows are the reduction), and the addend
            d["Q"] = d["D"] = _addresses(xsrc, batch)
            d["q_kmajor"] = 1
            d["C"] = _addresses(dst, batch)
            d["ldp"] = mp
            d["ldq"] = d["ldd"] = d["ldc"] = np_
            d["K"], d["rows"], d["colsn"] = mp, mp, np_
            prod.launch(d, 1.0, float(a), _lib.ROUND_FUSED | _lib.GEMM_Q_KMAJOR)
            if dst is not out3:
                out3.copy_(dst[:, :M, :N])
    return out
