"""Functional API with the reference's names and argument order (reference muon.py:8-15,
104-109, 265-291), executed by the gfx950 kernels of libmuon_amd.so."""
from __future__ import annotations

import threading
from collections import OrderedDict
from contextlib import contextmanager

import torch

from . import _lib
from .engine import AdamGroupEngine, MuonGroupEngine, require_gpu_tensor
from .plan import AOL_COEFFS

_ROUNDINGS = {"reference": True, "fused": False}
_ENGINE_CACHE: "OrderedDict[tuple, object]" = OrderedDict()
_ENGINE_CACHE_MAX = 4     # each cached engine holds its bf16 workspace


_CACHE_LOCK = threading.Lock()


_PRODUCT_CACHE: "OrderedDict[tuple, object]" = OrderedDict()      # job tables of the stand-alone products: small
_PRODUCT_CACHE_MAX = 64


def _cached(key, make, cache=None, limit=_ENGINE_CACHE_MAX):
    cache = _ENGINE_CACHE if cache is None else cache
    with _CACHE_LOCK:
        eng = cache.get(key)
        if eng is None:
            eng = make()
            eng._fn_lock = threading.Lock()       # one caller at a time enqueues on this engine
            eng._fn_done = None                   # event after the launches of its last call
            cache[key] = eng
            while len(cache) > limit:
                cache.popitem(last=False)
        else:
            cache.move_to_end(key)
        return eng


@contextmanager
def _exclusive(eng, device):
    """A cached engine owns one workspace, so its calls must not overlap, neither on the host (two
    threads enqueueing at once) nor on the device (two streams running its launches side by side):
    callers take the engine's lock, and the stream of a call waits for the launches of the call
    before it.  (Not while a HIP graph is being captured: the event of an earlier, uncaptured call
    cannot be waited for there, and a capture runs on one stream anyway.)"""
    with eng._fn_lock:
        stream = torch.cuda.current_stream(device)
        capturing = torch.cuda.is_current_stream_capturing()
        if eng._fn_done is not None and not capturing:
            stream.wait_event(eng._fn_done)
        yield
        if not capturing:
            done = torch.cuda.Event()
            done.record(stream)
            eng._fn_done = done


def clear_engine_cache() -> None:
    """Drop the workspaces cached by the functional entry points."""
    with _CACHE_LOCK:
        _ENGINE_CACHE.clear()
        _PRODUCT_CACHE.clear()


def _rounding_flag(rounding: str) -> bool:
    if rounding not in _ROUNDINGS:
        raise ValueError(f"rounding must be one of {sorted(_ROUNDINGS)}, got {rounding!r}")
    return _ROUNDINGS[rounding]


def _src_dtype(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return _lib.SRC_F32
    if t.dtype == torch.bfloat16:
        return _lib.SRC_BF16
    raise TypeError(f"unsupported dtype {t.dtype}")


def _orthogonalise(G: torch.Tensor, steps: int, epsilon: float, ref: bool, variant: str) -> torch.Tensor:
    assert G.ndim >= 2                                     # muon.py:275
    require_gpu_tensor(G, "G")
    if G.dtype not in (torch.float32, torch.bfloat16):
        G = G.float()
    G = G.contiguous()
    rows, cols = G.size(-2), G.size(-1)
    batch = G.numel() // (rows * cols) if rows * cols else 0
    out = torch.empty(G.shape, dtype=torch.bfloat16, device=G.device)
    if G.numel() == 0:
        return out
    with torch.cuda.device(G.device):
        eng = _cached(("ns", G.device, rows, cols, batch, int(steps), ref, variant),
                      lambda: MuonGroupEngine([(rows, cols)] * batch, G.device, int(steps), ref, variant=variant))
        gsz, osz = rows * cols * G.element_size(), rows * cols * 2
        with _exclusive(eng, G.device):
            eng.run([G.data_ptr() + b * gsz for b in range(batch)], [0] * batch, [0] * batch,
                    [out.data_ptr() + b * osz for b in range(batch)], [1.0] * batch,
                    [_src_dtype(G)] * batch, beta=0.0, nesterov=False, mutate_grad=False,
                    eps=float(epsilon), lr=0.0, weight_decay=0.0)
    return out


def zeropower_via_newtonschulz5(G: torch.Tensor, steps: int = 5, epsilon: float = 1e-7, *,
                                rounding: str = "reference") -> torch.Tensor:
    """Newton-Schulz orthogonalisation of G (reference muon.py:265-291): bf16 result of the
    shape of G; leading dimensions are a batch.

    rounding="reference" rounds to bf16 wherever the reference's bf16 tensor expression does;
    "fused" rounds once per stored matrix (closer to the fp32 result).

    The second positional argument is the iteration count, as in the specification
    (muon.py:265-266); the reference's live function takes epsilon there (muon.py:749), so a
    non-integral value in that place is refused rather than truncated to zero iterations.
    """
    if isinstance(steps, bool) or int(steps) != steps or steps < 0:
        raise TypeError(f"steps must be a non-negative integer, got {steps!r} (pass epsilon by keyword)")
    return _orthogonalise(G, steps, epsilon, _rounding_flag(rounding), "ns5")


def zeropower_via_aol4(G: torch.Tensor, epsilon: float = 1e-7, *, rescale: str = "symmetric") -> torch.Tensor:
    """The 4-iteration variant with AOL rescaling (reference muon.py:748-799): instead of the
    Frobenius pre-scale, the rows of X are divided by sqrt(sum_j |(X X^T)_ij|), which bounds the
    spectral norm by 1 and starts closer to orthogonal; four quintic iterations with the
    coefficients of muon.py:754-759 follow, the first reusing the rescaled Gram matrix.

    rescale="symmetric" (default) rescales the Gram matrix on both sides, diag(r) A diag(r): it
    then is the Gram matrix of the rescaled X, which the iteration assumes.  rescale="rows" divides
    its rows only, `A / s`, as muon.py:785 is written: A is then not symmetric, the first
    polynomial c * A A^T + b * A is computed over every tile, and for matrices with uneven row
    norms the iteration loses its contraction (the reference's own result further depends on the
    tile its autotuner picked, through the mirrored store of its polynomial kernel).
    """
    if rescale not in ("symmetric", "rows"):
        raise ValueError(f"rescale must be 'symmetric' or 'rows', got {rescale!r}")
    return _orthogonalise(G, len(AOL_COEFFS), epsilon, False, "aol4" if rescale == "symmetric" else "aol4_rows")


def muon_update(grad: torch.Tensor, momentum: torch.Tensor, beta: float = 0.95,
                nesterov: bool = True, ns_steps: int = 5, *, rounding: str = "reference",
                ns_variant: str = "ns5") -> torch.Tensor:
    """Reference muon.py:8-15.  Updates `momentum` in place, overwrites `grad` with the Nesterov
    blend (as the reference's grad.lerp_ does) and returns the scaled bf16 orthogonalised update
    (2-D for 4-D conv filters, else the shape of grad)."""
    require_gpu_tensor(grad, "grad")
    require_gpu_tensor(momentum, "momentum")
    assert grad.ndim >= 2                                  # muon.py:275 via muon.py:13
    if grad.dtype != momentum.dtype or grad.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError("muon_update needs grad and momentum of one dtype, fp32 or bf16")
    if not (grad.is_contiguous() and momentum.is_contiguous()):
        raise ValueError("muon_update needs contiguous grad and momentum (they are updated in place)")
    assert grad.shape == momentum.shape
    ref = _rounding_flag(rounding)
    if grad.ndim == 4:                                     # muon.py:11-12
        rows, cols = grad.size(0), grad.numel() // max(grad.size(0), 1)
        batch, out_shape = 1, (rows, cols)
    else:
        rows, cols = grad.size(-2), grad.size(-1)
        batch, out_shape = (grad.numel() // (rows * cols) if rows * cols else 0), tuple(grad.shape)
    scale = max(1, grad.size(-2) / grad.size(-1)) ** 0.5   # muon.py:14 (sizes of the un-flattened grad)
    out = torch.empty(out_shape, dtype=torch.bfloat16, device=grad.device)
    if grad.numel() == 0:
        return out
    with torch.cuda.device(grad.device):
        eng = _cached(("ns", grad.device, rows, cols, batch, int(ns_steps), ref, ns_variant),
                      lambda: MuonGroupEngine([(rows, cols)] * batch, grad.device, int(ns_steps), ref,
                                              variant=ns_variant))
        gsz, osz = rows * cols * grad.element_size(), rows * cols * 2
        with _exclusive(eng, grad.device):
            eng.run([grad.data_ptr() + b * gsz for b in range(batch)],
                    [momentum.data_ptr() + b * gsz for b in range(batch)], [0] * batch,
                    [out.data_ptr() + b * osz for b in range(batch)], [scale] * batch,
                    [_src_dtype(grad)] * batch, beta=beta, nesterov=bool(nesterov), mutate_grad=True,
                    eps=1e-7, lr=0.0, weight_decay=0.0)
    return out


def adam_update(grad, buf1, buf2, step, betas, eps) -> torch.Tensor:
    """Reference muon.py:104-109: updates both moment buffers in place and returns the
    bias-corrected Adam direction (in the dtype of the inputs: fp32 or bf16)."""
    for name, t in (("grad", grad), ("buf1", buf1), ("buf2", buf2)):
        require_gpu_tensor(t, name)
        if t.dtype != grad.dtype or t.dtype not in (torch.float32, torch.bfloat16):
            raise TypeError("adam_update needs tensors of one dtype, fp32 or bf16")
    if not (buf1.is_contiguous() and buf2.is_contiguous()):
        raise ValueError("adam_update needs contiguous moment buffers (they are updated in place)")
    grad = grad.contiguous()
    out = torch.empty_like(grad)
    if grad.numel() == 0:
        return out
    with torch.cuda.device(grad.device):
        eng = _cached(("adam", grad.device, grad.numel()), lambda: AdamGroupEngine([grad.numel()], grad.device))
        with _exclusive(eng, grad.device):
            eng.run([0], [grad.data_ptr()], [buf1.data_ptr()], [buf2.data_ptr()], [out.data_ptr()],
                    lr=0.0, weight_decay=0.0, betas=betas, eps=float(eps), step=step, dtypes=[_src_dtype(grad)])
    return out
