"""Device-side driver of the grouped Muon / Adam launches (torch for memory and streams only)."""
from __future__ import annotations

import contextlib
import os

import numpy as np
import torch

from . import _lib, plan as _plan

DEFAULT_WORKSPACE_CAP = int(os.environ.get("MUON_AMD_WORKSPACE_BYTES", 16 << 30))


def require_gpu_tensor(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise _lib.MuonAmdError(
            f"{what} is on {t.device}: muon_amd runs on an MI355X (gfx950) GPU only and has no "
            "CPU implementation")


# When set to a list, every launch is bracketed by a pair of HIP events recorded on the stream it
# runs on, and (label, algorithmic work, start, stop) is appended.  Work is flops for the GEMM
# launches (the minimum given symmetry, on the unpadded sizes) and bytes for the others.
PROFILE = None


def _launch(label, work, call):
    if PROFILE is None:
        call()
        return
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    call()
    e1.record()
    PROFILE.append((label, work, e0, e1))


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _upload(arr: np.ndarray, device) -> torch.Tensor:
    """Async host->device copy of a table that is uploaded once, through pinned staging (no stream
    or host sync)."""
    host = torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).reshape(-1)).pin_memory()
    return host.to(device, non_blocking=True)


class _Staging:
    """One pinned host buffer for the tables an engine uploads again and again (matrix descriptors
    after a tensor moved, Adam descriptors, a graph's scalars): the bytes are copied into it and from
    there to the device asynchronously.  Before the buffer is overwritten the host waits for the
    copy that last read it, which has normally finished long ago."""

    def __init__(self, device):
        self.device = device
        self.host = None
        self.event = None

    def upload(self, arr: np.ndarray, into: torch.Tensor) -> torch.Tensor:
        src = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
        n = src.size
        assert into.numel() == n, (into.numel(), n)
        if self.host is None or self.host.numel() < n:
            if self.event is not None:
                self.event.synchronize()
            self.host = torch.empty(max(n, 4096), dtype=torch.uint8, pin_memory=True)
            self.event = torch.cuda.Event()
        else:
            self.event.synchronize()
        self.host[:n].numpy()[:] = src
        into.copy_(self.host[:n], non_blocking=True)
        self.event.record(torch.cuda.current_stream(self.device))
        return into


class _ChunkRuntime:
    def __init__(self, chunk: _plan.ChunkPlan, base: int, device):
        self.staging = _Staging(device)
        lib = _lib.load()
        self.chunk = chunk
        self.device = device
        gemm = chunk.gemm_descs(base)
        for ph in range(_plan.N_PHASES):
            if ph == _plan.PH_POLY_FULL and chunk.poly_full_jobs is None:
                continue
            jobs = (chunk.syrk_jobs if ph in (_plan.PH_SYRK, _plan.PH_SYRK_ODD) else
                    chunk.sym_jobs if ph == _plan.PH_POLY else
                    chunk.poly_full_jobs if ph == _plan.PH_POLY_FULL else chunk.full_jobs)
            full = ph in (_plan.PH_UPD_EVEN, _plan.PH_UPD_ODD, _plan.PH_UPD_LAST)
            _lib.check(lib.muon_amd_validate_gemm(_lib.host_ptr(gemm[ph]), chunk.nmat,
                                                  _lib.host_ptr(jobs), len(jobs),
                                                  chunk.update_class if full else chunk.tile_class,
                                                  chunk.split_slots if ph in (_plan.PH_SYRK, _plan.PH_SYRK_ODD) else 0),
                       "validate_gemm")
        self.mat_template = chunk.mat_descs(base)
        # one static device blob: gemm descs | sym jobs | full jobs | block prefix | tile prefix |
        # syrk jobs (| AOL descs | AOL row prefix | AOL segment prefix), each part 256-byte aligned
        parts = [gemm.reshape(-1).view(np.uint8), chunk.sym_jobs.view(np.uint8),
                 chunk.full_jobs.view(np.uint8), chunk.block_prefix.view(np.uint8),
                 chunk.tile_prefix.view(np.uint8), chunk.syrk_jobs.view(np.uint8)]
        if chunk.aol:
            aol = chunk.aol_descs(base)
            _lib.check(lib.muon_amd_validate_aol(_lib.host_ptr(aol), chunk.nmat,
                                                 _lib.host_ptr(chunk.aol_row_prefix),
                                                 _lib.host_ptr(chunk.aol_seg_prefix)), "validate_aol")
            parts += [aol.view(np.uint8), chunk.aol_row_prefix.view(np.uint8),
                      chunk.aol_seg_prefix.view(np.uint8)]
            if chunk.poly_full_jobs is not None:
                parts.append(chunk.poly_full_jobs.view(np.uint8))
        # {0, blocks of matrix k} for every k: the prefix table of a momentum launch over matrix k alone
        single = np.zeros((chunk.nmat, 2), dtype=np.int32)
        single[:, 1] = np.diff(chunk.block_prefix)
        parts.append(single.reshape(-1).view(np.uint8))
        offs, blob, cur = [], [], 0
        for p in parts:
            offs.append(cur)
            pad = (-len(p)) % 256
            blob.append(p)
            if pad:
                blob.append(np.zeros(pad, dtype=np.uint8))
            cur += len(p) + pad
        self.static = _upload(np.concatenate(blob), device)
        b = self.static.data_ptr()
        self.gemm_ptr = [b + offs[0] + ph * chunk.nmat * _lib.GEMM_DESC.itemsize for ph in range(_plan.N_PHASES)]
        self.sym_jobs_ptr = b + offs[1]
        self.full_jobs_ptr = b + offs[2]
        self.block_prefix_ptr = b + offs[3]
        self.tile_prefix_ptr = b + offs[4]
        self.syrk_jobs_ptr = b + offs[5]
        # counters of the split groups: zero now, and every launch that uses them leaves them zero
        self.split_counters = torch.zeros(max(chunk.split_slots, 1), dtype=torch.int32, device=device)
        self.split_partials_ptr = base + chunk.off_split_partials if chunk.split_slots else None
        self.split_counters_ptr = self.split_counters.data_ptr() if chunk.split_slots else None
        if chunk.aol:
            self.aol_ptr, self.aol_row_prefix_ptr, self.aol_seg_prefix_ptr = (b + o for o in offs[6:9])
            self.poly_full_jobs_ptr = b + offs[9] if chunk.poly_full_jobs is not None else None
        self.single_prefix_ptr = b + offs[-1]
        self.single_blocks = single[:, 1].tolist()
        self.mat_dev = None
        self.mat_key = None
        self.mat_host = None

    def bind(self, grads, momenta, params, outs, scales, src_dtypes):
        """(Re)upload the matrix descriptors if any tensor address changed since the last call."""
        key = (tuple(grads), tuple(momenta), tuple(params), tuple(outs), tuple(scales), tuple(src_dtypes))
        if key == self.mat_key:
            return
        lib = _lib.load()
        d = self.mat_template.copy()
        d["grad"] = grads
        d["momentum"] = momenta
        d["param"] = params
        d["out"] = outs
        d["scale"] = scales
        d["src_dtype"] = src_dtypes
        _lib.check(lib.muon_amd_validate_mats(_lib.host_ptr(d), self.chunk.nmat,
                                              _lib.host_ptr(self.chunk.block_prefix),
                                              _lib.host_ptr(self.chunk.tile_prefix), self.chunk.tile),
                   "validate_mats")
        if self.mat_dev is None:
            self.mat_dev = torch.empty(d.nbytes, dtype=torch.uint8, device=self.device)
        self.staging.upload(d, self.mat_dev)
        self.mat_key = key
        self.mat_host = d
        self.src_dtypes = list(src_dtypes)
        self.present = [(bool(m), bool(p), bool(o)) for m, p, o in zip(momenta, params, outs)]

    def rebind_row(self, k, grad, momentum):
        """Matrix k now has these gradient / momentum addresses: rewrite its descriptor in place
        (on the current stream) and remember the addresses, so that the next `bind` with the same
        ones uploads nothing."""
        lib = _lib.load()
        d = self.mat_host
        d["grad"][k] = grad
        d["momentum"][k] = momentum
        _lib.check(lib.muon_amd_validate_mats(_lib.host_ptr(d), self.chunk.nmat,
                                              _lib.host_ptr(self.chunk.block_prefix),
                                              _lib.host_ptr(self.chunk.tile_prefix), self.chunk.tile),
                   "validate_mats")
        sz = _lib.MAT_DESC.itemsize
        self.staging.upload(d[k:k + 1], self.mat_dev[k * sz:(k + 1) * sz])
        g, m, *rest = self.mat_key
        g, m = list(g), list(m)
        g[k], m[k] = grad, momentum
        self.mat_key = (tuple(g), tuple(m), *rest)

    def momentum_of(self, k, one_minus_beta, beta, nesterov, mutate_grad, scalars_ptr=0, stream=None):
        """The momentum launch over matrix k alone: on the current stream, or on `stream` (a raw
        handle of a stream of this device, which must be the current device)."""
        lib = _lib.load()

        def call():
            _lib.check(lib.muon_amd_momentum(
                self.mat_dev.data_ptr() + k * _lib.MAT_DESC.itemsize, self.single_prefix_ptr + 8 * k, 1,
                self.single_blocks[k], one_minus_beta, beta, int(nesterov), int(mutate_grad),
                scalars_ptr or None, stream if stream is not None else _stream_ptr(self.device)), "momentum")

        if stream is not None:          # per-launch events are recorded on the current stream only
            call()
            return
        lay = self.chunk.layouts[k]
        sz = 2 if self.src_dtypes[k] == _lib.SRC_BF16 else 4
        _launch("momentum", lay.numel * (sz + 2 + (2 * sz if self.present[k][0] else 0)), call)

    def run(self, one_minus_beta, beta, nesterov, mutate_grad, eps, lr, wd_factor, scalars_ptr=0,
            momentum_done=frozenset()):
        """Enqueue the chunk's launches.  scalars_ptr: device address of {one_minus_beta, beta, lr,
        wd_factor}, read by the kernels at run time in place of the by-value arguments.
        momentum_done: matrices (positions in the chunk) whose momentum stage already ran."""
        lib = _lib.load()
        c = self.chunk
        s = _stream_ptr(self.device)
        sc_mom = scalars_ptr or None
        sc_apply = scalars_ptr + 8 if scalars_ptr else None
        flags = _lib.ROUND_REFERENCE if c.reference_rounding else _lib.ROUND_FUSED
        mats = self.mat_dev.data_ptr()
        elts = sum(lay.numel for lay in c.layouts)
        padded = sum(lay.mp * lay.np_ for lay in c.layouts)
        # algorithmic bytes: gradient, momentum (read + write) and parameter (read + write) in
        # their storage type, the bf16 update written once and read once
        store = [2 if t == _lib.SRC_BF16 else 4 for t in self.src_dtypes]
        mom_bytes = sum(lay.numel * (sz + 2 + (2 * sz if has_m else 0))
                        for lay, sz, (has_m, _, _) in zip(c.layouts, store, self.present))
        apply_bytes = sum(lay.numel * (2 + (2 * sz if has_p else 0) + (2 if has_o else 0))
                          for lay, sz, (_, has_p, has_o) in zip(c.layouts, store, self.present))
        if c.split_slots:
            # every launch leaves the counters of the split groups zero; clearing them here as well
            # (a fill kernel, recordable into a graph) keeps a launch that died half way from
            # poisoning every later step
            self.split_counters.zero_()
        if not momentum_done:
            _launch("momentum", mom_bytes, lambda: _lib.check(lib.muon_amd_momentum(
                mats, self.block_prefix_ptr, c.nmat, c.nblocks, one_minus_beta, beta, int(nesterov),
                int(mutate_grad), sc_mom, s), "momentum"))
        else:
            for k in range(c.nmat):
                if k not in momentum_done:
                    self.momentum_of(k, one_minus_beta, beta, nesterov, mutate_grad, scalars_ptr)
        norm_flags = flags | (_lib.NORM_UNIT if c.aol else 0)
        _launch("norm_finalize", c.nblocks * 4, lambda: _lib.check(lib.muon_amd_norm_finalize(
            mats, c.nmat, eps, norm_flags, s), "norm_finalize"))
        _launch("normalize", elts * 2 + padded * 2, lambda: _lib.check(lib.muon_amd_normalize(
            mats, self.tile_prefix_ptr, c.nmat, c.ntiles, s), "normalize"))
        flops = {
            _plan.PH_SYRK: sum(lay.m * (lay.m + 1) * lay.n for lay in c.layouts),
            _plan.PH_POLY: sum(lay.m * lay.m * (lay.m + 1) for lay in c.layouts),
        }
        f_upd = sum(2 * lay.m * lay.m * lay.n for lay in c.layouts)

        def gemm(name, ph, it, jobs_ptr, njobs, work, extra_flags=0):
            al, be, ga = c.phase_scalars(ph, it)
            split = ph in (_plan.PH_SYRK, _plan.PH_SYRK_ODD)
            tile_class = c.update_class if jobs_ptr == self.full_jobs_ptr else c.tile_class
            _launch(name, work, lambda: _lib.check(lib.muon_amd_ns_gemm(
                self.gemm_ptr[ph], jobs_ptr, njobs, tile_class, al, be, ga, flags | extra_flags,
                self.split_partials_ptr if split else None, self.split_counters_ptr if split else None, s),
                "ns_gemm"))

        for it in range(c.steps):
            first_aol = c.aol and it == 0
            gemm("ns_gemm/syrk", _plan.PH_SYRK if it % 2 == 0 else _plan.PH_SYRK_ODD, it, self.syrk_jobs_ptr,
                 len(c.syrk_jobs), flops[_plan.PH_SYRK], _lib.GEMM_ROWSUM if first_aol else 0)
            if first_aol:
                # muon.py:776-785: the row sums of |A| come out of the product's epilogue as partial
                # sums (one small launch adds them up), then X and A are rescaled in place (A becomes
                # the Gram matrix of the rescaled X, so this iteration needs no second X X^T)
                gram_bytes = sum(lay.mp * lay.mp * 2 for lay in c.layouts)
                part_bytes = sum(lay.mp * (lay.mp // _plan.ROWSUM_SLOT) * 4 for lay in c.layouts)
                _launch("aol_rowsum_finalize", part_bytes, lambda: _lib.check(lib.muon_amd_aol_rowsum_finalize(
                    self.aol_ptr, self.aol_row_prefix_ptr, c.nmat, int(c.aol_row_prefix[-1]), eps, s),
                    "aol_rowsum_finalize"))
                mode = _lib.AOL_ROWS_ONLY if c.variant == "aol4_rows" else _lib.AOL_SYMMETRIC
                _launch("aol_rescale", 2 * gram_bytes + 4 * padded, lambda: _lib.check(lib.muon_amd_aol_rescale(
                    self.aol_ptr, self.aol_seg_prefix_ptr, c.nmat, int(c.aol_seg_prefix[-1]), mode, s),
                    "aol_rescale"))
            if first_aol and c.variant == "aol4_rows":
                # A / s is not symmetric: c * A A^T + b * A over every tile, no mirrored store
                gemm("ns_gemm/poly", _plan.PH_POLY_FULL, it, self.poly_full_jobs_ptr, len(c.poly_full_jobs),
                     2 * flops[_plan.PH_POLY])
            else:
                gemm("ns_gemm/poly", _plan.PH_POLY, it, self.sym_jobs_ptr, len(c.sym_jobs), flops[_plan.PH_POLY])
            if it == c.steps - 1:
                # the last update product takes the parameter step in its epilogue (muon.py:14, 98-99)
                al, be, _ = c.phase_scalars(_plan.PH_UPD_LAST, it)
                _launch("ns_gemm/update_apply", f_upd, lambda: _lib.check(lib.muon_amd_ns_gemm_apply(
                    self.gemm_ptr[_plan.PH_UPD_LAST], self.full_jobs_ptr, len(c.full_jobs), c.update_class, al, be,
                    flags, mats, lr, wd_factor, sc_apply, s), "ns_gemm_apply"))
                return
            gemm("ns_gemm/update", _plan.PH_UPD_EVEN if it % 2 == 0 else _plan.PH_UPD_ODD, it, self.full_jobs_ptr,
                 len(c.full_jobs), f_upd, _lib.GEMM_Q_KMAJOR)
        # no iteration (steps == 0): the parameter step is a launch of its own
        _launch("apply", apply_bytes, lambda: _lib.check(lib.muon_amd_apply(
            mats, self.block_prefix_ptr, c.nmat, c.nblocks, lr, wd_factor, sc_apply, s), "apply"))


class MuonGroupEngine:
    """Runs the Muon update of a fixed list of matrix shapes on one device.

    Built once per (shapes, steps, rounding).  A step is `prepare` (bind the current tensor
    addresses, take the hyper-parameters) followed by `enqueue` (the launches); `run` does both.
    `enqueue` either passes the hyper-parameters by value or, given the device address of a copy
    of `scalars()`, lets the kernels read them at run time -- which is what a caller does who
    records the launches into a HIP graph once and replays them with new values.
    """

    N_SCALARS = 4          # {1 - beta, beta, lr, 1 - lr * weight_decay}

    def __init__(self, shapes, device, steps: int = 5, reference_rounding: bool = True,
                 workspace_cap: int | None = None, variant: str = "ns5", allow_lanes: bool = True):
        self.device = torch.device(device)
        with torch.cuda.device(self.device):
            _lib.check(_lib.load().muon_amd_init(), "init")
        self.shapes = [(int(r), int(c)) for r, c in shapes]
        cap = DEFAULT_WORKSPACE_CAP if workspace_cap is None else int(workspace_cap)
        # Lanes: disjoint sets of matrices with a workspace and (beyond the first, which runs on the
        # caller's stream) a stream each; the chunks of a lane share its workspace and run back to back.
        lanes = _plan.plan_lanes(self.shapes, steps, reference_rounding, cap, variant, allow_lanes)
        self.chunks = [c for lane in lanes for c in lane]
        self.workspaces = [torch.empty(max(c.workspace_bytes for c in lane), dtype=torch.uint8, device=self.device)
                           for lane in lanes]
        self.workspace = self.workspaces[0]
        assert all(ws.data_ptr() % 256 == 0 for ws in self.workspaces)
        self.lane_runtimes = [[_ChunkRuntime(c, ws.data_ptr(), self.device) for c in lane]
                              for lane, ws in zip(lanes, self.workspaces)]
        self.runtimes = [rt for lane in self.lane_runtimes for rt in lane]
        self.lane_streams = [None] + [torch.cuda.Stream(self.device) for _ in lanes[1:]]      # default priority
        self._hyper = None
        # matrices whose momentum stage may run ahead of the step: those of the first chunk (the
        # later chunks reuse its workspace while the step runs); matrix index -> position in the chunk
        self._early_pos = {lay.index: k for k, lay in enumerate(self.chunks[0].layouts)}
        self._early_stream = None
        self._early_events = {}
        self._early_done = {}         # position -> (gradient address, caller's token) the stage consumed
        self._skip = frozenset()

    def prepare(self, grads, momenta, params, outs, scales, src_dtypes, *, beta, nesterov, mutate_grad,
                eps, lr, weight_decay):
        """All list arguments are per matrix in the order of `shapes` (device addresses or 0)."""
        if self._early_done:
            # the stages enqueued by early_momentum since the last step: order them before what
            # follows on this stream, and insist that they consumed the gradients of this step
            torch.cuda.current_stream(self.device).wait_stream(self._early_stream)
            layouts = self.chunks[0].layouts
            done, self._early_done = self._early_done, {}
            for k, (used, _) in done.items():
                if grads[layouts[k].index] != used:
                    raise _lib.MuonAmdError(
                        f"the gradient of matrix {layouts[k].index} was replaced after its momentum stage ran "
                        "during backward (overlap with backward needs the gradient tensors left alone "
                        "between backward and step)")
            self._skip = frozenset(done)
        else:
            self._skip = frozenset()
        for rt in self.runtimes:
            idx = [lay.index for lay in rt.chunk.layouts]
            rt.bind([grads[i] for i in idx], [momenta[i] for i in idx], [params[i] for i in idx],
                    [outs[i] for i in idx], [scales[i] for i in idx], [src_dtypes[i] for i in idx])
        # 1 - beta and 1 - lr * weight_decay are python doubles, as in muon.py:9 and muon.py:98
        self._hyper = dict(one_minus_beta=1 - beta, beta=beta, nesterov=bool(nesterov),
                           mutate_grad=bool(mutate_grad), eps=float(eps), lr=lr, wd_factor=1 - lr * weight_decay)

    def scalars(self):
        h = self._hyper
        return [h["one_minus_beta"], h["beta"], h["lr"], h["wd_factor"]]

    def structure_key(self):
        """What a recorded sequence of launches depends on besides device memory."""
        h = self._hyper
        return (id(self), h["nesterov"], h["mutate_grad"], h["eps"], self._skip)

    def enqueue(self, scalars_ptr: int = 0, join: bool = True):
        """The launches of every lane: the first lane on the current stream, the others on their own
        streams, which wait for what the current stream holds so far (the descriptor uploads of
        `prepare`, the gradients) and which the current stream waits for before it goes on -- here,
        or (join=False) when the caller calls `join`, having enqueued work that does not depend on
        these matrices in between (the Adam launch of the same step)."""
        h = self._hyper
        main = torch.cuda.current_stream(self.device)
        for side in self.lane_streams[1:]:
            side.wait_stream(main)
        for li, runtimes in enumerate(self.lane_runtimes):
            with (torch.cuda.stream(self.lane_streams[li]) if li else contextlib.nullcontext()):
                for n, rt in enumerate(runtimes):
                    rt.run(h["one_minus_beta"], h["beta"], h["nesterov"], h["mutate_grad"], h["eps"], h["lr"],
                           h["wd_factor"], scalars_ptr=scalars_ptr,
                           momentum_done=self._skip if (li == 0 and n == 0) else frozenset())
        if join:
            self.join()

    def join(self):
        """The current stream waits for the lanes that run on streams of their own."""
        main = torch.cuda.current_stream(self.device)
        for side in self.lane_streams[1:]:
            main.wait_stream(side)

    def early_stream(self):
        """The side stream the early stages run on (default priority; created on first use)."""
        if self._early_stream is None:
            self._early_stream = torch.cuda.Stream(self.device)
        return self._early_stream

    def early_eligible(self, i) -> bool:
        """Whether `early_momentum` would act on matrix `i`: it is in the first chunk and a step has run."""
        return i in self._early_pos and self.runtimes[0].mat_key is not None

    def early_pending(self, i):
        """(gradient address, token) the pending early stage of matrix `i` consumed, or None."""
        k = self._early_pos.get(i)
        return None if k is None else self._early_done.get(k)

    def early_discard(self, i) -> None:
        """Forget the pending early stage of matrix `i`: the next step runs its momentum stage itself.
        The caller has put the momentum buffer back to what it was before that stage."""
        k = self._early_pos.get(i)
        if k is not None:
            self._early_done.pop(k, None)

    def early_momentum(self, i, grad, momentum, *, beta, nesterov, mutate_grad, token=None, redo=False) -> bool:
        """Run the first stage of matrix `i` (position in `shapes`) -- momentum, Nesterov blend,
        bf16 cast, sums of squares -- now, on a side stream that first waits for everything enqueued
        so far on the current stream (the work that produced the gradient), instead of inside the
        step.  The next `prepare` joins the side stream, and that step's `enqueue` leaves the matrix
        out of its momentum launch.  Meant to be called from a hook that fires during backward once
        the gradient at address `grad` is complete; `token` is kept beside the address for the
        caller (`early_pending`).  A second stage for a matrix before a step raises unless `redo`
        says that the caller has put the momentum buffer back (on the side stream) to what it was
        before the first one.  Returns False, having done nothing, for a matrix outside the first
        chunk or an engine that has not run a step yet."""
        k = self._early_pos.get(i)
        rt = self.runtimes[0]
        if k is None or rt.mat_key is None:
            return False
        if k in self._early_done and not redo:
            raise _lib.MuonAmdError(
                f"matrix {i}: a second gradient arrived before step() (the momentum buffer has already "
                "taken the first one; restore it and pass redo=True)")
        side = self.early_stream()
        ev = self._early_events.get(k)
        if ev is None:
            ev = self._early_events[k] = torch.cuda.Event()
        ev.record(torch.cuda.current_stream(self.device))
        side.wait_event(ev)
        moved = rt.mat_key[0][k] != grad or rt.mat_key[1][k] != momentum
        if moved or torch.cuda.current_device() != self.device.index:
            with torch.cuda.stream(side):
                if moved:
                    rt.rebind_row(k, grad, momentum)
                rt.momentum_of(k, 1 - beta, beta, nesterov, mutate_grad)
        else:       # the common case, kept cheap: this runs once per matrix inside backward
            rt.momentum_of(k, 1 - beta, beta, nesterov, mutate_grad, stream=side.cuda_stream)
        self._early_done[k] = (grad, token)
        return True

    def run(self, grads, momenta, params, outs, scales, src_dtypes, **hyper):
        self.prepare(grads, momenta, params, outs, scales, src_dtypes, **hyper)
        self.enqueue()


class AdamGroupEngine:
    """Fused auxiliary-Adam launch over a fixed list of tensors (prepare / enqueue as above)."""

    N_SCALARS = 7          # {lr, 1 - lr * weight_decay, 1 - beta1, 1 - beta2, eps, 1 - beta1**t, 1 - beta2**t}

    def __init__(self, numels, device):
        _lib.load()
        self.device = torch.device(device)
        self.numels = [int(n) for n in numels]
        self.prefix = _plan.adam_block_prefix(self.numels)
        self.nblocks = int(self.prefix[-1])
        self.prefix_dev = _upload(self.prefix, self.device)
        # one buffer for the descriptors, rewritten in place: recorded launches keep its address
        self.desc_dev = torch.empty(len(self.numels) * _lib.ADAM_DESC.itemsize, dtype=torch.uint8, device=self.device)
        self.staging = _Staging(self.device)
        self.key = None
        self._hyper = None

    def prepare(self, params, grads, exp_avgs, exp_avg_sqs, updates, *, lr, weight_decay, betas, eps, step,
                dtypes=None):
        dtypes = [_lib.SRC_F32] * len(self.numels) if dtypes is None else list(dtypes)
        key = (tuple(params), tuple(grads), tuple(exp_avgs), tuple(exp_avg_sqs), tuple(updates), tuple(dtypes))
        if key != self.key:
            d = np.zeros(len(self.numels), dtype=_lib.ADAM_DESC)
            d["param"] = params
            d["grad"] = grads
            d["exp_avg"] = exp_avgs
            d["exp_avg_sq"] = exp_avg_sqs
            d["update"] = updates
            d["numel"] = self.numels
            d["dtype"] = dtypes
            self.staging.upload(d, self.desc_dev)
            self.key = key
            self.nbytes = sum(n * (14 if t == _lib.SRC_BF16 else 28) for n, t in zip(self.numels, dtypes))
        # python doubles, as muon.py:105-108 and 257
        self._hyper = [lr, 1 - lr * weight_decay, 1 - betas[0], 1 - betas[1], eps,
                       1 - betas[0] ** step, 1 - betas[1] ** step]

    def scalars(self):
        return list(self._hyper)

    def structure_key(self):
        return (id(self),)

    def join(self):
        pass

    def enqueue(self, scalars_ptr: int = 0, join: bool = True):
        lib = _lib.load()
        lr, wd_factor, w1, w2, eps, bias1, bias2 = self._hyper
        _launch("adam", self.nbytes, lambda: _lib.check(lib.muon_amd_adam(
            self.desc_dev.data_ptr(), self.prefix_dev.data_ptr(), len(self.numels), self.nblocks, lr,
            wd_factor, w1, w2, eps, bias1, bias2, scalars_ptr or None, _stream_ptr(self.device)), "adam"))

    def run(self, params, grads, exp_avgs, exp_avg_sqs, updates, **hyper):
        self.prepare(params, grads, exp_avgs, exp_avg_sqs, updates, **hyper)
        self.enqueue()


class StepGraph:
    """A whole optimizer step on one device as one HIP graph: the launches of every engine of the
    step are recorded once and replayed afterwards.  What changes between steps is read by the
    recorded kernels from device memory: tensor addresses from the descriptor tables (rewritten in
    place by the engines' `prepare` when a tensor moved) and the hyper-parameters (learning rates,
    decay factors, Adam's bias corrections) from one block of scalars that a small asynchronous
    copy refreshes ahead of every replay.  No memset node is recorded."""

    def __init__(self, device):
        self.device = torch.device(device)
        self.graph = None
        self.key = None
        self.scalars = None
        self.staging = _Staging(self.device)
        self.replays = 0

    def run(self, engines):
        """`engines`: prepared engines in launch order."""
        offsets, host = [], []
        for e in engines:
            offsets.append(len(host))
            vals = e.scalars()
            host += vals + [0.0] * ((-len(vals)) % 4)          # every block 16-byte aligned
        if self.scalars is None or self.scalars.numel() < len(host):
            self.scalars = torch.zeros(max(len(host), 16), dtype=torch.float32, device=self.device)
            self.graph = None                                    # recorded launches hold the old address
        self.staging.upload(np.asarray(host, dtype=np.float32), self.scalars.view(torch.uint8)[: 4 * len(host)])
        key = tuple(e.structure_key() for e in engines)
        if self.graph is None or key != self.key:
            graph = torch.cuda.CUDAGraph()
            base = self.scalars.data_ptr()
            with torch.cuda.graph(graph):
                try:
                    for e, off in zip(engines, offsets):
                        e.enqueue(base + 4 * off, join=False)
                finally:
                    for e in engines:
                        e.join()
            self.graph, self.key = graph, key
        self.graph.replay()
        self.replays += 1
