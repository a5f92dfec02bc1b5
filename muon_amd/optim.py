"""Optimizer classes with the reference's names, constructor signatures, defaults, state keys and
assertions (reference muon.py:18-70, 73-101, 112-199, 202-260), single-GPU semantics.

Each `step()` issues, per Muon parameter group, a handful of grouped launches over all matrices
of the group (momentum -> norm -> normalise -> 15 Newton-Schulz GEMM launches, the last of which
applies the update to the parameters) and one fused launch per Adam group; nothing in it
synchronises with the host.
"""
from __future__ import annotations

import weakref

import torch

from . import engine as _engine
from .engine import AdamGroupEngine, MuonGroupEngine, StepGraph, require_gpu_tensor
from .functional import _rounding_flag, _src_dtype

NS_STEPS = 5          # the reference classes never pass a step count: muon_update's default rules
NESTEROV = True       # likewise (muon.py:8)


def _world_size() -> int:
    import torch.distributed as dist
    return dist.get_world_size() if dist.is_available() and dist.is_initialized() else 1


class _MuonBase(torch.optim.Optimizer):
    """Shared machinery: engine caches and the two per-group update paths."""

    def _init_runtime(self, ns_rounding, mutate_grad, workspace_bytes, ns_variant="ns5", use_graph=False,
                      overlap_backward=False):
        self._use_graph = bool(use_graph)
        self._overlap_backward = bool(overlap_backward)
        self._early_params = {}       # Muon parameter -> (engine, first matrix, matrices, group index), set by each step
        self._early_shadow = {}       # Muon parameter -> copy of its momentum buffer from before a pending early stage
        self._install_overlap_hooks()
        if ns_variant not in ("ns5", "aol4", "aol4_rows"):
            raise ValueError(f"ns_variant must be 'ns5', 'aol4' or 'aol4_rows', got {ns_variant!r}")
        self._ns_variant = ns_variant
        self._ns_rounding = ns_rounding
        self._reference_rounding = _rounding_flag(ns_rounding)
        self._mutate_grad = bool(mutate_grad)
        self._workspace_bytes = workspace_bytes
        self._muon_engines = {}
        self._adam_engines = {}
        self._graphs = {}             # device -> StepGraph (use_graph=True)
        self._pending = []            # engines prepared by the group loop of the current step, in launch order
        self._writebacks = []         # (destination, contiguous copy) pairs to copy back after the launches
        self._keepalive = []          # temporaries whose addresses the pending launches use
        self._step_bumps = []         # (Adam state, new step count) written when the launches go out

    _RUNTIME_OPTIONS = ("_ns_rounding", "_mutate_grad", "_workspace_bytes", "_ns_variant", "_use_graph",
                        "_overlap_backward")

    # ---- overlap with backward: the first Muon stage of a matrix runs when its gradient is ready ----
    def _install_overlap_hooks(self):
        for h in getattr(self, "_hook_handles", []):
            h.remove()
        self._hook_handles = []
        self._hooked = set()
        if self._overlap_backward:
            for group in self.param_groups:
                self._hook_group(group)

    def _hook_group(self, group):
        if not group.get("use_muon", True):
            return
        ref = weakref.ref(self)           # the parameters must not keep the optimizer alive

        def grad_ready(p):
            opt = ref()
            if opt is not None:
                opt._grad_ready(p)

        for p in group["params"]:
            if isinstance(p, torch.Tensor) and p.requires_grad and p.is_leaf and id(p) not in self._hooked:
                self._hook_handles.append(p.register_post_accumulate_grad_hook(grad_ready))
                self._hooked.add(id(p))

    def add_param_group(self, param_group):
        super().add_param_group(param_group)
        if getattr(self, "_overlap_backward", False):
            self._hook_group(self.param_groups[-1])

    @torch.no_grad()
    def _grad_ready(self, p):
        """Autograd has finished accumulating p.grad (post-accumulate-grad hook).  Once a step has
        built the group's engine, enqueue the momentum stage of the parameter's matrices on the
        engine's side stream; step() then skips it.  The momentum buffer is copied aside first, so
        that the stage can be taken back: when a second gradient arrives before step() (gradients
        accumulated over micro-batches, or a step that was skipped) the buffer is restored and the
        stage runs again on the gradient as it is now, and step() takes the stage back when the
        gradient was touched after it ran (`_early_settle`).  Anything out of the ordinary (no
        engine yet, strided tensors, a gradient of another dtype, mutate_grad) is left to step()."""
        info = self._early_params.get(p)
        if info is None or self._mutate_grad:     # a stage that overwrote the gradient could not run again
            return
        eng, first, count, gi = info
        if gi >= len(self.param_groups):
            return
        group = self.param_groups[gi]             # looked up now: load_state_dict replaces the group dicts
        g, m = p.grad, self.state[p].get("momentum_buffer")
        if (g is None or m is None or g.is_sparse or g.dtype != p.dtype or m.dtype != p.dtype or
                m.shape != p.shape or g.device != p.device or m.device != p.device or
                not (g.is_contiguous() and m.is_contiguous() and p.is_contiguous())):
            return
        if not all(eng.early_eligible(first + k) for k in range(count)):
            return
        pending = eng.early_pending(first)
        if pending is not None and pending[1][2] != m.data_ptr():
            for k in range(count):                # the state tensor was replaced since: nothing to take back
                eng.early_discard(first + k)
            pending = None
        shadow = self._early_shadow.get(p)
        if pending is None and (shadow is None or shadow.shape != m.shape or shadow.dtype != m.dtype or
                                shadow.device != m.device):
            shadow = self._early_shadow[p] = torch.empty_like(m)
        side = eng.early_stream()
        side.wait_stream(torch.cuda.current_stream(p.device))
        with torch.cuda.stream(side):
            if pending is not None:
                m.copy_(shadow)                   # the buffer as it was before the stage that is discarded
            else:
                shadow.copy_(m)
        stride = (p.numel() // count) * p.element_size()
        # The gradient tensor itself is part of the token: holding it keeps its memory from being
        # handed out again while the side stream reads it, and lets step() tell this tensor from a
        # new one that the allocator put at the same address.
        token = (g, g._version, m.data_ptr())
        for k in range(count):
            eng.early_momentum(first + k, g.data_ptr() + k * stride, m.data_ptr() + k * stride,
                               beta=float(group["momentum"]), nesterov=NESTEROV, mutate_grad=False,
                               token=token, redo=pending is not None)

    def _early_settle(self, p, eng, first, g, m, plain):
        """step() is about to use parameter p as matrices first.. of engine `eng` (None: another
        engine).  A pending early stage stands if it consumed exactly this gradient (the same tensor
        object, not written since: torch counts in-place writes in `_version`) into this momentum
        buffer; otherwise it is taken back: the buffer is restored from the copy made before the
        stage, and the step runs the stage itself."""
        info = self._early_params.get(p)
        if info is None:
            return
        old_eng, old_first, count, _ = info
        pending = old_eng.early_pending(old_first)
        if pending is None:
            return
        addr, (staged_grad, version, m_addr) = pending
        if (plain and old_eng is eng and old_first == first and g is staged_grad and g.data_ptr() == addr and
                g._version == version and m.data_ptr() == m_addr):
            return
        if m.data_ptr() == m_addr:
            torch.cuda.current_stream(p.device).wait_stream(old_eng.early_stream())
            m.copy_(self._early_shadow[p])
        for k in range(count):
            old_eng.early_discard(old_first + k)

    def __getstate__(self):
        # torch's Optimizer pickles defaults/state/param_groups only; the keyword-only options of
        # this build select the algorithm (ns_variant, ns_rounding), so a copy must carry them.
        # Engines (device workspaces, raw addresses, recorded graphs) are rebuilt on the next step.
        state = super().__getstate__()
        state["muon_amd_options"] = {k: getattr(self, k) for k in self._RUNTIME_OPTIONS}
        return state

    def __setstate__(self, state):
        state = dict(state)
        opts = state.pop("muon_amd_options", None)
        super().__setstate__(state)
        if opts is not None:
            self._init_runtime(opts["_ns_rounding"], opts["_mutate_grad"], opts["_workspace_bytes"],
                               opts["_ns_variant"], opts["_use_graph"], opts.get("_overlap_backward", False))
        elif not hasattr(self, "_muon_engines"):
            self._init_runtime("reference", False, None)

    @staticmethod
    def _check_param(p):
        require_gpu_tensor(p, "parameter")
        if p.dtype not in (torch.float32, torch.bfloat16):
            raise NotImplementedError(f"muon_amd updates fp32 and bf16 parameters; got {p.dtype}")

    @staticmethod
    def _grad_of(p):
        if p.grad is None:
            p.grad = torch.zeros_like(p)          # muon.py:91-93 "Force synchronization"
        g = p.grad
        if g.dtype != p.dtype or g.is_sparse:
            raise NotImplementedError("muon_amd needs dense gradients of the parameter's dtype")
        return g

    @staticmethod
    def _dense(t, writebacks, written=True):
        """The kernels address row-major memory.  A tensor with other strides (a transposed view
        used as a parameter, say) goes through a contiguous copy that is copied back after the
        launches; the reference takes any strides because torch does (muon.py:9-10, 98-99)."""
        if t.is_contiguous():
            return t
        c = t.contiguous()
        if written:
            writebacks.append((t, c))
        return c

    @staticmethod
    def _state_tensor(state, key, p):
        t = state[key]
        if t.dtype != p.dtype or t.device != p.device or t.shape != p.shape:
            raise NotImplementedError(f"{key} must be a tensor of the parameter's dtype and shape on its device")
        return t

    def _muon_group_step(self, gi, group):
        params = [p for p in group["params"] if p.numel() > 0]
        if not params:
            return
        grads, moms, ptrs, shapes, scales, dtypes, writebacks, keep = [], [], [], [], [], [], [], []
        spans = []                                # (parameter, first matrix, matrices) of plain row-major parameters
        for p in params:
            self._check_param(p)
            assert p.ndim >= 2                    # muon.py:275 (reached through muon.py:13)
            g = self._grad_of(p)
            state = self.state[p]
            if len(state) == 0:                   # muon.py:95-96
                state["momentum_buffer"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
            m = self._dense(self._state_tensor(state, "momentum_buffer", p), writebacks)
            g = self._dense(g, writebacks, written=self._mutate_grad)
            pc = self._dense(p, writebacks)
            keep.append((g, m, pc))               # copies stay allocated until the launches are enqueued
            if p.ndim == 4:                       # muon.py:11-12: conv filters are flattened
                batch, rows, cols = 1, p.size(0), p.numel() // p.size(0)
            else:                                 # muon.py:275, 282: leading dims are a batch
                rows, cols = p.shape[-2:]
                batch = p.numel() // (rows * cols)
            scale = max(1, p.size(-2) / p.size(-1)) ** 0.5             # muon.py:14
            if g is p.grad and pc is p and m is state["momentum_buffer"]:
                spans.append((p, len(shapes), batch))
            for k in range(batch):
                off = k * rows * cols * p.element_size()
                shapes.append((rows, cols))
                scales.append(scale)
                dtypes.append(_src_dtype(p))
                grads.append(g.data_ptr() + off)
                moms.append(m.data_ptr() + off)
                ptrs.append(pc.data_ptr() + off)
        device = params[0].device
        key = (gi, device, tuple(shapes))
        eng = self._muon_engines.get(key)
        if eng is None:
            self._muon_engines = {k: v for k, v in self._muon_engines.items() if k[0] != gi}
            with torch.cuda.device(device):
                # (the stages that run during backward write into the first chunk's workspace: one lane)
                eng = MuonGroupEngine(shapes, device, NS_STEPS, self._reference_rounding, self._workspace_bytes,
                                      variant=self._ns_variant, allow_lanes=not self._overlap_backward)
            self._muon_engines[key] = eng
            self._graphs.pop(device, None)        # a recorded step refers to the engine that was replaced
        if self._overlap_backward:
            plain = {id(p): first for p, first, _ in spans}
            for p in params:
                self._early_settle(p, eng, plain.get(id(p)), p.grad, self.state[p]["momentum_buffer"], id(p) in plain)
        n = len(shapes)
        # float(): schedulers and checkpoints may leave 0-dim tensors in the group (the reference's
        # tensor arithmetic takes them as they are)
        eng.prepare(grads, moms, ptrs, [0] * n, scales, dtypes,
                    beta=float(group["momentum"]), nesterov=NESTEROV, mutate_grad=self._mutate_grad,
                    eps=1e-7, lr=float(group["lr"]), weight_decay=float(group["weight_decay"]))
        self._pending.append(eng)
        self._writebacks += writebacks
        self._keepalive.append(keep)
        if self._overlap_backward:
            for p in params:
                self._early_params.pop(p, None)
            for p, first, count in spans:
                self._early_params[p] = (eng, first, count, gi)

    def _adam_group_step(self, gi, group):
        by_step, writebacks = {}, []
        for p in group["params"]:
            self._check_param(p)
            g = self._grad_of(p)
            state = self.state[p]
            if len(state) == 0:                   # muon.py:250-253
                state["exp_avg"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                state["step"] = 0
            # muon.py:254 increments before the update; the new count is written to the state when the
            # launches go out (_launch_pending), so that a step that raises while a later group is
            # prepared leaves every counter where it was
            step_now = int(state["step"]) + 1
            self._step_bumps.append((state, step_now))
            if p.numel() > 0:
                item = (self._dense(p, writebacks), self._dense(g, writebacks, written=False),
                        self._dense(self._state_tensor(state, "exp_avg", p), writebacks),
                        self._dense(self._state_tensor(state, "exp_avg_sq", p), writebacks))
                by_step.setdefault(step_now, []).append((p, item))
        for step, items in by_step.items():
            device = items[0][0].device
            key = (gi, device, tuple(id(p) for p, _ in items))
            eng = self._adam_engines.get(key)
            if eng is None:
                eng = AdamGroupEngine([p.numel() for p, _ in items], device)
                self._adam_engines[key] = eng
            eng.prepare([t[0].data_ptr() for _, t in items], [t[1].data_ptr() for _, t in items],
                        [t[2].data_ptr() for _, t in items], [t[3].data_ptr() for _, t in items],
                        [0] * len(items),
                        lr=float(group["lr"]), weight_decay=float(group["weight_decay"]),
                        betas=(float(group["betas"][0]), float(group["betas"][1])),
                        eps=float(group["eps"]), step=step, dtypes=[_src_dtype(p) for p, _ in items])
            self._pending.append(eng)
            self._keepalive.append(items)
        self._writebacks += writebacks

    def _launch_pending(self):
        """Enqueue what the group loop prepared: eagerly, or (use_graph=True) as one recorded graph
        per device that is replayed every step; then copy back tensors that went through a
        contiguous copy (stream ordered after the launches)."""
        try:
            for state, step_now in self._step_bumps:
                state["step"] = step_now
            by_device = {}
            for eng in self._pending:
                by_device.setdefault(eng.device, []).append(eng)
            for device, engines in by_device.items():
                with torch.cuda.device(device):
                    if self._use_graph and _engine.PROFILE is None:
                        graph = self._graphs.get(device)
                        if graph is None:
                            graph = self._graphs[device] = StepGraph(device)
                        graph.run(engines)
                    else:
                        # lanes on streams of their own are joined after everything is enqueued: the
                        # Adam launch does not wait for the last Muon launch of another lane
                        try:
                            for eng in engines:
                                eng.enqueue(join=False)
                        finally:                  # also when a launch was refused: nothing stays unjoined
                            for eng in engines:
                                eng.join()
            for dst, src in self._writebacks:
                dst.copy_(src)
        finally:
            self._pending, self._writebacks, self._keepalive, self._step_bumps = [], [], [], []

    def _run_closure(self, closure):
        # nothing left over from a step that raised
        self._pending, self._writebacks, self._keepalive, self._step_bumps = [], [], [], []
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        return loss


class SingleDeviceMuon(_MuonBase):
    """Muon for one device (reference muon.py:73-101).

    Keyword-only extras (not in the reference): ns_rounding ("reference" | "fused"),
    mutate_grad (write the Nesterov blend back into p.grad as the reference's in-place lerp does;
    off by default because nothing reads it), workspace_bytes (cap of the bf16 workspace),
    ns_variant ("ns5": the five-iteration specification muon.py:265-291; "aol4": the
    four-iteration AOL-rescaled variant muon.py:748-799 with the Gram matrix rescaled on both
    sides, "aol4_rows": the same with `A / s` by rows only as muon.py:785 is written; see
    zeropower_via_aol4), use_graph
    (record every launch of a step -- all Muon groups and all Adam groups on a device -- into one
    HIP graph once and replay it every step; tensor addresses and hyper-parameters are read from
    device memory, so gradients may be reallocated and learning rates scheduled between steps),
    overlap_backward (post-accumulate-grad hooks on the Muon parameters run a matrix's first stage
    -- momentum, Nesterov blend, bf16 cast, sums of squares -- on a side stream as soon as backward
    has produced its gradient, and step() skips it; from the second step on, for the matrices of
    the first workspace chunk.  The stage can be taken back: the momentum buffer is copied aside
    before it runs, a second gradient before step() -- accumulation over micro-batches, or a step
    that was skipped, as a loss scaler does after an overflow -- restores the buffer and runs the
    stage again on the gradient as it then is, and step() restores the buffer and runs the stage
    itself when the gradient was written after the stage (in-place clipping or unscaling: torch's
    version counter of the gradient tensor tells) or replaced.  What remains: between backward and
    step() the momentum buffer of a staged parameter holds the not-yet-committed value, and
    mutate_grad=True switches the early stage off).  Hyper-parameters kept as 0-dim tensors on the
    GPU are read with float(), which waits for the device once per step and group.
    """

    def __init__(self, params, lr=0.02, weight_decay=0, momentum=0.95, *, ns_rounding="reference",
                 mutate_grad=False, workspace_bytes=None, ns_variant="ns5", use_graph=False,
                 overlap_backward=False):
        defaults = dict(lr=lr, weight_decay=weight_decay, momentum=momentum)
        super().__init__(params, defaults)
        self._init_runtime(ns_rounding, mutate_grad, workspace_bytes, ns_variant, use_graph, overlap_backward)

    @torch.no_grad()
    def step(self, closure=None):
        loss = self._run_closure(closure)
        for gi, group in enumerate(self.param_groups):
            self._muon_group_step(gi, group)
        self._launch_pending()
        return loss


class Muon(SingleDeviceMuon):
    """Reference muon.py:18-70 on one GPU: asserts a non-empty list of Parameters and sorts it by
    size (descending) as the reference does; the cross-rank update sharding is not part of this
    library, so a process group with more than one rank is refused."""

    def __init__(self, params, lr=0.02, weight_decay=0, momentum=0.95, **extras):
        assert isinstance(params, list) and len(params) >= 1 and isinstance(params[0], torch.nn.Parameter)
        params = sorted(params, key=lambda x: x.size(), reverse=True)      # muon.py:42
        super().__init__(params, lr=lr, weight_decay=weight_decay, momentum=momentum, **extras)

    @torch.no_grad()
    def step(self, closure=None):
        if _world_size() > 1:
            raise NotImplementedError("muon_amd.Muon runs on one GPU; sharded updates across ranks are not provided")
        return super().step(closure)


def _fill_aux_adam_groups(param_groups, sort_muon: bool):
    for group in param_groups:
        assert "use_muon" in group
        if group["use_muon"]:
            if sort_muon:
                group["params"] = sorted(group["params"], key=lambda x: x.size(), reverse=True)  # muon.py:143
            group["lr"] = group.get("lr", 0.02)
            group["momentum"] = group.get("momentum", 0.95)
            group["weight_decay"] = group.get("weight_decay", 0)
            assert set(group.keys()) == set(["params", "lr", "momentum", "weight_decay", "use_muon"])
        else:
            group["lr"] = group.get("lr", 3e-4)
            group["betas"] = group.get("betas", (0.9, 0.95))
            group["eps"] = group.get("eps", 1e-10)
            group["weight_decay"] = group.get("weight_decay", 0)
            assert set(group.keys()) == set(["params", "lr", "betas", "eps", "weight_decay", "use_muon"])


class SingleDeviceMuonWithAuxAdam(_MuonBase):
    """Reference muon.py:202-260: Muon for `use_muon=True` groups, Adam for the others."""

    _SORT_MUON = False

    def __init__(self, param_groups, *, ns_rounding="reference", mutate_grad=False, workspace_bytes=None,
                 ns_variant="ns5", use_graph=False, overlap_backward=False):
        _fill_aux_adam_groups(param_groups, self._SORT_MUON)
        super().__init__(param_groups, dict())
        self._init_runtime(ns_rounding, mutate_grad, workspace_bytes, ns_variant, use_graph, overlap_backward)

    @torch.no_grad()
    def step(self, closure=None):
        loss = self._run_closure(closure)
        for gi, group in enumerate(self.param_groups):
            if group["use_muon"]:
                self._muon_group_step(gi, group)
            else:
                self._adam_group_step(gi, group)
        self._launch_pending()
        return loss


class MuonWithAuxAdam(SingleDeviceMuonWithAuxAdam):
    """Reference muon.py:112-199 on one GPU (Muon groups sorted by size as the reference does)."""

    _SORT_MUON = True

    @torch.no_grad()
    def step(self, closure=None):
        if _world_size() > 1:
            raise NotImplementedError("muon_amd.MuonWithAuxAdam runs on one GPU; sharded updates across ranks are not provided")
        return super().step(closure)
