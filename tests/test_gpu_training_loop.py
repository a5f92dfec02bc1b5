"""What a training loop does around the optimizer, on the GPU, with gradients that a real autograd
backward produces.

overlap_backward=True: post-accumulate-grad hooks run a matrix's first Muon stage (muon.py:9-10 and
the cast of muon.py:277) on a side stream while autograd is still producing the other gradients,
and step() skips that stage for those matrices.  The result must be the bits of the plain step,
the step itself must match the oracle, and a gradient that changes after its early stage ran
(accumulation, clipping, replacement, a skipped step) must give the plain optimizer's bits too.

Also: 0-dim tensors as hyper-parameters, steps issued on side streams, and a scheduler, gradient
clipping and a gradient scaler wrapped around the optimizer.
"""
import pytest
import torch

from oracle import muon_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def M():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need an MI355X; torch.cuda.is_available() is False")
    import muon_amd
    from muon_amd import _lib
    _lib.load()
    return muon_amd


SHAPES = [(768, 768), (256, 640), (640, 256), (3, 128, 192), (16, 8, 3, 3), (130, 300)]


def _params(seed, device="cuda"):
    torch.manual_seed(seed)
    return [torch.nn.Parameter((torch.randn(*s) * 0.02).to(device)) for s in SHAPES]


def _inputs(params, seed):
    """Per parameter a layer input x and an output gradient dy: the loss below makes autograd produce
    every weight gradient as the matrix product x^T . dy of a linear layer's backward (full rank:
    512 rows)."""
    gen = torch.Generator().manual_seed(seed)
    out = []
    for p in params:
        rows, cols = (p.shape[0], p.numel() // p.shape[0]) if p.ndim == 4 else p.shape[-2:]
        lead = tuple(p.shape[:-2]) if p.ndim == 3 else ()
        out.append((torch.randn(*lead, 512, rows, generator=gen) * 1e-2, torch.randn(*lead, 512, cols, generator=gen) * 1e-2))
    return out


def _loss(params, xs):
    total = 0.0
    for p, (x, dy) in zip(params, xs):
        w = p.reshape(p.shape[0], -1) if p.ndim == 4 else p
        total = total + ((x.to(p.device) @ w) * dy.to(p.device)).sum()
    return total


def _make(M, params, gain, **kw):
    return M.SingleDeviceMuonWithAuxAdam(
        [dict(params=params, use_muon=True, lr=0.02, weight_decay=0.01),
         dict(params=[gain], use_muon=False, lr=3e-4, weight_decay=0.0)], **kw)


@pytest.mark.parametrize("use_graph,cap", [(False, None), (True, None), (False, 3 << 20)])
def test_overlap_with_backward_equals_the_plain_step(M, use_graph, cap):
    pa, pb = _params(77), _params(77)
    ga, gb = (torch.nn.Parameter(torch.ones(40, device="cuda")) for _ in range(2))
    plain = _make(M, pa, ga, workspace_bytes=cap)
    early = _make(M, pb, gb, workspace_bytes=cap, use_graph=use_graph, overlap_backward=True)
    skipped = []
    for step in range(5):
        xs = _inputs(pa, 100 + step)
        if step == 3:        # the hooks read the group's momentum when they fire: change it before backward
            plain.param_groups[0]["momentum"] = early.param_groups[0]["momentum"] = 0.9
        for opt, params, gain in ((plain, pa, ga), (early, pb, gb)):
            opt.zero_grad(set_to_none=(step % 2 == 0))      # reallocated and reused gradient tensors
            (_loss(params, xs) + (gain * gain).sum()).backward()
        plain.step()
        early.step()
        eng = next(iter(early._muon_engines.values()))
        skipped.append(len(eng._skip))
        torch.cuda.synchronize()
        for a, b in zip(pa + [ga], pb + [gb]):
            assert torch.equal(a.detach(), b.detach()), (step, tuple(a.shape))
        for a, b in zip(pa, pb):
            assert torch.equal(plain.state[a]["momentum_buffer"], early.state[b]["momentum_buffer"]), (step, tuple(a.shape))
    eng = next(iter(early._muon_engines.values()))
    first_chunk = len(eng.chunks[0].layouts)
    # the first step builds the engine; from the second on, every matrix of the first chunk is done early
    assert skipped[0] == 0 and all(s == first_chunk for s in skipped[1:]), (skipped, first_chunk)
    if cap is None:
        assert first_chunk == len(eng.shapes) == len(SHAPES) + 2          # the 3-D parameter is three matrices
    else:
        assert len(eng.runtimes) > 1 and first_chunk < len(eng.shapes)


def test_overlapped_step_matches_the_oracle(M):
    gpu = _params(78)
    cpu = [torch.nn.Parameter(p.detach().cpu().clone()) for p in gpu]
    og = M.SingleDeviceMuon(gpu, lr=0.02, weight_decay=0.01, overlap_backward=True)
    oc = O.OracleSingleDeviceMuon(cpu, lr=0.02, weight_decay=0.01)
    for step in range(3):
        xs = _inputs(gpu, 200 + step)
        for opt, params in ((og, gpu), (oc, cpu)):
            opt.zero_grad(set_to_none=True)
            _loss(params, xs).backward()
        og.step()
        oc.step()
        for pc, pg in zip(cpu, gpu):
            tol = (1e-3 if pc.ndim == 2 else 3e-3) * (step + 1) ** 0.5
            assert O.rel_fro(pg.detach().cpu(), pc.detach()) <= tol, (step, tuple(pc.shape))
    assert len(next(iter(og._muon_engines.values()))._skip) == len(SHAPES) + 2       # the 3-D parameter is three matrices


def _drive(M, scenario, overlap):
    """Six iterations of one training-loop scenario; returns parameters and momentum buffers."""
    params = _params(79)
    opt = M.SingleDeviceMuon(params, lr=0.02, weight_decay=0.01, overlap_backward=overlap)
    for it in range(6):
        xs = _inputs(params, 300 + it)
        opt.zero_grad(set_to_none=(it % 2 == 0))
        _loss(params, xs).backward()
        if scenario == "accumulate":             # a second micro-batch accumulates into the same gradients
            _loss(params, _inputs(params, 900 + it)).backward()
        elif scenario == "clip_in_place":        # writes the gradients after the hooks consumed them
            torch.nn.utils.clip_grad_norm_(params, 0.05)
        elif scenario == "replace":              # what a clipping routine that reallocates does
            for p in params[::2]:
                p.grad = p.grad.clone() * 0.5
        elif scenario == "skip" and it in (2, 3):
            continue                             # a loss scaler after an overflow: no step() this iteration
        elif scenario == "skip_none" and it == 2:
            opt.zero_grad(set_to_none=True)      # skipped, and the next step sees no gradient at all
            opt.step()
            continue
        opt.step()
    torch.cuda.synchronize()
    staged = len(next(iter(opt._muon_engines.values()))._skip)
    return [p.detach().clone() for p in params], [opt.state[p]["momentum_buffer"].clone() for p in params], staged


@pytest.mark.parametrize("scenario", ["accumulate", "clip_in_place", "replace", "skip", "skip_none"])
def test_overlap_takes_its_early_stage_back_when_the_gradient_changes(M, scenario):
    """Gradient accumulation, in-place clipping, replaced gradient tensors and skipped steps under
    overlap_backward give the bits of the plain optimizer driven the same way: a stage that ran on a
    gradient that is no longer the one step() sees is undone (the momentum buffer restored) and run
    again, and a skipped step leaves the momentum untouched as the reference does (muon.py:97 runs
    inside step() only)."""
    pa, ma, _ = _drive(M, scenario, overlap=False)
    pb, mb, staged = _drive(M, scenario, overlap=True)
    for a, b in zip(pa + ma, pb + mb):
        assert torch.equal(a, b), (scenario, tuple(a.shape))
    assert all(torch.isfinite(p).all() for p in pb)
    if scenario in ("accumulate", "skip", "skip_none"):
        assert staged == len(SHAPES) + 2         # the last step still found every stage done early
    elif scenario == "clip_in_place":
        assert staged == 0                       # every stage was taken back
    else:
        assert 0 < staged < len(SHAPES) + 2


def test_a_step_that_raises_leaves_the_adam_counters_alone(M):
    """Groups are prepared before anything is launched; a later group that raises must not leave the
    Adam step counters of an earlier one advanced (muon.py:254 increments inside the update)."""
    gain = torch.nn.Parameter(torch.ones(50, device="cuda"))
    w = torch.nn.Parameter(torch.randn(64, 64, device="cuda") * 0.02)
    bad = torch.nn.Parameter(torch.randn(64, 64, device="cuda").half())
    opt = M.SingleDeviceMuonWithAuxAdam([dict(params=[gain], use_muon=False), dict(params=[w], use_muon=True)])
    for p in (gain, w):
        p.grad = torch.randn_like(p) * 1e-2
    opt.step()
    assert opt.state[gain]["step"] == 1
    opt.add_param_group(dict(params=[bad], use_muon=True, lr=0.02, momentum=0.95, weight_decay=0))
    bad.grad = torch.randn_like(bad)
    before = gain.detach().clone()
    with pytest.raises(NotImplementedError):
        opt.step()
    torch.cuda.synchronize()
    assert opt.state[gain]["step"] == 1 and torch.equal(gain.detach(), before)


def test_tensor_hyper_parameters_and_side_streams_change_nothing(M):
    """0-dim tensors as lr / weight decay / momentum / betas (schedulers and checkpoints leave them
    in the groups) give the bits of the same values as floats, and so do steps issued under
    torch.cuda.stream(...) of alternating streams with the usual event ordering between them."""
    pa, pb = _params(80), _params(80)
    ga, gb = (torch.nn.Parameter(torch.ones(33, device="cuda")) for _ in range(2))
    plain = _make(M, pa, ga)
    t64 = lambda v: torch.tensor(v, dtype=torch.float64)       # the same double as the python float
    other = M.SingleDeviceMuonWithAuxAdam(
        [dict(params=pb, use_muon=True, lr=t64(0.02), weight_decay=t64(0.01).cuda(), momentum=t64(0.95)),
         dict(params=[gb], use_muon=False, lr=t64(3e-4), weight_decay=0.0, betas=(t64(0.9), t64(0.95)),
              eps=t64(1e-10))])
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    main = torch.cuda.current_stream()
    for step in range(4):
        xs = _inputs(pa, 400 + step)
        for opt, params, gain in ((plain, pa, ga), (other, pb, gb)):
            opt.zero_grad(set_to_none=True)
            (_loss(params, xs) + (gain * gain).sum()).backward()
        plain.step()
        s = streams[step % 2]
        s.wait_stream(main)
        with torch.cuda.stream(s):
            other.step()
        main.wait_stream(s)
        torch.cuda.synchronize()
        for a, b in zip(pa + [ga], pb + [gb]):
            assert torch.equal(a.detach(), b.detach()), (step, tuple(a.shape))


def test_functional_calls_from_several_threads_and_streams_share_an_engine_safely(M):
    """The functional entry points cache one engine (one workspace) per shape.  Calls of the same
    shape from several threads, each on a stream of its own, must not run side by side in that
    workspace: every result equals the one computed alone."""
    import threading
    torch.manual_seed(11)
    M.clear_engine_cache()
    inputs = [torch.randn(256, 512, device="cuda") * 0.02 for _ in range(8)]
    want = [M.zeropower_via_newtonschulz5(g).clone() for g in inputs]
    torch.cuda.synchronize()
    got, errors = [None] * len(inputs), []

    def work(lo, hi):
        try:
            s = torch.cuda.Stream()
            s.wait_stream(torch.cuda.default_stream())
            with torch.cuda.stream(s):
                for rep in range(3):
                    for i in range(lo, hi):
                        got[i] = M.zeropower_via_newtonschulz5(inputs[i])
            s.synchronize()
        except Exception as e:          # surfaces in the main thread below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(k * 2, k * 2 + 2)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for w, g in zip(want, got):
        assert torch.equal(w, g)


def test_usual_training_loop_companions(M):
    """A learning-rate scheduler, gradient clipping and a gradient scaler around the optimizer, as a
    training script has them: the scheduler's `initial_lr` key in the groups, its wrapped step(),
    clipped (in place) gradients and the scaler's unscale / conditional step all go through, and
    the parameters follow the oracle optimizer driven the same way on the CPU."""
    gpu = _params(81)
    cpu = [torch.nn.Parameter(p.detach().cpu().clone()) for p in gpu]
    og = M.SingleDeviceMuon(gpu, lr=0.02, weight_decay=0.01)
    oc = O.OracleSingleDeviceMuon(cpu, lr=0.02, weight_decay=0.01)
    schedule = lambda step: 1.0 / (1 + step)
    sg = torch.optim.lr_scheduler.LambdaLR(og, schedule)
    sc = torch.optim.lr_scheduler.LambdaLR(oc, schedule)
    scaler = torch.amp.GradScaler("cuda", init_scale=1024.0)          # a power of two: unscaling is exact
    for step in range(3):
        xs = _inputs(gpu, 500 + step)
        og.zero_grad(set_to_none=True)
        oc.zero_grad(set_to_none=True)
        scaler.scale(_loss(gpu, xs)).backward()
        _loss(cpu, xs).backward()
        scaler.unscale_(og)
        torch.nn.utils.clip_grad_norm_(gpu, 0.05)
        torch.nn.utils.clip_grad_norm_(cpu, 0.05)
        scaler.step(og)
        scaler.update()
        oc.step()
        sg.step()
        sc.step()
        assert og.param_groups[0]["lr"] == oc.param_groups[0]["lr"] == 0.02 * schedule(step + 1)
        for pc, pg in zip(cpu, gpu):
            # (the gradients themselves come from two matmul implementations here, and lr / |p| is large
            # for the small matrices: 2e-3 below 256 rows or columns, as for the conv-sized shapes elsewhere)
            small = pc.ndim != 2 or min(pc.shape) < 256
            tol = (2e-3 if small else 1e-3) * (1.5 if pc.ndim != 2 else 1.0) * (step + 1) ** 0.5
            assert O.rel_fro(pg.detach().cpu(), pc.detach()) <= tol, (step, tuple(pc.shape))
