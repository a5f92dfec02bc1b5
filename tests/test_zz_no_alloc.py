"""muon_amd_ns_gemm_noalloc (split-reduction scratch in a static device array inside the library)
against muon_amd_ns_gemm (caller-owned scratch), through the C ABI: the same bits, on two calls in a
row, the second with a smaller input; sizes beyond the static maximum are refused."""
import numpy as np
import pytest
import torch

from muon_amd import _lib, plan

pytestmark = pytest.mark.gpu


def _upload(arr):
    return torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).reshape(-1).copy()).cuda()


def _syrk_both_ways(lib, shapes, seed):
    """X X^T (with its c*A copy) of every matrix of `shapes` through both entry points."""
    chunk = plan.ChunkPlan([(i, r, c) for i, (r, c) in enumerate(shapes)], 0, 5, True)
    assert 0 < chunk.split_slots <= lib.muon_amd_noalloc_max_split_slots()
    ws = torch.zeros(chunk.workspace_bytes, dtype=torch.uint8, device="cuda")
    base = ws.data_ptr()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    for lay in chunk.layouts:       # the operand: X, zero padded, rows of pitch ldn
        x = ws[lay.off["X0"]: lay.off["X0"] + lay.mp * lay.ldn * 2].view(torch.bfloat16).view(lay.mp, lay.ldn)
        x[:lay.m, :lay.n] = (torch.randn(lay.m, lay.n, device="cuda", generator=gen) * 0.05).bfloat16()
    gemm = chunk.gemm_descs(base)[plan.PH_SYRK]
    jobs = chunk.syrk_jobs
    assert lib.muon_amd_validate_gemm(_lib.host_ptr(gemm), chunk.nmat, _lib.host_ptr(jobs), len(jobs), 0,
                                      chunk.split_slots) == 0
    gemm_dev, jobs_dev = _upload(gemm), _upload(jobs)
    stream = torch.cuda.current_stream().cuda_stream
    flags = _lib.ROUND_REFERENCE

    def outputs():
        torch.cuda.synchronize()
        res = []
        for lay in chunk.layouts:
            for name in ("A", "CA"):
                res.append(ws[lay.off[name]: lay.off[name] + lay.mp * lay.ldm * 2].clone())
        return res

    def clear_outputs():
        for lay in chunk.layouts:
            for name in ("A", "CA"):
                ws[lay.off[name]: lay.off[name] + lay.mp * lay.ldm * 2].fill_(0x5a)

    clear_outputs()
    counters = torch.zeros(chunk.split_slots, dtype=torch.int32, device="cuda")
    _lib.check(lib.muon_amd_ns_gemm(gemm_dev.data_ptr(), jobs_dev.data_ptr(), len(jobs), 0, 1.0, 0.0, 2.0315, flags,
                                    base + chunk.off_split_partials, counters.data_ptr(), stream), "ns_gemm")
    want = outputs()
    assert int(counters.abs().sum()) == 0
    clear_outputs()
    _lib.check(lib.muon_amd_ns_gemm_noalloc(gemm_dev.data_ptr(), jobs_dev.data_ptr(), len(jobs), 0, 1.0, 0.0, 2.0315,
                                            flags, chunk.split_slots, stream), "ns_gemm_noalloc")
    got = outputs()
    for w, g in zip(want, got):
        assert torch.equal(w, g)
    # and the product is the right one (fp32 matmul of the same bf16 operand)
    lay = chunk.layouts[0]
    x = ws[lay.off["X0"]: lay.off["X0"] + lay.mp * lay.ldn * 2].view(torch.bfloat16).view(lay.mp, lay.ldn)[:lay.m, :lay.n].float()
    a = got[0].view(torch.bfloat16).view(lay.mp, lay.ldm)[:lay.m, :lay.m].float()
    ref = x @ x.T
    assert float((a - ref).norm() / ref.norm()) < 5e-3
    return chunk.split_slots


def test_noalloc_gemm_equals_the_caller_scratch_entry_point_twice_in_a_row():
    lib = _lib.load()
    _lib.check(lib.muon_amd_init(), "init")
    first = _syrk_both_ways(lib, [(128, 8192), (128, 16384), (256, 4608), (512, 2304)], seed=1)
    second = _syrk_both_ways(lib, [(128, 4096)], seed=2)          # smaller: fewer slots, stale contents beyond them
    assert second < first
    third = _syrk_both_ways(lib, [(16384, 128), (128, 8192)], seed=3)
    assert third > second


def test_noalloc_gemm_refuses_more_slots_than_the_static_array_holds():
    lib = _lib.load()
    cap = lib.muon_amd_noalloc_max_split_slots()
    assert cap == 256
    dummy = torch.zeros(64, dtype=torch.uint8, device="cuda")
    rc = lib.muon_amd_ns_gemm_noalloc(dummy.data_ptr(), dummy.data_ptr(), 1, 0, 1.0, 0.0, 0.0, 0, cap + 1, None)
    assert rc == -1 and b"split slots" in lib.muon_amd_last_error()
    rc = lib.muon_amd_ns_gemm_noalloc(dummy.data_ptr(), dummy.data_ptr(), 1, 1, 1.0, 0.0, 0.0, 0, 4, None)
    assert rc == -1 and b"does not split" in lib.muon_amd_last_error()
