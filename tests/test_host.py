"""Host-side logic that needs no GPU: the C ABI library loads and exports every declared symbol,
descriptor layouts match, launch plans are well formed, and the optimizer classes keep the
reference's constructor contract (reference muon.py:39-43, 77-79, 139-156, 206-222)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import muon_amd
from muon_amd import _lib, plan

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------------------------------
# C ABI
# ------------------------------------------------------------------------------------------
def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "muon_amd.h")).read()
    declared = set(re.findall(r"\b(muon_amd_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    lib = _lib.load()
    assert lib.muon_amd_abi_version() == 3
    for tc, (tr, tcol) in plan.TILE_DIMS.items():
        assert (lib.muon_amd_gemm_tile_rows(tc), lib.muon_amd_gemm_tile_cols(tc)) == (tr, tcol)
    assert lib.muon_amd_gemm_tile_rows(7) < 0 and b"tile class" in lib.muon_amd_last_error()
    assert lib.muon_amd_elementwise_block_elems() == plan.EW_BLOCK_ELEMS
    assert lib.muon_amd_normalize_tile() == plan.NT_TILE


def test_struct_layouts_match_the_library():
    lib = _lib.load()
    assert _lib.MAT_DESC.itemsize == lib.muon_amd_sizeof_mat_desc() == 120
    assert _lib.GEMM_DESC.itemsize == lib.muon_amd_sizeof_gemm_desc() == 104
    assert _lib.TILE_JOB.itemsize == lib.muon_amd_sizeof_tile_job() == 32
    assert _lib.ADAM_DESC.itemsize == lib.muon_amd_sizeof_adam_desc() == 56


def test_entry_points_reject_bad_arguments_without_a_gpu():
    lib = _lib.load()
    assert lib.muon_amd_ns_gemm(None, None, 1, 0, 1.0, 0.0, 0.0, 0, None, None, None) == -1
    assert lib.muon_amd_momentum(None, None, 1, 1, 0.05, 0.95, 1, 0, None, None) == -1
    assert lib.muon_amd_adam(None, None, 1, 1, 1e-3, 1.0, 0.1, 0.05, 1e-10, 0.1, 0.05, None, None) == -1
    with pytest.raises(_lib.MuonAmdError):
        _lib.check(lib.muon_amd_apply(None, None, 0, 0, 0.0, 1.0, None, None), "apply")


# ------------------------------------------------------------------------------------------
# planning
# ------------------------------------------------------------------------------------------
SHAPES = [(768, 3072), (3072, 768), (768, 768), (4096, 4096), (64, 216), (16384, 128), (5, 3), (1024, 4096)]


def _check_chunk(lib, c):
    """Tables of one chunk: accepted by the library's validators, every tile of every product
    covered exactly once, workspace regions disjoint and inside the workspace."""
    T = c.tile
    assert all(plan.tile_class_for(l.m) == c.tile_class for l in c.layouts)
    g = c.gemm_descs(1 << 20)
    syrk_phases = (plan.PH_SYRK, plan.PH_SYRK_ODD)
    for ph in (plan.PH_SYRK, plan.PH_SYRK_ODD, plan.PH_POLY, plan.PH_UPD_EVEN, plan.PH_UPD_ODD, plan.PH_UPD_LAST):
        jobs = c.syrk_jobs if ph in syrk_phases else c.sym_jobs if ph == plan.PH_POLY else c.full_jobs
        tile_class = c.update_class if jobs is c.full_jobs else c.tile_class     # the update products may use larger tiles
        rc = lib.muon_amd_validate_gemm(_lib.host_ptr(g[ph]), c.nmat, _lib.host_ptr(jobs), len(jobs), tile_class,
                                        c.split_slots if ph in syrk_phases else 0)
        assert rc == 0, lib.muon_amd_last_error()
    # the update product reads X itself, k-major, and writes the other buffer; X X^T follows the iterate
    for k, l in enumerate(c.layouts):
        x0, x1 = (1 << 20) + l.off["X0"], (1 << 20) + l.off["X1"]
        assert g[plan.PH_SYRK, k]["P"] == g[plan.PH_UPD_EVEN, k]["Q"] == g[plan.PH_UPD_EVEN, k]["D"] == x0
        assert g[plan.PH_SYRK_ODD, k]["P"] == g[plan.PH_UPD_ODD, k]["Q"] == g[plan.PH_UPD_EVEN, k]["C"] == x1
        assert g[plan.PH_UPD_ODD, k]["C"] == x0
        assert all(g[ph, k]["q_kmajor"] == 1 and g[ph, k]["CT"] == 0 for ph in (plan.PH_UPD_EVEN, plan.PH_UPD_ODD, plan.PH_UPD_LAST))
        assert all(g[ph, k]["q_kmajor"] == 0 for ph in (plan.PH_SYRK, plan.PH_SYRK_ODD, plan.PH_POLY))
    assert c.update_class in (c.tile_class, 1)
    TR, TC = c.tile_rows, c.tile_cols
    UR, UC = plan.TILE_DIMS[c.update_class]
    for k, l in enumerate(c.layouts):
        mt, nt, ratio = l.mp // TR, l.np_ // TC, TR // TC
        sj = c.sym_jobs[c.sym_jobs["desc"] == k]
        got = sorted(zip((sj["i0"] // TR).tolist(), (sj["j0"] // TC).tolist()))
        assert got == [(i, j) for i in range(mt) for j in range(i * ratio, l.mp // TC)]
        assert np.array_equal(sj["diag"], (sj["i0"] // TR == sj["j0"] // TR).astype(np.int32))
        # direct tiles plus mirrors of the off-diagonal-block tiles cover the matrix exactly once
        cover = np.zeros((l.mp // TC, l.mp // TC), dtype=int)
        for i0, j0, dg in zip(sj["i0"].tolist(), sj["j0"].tolist(), sj["diag"].tolist()):
            cover[i0 // TC:(i0 + TR) // TC, j0 // TC] += 1
            if not dg:
                cover[j0 // TC, i0 // TC:(i0 + TR) // TC] += 1
        assert (cover == 1).all()
        fj = c.full_jobs[c.full_jobs["desc"] == k]
        got = sorted(zip((fj["i0"] // UR).tolist(), (fj["j0"] // UC).tolist()))
        assert got == [(i, j) for i in range(l.mp // UR) for j in range(l.np_ // UC)]
        assert np.all(fj["i0"] % UR == 0) and np.all(fj["j0"] % UC == 0)
        assert l.mp % T == 0 and l.np_ % T == 0 and l.mp >= l.m and l.np_ >= l.n
        assert l.wide == (l.rows <= l.cols)
    # workspace regions do not overlap and stay inside the chunk's workspace
    regions = []
    for l in c.layouts:
        size = {"X0": l.mp * l.ldn * 2, "X1": l.mp * l.ldn * 2,
                "A": l.mp * l.ldm * 2, "B": l.mp * l.ldm * 2, "CA": l.mp * l.ldm * 2}
        assert set(l.off) == set(size)            # two copies of X, no transposed one: 2 m n + 3 m^2
        for name in size:
            regions.append((l.off[name], l.off[name] + size[name]))
    regions += [(c.off_partials, c.off_partials + 4 * c.nblocks), (c.off_denoms, c.off_denoms + 4 * c.nmat)]
    regions.sort()
    assert all(a[1] <= b[0] for a, b in zip(regions, regions[1:])) and regions[-1][1] <= c.workspace_bytes
    assert all(r[0] % 256 == 0 for r in regions)
    md = c.mat_descs(1 << 20)
    md["grad"] = 4096
    md["out"] = 8192
    rc = lib.muon_amd_validate_mats(_lib.host_ptr(md), c.nmat, _lib.host_ptr(c.block_prefix),
                                    _lib.host_ptr(c.tile_prefix), c.tile)
    assert rc == 0, lib.muon_amd_last_error()




@pytest.mark.parametrize("ref", [True, False])
def test_plans_validate_and_cover_every_tile_once(ref):
    lib = _lib.load()
    chunks = plan.plan_chunks(SHAPES, 5, ref, 1 << 30)
    seen = sorted(l.index for c in chunks for l in c.layouts)
    assert seen == list(range(len(SHAPES)))
    for c in chunks:
        _check_chunk(lib, c)


def test_random_parameter_lists_plan_into_valid_tables():
    """Seeded random lists of shapes (tiny, around the tile edges, tall, wide), random workspace
    caps, both roundings and the AOL variants: every chunk passes the same checks."""
    import random
    lib = _lib.load()
    rng = random.Random(7)
    edge = [1, 2, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 767, 768, 1023, 1024, 1025, 2048, 4096]

    def dim():
        k = rng.random()
        return rng.randint(1, 70) if k < 0.3 else rng.choice(edge) if k < 0.7 else rng.randint(64, 5000)

    for case in range(60):
        shapes = [(dim(), dim()) for _ in range(rng.randint(1, 12))]
        variant = rng.choice(["ns5", "ns5", "aol4", "aol4_rows"])
        if variant == "aol4_rows":      # refused below a side of 32
            shapes = [(max(r, plan.AOL_ROWS_MIN_SIDE), max(c, plan.AOL_ROWS_MIN_SIDE)) for r, c in shapes]
        aol = variant != "ns5"
        biggest = max(plan.matrix_workspace_bytes(r, c, plan.pad_unit(plan.tile_class_for(min(r, c)))) +
                      plan.matrix_scratch_bytes(r, c, plan.tile_class_for(min(r, c)), aol) for r, c in shapes)
        cap = max(biggest, rng.choice([1 << 20, 16 << 20, 256 << 20, 1 << 34]))
        chunks = plan.plan_chunks(shapes, 5, rng.random() < 0.5, cap, variant)
        assert sorted(l.index for c in chunks for l in c.layouts) == list(range(len(shapes))), (case, shapes)
        for c in chunks:
            assert c.workspace_bytes <= cap, (case, shapes, cap)
            _check_chunk(lib, c)
            if c.aol:
                aol = c.aol_descs(1 << 20)
                rc = lib.muon_amd_validate_aol(_lib.host_ptr(aol), c.nmat, _lib.host_ptr(c.aol_row_prefix),
                                               _lib.host_ptr(c.aol_seg_prefix))
                assert rc == 0, lib.muon_amd_last_error()


def test_validation_catches_a_bad_table():
    lib = _lib.load()
    c = plan.plan_chunks([(768, 3072)], 5, True, 1 << 30)[0]
    g = c.gemm_descs(1 << 20)
    bad = c.full_jobs.copy()
    bad["j0"][0] = c.layouts[0].np_          # one tile past the last column
    assert lib.muon_amd_validate_gemm(_lib.host_ptr(g[2]), 1, _lib.host_ptr(bad), len(bad), c.tile_class, 0) == -1
    gd = g[0].copy()
    gd["K"] = 100                            # not a multiple of the k-block
    assert lib.muon_amd_validate_gemm(_lib.host_ptr(gd), 1, _lib.host_ptr(c.syrk_jobs), len(c.syrk_jobs), c.tile_class, 0) == -1
    low = c.syrk_jobs.copy()
    low["i0"][0], low["j0"][0] = c.tile_rows, 0      # below the diagonal of a mirrored GEMM
    assert lib.muon_amd_validate_gemm(_lib.host_ptr(g[0]), 1, _lib.host_ptr(low), len(low), c.tile_class, 0) == -1
    short = c.syrk_jobs.copy()
    short["k1"][0] -= 64                     # an unsplit job that does not reduce over all of K
    assert lib.muon_amd_validate_gemm(_lib.host_ptr(g[0]), 1, _lib.host_ptr(short), len(short), c.tile_class, 0) == -1


def test_split_reduction_plan():
    """X X^T of a short, very wide matrix is split along K by a rule that looks at the matrix alone."""
    lib = _lib.load()
    assert [plan.split_factor(128, 16384), plan.split_factor(512, 4608), plan.split_factor(512, 2304),
            plan.split_factor(256, 576), plan.split_factor(768, 3072), plan.split_factor(4096, 14336)] == [10, 3, 1, 1, 1, 1]
    c = plan.plan_chunks([(128, 16384), (16384, 128), (512, 4608), (64, 216)], 5, True, 1 << 30)[0]
    g = c.gemm_descs(1 << 20)
    assert c.split_slots == 10 + 10 + 10 * 3 and len(c.syrk_jobs) == c.split_slots + 1
    assert np.all(c.sym_jobs["split"] == 0) and np.all(c.full_jobs["split"] == 0)      # only X X^T is split
    rc = lib.muon_amd_validate_gemm(_lib.host_ptr(g[plan.PH_SYRK]), c.nmat, _lib.host_ptr(c.syrk_jobs),
                                    len(c.syrk_jobs), c.tile_class, c.split_slots)
    assert rc == 0, lib.muon_amd_last_error()
    for k, l in enumerate(c.layouts):        # every tile's jobs tile [0, K) in 64-wide blocks, one slot each
        jk = c.syrk_jobs[c.syrk_jobs["desc"] == k]
        for i0, j0 in {(a, b) for a, b in zip(jk["i0"].tolist(), jk["j0"].tolist())}:
            t = np.sort(jk[(jk["i0"] == i0) & (jk["j0"] == j0)], order="k0")
            assert t["k0"][0] == 0 and t["k1"][-1] == l.np_ and np.array_equal(t["k1"][:-1], t["k0"][1:])
            assert np.all(t["k0"] % 64 == 0) and len(t) == plan.split_factor(l.mp, l.np_)
            if len(t) > 1:
                assert np.array_equal(np.sort(t["split"] & 0xffff), np.arange(len(t))) and len(set(t["part_base"].tolist())) == 1
    groups = c.syrk_jobs[c.syrk_jobs["split"] != 0]
    slots = sorted((groups["part_base"] + (groups["split"] & 0xffff)).tolist())
    assert slots == list(range(c.split_slots))                                        # no two jobs share a slot
    assert c.off_split_partials + c.split_slots * c.tile_rows * c.tile_cols * 4 <= c.workspace_bytes
    # the library refuses too few slots, a hole in a group's K range and a job counted twice
    args = (_lib.host_ptr(g[plan.PH_SYRK]), c.nmat)
    assert lib.muon_amd_validate_gemm(*args, _lib.host_ptr(c.syrk_jobs), len(c.syrk_jobs), c.tile_class, c.split_slots - 1) == -1
    hole = c.syrk_jobs.copy()
    first = np.flatnonzero(hole["split"] != 0)[0]
    hole["k1"][first] -= 64
    assert lib.muon_amd_validate_gemm(*args, _lib.host_ptr(hole), len(hole), c.tile_class, c.split_slots) == -1
    twice = np.concatenate([c.syrk_jobs, c.syrk_jobs[first:first + 1]])
    assert lib.muon_amd_validate_gemm(*args, _lib.host_ptr(twice), len(twice), c.tile_class, c.split_slots) == -1


def test_xcd_permutation_and_orientation_of_the_iterate():
    for n in (1, 7, 8, 9, 136, 1000, 4352):
        for group in (32, 64):
            p = plan.xcd_permutation(n, group)
            assert sorted(p.tolist()) == list(range(n))
    # a job count that is no multiple of eight groups: what is left over still reaches every XCD as
    # one contiguous run of the list (block b is on XCD b % 8), no XCD gets more than one job more than
    # another, and nothing shifts the whole groups before it
    for n, group in ((966, 64), (1296, 32), (454, 64), (1000, 16)):
        p = plan.xcd_permutation(n, group)
        full = n // (8 * group) * (8 * group)
        assert p[:full].tolist() == plan.xcd_permutation(full, group).tolist()
        runs = [p[full:][x::8] for x in range(8)]
        assert all(len(r) == 0 or r.tolist() == list(range(r[0], r[0] + len(r))) for r in runs)
        assert max(map(len, runs)) - min(map(len, runs)) <= 1
    p = plan.xcd_permutation(512, 32)            # block b runs on XCD b % 8, slot b // 8
    assert p[:8].tolist() == [0, 32, 64, 96, 128, 160, 192, 224] and p[8] == 1      # a 32-job group per XCD
    assert p[256:264].tolist() == [256, 288, 320, 352, 384, 416, 448, 480]           # next round of groups
    # the normalise launch writes X0 in one orientation: the parameter's for a wide matrix and for a run
    # without iterations (where it is the result), the transposed one for a tall matrix that iterates
    for steps in (0, 1, 2, 5):
        c = plan.ChunkPlan([(0, 300, 100), (1, 100, 300)], 0, steps, True)
        md = c.mat_descs(1 << 20)
        x0 = [(1 << 20) + l.off["X0"] for l in c.layouts]
        tall, wide = md[0], md[1]
        assert wide["direct"] == x0[1] and wide["transp"] == 0
        assert (tall["direct"], tall["transp"]) == ((x0[0], 0) if steps == 0 else (0, x0[0]))
        assert all(m["result"] == (m["direct"] if steps == 0 else 0) for m in md)
        assert all(m["u"] == (1 << 20) + l.off["X1"] for m, l in zip(md, c.layouts))
    # workspace per matrix: 2 m n + 3 m^2 bf16 elements (padded)
    assert plan.matrix_workspace_bytes(4096, 14336, 256) == 2 * (2 * 4096 * 14336 + 3 * 4096 * 4096)


def test_chunking_respects_the_workspace_cap():
    shapes = [(4096, 14336)] * 6 + [(1024, 4096)] * 4 + [(768, 768)] * 3
    one = plan.matrix_workspace_bytes(4096, 14336, 256)
    chunks = plan.plan_chunks(shapes, 5, True, 2 * one + (1 << 20))
    big = [c for c in chunks if any(l.n == 14336 for l in c.layouts)]
    assert all(sum(1 for l in c.layouts if l.n == 14336) <= 2 for c in big) and len(big) >= 3
    assert all(len({plan.tile_class_for(l.m) for l in c.layouts}) == 1 for c in chunks)
    tiny_cap = plan.plan_chunks(shapes, 5, True, 1)           # every matrix still gets a chunk
    assert sum(c.nmat for c in tiny_cap) == len(shapes)


# ------------------------------------------------------------------------------------------
# optimizer constructors (CPU tensors: construction works, stepping refuses loudly)
# ------------------------------------------------------------------------------------------
def test_constructor_contract_matches_the_reference():
    a = torch.nn.Parameter(torch.zeros(4, 8))
    b = torch.nn.Parameter(torch.zeros(16, 8))
    c = torch.nn.Parameter(torch.zeros(8))
    opt = muon_amd.SingleDeviceMuon([a, b])
    assert opt.defaults == dict(lr=0.02, weight_decay=0, momentum=0.95)
    assert [tuple(p.shape) for p in opt.param_groups[0]["params"]] == [(4, 8), (16, 8)]     # order kept
    srt = muon_amd.Muon([a, b], lr=0.05)
    assert [tuple(p.shape) for p in srt.param_groups[0]["params"]] == [(16, 8), (4, 8)]     # muon.py:42
    with pytest.raises(AssertionError):
        muon_amd.Muon((a, b))                                                             # must be a list (muon.py:41)
    with pytest.raises(AssertionError):
        muon_amd.Muon([])
    groups = [dict(params=[a, b], use_muon=True), dict(params=[c], use_muon=False)]
    aux = muon_amd.MuonWithAuxAdam(groups)
    g0, g1 = aux.param_groups
    assert (g0["lr"], g0["momentum"], g0["weight_decay"]) == (0.02, 0.95, 0)
    assert (g1["lr"], g1["betas"], g1["eps"], g1["weight_decay"]) == (3e-4, (0.9, 0.95), 1e-10, 0)
    assert [tuple(p.shape) for p in g0["params"]] == [(16, 8), (4, 8)]                      # muon.py:143
    sd = muon_amd.SingleDeviceMuonWithAuxAdam([dict(params=[a, b], use_muon=True)])
    assert [tuple(p.shape) for p in sd.param_groups[0]["params"]] == [(4, 8), (16, 8)]      # not sorted
    for bad in ([dict(params=[a])], [dict(params=[a], use_muon=True, betas=(0.9, 0.9))],
                [dict(params=[c], use_muon=False, momentum=0.9)]):
        with pytest.raises(AssertionError):
            muon_amd.SingleDeviceMuonWithAuxAdam(bad)
    with pytest.raises(ValueError):
        muon_amd.SingleDeviceMuon([a], ns_rounding="nearest")


def test_copies_and_pickles_keep_the_algorithm_options():
    """torch pickles only defaults/state/param_groups; the keyword-only options that select the
    algorithm must survive copy.deepcopy and pickle, or a copied optimizer silently runs another
    iteration."""
    import copy
    import pickle
    a = torch.nn.Parameter(torch.zeros(4, 8))
    opt = muon_amd.SingleDeviceMuon([a], ns_variant="aol4", ns_rounding="fused", mutate_grad=True,
                                    use_graph=True, workspace_bytes=1 << 20)
    for dup in (copy.deepcopy(opt), pickle.loads(pickle.dumps(opt))):
        assert dup._ns_variant == "aol4" and dup._reference_rounding is False
        assert dup._mutate_grad is True and dup._use_graph is True and dup._workspace_bytes == 1 << 20
        assert dup._muon_engines == {} and dup.param_groups[0]["lr"] == 0.02
    aux = muon_amd.MuonWithAuxAdam([dict(params=[a], use_muon=True)], ns_variant="aol4")
    assert copy.deepcopy(aux)._ns_variant == "aol4"
    plain = copy.deepcopy(muon_amd.SingleDeviceMuon([a]))
    assert plain._ns_variant == "ns5" and plain._reference_rounding is True and plain._use_graph is False


def test_no_cpu_fallback():
    a = torch.nn.Parameter(torch.zeros(4, 8))
    a.grad = torch.ones(4, 8)
    with pytest.raises(muon_amd.MuonAmdError, match="no CPU implementation"):
        muon_amd.SingleDeviceMuon([a]).step()
    with pytest.raises(muon_amd.MuonAmdError):
        muon_amd.zeropower_via_newtonschulz5(torch.ones(4, 8))
    with pytest.raises(muon_amd.MuonAmdError):
        muon_amd.adam_update(torch.ones(4), torch.zeros(4), torch.zeros(4), 1, (0.9, 0.95), 1e-10)
    with pytest.raises(muon_amd.MuonAmdError):
        muon_amd.muon_update(torch.ones(4, 8), torch.zeros(4, 8))
    with pytest.raises(AssertionError):
        muon_amd.zeropower_via_newtonschulz5(torch.ones(4))                                  # muon.py:275
    # the live function's second positional argument is epsilon (muon.py:749), the specification's the
    # iteration count (muon.py:265): an epsilon in that place must not become zero iterations
    for bad in (1e-7, 2.5, -1):
        with pytest.raises(TypeError, match="steps must be a non-negative integer"):
            muon_amd.zeropower_via_newtonschulz5(torch.ones(4, 8), bad)


def test_reference_module_name_is_importable():
    import muon
    assert muon.MuonWithAuxAdam is muon_amd.MuonWithAuxAdam
    assert muon.zeropower_via_newtonschulz5 is muon_amd.zeropower_via_newtonschulz5
    import inspect
    sig = inspect.signature(muon.muon_update)
    assert list(sig.parameters)[:4] == ["grad", "momentum", "beta", "nesterov"]
    assert sig.parameters["beta"].default == 0.95 and sig.parameters["nesterov"].default is True
    assert sig.parameters["ns_steps"].default == 5
    assert list(inspect.signature(muon.adam_update).parameters) == ["grad", "buf1", "buf2", "step", "betas", "eps"]
    z = inspect.signature(muon.zeropower_via_newtonschulz5).parameters
    assert z["steps"].default == 5 and z["epsilon"].default == 1e-7
    assert plan.NS_COEFFS == (3.4445, -4.7750, 2.0315)
    # the three products as operators: muon.py:420, 547, 705
    K = inspect.Parameter.KEYWORD_ONLY
    for fn, names in ((muon.ns_line_1, ["A", "out"]), (muon.ns_line_2, ["A", "alpha", "beta", "out"]),
                      (muon.ns_line_3, ["B", "X", "a", "out"])):
        ps = inspect.signature(fn).parameters
        assert list(ps) == names and ps["out"].kind == K and ps["out"].default is None
        assert all(ps[n].default is inspect.Parameter.empty for n in names[:-1])


def test_product_operators_check_shapes_before_anything_else_and_their_job_lists_validate():
    import muon
    from muon_amd import ops
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="must be 2D or 3D, but got 4D"):        # muon.py:424-425
        muon.ns_line_1(z(2, 2, 4, 4))
    with pytest.raises(ValueError, match="symmetric square matrix"):             # muon.py:555-558
        muon.ns_line_2(z(4, 6), 1.0, 1.0)
    with pytest.raises(ValueError, match="B must be square"):                    # muon.py:710-711
        muon.ns_line_3(z(4, 6), z(4, 6), 1.0)
    with pytest.raises(ValueError, match="same number of rows"):                 # muon.py:713-714
        muon.ns_line_3(z(4, 4), z(6, 6), 1.0)
    with pytest.raises(muon_amd.MuonAmdError, match="no CPU implementation"):
        muon.ns_line_1(z(4, 4))
    # the job list of a product: every tile on or above the diagonal once (mirrored products) or every
    # tile once, each over the whole reduction, in an order the library accepts
    lib = _lib.load()
    for tile_class, batch, rows_p, cols_p, kdim, sym, nsplit in (
            (0, 3, 384, 384, 192, True, 1), (1, 2, 1024, 1024, 1024, True, 1), (0, 1, 256, 640, 256, False, 1),
            (1, 2, 1280, 1536, 1280, False, 1), (0, 1, 128, 128, 16384, True, 10), (0, 3, 256, 256, 8256, True, 5)):
        jobs = ops._product_jobs(tile_class, batch, rows_p, cols_p, kdim, sym, nsplit)
        T = plan.TILE_DIMS[tile_class][0]
        mt, nt = rows_p // T, cols_p // T
        assert len(jobs) == batch * (mt * (mt + 1) // 2 if sym else mt * nt) * nsplit
        assert len({(j["desc"], j["i0"], j["j0"], j["k0"]) for j in jobs}) == len(jobs)
        if nsplit == 1:
            assert (jobs["k0"] == 0).all() and (jobs["k1"] == kdim).all() and (jobs["split"] == 0).all()
        else:       # every job its own slot; the jobs of a tile cover its reduction once
            assert sorted(jobs["part_base"] + (jobs["split"] & 0xffff)) == list(range(len(jobs)))
            assert ((jobs["split"] >> 16) == nsplit).all()
            assert int((jobs["k1"] - jobs["k0"]).sum()) == kdim * len(jobs) // nsplit
        if sym:
            assert (jobs["j0"] >= jobs["i0"]).all() and ((jobs["i0"] == jobs["j0"]) == (jobs["diag"] == 1)).all()
        d = np.zeros(batch, dtype=_lib.GEMM_DESC)
        d["P"] = d["Q"] = 1 << 20
        d["C"] = 1 << 24
        if sym:
            d["CT"] = d["C"]
        d["ldp"] = kdim
        d["ldq"] = kdim if sym else cols_p
        d["q_kmajor"] = 0 if sym else 1
        d["ldc"] = d["ldct"] = cols_p
        d["K"], d["rows"], d["colsn"] = kdim, rows_p, cols_p
        rc = lib.muon_amd_validate_gemm(_lib.host_ptr(d), batch, _lib.host_ptr(jobs), len(jobs), tile_class,
                                        len(jobs) if nsplit > 1 else 0)
        assert rc == 0, lib.muon_amd_last_error()


def test_product_never_imports_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "muon_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, os.path.join(dirpath, f)
    assert "oracle" not in open(os.path.join(ROOT, "muon.py")).read()


def test_aol_variant_plan_validates():
    """The 4-iteration variant: fixed schedule, one rounding per stored matrix, row-scale vectors
    in the workspace, and block prefixes the library accepts."""
    lib = _lib.load()
    assert lib.muon_amd_aol_rows_per_block() == plan.AOL_ROWS
    assert _lib.AOL_DESC.itemsize == lib.muon_amd_sizeof_aol_desc() == 64
    for variant in ("aol4", "aol4_rows"):
        shapes = [sh for sh in SHAPES if variant == "aol4" or min(sh) >= plan.AOL_ROWS_MIN_SIDE]
        chunks = plan.plan_chunks(shapes, 5, True, 1 << 30, variant)
        for c in chunks:
            assert c.variant == variant and c.aol and c.steps == len(plan.AOL_COEFFS) == 4 and not c.reference_rounding
            d = c.aol_descs(1 << 20)
            rc = lib.muon_amd_validate_aol(_lib.host_ptr(d), c.nmat, _lib.host_ptr(c.aol_row_prefix),
                                           _lib.host_ptr(c.aol_seg_prefix))
            assert rc == 0, lib.muon_amd_last_error()
            assert [c.phase_scalars(plan.PH_POLY, it) for it in range(4)] == [(co[2], co[1], 0.0) for co in plan.AOL_COEFFS]
            assert c.phase_scalars(plan.PH_UPD_EVEN, 2) == (1.0, plan.AOL_COEFFS[2][0], 0.0)
            g = c.gemm_descs(1 << 20)
            for k, l in enumerate(c.layouts):
                # the r vectors and the partial row sums lie inside the workspace, apart from everything else
                assert c.off_denoms + 4 * c.nmat <= c.off_rvec[k] and c.off_rvec[k] + 4 * l.mp <= c.off_rowsum[k]
                assert c.off_rowsum[k] + 4 * l.mp * (l.mp // 64) <= c.workspace_bytes
                assert g[plan.PH_SYRK, k]["rowsum"] == (1 << 20) + c.off_rowsum[k] == d[k]["rowsum"]
                assert g[plan.PH_SYRK, k]["ld_rowsum"] == l.mp // 64 == d[k]["ld_rowsum"]
            rc = lib.muon_amd_validate_gemm(_lib.host_ptr(g[plan.PH_SYRK]), c.nmat, _lib.host_ptr(c.syrk_jobs),
                                            len(c.syrk_jobs), c.tile_class, c.split_slots)
            assert rc == 0, lib.muon_amd_last_error()
            if variant == "aol4_rows":      # every tile of the m x m polynomial once, stored in one orientation
                TR, TC = c.tile_rows, c.tile_cols
                rc = lib.muon_amd_validate_gemm(_lib.host_ptr(g[plan.PH_POLY_FULL]), c.nmat, _lib.host_ptr(c.poly_full_jobs),
                                                len(c.poly_full_jobs), c.tile_class, 0)
                assert rc == 0, lib.muon_amd_last_error()
                assert g[plan.PH_POLY_FULL, 0]["CT"] == 0 and g[plan.PH_POLY_FULL, 0]["C"] == g[plan.PH_POLY, 0]["C"]
                for k, l in enumerate(c.layouts):
                    pj = c.poly_full_jobs[c.poly_full_jobs["desc"] == k]
                    got = sorted(zip((pj["i0"] // TR).tolist(), (pj["j0"] // TC).tolist()))
                    assert got == [(i, j) for i in range(l.mp // TR) for j in range(l.mp // TC)]
            else:
                assert c.poly_full_jobs is None
            bad = c.aol_seg_prefix.copy()
            bad[1] += 1
            assert lib.muon_amd_validate_aol(_lib.host_ptr(d), c.nmat, _lib.host_ptr(c.aol_row_prefix), _lib.host_ptr(bad)) == -1
    chunks = plan.plan_chunks(SHAPES, 5, True, 1 << 30, "aol4")
    ns5 = plan.plan_chunks(SHAPES, 5, True, 1 << 30)
    assert all(a.workspace_bytes > b.workspace_bytes for a, b in zip(chunks, ns5))


def test_header_is_plain_c_and_field_offsets_match_the_binding(tmp_path):
    """include/muon_amd.h compiles as C99 on its own, and every struct field sits where the numpy
    mirror of the binding puts it."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    structs = {"MuonMatDesc": _lib.MAT_DESC, "MuonGemmDesc": _lib.GEMM_DESC, "MuonTileJob": _lib.TILE_JOB,
               "MuonAdamDesc": _lib.ADAM_DESC, "MuonAolDesc": _lib.AOL_DESC}
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "muon_amd.h"', 'int main(void) {']
    for name, dt in structs.items():
        lines.append(f'  printf("{name} size %zu\\n", sizeof({name}));')
        for field in dt.names:
            lines.append(f'  printf("{name} {field} %zu\\n", offsetof({name}, {field}));')
    lines += ['  return 0;', '}']
    src = tmp_path / "offsets.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "offsets"
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-I", inc, str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    got = {tuple(l.split()[:2]): int(l.split()[2]) for l in out if l}
    for name, dt in structs.items():
        assert got[(name, "size")] == dt.itemsize
        for field in dt.names:
            assert got[(name, field)] == dt.fields[field][1], (name, field)


def test_overlap_backward_option_installs_hooks_and_survives_copies():
    """overlap_backward=True registers one post-accumulate-grad hook per Muon parameter (none on
    Adam parameters), new groups get theirs, copies of the optimizer re-register on their own
    parameters, and before the first step the hooks do nothing (there is no engine yet)."""
    import copy
    import muon_amd as M
    w = [torch.nn.Parameter(torch.randn(8, 4)), torch.nn.Parameter(torch.randn(4, 8))]
    gain = torch.nn.Parameter(torch.ones(4))
    opt = M.SingleDeviceMuonWithAuxAdam([dict(params=w, use_muon=True), dict(params=[gain], use_muon=False)],
                                        overlap_backward=True)
    assert len(opt._hook_handles) == 2 and opt._overlap_backward
    (w[0].sum() + w[1].sum() + gain.sum()).backward()          # hooks fire: nothing to do yet, no GPU touched
    assert all(p.grad is not None for p in w) and not opt._early_params
    extra = torch.nn.Parameter(torch.randn(4, 4))
    opt.add_param_group(dict(params=[extra], use_muon=True, lr=0.02, momentum=0.95, weight_decay=0))
    assert len(opt._hook_handles) == 3
    dup = copy.deepcopy(opt)
    assert dup._overlap_backward and len(dup._hook_handles) == 3
    assert all(p._post_accumulate_grad_hooks for g in dup.param_groups if g["use_muon"] for p in g["params"])
    plain = M.SingleDeviceMuon([torch.nn.Parameter(torch.randn(4, 4))])
    assert not plain._overlap_backward and plain._hook_handles == []


def test_update_products_take_large_tiles_only_where_they_fill_the_gpu():
    gpt2 = [(768, 2304), (768, 768), (768, 3072), (3072, 768)] * 12
    (c,) = plan.plan_chunks(gpt2, 5, True, 16 << 30)
    assert c.tile_class == 0 and c.update_class == 1 and len(c.full_jobs) == 12 * (3 * 9 + 3 * 3 + 3 * 12 + 3 * 12)
    (c,) = plan.plan_chunks([(768, 3072)], 5, True, 16 << 30)            # 36 large tiles: too few for 256 CUs
    assert c.tile_class == 0 and c.update_class == 0
    (c,) = plan.plan_chunks([(768, 3072)] * 16 + [(640, 1280)], 5, True, 16 << 30)      # 640 is not a multiple of 256
    assert c.update_class == 0
    (c,) = plan.plan_chunks([(4096, 4096)] * 2, 5, True, 16 << 30)
    assert c.tile_class == 1 and c.update_class == 1


def test_jobs_of_unequal_length_are_dealt_so_that_the_cus_stay_balanced():
    """A launch whose matrices differ in shape has jobs of different lengths; the planner deals them to
    the XCDs in half or quarter super-blocks when whole ones would leave some CUs with much more work."""
    gpt2 = [(768, 2304), (768, 768), (768, 3072), (3072, 768)] * 12
    (c,) = plan.plan_chunks(gpt2, 5, True, 16 << 30)
    kb = (c.syrk_jobs["k1"] - c.syrk_jobs["k0"]) // plan.GEMM_BK
    assert sorted(set(kb.tolist())) == [12, 36, 48] and len(kb) == 48 * 21
    cu, xcd = plan.launch_imbalance(kb, 0)
    assert cu < 1.03 and xcd < 1.02                       # (whole super-blocks: 1.14 and 1.10)
    logical = np.sort(kb)[::-1]                           # the list order: same-shape matrices adjacent
    whole = plan.launch_imbalance(logical[plan.xcd_permutation(len(kb), 64)], 0)
    assert whole[0] > 1.12 and plan.choose_xcd_group(logical, 0, 64) in (16, 32)
    # jobs of equal length: nothing to gain, the super-block stays whole
    assert plan.choose_xcd_group(np.full(1008, 12), 0, 64) == 64
    assert plan.choose_xcd_group(np.full(4352, 64), 1, 32) == 32
    # every job still appears exactly once
    assert sorted(zip(c.syrk_jobs["desc"].tolist(), c.syrk_jobs["i0"].tolist(), c.syrk_jobs["j0"].tolist())) == \
        sorted((d, i, j) for d in range(48) for i in range(0, 768, 128) for j in range(i, 768, 128))


def test_chunk_cuts_move_to_where_the_launches_fill_their_last_rounds():
    """When the workspace cap forces a cut inside a run of matrices, the cut goes where the launches of
    the chunk (and of what it leaves behind) waste least on partial last rounds; a run that fits one
    chunk is never split, and every matrix still lands in exactly one chunk, in list order."""
    llama = [(4096, 4096)] * 64 + [(1024, 4096)] * 64 + [(14336, 4096)] * 64 + [(4096, 14336)] * 32
    chunks = plan.plan_chunks(llama, 5, True, 16 << 30)
    assert [len(c.layouts) for c in chunks] == [50, 47, 127]
    assert all(c.workspace_bytes <= (16 << 30) for c in chunks)
    assert sorted(l.index for c in chunks for l in c.layouts) == list(range(len(llama)))
    # 47 matrices of m = 4096: 47 * 136 symmetric tiles = 24.97 rounds of 256 workgroups
    assert len(chunks[1].syrk_jobs) == 47 * 136 and 47 * 136 / 256 > 24.9
    for cap in (4 << 30, 8 << 30, 12 << 30):
        cs = plan.plan_chunks(llama, 5, True, cap)
        assert all(c.workspace_bytes <= cap for c in cs)
        assert sorted(l.index for c in cs for l in c.layouts) == list(range(len(llama)))
    # est >= ideal, equal jobs on a multiple of the grid are ideal
    est, ideal = plan._chunk_time_us([(4096, 4096)] * 32, 1)
    assert abs(est - ideal) < 1e-6 * ideal
    est, ideal = plan._chunk_time_us([(4096, 4096)] * 33, 1)
    assert est > 1.01 * ideal
    (c,) = plan.plan_chunks([(768, 3072)] * 46 + [(768, 768)] * 2, 5, True, 16 << 30)      # fits: stays whole
    assert len(c.layouts) == 48


def test_rows_only_aol_is_refused_below_its_stated_size():
    """plan_chunks refuses the rows-only AOL rescaling for a matrix with a side below
    AOL_ROWS_MIN_SIDE (the map does not contract there), and only that variant."""
    from muon_amd import plan
    for shape in [(18, 63), (63, 18), (31, 4096)]:
        with pytest.raises(ValueError, match="rows-only"):
            plan.plan_chunks([(256, 256), shape], 4, False, 1 << 30, "aol4_rows")
        assert plan.plan_chunks([(256, 256), shape], 4, False, 1 << 30, "aol4")
        assert plan.plan_chunks([(256, 256), shape], 5, True, 1 << 30, "ns5")
    assert plan.plan_chunks([(plan.AOL_ROWS_MIN_SIDE, 63)], 4, False, 1 << 30, "aol4_rows")


def test_update_launches_of_matrices_with_ragged_super_blocks_deal_whole_matrices_to_the_xcds():
    """Three tile rows (m = 768) against the super-block's four: the 256 x 256 update list is dealt
    in groups of 108 jobs = 4, 12 or 3 whole matrices, so an XCD sees few matrices; matrices whose
    tile rows fill the super-blocks (m = 1024, 4096) keep the super-block groups."""
    assert plan.whole_matrix_group([27, 9, 36, 36], 32) == 108
    assert plan.whole_matrix_group([75, 25, 100], 32) == 100           # lcm 300 is more than four super-blocks
    assert plan.whole_matrix_group([243, 81, 324], 32) == 32           # matrices this large keep the super-block groups
    gpt2 = [(768, 2304), (768, 768), (768, 3072), (3072, 768)] * 12
    (c,) = plan.plan_chunks(gpt2, 5, True, 16 << 30)
    assert c.update_class == 1 and len(c.full_jobs) == 1296
    x = np.arange(1296) % 8
    per_xcd = [len(set(c.full_jobs["desc"][x == k].tolist())) for k in range(8)]
    assert max(per_xcd) <= 9 and sum(per_xcd) == 48                     # no matrix on two XCDs
    assert sorted(map(tuple, c.full_jobs[["desc", "i0", "j0"]].tolist())) == sorted(
        (k, i, j) for k, lay in enumerate(c.layouts) for i in range(0, lay.mp, 256) for j in range(0, lay.np_, 256))
    medium = [(1024, 3072), (1024, 1024), (1024, 4096), (4096, 1024)] * 4
    (c,) = plan.plan_chunks(medium, 5, True, 16 << 30)
    ref = c.full_jobs.copy()
    old, plan.WHOLE_MATRIX_GROUPS = plan.WHOLE_MATRIX_GROUPS, False
    try:
        (c2,) = plan.plan_chunks(medium, 5, True, 16 << 30)
    finally:
        plan.WHOLE_MATRIX_GROUPS = old
    assert (c2.full_jobs == ref).all()


def test_lanes_split_groups_like_gpt2_small_and_nothing_else():
    """Two lanes (every other matrix of the sorted list, planned separately) for one chunk of the
    128 x 128 class whose update products run in 600-2600 tiles of 256 x 256; one lane for everything
    that measured slower in two: more tiles, update products in small tiles, the 256 x 256 class, short
    launches, several chunks, and on request."""
    gpt2 = [(768, 2304), (768, 768), (768, 3072), (3072, 768)] * 12
    lanes = plan.plan_lanes(gpt2, 5, True, 16 << 30)
    assert len(lanes) == 2 and all(len(lane) == 1 and lane[0].nmat == 24 for lane in lanes)
    idx = [sorted(lay.index for c in lane for lay in c.layouts) for lane in lanes]
    assert sorted(idx[0] + idx[1]) == list(range(48)) and not set(idx[0]) & set(idx[1])
    for lane in lanes:       # the same mix of shapes in both
        assert sorted((lay.m, lay.n) for lay in lane[0].layouts) == sorted([(768, 2304), (768, 768), (768, 3072), (768, 3072)] * 6)
        assert lane[0].update_class == 1
    assert len(plan.plan_lanes([(512, 1536), (512, 512), (512, 2048), (2048, 512)] * 24, 5, True, 16 << 30)) == 2
    assert len(plan.plan_lanes(gpt2 * 2, 5, True, 16 << 30)) == 2
    conv = [(64, 216), (256, 576), (256, 2304), (256, 2304), (512, 2304), (512, 4608), (512, 4608), (512, 4608),
            (128, 16384), (16384, 128)]
    llama = [(4096, 4096)] * 64 + [(1024, 4096)] * 64 + [(14336, 4096)] * 64 + [(4096, 14336)] * 32
    one = (conv, llama, [(4096, 4096)] * 32, gpt2[:4], gpt2 * 4,
           [(896, 2688), (896, 896), (896, 3584), (3584, 896)] * 12,            # update products in 128 x 128 tiles
           [(1024, 3072), (1024, 1024), (1024, 4096), (4096, 1024)] * 24,       # the 256 x 256 class
           [(1536, 4608), (1536, 1536), (1536, 6144), (6144, 1536)] * 8)
    for shapes in one:
        assert len(plan.plan_lanes(shapes, 5, True, 16 << 30)) == 1
    assert len(plan.plan_lanes(gpt2, 5, True, 16 << 30, allow_lanes=False)) == 1
    assert len(plan.plan_lanes(gpt2, 5, True, 64 << 20)) == 1                     # several chunks: one lane
