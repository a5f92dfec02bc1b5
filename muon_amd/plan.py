"""Host-side planning of the grouped Newton-Schulz launches (pure numpy; no GPU needed).

A *chunk* is a set of matrices that runs through the whole Muon step together: one momentum
launch, one norm launch, one normalise launch, 3 GEMM launches per Newton-Schulz iteration and
one apply launch, however many matrices it holds.  Chunks exist only to bound the bf16
workspace; they share one workspace and run back to back on the stream.

Per matrix (m = min(rows, cols), n = max(rows, cols), padded to the chunk's GEMM tile) the
workspace holds two m x n buffers X0 and X1 (the iterate and its successor: the update product
a X + B X reads X itself as its k-major second operand, every tile of a column block reading all
rows of it, so it cannot be overwritten in place), and A, B, c*A (m x m): 2 m n + 3 m^2 elements
against the reference's A, B, C beside X (muon.py:765-767).  No transposed copy of X exists.  The
un-normalised bf16 update produced by the momentum kernel is parked in X1, which the iteration does
not touch before the normalise kernel has consumed it.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from functools import lru_cache

import numpy as np

from . import _lib

NS_COEFFS = (3.4445, -4.7750, 2.0315)   # reference muon.py:276
# per-iteration coefficients of the 4-iteration AOL-rescaled variant, reference muon.py:754-759
AOL_COEFFS = ((4.0098, -7.0585, 2.4635), (3.4585, -5.5479, 2.5959),
              (2.7573, -3.2939, 1.4254), (2.7215, -3.0494, 1.3169))
# "aol4": the Gram matrix rescaled on both sides; "aol4_rows": by rows only, as muon.py:785 writes it
VARIANTS = ("ns5", "aol4", "aol4_rows")
# The rows-only rescaling (muon.py:785 as written) is refused for matrices with a side shorter than
# this.  Dividing the rows of A by s while X is divided by sqrt(s) leaves the first polynomial with a
# matrix that is not the Gram matrix of X; for a short matrix the row sums s_i scatter enough that the
# iteration stops contracting: in float64, on Gaussian matrices whose row norms vary by +-5 %, the
# largest singular value of the result reaches 1.4 for 32 x 32, 58 for 28 x 28, 1e3 for 24 x 24 and
# 1e18 for 6 x 30, and rounding differences are amplified alike (a bf16 evaluation is up to 1.1 in
# relative Frobenius norm from the float64 one at 18 x 63), so no error bound can be stated below it.
AOL_ROWS_MIN_SIDE = 32
AOL_ROWS = 4                            # must match muon_amd_aol_rows_per_block()
TILE_DIMS = {0: (128, 128), 1: (256, 256)}   # must match muon_amd_gemm_tile_rows/cols()
# output tiles (rows, cols) of one XCD-resident super-block: as many tiles as an XCD holds workgroups
SUPER_DIMS = {0: (8, 8), 1: (4, 8)}
if os.environ.get("MUON_AMD_SUPER"):     # measurement knob: "rows,cols" of the 256 x 256 class super-block
    SUPER_DIMS[1] = tuple(int(v) for v in os.environ["MUON_AMD_SUPER"].split(","))
EW_BLOCK_ELEMS = 8192                   # must match muon_amd_elementwise_block_elems()
NT_TILE = 128                           # must match muon_amd_normalize_tile()
N_XCD = 8                               # workgroups are dealt round-robin to the 8 XCDs
RESIDENT_BIG_TILE_WORKGROUPS = 256      # one 256 x 256 workgroup per CU of an MI355X
# Workspace rows may be made this many elements longer than the padded width (a knob for
# measurements: on MI355X a power-of-two row pitch measured no slower than a padded one).
LD_PAD = int(os.environ.get("MUON_AMD_LD_PAD", "0"))
_ALIGN = 256

# X X^T and the update of an even iteration read X0 (and the update writes X1), those of an odd one X1
PH_SYRK, PH_POLY, PH_UPD_EVEN, PH_UPD_ODD, PH_UPD_LAST, PH_POLY_FULL, PH_SYRK_ODD = range(7)
N_PHASES = 7
ROWSUM_SLOT = 64                        # columns per slot of the fused row sums (the wave tile's width)


BIG_TILE_MIN_M = int(os.environ.get("MUON_AMD_BIG_TILE_MIN_M", "1024"))


def tile_class_for(m: int) -> int:
    """256 x 256 tiles once the short side is long enough to fill them; 128 x 128 tiles below."""
    return 1 if m >= BIG_TILE_MIN_M else 0


GEMM_BK = 64                            # k-block of the GEMM kernel: K and every job's K range are multiples
# (measurement knob: MUON_AMD_SPLIT = "max_m,min_kblocks,kblocks_per_job,max")
_SPLIT = [int(v) for v in os.environ.get("MUON_AMD_SPLIT", "512,32,24,16").split(",")]
SPLIT_MAX_M = _SPLIT[0]                 # X X^T of a matrix this short ...
SPLIT_MIN_KBLOCKS = _SPLIT[1]           # ... and at least this long (in k-blocks) is split ...
SPLIT_KBLOCKS_PER_JOB = _SPLIT[2]       # ... into jobs of about this many k-blocks, at most SPLIT_MAX
SPLIT_MAX = _SPLIT[3]


def split_factor(mp: int, kdim: int) -> int:
    """Into how many jobs each tile of X X^T is split along its reduction.  The rule looks at the
    matrix alone, so its result is the same bits whatever else shares the launch: a short, very
    wide matrix has a handful of tiles with thousands of k-blocks each (one tile with 256 for
    128 x 16384), which one workgroup per tile would grind through while the rest of the GPU idles."""
    kblocks = kdim // GEMM_BK
    if mp > SPLIT_MAX_M or kblocks < SPLIT_MIN_KBLOCKS:
        return 1
    return max(1, min(SPLIT_MAX, kblocks // SPLIT_KBLOCKS_PER_JOB))


def pad_unit(tile_class: int) -> int:
    return max(TILE_DIMS[tile_class])


def _round_up(x: int, q: int) -> int:
    return (x + q - 1) // q * q


@dataclass
class MatLayout:
    index: int            # position in the caller's matrix list
    rows: int
    cols: int
    m: int
    n: int
    mp: int
    np_: int
    wide: bool            # rows <= cols: X is the matrix itself; else X is its transpose
    off: dict = field(default_factory=dict)   # byte offsets of X0, X1, A, B, CA

    @property
    def ldn(self) -> int:     # leading dimension of X (rows of length np_)
        return self.np_ + LD_PAD

    @property
    def ldm(self) -> int:     # leading dimension of A, B, c*A (rows of length mp)
        return self.mp + LD_PAD

    @property
    def rows_p(self) -> int:
        return self.mp if self.wide else self.np_

    @property
    def cols_p(self) -> int:
        return self.np_ if self.wide else self.mp

    @property
    def numel(self) -> int:
        return self.rows * self.cols


def matrix_workspace_bytes(rows: int, cols: int, unit: int) -> int:
    m, n = min(rows, cols), max(rows, cols)
    mp, np_ = _round_up(m, unit), _round_up(n, unit)
    return (2 * _round_up(max(mp * (np_ + LD_PAD), np_ * (mp + LD_PAD)) * 2, _ALIGN) +
            3 * _round_up(mp * (mp + LD_PAD) * 2, _ALIGN))


UPDATE_CLASS = os.environ.get("MUON_AMD_UPDATE_CLASS", "auto")      # measurement knob: "0", "1" or "auto"


def update_class_for(tile_class: int, layouts) -> int:
    """Tile class of the update products X' = a X + B X of a chunk.  They have m x n tiles to
    spread over the GPU where the symmetric products have only m x m / 2, so a chunk of the
    128 x 128 class can afford 256 x 256 tiles for them (half the operand traffic per flop, a
    quarter of the tiles) when its padded sizes are all multiples of 256 and the larger tiles
    still give every CU one: measured on the 48 matrices of GPT-2-124M, 4 % off the update
    launches.  Which tiles compute an element does not change its bits."""
    if tile_class != 0 or UPDATE_CLASS == "0":
        return tile_class
    if any(lay.mp % 256 or lay.np_ % 256 for lay in layouts):
        return tile_class
    big_tiles = sum((lay.mp // 256) * (lay.np_ // 256) for lay in layouts)
    if UPDATE_CLASS == "auto" and big_tiles < RESIDENT_BIG_TILE_WORKGROUPS:
        return tile_class
    return 1


def matrix_scratch_bytes(rows: int, cols: int, tile_class: int, aol: bool) -> int:
    """Upper bound of what a matrix adds to a chunk's workspace besides its six bf16 buffers: the
    sums of squares of its elementwise blocks, its denominator, the fp32 slots of its split
    reductions and, for the AOL variants, its row scales and partial row sums (each rounded up to
    the alignment: the chunk rounds the first two once for all its matrices)."""
    unit = pad_unit(tile_class)
    tr, tc = TILE_DIMS[tile_class]
    m, n = min(rows, cols), max(rows, cols)
    mp, np_ = _round_up(m, unit), _round_up(n, unit)
    total = _round_up(-(-rows * cols // EW_BLOCK_ELEMS) * 4, _ALIGN) + _ALIGN
    nsplit = split_factor(mp, np_)
    if nsplit > 1:
        tiles = (mp // tr) * (mp // tr + 1) // 2 * (tr // tc) if tr != tc else (mp // tr) * (mp // tr + 1) // 2
        total += _round_up(tiles * nsplit * tr * tc * 4, _ALIGN)
    if aol:
        total += _round_up(mp * 4, _ALIGN) + _round_up(mp * (mp // ROWSUM_SLOT) * 4, _ALIGN)
    return total


@lru_cache(maxsize=256)
def _tile_order(mt: int, nt: int, sym: bool, ratio: int, super_i: int, super_j: int):
    """Tiles of an mt x nt grid in super-block order.  `ratio` = tile rows / tile cols; with sym
    only tiles whose column block (j // ratio) is on or above their row block are kept."""
    ti, tj = [], []
    for bi in range(0, mt, super_i):
        for bj in range(0, nt, super_j):
            for i in range(bi, min(bi + super_i, mt)):
                for j in range(bj, min(bj + super_j, nt)):
                    if sym and j // ratio < i:
                        continue
                    ti.append(i)
                    tj.append(j)
    return np.asarray(ti, dtype=np.int32), np.asarray(tj, dtype=np.int32)


XCD_MODE = os.environ.get("MUON_AMD_XCD_MODE", "interleave")


def xcd_permutation(njobs: int, group: int = 32) -> np.ndarray:
    """physical block b runs logical job perm[b].  Block b lands on XCD b % 8, as slot b // 8 of
    that XCD.  Consecutive groups of `group` logical jobs (one super-block: as many tiles as an XCD
    holds workgroups) are dealt round-robin to the XCDs: the workgroups resident on one XCD share
    operand panels in its L2, and the eight XCDs work on neighbouring super-blocks of the same
    matrix at the same time, so a panel one XCD pulled from HBM is found in the memory-side cache
    by the others."""
    if XCD_MODE == "segment":      # each XCD walks one contiguous eighth of the list
        seg = -(-njobs // N_XCD)
        idx = np.arange(N_XCD * seg, dtype=np.int64).reshape(N_XCD, seg).T.reshape(-1)
        return idx[idx < njobs]
    full = njobs // (N_XCD * group) * (N_XCD * group)
    perm = np.empty(njobs, dtype=np.int64)
    b = np.arange(full, dtype=np.int64)
    x, s = b % N_XCD, b // N_XCD
    perm[:full] = ((s // group) * N_XCD + x) * group + (s % group)
    # What is left over after the last whole set of eight groups still goes to the XCDs in contiguous
    # runs: block full + 8 i + x is slot i of XCD x, which takes the i-th job of its run.  (Dealing
    # whole groups and dropping the missing jobs would shift every later block to another XCD.)
    rem = njobs - full
    if rem:
        count = (rem - np.arange(N_XCD) + N_XCD - 1) // N_XCD       # blocks XCD x has in the remainder
        start = full + np.concatenate([[0], np.cumsum(count)[:-1]])
        t = np.arange(rem, dtype=np.int64)
        perm[full:] = start[t % N_XCD] + t // N_XCD
    return perm


# Cost of a job in k-blocks for balancing a launch: its reduction plus what its prologue and
# epilogue cost in the same unit (measured: about 8 us against 0.65 us per k-block for the
# 128 x 128 class, 12 us against 1.6 us for the 256 x 256 class).
JOB_FIXED_KBLOCKS = {0: 12, 1: 8}
WORKGROUPS_PER_CU = {0: 2, 1: 1}        # must match the kernels' launch bounds
N_CU = 256


def launch_imbalance(kblocks: np.ndarray, tile_class: int) -> tuple[float, float]:
    """(busiest CU, busiest XCD) over their means for a job list in launch order.  A launch has
    min(jobs, resident workgroups) workgroups; workgroup b computes jobs b, b + grid, ... and sits on
    XCD b % 8; the workgroups of an XCD fill its 32 CUs in turn, so with two workgroups per CU
    workgroups b and b + 256 share one and split its throughput."""
    cost = kblocks.astype(np.float64) + JOB_FIXED_KBLOCKS[tile_class]
    grid = min(len(cost), N_CU * WORKGROUPS_PER_CU[tile_class])
    b = np.arange(len(cost)) % grid
    cu = np.bincount(b % N_CU, weights=cost, minlength=N_CU)
    xcd = np.bincount(b % N_XCD, weights=cost, minlength=N_XCD)
    return float(cu.max() / cu.mean()), float(xcd.max() / xcd.mean())


def choose_xcd_group(kblocks: np.ndarray, tile_class: int, default: int) -> int:
    """How many consecutive jobs of the logical list go to one XCD together: the super-block (as many
    tiles as an XCD holds workgroups) unless a half or a quarter of it leaves the CUs noticeably
    better balanced.  Jobs of one launch differ in length when its matrices differ in shape (the
    list keeps same-shape matrices adjacent): GPT-2's X X^T launch has 504 jobs of 48 k-blocks, 252
    of 36 and 252 of 12 on 512 workgroup slots, and dealt in groups of 64 its busiest CU carries
    1.14 times the mean, in groups of 32 1.02 times (measured: 111 against 102 us)."""
    best, best_key = default, None
    for g in (default, default // 2, default // 4):
        cu, xcd = launch_imbalance(kblocks[xcd_permutation(len(kblocks), g)], tile_class)
        key = max(cu, xcd)
        if best_key is None or key < best_key - 0.02:     # a smaller group must earn its place
            best, best_key = g, key
    return best


WHOLE_MATRIX_GROUPS = os.environ.get("MUON_AMD_WHOLE_MATRIX_GROUPS", "1") != "0"      # measurement knob


def whole_matrix_group(tiles_per_matrix, default: int) -> int:
    """Group size for a launch of 256 x 256 tiles over matrices whose tile rows do not fill the
    super-block (3 or 5 tile rows against its 4): groups of `default` jobs then straddle super-blocks
    and matrices, and several XCDs fetch the same small B and X.  Whole matrices per XCD instead: the
    least common multiple of the matrices' tile counts, or else the largest count, when that is at
    most four super-blocks (measured on the update launches of GPT-2-124M, m = 768, groups of 108: 0.187
    -> 0.180 ms, and of m = 1280, groups of 100: 0.647 -> 0.622 ms).  Larger matrices keep the
    super-block groups: m = 1536 and 1792 (groups of 144, 147) measured the same either way, m = 2304
    (324) 2 % slower in whole matrices; matrices with 4 or 16 tile rows are best left in super-blocks."""
    counts = sorted(set(int(t) for t in tiles_per_matrix))
    for g in (int(np.lcm.reduce(counts)), max(counts)):
        if g <= 4 * default:
            return g
    return default


class ChunkPlan:
    """Layout, descriptor tables and tile job lists of one chunk."""

    def __init__(self, mats, tile_class: int, steps: int, reference_rounding: bool, variant: str = "ns5"):
        # mats: list of (index, rows, cols)
        assert variant in VARIANTS
        self.aol = variant in ("aol4", "aol4_rows")
        if self.aol:                    # fixed schedule, one rounding per stored matrix
            steps, reference_rounding = len(AOL_COEFFS), False
        self.variant = variant
        self.tile_class = tile_class
        self.tile_rows, self.tile_cols = TILE_DIMS[tile_class]
        self.tile = pad_unit(tile_class)          # padding unit of the chunk
        self.steps = steps
        self.reference_rounding = reference_rounding
        T = self.tile
        self.layouts: list[MatLayout] = []
        off = 0
        for index, rows, cols in mats:
            m, n = min(rows, cols), max(rows, cols)
            lay = MatLayout(index, rows, cols, m, n, _round_up(m, T), _round_up(n, T), rows <= cols)
            # (an m x n buffer also holds the n x m matrix of a run without iterations, in either pitch)
            xb = _round_up(max(lay.mp * lay.ldn, lay.np_ * lay.ldm) * 2, _ALIGN)
            ab = _round_up(lay.mp * lay.ldm * 2, _ALIGN)
            for name, nbytes in (("X0", xb), ("X1", xb), ("A", ab), ("B", ab), ("CA", ab)):
                lay.off[name] = off
                off += nbytes
            self.layouts.append(lay)
        self.nmat = len(self.layouts)
        # elementwise block prefix (momentum / apply) and normalise tile prefix
        nblk = [-(-lay.numel // EW_BLOCK_ELEMS) for lay in self.layouts]
        self.block_prefix = np.concatenate([[0], np.cumsum(nblk)]).astype(np.int32)
        self.nblocks = int(self.block_prefix[-1])
        ntile = [(lay.rows_p // NT_TILE) * (lay.cols_p // NT_TILE) for lay in self.layouts]
        self.tile_prefix = np.concatenate([[0], np.cumsum(ntile)]).astype(np.int32)
        self.ntiles = int(self.tile_prefix[-1])
        # scalars at the tail of the workspace
        self.off_partials = off
        off += _round_up(self.nblocks * 4, _ALIGN)
        self.off_denoms = off
        off += _round_up(self.nmat * 4, _ALIGN)
        # AOL variants: r = s^-1/2 per row of each Gram matrix, the partial row sums the first X X^T
        # launch leaves (one float per row and 64-column slot), and the block prefixes of the launches
        self.off_rvec, self.off_rowsum = [], []
        for lay in self.layouts:
            self.off_rvec.append(off)
            off += _round_up(lay.mp * 4, _ALIGN) if self.aol else 0
            self.off_rowsum.append(off)
            off += _round_up(lay.mp * (lay.mp // ROWSUM_SLOT) * 4, _ALIGN) if self.aol else 0
        rowblk = [lay.mp // AOL_ROWS for lay in self.layouts]
        self.aol_row_prefix = np.concatenate([[0], np.cumsum(rowblk)]).astype(np.int32)
        # segments of the rescaling launch per matrix: rows of X, (rows of X^T: none is kept), rows of A
        segblk = [b for lay in self.layouts for b in (lay.mp // AOL_ROWS, 0, lay.mp // AOL_ROWS)]
        self.aol_seg_prefix = np.concatenate([[0], np.cumsum(segblk)]).astype(np.int32)
        # job lists: the symmetric products share their tiles but not their reduction length
        # (X X^T reduces over n, the polynomial over m), and only the former is ever split
        self.split_slots = 0
        self.syrk_jobs = self._jobs(sym=True, reduce_over_n=True)
        self.sym_jobs = self._jobs(sym=True, reduce_over_n=False)
        # The update products may run in the 256 x 256 class where the chunk as a whole is in the
        # 128 x 128 class (see update_class_for).
        self.update_class = update_class_for(tile_class, self.layouts)
        self.full_jobs = self._jobs(sym=False, reduce_over_n=False, tile_class=self.update_class)
        # every tile of the m x m polynomial (no mirrored store): the first iteration of "aol4_rows",
        # whose Gram matrix is not symmetric after the row-only rescaling
        self.poly_full_jobs = self._jobs(sym=False, reduce_over_n=False, square=True) if variant == "aol4_rows" else None
        # fp32 slots of the split jobs (scratch like the rest; the per-slot counters are not part
        # of the workspace: they must stay zero between launches, and chunks share the workspace)
        self.off_split_partials = off
        off += _round_up(self.split_slots * self.tile_rows * self.tile_cols * 4, _ALIGN)
        self.workspace_bytes = off

    # ---- tile job lists -----------------------------------------------------------------
    def _jobs(self, sym: bool, reduce_over_n: bool, square: bool = False, tile_class: int | None = None) -> np.ndarray:
        tile_class = self.tile_class if tile_class is None else tile_class
        TR, TC = TILE_DIMS[tile_class]
        ratio = TR // TC
        si, sj = SUPER_DIMS[tile_class]
        parts = []
        for k, lay in enumerate(self.layouts):
            mt = lay.mp // TR
            nt = (lay.mp if (sym or square) else lay.np_) // TC
            ti, tj = _tile_order(mt, nt, sym, ratio, si, sj)
            kdim = lay.np_ if reduce_over_n else lay.mp
            nsplit = split_factor(lay.mp, kdim) if reduce_over_n else 1
            j = np.zeros(len(ti) * nsplit, dtype=_lib.TILE_JOB)
            j["desc"] = k
            j["i0"] = np.repeat(ti * TR, nsplit)
            j["j0"] = np.repeat(tj * TC, nsplit)
            j["diag"] = np.repeat((ti == tj // ratio).astype(np.int32), nsplit) if sym else 0
            if nsplit == 1:
                j["k1"] = kdim
            else:      # k-blocks dealt as evenly as 64-wide blocks allow; one group of slots per tile
                edges = (np.arange(nsplit + 1) * (kdim // GEMM_BK) // nsplit) * GEMM_BK
                idx = np.tile(np.arange(nsplit), len(ti))
                j["k0"], j["k1"] = edges[idx], edges[idx + 1]
                j["part_base"] = self.split_slots + np.repeat(np.arange(len(ti)) * nsplit, nsplit)
                j["split"] = idx | (nsplit << 16)
                self.split_slots += len(ti) * nsplit
            parts.append(j)
        logical = np.concatenate(parts)
        if os.environ.get("MUON_AMD_XCD_GROUP"):                        # measurement knob
            group = int(os.environ["MUON_AMD_XCD_GROUP"])
        elif tile_class == 1 and not sym and WHOLE_MATRIX_GROUPS and any((lay.mp // TR) % si for lay in self.layouts):
            group = whole_matrix_group([len(p) for p in parts], si * sj)
        else:
            group = choose_xcd_group((logical["k1"] - logical["k0"]) // GEMM_BK, tile_class, si * sj)
        return np.ascontiguousarray(logical[xcd_permutation(len(logical), group)])

    # ---- descriptor tables -----------------------------------------------------------------
    def gemm_descs(self, base: int) -> np.ndarray:
        """[N_PHASES, nmat] MuonGemmDesc table for a workspace at device address `base`."""
        d = np.zeros((N_PHASES, self.nmat), dtype=_lib.GEMM_DESC)
        for k, lay in enumerate(self.layouts):
            p = {name: base + o for name, o in lay.off.items()}
            mp, np_ = lay.mp, lay.np_
            for ph, src in ((PH_SYRK, "X0"), (PH_SYRK_ODD, "X1")):
                s = d[ph, k]
                s["P"] = s["Q"] = p[src]
                s["ldp"] = s["ldq"] = lay.ldn
                s["K"] = np_
                s["C"] = s["CT"] = p["A"]
                if self.reference_rounding:
                    s["C2"] = s["C2T"] = p["CA"]
                s["ldc"] = s["ldct"] = lay.ldm
                s["rows"] = s["colsn"] = mp
                if self.aol:                # used by the launch that carries MUON_AMD_GEMM_ROWSUM only
                    s["rowsum"] = base + self.off_rowsum[k]
                    s["ld_rowsum"] = mp // ROWSUM_SLOT
            q = d[PH_POLY, k]
            q["P"] = p["CA"] if self.reference_rounding else p["A"]
            q["Q"] = q["D"] = p["A"]
            q["ldp"] = q["ldq"] = q["ldd"] = lay.ldm
            q["K"] = mp
            q["C"] = q["CT"] = p["B"]
            q["ldc"] = q["ldct"] = lay.ldm
            q["rows"] = q["colsn"] = mp
            f = d[PH_POLY_FULL, k]      # the polynomial over every tile, stored in one orientation
            for name in _lib.GEMM_DESC.names:
                f[name] = q[name]
            f["CT"] = 0
            # X' = a X + B X: P = B (row-major along k), Q = X itself, k-major; X' goes to the other buffer
            for ph, src, dst in ((PH_UPD_EVEN, "X0", "X1"), (PH_UPD_ODD, "X1", "X0")):
                u = d[ph, k]
                u["P"] = p["B"]
                u["ldp"] = lay.ldm
                u["Q"] = u["D"] = p[src]
                u["ldq"] = u["ldd"] = lay.ldn
                u["q_kmajor"] = 1
                u["K"] = mp
                u["C"] = p[dst]
                u["ldc"] = lay.ldn
                u["rows"] = mp
                u["colsn"] = np_
            # the last update product carries the parameter step in its epilogue and stores nothing
            # itself (validate_gemm still wants an output: the buffer it would write is named)
            last = d[PH_UPD_LAST, k]
            last_src = d[PH_UPD_EVEN if (max(self.steps, 1) - 1) % 2 == 0 else PH_UPD_ODD, k]
            for name in _lib.GEMM_DESC.names:
                last[name] = last_src[name]
        return d

    def mat_descs(self, base: int) -> np.ndarray:
        """MuonMatDesc table with the workspace fields filled; tensor pointers are left zero.
        The normalise launch leaves X0 in the orientation the iteration wants: the parameter's own
        for a wide matrix (`direct`), its transpose for a tall one (`transp`); the other pointer is
        null and that orientation is not written.  Without iterations (steps = 0) the normalised
        matrix is the result and is written in the parameter's orientation either way."""
        d = np.zeros(self.nmat, dtype=_lib.MAT_DESC)
        for k, lay in enumerate(self.layouts):
            p = {name: base + o for name, o in lay.off.items()}
            r = d[k]
            r["u"] = p["X1"]
            as_param = lay.wide or self.steps == 0
            r["direct"] = p["X0"] if as_param else 0
            r["transp"] = 0 if as_param else p["X0"]
            r["result"] = p["X0"] if self.steps == 0 else 0
            r["partials"] = base + self.off_partials
            r["denom"] = base + self.off_denoms + 4 * k
            r["rows"], r["cols"] = lay.rows, lay.cols
            r["rows_p"], r["cols_p"] = lay.rows_p, lay.cols_p
            r["ld_direct"] = lay.ldn if lay.wide else lay.ldm
            r["ld_transp"] = lay.ldm if lay.wide else lay.ldn
            r["part_begin"] = self.block_prefix[k]
            r["part_end"] = self.block_prefix[k + 1]
            r["scale"] = 1.0
        return d

    def aol_descs(self, base: int) -> np.ndarray:
        """MuonAolDesc table: after the normalise launch X is in `X0` (no transposed copy: `xc` is null)."""
        d = np.zeros(self.nmat, dtype=_lib.AOL_DESC)
        for k, lay in enumerate(self.layouts):
            r = d[k]
            r["xr"] = base + lay.off["X0"]
            r["xc"] = 0
            r["gram"] = base + lay.off["A"]
            r["rvec"] = base + self.off_rvec[k]
            r["rowsum"] = base + self.off_rowsum[k]
            r["ld_rowsum"] = lay.mp // ROWSUM_SLOT
            r["m_p"], r["n_p"], r["ld_n"], r["ld_m"] = lay.mp, lay.np_, lay.ldn, lay.ldm
        return d

    def phase_scalars(self, phase: int, iteration: int = 0):
        """(alpha, beta, gamma) of the GEMM epilogue for a phase of an iteration."""
        a, b, c = AOL_COEFFS[iteration] if self.aol else NS_COEFFS
        if phase in (PH_SYRK, PH_SYRK_ODD):
            return 1.0, 0.0, c
        if phase in (PH_POLY, PH_POLY_FULL):
            return (1.0, b, 0.0) if self.reference_rounding else (c, b, 0.0)
        return 1.0, a, 0.0


def _shape_order_key(shapes, i):
    return (-tile_class_for(min(shapes[i])), -min(shapes[i]), -max(shapes[i]), -shapes[i][0], i)


LANES = os.environ.get("MUON_AMD_LANES", "auto")        # "auto", or a number of lanes to force ("1" switches them off)
LANE_UPDATE_TILES = (600, 2600)


def plan_lanes(shapes, steps: int, reference_rounding: bool, workspace_cap: int, variant: str = "ns5",
               allow_lanes: bool = True):
    """-> lanes, each a list of chunks.  Lanes have workspaces of their own and run side by side on
    streams of their own, so that the launches of one fill the CUs that the last, partly filled
    rounds of the other's leave idle (every launch is persistent: while one runs in full, the other
    lane's next launch waits for CUs and starts where they free up).

    Two lanes, each with every other matrix of the sorted list, are taken for what measured faster
    that way: one chunk of the 128 x 128 class whose update products run in 600 to 2600 tiles of
    256 x 256, a few rounds with a ragged last one (Muon part of a step: the 48 GPT-2-124M matrices
    2.07 -> 1.975 ms, 96 matrices of m = 512 1.60 -> 1.52, 96 of GPT-2's shapes 4.01 -> 3.94, 24 of them
    1.08 -> 1.08).  Everything else measured slower in two lanes and stays in one: more tiles (192
    GPT-2 shapes 7.81 -> 8.2 ms), chunks whose update products stay in 128 x 128 tiles (m = 896, 640,
    384: +4 to +20 %), the 256 x 256 class (m = 1024 and 1280 gain 2-3 % with 96 / 48 matrices and lose
    7-8 % with twice as many; m = 1536, 2048, 4096 and the Llama-3-8B matrices lose 2-14 %: two large
    kernels side by side evict each other's panels), and short launches (conv: the host then issues
    two streams' worth of them).  Three lanes measured like two, four slower.  Which lane computes a
    matrix does not change its bits."""
    chunks = plan_chunks(shapes, steps, reference_rounding, workspace_cap, variant)
    n = 1
    if allow_lanes and LANES != "auto":
        n = max(1, min(int(LANES), len(shapes)))
    elif allow_lanes and len(chunks) == 1:
        c = chunks[0]
        if (c.tile_class == 0 and c.update_class == 1 and
                LANE_UPDATE_TILES[0] <= len(c.full_jobs) <= LANE_UPDATE_TILES[1]):
            n = 2
    if n == 1:
        return [chunks]
    order = sorted(range(len(shapes)), key=lambda i: _shape_order_key(shapes, i))
    lanes = [plan_chunks(shapes, steps, reference_rounding, workspace_cap, variant, subset=order[k::n])
             for k in range(n)]
    if LANES == "auto" and any(c.update_class != chunks[0].update_class for lane in lanes for c in lane):
        return [chunks]            # half the matrices would no longer fill the larger update tiles
    return lanes


def plan_chunks(shapes, steps: int, reference_rounding: bool, workspace_cap: int, variant: str = "ns5",
                subset=None):
    """Split matrices [(rows, cols), ...] into chunks of one tile class each whose workspace (the bf16
    buffers and the scratch beside them) stays under `workspace_cap` bytes (a single matrix larger
    than the cap gets a chunk of its own).
    Same-shape matrices are kept together so that their tiles batch into full waves of the GPU.
    `subset`: positions in `shapes` to plan for (all of them when None)."""
    if variant == "aol4_rows":
        short = [tuple(sh) for sh in shapes if min(sh) < AOL_ROWS_MIN_SIDE]
        if short:
            raise ValueError(
                f"the rows-only AOL rescaling is not offered for matrices with a side below {AOL_ROWS_MIN_SIDE} "
                f"(got {short[0][0]} x {short[0][1]}): the iteration does not contract there and amplifies rounding "
                "differences without bound; use the symmetric rescaling (ns_variant='aol4', rescale='symmetric')")
    order = sorted(range(len(shapes)) if subset is None else subset, key=lambda i: _shape_order_key(shapes, i))
    need = [matrix_workspace_bytes(*shapes[i], pad_unit(tile_class_for(min(shapes[i])))) +
            matrix_scratch_bytes(*shapes[i], tile_class_for(min(shapes[i])), variant in ("aol4", "aol4_rows"))
            for i in order]
    chunks, pos = [], 0
    while pos < len(order):
        tc = tile_class_for(min(shapes[order[pos]]))
        end = pos                                          # the run of this tile class in the list
        while end < len(order) and tile_class_for(min(shapes[order[end]])) == tc:
            end += 1
        kmax, nbytes = 0, 0                                # as many of it as stay under the cap ...
        while pos + kmax < end and (kmax == 0 or nbytes + need[pos + kmax] <= workspace_cap):
            nbytes += need[pos + kmax]
            kmax += 1
        # ... cut where the launches of this chunk and of what it leaves behind fill their last rounds best
        k = kmax
        if TAIL_AWARE_CHUNKS and pos + kmax < end:         # (a run that fits one chunk stays whole)
            k = _best_cut([shapes[i] for i in order[pos:end]], need[pos:end], tc, kmax, workspace_cap)
        chunks.append(ChunkPlan([(i, *shapes[i]) for i in order[pos:pos + k]], tc, steps, reference_rounding, variant))
        pos += k
    return chunks


TAIL_AWARE_CHUNKS = os.environ.get("MUON_AMD_TAIL_AWARE_CHUNKS", "1") != "0"      # measurement knob
KBLOCK_US = {0: 0.645, 1: 1.58}         # a CU's time per k-block of its tiles (two co-resident 128 x 128 tiles share it)
CHUNK_FIXED_US = 200.0                  # what one more chunk costs: 18 more launches that fill and drain the GPU


def _chunk_time_us(mats, tile_class: int) -> tuple[float, float]:
    """(estimated, ideal) time of the fifteen GEMM launches of one iteration-set of a chunk holding
    `mats` [(rows, cols)], from the busiest CU of every launch (jobs in list order, job j on
    workgroup j % grid; see launch_imbalance).  The ideal has every CU equally busy."""
    unit = pad_unit(tile_class)
    dims = [(_round_up(min(r, c), unit), _round_up(max(r, c), unit)) for r, c in mats]
    big = (tile_class == 1 or
           (UPDATE_CLASS != "0" and all(mp % 256 == 0 and np_ % 256 == 0 for mp, np_ in dims) and
            (UPDATE_CLASS == "1" or sum((mp // 256) * (np_ // 256) for mp, np_ in dims) >= RESIDENT_BIG_TILE_WORKGROUPS)))
    est = ideal = 0.0
    T = TILE_DIMS[tile_class][0]
    for kind in ("syrk", "poly", "update"):
        tc = (1 if big else 0) if kind == "update" else tile_class
        TT = TILE_DIMS[tc][0] if kind == "update" else T
        counts, costs = [], []
        for mp, np_ in dims:
            mt = mp // TT
            if kind == "update":
                counts.append(mt * (np_ // TT)); costs.append(mp // GEMM_BK)
            else:
                kb = (np_ if kind == "syrk" else mp) // GEMM_BK
                ns = split_factor(mp, np_) if kind == "syrk" else 1
                counts.append(mt * (mt + 1) // 2 * ns); costs.append(kb // ns)
        cost = np.repeat(np.asarray(costs, dtype=np.float64) + JOB_FIXED_KBLOCKS[tc], counts)
        grid = min(len(cost), N_CU * WORKGROUPS_PER_CU[tc])
        cu = np.bincount((np.arange(len(cost)) % grid) % N_CU, weights=cost, minlength=N_CU)
        est += cu.max() * KBLOCK_US[tc]
        ideal += cost.sum() / N_CU * KBLOCK_US[tc]
    return est, ideal


def _best_cut(mats, nbytes, tile_class: int, kmax: int, cap: int) -> int:
    """How many of the first kmax matrices of the run `mats` (one tile class, in list order; `nbytes`
    their workspace needs) the next chunk takes: the count, between half of kmax and kmax, that makes
    the whole run cheapest.  A chunk costs what the busiest CU of each of its launches takes plus the
    launches themselves; what it leaves behind is charged as the chunk it would make if it fits one,
    else at 3 % over its ideal time plus the chunks its bytes need.  So a cut moves to where the
    launches fill their last rounds (51 matrices of 4096 x 14336 are 27.09 rounds of X X^T tiles on 256
    CUs, 47 of them 24.97), but never splits off a handful of matrices into launches of their own."""
    if kmax <= 2:
        return kmax
    fixed = CHUNK_FIXED_US / 5                             # per iteration, like the launch times
    best, best_cost = kmax, None
    for k in range(kmax, max(kmax // 2, 1) - 1, -1):
        est, _ = _chunk_time_us(mats[:k], tile_class)
        cost = est + fixed
        rest = mats[k:]
        if rest:
            rest_bytes = sum(nbytes[k:])
            r_est, r_ideal = _chunk_time_us(rest, tile_class)
            cost += (r_est + fixed) if rest_bytes <= cap else (r_ideal * 1.03 + fixed * rest_bytes / cap)
        if best_cost is None or cost < best_cost * 0.997:     # ties go to the larger chunk
            best, best_cost = k, cost
    return best


def adam_block_prefix(numels) -> np.ndarray:
    nblk = [-(-int(n) // EW_BLOCK_ELEMS) for n in numels]
    return np.concatenate([[0], np.cumsum(nblk)]).astype(np.int32)
