"""muon_amd -- the Muon optimizer step for AMD Instinct MI355X (gfx950).

Drop-in for the single-GPU surface of the reference `muon` module: the same class and function
names, argument order, defaults and optimizer state keys, with the device work done by
hand-written HIP kernels in libmuon_amd.so (see include/muon_amd.h for its C ABI).
"""
from .functional import (adam_update, clear_engine_cache, muon_update, zeropower_via_aol4,
                         zeropower_via_newtonschulz5)
from .ops import ns_line_1, ns_line_2, ns_line_3
from .optim import Muon, MuonWithAuxAdam, SingleDeviceMuon, SingleDeviceMuonWithAuxAdam
from ._lib import MuonAmdError

__all__ = [
    "Muon", "SingleDeviceMuon", "MuonWithAuxAdam", "SingleDeviceMuonWithAuxAdam",
    "zeropower_via_newtonschulz5", "zeropower_via_aol4", "muon_update", "adam_update", "clear_engine_cache",
    "ns_line_1", "ns_line_2", "ns_line_3",
    "MuonAmdError",
]
