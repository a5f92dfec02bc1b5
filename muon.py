"""`from muon import MuonWithAuxAdam` keeps working: this module re-exports the muon_amd
implementations under the reference module's name."""
from muon_amd import (Muon, MuonWithAuxAdam, SingleDeviceMuon, SingleDeviceMuonWithAuxAdam,  # noqa: F401
                      adam_update, muon_update, ns_line_1, ns_line_2, ns_line_3, zeropower_via_aol4,
                      zeropower_via_newtonschulz5)
