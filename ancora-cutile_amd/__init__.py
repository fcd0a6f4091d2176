"""MI355X-native Muon + AdamW optimizer step: drop-in for ancora/optim of
MythosAd/ancora-cutile. Pure Python + numpy on the host, hand-written gfx950 HIP kernels
behind a ctypes-loaded C ABI (include/anc_optim.h). No PyTorch, no CPU fallback.

Import name: `ancora_cutile_amd` (the directory `ancora-cutile_amd/` is not a valid
Python identifier; the sibling package `ancora_cutile_amd/` points its search path here).
"""
from .devbuf import DevBuf                                                   # noqa: F401
from .adamw import AdamW, _adamw, _pick_otm, C                               # noqa: F401
from .gradnorm import StepGuard                                              # noqa: F401
from .muon_ns import (newton_schulz_resident, newton_schulz_resident_e, ns_fp32_batched,  # noqa: F401
                      set_polar_express, PE_SCHEDULE, A_COEF, B_COEF, C_COEF, NTM, NTN, NTK)
from .muon import (Muon, DeviceMuon, MuonScratch, ResidentMuon, BatchedProjMuon,  # noqa: F401
                   newton_schulz5)
from .moe import ExpertMuonScratch, ExpertOptimizer, GroupedMoEFFNOptim                          # noqa: F401
from .hybrid import HybridOptimizer, default_is_muon, resident_is_muon       # noqa: F401
from .quant import Mxfp8WeightCache, quant_mxfp8_w                          # noqa: F401
from .grads import gemm_dW, transpose_acts, DwWorkspace                       # noqa: F401
