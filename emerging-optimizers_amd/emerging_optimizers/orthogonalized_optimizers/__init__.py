from . import muon_utils
from .adaptive_muon import AdaptiveMuon
from .muon import Muon, get_muon_scale_factor
from .muon_hyperball import MuonHyperball
from .muon_utils import newton_schulz, newton_schulz_tp
from .orthogonalized_optimizer import OrthogonalizedOptimizer
from .polargrad import PolarGrad
from .scion import Scion
from .spectral_clipping_utils import spectral_clip, spectral_clipped_weight_decay, spectral_hardcap
from .spel import Spel

__all__ = [
    "AdaptiveMuon",
    "Muon",
    "MuonHyperball",
    "OrthogonalizedOptimizer",
    "PolarGrad",
    "Scion",
    "Spel",
    "get_muon_scale_factor",
    "muon_utils",
    "newton_schulz",
    "newton_schulz_tp",
    "spectral_clip",
    "spectral_clipped_weight_decay",
    "spectral_hardcap",
]
