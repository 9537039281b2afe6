from . import muon_utils
from .muon import Muon, get_muon_scale_factor
from .muon_utils import newton_schulz, newton_schulz_tp
from .orthogonalized_optimizer import OrthogonalizedOptimizer

__all__ = ["Muon", "OrthogonalizedOptimizer", "get_muon_scale_factor", "muon_utils", "newton_schulz", "newton_schulz_tp"]
