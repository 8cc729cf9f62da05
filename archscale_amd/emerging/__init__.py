"""Mirror of the reference's ``emerging_optimizers.orthogonalized_optimizers`` Muon family for MI355X."""
from .mixin import WeightDecayMixin, WeightDecayT  # noqa: F401
from .muon import Muon, get_muon_scale_factor  # noqa: F401
from .muon_ball import MuonBall  # noqa: F401
from .muon_utils import newton_schulz, newton_schulz_step_tsyrk  # noqa: F401
from .orthogonalized_optimizer import OrthogonalizedOptimizer  # noqa: F401
from .spectral_ball_utils import (apply_retract, compute_target_radius, get_spectral_ball_scale_factor, msign,  # noqa: F401
                                  power_iteration, spectral_norm)
