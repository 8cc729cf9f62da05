"""Mirror of the reference's ``emerging_optimizers.orthogonalized_optimizers`` Muon family for MI355X."""
from .mixin import WeightDecayMixin, WeightDecayT  # noqa: F401
from .muon import Muon, get_muon_scale_factor  # noqa: F401
from .muon_utils import newton_schulz  # noqa: F401
from .orthogonalized_optimizer import OrthogonalizedOptimizer  # noqa: F401
from .spectral_ball_utils import msign  # noqa: F401
