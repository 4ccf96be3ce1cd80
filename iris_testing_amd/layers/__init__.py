"""Layer-level operators with the reference's call signatures (layers/all_to_all.py,
layers/token_shuffle.py, layers/expert.py) plus the two the path needs that the reference lacks
(expert MLP, combine)."""
from .all_to_all import custom_a2a, SimulatedWorld, simulated_world  # noqa: F401
from .token_shuffle import shuffle  # noqa: F401
from .expert import expert, expert_mlp, ExpertWeights  # noqa: F401
from .combine import combine, pack_fixed_m  # noqa: F401
