"""MI355X-native fused gated MLP with the import surface of matteobonotto/triton-gated-mlp."""

from . import const, gated_mlp, utils  # noqa: F401
from .gated_mlp import (  # noqa: F401
    ACT_FWD,
    EagerGatedMLP,
    FusedGatedMLP,
    FusedGatedMLPFullFunction,
    FusedGatedMLPFunction,
    eager_bwd,
    eager_fwd,
    mlp_hidden_states_bwd,
    mlp_hidden_states_fwd,
)
from .utils import copy_weights, get_device  # noqa: F401
