"""MI355X-native fused linear + cross-entropy loss (drop-in for ``linear_cross_entropy``)."""
from .ops import fwd_configs, bwd_configs, LinearCrossEntropyLoss, linear_cross_entropy, LinearXentImplementation

__all__ = ["fwd_configs", "bwd_configs", "LinearCrossEntropyLoss", "linear_cross_entropy",
           "LinearXentImplementation"]
