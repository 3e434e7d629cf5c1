"""optimi_amd: the fused optimizer step of optimi, hand-written for MI355X (gfx950).

Drop-in for the accelerated path of warner-benjamin/optimi: the same optimizer classes,
functional forms, gradient-release hooks and ``state_dict`` layout, with ``triton=True``
served by HIP kernels behind a C ABI (``include/optimi_hip.h``).
"""

__version__ = "0.1.0"

from .functional import adam, adamw, adan, lion, radam, ranger, sgd, stableadamw
from .gradient_release import prepare_for_gradient_release, remove_gradient_release
from .optimizers import SGD, Adam, AdamW, Adan, Lion, OptimiOptimizer, RAdam, Ranger, StableAdamW
from .utils import param_groups_weight_decay, to_low_precision

__all__ = [
    "Adam", "AdamW", "Adan", "Lion", "StableAdamW", "SGD", "RAdam", "Ranger", "OptimiOptimizer",
    "adam", "adamw", "adan", "lion", "stableadamw", "sgd", "radam", "ranger",
    "prepare_for_gradient_release", "remove_gradient_release", "param_groups_weight_decay", "to_low_precision",
]
