"""olmax_amd — MI355X-native (gfx950) implementation of OLMax's transformer training hot path.

All arithmetic lives in hand-written HIP kernels behind the C ABI of ``libolmax_hip.so``
(declared in ``include/olmax_hip.h``); this package is the thin Python host side.
"""
from .optim import AdamWConfig, ConstantSchedule, WarmupCosineDecaySchedule, WarmupStableDecaySchedule  # noqa: F401
from .transformer import Transformer, TransformerConfig, TransformerRecipe  # noqa: F401
from .train import Trainer  # noqa: F401
from . import data  # noqa: F401,E402
