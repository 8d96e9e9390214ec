"""Architectures: each module registers itself under the names its config.json uses."""
from . import bitonex, digasun, fuvirax, girelix, llama  # noqa: F401
from .plan import LayerPlan, ModelPlan, Place  # noqa: F401
