"""Layer parts. Importing this package registers the shipped kinds."""

from . import attention, block, embedding, mlp, norm, rope  # noqa: F401
from .base import (  # noqa: F401
    Block,
    CacheView,
    FeedForward,
    GroupView,
    Mixer,
    Norm,
    Part,
    PositionEncoding,
    StepContext,
    StepCost,
)
from .model import DecoderModel, build_part  # noqa: F401
from .plan import CacheSpec, LayerSpec, ModelPlan, PagedStream, PartSpec, RunStep, TensorDecl  # noqa: F401
