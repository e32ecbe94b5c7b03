from .generate import generate, plan_batches  # noqa: F401
from .model import DecoderModel, LayerBinding, require_gpu  # noqa: F401
from .step import Engine, StepContext, StepEntry, StepError  # noqa: F401
