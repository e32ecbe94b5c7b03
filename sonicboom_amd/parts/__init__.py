"""Parts a model is assembled from; importing the package registers the built-in kinds."""
from .base import (CATEGORIES, KVSpec, Mixer, Part, RowsSpec, Runtime, StateSpec, build_part,  # noqa: F401
                   register_part, registered_parts)
from .spec import ModelSpec, OrderEntry, PartSpec, TensorSpec  # noqa: F401
from . import attention, block, embedding, ffn, norm, position  # noqa: F401
