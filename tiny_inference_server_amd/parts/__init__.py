"""Parts that layers are put together from: norms, position encodings, mixers, feed-forwards,
block arrangements and stage inputs. Importing this package registers the built-in kinds."""
from .base import (ARRANGEMENTS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, STAGE_INPUTS, Arrangement, CallContext,
                   Tensors, build_part, expected_tensors, part_class, to_compute, to_gain)
from .spec import LayerCall, LayerSpec, ModelSpec, PagedKvNeed, PartSpec, StageSpec, StateNeed
from . import attention, block, feed_forward, norm, position, stage_input  # noqa: F401  (registration)
