"""Parts a model is put together from.  Importing the package registers the
built-in parts under their names."""

from tokasaurus_amd.parts import (attention, block, delta_rule, embedding, feedforward, grouped_attention, latent_attention, linear_attention, min_gru, mixer_pair,  # noqa: F401
                                   norm, position, routed_experts)
from tokasaurus_amd.parts.base import (  # noqa: F401
    BLOCKS,
    EMBEDDINGS,
    HEADS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    CacheNeed,
    CacheView,
    Normed,
    Prepared,
    PartSpec,
    StateNeed,
    StepContext,
    TensorSpec,
)
