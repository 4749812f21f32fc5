"""Parts of a layer (mixer, feed-forward, norm, position encoding, block) and their registries."""
from .base import (FeedForward, LayerCache, Mixer, Norm, Part, PositionEncoding, RowTransform, StepContext, block_class,
                   feed_forward_class, mixer_class, norm_class, position_class, register_block, register_feed_forward,
                   register_mixer, register_norm, register_position_encoding, register_row_transform, row_transform_class,
                   weight_bytes, weight_tensors)
from . import norm, rope, attention, mlp, block, transform          # registers the built-in kinds
from .linear import linear, linear_onto
from .attention import qkv_rotate_store_attend
from ..weights.loader import TensorNeed


def model_tensor_needs(spec):
    """Every tensor a model of this spec reads, in the model's own order."""
    needs = [TensorNeed(spec.embedding, (spec.vocab_size, spec.hidden_size))]
    for layer in spec.layers:
        needs += block_class(layer.block).tensor_needs(layer)
    needs += norm_class(spec.final_norm).tensor_needs(spec.final_norm)
    needs.append(TensorNeed(spec.lm_head, (spec.vocab_size, spec.hidden_size)))
    return needs
