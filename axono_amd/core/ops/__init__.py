from .llm import add, linear, linear_nobias, rms_norm
from .sequence import (argmax, concat, embedding, mrope_cos_sin, rope, rope_thd, rope_with_cos_sin,
                       scaled_dot_product_attention, slice_)

__all__ = ["add", "linear", "linear_nobias", "rms_norm", "argmax", "concat", "embedding", "mrope_cos_sin", "rope",
           "rope_thd", "rope_with_cos_sin", "scaled_dot_product_attention", "slice_"]
