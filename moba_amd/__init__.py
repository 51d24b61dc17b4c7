"""MI355X-native MoBA attention: drop-in for the reference package's public surface
(moba/__init__.py:1-11): ``MoBAConfig``, ``register_moba``, ``moba_attn_varlen``."""

from functools import partial

from .config import MoBAConfig
from .moba_efficient import moba_attn_varlen, moba_attn_varlen_gqa
from .wrapper import moba_layer

__all__ = ["MoBAConfig", "register_moba", "moba_attn_varlen", "moba_attn_varlen_gqa", "moba_layer"]


def register_moba(cfg: MoBAConfig):
    """Register the attention implementations under the reference's names
    (moba/__init__.py:9-11): "moba" (HIP kernels) and "moba_naive" (dense-mask torch ops)."""
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS

    from .moba_naive import moba_attn_varlen_naive

    ALL_ATTENTION_FUNCTIONS["moba_naive"] = partial(moba_layer, moba_attn_varlen_naive, cfg)
    ALL_ATTENTION_FUNCTIONS["moba"] = partial(moba_layer, moba_attn_varlen, cfg)
