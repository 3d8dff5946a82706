from . import (attention, block, dense_mlp, embedding, gated_delta, hgrn2, latent_attention, mlstm, moe, norm, polynorm_mlp,
               rope, shaped_attention, side_by_side, slopes, swiglu, time_conv)  # noqa: F401  (registers the parts)
from .base import Part, build_part, part, register_part, unregister_part

__all__ = ["Part", "build_part", "part", "register_part", "unregister_part"]
