"""The parts a model is put together from, and their registries."""
from .base import BuildContext, Part, part_factory, register_part, unregister_part
from . import rope, norm, attention, latent_attention, ffn, moe, block  # register the built-in parts
from . import wide_attention, gated_delta, parallel, state_space  # noqa: E402,F401
from .model import DecoderModel

__all__ = ["BuildContext", "Part", "part_factory", "register_part", "unregister_part", "DecoderModel"]
