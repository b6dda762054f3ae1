from .base import (FeedForward, LayerSpec, Mixer, ModelSpec, Norm, Part, PartSpec, Position, Run,
                   RunBinding, StepContext, Workspace, make_part, register_part, registered_parts,
                   unregister_part)
from . import (attention, attention_diff, attention_heads, attention_latent, attention_scored, block,   # noqa: F401
               embedding, ffn, ffn_routed, norms, position, recurrence, state_space, stream_mix)
from .linear import Linear

__all__ = ["FeedForward", "LayerSpec", "Linear", "Mixer", "ModelSpec", "Norm", "Part", "PartSpec",
           "Position", "Run", "RunBinding", "StepContext", "Workspace", "make_part",
           "register_part", "registered_parts", "unregister_part"]
