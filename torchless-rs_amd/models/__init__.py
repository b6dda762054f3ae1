"""Architectures: each module registers a name from config.json's
`architectures` with its configuration class and its `ModelSpec` builder."""
from ..config.base import ModelConfig, get_architecture
from ..parts import base as _parts_base
from .. import parts as _parts            # registers the parts
from . import mistral as _mistral         # registers MistralForCausalLM
from . import sozetar as _sozetar         # registers Sozetar
from . import fanitar as _fanitar         # registers Fanitar
from . import nepisun as _nepisun         # registers Nepisun
from . import giforax as _giforax         # registers Giforax


def model_spec_for(cfg: ModelConfig):
    return get_architecture(cfg.architecture).build_spec(cfg)
