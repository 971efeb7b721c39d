"""Typed configuration and the registries of architectures and parts."""

from tokamak_amd.config.model_config import (
    LayerCall,
    LayerSpec,
    ModelPlan,
    PartSpec,
    SubPart,
    default_order,
)
from tokamak_amd.config.registry import (
    Architecture,
    get_architecture,
    find_preset,
    get_part,
    load_model_description,
    preset_names,
    read_eos_token_ids,
    register_architecture,
    register_part,
    supported_architectures,
)

__all__ = [
    "Architecture",
    "LayerCall",
    "LayerSpec",
    "ModelPlan",
    "PartSpec",
    "SubPart",
    "default_order",
    "get_architecture",
    "find_preset",
    "get_part",
    "preset_names",
    "load_model_description",
    "read_eos_token_ids",
    "register_architecture",
    "register_part",
    "supported_architectures",
]
