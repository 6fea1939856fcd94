from .spec import PartSpec, LayerSpec, ScheduleEntry, ModelSpec, default_schedule, prenorm_layer
from .registry import (Architecture, register_architecture, unregister_architecture,
                       registered_architectures, architecture_of, architecture_of_config,
                       read_config_json, config_from_dict, config_from_folder, spec_of, generation_stop_tokens)
from .mistral import MistralConfig, PRESETS, preset, build_spec as build_mistral_spec, ARCHITECTURE as MISTRAL
from .kesitar import KesitarConfig, build_spec as build_kesitar_spec, ARCHITECTURE as KESITAR
from .sidirax import SidiraxConfig, build_spec as build_sidirax_spec, ARCHITECTURE as SIDIRAX
from .zivovik import ZivovikConfig, build_spec as build_zivovik_spec, ARCHITECTURE as ZIVOVIK
from .ladadra import LadadraConfig, build_spec as build_ladadra_spec, ARCHITECTURE as LADADRA
from . import kesitar as _kesitar
from . import ladadra as _ladadra
from . import zivovik as _zivovik
from . import sidirax as _sidirax

register_architecture(MISTRAL, MistralConfig, build_mistral_spec, model_type="mistral", replace=True)
register_architecture(KESITAR, KesitarConfig, build_kesitar_spec, model_type="kesitar", replace=True)
register_architecture(SIDIRAX, SidiraxConfig, build_sidirax_spec, model_type="sidirax", replace=True)
register_architecture(ZIVOVIK, ZivovikConfig, build_zivovik_spec, model_type="zivovik", replace=True)
register_architecture(LADADRA, LadadraConfig, build_ladadra_spec, model_type="ladadra", replace=True)
PRESET_FAMILIES = {MISTRAL: (PRESETS, preset), KESITAR: (_kesitar.PRESETS, _kesitar.preset),
                   SIDIRAX: (_sidirax.PRESETS, _sidirax.preset), ZIVOVIK: (_zivovik.PRESETS, _zivovik.preset),
                   LADADRA: (_ladadra.PRESETS, _ladadra.preset)}


def any_preset(name: str, **overrides):
    """A preset of any registered architecture by its name."""
    for presets, make in PRESET_FAMILIES.values():
        if name in presets:
            return make(name, **overrides)
    from ..errors import ConfigError
    raise ConfigError(f"unknown preset {name!r}; known: {sorted(n for p, _ in PRESET_FAMILIES.values() for n in p)}")

__all__ = [
    "PartSpec", "LayerSpec", "ScheduleEntry", "ModelSpec", "default_schedule", "prenorm_layer",
    "Architecture", "register_architecture", "unregister_architecture", "registered_architectures",
    "architecture_of", "architecture_of_config", "read_config_json", "config_from_dict",
    "config_from_folder", "spec_of", "generation_stop_tokens", "MistralConfig", "PRESETS", "preset",
    "KesitarConfig", "SidiraxConfig", "ZivovikConfig", "LadadraConfig", "any_preset", "PRESET_FAMILIES",
]
