from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec
from .registry import (Architecture, architecture_name, load_config, lookup, read_config_json,
                       register_architecture, registered_architectures)
from .qwen2 import ConfigError, Qwen2Config, qwen2_model_spec

from .qwen2 import QWEN2_WEIGHT_ALIASES

register_architecture("Qwen2ForCausalLM", Qwen2Config.from_dict, qwen2_model_spec, aliases=("qwen2",),
                      weight_aliases=QWEN2_WEIGHT_ALIASES)

from .tovasun import TovasunConfig, tovasun_model_spec

register_architecture("Tovasun", TovasunConfig.from_dict, tovasun_model_spec, aliases=("tovasun",))

from .sogenex import SogenexConfig, sogenex_model_spec

register_architecture("Sogenex", SogenexConfig.from_dict, sogenex_model_spec, aliases=("sogenex",))

from .nusuvik import NusuvikConfig, nusuvik_model_spec

register_architecture("Nusuvik", NusuvikConfig.from_dict, nusuvik_model_spec, aliases=("nusuvik",))

from .kufolorn import KufolornConfig, kufolorn_model_spec

register_architecture("Kufolorn", KufolornConfig.from_dict, kufolorn_model_spec, aliases=("kufolorn",))

__all__ = ["KufolornConfig", "kufolorn_model_spec", "NusuvikConfig", "nusuvik_model_spec", "TovasunConfig", "tovasun_model_spec", "SogenexConfig", "sogenex_model_spec", "ExecEntry", "LayerSpec", "ModelSpec", "PartSpec", "Architecture", "architecture_name",
           "load_config", "lookup", "read_config_json", "register_architecture",
           "registered_architectures", "ConfigError", "Qwen2Config", "qwen2_model_spec"]
