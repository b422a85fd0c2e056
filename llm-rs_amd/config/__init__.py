from .llama import ConfigError, LlamaConfig, RopeScaling
from .gokosun import GokosunConfig
from .lilatar import LilatarConfig
from .tuvodra import TuvodraConfig
from .vivisun import VivisunConfig
from .registry import architectures, config_from_dict, load_config, register_architecture
from .spec import ExtraPart, LayerSpec, ModelSpec, PartSpec, RunSpec

__all__ = ["ConfigError", "LlamaConfig", "TuvodraConfig", "LilatarConfig", "VivisunConfig", "GokosunConfig", "RopeScaling", "architectures", "config_from_dict",
           "load_config", "register_architecture", "ExtraPart", "LayerSpec", "ModelSpec", "PartSpec", "RunSpec"]
