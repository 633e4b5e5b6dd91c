from .spec import PartSpec, SubLayerSpec, LayerSpec, ScheduleEntry, ModelSpec, ConfigError
from .llama import LlamaConfig
from .manirax import ManiraxConfig
from .risonex import RisonexConfig
from .dupolorn import DupolornConfig
from .favizen import FavizenConfig

__all__ = ["PartSpec", "SubLayerSpec", "LayerSpec", "ScheduleEntry", "ModelSpec", "ConfigError", "LlamaConfig", "ManiraxConfig", "RisonexConfig", "DupolornConfig", "FavizenConfig"]
