from .base import ConfigError, ModelConfig, architecture_name, field_from, read_config_json, require
from .minicpm import MiniCPMConfig, RopeScaling, SparseConfig
from .duvulix import DuvulixConfig
from .gumodra import GumodraConfig
from .sagedra import SagedraConfig
from .nelutar import NelutarConfig
