from .model_config import ConfigError, ConfigReader, DenseDecoderConfig, RopeScaling, read_config_json
from .registry import ARCHITECTURES, Architecture, architecture_of, register_architecture
