from .model import LayerSpec, Model, ModelSpec, ScheduleEntry, build_layer
from .dense_decoder import dense_decoder_spec
