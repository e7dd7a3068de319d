from .loader import CheckpointError, load_checkpoint
from .random_init import draw_all, write_model_folder
from .safetensors_io import SafetensorsError, SafetensorsFile, open_checkpoint, write_safetensors
from .spec import ParamSpec

__all__ = ["CheckpointError", "load_checkpoint", "draw_all", "write_model_folder", "SafetensorsError",
           "SafetensorsFile", "open_checkpoint", "write_safetensors", "ParamSpec"]
