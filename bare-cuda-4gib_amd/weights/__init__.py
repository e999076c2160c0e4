from .safetensors_io import SafetensorsFile, SafetensorsWriter, open_model_tensors  # noqa: F401
from .loader import WeightSpec, load_weights  # noqa: F401
from .random_init import write_random_model  # noqa: F401
