from .safetensors_io import SafetensorsFile, SafetensorsReader, WeightError, write_safetensors
from .loader import check_checkpoint, load_weights
from .random_init import init_random_weights, random_tensor, random_tensors, write_random_model
