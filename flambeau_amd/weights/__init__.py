from .loader import SafetensorsDir, WeightError, check_against_manifest, load_weights
from .random_init import RandomSource, write_random_model
from .safetensors_io import SafetensorsFile, TensorInfo, WeightFileError, write_safetensors
