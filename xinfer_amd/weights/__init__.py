from .safetensors_io import SafetensorsFile, write_safetensors
from .store import RandomStore, SafetensorsStore, TensorDecl, WeightError, WeightStore
from .random_init import write_random_model
