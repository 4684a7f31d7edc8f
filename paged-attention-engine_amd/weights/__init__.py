from .loader import WeightsError, load_weights
from .random_init import RandomWeights, random_tensor, random_weights, write_model_folder
from .safetensors_io import SafetensorsError, SafetensorsFile, save_file
