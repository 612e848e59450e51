from .safetensors_io import SafetensorsFile, SafetensorsError, save_file
from .loader import TensorDecl, WeightsError, load_weights, WEIGHTS_FILE
from .random_init import write_random_model, random_tensor
