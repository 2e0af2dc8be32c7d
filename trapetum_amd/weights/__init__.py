from .loader import WeightError, check_source, load_folder, load_into   # noqa: F401
from .random_init import RandomWeights, write_model_folder   # noqa: F401
from .safetensors_io import (SafeTensorsFile, WeightFileError, WeightFolder, write_safetensors,   # noqa: F401
                             write_safetensors_streamed)
