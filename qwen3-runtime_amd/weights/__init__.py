from .loader import WeightError, WeightLoader, check_source, load_model  # noqa: F401
from .source import RandomSource, SafetensorsSource, write_model_folder  # noqa: F401
