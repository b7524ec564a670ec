from .loader import (MemoryBudgetError, WeightArena, WeightError, WeightSpec, check_names, device_budget,
                     load_weights, open_model_folder, plan_arena, stacked)
from .random_init import random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["MemoryBudgetError", "WeightArena", "device_budget", "plan_arena", "stacked", "WeightError", "WeightSpec", "check_names", "load_weights", "open_model_folder",
           "random_tensors", "write_random_model", "SafetensorsError", "SafetensorsFile",
           "write_safetensors"]
