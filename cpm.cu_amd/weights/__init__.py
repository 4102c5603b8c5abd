from .loader import WeightError, checkpoint_files, checkpoint_names, load_tensors, stored_dtype
from .random_init import INIT_RULES, draw, random_tensors, register_init_rule, write_model_dir
