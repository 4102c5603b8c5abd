from .loader import WeightError, checkpoint_files, checkpoint_names, load_tensors, stored_dtype
from .random_init import draw, random_tensors, write_model_dir
