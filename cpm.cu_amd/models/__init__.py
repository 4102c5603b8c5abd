"""Model files.  Importing this package registers the built-in architectures."""
from .decoder import DecoderModel, Run, sequential_schedule
from . import minicpm
