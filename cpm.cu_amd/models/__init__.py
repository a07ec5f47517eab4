"""Model files.  Importing this package registers the built-in architectures."""
from .decoder import DecoderModel, Run, sequential_schedule
from . import minicpm
from . import duvulix
from . import gumodra
from . import sagedra
from . import nelutar
