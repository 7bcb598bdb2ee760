from .format import CheckpointReader
from .loader import Loader
from .saver import Saver

__all__ = ["Saver", "Loader", "CheckpointReader"]
