"""MI355X-native drop-in for sharktank's quantized mixture-of-experts layer path."""

from . import types, ops, layers
from ._hip import load_library, library_path
