from .tensors import *
from .layouts import *
from .layout_utils import *
from .gguf_interop import *
from .quantizers import *
from .theta import *
