"""numml_amd: MI355X (gfx950) backend for numml's differentiable sparse-CSR path."""
from . import numml_torch_cpp  # noqa: F401
from . import _binding  # noqa: F401
from ._binding import install, load_compiled  # noqa: F401
from . import sparse  # noqa: F401

__version__ = "0.1.0"
