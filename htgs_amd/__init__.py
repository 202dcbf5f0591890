"""MI355X-native rasterizer for Hybrid-Transparency Gaussian Splatting (drop-in for HTGSCudaBackend)."""
from .torch_bindings import *  # noqa: F401,F403
from .torch_bindings import __all__  # noqa: F401
