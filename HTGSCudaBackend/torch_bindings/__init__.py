from htgs_amd.torch_bindings import *  # noqa: F401,F403
from htgs_amd.torch_bindings import __all__  # noqa: F401
