"""Import-path alias: code written against the reference (`from HTGSCudaBackend.torch_bindings import rasterize,
RasterizerSettings`, README.md:63-65 of the reference) runs on the MI355X implementation unchanged."""
from htgs_amd.torch_bindings import *  # noqa: F401,F403
from htgs_amd.torch_bindings import __all__  # noqa: F401
