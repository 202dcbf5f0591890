from .rasterization import rasterize, RasterizerSettings, RasterizerMode, FrameBuffers

__all__ = ['rasterize', 'RasterizerSettings', 'RasterizerMode', 'FrameBuffers']
