from .rasterization import diff_rasterize, rasterize, RasterizerSettings, RasterizerMode, FrameBuffers

__all__ = ['diff_rasterize', 'rasterize', 'RasterizerSettings', 'RasterizerMode', 'FrameBuffers']
