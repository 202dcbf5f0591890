from .rasterization import diff_rasterize, rasterize, update_max_weights, RasterizerSettings, RasterizerMode, FrameBuffers

__all__ = ['diff_rasterize', 'rasterize', 'update_max_weights', 'RasterizerSettings', 'RasterizerMode', 'FrameBuffers']
