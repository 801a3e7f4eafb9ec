"""MI355X-native one-pixel point rasterizer with the entry points of ADOP's render stage.

``adop_amd._capi``  ctypes mirror of the C-ABI (``include/adop_raster.h``) and the library loader
``adop_amd.render`` host-side mirror of the reference's render interface (NeuralPointCloud, PointRendererCache,
                    NeuralRenderInfo, BlendPointCloud / PointRender)
``adop_amd.scenes`` synthetic scenes (the benchmark configurations)
"""
__version__ = "0.1.0"
