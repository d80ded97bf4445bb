"""MI355X-native forward rasterizer for 3D Gaussian Splatting behind FlashGS's op surface.

``flashgs_amd.cabi``        ctypes binding of the C ABI (libflashgs_hip.so)
``flashgs_amd.rasterizer``  Scene / Camera / Rasterizer driver on top of ``flash_gaussian_splatting.ops``
``flashgs_amd.scenes``      deterministic synthetic scenes of the benchmark configurations
``flashgs_amd.build``       build recipe of the native parts
"""
__version__ = "0.1.0"
