"""MI355X-native (gfx950) low-rank decode path: hand-written HIP kernels behind a C ABI
(libflashsvd_hip.so), exposed through the operator names of the FlashSVD Python runtime."""
__version__ = "0.1.0"
