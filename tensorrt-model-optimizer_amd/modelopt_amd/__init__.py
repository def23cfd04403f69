"""MI355X-native ModelOpt quantization hot path (gfx950 HIP kernels behind the ModelOpt API)."""

__version__ = "0.1.0"
