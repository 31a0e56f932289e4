"""keops_amd: MI355X-native backend for KeOps-style tiled map-reduce (Genred / LazyTensor API)."""
__version__ = "0.1.0"
