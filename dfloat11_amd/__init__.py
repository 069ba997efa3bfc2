"""MI355X-native DFloat11 weight decompression (drop-in for the `dfloat11` package API)."""
__version__ = "0.5.0"
