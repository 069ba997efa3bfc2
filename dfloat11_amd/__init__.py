"""MI355X-native DFloat11 weight decompression: a drop-in for the `dfloat11`
package API (`from dfloat11_amd import DFloat11Model, compress_model`)."""
__version__ = "0.5.0"


def __getattr__(name):
    # torch and the native libraries are loaded on first use, not at import
    if name in ("DFloat11Model", "compress_model", "TensorManager", "get_hook",
                "load_and_replace_tensors", "get_no_split_classes"):
        from . import dfloat11
        return getattr(dfloat11, name)
    raise AttributeError(f"module 'dfloat11_amd' has no attribute {name!r}")
