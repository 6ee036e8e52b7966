"""MI355X-native Dynamic Grained Encoder query path (drop-in for vtpack.layers / vtpack._C)."""
from . import _lib  # noqa: F401

__version__ = "0.1.0"


def install_as_vtpack():
    """Register this package's operator module under the name the reference imports.

    After this call `from vtpack import _C` (vtpack/layers/dge.py:16, grained_sample.py:8,
    sparse_ops.py:8 of the reference) resolves to the HIP-backed module, so the reference's
    own layer and model files run unchanged on top of it.
    """
    import sys
    import types
    from . import _C
    pkg = sys.modules.get("vtpack")
    if pkg is None:
        pkg = types.ModuleType("vtpack")
        pkg.__path__ = []
        sys.modules["vtpack"] = pkg
    pkg._C = _C
    sys.modules["vtpack._C"] = _C
    return _C
