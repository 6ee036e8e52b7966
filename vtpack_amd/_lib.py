"""ctypes binding of libvtdge.so (the C ABI declared in include/vtdge.h).

The library is loaded lazily on first use and the load fails loudly: there is
no CPU or PyTorch fallback for any operator of this package.
"""
import ctypes
import os
import subprocess

import torch  # noqa: F401  (loaded first so that libvtdge binds to the HIP runtime torch already holds)

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("VTDGE_LIB", os.path.join(_PKG, "libvtdge.so"))   # override: kernel experiments only
CSRC = os.path.join(_PKG, "csrc")

F32, BF16 = 0, 1
ACT_NONE, ACT_GELU = 0, 1
ERR_ARG, ERR_UNSUPPORTED, ERR_LAUNCH = -1, -2, -3      # include/vtdge.h
MAX_SPLITS = 8

_p = ctypes.c_void_p
_i = ctypes.c_int
_l = ctypes.c_int64
_f = ctypes.c_float

# name -> argtypes, in the order of include/vtdge.h
SIGNATURES = {
    "vtdge_router": [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_router_layernorm": [_p, _p, _p, _p, _p, _p, _p, _f, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_index_to_patch": [_p, _p, _i, _i, _i, _i, _i, _i, _p, _l, _p, _p, _p],
    "vtdge_index_to_patch_dense": [_p, _i, _i, _i, _i, _i, _i, _p, _p],
    "vtdge_compress": [_p, _p, _p, _l, _p, _p, _p, _p, _f, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_decompress": [_p, _p, _p, _p, _l, _p, _p, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_decompress_layernorm": [_p, _p, _p, _p, _l, _p, _p, _p, _p, _p, _f, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_decompress_router": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _f, _p, _p, _p, _p, _i, _i, _i, _i,
                                _i, _i, _i, _i, _i, _p],
    "vtdge_decompress_router_compress": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _f, _p, _p, _p, _p,
                                         _p, _p, _f, _p, _l, _p, _p, _p, _l, _i,
                                         _i, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_decompress_router_compress_static": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _f, _p, _p, _p, _p,
                                                _p, _p, _f, _p, _l, _p, _p,
                                                _i, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_router_stats": [_p, _p, _p, _p, _p, _p, _p, _f, _p, _p, _p, _l, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_compress_regions": [_p, _p, _p, _p, _p, _p, _f, _p, _l, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_layernorm": [_p, _p, _p, _p, _p, _l, _i, _f, _i, _p],
    "vtdge_patch_embed_norm": [_p, _p, _p, _p, _p, _f, _p, _p, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_layernorm_add": [_p, _p, _p, _p, _l, _p, _l, _i, _f, _i, _p],
    "vtdge_layernorm_rows": [_p, _l, _i, _p, _p, _p, _l, _i, _f, _i, _p],
    "vtdge_linear": [_p, _l, _p, _p, _p, _l, _p, _l, _p, _l, _i, _i, _i, _i, _p],
    "vtdge_patch_embed": [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_patch_linear": [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p],
    "vtdge_linear_packed_size": [_i, _i, _i, _p],
    "vtdge_linear_prepack": [_p, _i, _i, _i, _p, _p],
    "vtdge_linear_prepacked": [_p, _l, _p, _p, _p, _p, _l, _p, _l, _p, _l, _i, _i, _i, _i, _p],
    "vtdge_linear_stats": [_p, _l, _p, _p, _p, _p, _l, _p, _l, _p, _f, _p, _l, _i, _i, _i, _p],
    "vtdge_layernorm_stats": [_p, _p, _p, _l, _i, _f, _i, _p],
    "vtdge_layernorm_fold": [_p, _p, _p, _p, _i, _i, _i, _p, _p, _p],
    "vtdge_linear_layernorm": [_p, _l, _p, _p, _p, _p, _p, _l, _p, _l, _i, _i, _i, _i, _p],
    "vtdge_linear_layernorm_pair": [_p, _l, _p, _p, _p, _p, _p, _l, _p, _l, _i, _p, _l, _p, _p, _p, _p, _p, _l, _p, _l,
                                    _i, _i, _i, _p],
    "vtdge_sparse_attention": [_p, _l, _l, _p, _p, _l, _l, _l, _p, _p, _l, _l, _i, _i, _i, _i, _i, _f, _i, _p],
    "vtdge_batched_sparse_gemm": [_p, _p, _p, _p, _p, _i, _i, _l, _i, _l, _i, _i, _i, _l, _l, _l, _i, _p],
}
EXPORTS = ["vtdge_version", "vtdge_last_error", "vtdge_last_kernel"] + list(SIGNATURES)

_lib = None


class VtdgeError(RuntimeError):
    """A libvtdge entry point returned a negative status."""


def build(verbose=False):
    """Compile every kernel for gfx950 with hipcc (cross-compiles without a GPU)."""
    cmd = ["make", "-B", "-j8", "-C", CSRC]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout[-4000:])
        print(res.stderr[-4000:])
    if res.returncode != 0:
        raise RuntimeError("building libvtdge.so failed")
    return LIB_PATH


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP kernels are not built. Run `make -C {CSRC}` "
            "(or __graft_entry__.build()); this package has no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    lib.vtdge_version.restype = _i
    lib.vtdge_version.argtypes = []
    lib.vtdge_last_error.restype = ctypes.c_char_p
    lib.vtdge_last_error.argtypes = []
    lib.vtdge_last_kernel.restype = ctypes.c_char_p
    lib.vtdge_last_kernel.argtypes = []
    lib.vtdge_decompress_router_compress_workspace.restype = _l
    lib.vtdge_decompress_router_compress_workspace.argtypes = [_i, _i, _i, _i]
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = _i
        fn.argtypes = args
    _lib = lib
    return lib


# Optional per-launch timer (benchmarks only): an object with begin(name, tag) / end(); None = off.
timer = None


def call(name, *args, tag=None):
    lib = load()
    if timer is not None:
        timer.begin(name, tag)
    rc = getattr(lib, name)(*args)
    if timer is not None:
        timer.end()
    if rc != 0:
        msg = lib.vtdge_last_error().decode("utf-8", "replace")
        raise VtdgeError(f"{name} failed ({rc}): {msg}")


def last_kernel():
    """Name of the kernel the latest libvtdge launch of this thread was, as rocprofv3 lists it (without the
    namespace and the argument list)."""
    name = load().vtdge_last_kernel().decode("utf-8", "replace")
    if name.startswith("void "):
        name = name[5:]
    depth, cut = 0, len(name)
    for i, ch in enumerate(name):            # the argument list opens at the first '(' outside the template brackets
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0:
            cut = i
            break
    name = name[:cut]
    return name[len("vtdge::"):] if name.startswith("vtdge::") else name


def dtype_code(t):
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise TypeError(f"vtdge kernels are built for float32 and bfloat16, got {t.dtype}")


def stream_ptr():
    return torch.cuda.current_stream().cuda_stream


def ptr(t):
    return 0 if t is None else t.data_ptr()
