"""ctypes front end of oracle/dge_oracle.c (numpy in, numpy out).

TEST INFRASTRUCTURE ONLY.  See the header of dge_oracle.c for what each
function restates and how it is pinned.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdge_oracle.so")
_lib = None

_i64p = ctypes.POINTER(ctypes.c_int64)
_f32p = ctypes.POINTER(ctypes.c_float)


def build(force=False):
    """Compile the C checker with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libdge_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.dge_index_to_patch.restype = ctypes.c_int64
        L.dge_index_to_patch.argtypes = [_i64p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _i64p,
                                         ctypes.c_int, ctypes.c_int, ctypes.c_int, _i64p, _i64p]
        L.dge_index_to_patch_dense.restype = ctypes.c_int64
        L.dge_index_to_patch_dense.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, _i64p, ctypes.c_int,
                                               ctypes.c_int, ctypes.c_int, _i64p, _i64p]
        L.dge_compress_f32.restype = None
        L.dge_compress_f32.argtypes = [_f32p, _i64p, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                       ctypes.c_int, ctypes.c_int, _f32p]
        L.dge_decompress_f32.restype = None
        L.dge_decompress_f32.argtypes = [_f32p, _i64p, ctypes.c_int64, _f32p, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_int, ctypes.c_int, ctypes.c_int, _f32p]
        L.dge_attention_f32.restype = ctypes.c_int
        L.dge_attention_f32.argtypes = [_f32p, _f32p, _f32p, _i64p, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                        ctypes.c_int, ctypes.c_int, ctypes.c_float, _f32p]
        L.dge_sparse_gemm_f32.restype = ctypes.c_int64
        L.dge_sparse_gemm_f32.argtypes = [_f32p, _f32p, _i64p, _i64p, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                          ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          _f32p, ctypes.c_int64, ctypes.c_int64]
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _p(a, t):
    return a.ctypes.data_as(t)


def index_to_patch(indices, splits, region_size, num_extra_tokens):
    """-> (patches int64 [L,4], batch_lengths int64 [B]).  grained_sample.cu:302-345."""
    indices = _i64(indices)
    splits = _i64(splits)
    B, Hr, Wr = indices.shape
    lengths = np.zeros(B, dtype=np.int64)
    L = lib().dge_index_to_patch(_p(indices, _i64p), B, Hr, Wr, _p(splits, _i64p), len(splits),
                                 region_size, num_extra_tokens, None, _p(lengths, _i64p))
    if L < 0:
        raise ValueError("gate index outside [0, len(splits))")
    patches = np.zeros((L, 4), dtype=np.int64)
    lib().dge_index_to_patch(_p(indices, _i64p), B, Hr, Wr, _p(splits, _i64p), len(splits),
                             region_size, num_extra_tokens, _p(patches, _i64p), _p(lengths, _i64p))
    return patches, lengths


def index_to_patch_dense(indices, splits, region_size, num_extra_tokens):
    """-> (patches, batch_lengths) for every granularity.  grained_sample.cu:347-433."""
    B, Hr, Wr = np.asarray(indices).shape
    splits = _i64(splits)
    lengths = np.zeros(B, dtype=np.int64)
    L = lib().dge_index_to_patch_dense(B, Hr, Wr, _p(splits, _i64p), len(splits), region_size,
                                       num_extra_tokens, None, _p(lengths, _i64p))
    patches = np.zeros((L, 4), dtype=np.int64)
    lib().dge_index_to_patch_dense(B, Hr, Wr, _p(splits, _i64p), len(splits), region_size,
                                   num_extra_tokens, _p(patches, _i64p), _p(lengths, _i64p))
    return patches, lengths


def compress(x, patches, height, width, num_extra_tokens):
    """x [B,N,C] fp32 -> [L,C] fp32.  grained_sample.cu:31-69."""
    x = _f32(x)
    patches = _i64(patches)
    B, N, C = x.shape
    out = np.empty((patches.shape[0], C), dtype=np.float32)
    lib().dge_compress_f32(_p(x, _f32p), _p(patches, _i64p), patches.shape[0], N, C, width,
                           num_extra_tokens, _p(out, _f32p))
    return out


def decompress(inp, patches, reference, height, width, num_extra_tokens, is_add_ref, fill=np.nan):
    """inp [L,C], reference [B,N,C] -> [B,N,C].  grained_sample.cu:71-144."""
    inp = _f32(inp)
    patches = _i64(patches)
    reference = _f32(reference)
    B, N, C = reference.shape
    out = np.full((B, N, C), fill, dtype=np.float32)
    lib().dge_decompress_f32(_p(inp, _f32p), _p(patches, _i64p), patches.shape[0], _p(reference, _f32p),
                             N, C, width, num_extra_tokens, int(bool(is_add_ref)), _p(out, _f32p))
    return out


def attention(q, k, v, lengths, scale):
    """q [h,L,d], k,v [h,B,n,d], lengths [B] -> [h,L,d].  batched_sparse_gemm.cu:219-305."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    lengths = _i64(lengths)
    h, L, d = q.shape
    _, B, n, _ = k.shape
    assert int(lengths.sum()) == L and len(lengths) == B
    out = np.empty_like(q)
    rc = lib().dge_attention_f32(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(lengths, _i64p), B, h, L, n, d,
                                 float(np.float32(scale)), _p(out, _f32p))
    assert rc == 0
    return out


def sparse_gemm(a, b, a_lengths, b_lengths, is_a_transposed, is_b_transposed):
    """a [h,La,ka], b [h,Lb,kb] -> concatenated per-sample products.  batched_sparse_gemm.cu:150-195."""
    a, b = _f32(a), _f32(b)
    a_lengths, b_lengths = _i64(a_lengths), _i64(b_lengths)
    h, La, ka = a.shape
    _, Lb, kb = b.shape
    B = len(a_lengths)
    ncols = int(b_lengths[0]) if is_b_transposed else kb
    rows = B * ka if is_a_transposed else int(a_lengths.sum())
    out = np.empty((h, rows, ncols), dtype=np.float32)
    r = lib().dge_sparse_gemm_f32(_p(a, _f32p), _p(b, _f32p), _p(a_lengths, _i64p), _p(b_lengths, _i64p), B, h,
                                  La, ka, Lb, kb, int(is_a_transposed), int(is_b_transposed), _p(out, _f32p),
                                  rows, ncols)
    if r != rows:
        raise ValueError("per-sample shapes do not chain (inner dims or output widths differ)")
    return out
