"""vtdge_decompress_router_compress_static: the scatter-back that packs the next block's queries with its status
words inside the library (no device allocation in the call), against vtdge_decompress_router_compress with a
workspace from the caller - bit for bit, on two calls in a row that share the built-in array, the second smaller."""
import ctypes

import pytest
import torch

from util import SPLITS, random_indices

pytestmark = pytest.mark.gpu
EPS = 1e-6


def case(dev, B, H, W, Cc, extra, seed):
    from vtpack_amd import ops
    N = extra + H * W
    g = torch.Generator().manual_seed(seed)
    idx = torch.from_numpy(random_indices(seed, B, H // 4, W // 4)).to(dev)
    splits = torch.tensor(SPLITS, dtype=torch.int64, device=dev)
    x = (torch.randn(B, N, Cc, generator=g) * 2 + 3 * torch.randn(B, N, 1, generator=g)).bfloat16().to(dev)
    comp, _, _, offsets, _ = ops.compress_regions(x, idx, splits, H, W, 4)
    q = torch.randn(B * N, Cc, generator=g).bfloat16().to(dev)
    wgt = (torch.randn(3, Cc, generator=g) * 0.3).bfloat16().to(dev)
    bias = (torch.randn(3, generator=g) * 0.3).bfloat16().to(dev)

    def run(workspace):
        return ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=comp, next_weight=wgt, next_bias=bias,
                                     stats_eps=EPS, next_splits=splits, pack_next=True, pack_eps=EPS,
                                     workspace=workspace)
    return run


def same(got, want, B):
    total = int(want[5]["offsets"][B])
    assert total == int(got[5]["offsets"][B]) and 0 < total <= want[5]["comp"].shape[0]
    for a, b in zip(got[:4], want[:4]):
        assert torch.equal(a, b)
    regions = got[2].numel()              # the count bytes come in a buffer padded to whole 16 bytes
    assert torch.equal(got[4][:regions], want[4][:regions])
    for key in ("offsets", "region_rows"):
        assert torch.equal(got[5][key], want[5][key])
    for key in ("comp", "records", "patches"):
        assert torch.equal(got[5][key][:total], want[5][key][:total])


def test_built_in_workspace_matches_the_callers(dev):
    big = case(dev, 16, 32, 32, 384, 1, seed=5)            # 1024 regions, 256 status words
    small = case(dev, 2, 8, 8, 384, 1, seed=6)             # 8 regions, 2 status words
    want_big, want_small = big(None), small(None)
    got_big = big("static")
    got_small = small("static")                            # the array still holds the first call's words
    assert got_big[5]["workspace"] is None
    same(got_big, want_big, 16)
    same(got_small, want_small, 2)
    same(big("static"), want_big, 16)                      # and the large case after the small one


def test_built_in_workspace_has_a_limit(dev):
    from vtpack_amd import _lib
    lib = _lib.load()
    p = ctypes.c_void_p(256)                               # never dereferenced: the sizes are refused first
    args = [p] * 12 + [ctypes.c_float(EPS)] + [p] * 6 + [ctypes.c_float(EPS), p, ctypes.c_int64(1 << 30), p, p]
    rc = lib.vtdge_decompress_router_compress_static(*args, 1025, 32, 32, 384, 0, 4, 3, 3, _lib.BF16, None)
    assert rc == _lib.ERR_UNSUPPORTED
    assert b"65536" in lib.vtdge_last_error()
