"""Pins for the CPU oracle (oracle/dge_oracle.c, oracle/torch_ref.py).  No GPU needed.

The reference ships no tests, fixtures or golden vectors for this path, and its own implementation
is CUDA only, so each oracle function is held in place by something it does not itself compute:
a hand-worked example, the reference's own *dense* closed forms (vtpack/layers/grained_sample.py:126-177,
written here with torch library routines), algebraic invariants (partition of the grid, adjointness,
round trips) and float64 library evaluations.  A dropped term, a wrong sign, a swapped y/x or a
transposed operand fails at least one of these.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import dge_oracle as orc
from oracle import torch_ref
from util import SPLITS, randn, random_indices, rng

R = 4


# ------------------------------------------------------------------ index -> patch
def test_index_to_patch_worked_example():
    # one 4x4 region, gate index 1 -> 2x2 sub-patches of 2x2 tokens, one class token
    p, l = orc.index_to_patch(np.array([[[1]]]), SPLITS, R, 1)
    assert l.tolist() == [5]
    assert p.tolist() == [[0, -1, 0, 1], [0, 0, 0, 2], [0, 0, 2, 2], [0, 2, 0, 2], [0, 2, 2, 2]]
    # two regions side by side, finest then coarsest; y is column 1, x is column 2
    p, l = orc.index_to_patch(np.array([[[2, 0]]]), SPLITS, R, 0)
    assert l.tolist() == [17]
    assert p[0].tolist() == [0, 0, 0, 4]
    assert p[1].tolist() == [0, 0, 4, 1] and p[2].tolist() == [0, 0, 5, 1] and p[5].tolist() == [0, 1, 4, 1]
    assert p[16].tolist() == [0, 3, 7, 1]


@pytest.mark.parametrize("B,Hr,Wr,extra,splits", [(6, 4, 4, 1, [4, 2, 1]), (3, 2, 5, 0, [4, 2, 1]),
                                                    (4, 8, 8, 2, [4, 2, 1]), (5, 3, 3, 1, [2, 1])])
def test_index_to_patch_invariants(B, Hr, Wr, extra, splits):
    Rr = max(splits)
    H, W = Hr * Rr, Wr * Rr
    idx = random_indices(B + Hr, B, Hr, Wr, S=len(splits))
    p, l = orc.index_to_patch(idx, splits, Rr, extra)
    ps = np.array(splits)[idx]
    # per-sample query counts: closed form
    assert np.array_equal(l, extra + (ps ** 2).reshape(B, -1).sum(1))
    assert p.shape == (l.sum(), 4)
    # windows partition the token grid: every token of every sample is covered exactly once
    cover = np.zeros((B, extra + H * W), dtype=np.int64)
    for b, y0, x0, s in p:
        if y0 < 0:
            assert s == 1
            cover[b, -y0 - 1] += 1
        else:
            assert y0 % s == 0 and x0 % s == 0
            for dy in range(s):
                for dx in range(s):
                    cover[b, (y0 + dy) * W + x0 + dx + extra] += 1
    assert (cover == 1).all()
    # sum of window areas per sample = number of tokens
    area = np.where(p[:, 1] < 0, 1, p[:, 3] ** 2)
    assert np.array_equal(np.bincount(p[:, 0], weights=area, minlength=B), np.full(B, extra + H * W))
    # ordering: sample-major; extras first; regions row-major; sub-patches row-major
    key = []
    for b, y0, x0, s in p:
        if y0 < 0:
            key.append((b, 0, -y0 - 1, 0, 0))
        else:
            key.append((b, 1, (y0 // Rr) * Wr + x0 // Rr, y0 % Rr, x0 % Rr))
    assert key == sorted(key) and len(set(key)) == len(key)
    # each region carries the window size its gate index selects
    for b, y0, x0, s in p:
        if y0 >= 0:
            assert s == Rr // ps[b, y0 // Rr, x0 // Rr]


def test_index_to_patch_uniform_gates():
    B, Hr, Wr = 2, 4, 4
    fine, lf = orc.index_to_patch(np.zeros((B, Hr, Wr), dtype=np.int64), SPLITS, R, 1)
    coarse, lc = orc.index_to_patch(np.full((B, Hr, Wr), 2, dtype=np.int64), SPLITS, R, 1)
    assert lf.tolist() == [257, 257] and lc.tolist() == [17, 17]
    assert (fine[fine[:, 1] >= 0, 3] == 1).all() and (coarse[coarse[:, 1] >= 0, 3] == 4).all()


def test_index_to_patch_rejects_bad_gate():
    with pytest.raises(ValueError):
        orc.index_to_patch(np.array([[[3]]]), SPLITS, R, 1)


def test_index_to_patch_dense_closed_form():
    B, Hr, Wr, extra = 2, 2, 3, 1
    p, l = orc.index_to_patch_dense(np.zeros((B, Hr, Wr)), SPLITS, R, extra)
    per = extra + Hr * Wr * (16 + 4 + 1)
    assert l.tolist() == [per] * B and p.shape == (B * per, 4)
    want = []
    for b in range(B):
        want.append([b, -1, 0, 1])
        for ps in SPLITS:
            step = R // ps
            for sp in range(Hr * Wr * ps * ps):
                want.append([b, (sp // (Wr * ps)) * step, (sp % (Wr * ps)) * step, step])
    assert p.tolist() == want


# ------------------------------------------------------------------ compress
def _dense_compress(x, H, W, extra):
    """The reference's dense statement (grained_sample.py:126-147): extras, then avg_pool2d at every granularity."""
    B, N, C = x.shape
    grid = x[:, extra:].reshape(B, H, W, C).permute(0, 3, 1, 2)
    parts = [x[:, :extra]] if extra else []
    for ps in SPLITS:
        k = R // ps
        parts.append(F.avg_pool2d(grid, kernel_size=k, stride=k).permute(0, 2, 3, 1).reshape(B, -1, C))
    return torch.cat(parts, dim=1)


def _dense_position(p, H, W, extra):
    """Row of a sparse patch inside the dense layout above."""
    b, y0, x0, s = p
    if y0 < 0:
        return -y0 - 1
    pos = extra
    for ps in SPLITS:
        k = R // ps
        if k == s:
            return pos + (y0 // s) * (W // s) + x0 // s
        pos += (H // k) * (W // k)
    raise AssertionError


@pytest.mark.parametrize("B,H,W,extra,C", [(3, 16, 16, 1, 24), (2, 8, 12, 0, 16), (2, 32, 32, 2, 8)])
def test_compress_equals_dense_avg_pool(B, H, W, extra, C):
    idx = random_indices(C, B, H // R, W // R)
    patches, _ = orc.index_to_patch(idx, SPLITS, R, extra)
    x = randn(C + 1, B, extra + H * W, C)
    got = orc.compress(x, patches, H, W, extra)
    dense = _dense_compress(torch.from_numpy(x), H, W, extra).numpy()
    want = np.stack([dense[p[0], _dense_position(p, H, W, extra)] for p in patches])
    # same sums in fp32; library pooling may order the 4 / 16 additions differently
    np.testing.assert_allclose(got, want, rtol=0, atol=4e-7 * np.abs(x).max() * 4)


def test_compress_special_cases():
    B, H, W, C = 2, 16, 16, 12
    x = randn(5, B, 1 + H * W, C)
    coarse, _ = orc.index_to_patch(np.full((B, 4, 4), 2), SPLITS, R, 1)
    got = orc.compress(x, coarse, H, W, 1).reshape(B, 17, C)
    assert np.array_equal(got[:, 0], x[:, 0])                                  # class token copied
    pooled = F.avg_pool2d(torch.from_numpy(x[:, 1:]).reshape(B, H, W, C).permute(0, 3, 1, 2), 4)
    np.testing.assert_allclose(got[:, 1:], pooled.permute(0, 2, 3, 1).reshape(B, 16, C).numpy(), atol=1e-6)
    fine, _ = orc.index_to_patch(np.zeros((B, 4, 4)), SPLITS, R, 1)
    got = orc.compress(x, fine, H, W, 1).reshape(B, 257, C)
    # all-fine gate: a pure permutation of the tokens (region-major order), bit exact
    assert np.array_equal(np.sort(got.reshape(B, -1), axis=1), np.sort(x.reshape(B, -1), axis=1))
    tok = fine[:257, 1] * W + fine[:257, 2] + 1
    tok[0] = 0
    assert np.array_equal(got[0], x[0, tok])


def test_compress_accumulation_order_is_sequential_fp32():
    # values chosen so that (a+b)+c+d in fp32 differs from pairwise or float64 summation
    x = np.zeros((1, 16, 4), dtype=np.float32)
    x[0, [0, 1, 4, 5], 0] = [1e8, 1.0, -1e8, 1.0]          # the 2x2 window at (0,0), row-major
    p = np.array([[0, 0, 0, 2]], dtype=np.int64)
    got = orc.compress(x, p, 4, 4, 0)[0, 0]
    seq = np.float32(0)
    for v in [1e8, 1.0, -1e8, 1.0]:
        seq = np.float32(seq + np.float32(v))
    assert got == seq / np.float32(4) == np.float32(0.25)    # float64 summation would give 0.5


# ------------------------------------------------------------------ decompress
def _dense_decompress(xd, gate, reference, H, W, extra, add_ref):
    """The reference's dense statement (grained_sample.py:150-177) with a one-hot gate."""
    B, N, C = reference.shape
    Hr, Wr = gate.shape[1:3]
    out = 0
    start = extra
    for i, ps in enumerate(SPLITS):
        step = R // ps
        Hi, Wi = H // step, W // step
        xi = xd[:, start:start + Hi * Wi].reshape(B, Hi, 1, Wi, 1, C).repeat(1, 1, step, 1, step, 1)
        xi = xi.reshape(B, Hr, H // Hr, Wr, W // Wr, C)
        out = out + (xi * gate[..., i].reshape(B, Hr, 1, Wr, 1, 1)).reshape(B, H, W, C)
        start += Hi * Wi
    out = out.reshape(B, -1, C)
    if extra:
        out = torch.cat([xd[:, :extra], out], dim=1)
    return out + reference if add_ref else out


@pytest.mark.parametrize("add_ref", [True, False])
@pytest.mark.parametrize("B,H,W,extra,C", [(3, 16, 16, 1, 10), (2, 8, 12, 0, 6)])
def test_decompress_equals_dense_one_hot(add_ref, B, H, W, extra, C):
    idx = random_indices(C + 3, B, H // R, W // R)
    patches, _ = orc.index_to_patch(idx, SPLITS, R, extra)
    d = randn(C + 4, patches.shape[0], C)
    ref = randn(C + 5, B, extra + H * W, C)
    got = orc.decompress(d, patches, ref, H, W, extra, add_ref)
    n_dense = extra + sum((H * ps // R) * (W * ps // R) for ps in SPLITS)
    xd = torch.from_numpy(randn(99, B, n_dense, C))          # rows of unselected granularities: arbitrary
    for row, p in enumerate(patches):
        xd[p[0], _dense_position(p, H, W, extra)] = torch.from_numpy(d[row])
    gate = F.one_hot(torch.from_numpy(idx), len(SPLITS)).float()
    want = _dense_decompress(xd, gate, torch.from_numpy(ref), H, W, extra, add_ref).numpy()
    np.testing.assert_array_equal(got, want)


def test_decompress_invariants():
    B, H, W, extra, C = 3, 16, 16, 1, 8
    idx = random_indices(1, B, 4, 4)
    patches, _ = orc.index_to_patch(idx, SPLITS, R, extra)
    L = patches.shape[0]
    ref = randn(2, B, extra + H * W, C)
    # zero delta leaves the reference untouched, bit exact
    assert np.array_equal(orc.decompress(np.zeros((L, C), np.float32), patches, ref, H, W, extra, True), ref)
    # compress after a plain scatter returns the packed rows (mean of equal values)
    y = randn(3, L, C)
    back = orc.compress(orc.decompress(y, patches, ref, H, W, extra, False), patches, H, W, extra)
    np.testing.assert_allclose(back, y, rtol=2e-6)
    # adjointness (vtpack/layers/grained_sample.py:36-37): <compress(x), y> == <x, scatter(y / size^2)>
    x = randn(4, B, extra + H * W, C).astype(np.float64)
    area = (patches[:, 3:4] ** 2).astype(np.float64)
    lhs = (orc.compress(x.astype(np.float32), patches, H, W, extra).astype(np.float64) * y).sum()
    rhs = (x * orc.decompress((y / area).astype(np.float32), patches, ref, H, W, extra, False)).sum()
    assert abs(lhs - rhs) <= 1e-4 * abs(lhs)


# ------------------------------------------------------------------ attention / sparse gemm
def test_attention_against_float64_library_softmax():
    B, h, d, n = 3, 2, 16, 37
    lengths = np.array([5, 1, 11])
    L = lengths.sum()
    q, k, v = randn(1, h, L, d), randn(2, h, B, n, d), randn(3, h, B, n, d)
    scale = 0.37
    got = orc.attention(q, k, v, lengths, scale)
    tq, tk, tv = (torch.from_numpy(a).double() for a in (q, k, v))
    off = 0
    for i, m in enumerate(lengths):
        s = torch.einsum("hqd,hkd->hqk", tq[:, off:off + m], tk[:, i]) * scale
        want = torch.einsum("hqk,hkd->hqd", torch.softmax(s, -1), tv[:, i])
        np.testing.assert_allclose(got[:, off:off + m], want.numpy(), rtol=0, atol=2e-6)
        off += m


def test_attention_special_cases():
    h, d, n = 2, 8, 9
    lengths = np.array([4, 3])
    q, k = randn(1, h, 7, d), randn(2, h, 2, n, d)
    v = np.broadcast_to(randn(3, h, 2, 1, d), (h, 2, n, d)).copy()      # every key holds the same value row
    got = orc.attention(q, k, v, lengths, 1.0)
    np.testing.assert_allclose(got[:, :4], np.broadcast_to(v[:, 0, :1], (h, 4, d)), atol=1e-6)   # weights sum to 1
    np.testing.assert_allclose(got[:, 4:], np.broadcast_to(v[:, 1, :1], (h, 3, d)), atol=1e-6)   # and sample 1 uses ITS K/V
    # a single key: output is that key's value whatever the query
    got = orc.attention(q, k[:, :, :1], randn(4, h, 2, 1, d), lengths, 3.0)
    assert np.allclose(got[:, :4], randn(4, h, 2, 1, d)[:, 0])
    # scale matters and enters before the softmax: scale 0 -> plain average of V
    vv = randn(5, h, 2, n, d)
    got = orc.attention(q, k, vv, lengths, 0.0)
    np.testing.assert_allclose(got[:, :4], np.broadcast_to(vv[:, 0].mean(1, keepdims=True), (h, 4, d)), atol=1e-6)


@pytest.mark.parametrize("ta,tb", [(False, True), (False, False), (True, False), (True, True)])
def test_sparse_gemm_against_bmm(ta, tb):
    B, h = 4, 2
    la = rng(1).randint(1, 9, size=B)
    if not ta and tb:
        lb, ka, kb = rng(2).randint(1, 7, size=B) * 0 + 5, 6, 6
    elif not ta and not tb:
        lb, ka, kb = np.full(B, 5), 5, 7
    elif ta and not tb:
        lb, ka, kb = la.copy(), 6, 7
    else:
        la, lb, ka, kb = np.full(B, 5), np.full(B, 3), 6, 5
    a, b = randn(3, h, la.sum(), ka), randn(4, h, lb.sum(), kb)
    got = orc.sparse_gemm(a, b, la, lb, ta, tb)
    want = torch_ref.sparse_gemm(torch.from_numpy(a).double(), torch.from_numpy(b).double(), torch.from_numpy(la),
                                 torch.from_numpy(lb), ta, tb)
    np.testing.assert_allclose(got, want.numpy(), atol=1e-5)


def test_sparse_gemm_rejects_mismatch():
    a, b = randn(1, 1, 5, 4), randn(2, 1, 6, 3)
    with pytest.raises(ValueError):
        orc.sparse_gemm(a, b, np.array([5]), np.array([6]), False, False)    # inner dims 4 vs 6


# ------------------------------------------------------------------ torch restatement == C restatement
def test_torch_ref_operators_match_c_oracle():
    B, H, W, extra, C, h = 4, 16, 16, 1, 48, 3
    idx = random_indices(7, B, 4, 4)
    p_c, l_c = orc.index_to_patch(idx, SPLITS, R, extra)
    p_t, l_t = torch_ref.index_to_patch(torch.from_numpy(idx), torch.tensor(SPLITS), R, extra)
    assert np.array_equal(p_t.numpy(), p_c) and np.array_equal(l_t.numpy(), l_c)
    x = randn(8, B, extra + H * W, C)
    comp_c = orc.compress(x, p_c, H, W, extra)
    comp_t = torch_ref.compress(torch.from_numpy(x), p_t, H, W, extra).numpy()
    np.testing.assert_allclose(comp_t, comp_c, atol=1e-6)
    d = randn(9, p_c.shape[0], C)
    np.testing.assert_array_equal(torch_ref.decompress(torch.from_numpy(d), p_t, torch.from_numpy(x), H, W, extra,
                                                       True).numpy(),
                                  orc.decompress(d, p_c, x, H, W, extra, True))
    dd = C // h
    q, k, v = randn(10, h, p_c.shape[0], dd), randn(11, h, B, 257, dd), randn(12, h, B, 257, dd)
    att_t = torch_ref.attention(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), l_t, dd ** -0.5)
    np.testing.assert_allclose(att_t.numpy(), orc.attention(q, k, v, l_c, dd ** -0.5), atol=2e-6)


def test_router_restatement_matches_manual_pooling():
    B, H, W, extra, C = 2, 8, 8, 1, 12
    x = randn(1, B, extra + H * W, C)
    w, b = randn(2, 3, C), randn(3, 3)
    got = torch_ref.router_gate(torch.from_numpy(x), H, W, torch.from_numpy(w), torch.from_numpy(b), R).numpy()
    grid = x[:, extra:].reshape(B, H // R, R, W // R, R, C).astype(np.float64).mean(axis=(2, 4))
    np.testing.assert_allclose(got, grid @ w.T.astype(np.float64) + b, atol=1e-5)
