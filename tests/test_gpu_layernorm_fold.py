"""LayerNorm folded into the Linear behind it (norm1 -> kv, norm2 -> fc1; vtpack/models/dge/deit_dge.py:127-128 with
:73 and :38-44): the statistics records and their three producers, the Linear that consumes them, and the model with
the folding on and off.

The reference for every value is torch in fp64 on the same bf16 inputs: F.layer_norm followed by a matrix product
(+ GELU).  Inputs are scaled so that expected values stay below 4 in magnitude, where the plain 2e-2 max-abs bar of
the bf16 tests applies.
"""
import pytest
import torch

from util import BF16_ABS, SPLITS, abs_err, random_indices

pytestmark = pytest.mark.gpu

C = 384
EPS = 1e-6


def decode(rec):
    """records [rows, 16] bf16 -> (mean, sigma) as the consuming kernel sums them, and the raw values."""
    r = rec.float()
    return r[:, 0] + r[:, 2] + r[:, 5], r[:, 6] + r[:, 7], r


def assert_record_layout(rec):
    """lo = (m1, m1, m2, m1, m2, m3, s1, s2), hi = (s1, s2, 0, ...): what one MFMA K step multiplies by the column
    record (-c1, -c2, -c1, -c3, -c2, -c1, b1, b1 | b2, 0, ...)."""
    r = rec.float()
    assert bool((r[:, 0] == r[:, 1]).all() and (r[:, 0] == r[:, 3]).all() and (r[:, 2] == r[:, 4]).all())
    assert bool((r[:, 6] == r[:, 8]).all() and (r[:, 7] == r[:, 9]).all() and (r[:, 10:] == 0).all())


def want_stats(x):
    xd = x.double().reshape(-1, x.shape[-1])
    return xd.mean(1), (xd.var(1, unbiased=False) + EPS).sqrt()


def rows_like_tokens(M, seed, shift=0.0, dev="cuda"):
    """Rows with per-row scale between 0.5 and 2.5 and a per-row offset of `shift` standard deviations."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, C, generator=g) * (0.5 + 2 * torch.rand(M, 1, generator=g))
    return (x + shift * torch.randn(M, 1, generator=g)).bfloat16().to(dev)


def layer(N, seed, dev):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(N, C, generator=g) * 0.03).bfloat16().to(dev)
    b = (torch.randn(N, generator=g) * 0.2).bfloat16().to(dev)
    gamma = (1 + 0.3 * torch.randn(C, generator=g)).bfloat16().to(dev)
    beta = (0.2 * torch.randn(C, generator=g)).bfloat16().to(dev)
    return w, b, gamma, beta


def want_linear_layernorm(x, w, b, gamma, beta, act):
    y = torch.nn.functional.layer_norm(x.double(), (C,), gamma.double(), beta.double(), EPS)
    want = y @ w.double().T + (b.double() if b is not None else 0.0)
    return torch.nn.functional.gelu(want) if act == "gelu" else want


# ----------------------------------------------------------------------------- records from the statistics kernel
@pytest.mark.parametrize("shift", [0.0, 3.0, 200.0])
@pytest.mark.parametrize("live", [None, 0, 1, 5, 4097])
def test_statistics_records(dev, live, shift):
    from vtpack_amd import ops
    M = 5000
    x = rows_like_tokens(M, 11, shift, dev)
    rows_dev = None if live is None else torch.tensor([live], dtype=torch.int64, device=dev)
    rec = torch.full((M, 16), 7.0, dtype=torch.bfloat16, device=dev)
    ops.layernorm_stats(x, EPS, rows_dev=rows_dev, out=rec)
    L = M if live is None else live
    assert bool((rec[L:] == 7.0).all())
    if L:
        mean, sigma, _ = decode(rec[:L])
        m_ref, s_ref = want_stats(x[:L])
        assert_record_layout(rec[:L])
        # mean to fp32 accuracy relative to the row's magnitude (three bf16 parts), sigma to 2^-16 (two parts)
        assert float(((mean.double().cpu() - m_ref.cpu()).abs() / x[:L].double().abs().amax(1).cpu()).max()) < 1e-6
        assert float(((sigma.double().cpu() - s_ref.cpu()) / s_ref.cpu()).abs().max()) < 2e-5


# ----------------------------------------------------------------------------- the consuming Linear
@pytest.mark.parametrize("live", [None, 0, 1, 7, 31, 32, 33, 63, 65, 2047, 2500])
@pytest.mark.parametrize("N,act", [(768, "none"), (1536, "gelu"), (384, "none")])
@pytest.mark.parametrize("packed", [True, False])
def test_linear_layernorm_live_rows(dev, live, N, act, packed):
    from vtpack_amd import ops
    M = 2600
    x = rows_like_tokens(M, 3 + (live or 0), 1.0, dev)
    w, b, gamma, beta = layer(N, 5, dev)
    rows_dev = None if live is None else torch.tensor([live], dtype=torch.int64, device=dev)
    L = M if live is None else live
    rec = ops.layernorm_stats(x, EPS, rows_dev=rows_dev)
    out = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=dev)
    ops.PACK_WEIGHTS = packed
    try:
        ops.invalidate_packed()
        ops.linear_layernorm(x, rec, w, b, gamma, beta, act=act, rows_dev=rows_dev, out=out)
    finally:
        ops.PACK_WEIGHTS = True
        ops.invalidate_packed()
    if L:
        want = want_linear_layernorm(x[:L], w, b, gamma, beta, act)
        assert float(want.abs().max()) < 4.0
        assert abs_err(out[:L], want) <= BF16_ABS
    assert bool((out[L:] == 7.0).all())


@pytest.mark.parametrize("shift", [0.0, 30.0, 100.0])
def test_linear_layernorm_rows_far_from_zero(dev, shift):
    """Rows whose mean is up to a few hundred standard deviations from zero: the rank-one correction
    mean * colsum(W') is as large as the product itself and cancels it to fp32 accuracy, so the error stays that of
    the two-kernel path.  (What is left of the cancellation is the fp32 rounding of the product, about
    2^-22 |mean| sum|W'|, times rstd: it reaches the bf16 bar only where |mean| / sigma passes ~10^4, i.e. for rows
    that bf16 cannot tell from constant ones.)"""
    from vtpack_amd import ops
    M, N = 4096, 768
    x = rows_like_tokens(M, 21, shift, dev)
    _, s_ref = want_stats(x)
    keep = (x.double().mean(1).abs() / s_ref) < 1e3          # drop rows that rounding has made constant
    x = x[keep][:2304 + (int(keep.sum()) - 2304) // 32 * 32].contiguous()
    w, b, gamma, beta = layer(N, 22, dev)
    got = ops.linear_layernorm(x, ops.layernorm_stats(x, EPS), w, b, gamma, beta)
    two = ops.linear(ops.layernorm(x, gamma, beta, EPS), w, b)
    want = want_linear_layernorm(x, w, b, gamma, beta, "none")
    assert float(want.abs().max()) < 4.0
    assert abs_err(got, want) <= BF16_ABS
    assert abs_err(got, want) <= 1.25 * abs_err(two, want) + 2 ** -9


def test_linear_layernorm_of_zero_rows_is_the_folded_bias(dev):
    """All-zero rows (padding): LayerNorm gives beta, the Linear bias + W beta, and the folded form reproduces it
    through sigma * b' * rstd with no product to cancel."""
    from vtpack_amd import ops
    M, N = 2304, 768
    x = rows_like_tokens(M, 5, 0.0, dev)
    x[::7] = 0
    w, b, gamma, beta = layer(N, 6, dev)
    got = ops.linear_layernorm(x, ops.layernorm_stats(x, EPS), w, b, gamma, beta)
    want = want_linear_layernorm(x, w, b, gamma, beta, "none")
    assert abs_err(got[::7], want[::7]) <= 2 ** -8 * float(want[::7].abs().max())     # one bf16 rounding
    assert abs_err(got, want) <= BF16_ABS


def test_linear_layernorm_full_shapes_and_repeatable(dev):
    """The two shapes of the headline model (kv: 65 792 x 768, fc1 + GELU: ~27 000 live rows x 1536) and bit-equal
    repeats."""
    from vtpack_amd import ops
    for M, N, act, live in ((65792, 768, "none", None), (65792, 1536, "gelu", 27113)):
        x = rows_like_tokens(M, M % 97, 0.5, dev)
        w, b, gamma, beta = layer(N, N, dev)
        rows_dev = None if live is None else torch.tensor([live], dtype=torch.int64, device=dev)
        L = M if live is None else live
        rec = ops.layernorm_stats(x, EPS, rows_dev=rows_dev)
        first = ops.linear_layernorm(x, rec, w, b, gamma, beta, act=act, rows_dev=rows_dev)
        want = want_linear_layernorm(x[:L], w, b, gamma, beta, act)
        assert float(want.abs().max()) < 4.0
        assert abs_err(first[:L], want) <= BF16_ABS
        for _ in range(2):
            assert torch.equal(ops.linear_layernorm(x, rec, w, b, gamma, beta, act=act, rows_dev=rows_dev)[:L], first[:L])


def test_folded_weights_follow_edits(dev):
    """The folded copy is keyed on all four tensors: an in-place edit of the LayerNorm's scale or of the Linear's bias
    is seen at the next call; a write through .data needs invalidate_packed."""
    from vtpack_amd import ops
    M, N = 2304, 768
    x = rows_like_tokens(M, 1, 0.0, dev)
    w, b, gamma, beta = layer(N, 2, dev)
    rec = ops.layernorm_stats(x, EPS)

    def check():
        got = ops.linear_layernorm(x, rec, w, b, gamma, beta)
        assert abs_err(got, want_linear_layernorm(x, w, b, gamma, beta, "none")) <= BF16_ABS
        return got

    base = check()
    gamma.mul_(0.5)
    assert not torch.equal(check(), base)
    b.add_(0.25)
    check()
    w.data.mul_(0.5)                       # not counted by torch
    ops.invalidate_packed(w)
    check()


def test_operand_checks(dev):
    from vtpack_amd import ops
    x = rows_like_tokens(2304, 1, 0.0, dev)
    w, b, gamma, beta = layer(768, 2, dev)
    rec = ops.layernorm_stats(x, EPS)
    with pytest.raises(TypeError):
        ops.layernorm_stats(x.float(), EPS)
    with pytest.raises(ValueError):
        ops.linear_layernorm(x, rec[:100], w, b, gamma, beta)
    with pytest.raises(ValueError):
        ops.linear_layernorm(x[:100], rec[:100], w, b, gamma, beta)            # too few rows for the kernel
    with pytest.raises(TypeError):
        ops.linear_layernorm(x, rec, w, b, gamma.float(), beta)
    with pytest.raises(ValueError):
        ops.linear_layernorm(x, rec, w, b, gamma[:100], beta[:100])
    with pytest.raises(ValueError):
        ops.linear(x, w, b, stats_eps=EPS)                                     # records need N = 384
    assert not ops.fits_linear_layernorm(x.float(), w)
    assert not ops.fits_linear_layernorm(x, torch.zeros(100, C, dtype=torch.bfloat16, device=dev))


@pytest.mark.parametrize("live1", [None, 0, 1, 31, 33, 700, 2599, 11000, 60000])
@pytest.mark.parametrize("M0,N0,N1", [(65792, 768, 384), (2600, 768, 384), (4097, 384, 1536)])
def test_two_linears_in_one_launch(dev, M0, N0, N1, live1):
    """norm1 -> kv on all tokens and norm1 -> q on the packed rows as one launch whose workgroups are shared out by
    the live row counts: the same bytes as the two separate launches, whatever the split."""
    from vtpack_amd import ops
    M1 = max(M0, 2048 if live1 is None else live1)
    x0 = rows_like_tokens(M0, 31, 1.0, dev)
    x1 = rows_like_tokens(M1, 32, 0.5, dev)
    w0, b0, gamma, beta = layer(N0, 33, dev)
    w1, b1, _, _ = layer(N1, 34, dev)
    rows_dev1 = None if live1 is None else torch.tensor([live1], dtype=torch.int64, device=dev)
    L1 = M1 if live1 is None else live1
    rec0 = ops.layernorm_stats(x0, EPS)
    rec1 = ops.layernorm_stats(x1, EPS, rows_dev=rows_dev1)
    want0 = ops.linear_layernorm(x0, rec0, w0, b0, gamma, beta)
    want1 = ops.linear_layernorm(x1, rec1, w1, b1, gamma, beta, rows_dev=rows_dev1)
    got0, got1 = ops.linear_layernorm_pair(x0, rec0, w0, b0, x1, rec1, w1, b1, gamma, beta, rows_dev1=rows_dev1)
    assert torch.equal(got0, want0)
    assert torch.equal(got1[:L1], want1[:L1])
    # the other way round, and the first one short
    rows_dev0 = torch.tensor([min(M0, 777)], dtype=torch.int64, device=dev)
    a, b = ops.linear_layernorm_pair(x1, rec1, w1, b1, x0, rec0, w0, b0, gamma, beta, rows_dev0=rows_dev1, rows_dev1=rows_dev0)
    assert torch.equal(a[:L1], want1[:L1]) and torch.equal(b[:min(M0, 777)], want0[:min(M0, 777)])


# ----------------------------------------------------------------------------- records from the producing kernels
@pytest.mark.parametrize("live", [None, 0, 17, 33, 64, 2599])
@pytest.mark.parametrize("has_bias,has_res", [(True, True), (True, False), (False, True), (False, False)])
def test_linear_writes_records_of_its_rows(dev, live, has_bias, has_res):
    """proj + residual with the records of its output rows: the output is the plain Linear's bit for bit, the records
    are the statistics of the fp32 sums."""
    from vtpack_amd import ops
    M = 2600
    g = torch.Generator().manual_seed(7 + (live or 0))
    a = torch.randn(M, C, generator=g).bfloat16().to(dev)
    w = (torch.randn(C, C, generator=g) * 0.05).bfloat16().to(dev)
    # a bias far from zero: without a residual it is what moves the rows' means away from zero (|mean| ~ 30 sigma), the
    # case the pivoted sums are there for
    b = (torch.randn(C, generator=g) * 0.2 + (0.0 if has_res else 30.0)).bfloat16().to(dev) if has_bias else None
    res = (torch.randn(M, C, generator=g) * 2 + 3 * torch.randn(M, 1, generator=g)).bfloat16().to(dev) if has_res else None
    rows_dev = None if live is None else torch.tensor([live], dtype=torch.int64, device=dev)
    L = M if live is None else live
    plain = ops.linear(a, w, b, residual=res, rows_dev=rows_dev)
    out, rec = ops.linear(a, w, b, residual=res, rows_dev=rows_dev, stats_eps=EPS)
    assert torch.equal(out[:L], plain[:L])
    if not L:
        return
    want = a[:L].double() @ w.double().T
    if has_bias:
        want = want + b.double()
    if has_res:
        want = want + res[:L].double()
    mean, sigma, _ = decode(rec[:L])
    m_ref, s_ref = want_stats(want)
    assert_record_layout(rec[:L])
    assert float((mean.double() - m_ref).abs().max()) < 1e-5 * max(1.0, float(m_ref.abs().max()) / 8)
    assert float(((sigma.double() - s_ref) / s_ref).abs().max()) < 3e-5


def test_linear_records_at_full_size_feed_the_next_linear(dev):
    """proj -> (records) -> fc1 at the headline shape, against LayerNorm of the stored rows in fp64."""
    from vtpack_amd import ops
    M, live = 65792, 27113
    g = torch.Generator().manual_seed(3)
    a = torch.randn(M, C, generator=g).bfloat16().to(dev)
    wp = (torch.randn(C, C, generator=g) * 0.05).bfloat16().to(dev)
    res = torch.randn(M, C, generator=g).bfloat16().to(dev)
    w1, b1, gamma, beta = layer(1536, 9, dev)
    rows_dev = torch.tensor([live], dtype=torch.int64, device=dev)
    q1, rec = ops.linear(a, wp, None, residual=res, rows_dev=rows_dev, stats_eps=EPS)
    hid = ops.linear_layernorm(q1, rec, w1, b1, gamma, beta, act="gelu", rows_dev=rows_dev)
    want = want_linear_layernorm(q1[:live], w1, b1, gamma, beta, "gelu")
    assert float(want.abs().max()) < 4.0
    assert abs_err(hid[:live], want) <= BF16_ABS


@pytest.mark.parametrize("B,H,Cc,extra", [(8, 16, 384, 1), (4, 32, 384, 2), (3, 8, 512, 0), (2, 8, 264, 1)])
def test_scatter_back_writes_records_of_the_tokens(dev, B, H, Cc, extra):
    from vtpack_amd import ops
    W = H
    N = extra + H * W
    g = torch.Generator().manual_seed(B)
    idx = torch.from_numpy(random_indices(B, B, H // 4, W // 4)).to(dev)
    splits = torch.tensor(SPLITS, dtype=torch.int64, device=dev)
    patches, offsets, lengths = ops.index_to_patch(idx, splits, 4, extra, capacity=B * N)
    x = (torch.randn(B, N, Cc, generator=g) * 2 + 5 * torch.randn(B, N, 1, generator=g)).bfloat16().to(dev)
    q = torch.randn(B * N, Cc, generator=g).bfloat16().to(dev)
    sub = torch.randn(B * N, Cc, generator=g).bfloat16().to(dev)
    wgt = (torch.randn(3, Cc, generator=g) * 0.1).bfloat16().to(dev)
    bias = torch.zeros(3, dtype=torch.bfloat16, device=dev)
    o0, g0, i0 = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=sub, next_weight=wgt, next_bias=bias)
    o1, g1, i1, rec = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=sub, next_weight=wgt,
                                            next_bias=bias, stats_eps=EPS)
    assert torch.equal(o0, o1) and torch.equal(g0, g1) and torch.equal(i0, i1)
    mean, sigma, _ = decode(rec)
    m_ref, s_ref = want_stats(o1)
    assert_record_layout(rec)
    assert float((mean.double() - m_ref).abs().max()) < 5e-6 * float(o1.double().abs().max())
    assert float(((sigma.double() - s_ref) / s_ref).abs().max()) < 3e-5
    # without the next router as well
    o2, _, _, rec2 = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=None, stats_eps=EPS)
    m2, s2, _ = decode(rec2)
    m_ref2, s_ref2 = want_stats(o2)
    assert float(((s2.double() - s_ref2) / s_ref2).abs().max()) < 3e-5


@pytest.mark.parametrize("B,H,Cc,extra,with_front", [(8, 16, 384, 1, True), (4, 32, 384, 2, True), (3, 8, 512, 0, False),
                                                    (2, 8, 264, 1, False)])
def test_router_with_records_of_all_tokens(dev, B, H, Cc, extra, with_front):
    """The first block's kernel: gate logits and indices bit for bit those of the router, the records of every token
    row, the query counts per region, and the rows given for the extra tokens stored in every sample."""
    from vtpack_amd import ops
    W = H
    N = extra + H * W
    g = torch.Generator().manual_seed(B + Cc)
    x = (torch.randn(B, N, Cc, generator=g) * 2 + 5 * torch.randn(B, N, 1, generator=g)).bfloat16().to(dev)
    wgt = (torch.randn(3, Cc, generator=g) * 0.1).bfloat16().to(dev)
    bias = (torch.randn(3, generator=g) * 0.1).bfloat16().to(dev)
    splits = torch.tensor(SPLITS, dtype=torch.int64, device=dev)
    front = (torch.randn(extra, Cc, generator=g) * 3).bfloat16().to(dev) if with_front else None
    want_x = x.clone()
    if with_front:
        want_x[:, :extra] = front
    want_gate, want_idx = ops.router(want_x, wgt, bias, H, W, 4)
    gate, idx, rec, counts = ops.router_stats(x, wgt, bias, H, W, 4, EPS, front_rows=front, splits=splits)
    assert torch.equal(x, want_x)                       # only the extra-token rows were written
    assert torch.equal(gate, want_gate) and torch.equal(idx, want_idx)
    assert torch.equal(counts[:idx.numel()].long(), splits[idx.reshape(-1)] ** 2)
    mean, sigma, _ = decode(rec)
    m_ref, s_ref = want_stats(want_x)
    assert_record_layout(rec)
    assert float((mean.double() - m_ref).abs().max()) < 5e-6 * float(want_x.double().abs().max())
    assert float(((sigma.double() - s_ref) / s_ref).abs().max()) < 3e-5
    # words to clear on the way (more of them than the launch has threads at the small shapes)
    scratch = torch.full((5001,), -1, dtype=torch.int64, device=dev)
    _, _, rec2, none = ops.router_stats(x, wgt, bias, H, W, 4, EPS, clear=scratch[:5000])
    assert none is None and torch.equal(rec2, rec)
    assert int(scratch[:5000].abs().sum()) == 0 and int(scratch[5000]) == -1


def test_scatter_records_refused_for_other_rows(dev):
    from vtpack_amd import ops
    from vtpack_amd._lib import VtdgeError
    B, H, Cc = 2, 8, 192
    idx = torch.zeros(B, 2, 2, dtype=torch.int64, device=dev)
    splits = torch.tensor(SPLITS, dtype=torch.int64, device=dev)
    patches, offsets, lengths = ops.index_to_patch(idx, splits, 4, 1, capacity=B * 65)
    x = torch.zeros(B, 65, Cc, dtype=torch.bfloat16, device=dev)
    q = torch.zeros(B * 65, Cc, dtype=torch.bfloat16, device=dev)
    with pytest.raises(VtdgeError):
        ops.decompress_router(q, idx, splits, offsets, x, H, H, 4, stats_eps=EPS)
    assert not ops.fits_scatter_stats(x) and not ops.fits_scatter_stats(x.float())


# ----------------------------------------------------------------------------- the scatter-back that packs the
# next block's queries (vtpack/layers/dge.py:87-112, then :145-150, :75-79 of the next block) against the two kernels
# it stands for: every output bit for bit
@pytest.mark.parametrize("B,H,W,Cc,extra,with_sub", [(8, 16, 16, 384, 1, True), (4, 32, 32, 384, 2, True),
                                                     (4, 8, 8, 512, 0, False), (2, 8, 8, 264, 1, True),
                                                     (3, 8, 16, 384, 1, True), (256, 16, 16, 384, 1, True),
                                                     (64, 32, 32, 384, 0, True),
                                                     # four times as many workgroups as the chip holds at once
                                                     (256, 32, 32, 384, 1, True)])
def test_scatter_back_packs_the_next_queries(dev, B, H, W, Cc, extra, with_sub):
    from vtpack_amd import ops
    N = extra + H * W
    g = torch.Generator().manual_seed(B + Cc)
    idx = torch.from_numpy(random_indices(B, B, H // 4, W // 4)).to(dev)
    splits = torch.tensor(SPLITS, dtype=torch.int64, device=dev)
    next_splits = torch.tensor(SPLITS[::-1], dtype=torch.int64, device=dev)
    x = (torch.randn(B, N, Cc, generator=g) * 2 + 3 * torch.randn(B, N, 1, generator=g)).bfloat16().to(dev)
    assert ops.fits_pack_next(x, H, W, 4, SPLITS)
    comp, _, patches, offsets, lengths, rrows = ops.compress_regions(x, idx, splits, H, W, 4, want_region_rows=True)
    q = torch.randn(B * N, Cc, generator=g).bfloat16().to(dev)
    wgt = (torch.randn(3, Cc, generator=g) * 0.3).bfloat16().to(dev)
    bias = (torch.randn(3, generator=g) * 0.3).bfloat16().to(dev)
    sub = comp if with_sub else None
    want = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=sub, next_weight=wgt, next_bias=bias,
                                 stats_eps=EPS, next_splits=next_splits)
    w_out, w_gate, w_idx, w_rec, w_cnt = want
    assert len(set(w_idx.reshape(-1).tolist())) >= 2            # a mix of splits
    w_comp, w_crec, w_pat, w_off, w_len, w_rows = ops.compress_regions(
        w_out, w_idx, next_splits, H, W, 4, counts=w_cnt, stats_eps=2 * EPS, want_region_rows=True)
    total = int(w_off[B])
    words = ops.pack_next_workspace_words(B, H, W, 4)
    ws = torch.zeros(words + 3, dtype=torch.int64, device=dev)
    for trial in range(4):
        kw = dict(workspace=ws) if trial % 2 else {}
        if trial % 2:
            ws.zero_()
        got = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=sub, next_weight=wgt, next_bias=bias,
                                    stats_eps=EPS, next_splits=next_splits, pack_next=True, pack_eps=2 * EPS, **kw)
        out, gate, nidx, rec, cnt, packed = got
        assert int(packed["workspace"][0]) == 0
        assert torch.equal(out, w_out) and torch.equal(gate, w_gate) and torch.equal(nidx, w_idx)
        assert torch.equal(rec, w_rec) and torch.equal(cnt[:nidx.numel()], w_cnt[:nidx.numel()])
        assert torch.equal(packed["offsets"], w_off)
        assert torch.equal(packed["region_rows"], w_rows)
        assert torch.equal(packed["comp"][:total], w_comp[:total])
        assert torch.equal(packed["records"][:total], w_crec[:total])
        assert torch.equal(packed["patches"][:total], w_pat[:total])
    # the regions' first rows of this block handed over as well
    got = ops.decompress_router(q, idx, splits, offsets, x, H, W, 4, sub=sub, next_weight=wgt, next_bias=bias,
                                stats_eps=EPS, next_splits=next_splits, pack_next=True, pack_eps=2 * EPS,
                                region_rows=rrows, cur_counts=(splits[idx.reshape(-1)] ** 2).to(torch.uint8))
    assert torch.equal(got[0], w_out) and torch.equal(got[5]["records"][:total], w_crec[:total])
    assert torch.equal(got[5]["comp"][:total], w_comp[:total]) and torch.equal(got[5]["offsets"], w_off)


def test_pack_next_refuses_partial_workgroups(dev):
    from vtpack_amd import ops
    x = torch.zeros(3, 1 + 8 * 8, 384, dtype=torch.bfloat16, device=dev)     # 3 * 4 regions: fine
    assert ops.fits_pack_next(x, 8, 8, 4, SPLITS)
    x = torch.zeros(3, 1 + 12 * 4, 384, dtype=torch.bfloat16, device=dev)    # 3 * 3 regions
    assert not ops.fits_pack_next(x, 12, 4, 4, SPLITS)


# ----------------------------------------------------------------------------- the model with and without
def test_model_with_and_without_folded_norms(dev):
    """DeiT-S+DGE, bf16, 256 px, batch 16 (enough rows for the weight-stationary kernels): with the folding on the
    forward launches one LayerNorm (the final one, on the class-token rows) instead of 37, the statistics of the first block's tokens coming
    from its router's kernel.  Rounding differs between the two forms, so a near-tie of some router may fall the other way and the
    two runs need not route alike after the first block: each run is therefore compared with the CPU restatement
    under its OWN gate choices (logits within the bf16 bar, integer outputs of every layer exact)."""
    from vtpack_amd import _lib, engine
    from vtpack_amd.models import dge as zoo
    from vtpack_amd.synthetic import set_synthetic_router, synthetic_images
    from util import LaunchNames, forced_reference

    torch.manual_seed(0)
    m = zoo.deit_dge_s124_small_patch16_256()
    set_synthetic_router(m, 0)
    m = m.eval().to(dev).to(torch.bfloat16)
    img = synthetic_images(16, 256, seed=0, dtype=torch.bfloat16, device=dev)
    runs = {}
    try:
        for fold in (True, False):
            engine.FOLD_NORMS = fold
            _lib.timer = LaunchNames()
            with torch.no_grad():
                out = m(img)
            names = _lib.timer.names
            _lib.timer = None
            want, traces = forced_reference(m, img.float().cpu(), 6, 12)
            for blk, tr in zip(m.blocks, traces):
                assert torch.equal(blk.dge.states["patches"].cpu(), tr["patches"])
                assert torch.equal(blk.dge.states["batches"], tr["lengths"])
            assert abs_err(out.float(), want) <= BF16_ABS, f"folded LayerNorms {'on' if fold else 'off'}"
            runs[fold] = (out.float(), [blk.dge.states["batches_device"].clone() for blk in m.blocks], names)
    finally:
        engine.FOLD_NORMS = True
        _lib.timer = None
    (on, len_on, names_on), (off, len_off, names_off) = runs[True], runs[False]
    assert names_off.count("vtdge_layernorm") == 36 and names_off.count("vtdge_linear_layernorm") == 0
    assert names_off.count("vtdge_layernorm_rows") == 1 and names_on.count("vtdge_layernorm_rows") == 1
    assert names_on.count("vtdge_layernorm") == 0 and names_on.count("vtdge_layernorm_stats") == 0
    assert names_on.count("vtdge_router_stats") == 1 and names_on.count("vtdge_router") == 0
    assert names_on.count("vtdge_linear_layernorm") == 12 and names_on.count("vtdge_linear_layernorm_pair") == 12
    assert names_on.count("vtdge_linear_stats") == 12
    assert torch.equal(len_on[0], len_off[0])
    if all(torch.equal(a, b) for a, b in zip(len_on, len_off)):
        assert abs_err(on, off) <= 2 * BF16_ABS
