"""The headline configuration (DeiT-S+DGE, bf16, batch 256, 256 px: 65 792 tokens of 384 channels, about 27 000
packed queries per layer) and the high-resolution one (batch 64, 512 px: 1025 tokens and 64 regions per sample, key
/ value length 1025) at their full sizes, where the CPU oracle would take minutes: every kernel of the path is
checked through properties that hold at any size and whose expected values are exact."""
import numpy as np
import pytest
import torch

from util import random_indices

pytestmark = pytest.mark.gpu

C, R, EXTRA, HEADS = 384, 4, 1, 6
SPLITS = [4, 2, 1]
B = H = W = N = IMG = 0      # set per configuration by the fixture below


@pytest.fixture(scope="module", params=["b256_256px", "b64_512px"], autouse=True)
def geometry(request):
    global B, H, W, N, IMG
    B, H, IMG = (256, 16, 256) if request.param == "b256_256px" else (64, 32, 512)
    W = H
    N = EXTRA + H * W
    return request.param


@pytest.fixture(scope="module")
def routed(dev, geometry):
    """Gate indices with the mix the benchmark's router produces, and their packed descriptors."""
    from vtpack_amd import ops
    idx = torch.from_numpy(random_indices(5, B, H // R, W // R, p=[0.1, 0.25, 0.65])).to(dev)
    splits = torch.tensor(SPLITS, dtype=torch.int64, device=dev)
    patches, offsets, lengths = ops.index_to_patch(idx, splits, R, EXTRA, capacity=B * N)
    return idx, splits, patches, offsets, lengths


def test_descriptors_partition_every_sample(routed):
    """Rows sorted by sample, extra tokens first; the windows of a sample tile its token grid exactly once;
    lengths and offsets follow from the gate indices in closed form."""
    idx, splits, patches, offsets, lengths = routed
    ps = splits[idx]                                            # [B, Hr, Wr]
    want_len = EXTRA + (ps * ps).sum(dim=(1, 2))
    assert torch.equal(lengths, want_len)
    assert torch.equal(offsets, torch.cat([torch.zeros(1, dtype=torch.int64, device=idx.device), want_len.cumsum(0)]))
    L = int(offsets[-1])
    p = patches[:L].cpu().numpy()
    assert (np.diff(p[:, 0]) >= 0).all() and p[0, 0] == 0 and p[-1, 0] == B - 1
    cover = np.zeros((B, H, W), dtype=np.int32)
    spatial = p[p[:, 1] >= 0]
    for sz in (1, 2, 4):
        rows = spatial[spatial[:, 3] == sz]
        for dy in range(sz):
            for dx in range(sz):
                np.add.at(cover, (rows[:, 0], rows[:, 1] + dy, rows[:, 2] + dx), 1)
    assert (cover == 1).all()
    extras = p[p[:, 1] < 0]
    assert len(extras) == B * EXTRA and (extras[:, 1] == -1).all() and (extras[:, 3] == 1).all()
    # a sample's first row is its extra token
    assert (p[offsets[:-1].cpu().numpy(), 1] == -1).all()


def test_compress_inverts_scatter(dev, routed):
    """Scattering packed rows over their windows and taking the window means again returns the rows, bit for bit
    (the mean of equal values is that value), and with every window of size 1 compress is a row gather."""
    from vtpack_amd import ops
    idx, splits, patches, offsets, lengths = routed
    L = int(offsets[-1])
    g = torch.Generator().manual_seed(1)
    q = torch.randn(B * N, C, generator=g).bfloat16().to(dev)
    zeros = torch.zeros(B, N, C, dtype=torch.bfloat16, device=dev)
    spread = ops.decompress(q, patches, zeros, W, EXTRA, add_ref=False, rows_dev=offsets[B:], rows=B * N)
    back = ops.compress(spread, patches, W, EXTRA, rows_dev=offsets[B:], rows=B * N)
    back = back[0] if isinstance(back, tuple) else back
    assert torch.equal(back[:L], q[:L])
    # the fused form of the block: out = ref + (q - comp) is ref itself when q == comp
    x = torch.randn(B, N, C, generator=g).bfloat16().to(dev)
    comp = ops.compress(x, patches, W, EXTRA, rows_dev=offsets[B:], rows=B * N)
    comp = comp[0] if isinstance(comp, tuple) else comp
    same = ops.decompress(comp, patches, x, W, EXTRA, add_ref=True, sub=comp, rows_dev=offsets[B:], rows=B * N)
    assert torch.equal(same, x)
    # all-fine routing: one window per token, compress only reorders rows
    fine = torch.full((B, H // R, W // R), 0, dtype=torch.int64, device=dev)
    p_f, o_f, _ = ops.index_to_patch(fine, splits, R, EXTRA, capacity=B * N)
    assert int(o_f[-1]) == B * N
    c_f = ops.compress(x, p_f, W, EXTRA, rows_dev=o_f[B:], rows=B * N)
    c_f = c_f[0] if isinstance(c_f, tuple) else c_f
    tok = torch.where(p_f[:, 1] < 0, -p_f[:, 1] - 1, EXTRA + p_f[:, 1] * W + p_f[:, 2])
    assert torch.equal(c_f, x[p_f[:, 0], tok])


def test_router_picks_the_planted_split(dev):
    """Channel s of every token is set from the split planted for its region and the gate weight reads exactly
    that channel: the router returns the planted split for every region of the batch."""
    from vtpack_amd import ops
    want = torch.from_numpy(random_indices(9, B, H // R, W // R)).to(dev)
    x = torch.zeros(B, N, C, dtype=torch.bfloat16, device=dev)
    onehot = torch.nn.functional.one_hot(want, 3).to(torch.bfloat16)               # [B, Hr, Wr, 3]
    grid = onehot.repeat_interleave(R, dim=1).repeat_interleave(R, dim=2)             # [B, H, W, 3]
    x[:, EXTRA:, :3] = grid.reshape(B, H * W, 3)
    x[:, :EXTRA] = 7.0                                                                # extra tokens are not pooled
    wgt = torch.zeros(3, C, dtype=torch.bfloat16, device=dev)
    wgt[0, 0] = wgt[1, 1] = wgt[2, 2] = 1.0
    bias = torch.zeros(3, dtype=torch.bfloat16, device=dev)
    gate, got = ops.router(x, wgt, bias, H, W, R)
    assert torch.equal(got, want)
    assert torch.equal(gate, onehot)


def test_linear_with_selector_weights_is_exact(dev):
    """Weights made of 0 and 1 turn the Linears of the block into exact row arithmetic at their full shapes:
    q / proj / kv / fc1 (K = 384) copy or add channels, fc2 (K = 1536) adds its four K quarters in the kernel's
    documented order."""
    from vtpack_amd import ops
    g = torch.Generator().manual_seed(3)
    L = 27001 if H == 16 else 28703
    a = torch.randn(L, C, generator=g).bfloat16().to(dev)
    eye = torch.eye(C, dtype=torch.bfloat16, device=dev)
    assert torch.equal(ops.linear(a, eye), a)                                          # q / proj shape
    res = torch.randn(L, C, generator=g).bfloat16().to(dev)
    want = (a.float() + res.float()).bfloat16()
    assert torch.equal(ops.linear(a, eye, residual=res), want)
    tokens = torch.randn(B * N, C, generator=g).bfloat16().to(dev)
    w_kv = torch.cat([eye, eye.flip(0)])                                               # kv shape: [768, 384]
    kv = ops.linear(tokens, w_kv)
    assert torch.equal(kv[:, :C], tokens) and torch.equal(kv[:, C:], tokens.flip(1))
    w1 = torch.cat([eye, eye, eye.flip(0), eye])                                       # fc1 shape: [1536, 384]
    hid = ops.linear(a, w1)
    assert torch.equal(hid[:, :C], a) and torch.equal(hid[:, 2 * C:3 * C], a.flip(1))
    w2 = torch.cat([eye, eye, eye, eye], dim=1)                                        # fc2 shape: [384, 1536]
    h4 = torch.randn(L, 4 * C, generator=g).bfloat16().to(dev)
    parts = [h4[:, i * C:(i + 1) * C].float() for i in range(4)]
    bias = torch.randn(C, generator=g).bfloat16().to(dev)
    want = ((((parts[0] + parts[1]) + parts[2]) + parts[3]) + bias.float() + res.float()).bfloat16()
    assert torch.equal(ops.linear(h4, w2, bias, residual=res), want)


def test_attention_of_constant_values_and_sample_isolation(dev, routed):
    """With V constant along the keys the softmax weights sum out: every output row is that constant, whatever
    q and k are.  And a sample's output depends on its own keys and values only."""
    from vtpack_amd import ops
    idx, splits, patches, offsets, lengths = routed
    L = int(offsets[-1])
    g = torch.Generator().manual_seed(4)
    q = torch.randn(L, C, generator=g).bfloat16().to(dev)
    kv = torch.randn(B, N, 2 * C, generator=g).bfloat16().to(dev)
    level = torch.randn(B, 1, C, generator=g).bfloat16().to(dev)
    kv[:, :, C:] = level
    out = ops.sparse_attention(q, kv[:, :, :C], kv[:, :, C:], offsets, 0.125, HEADS, N)
    sample = torch.repeat_interleave(torch.arange(B, device=dev), lengths)
    assert torch.equal(out, level[sample, 0])
    # isolation: new keys and values for the odd samples leave the even samples' rows as they were
    kv2 = torch.randn(B, N, 2 * C, generator=g).bfloat16().to(dev)
    base = ops.sparse_attention(q, kv2[:, :, :C], kv2[:, :, C:], offsets, 0.125, HEADS, N)
    kv2[1::2] = torch.randn(B // 2, N, 2 * C, generator=g).bfloat16().to(dev)
    again = ops.sparse_attention(q, kv2[:, :, :C], kv2[:, :, C:], offsets, 0.125, HEADS, N)
    even = sample % 2 == 0
    assert torch.equal(again[even], base[even])
    assert not torch.equal(again[~even], base[~even])


def test_model_batch_is_its_first_quarter_four_times(dev):
    """The whole forward at the full batch: samples do not see each other, so the logits of the first quarter of the
    images are the logits of those images run alone (same kernels on both sides: each run has well over 2048 packed
    rows per layer), and a second run of the batch returns the same bits."""
    from vtpack_amd.models import dge as zoo
    from vtpack_amd.synthetic import set_synthetic_router, synthetic_images
    torch.manual_seed(0)
    m = zoo.deit_dge_s124_small_patch16_256(img_size=IMG)
    set_synthetic_router(m, 0)
    m = m.eval().to(dev).to(torch.bfloat16)
    img = synthetic_images(B, IMG, seed=0, dtype=torch.bfloat16, device=dev)
    with torch.no_grad():
        full = m(img)
        lens = [blk.dge.states["batches_device"].clone() for blk in m.blocks]
        again = m(img)
        part = m(img[:B // 4].contiguous())
    assert full.shape == (B, 1000) and bool(torch.isfinite(full.float()).all())
    assert torch.equal(full, again)
    assert torch.equal(full[:B // 4], part)
    # the router really mixes grains at this size: between a third and two thirds of the tokens stay queries
    ratio = float(sum(int(l.sum()) for l in lens)) / (len(lens) * B * N)
    assert 0.3 < ratio < 0.7
