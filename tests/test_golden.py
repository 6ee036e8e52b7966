"""Committed golden vectors (tests/golden/): the oracle reproduces them on any box, the HIP path matches them."""
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import recipe  # noqa: E402

from oracle import dge_oracle as orc  # noqa: E402
from oracle import torch_ref  # noqa: E402
from util import FP32_REL, rel_err  # noqa: E402


@pytest.fixture(scope="module")
def gold():
    return dict(np.load(os.path.join(HERE, "golden", recipe.FIXTURE), allow_pickle=False))


def test_oracle_reproduces_golden(gold):
    x, gate = recipe.inputs()
    # integer part through the C restatement
    idx = gate.argmax(-1)
    assert np.array_equal(idx, gold["indices"])
    p, l = orc.index_to_patch(idx, recipe.SPLITS, 4, recipe.EXTRA)
    assert np.array_equal(p, gold["patches"]) and np.array_equal(l, gold["lengths"])
    np.testing.assert_allclose(orc.compress(x, p, recipe.H, recipe.W, recipe.EXTRA), gold["comp"], atol=1e-6)
    # whole block through the torch restatement (library GEMMs: tolerance, not bit equality)
    tr = {}
    out = torch_ref.block_forward(recipe.state_dict(), "", torch.from_numpy(x), recipe.HEADS,
                                  gate=torch.from_numpy(gate), trace=tr)
    assert rel_err(tr["attn"], gold["attn"]) <= FP32_REL
    assert rel_err(out, gold["out"]) <= FP32_REL


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [True, False])
def test_hip_block_matches_golden(dev, gold, fused):
    from vtpack_amd.models.dge.deit_dge import Block
    blk = Block(recipe.C, recipe.HEADS, mlp_ratio=4, qkv_bias=True,
                norm_layer=lambda d: torch.nn.LayerNorm(d, eps=1e-6), split_sizes=recipe.SPLITS, fused=fused)
    blk.load_state_dict(recipe.state_dict())
    blk = blk.eval().to(dev)
    x, gate = recipe.inputs()
    with torch.no_grad():
        out = blk(torch.from_numpy(x).to(dev), gate=torch.from_numpy(gate).to(dev))
    st = blk.dge.states
    L = int(gold["lengths"].sum())
    assert np.array_equal(st["patches"][:L].cpu().numpy(), gold["patches"])
    lengths = st["batches"] if st["batches"] is not None else st["batches_device"].cpu()
    assert np.array_equal(lengths.numpy(), gold["lengths"])
    assert np.array_equal(st["comp"][:L].cpu().numpy(), gold["comp"])
    assert rel_err(out, gold["out"]) <= FP32_REL
