#!/usr/bin/env python3
"""Writes tests/golden/dge_block_b2_c64.npz: one DGE block (C=64, 1 head, batch 2, injected gate logits)
evaluated by the CPU oracle.  Run from the repository root:  python tests/golden/make_golden.py

The reference itself cannot produce these vectors in this environment (its operators exist only as CUDA
kernels and its Python needs the compiled module plus timm), so they come from the restatement in oracle/,
after that restatement passed tests/test_oracle_pins.py.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

import recipe  # noqa: E402
from oracle import torch_ref  # noqa: E402


def main():
    x, gate = recipe.inputs()
    tr = {}
    out = torch_ref.block_forward(recipe.state_dict(), "", torch.from_numpy(x), recipe.HEADS,
                                  gate=torch.from_numpy(gate), trace=tr)
    np.savez(os.path.join(HERE, recipe.FIXTURE), indices=tr["indices"].numpy(), lengths=tr["lengths"].numpy(),
             patches=tr["patches"].numpy(), comp=tr["comp"].numpy(), attn=tr["attn"].numpy(), q2=tr["q2"].numpy(),
             out=out.numpy())
    print("wrote", recipe.FIXTURE, "L =", int(tr["lengths"].sum()))


if __name__ == "__main__":
    main()
