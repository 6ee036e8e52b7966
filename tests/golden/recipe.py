"""Deterministic inputs of the golden fixture (numpy RandomState streams are frozen across versions)."""
import numpy as np
import torch

B, H, W, EXTRA, C, HEADS = 2, 16, 16, 1, 64, 1
SPLITS = [4, 2, 1]
FIXTURE = "dge_block_b2_c64.npz"


def inputs():
    r = np.random.RandomState(20211206)
    x = r.standard_normal((B, EXTRA + H * W, C)).astype(np.float32)
    gate = r.standard_normal((B, H // 4, W // 4, 3)).astype(np.float32)
    return x, gate


def state_dict():
    r = np.random.RandomState(777)
    n = lambda *s, std=1.0: torch.from_numpy((r.standard_normal(s) * std).astype(np.float32))  # noqa: E731
    sd = {}
    for name in ("norm1", "norm2"):
        sd[f"{name}.weight"] = 1.0 + n(C, std=0.1)
        sd[f"{name}.bias"] = n(C, std=0.1)
    for name, (o, i) in {"attn.q": (C, C), "attn.kv": (2 * C, C), "attn.proj": (C, C), "mlp.fc1": (4 * C, C),
                         "mlp.fc2": (C, 4 * C)}.items():
        sd[f"{name}.weight"] = n(o, i, std=0.08)
        sd[f"{name}.bias"] = n(o, std=0.05)
    sd["dge.splits"] = torch.tensor(SPLITS, dtype=torch.int64)
    sd["dge.router.gate.weight"] = n(3, C, std=0.1)
    sd["dge.router.gate.bias"] = torch.zeros(3)
    return sd
