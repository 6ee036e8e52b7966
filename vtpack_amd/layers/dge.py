"""DynamicGrainedEncoder / DynamicRouter on the HIP kernels (mirror of vtpack/layers/dge.py).

Module, parameter and `states` key names follow the reference so that its checkpoints and the
code that reads `states` (the transformer block, the complexity counter) keep working.  The
inference branch (argmax gate, sparse compress / decompress; dge.py:74-79, :108-111) runs on the
HIP kernels.  The training branches (Gumbel hard gate; dense compress / decompress, or the sparse
operators with the straight-through gate scaling of `sparse_train`; dge.py:66-72, :91-106) are kept
for API completeness: the router and the dense forms are plain differentiable torch ops there, the
sparse operators use the kernels forward and backward.
"""
import math
from typing import List

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from .grained_sample import (grained_sample_compress, grained_sample_compress_dense, grained_sample_decompress,
                             grained_sample_decompress_dense, grained_sample_index_to_patch)


class Deferred:
    """A value of `states` that is only worked out when somebody reads it (see `States`)."""

    def __init__(self, make):
        self.make = make


class States(dict):
    """The `states` dict of a DynamicGrainedEncoder (vtpack/layers/dge.py:35-38, :81-84).

    The fused inference path never copies the query counts to the host and works on buffers sized for the worst
    case.  It therefore stores `batches` (CPU int64 lengths), `comp`, `patches` and `queries` as `Deferred` values:
    reading one of them performs the device->host copy of the counts and returns what the reference's code expects,
    tensors cut to the live rows.  Code that never reads them never synchronises.

    A Deferred value is worked out on EVERY read and never stored back: the tensors behind it are rewritten by
    each replay of a captured HIP graph (which runs no Python), so a cached count would go stale.  Every way of
    taking values out of the dict resolves them - indexing, get, items, values, pop, popitem, setdefault, copy,
    dict(states), {**states} - so code written against the reference's plain dict never sees a Deferred object."""

    @staticmethod
    def _resolve(value):
        return value.make() if isinstance(value, Deferred) else value

    def __getitem__(self, key):
        return self._resolve(dict.__getitem__(self, key))

    def get(self, key, default=None):
        return self[key] if key in self else default

    # overriding __iter__ / keys also takes dict(states) and {**states} off the C fast path, which would copy the
    # raw values: they then go through keys() and __getitem__
    def __iter__(self):
        return dict.__iter__(self)

    def keys(self):
        return dict.keys(self)

    def items(self):
        return [(k, self[k]) for k in self.keys()]

    def values(self):
        return [self[k] for k in self.keys()]

    def pop(self, key, *default):
        if key in self:
            value = self[key]
            dict.__delitem__(self, key)
            return value
        if default:
            return default[0]
        raise KeyError(key)

    def popitem(self):
        key, value = dict.popitem(self)
        return key, self._resolve(value)

    def setdefault(self, key, default=None):
        if key not in self:
            dict.__setitem__(self, key, default)
        return self[key]

    def copy(self):
        """A plain dict of the values as they are now (a snapshot: later forwards or graph replays do not change
        it)."""
        return {k: self[k] for k in self.keys()}

    snapshot = copy


class DynamicRouter(nn.Module):
    """Region mean -> Linear(C, #splits).  vtpack/layers/dge.py:115-150."""

    def __init__(self, num_channels, split_sizes, init_gate=0.95):
        super().__init__()
        self.num_channels = num_channels
        self.split_sizes = list(split_sizes)
        self.region_size = max(self.split_sizes)
        self.init_gate = init_gate
        self.gate = nn.Linear(num_channels, len(self.split_sizes))
        self.init_parameters()

    def init_parameters(self):
        # dge.py:129-138: tiny weights; bias so that the finest split starts with probability init_gate
        nn.init.trunc_normal_(self.gate.weight, std=.01)
        n = len(self.split_sizes)
        with torch.no_grad():
            if n == 1:
                self.gate.bias.zero_()
            else:
                b = math.log(math.sqrt(self.init_gate * (1 - n) / (self.init_gate - 1)))
                self.gate.bias.fill_(-b)
                self.gate.bias[0] = b

    def complexity(self, num_inputs, num_queries):
        per_region = num_inputs / (self.region_size ** 2) * self.num_channels
        return per_region + per_region * len(self.split_sizes)

    def route(self, x_tokens, H, W):
        """x_tokens [B, extra+H*W, C] -> (gate logits [B,Hr,Wr,S], argmax indices int64 [B,Hr,Wr])."""
        return ops.router(x_tokens, self.gate.weight, self.gate.bias, H, W, self.region_size)

    def forward(self, x):
        """x [B,H,W,C] -> gate logits [B,Hr,Wr,S] (the reference's call form, dge.py:145-150)."""
        B, H, W, C = x.shape
        if self.training or torch.is_grad_enabled() and x.requires_grad:     # differentiable composition
            pooled = F.avg_pool2d(x.permute(0, 3, 1, 2), self.region_size, self.region_size).permute(0, 2, 3, 1)
            return self.gate(pooled)
        return self.route(x.reshape(B, H * W, C), H, W)[0]


class DynamicGrainedEncoder(nn.Module):

    def __init__(self, in_channels: int, split_sizes: List[int], complexity_handler=None, sparse_train: bool = False):
        super().__init__()
        self.in_channels = in_channels
        self.region_size = max(split_sizes)
        for s in split_sizes:
            if s <= 0 or self.region_size % s:
                raise ValueError(f"split size {s} does not divide the region size {self.region_size}")
        self.splits = nn.Parameter(torch.tensor(list(split_sizes), dtype=torch.int64), requires_grad=False)
        self.router = DynamicRouter(in_channels, split_sizes)
        self.complexity_handler = complexity_handler
        self.sparse_train = sparse_train
        self.states = States({"comp": None, "input": None, "patches": None, "batches": None, "gate": None,
                              "size": None, "num_extra_tokens": 0})

    def get_complexity(self):
        # vtpack/layers/dge.py:40-59
        if self.complexity_handler is None:
            return {"static": None, "dynamic": None}
        B, N, _ = self.states["input"].shape
        gate = self.states["gate"]
        if not self.training:
            gate = torch.zeros_like(gate).scatter_(-1, gate.argmax(dim=-1, keepdim=True), 1.0)
        per_region = gate.double() * (self.splits.to(gate.device).double() ** 2)
        num_queries = per_region.reshape(B, -1).sum(-1) + self.states["num_extra_tokens"]
        num_inputs = torch.full_like(num_queries, N)
        router_cost = self.router.complexity(num_inputs, num_queries)
        return {"static": self.complexity_handler(num_inputs, num_inputs) + router_cost,
                "dynamic": self.complexity_handler(num_inputs, num_queries) + router_cost}

    def compress(self, x, H, W, gate=None):
        """x [B, extra+H*W, C] -> packed queries [L, C].  `gate` overrides the router output (tests)."""
        B, N, C = x.shape
        extra = N - H * W
        if self.training:
            # dge.py:64-72: hard Gumbel sample of the gate; every granularity (dense) or the sampled one (sparse)
            if gate is None:
                gate = self.router(x[:, extra:, :].reshape(B, H, W, C))
            gate = F.gumbel_softmax(gate, dim=-1, hard=True)
            if not self.sparse_train:
                comp, batches = grained_sample_compress_dense(x, self.splits, self.region_size, H, W, extra)
                self.states.update({"comp": comp, "input": x, "patches": None, "batches": batches, "gate": gate,
                                    "size": (H, W), "num_extra_tokens": extra})
                return comp
            indices = gate.argmax(dim=-1)
        elif gate is None:
            gate, indices = self.router.route(x, H, W)
        else:
            indices = gate.argmax(dim=-1)
        patches, batches = grained_sample_index_to_patch(indices, self.splits, self.region_size, extra)
        comp = grained_sample_compress(x, patches, H, W, extra)
        self.states.update({"comp": comp, "input": x, "patches": patches, "batches": batches, "gate": gate,
                            "size": (H, W), "num_extra_tokens": extra})
        return comp

    def decompress(self, x):
        """packed [L, C] -> tokens [B, N, C]: input + broadcast(x - comp).  dge.py:87-111."""
        st = self.states
        x = x - st["comp"]
        if self.training and not self.sparse_train:
            return grained_sample_decompress_dense(x, st["gate"], st["input"], self.splits, self.region_size,
                                                   *st["size"], st["num_extra_tokens"], True)
        if self.training:
            # dge.py:96-106: scale each query by its region's (hard, value 1) gate so the router receives a gradient
            B, N, C = st["input"].shape
            extra = st["num_extra_tokens"]
            g = st["gate"].max(dim=-1, keepdim=True)[0]
            g = g.repeat_interleave(self.region_size, 1).repeat_interleave(self.region_size, 2).reshape(B, -1, 1)
            if extra > 0:
                g = torch.cat([g.new_ones([B, extra, 1]), g], dim=1)
            x = x * grained_sample_compress(g, st["patches"], *st["size"], extra)
        return grained_sample_decompress(x, st["patches"], st["input"], *st["size"], st["num_extra_tokens"], True)
