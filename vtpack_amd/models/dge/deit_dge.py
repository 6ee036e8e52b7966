"""DeiT + Dynamic Grained Encoder, the caller of the query path (vtpack/models/dge/deit_dge.py).

Self-contained (no timm): the patch embedding is the Conv2d(3, C, 16, stride 16) timm's PatchEmbed
wraps, DropPath/Dropout are identities at inference.  Sub-module and parameter names are the
reference's, so its state dicts load with `load_state_dict` unchanged.

In training mode a block runs the reference's training composition (Gumbel-sampled gate, dense or sparse
operators, differentiable attention; deit_dge.py:79-95) with torch autograd around the operators.

Every block can run two ways at inference:
  * layer mode  - the reference's composition (deit_dge.py:123-130): nn.LayerNorm / nn.Linear from
    torch around the `vtpack.layers` operators, one device->host copy of the query counts per block;
  * fused mode (default) - the whole block on libvtdge kernels with the query count kept on the
    device, see `vtpack_amd.engine.block_forward`.
"""
import math
from collections import OrderedDict
from functools import partial

import torch
from torch import nn

from ... import engine
from ...layers import DynamicGrainedEncoder
from ...layers.sparse_ops import batched_sparse_attention, sparse_attention_train

__all__ = ["VisionTransformer", "Block", "Attention", "Mlp", "PatchEmbed", "deit_dge_s124_tiny_patch16_256",
           "deit_dge_s124_small_patch16_256", "deit_dge_s124_base_patch16_256"]


class Mlp(nn.Module):
    def __init__(self, in_features, hidden_features=None, out_features=None):
        super().__init__()
        self.fc1 = nn.Linear(in_features, hidden_features or in_features)
        self.act = nn.GELU()
        self.fc2 = nn.Linear(hidden_features or in_features, out_features or in_features)

    def complexity(self, num_inputs, num_queries):
        # deit_dge.py:32-36
        f1, f2 = self.fc1, self.fc2
        return num_queries * (f1.in_features * f1.out_features + f1.out_features + f2.in_features * f2.out_features)

    def forward(self, x):
        return self.fc2(self.act(self.fc1(x)))


class Attention(nn.Module):
    """Separate q and kv projections; packed queries attend to every token of their own sample."""

    def __init__(self, dim, num_heads=8, qkv_bias=False, qk_scale=None):
        super().__init__()
        self.dim, self.num_heads = dim, num_heads
        self.scale = qk_scale or (dim // num_heads) ** -0.5
        self.q = nn.Linear(dim, dim, bias=qkv_bias)
        self.kv = nn.Linear(dim, dim * 2, bias=qkv_bias)
        self.proj = nn.Linear(dim, dim)

    def complexity(self, num_inputs, num_queries):
        # deit_dge.py:61-68
        c = self.dim
        return (num_queries * c * c + 2 * num_inputs * c * c + 2 * num_queries * num_inputs * c
                + 3 * num_queries * num_inputs * self.num_heads + num_queries * c * c)

    def forward(self, x, q, q_lengths):
        # deit_dge.py:70-78,96 
        B, N, C = x.shape
        h, d = self.num_heads, C // self.num_heads
        q = self.q(q).reshape(-1, h, d).permute(1, 0, 2)
        kv = self.kv(x).reshape(B, N, 2, h, d).permute(2, 3, 0, 1, 4)
        if self.training:
            return self.proj(sparse_attention_train(q, kv[0], kv[1], q_lengths, self.scale))
        o = batched_sparse_attention(q, kv[0], kv[1], q_lengths, self.scale)
        return self.proj(o.transpose(0, 1).reshape(-1, C))


class Block(nn.Module):
    def __init__(self, dim, num_heads, mlp_ratio=4., qkv_bias=False, qk_scale=None, norm_layer=nn.LayerNorm,
                 split_sizes=(2, 1), fused=True):
        super().__init__()
        self.dim = dim
        self.fused = fused
        self.norm1 = norm_layer(dim)
        self.attn = Attention(dim, num_heads=num_heads, qkv_bias=qkv_bias, qk_scale=qk_scale)
        self.norm2 = norm_layer(dim)
        self.mlp = Mlp(dim, int(dim * mlp_ratio))
        self.dge = DynamicGrainedEncoder(dim, list(split_sizes), complexity_handler=self.complexity)

    def complexity(self, num_inputs, num_queries):
        # deit_dge.py:117-121
        return (num_inputs * self.dim * 2 + self.attn.complexity(num_inputs, num_queries)
                + self.mlp.complexity(num_inputs, num_queries))

    def forward(self, x, gate=None):
        B, N, C = x.shape
        H = W = int(math.sqrt(N))
        if self.fused and not self.training:
            return engine.block_forward(self, x, H, W, gate=gate)
        q = self.dge.compress(x, H, W, gate=gate)
        q = q + self.attn(self.norm1(x), self.norm1(q), self.dge.states["batches"])
        q = q + self.mlp(self.norm2(q))
        return self.dge.decompress(q)


class PatchEmbed(nn.Module):
    """Non-overlapping patches -> tokens (what timm's PatchEmbed does for the reference, deit_dge.py:176-177)."""

    def __init__(self, img_size=224, patch_size=16, in_chans=3, embed_dim=768):
        super().__init__()
        self.img_size, self.patch_size = (img_size, img_size), (patch_size, patch_size)
        self.grid_size = (img_size // patch_size, img_size // patch_size)
        self.num_patches = self.grid_size[0] * self.grid_size[1]
        self.proj = nn.Conv2d(in_chans, embed_dim, kernel_size=patch_size, stride=patch_size)

    def forward(self, x):
        if tuple(x.shape[-2:]) != self.img_size:
            raise ValueError(f"input {tuple(x.shape[-2:])} does not match the model's image size {self.img_size}")
        return self.proj(x).flatten(2).transpose(1, 2)


class VisionTransformer(nn.Module):
    """vtpack/models/dge/deit_dge.py:133-299: class token, optional distillation token and second head
    (`distilled`), optional pre-logits layer (`representation_size`, ignored with `distilled` as in the reference),
    optional absence of the class token (`cls_token=False`: the head sees the mean over the tokens)."""

    def __init__(self, img_size=224, patch_size=16, in_chans=3, num_classes=1000, embed_dim=768, depth=12,
                 num_heads=12, mlp_ratio=4., qkv_bias=True, qk_scale=None, representation_size=None, distilled=False,
                 drop_rate=0., attn_drop_rate=0., drop_path_rate=0., norm_layer=None, cls_token=True,
                 split_sizes=(2, 1), fused=True):
        super().__init__()
        # Dropout / stochastic depth are identities at inference; the rates are kept so that a training-mode forward
        # can refuse them instead of silently training without the regularisers.
        self.drop_rates = (drop_rate, attn_drop_rate, drop_path_rate)
        self.num_classes = num_classes
        self.num_features = self.embed_dim = embed_dim
        self.num_tokens = (1 if cls_token else 0) + (1 if distilled else 0)
        norm_layer = norm_layer or partial(nn.LayerNorm, eps=1e-6)
        self.patch_embed = PatchEmbed(img_size, patch_size, in_chans, embed_dim)
        self.cls_token = nn.Parameter(torch.zeros(1, 1, embed_dim)) if cls_token else None
        self.dist_token = nn.Parameter(torch.zeros(1, 1, embed_dim)) if distilled else None
        self.pos_embed = nn.Parameter(torch.zeros(1, self.patch_embed.num_patches + self.num_tokens, embed_dim))
        self.blocks = nn.Sequential(*[
            Block(embed_dim, num_heads, mlp_ratio, qkv_bias, qk_scale, norm_layer, split_sizes, fused)
            for _ in range(depth)])
        self.norm = norm_layer(embed_dim)
        if representation_size and not distilled:
            self.num_features = representation_size
            self.pre_logits = nn.Sequential(OrderedDict([("fc", nn.Linear(embed_dim, representation_size)),
                                                         ("act", nn.Tanh())]))
        else:
            self.pre_logits = nn.Identity()
        self.head = nn.Linear(self.num_features, num_classes) if num_classes > 0 else nn.Identity()
        self.head_dist = None
        if distilled:
            self.head_dist = nn.Linear(embed_dim, num_classes) if num_classes > 0 else nn.Identity()
        self.fused = fused
        self._init_weights()

    def _init_weights(self):
        # timm's _init_vit_weights for the default scheme: trunc_normal(.02) weights, zero biases, unit LayerNorm
        nn.init.trunc_normal_(self.pos_embed, std=.02)
        for tok in (self.cls_token, self.dist_token):
            if tok is not None:
                nn.init.trunc_normal_(tok, std=.02)
        for m in self.modules():
            if isinstance(m, nn.Linear):
                nn.init.trunc_normal_(m.weight, std=.02)
                if m.bias is not None:
                    nn.init.zeros_(m.bias)
            elif isinstance(m, nn.LayerNorm):
                nn.init.ones_(m.weight)
                nn.init.zeros_(m.bias)
        for m in self.modules():
            if isinstance(m, DynamicGrainedEncoder):
                m.router.init_parameters()

    def set_fused(self, fused):
        self.fused = fused
        for blk in self.blocks:
            blk.fused = fused
        return self

    def no_weight_decay(self):
        return {"pos_embed", "cls_token"}

    def get_classifier(self):
        return self.head if self.dist_token is None else (self.head, self.head_dist)

    def reset_classifier(self, num_classes, global_pool=""):
        self.num_classes = num_classes
        self.head = nn.Linear(self.embed_dim, num_classes) if num_classes > 0 else nn.Identity()
        if self.num_tokens == 2:
            self.head_dist = nn.Linear(self.embed_dim, num_classes) if num_classes > 0 else nn.Identity()

    def complexity(self, x):
        # deit_dge.py:234-249; call after a forward pass on x
        n = x.shape[1] * x.shape[2]
        base = n * self.num_features * 3 + self.num_features * self.num_classes
        per = [blk.dge.get_complexity() for blk in self.blocks]
        return {"static": (sum(p["static"] for p in per) + base).mean(),
                "dynamic": (sum(p["dynamic"] for p in per) + base).mean()}

    def embed_tokens(self, x):
        """Patch tokens with the extra tokens in front (class, then distillation) plus the positions."""
        x = self.patch_embed(x)
        front = [t.expand(x.shape[0], -1, -1) for t in (self.cls_token, self.dist_token) if t is not None]
        if self.cls_token is None and self.dist_token is not None:
            raise ValueError("a distillation token needs a class token (deit_dge.py:270-275)")
        return torch.cat(front + [x], dim=1) + self.pos_embed

    def forward_features(self, x):
        x = self.norm(self.blocks(self.embed_tokens(x)))
        if self.cls_token is None:
            return x
        if self.dist_token is None:
            return self.pre_logits(x[:, 0])
        return x[:, 0], x[:, 1]

    def classify(self, feats):
        """deit_dge.py:286-299 on the output of forward_features."""
        if self.head_dist is not None:
            a, b = self.head(feats[0]), self.head_dist(feats[1])
            return (a, b) if self.training else (a + b) / 2
        return self.head(feats if self.cls_token is not None else feats.mean(dim=1))

    def forward(self, x):
        if self.fused and not self.training:
            return engine.model_forward(self, x)
        if self.training and any(self.drop_rates):
            raise NotImplementedError("dropout / stochastic depth in training mode are not part of this package")
        return self.classify(self.forward_features(x))


def _deit_dge_s124(embed_dim, num_heads, **kwargs):
    kwargs.setdefault("img_size", 256)
    return VisionTransformer(patch_size=16, embed_dim=embed_dim, depth=12, num_heads=num_heads, mlp_ratio=4,
                             qkv_bias=True, norm_layer=partial(nn.LayerNorm, eps=1e-6), split_sizes=[4, 2, 1],
                             **kwargs)


def deit_dge_s124_tiny_patch16_256(pretrained=False, **kwargs):
    return _deit_dge_s124(192, 3, **kwargs)


def deit_dge_s124_small_patch16_256(pretrained=False, **kwargs):
    return _deit_dge_s124(384, 6, **kwargs)


def deit_dge_s124_base_patch16_256(pretrained=False, **kwargs):
    return _deit_dge_s124(768, 12, **kwargs)
