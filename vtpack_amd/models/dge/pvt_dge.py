"""Pyramid Vision Transformer + Dynamic Grained Encoder (vtpack/models/dge/pvt_dge.py), the second caller of
the query path: four stages of differing width, no extra tokens before the last stage, and keys/values taken
from a spatially reduced token grid (KV length != number of tokens).

Self-contained (no timm).  Sub-module and parameter names are the reference's (`patch_embed{i}`, `pos_embed{i}`,
`block{i}.{j}.attn.sr`, ...), so its state dicts load unchanged.  As for DeiT, every block runs either in layer
mode (the reference's composition around the `vtpack.layers` operators) or fused on libvtdge
(`vtpack_amd.engine.block_forward`, default); in training mode it runs the reference's training composition.
"""
from functools import partial

import torch
import torch.nn.functional as F
from torch import nn

from ... import engine
from ...layers import DynamicGrainedEncoder
from ...layers.sparse_ops import batched_sparse_attention, sparse_attention_train
from .deit_dge import Mlp

__all__ = ["PyramidVisionTransformer", "Block", "Attention", "PatchEmbed", "pvt_dge_s124_tiny", "pvt_dge_s124_small",
           "pvt_dge_s124_tiny_256", "pvt_dge_s124_small_256", "pvt_dge_s124_medium_256", "pvt_dge_s124_large_256"]


class Attention(nn.Module):
    """q from the packed queries; k, v from all tokens, or from the sr x sr reduced grid when sr_ratio > 1."""

    def __init__(self, dim, num_heads=8, qkv_bias=False, qk_scale=None, sr_ratio=1):
        super().__init__()
        if dim % num_heads:
            raise ValueError(f"dim {dim} should be divided by num_heads {num_heads}.")
        self.dim, self.num_heads = dim, num_heads
        self.scale = qk_scale or (dim // num_heads) ** -0.5
        self.q = nn.Linear(dim, dim, bias=qkv_bias)
        self.kv = nn.Linear(dim, dim * 2, bias=qkv_bias)
        self.proj = nn.Linear(dim, dim)
        self.sr_ratio = sr_ratio
        if sr_ratio > 1:
            self.sr = nn.Conv2d(dim, dim, kernel_size=sr_ratio, stride=sr_ratio)
            self.norm = nn.LayerNorm(dim)

    def complexity(self, num_inputs, num_queries):
        # pvt_dge.py:65-75
        c, r2 = self.dim, self.sr_ratio ** 2
        comp = num_queries * c * c
        if self.sr_ratio > 1:
            comp = comp + num_inputs * c * c + num_inputs / r2 * c
        comp = comp + num_inputs / r2 * c * c * 2
        comp = comp + num_queries * num_inputs / r2 * c
        comp = comp + num_queries * num_inputs / r2 * self.num_heads * 3
        return comp + num_queries * c * c

    def forward(self, x, q, H, W, q_lengths):
        # pvt_dge.py:77-92,108 
        B, N, C = x.shape
        h, d = self.num_heads, C // self.num_heads
        q = self.q(q).reshape(-1, h, d).permute(1, 0, 2)
        if self.sr_ratio > 1:
            x = self.sr(x.permute(0, 2, 1).reshape(B, C, H, W)).reshape(B, C, -1).permute(0, 2, 1)
            x = self.norm(x)
        kv = self.kv(x).reshape(B, -1, 2, h, d).permute(2, 3, 0, 1, 4)
        if self.training:
            return self.proj(sparse_attention_train(q, kv[0], kv[1], q_lengths, self.scale))
        o = batched_sparse_attention(q, kv[0], kv[1], q_lengths, self.scale)
        return self.proj(o.transpose(0, 1).reshape(-1, C))


class Block(nn.Module):
    def __init__(self, dim, num_heads, mlp_ratio=4., qkv_bias=False, qk_scale=None, norm_layer=nn.LayerNorm,
                 sr_ratio=1, split_sizes=(2, 1), fused=True):
        super().__init__()
        self.dim = dim
        self.fused = fused
        self.norm1 = norm_layer(dim)
        self.attn = Attention(dim, num_heads=num_heads, qkv_bias=qkv_bias, qk_scale=qk_scale, sr_ratio=sr_ratio)
        self.norm2 = norm_layer(dim)
        self.mlp = Mlp(dim, int(dim * mlp_ratio))
        self.dge = DynamicGrainedEncoder(dim, list(split_sizes), complexity_handler=self.complexity)

    def complexity(self, num_inputs, num_queries):
        # pvt_dge.py:128-132
        return (num_inputs * self.dim * 2 + self.attn.complexity(num_inputs, num_queries)
                + self.mlp.complexity(num_inputs, num_queries))

    def forward(self, x, H, W, gate=None):
        # pvt_dge.py:134-140
        if self.fused and not self.training:
            return engine.block_forward(self, x, H, W, gate=gate)
        q = self.dge.compress(x, H, W, gate=gate)
        q = q + self.attn(self.norm1(x), self.norm1(q), H, W, self.dge.states["batches"])
        q = q + self.mlp(self.norm2(q))
        return self.dge.decompress(q)


class PatchEmbed(nn.Module):
    """Stride-k k x k convolution + LayerNorm; returns tokens and their grid.  pvt_dge.py:143-174."""

    def __init__(self, img_size=224, patch_size=16, in_chans=3, embed_dim=768):
        super().__init__()
        self.img_size, self.patch_size = (img_size, img_size), (patch_size, patch_size)
        self.H, self.W = img_size // patch_size, img_size // patch_size
        self.num_patches = self.H * self.W
        self.proj = nn.Conv2d(in_chans, embed_dim, kernel_size=patch_size, stride=patch_size)
        self.norm = nn.LayerNorm(embed_dim)

    def complexity(self, num_inputs, num_queries):
        comp = num_inputs * self.proj.in_channels * self.proj.out_channels
        return comp + num_inputs / (self.patch_size[0] * self.patch_size[1]) * self.proj.out_channels

    def forward(self, x):
        H, W = x.shape[2] // self.patch_size[0], x.shape[3] // self.patch_size[1]
        return self.norm(self.proj(x).flatten(2).transpose(1, 2)), (H, W)


class PyramidVisionTransformer(nn.Module):
    def __init__(self, img_size=224, patch_size=16, in_chans=3, num_classes=1000, embed_dims=(64, 128, 256, 512),
                 num_heads=(1, 2, 4, 8), mlp_ratios=(4, 4, 4, 4), qkv_bias=False, qk_scale=None, norm_layer=nn.LayerNorm,
                 depths=(3, 4, 6, 3), sr_ratios=(8, 4, 2, 1), num_stages=4,
                 split_sizes=((2, 1), (2, 1), (2, 1), (2, 1)), fused=True):
        super().__init__()
        self.embed_dims, self.num_classes, self.depths, self.num_stages = list(embed_dims), num_classes, list(depths), \
            num_stages
        self.fused = fused
        last = num_stages - 1
        for i in range(num_stages):
            pe = PatchEmbed(img_size if i == 0 else img_size // (2 ** (i + 1)), patch_size if i == 0 else 2,
                            in_chans if i == 0 else embed_dims[i - 1], embed_dims[i])
            setattr(self, f"patch_embed{i + 1}", pe)
            setattr(self, f"pos_embed{i + 1}",
                    nn.Parameter(torch.zeros(1, pe.num_patches + (1 if i == last else 0), embed_dims[i])))
            setattr(self, f"block{i + 1}", nn.ModuleList([
                Block(embed_dims[i], num_heads[i], mlp_ratios[i], qkv_bias, qk_scale, norm_layer, sr_ratios[i],
                      split_sizes[i], fused) for _ in range(depths[i])]))
        self.norm = norm_layer(embed_dims[last]) if num_classes > 0 else nn.Identity()
        self.cls_token = nn.Parameter(torch.zeros(1, 1, embed_dims[last]))
        self.head = nn.Linear(embed_dims[last], num_classes) if num_classes > 0 else nn.Identity()
        self._init_weights()

    def _init_weights(self):
        # pvt_dge.py:226-244: trunc_normal(.02) Linear weights and embeddings, zero biases, unit LayerNorm, router init
        for i in range(self.num_stages):
            nn.init.trunc_normal_(getattr(self, f"pos_embed{i + 1}"), std=.02)
        nn.init.trunc_normal_(self.cls_token, std=.02)
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
        for m in self.modules():
            if isinstance(m, Block):
                m.fused = fused
        return self

    def complexity(self, x):
        # pvt_dge.py:246-266; call after a forward pass on x
        n = x.shape[1] * x.shape[2]
        comp = self.embed_dims[-1] * self.num_classes
        for i in range(self.num_stages):
            pe = getattr(self, f"patch_embed{i + 1}")
            comp = comp + pe.complexity(n, n)
            n = n / (pe.patch_size[0] * pe.patch_size[1])
        per = [m.get_complexity() for m in self.modules() if isinstance(m, DynamicGrainedEncoder)]
        return {"static": (sum(p["static"] for p in per) + comp).mean(),
                "dynamic": (sum(p["dynamic"] for p in per) + comp).mean()}

    def _get_pos_embed(self, pos_embed, patch_embed, H, W):
        # pvt_dge.py:281-288
        if H * W == patch_embed.num_patches:
            return pos_embed
        grid = pos_embed.reshape(1, patch_embed.H, patch_embed.W, -1).permute(0, 3, 1, 2)
        return F.interpolate(grid, size=(H, W), mode="bilinear", align_corners=False).reshape(1, -1, H * W) \
            .permute(0, 2, 1)

    def forward_features(self, x):
        # pvt_dge.py:290-330
        B = x.shape[0]
        outputs = {}
        last = self.num_stages - 1
        for i in range(self.num_stages):
            pe = getattr(self, f"patch_embed{i + 1}")
            pos = getattr(self, f"pos_embed{i + 1}")
            x, (H, W) = pe(x)
            if i == last:
                x = torch.cat((self.cls_token.expand(B, -1, -1), x), dim=1)
                pos = torch.cat((pos[:, 0:1], self._get_pos_embed(pos[:, 1:], pe, H, W)), dim=1)
            else:
                pos = self._get_pos_embed(pos, pe, H, W)
            x = x + pos
            for blk in getattr(self, f"block{i + 1}"):
                x = blk(x, H, W)
            if i != last:
                x = x.reshape(B, H, W, -1).permute(0, 3, 1, 2).contiguous()
                outputs[f"res{i + 2}"] = x
            elif self.num_classes == 0:
                outputs[f"res{i + 2}"] = x[:, 1:].reshape(B, H, W, -1).permute(0, 3, 1, 2).contiguous()
        if self.num_classes == 0:
            return outputs
        return self.norm(x)[:, 0]

    def forward(self, x):
        if self.fused and not self.training:
            return engine.pvt_forward(self, x)
        x = self.forward_features(x)
        return self.head(x) if self.num_classes > 0 else x


def _pvt_dge_s124(depths, **kwargs):
    return PyramidVisionTransformer(
        patch_size=4, embed_dims=[64, 128, 320, 512], num_heads=[1, 2, 5, 8], mlp_ratios=[8, 8, 4, 4], qkv_bias=True,
        norm_layer=partial(nn.LayerNorm, eps=1e-6), depths=depths, sr_ratios=[8, 4, 2, 1],
        split_sizes=[[4, 2, 1]] * 4, **kwargs)


def pvt_dge_s124_tiny(pretrained=False, **kwargs):
    return _pvt_dge_s124([2, 2, 2, 2], **kwargs)


def pvt_dge_s124_small(pretrained=False, **kwargs):
    return _pvt_dge_s124([3, 4, 6, 3], **kwargs)


def pvt_dge_s124_tiny_256(pretrained=False, **kwargs):
    kwargs.setdefault("img_size", 256)
    return _pvt_dge_s124([2, 2, 2, 2], **kwargs)


def pvt_dge_s124_small_256(pretrained=False, **kwargs):
    kwargs.setdefault("img_size", 256)
    return _pvt_dge_s124([3, 4, 6, 3], **kwargs)


def pvt_dge_s124_medium_256(pretrained=False, **kwargs):
    kwargs.setdefault("img_size", 256)
    return _pvt_dge_s124([3, 4, 18, 3], **kwargs)


def pvt_dge_s124_large_256(pretrained=False, **kwargs):
    kwargs.setdefault("img_size", 256)
    return _pvt_dge_s124([3, 8, 27, 3], **kwargs)
