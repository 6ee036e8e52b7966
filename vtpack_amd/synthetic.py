"""Synthetic inputs and router settings for benchmarks and tests (no dataset, no checkpoint).

A randomly initialised DGE router always picks the finest split (its bias starts at +-1.82 in favour
of split 0, vtpack/layers/dge.py:135-138), which would make every benchmark a dense DeiT.  The
"budget 0.5" operating point of the trained models is emulated by zeroing the router bias and
drawing its weights at random, so that each region's argmax is close to uniform over the splits
(expected query count 1 + 7 per region, complexity ratio ~0.52 by the reference's own counter).
"""
import torch

IMAGENET_MEAN = (0.485, 0.456, 0.406)
IMAGENET_STD = (0.229, 0.224, 0.225)


def synthetic_images(batch, size, seed=0, dtype=torch.float32, device="cpu"):
    """Pixels ~ U(0,1), normalised per channel with the ImageNet statistics (vtpack/engine/datasets.py:108)."""
    g = torch.Generator().manual_seed(seed)
    img = torch.rand((batch, 3, size, size), generator=g)
    mean = torch.tensor(IMAGENET_MEAN).view(1, 3, 1, 1)
    std = torch.tensor(IMAGENET_STD).view(1, 3, 1, 1)
    return ((img - mean) / std).to(device=device, dtype=dtype)


def set_synthetic_router(model, seed=0):
    """Zero bias + seeded N(0, 1/C) weights for every block's router (mixed gate instead of all-fine)."""
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for mod in model.modules():
            if not hasattr(mod, "router") or not hasattr(mod, "splits"):
                continue                       # every DynamicGrainedEncoder, in execution order
            lin = mod.router.gate
            w = torch.randn(lin.weight.shape, generator=g) / lin.weight.shape[1] ** 0.5
            lin.weight.copy_(w.to(lin.weight.dtype))
            lin.bias.zero_()
    return model
