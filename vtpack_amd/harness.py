"""Evaluation-side mirror of the reference's harness for DGE models (vtpack/engine/engine.py, main.py:372-392).

Only what touches the query path is here: the complexity ratio, the budget loss built on it, an `evaluate` loop that
reports the same meters under the same names, and loading a `{"model": state_dict}` checkpoint.  Datasets,
samplers, optimisers, EMA, distillation and logging back-ends stay with the caller.
"""
import torch

from .layers import DynamicGrainedEncoder
from .synthetic import synthetic_images


def unwrap(model):
    """The model itself, or what a DistributedDataParallel-style wrapper holds in `.module`."""
    return model.module if hasattr(model, "module") and isinstance(model.module, torch.nn.Module) else model


def get_complexity(model):
    """dynamic / static complexity over every DynamicGrainedEncoder of the model, after a forward pass.
    vtpack/engine/engine.py:20-32."""
    static, dynamic = [], []
    for m in model.modules():
        if isinstance(m, DynamicGrainedEncoder):
            c = m.get_complexity()
            static.append(c["static"])
            dynamic.append(c["dynamic"])
    return sum(dynamic).mean() / sum(static).mean().clamp(min=1.0)


def budget_loss(model, samples, dge_budget=1.0, dge_lr_scale=1.0):
    """-> (loss_dge, comp_ratio, comp): dge_lr_scale * (dynamic / static - budget)^2 from the model's own complexity
    counter, after a forward pass on `samples`.  vtpack/engine/engine.py:58-63, :121-126.  In training mode the
    gate is the straight-through Gumbel sample, so the loss carries a gradient to every router."""
    comp = unwrap(model).complexity(samples)
    ratio = comp["dynamic"] / comp["static"].clamp(min=1.0)
    return dge_lr_scale * (ratio - dge_budget) ** 2, ratio, comp


class _Meter:
    """Running total / count: the `global_avg` of the reference's SmoothedValue (vtpack/engine/utils.py)."""

    def __init__(self):
        self.total, self.count = 0.0, 0

    def update(self, value, n=1):
        self.total += value * n
        self.count += n

    @property
    def global_avg(self):
        return self.total / max(self.count, 1)


def accuracy(output, target, topk=(1,)):
    """Top-k accuracies in percent (timm.utils.accuracy, as engine.py:133 calls it)."""
    maxk = min(max(topk), output.shape[1])
    pred = output.topk(maxk, dim=1).indices.t()
    correct = pred.eq(target.reshape(1, -1))
    return [correct[:min(k, maxk)].reshape(-1).float().sum() * 100.0 / target.shape[0] for k in topk]


@torch.no_grad()
def evaluate(data_loader, model, device, dge_enable=False, dge_budget=1.0, dge_lr_scale=1.0):
    """vtpack/engine/engine.py:102-147: eval mode, one forward per (images, target) batch, cross-entropy, top-1 / top-5
    and, with `dge_enable`, the complexity meters.  Returns {meter name: global average} with the reference's names:
    loss, acc1, acc5 and loss_cls, loss_dge, dge_ratio, comp_static, comp_dynamic."""
    criterion = torch.nn.CrossEntropyLoss()
    meters = {}

    def update(name, value, n=1):
        meters.setdefault(name, _Meter()).update(float(value), n)

    model.eval()
    for images, target in data_loader:
        images = images.to(device, non_blocking=True)
        target = target.to(device, non_blocking=True)
        output = model(images)
        loss_cls = criterion(output.float(), target)
        loss = loss_cls
        if dge_enable:
            loss_dge, ratio, comp = budget_loss(model, images, dge_budget, dge_lr_scale)
            loss = loss_dge + loss_cls
            update("loss_cls", loss_cls)
            update("loss_dge", loss_dge)
            update("dge_ratio", ratio)
            update("comp_static", comp["static"])
            update("comp_dynamic", comp["dynamic"])
        acc1, acc5 = accuracy(output, target, topk=(1, 5))
        update("loss", loss)
        update("acc1", acc1, n=images.shape[0])
        update("acc5", acc5, n=images.shape[0])
    return {k: m.global_avg for k, m in meters.items()}


def load_checkpoint(model, path, strict=True):
    """Load the `"model"` entry of a checkpoint written as main.py:430-440 writes it (`{"model": state_dict, ...}`),
    as main.py:372-379 reads it, with a loader that executes nothing from the file.  A bare state dict is accepted
    too.  Returns the rest of the checkpoint (epoch, optimiser state, ... when present)."""
    ckpt = torch.load(path, map_location="cpu", weights_only=True)
    sd = ckpt["model"] if isinstance(ckpt, dict) and "model" in ckpt else ckpt
    unwrap(model).load_state_dict(sd, strict=strict)
    return {k: v for k, v in ckpt.items() if k != "model"} if sd is not ckpt else {}


def synthetic_loader(batches, batch_size, image_size, num_classes=1000, seed=0, dtype=torch.float32):
    """A stand-in for the ImageNet validation loader: `batches` batches of seeded synthetic images with seeded labels."""
    g = torch.Generator().manual_seed(seed)
    for i in range(batches):
        yield (synthetic_images(batch_size, image_size, seed=seed * 1000 + i, dtype=dtype),
               torch.randint(0, num_classes, (batch_size,), generator=g))
