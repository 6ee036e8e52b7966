"""Shared helpers of the parity tests."""
import numpy as np
import torch

SPLITS = [4, 2, 1]

# Tolerances of the floating-point comparisons (integer outputs are always compared bit-exactly):
#   fp32: max|got - want| <= 1e-5 * max|want|   ("1e-5 relative", measured against the tensor's scale)
#   bf16: max|got - want| <= 2e-2               (max-abs, against the fp32 oracle fed the same bf16 inputs)
FP32_REL = 1e-5
BF16_ABS = 2e-2


def rel_err(got, want):
    got = torch.as_tensor(got).double().cpu()
    want = torch.as_tensor(want).double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def abs_err(got, want):
    return float((torch.as_tensor(got).double().cpu() - torch.as_tensor(want).double().cpu()).abs().max())


def assert_close(got, want, dtype, what=""):
    if dtype == torch.float32:
        e = rel_err(got, want)
        assert e <= FP32_REL, f"{what}: fp32 relative error {e:.3e} > {FP32_REL}"
    else:
        e = abs_err(got, want)
        assert e <= BF16_ABS, f"{what}: bf16 max-abs error {e:.3e} > {BF16_ABS}"


def rng(seed):
    return np.random.RandomState(seed)


def random_indices(seed, B, Hr, Wr, S=3, p=None):
    return rng(seed).choice(S, size=(B, Hr, Wr), p=p).astype(np.int64)


def randn(seed, *shape):
    return rng(seed).standard_normal(shape).astype(np.float32)


def bf16_round(a):
    """fp32 numpy -> the fp32 value of its bf16 rounding (round to nearest even), via torch."""
    return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).float().numpy()


def forced_reference(model, images, heads, depth):
    """The CPU restatement of a DeiT+DGE forward with the GPU run's gate choices forced (read from the model's
    `states` after its forward): -> (logits, per-layer traces).  Every layer's trace also carries the logits the CPU
    path's own router computes on its own activations (`gate_free`)."""
    from oracle import torch_ref
    sd = torch_ref.float_state_dict(model)
    forced = [blk.dge.states["gate"].float().argmax(-1).cpu() for blk in model.blocks]
    traces = []
    logits = torch_ref.deit_dge_forward(sd, images, heads, depth, forced_indices=forced, traces=traces)
    for tr in traces:
        tr["gate_free"] = tr["gate"]
    return logits, traces


class LaunchNames:
    """A stand-in for the library's launch timer that only notes which entry points were called."""

    def __init__(self):
        self.names = []

    def begin(self, name, tag):
        self.names.append(name)

    def end(self):
        pass
