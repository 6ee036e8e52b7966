#!/usr/bin/env python3
"""Benchmark of the DGE query path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3|cfg2|cfg5|cfg4|pvt] [--no-graph]

A step is one inference forward of DeiT+DGE over one batch of synthetic images already resident in HBM.
The headline workload is "cfg3": DeiT-S+DGE, 12 layers, bf16, 256 px, batch 256, router set for a ~0.5
complexity ratio (the configuration the images/s metric is quoted on).  One JSON line is printed:

  value         images/s over the K timed steps (wall clock between two device synchronisations)
  roofline      the kernel name with the largest share of GPU time: algorithmic flops (or bytes) of its launches
                divided by their HIP-event durations, against MI355X's published peak; a matrix kernel is priced
                against both roofs and reported against the one it is nearer to (the other under "other_roof")
  kernels       the same figures for every libvtdge kernel of the step
  cpu_baseline  the torch-CPU restatement of the same model (oracle/torch_ref.py) timed on this box's host cores
                on a bounded sample of the same workload
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"hbm": 8000.0,                         # GB/s
        "mfma": {"bf16": 2500.0, "f32": 157.3}}  # TFLOP/s, dense

WORKLOADS = {
    # name: (factory, img, batch, dtype, heads, description)
    "cfg2": ("deit_dge_s124_tiny_patch16_256", 256, 128, "f32", 3, "DeiT-Ti+DGE 12L fp32 256px B128"),
    "cfg3": ("deit_dge_s124_small_patch16_256", 256, 256, "bf16", 6, "DeiT-S+DGE 12L bf16 256px B256"),
    "cfg5": ("deit_dge_s124_small_patch16_256", 512, 64, "bf16", 6, "DeiT-S+DGE 12L bf16 512px B64"),
    # the second caller of the path (PVT: four stages, spatially reduced keys/values); not one of the five numbered configurations
    "pvt": ("pvt_dge_s124_small_256", 256, 256, "bf16", (1, 2, 5, 8), "PVT-S+DGE 16L bf16 256px B256"),
}


class EventTimer:
    """Brackets every libvtdge call with a pair of HIP events on the stream the kernels are launched on."""

    def __init__(self, torch, last_kernel):
        self.torch = torch
        self.last_kernel = last_kernel
        self.records = []
        self._open = None

    def begin(self, name, tag):
        s = self.torch.cuda.Event(enable_timing=True)
        e = self.torch.cuda.Event(enable_timing=True)
        s.record()
        self._open = (name, tag, s, e)

    def end(self):
        name, tag, s, e = self._open
        e.record()
        # the kernel the call has just launched, under the name the library itself reports for it (the one
        # rocprofv3 lists): the per-kernel table below cannot drift from the library's dispatch
        self.records.append((name, tag, s, e, self.last_kernel()))

    def durations(self):
        self.torch.cuda.synchronize()
        return [(n, t, s.elapsed_time(e) * 1e-3, k) for n, t, s, e, k in self.records]


def measured_traffic(workload):
    """HBM bytes per launch by kernel name, from the committed rocprofv3 --pmc summary of this workload
    (FETCH_SIZE / WRITE_SIZE scaled by a copy of known size); {} when there is none."""
    path = os.path.join(ROOT, "profiles", f"hbm_traffic_{workload}_pmc.txt")
    table = {}
    if os.path.exists(path):
        for line in open(path):
            if line.startswith("#") or "|" not in line:
                continue
            cols = [c.strip() for c in line.split("|")]
            table[cols[0]] = int(cols[4])
    return table


def algorithmic_work(name, tag, esz, geo):
    """(bound, amount) per launch: flops for MFMA kernels, bytes for HBM kernels.

    geo: dict with B, N, C, L (live packed rows), regions and extra of the block the launch belongs to."""
    B, N, C, L = geo["B"], geo["N"], geo["C"], geo["L"]
    if name in ("vtdge_linear", "vtdge_linear_prepacked"):
        _, _, _, has_res, rows, Nn, K, packed = tag
        M = L if packed else rows
        # operands once: A, W, the output and, when there is one, the residual
        return "mfma", 2.0 * M * Nn * K, (M * K + Nn * K + M * Nn * (2 if has_res else 1)) * esz
    if name == "vtdge_patch_embed":
        # images in, tokens out, the weight and the position table once
        _, Bp, S, patch, Cc = tag
        rows, K = Bp * (S // patch) ** 2, 3 * patch * patch
        return "mfma", 2.0 * rows * Cc * K, (rows * K + Cc * K + rows * Cc + (S // patch) ** 2 * Cc) * esz
    if name == "vtdge_patch_linear":
        # the tokens in, the weight once, the rows out
        _, Bp, Hp, Wp, Cp, kp, Np = tag
        rows, K = Bp * (Hp // kp) * (Wp // kp), kp * kp * Cp
        return "mfma", 2.0 * rows * Np * K, (rows * K + Np * K + rows * Np) * esz
    if name == "vtdge_linear_stats":
        _, _, has_res, rows, Nn, K, packed = tag
        M = L if packed else rows
        return "mfma", 2.0 * M * Nn * K, (M * K + Nn * K + M * Nn * (2 if has_res else 1)) * esz + 32 * M
    if name == "vtdge_linear_layernorm":
        _, _, rows, Nn, K, packed = tag
        M = L if packed else rows
        # raw rows, their 32-byte records, the folded weights and their records, the output
        return "mfma", 2.0 * M * Nn * K, (M * K + Nn * K + M * Nn) * esz + 32 * (M + Nn)
    if name == "vtdge_linear_layernorm_pair":
        # two Linears: (rows, N, packed) each; K is the width of the tokens
        flops = byts = 0.0
        for rows, Nn, packed in (tag[1:4], tag[4:7]):
            M = L if packed else rows
            flops += 2.0 * M * Nn * C
            byts += (M * C + Nn * C + M * Nn) * esz + 32 * (M + Nn)
        return "mfma", flops, byts
    if name == "vtdge_compress_regions":
        # every token once, the gate indices and count bytes, every query once with its record and descriptor
        return "hbm", B * N * C * esz + 9 * B * geo["regions"] + L * C * esz + (32 * L if tag[1] else 0) + 32 * L
    if name == "vtdge_layernorm_stats":
        rows = L if tag[1] != B * N else tag[1]
        return "hbm", rows * tag[2] * esz + 32.0 * rows
    if name == "vtdge_sparse_attention":
        # tag[4] = keys per sample; bytes: q in, out, every sample's K and V once
        return "mfma", 4.0 * L * tag[4] * C, (2 * L * C + 2 * B * tag[4] * C) * esz
    if name == "vtdge_compress":
        # read every token once, the descriptors, write every query once (+ the fused LayerNorm copy)
        return "hbm", B * N * C * esz + 32 * L + L * C * esz * (2 if tag[1] else 1)
    if name == "vtdge_decompress":
        return "hbm", (2 if tag[1] else 1) * L * C * esz + 32 * L + (2 if tag[2] else 1) * B * N * C * esz
    if name == "vtdge_decompress_router":
        # the scatter-back's bytes: routing the next block reads nothing more (gate indices in, logits out: KBs)
        return "hbm", ((2 if tag[1] else 1) * L * C * esz + 2 * B * N * C * esz + 16 * B * geo["regions"]
                       + (32 * B * N if tag[4] else 0))
    if name == "vtdge_decompress_router_compress":
        # the scatter-back's bytes plus the next block's queries with their records and descriptors (the tokens the
        # kernel reads back are the ones it has just written)
        Ln = geo["L_next"]
        return "hbm", ((2 if tag[1] else 1) * L * C * esz + 2 * B * N * C * esz + 16 * B * geo["regions"]
                       + 32 * B * N + Ln * C * esz + (32 * Ln if tag[3] else 0) + 32 * Ln)
    if name == "vtdge_decompress_layernorm":
        # the scatter-back plus one more write of every token (the next block's first LayerNorm)
        return "hbm", (2 if tag[1] else 1) * L * C * esz + 32 * L + 3 * B * N * C * esz
    if name == "vtdge_layernorm":
        rows = L if tag[1] else tag[2]
        return "hbm", 2.0 * rows * tag[3] * esz
    if name == "vtdge_router":
        return "hbm", B * (N - geo["extra"]) * C * esz
    if name == "vtdge_router_stats":
        # every token read once, a 32-byte record written per token
        return "hbm", B * N * C * esz + 32.0 * B * N
    if name == "vtdge_router_layernorm":
        return "hbm", 2.0 * B * N * C * esz              # every token read once, its LayerNorm written once
    if name == "vtdge_index_to_patch":
        return "hbm", 8.0 * B * geo["regions"] + 32 * L + 8 * B
    return "hbm", 0.0


def run_model_workload(args, torch):
    from vtpack_amd import _lib
    from vtpack_amd.models import dge as zoo
    from vtpack_amd.synthetic import set_synthetic_router, synthetic_images

    factory, img, batch, dt, heads, desc = WORKLOADS[args.workload]
    if args.batch:
        batch = args.batch
    dtype = torch.bfloat16 if dt == "bf16" else torch.float32
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    model = getattr(zoo, factory)(img_size=img)
    set_synthetic_router(model, 0)
    blocks = list(model.blocks) if hasattr(model, "blocks") else \
        [b for i in range(model.num_stages) for b in getattr(model, f"block{i + 1}")]
    model = model.eval().to(dev).to(dtype)
    images = synthetic_images(batch, img, seed=0, dtype=dtype, device=dev)

    from vtpack_amd import engine

    def step():
        with torch.no_grad():
            return model(images)

    for _ in range(max(args.warmup, 1)):
        out = step()
    torch.cuda.synchronize()

    # ---- optional HIP graph of the whole forward, validated against the eager result on several replays
    mode = "eager"
    runner = step
    if not args.no_graph:
        try:
            static_out = None
            g = torch.cuda.CUDAGraph()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream().wait_stream(side)
            with torch.cuda.graph(g):
                static_out = step()
            ok = True
            for _ in range(3):
                eager = step()
                torch.cuda.synchronize()
                g.replay()
                torch.cuda.synchronize()
                ok = ok and torch.equal(static_out, eager)
            if ok:
                mode = "hipgraph"
                runner = g.replay
            else:
                print("bench: graph replay differs from the eager result; timing the eager path", file=sys.stderr)
        except Exception as exc:  # capture is an optimisation, never a requirement
            print(f"bench: HIP graph capture unavailable ({exc}); timing the eager path", file=sys.stderr)
            torch.cuda.synchronize()

    for _ in range(args.warmup):
        runner()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        runner()
    torch.cuda.synchronize()
    dt_s = time.perf_counter() - t0
    ms_per_step = dt_s / args.steps * 1e3
    value = batch * args.steps / dt_s

    # ---- per-kernel HIP-event timing: the same steps again, eagerly, every libvtdge launch bracketed
    timer = EventTimer(torch, _lib.last_kernel)
    inst_steps = min(args.steps, 5)
    lens = []
    _lib.timer = timer
    engine.OVERLAP = False      # one kernel at a time on one stream
    try:
        for _ in range(inst_steps):
            step()
            lens.append([int(b.dge.states["offsets_device"][-1]) for b in blocks])
    finally:
        _lib.timer = None
        engine.OVERLAP = True
    recs = timer.durations()

    # geometry of every block (token count, width, regions), from the states its encoder keeps
    esz = 2 if dt == "bf16" else 4
    geos = []
    for b in blocks:
        st_ = b.dge.states
        Bn, Nn, Cn = st_["input"].shape
        H_, W_ = st_["size"]
        geos.append({"B": Bn, "N": Nn, "C": Cn, "regions": (H_ // 4) * (W_ // 4), "extra": st_["num_extra_tokens"]})
    per_step = len(recs) // inst_steps
    stats = {}
    blk = 0
    for i, (name, tag, sec, sym) in enumerate(recs):
        if i % per_step == 0:
            blk = 0
        # a block's launches end with its scatter; what precedes block 0 or follows the last block is dense
        at = min(blk, len(blocks) - 1)
        geo = dict(geos[at], L=lens[i // per_step][at], L_next=lens[i // per_step][min(at + 1, len(blocks) - 1)])
        bound, amount, *rest = algorithmic_work(name, tag, esz, geo)
        st = stats.setdefault(sym, {"bound": bound, "launches": 0, "seconds": 0.0, "work": 0.0, "bytes": 0.0})
        st["launches"] += 1
        st["seconds"] += sec
        st["work"] += amount
        st["bytes"] += rest[0] if rest else 0.0
        if name in ("vtdge_decompress", "vtdge_decompress_router", "vtdge_decompress_router_compress",
                    "vtdge_decompress_layernorm"):
            blk += 1
    kernels = {}
    for sym, st in stats.items():
        # A matrix kernel is priced against both roofs (the K = 384 and narrow-N GEMMs of this model sit near the
        # ridge, attention below it): the one it is nearer to is the one that binds, and the other is kept beside it.
        other = None
        if st["bound"] == "mfma" and st["bytes"] > 0:
            f_m = st["work"] / st["seconds"] / 1e12 / PEAK["mfma"][dt]
            f_h = st["bytes"] / st["seconds"] / 1e9 / PEAK["hbm"]
            if f_h > f_m:
                other = {"bound": "mfma", "achieved": round(st["work"] / st["seconds"] / 1e12, 2),
                         "peak": PEAK["mfma"][dt], "unit": "TFLOP/s", "frac": round(f_m, 4),
                         "algorithmic_per_launch": int(st["work"] / st["launches"])}
                st["bound"], st["work"] = "hbm", st["bytes"]
            else:
                other = {"bound": "hbm", "achieved": round(st["bytes"] / st["seconds"] / 1e9, 2), "peak": PEAK["hbm"],
                         "unit": "GB/s", "frac": round(f_h, 4),
                         "algorithmic_per_launch": int(st["bytes"] / st["launches"])}
        peak = PEAK["hbm"] if st["bound"] == "hbm" else PEAK["mfma"][dt]
        unit = "GB/s" if st["bound"] == "hbm" else "TFLOP/s"
        ach = st["work"] / st["seconds"] / (1e9 if st["bound"] == "hbm" else 1e12)
        kernels[sym] = {"bound": st["bound"], "achieved": round(ach, 2), "peak": peak, "unit": unit,
                        "frac": round(ach / peak, 4), "avg_us": round(st["seconds"] / st["launches"] * 1e6, 2),
                        "launches_per_step": st["launches"] // inst_steps,
                        "share": 0.0}
        if other is not None:
            kernels[sym]["other_roof"] = other
    tot = sum(st["seconds"] for st in stats.values())
    for sym, st in stats.items():
        kernels[sym]["share"] = round(st["seconds"] / tot, 4)
    dom = max(stats, key=lambda s: stats[s]["seconds"])
    roof = {k: kernels[dom][k] for k in ("bound", "achieved", "peak", "unit", "frac")}
    traffic = measured_traffic(args.workload)
    for sym in kernels:
        kernels[sym]["algorithmic_per_launch"] = int(stats[sym]["work"] / stats[sym]["launches"])
        kernels[sym]["traffic"] = traffic.get(sym)
    roof.update({"kernel": dom, "avg_us": kernels[dom]["avg_us"], "traffic": traffic.get(dom)})
    if "other_roof" in kernels[dom]:
        roof["other_roof"] = kernels[dom]["other_roof"]

    # one plain device-to-device copy of known size (256 MiB), so that a counter run of this script carries its
    # own yardstick for the HBM byte counters
    calib_src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    calib_dst = torch.empty_like(calib_src)
    calib_dst.copy_(calib_src)
    torch.cuda.synchronize()

    ratio = sum(sum(l) for l in lens) / (len(lens) * sum(g["B"] * g["N"] for g in geos))
    N = geos[-1]["N"]
    result = {
        "metric": "images/sec DeiT-S+DGE bf16 256px @1 MI355X" if args.workload == "cfg3"
        else f"images/sec {desc} @1 MI355X",
        "value": round(value, 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt, "data": "synthetic",
        "config": {"workload": f"{args.workload}: {desc}, budget~0.5 via synthetic router", "batch": batch,
                   "tokens": N, "query_ratio": round(ratio, 4), "mode": mode},
        "roofline": roof, "kernels": kernels,
    }
    return result, model, images, heads


def run_isolated_gemm(args, torch):
    """cfg4: packed A [L, 384] ~ N(0,1) against shared W [N, 384] ~ N(0, 0.02), bf16; 256 segments whose lengths
    follow a seeded skewed gate mix (1/4/16 queries per region with a heavy tail), clipped to [16, 256]."""
    import numpy as np
    from vtpack_amd import ops
    dev = torch.device("cuda:0")
    rng = np.random.RandomState(0)
    p_fine = np.clip(rng.beta(0.6, 2.0, size=256), 0, 1)          # most samples coarse, a heavy tail of fine ones
    lengths = []
    for pf in p_fine:
        probs = [pf, (1 - pf) * 0.4, (1 - pf) * 0.6]
        lengths.append(1 + int(rng.choice([16, 4, 1], size=16, p=probs).sum()))
    lengths = np.clip(np.array(lengths), 16, 256)
    L = int(lengths.sum())
    K = 384
    g = torch.Generator().manual_seed(0)
    A = torch.randn((L, K), generator=g).to(dev, torch.bfloat16)
    rows_dev = torch.tensor([L], dtype=torch.int64, device=dev)
    per_n, total_flops, total_s = {}, 0.0, 0.0
    for N in (384, 1152, 1536):
        Wt = (torch.randn((N, K), generator=g) * 0.02).to(dev, torch.bfloat16)
        bias = torch.zeros(N, device=dev, dtype=torch.bfloat16)
        out = torch.empty((L, N), device=dev, dtype=torch.bfloat16)
        for _ in range(args.warmup):
            ops.linear(A, Wt, bias, rows_dev=rows_dev, out=out)
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        s.record()
        for _ in range(args.steps):
            ops.linear(A, Wt, bias, rows_dev=rows_dev, out=out)
        e.record()
        torch.cuda.synchronize()
        sec = s.elapsed_time(e) * 1e-3 / args.steps
        fl = 2.0 * L * N * K
        byts = (L * K + N * K + L * N) * 2
        per_n[str(N)] = {"us": round(sec * 1e6, 2), "TFLOP/s": round(fl / sec / 1e12, 1),
                         "GB/s": round(byts / sec / 1e9, 1), "frac_mfma": round(fl / sec / 1e12 / 2500.0, 4)}
        total_flops += fl
        total_s += sec
    from vtpack_amd import _lib
    last_name = _lib.last_kernel()
    ach = total_flops / total_s / 1e12
    return {"metric": "TFLOP/s isolated packed-M GEMM bf16 K=384 @1 MI355X", "value": round(ach, 1),
            "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(total_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "cfg4: 256 segments, skewed lengths in [16,256], K=384, N in {384,1152,1536}",
                       "packed_rows": L},
            "roofline": {"bound": "mfma", "achieved": round(ach, 1), "peak": 2500.0, "unit": "TFLOP/s",
                         "frac": round(ach / 2500.0, 4),
                         "kernel": last_name, "traffic": None},
            "per_n": per_n}


def cpu_baseline(args, torch, model, images, heads):
    """The torch-CPU restatement on a bounded sample of the same workload, on this box's host cores."""
    from oracle import torch_ref
    sample = min(args.cpu_sample, images.shape[0])
    sd = torch_ref.float_state_dict(model)
    img = images[:sample].float().cpu()
    threads = torch.get_num_threads()
    if hasattr(model, "blocks"):
        depth = len(model.blocks)
        run = lambda: torch_ref.deit_dge_forward(sd, img, heads, depth)  # noqa: E731
    else:
        sr = [getattr(model, f"block{i + 1}")[0].attn.sr_ratio for i in range(model.num_stages)]
        run = lambda: torch_ref.pvt_dge_forward(sd, img, heads, model.depths, sr)  # noqa: E731
    with torch.no_grad():
        run()
        run()
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            run()
            times.append(time.perf_counter() - t0)
    med = sorted(times)[2]
    return {"value": round(sample / med, 2), "unit": "images/s", "cores": threads, "kind": "port",
            "sample": f"{sample} images of the same workload, fp32 torch-CPU restatement (oracle/torch_ref.py), "
                      f"median of 5 after 2 warm-ups, {threads} threads"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg3", choices=sorted(WORKLOADS) + ["cfg4"])
    ap.add_argument("--batch", type=int, default=0, help="override the workload's batch size")
    ap.add_argument("--no-graph", action="store_true", help="time the eager path instead of a HIP graph replay")
    ap.add_argument("--cpu-sample", type=int, default=128, help="images in the CPU baseline sample (0 = skip)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only (the path shards along the batch with no exchange step)."
              " Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.workload == "cfg4":
        print(json.dumps(run_isolated_gemm(args, torch)))
        return
    result, model, images, heads = run_model_workload(args, torch)
    if args.cpu_sample > 0:
        result["cpu_baseline"] = cpu_baseline(args, torch, model, images, heads)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
