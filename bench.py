#!/usr/bin/env python3
"""Headline benchmark: images/sec of fp16 NHWC ResNet-50 v1.5 at batch 256 on one MI355X,
one training step (forward + backward + mixed-precision Adam) and inference, through the
Saga Graph/Context/Program boundary on the hip engine.

    python bench.py --gpus 1 --steps K --warmup W

Prints ONE JSON line.  `value` is training images/sec over exactly K timed steps with the
input batch already resident in HBM; `infer_images_per_sec` is the inference program on the
same weights (`roofline_infer`: its dominant kernel family, timed the same way).  `roofline` describes the
kernel family that takes the most GPU time in the
training step (the convolutions; HIP-event timing of every operation on the engine's stream, taken in a
second pass of K steps so that the events do not sit inside the timed region), `roofline_hbm` the
HBM-bound family with the most time (batch norm); `families` and `kernels` list every family and
every operation kind the same way.  `cpu_baseline` is the CPU oracle (oracle/) running the same
training step on a small batch on the host cores - a reported baseline, not a target.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16 matrix
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

MATRIX_KINDS = ("convfwd", "convbwddata", "convbwdfilter", "fc.")
CONV_KINDS = ("convfwd", "convbwddata", "convbwddata.bn", "convbwdfilter")

# Operation kinds that share kernels and a roofline bound form a family; `roofline` describes the family with
# the most GPU time in the training step.
FAMILIES = {
    "conv": ("convfwd", "convfwd.bn", "convbwddata", "convbwddata.bn", "convbwdfilter"),
    "batchnorm": ("bntrain", "bntrain.fused", "bnbwd", "bnbwd.fused", "bnbwd.linked", "bnbwd.pooled"),
    "pool": ("poolfwd", "poolfwd.bn", "poolbwd"),
}

# HBM bytes per launch of a family, averaged over ALL launches of that family in one training step (the same
# population `algorithmic` is averaged over): rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE over
# `bench.py --train-only --no-cpu --no-profile`, summed over the kernels the family's operations launch, each
# counter scaled by what it reads for a plain copy of known size (`bench.py --copy-calibration`).  The command
# lines, the per-kernel table and the commit the counters were taken at are in
# profiles/resnet50_b256_fp16_hbm_counters.txt; they go stale when kernels change, hence the label.
MEASURED_HBM_BYTES_PER_LAUNCH = {
    "conv": 255579238,
    "batchnorm": 413304412,
}
TRAFFIC_SOURCE = "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE snapshot at commit 83e6fa4 (profiles/resnet50_b256_fp16_hbm_counters.txt)"


def by_kind(rows):
    """The engine reports one row per operation ("kind#position"); add them up per kind.  `roof_ms` is
    the time the same launches would take at the roofline: each operation at the larger of its
    algorithmic flops / MFMA peak and its algorithmic bytes / HBM peak (a 1x1 convolution over
    56x56 pixels is bound by HBM, a 3x3 one over 14x14 pixels by the matrix cores)."""
    agg = {}
    for r in rows:
        if r["launches"] == 0:
            continue
        kind = r["kind"].split("#")[0]
        a = agg.setdefault(kind, {"kind": kind, "launches": 0, "ms": 0.0, "flops": 0.0, "bytes": 0.0, "roof_ms": 0.0})
        a["launches"] += r["launches"]
        a["ms"] += r["ms"]
        a["flops"] += r["flops"]
        a["bytes"] += r["bytes"]
        a["roof_ms"] += max(r["flops"] / (PEAK_FP16_TFLOPS * 1e12), r["bytes"] / (PEAK_HBM_GBS * 1e9)) * 1e3
    return list(agg.values())


def write_per_op(path, rows, steps):
    """One line per operation, in program order: average time per launch, achieved rate, the time its
    algorithmic flops and bytes would take at the MFMA and HBM peaks, and which of the two bounds it."""
    def pos(r):
        return int(r["kind"].split("#")[1]) if "#" in r["kind"] else 0
    with open(path, "w") as f:
        f.write(f"per-operation profile of one training step (average over {steps} steps, HIP events on the engine's stream)\n")
        f.write("  #  kind                    us  GFLOP      MB   TFLOP/s    GB/s  bound  roof_us  frac\n")
        tot = roof = 0.0
        for r in sorted(rows, key=pos):
            if r["launches"] == 0:
                continue
            us = r["ms"] * 1e3 / r["launches"]
            fl, by = r["flops"] / r["launches"], r["bytes"] / r["launches"]
            t_m, t_h = fl / (PEAK_FP16_TFLOPS * 1e12) * 1e6, by / (PEAK_HBM_GBS * 1e9) * 1e6
            bound = max(t_m, t_h)
            tot += us
            roof += bound
            f.write(f"{pos(r):3d}  {r['kind'].split('#')[0]:18s} {us:8.1f} {fl / 1e9:6.1f} {by / 1e6:7.1f} "
                    f"{fl / us / 1e6 if us else 0:9.1f} {by / us / 1e3 if us else 0:7.0f}  {'mfma' if t_m >= t_h else 'hbm':5s} "
                    f"{bound:7.1f}  {bound / us if us else 0:.3f}\n")
        f.write(f"sum of operations {tot / 1e3:.3f} ms, sum of roofline bounds {roof / 1e3:.3f} ms, fraction {roof / tot:.3f}\n")


def profile_rows(rows):
    out = []
    for r in rows:
        if r["launches"] == 0 or r["ms"] <= 0:
            continue
        matrix = r["kind"].startswith(MATRIX_KINDS)
        sec = r["ms"] * 1e-3
        row = {"kind": r["kind"], "launches": r["launches"], "ms_total": round(r["ms"], 3),
               "avg_us": round(r["ms"] * 1e3 / r["launches"], 2),
               "frac_of_roofline": round(r["roof_ms"] / r["ms"], 4)}
        if matrix:
            a = r["flops"] / sec / 1e12
            row.update(bound="mfma", achieved=round(a, 2), peak=PEAK_FP16_TFLOPS, unit="TFLOP/s",
                       frac=round(a / PEAK_FP16_TFLOPS, 4))
        else:
            a = r["bytes"] / sec / 1e9
            row.update(bound="hbm", achieved=round(a, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                       frac=round(a / PEAK_HBM_GBS, 4))
        out.append(row)
    out.sort(key=lambda r: -r["ms_total"])
    return out


def family_rows(rows, steps, with_traffic=True):
    """Operation kinds grouped into families (FAMILIES; every other kind is its own family), most GPU time first.
    achieved = algorithmic flops (matrix families) or bytes (the others) of all launches / their summed time,
    both from this run; `algorithmic` and `traffic` are per launch, averaged over the same launches."""
    fam_of = {k: f for f, kinds in FAMILIES.items() for k in kinds}
    agg = {}
    for r in rows:
        if r["ms"] <= 0:
            continue
        f = fam_of.get(r["kind"], r["kind"])
        a = agg.setdefault(f, {"kernel": f, "kinds": [], "launches": 0, "ms": 0.0, "flops": 0.0, "bytes": 0.0, "roof_ms": 0.0})
        a["kinds"].append(r["kind"])
        for k in ("launches", "ms", "flops", "bytes", "roof_ms"):
            a[k] += r[k]
    out = []
    for a in agg.values():
        matrix = a["kernel"] == "conv" or a["kernel"].startswith("fc.")
        sec = a["ms"] * 1e-3
        if matrix:
            ach, peak, unit = a["flops"] / sec / 1e12, PEAK_FP16_TFLOPS, "TFLOP/s"
            alg = a["flops"] / a["launches"]
        else:
            ach, peak, unit = a["bytes"] / sec / 1e9, PEAK_HBM_GBS, "GB/s"
            alg = a["bytes"] / a["launches"]
        out.append({"kernel": a["kernel"], "kinds": sorted(a["kinds"]), "bound": "mfma" if matrix else "hbm",
                    "achieved": round(ach, 1), "peak": peak, "unit": unit, "frac": round(ach / peak, 4),
                    "traffic": MEASURED_HBM_BYTES_PER_LAUNCH.get(a["kernel"]) if with_traffic else None,
                    "traffic_source": TRAFFIC_SOURCE if with_traffic else None,
                    "algorithmic": round(alg), "algorithmic_unit": "flop/launch" if matrix else "byte/launch",
                    "algorithmic_bytes": round(a["bytes"] / a["launches"]),
                    "avg_launch_us": round(a["ms"] * 1e3 / a["launches"], 2), "launches": a["launches"],
                    "ms_per_step": round(a["ms"] / steps, 3),
                    "frac_of_own_roofline": round(a["roof_ms"] / a["ms"], 4)})
    out.sort(key=lambda r: -r["ms_per_step"])
    return out


def cpu_baseline(batch, image):
    """The CPU oracle's training step on a bounded sample (small batch, same network)."""
    from oracle.net import OracleNet
    from saga_amd import networks as N

    net = N.resnet50(batch, image=image)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((batch, 3, image, image)).astype(np.float16).astype(np.float32)
    labels = rng.integers(0, 1000, (batch, 1)).astype(np.int32)
    o = OracleNet(net, lr=1e-4, loss_scale=1024.0)
    t0 = time.perf_counter()
    o.train_step(x, labels)
    dt = time.perf_counter() - t0
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return {"value": round(batch / dt, 4), "unit": "images/sec", "cores": cores, "kind": "port",
            "sample": f"ONE ResNet-50 training step (fwd+bwd+Adam) at batch {batch}, {image}x{image}, not warmed "
                      f"up and not repeated ({dt:.1f} s of CPU work; ten warm repetitions would take minutes)"}


def hbm_copy_rate():
    """What a plain device copy reaches on this GPU, measured live: 1 GiB fp32 -> fp32 through saga_hip_axpby
    (alpha 1, beta 0; the same 16-byte-per-lane streaming loop the element-wise operators use), best of 5 after
    one warm-up, HIP events on the stream the kernel runs on.  Reported next to the HBM fractions: the distance
    between this and the 8 TB/s data-sheet peak is not the kernels'."""
    import ctypes as C
    import torch
    from saga_amd import kernels as K

    n = 1 << 28
    src = torch.ones(1, 1, 1, n, dtype=torch.float32, device="cuda")
    dst = torch.zeros_like(src)
    vs, vd = K.view(src), K.view(dst)
    best = None
    for i in range(6):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        K.check(K.lib().saga_hip_axpby(C.byref(vs), C.byref(vd), 1.0, 0.0, K.stream_ptr()))
        b.record()
        b.synchronize()
        ms = a.elapsed_time(b)
        if i and (best is None or ms < best):
            best = ms
    del src, dst
    torch.cuda.empty_cache()
    return {"value": round(2 * n * 4 / best / 1e6, 1), "unit": "GB/s", "sample": "1 GiB read + 1 GiB written per launch, best of 5",
            "frac_of_peak": round(2 * n * 4 / best / 1e6 / PEAK_HBM_GBS, 4)}


def copy_calibration():
    """Five plain copies of 1 GiB (fp32 -> fp32 through saga_hip_axpby, alpha 1, beta 0): under
    `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` the ew_flat kernel's counter value divided by
    1 GiB is the factor that turns the counters of the other kernels into bytes."""
    import ctypes as C
    import torch
    from saga_amd import kernels as K

    n = 1 << 28
    src = torch.ones(1, 1, 1, n, dtype=torch.float32, device="cuda")
    dst = torch.zeros_like(src)
    for _ in range(5):
        K.check(K.lib().saga_hip_axpby(C.byref(K.view(src)), C.byref(K.view(dst)), 1.0, 0.0, None))
    torch.cuda.synchronize()
    assert float(dst[0, 0, 0, -1]) == 1.0
    print(json.dumps({"copy_bytes": n * 4, "launches": 5}))


def conv_microbench(args):
    """The single-layer convolution microbenchmark (N=256, 56x56, 64 -> 64 channels, 3x3, stride 1, pad 1) in fp16
    NHWC and fp32 NCHW through the C ABI: forward, backward data and backward filter, inputs N(0,1), He-normal
    filter, 59.19 GFLOP per pass.  HIP events on the launch stream, `steps` launches per pass after 3 warm-ups."""
    import torch
    from saga_amd import kernels as K

    N, Cc, H, Kk, R = 256, 64, 56, 64, 3
    flops = 2.0 * N * Kk * H * H * Cc * R * R
    out = {}
    for name, dt, cl in (("fp16_nhwc", torch.float16, True), ("fp32_nchw", torch.float32, False)):
        g = torch.Generator(device="cuda").manual_seed(2)
        mk = lambda *shape: torch.randn(*shape, dtype=dt, device="cuda", generator=g)
        fmt = (lambda t: t.contiguous(memory_format=torch.channels_last)) if cl else (lambda t: t)
        x, dy = fmt(mk(N, Cc, H, H)), fmt(mk(N, Kk, H, H))
        w = fmt(mk(Kk, Cc, R, R) * (2.0 / (Cc * R * R)) ** 0.5)
        y, dx, dw = torch.zeros_like(dy), torch.zeros_like(x), torch.zeros_like(w)
        res = {}
        for kind, a in (("fwd", (K.CONV_FWD, x, w, y)), ("bwd_data", (K.CONV_BWD_DATA, dy, w, dx)),
                        ("bwd_filter", (K.CONV_BWD_FILTER, x, dy, dw))):
            for _ in range(3):
                K.conv2d(*a, 1, 1)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(args.steps):
                K.conv2d(*a, 1, 1)
            e1.record()
            e1.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / args.steps
            res[kind] = {"us": round(us, 1), "tflops": round(flops / us / 1e6, 1)}
        out[name] = res
    print(json.dumps({"conv_microbench": {"shape": "N256 C64 56x56 K64 3x3 s1 p1", "gflop_per_pass": round(flops / 1e9, 2),
                                          "peak_tflops": {"fp16_nhwc": PEAK_FP16_TFLOPS, "fp32_nchw": 157.3}, **out}}))


def host_input_rate(args):
    """The same two programs with the image batch and the labels declared as batched tensors: every step the
    engine uploads the host's back buffers (pinned memory, hipMemcpyAsync on the program's stream) before it
    runs, as it does for the reference's harness.  Reported beside the headline, never as `value`."""
    import torch
    from saga_amd import api as S
    from saga_amd import networks as N

    net = N.resnet50(args.batch, image=args.image)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((args.batch, 3, args.image, args.image)).astype(np.float16)
    ctx = S.Context()
    graph, t = N.build_graph(net, x)
    pre = 1  # Phase::PRE
    train = ctx.create_program(graph, args.batch, training=True, learning_rate=1e-4, initial_loss_scale=1024.0,
                               batched={t[net.input]: pre, t["labels"]: pre})
    infer = ctx.create_program(graph, args.batch, training=False, batched={t[net.input]: pre})
    ctx.resolve(t["loss"])
    ctx.resolve(t["pred"])
    out = {"host_bytes_per_step": int(x.nbytes + args.batch * 4)}
    for name, prog in (("train", train), ("infer", infer)):
        prog.run(args.warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        prog.run(args.steps)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        out[name + "_images_per_sec"] = round(args.batch * args.steps / dt, 1)
        out[name + "_ms_per_step"] = round(dt / args.steps * 1e3, 3)
    print(json.dumps({"pcie_inclusive": out}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--image", type=int, default=224)
    ap.add_argument("--cpu-batch", type=int, default=16)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-profile", action="store_true")
    ap.add_argument("--train-only", action="store_true",
                    help="skip the inference program (counter runs that must see training launches only)")
    ap.add_argument("--per-op", metavar="FILE",
                    help="also write one line per operation of the training step (time, rate, own roofline bound)")
    ap.add_argument("--host-input", action="store_true",
                    help="time the programs with the batch handed over from host memory every step (PCIe included) and exit")
    ap.add_argument("--conv-microbench", action="store_true",
                    help="time the single-layer convolution microbenchmark (fp16 NHWC and fp32 NCHW) and exit")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run a plain 1 GiB device copy five times and exit (reference for the HBM counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build drives exactly one GPU (no collectives, no sharding); run with --gpus 1")
    if args.copy_calibration:
        return copy_calibration()
    if args.host_input:
        return host_input_rate(args)
    if args.conv_microbench:
        return conv_microbench(args)

    os.environ.setdefault("SAGA_HIP_PROFILE_PER_OP", "1")  # profile rows per operation, see by_kind()
    from saga_amd import api as S
    from saga_amd import networks as N

    net = N.resnet50(args.batch, image=args.image)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((args.batch, 3, args.image, args.image)).astype(np.float16)
    labels = rng.integers(0, 1000, (args.batch, 1)).astype(np.int32)

    ctx = S.Context()
    graph, t = N.build_graph(net, x)
    train = ctx.create_program(graph, args.batch, training=True, learning_rate=1e-4, initial_loss_scale=1024.0)
    infer = None if args.train_only else ctx.create_program(graph, args.batch, training=False)
    ctx.resolve(t["labels"]).write(labels)
    loss = ctx.resolve(t["loss"])
    pred = ctx.resolve(t["pred"])
    train.finalize()
    if infer:
        infer.finalize()

    import torch  # device-wide synchronisation around the timed regions

    # ---- training: W warm-up steps, then exactly K timed steps
    train.run(args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    train.run(args.steps)
    torch.cuda.synchronize()
    t_train = time.perf_counter() - t0
    mean_loss = float(loss.read().mean())

    # ---- inference on the same weights
    t_infer = float("nan")
    if not args.train_only:
        infer.run(args.warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        infer.run(args.steps)
        torch.cuda.synchronize()
        t_infer = time.perf_counter() - t0
        pred.read()

    kernels, roof, roof_hbm, conv, families = [], None, None, None, []
    copy_rate = None if args.no_profile else hbm_copy_rate()
    if not args.no_profile:
        train.set_profiling(True)
        train.run(args.steps)
        raw = train.profile()
        if args.per_op:
            write_per_op(args.per_op, raw, args.steps)
        rows = by_kind(raw)
        kernels = profile_rows(rows)
        train.set_profiling(False)
        families = family_rows(rows, args.steps)
        if families:
            roof = families[0]
            hbm = [f for f in families if f["bound"] == "hbm"]
            roof_hbm = hbm[0] if hbm else None
        # the three convolution kinds together: the "conv MFMA util %" half of the metric
        cr = [r for r in rows if r["kind"] in CONV_KINDS and r["ms"] > 0]
        if cr:
            tf = sum(r["flops"] for r in cr) / (sum(r["ms"] for r in cr) * 1e-3) / 1e12
            conv = {"bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(tf / PEAK_FP16_TFLOPS, 4), "mfma_util_pct": round(100 * tf / PEAK_FP16_TFLOPS, 2),
                    "ms_per_step": round(sum(r["ms"] for r in cr) / args.steps, 3),
                    # against each layer's own bound (HBM for the wide 1x1 layers, MFMA for the others)
                    "frac_of_roofline": round(sum(r["roof_ms"] for r in cr) / sum(r["ms"] for r in cr), 4)}

    # the inference program the same way: its convolutions carry the folded batch norm, relu and residual add
    # ("convfwd.bn"), so one family holds nearly all of its time.  The HBM counters were taken on training
    # launches only, so `traffic` is null here.
    roof_infer, families_infer = None, []
    if infer and not args.no_profile:
        infer.set_profiling(True)
        infer.run(args.steps)
        families_infer = family_rows(by_kind(infer.profile()), args.steps, with_traffic=False)
        infer.set_profiling(False)
        roof_infer = families_infer[0] if families_infer else None

    flops_step = 3 * net.flops_fwd * args.batch  # fwd + bwd-data + bwd-filter (the stem has no bwd-data)
    ips = args.batch * args.steps / t_train
    out = {
        "metric": "images/sec fp16 NHWC ResNet-50 b256 infer+train step; conv MFMA util %",
        "value": round(ips, 1),
        "unit": "images/sec",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(t_train / args.steps * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"ResNet-50 v1.5 training step (fwd+bwd+Adam), fp16 NHWC, batch {args.batch}, "
                               f"{args.image}x{args.image}, 1000 classes", "global_batch": args.batch},
        "train_images_per_sec": round(ips, 1),
        "infer_images_per_sec": None if args.train_only else round(args.batch * args.steps / t_infer, 1),
        "infer_ms_per_batch": None if args.train_only else round(t_infer / args.steps * 1e3, 3),
        "train_tflops": round(flops_step / (t_train / args.steps) / 1e12, 1),
        "infer_tflops": None if args.train_only else round(net.flops_fwd * args.batch / (t_infer / args.steps) / 1e12, 1),
        "loss_scale": train.loss_scale(),
        "mean_loss": round(mean_loss, 4),
        "roofline": roof,
        "roofline_hbm": roof_hbm,
        "roofline_infer": roof_infer,
        "families_infer": families_infer,
        "hbm_copy_rate": copy_rate,
        "conv": conv,
        "families": families,
        "kernels": kernels,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.cpu_batch, args.image)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
