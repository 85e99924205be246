"""Benchmark of the PSA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c1|c3|c4|c5] [--no-cpu] [--no-dense] [--no-extras]

A step = one PSA attention layer over synthetic inputs already resident in HBM:
pyramid pooling -> sampled block-importance estimate -> level map -> tile schedule -> sparse attention forward.
Prints ONE JSON line (the headline metric of this path) with a `roofline` object for the dominant kernel
(the sparse forward, MFMA-bound) and a `cpu_baseline` object (the oracle on the host cores over a
bounded sample of the same workload).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "pyramid-sparse-attention_amd")
sys.path.insert(0, PKG)

METRIC = "PSA attn ms/layer + effective TFLOPS (% bf16 MFMA peak) at Wan2.1-1.3B shape, 1 GPU"
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_FP32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # c2, the configuration the metric is quoted on: Wan2.1-1.3B 480p self-attention layer
    "c2": dict(name="wan2.1-1.3b-480p B1 H12 N32760 D128 bf16 blk128 thresholdbound ~90% sparsity",
               B=1, H=12, grid=(21, 30, 52), D=128, bm=128, bn=128, tn=32, sparsity=0.90),
    # c1 (small, fp32 tensors: every stage computes in fp32 - the fp32 kernels run on the vector
    # units, so the peak its roofline line is priced against is the fp32 one)
    "c1": dict(name="small B1 H2 N4096 D64 fp32 blk64 thresholdbound ~80% sparsity",
               B=1, H=2, grid=(4, 32, 32), D=64, bm=64, bn=64, tn=16, sparsity=0.80, dtype="fp32"),
}
WORKLOADS.update({
    # c3: CogVideoX-5B joint text + video attention (text blocks last, always level 1)
    # (top-k with the ratios of the reference's CogVideo_5b / psa_4steps preset: density 0.15625 before the text columns)
    "c3": dict(name="cogvideox-5b B2 H48 N17776 (17550 video + 226 text) D64 bf16 blk128 topk psa_4steps ratios ~84% sparsity",
               B=2, H=48, grid=(13, 30, 45), D=64, bm=128, bn=128, tn=32, sparsity=0.84, text=226, mode="topk",
               ratios={1: (0.0, 0.05), 2: (0.05, 0.15), 4: (0.15, 0.25), 8: (0.25, 0.5), 0: (0.5, 1.0)}),
    # c4: training step = forward with lse + backward (dQ, dK, dV)
    "c4": dict(name="training step B1 H12 N32760 D128 bf16 blk128 thresholdbound ~85% sparsity, dO ~ N(0, 0.02)",
               B=1, H=12, grid=(21, 30, 52), D=128, bm=128, bn=128, tn=32, sparsity=0.85, kind="train"),
    # c5: causal GQA prefill at the Qwen2.5-VL-7B decoder shape
    # (the configuration names N = 32768 with tokens 1024.. on a 16x44x44 grid, which has 30976 positions: the vision
    # part here is the first 31744 positions of a 17x44x44 grid, so that N is the 32768 the configuration is about)
    "c5": dict(name="qwen2.5-vl-7b causal prefill B1 Hq28 Hkv4 N32768 (1024 text + 31744 vision tokens of a 44x44-per-frame grid) "
                    "D128 bf16 blk128 xattn estimate stride 8, energybound ~80% sparsity over the lower triangle",
               B=1, H=28, Hkv=4, grid=(17, 44, 44), tokens=32768, D=128, bm=128, bn=128, sparsity=0.80, text=1024, kind="causal",
               stride=8),
})
WAN13 = {1: (0.0, 0.5), 2: (0.5, 0.6), 4: (0.6, 0.7), 8: (0.7, 0.8), 0: (0.8, 1.0)}


def fwd_traffic_bytes(workload):
    """HBM-side bytes per launch of the forward kernel from the committed rocprofv3 counter summaries
    (profiles/*.txt, line `roofline.traffic <workload> <kernel> <bytes>`), or None."""
    import glob

    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.txt"))):
        try:
            for line in open(path):
                f = line.split()
                if len(f) >= 4 and f[0] == "roofline.traffic" and f[1] == workload:
                    return float(f[3])
        except OSError:
            pass
    return None


def scaled_ratios(tau):
    return {lv: (lo * tau if lv else 0.8 * tau, hi * tau if lv else 1.0) for lv, (lo, hi) in WAN13.items()}


def time_gpu(fn, iters, warm=20):
    import torch

    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in evs)
    return ts[len(ts) // 2], sum(ts) / len(ts)


def load_telemetry(fn, ms_per_call, flops_per_call=0.0):
    """What rocm-smi reports while fn runs back to back for about 3 s: the shader clock (the clock the launch's cycles are
    counted in - the published peak is quoted at the 2400 MHz maximum), and the board's average power over the run from
    its energy counter, with the energy per call (and per flop) that follows.  Fields are None where rocm-smi gives no
    reading."""
    import re
    import subprocess
    import threading

    import torch

    def smi(*args):
        try:
            return subprocess.run(["rocm-smi", *args], capture_output=True, text=True, timeout=20).stdout
        except Exception:
            return ""

    def energy_uj():
        m = re.search(r"Accumulated Energy \(uJ\):\s*([\d.]+)", smi("--showenergycounter"))
        return float(m.group(1)) if m else None

    reads, stop = [], threading.Event()

    def poll():
        while not stop.is_set():
            m = re.search(r"sclk clock level[^(]*\((\d+)Mhz\)", smi("--showclocks"))
            if m:
                reads.append(int(m.group(1)))
            stop.wait(0.1)

    th = threading.Thread(target=poll, daemon=True)
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    n = max(10, int(3000.0 / max(ms_per_call, 1e-3)))
    e0, t0 = energy_uj(), time.perf_counter()
    th.start()
    for _ in range(n):
        fn()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    e1 = energy_uj()
    stop.set()
    th.join(timeout=30)
    reads = sorted(reads[1:] or reads)  # (the first reading may predate the load)
    out = {"sclk_mhz": reads[len(reads) // 2] if reads else None, "avg_power_w": None, "joule_per_call": None, "pj_per_flop": None}
    if e0 is not None and e1 is not None and e1 > e0:
        joule = (e1 - e0) / 1e6
        out["avg_power_w"] = round(joule / dt, 0)
        out["joule_per_call"] = round(joule / n, 4)
        if flops_per_call:
            out["pj_per_flop"] = round(joule / n / flops_per_call * 1e12, 3)
    return out


def copy_calib(torch, dev):
    """1 GiB read + 1 GiB written by a plain elementwise kernel: the reference reading for FETCH_SIZE / WRITE_SIZE."""
    src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    for _ in range(3):
        torch.mul(src, 1.0, out=dst)
    torch.cuda.synchronize()
    del src, dst


def cpu_baseline_other(w, torch, q, k, v, mp, ratios, dout, dense_flops, density, causal):
    """The oracle on the host cores for the training-step and causal-prefill configurations, on a bounded sample of the
    workload scaled to the whole step (what the sample was is in `sample`)."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import psa_oracle as O

    ncores = os.cpu_count() or 1
    torch.set_num_threads(min(ncores, 32))
    B, H, D, bm, bn = w["B"], w["H"], w["D"], w["bm"], w["bn"]
    L = q.shape[2]
    Mq = -(-L // bm)
    qc, kc, vc = q[:, :1].float().cpu(), k[:, :1].float().cpu(), v[:, :1].float().cpu()
    mc = mp[:, :1].cpu().numpy().astype("int32")
    qblocks = list(range(0, Mq, max(1, Mq // 16)))[:16]
    if causal:
        t0 = time.perf_counter()
        est = O.estimate_xattn(qc, kc, block_size=bm, stride=w.get("stride", 8), causal=True)
        O.level_map_qwen(est.numpy(), ratios, w.get("text", 0), "energybound", block_size=bm, causal=True)
        t_front = time.perf_counter() - t0
        t1 = time.perf_counter()
        O.psa_attention_blockwalk(qc, kc, vc, mc, bm, bn, causal=True, qblocks=qblocks)
        t_attn = (time.perf_counter() - t1) * (Mq / len(qblocks))
        secs = (t_front + t_attn) * H
        sample = ("query head 0 of %d in fp32: full antidiagonal estimate + level map, causal attention on %d of %d q-blocks "
                  "(evenly spaced) scaled to all; then scaled by the head count" % (H, len(qblocks), Mq))
    else:
        t1 = time.perf_counter()
        O.psa_attention_blockwalk(qc, kc, vc, mc, bm, bn, qblocks=qblocks)
        t_fwd = (time.perf_counter() - t1) * (Mq / len(qblocks)) * H
        # backward: autograd through the dense restatement (fp64) on the first 2048 tokens of head 0 with the map's
        # top-left corner, scaled by the ratio of executed flops
        Lc = 2048
        nb = Lc // bm
        mcc = mc[:, :, :nb, :nb]
        t2 = time.perf_counter()
        O.psa_backward_dense(qc[:, :, :Lc], kc[:, :, :Lc], vc[:, :, :Lc], mcc, dout[:, :1, :Lc].float().cpu(), bm, bn)
        t_b = time.perf_counter() - t2
        dens_c = float(O.density(mcc))
        t_bwd = t_b * (density * float(L) * L * H) / max(dens_c * float(Lc) * Lc, 1.0)
        secs = t_fwd + t_bwd
        sample = ("head 0 of %d: forward in fp32 on %d of %d q-blocks scaled to all rows and heads; backward = fp64 autograd through the "
                  "dense restatement on the first %d tokens (map's top-left %dx%d blocks, density %.3f), scaled by executed flops"
                  % (H, len(qblocks), Mq, Lc, nb, nb, dens_c))
    return {"value": round(dense_flops / secs / 1e12, 5), "unit": "TFLOP/s (effective)", "ms_per_step": round(secs * 1e3, 1),
            "cores": torch.get_num_threads(), "host_cpus": ncores, "kind": "port", "sample": sample}


def run_other(args, w, torch, ops, make_qkv, sample_offsets, dev):
    """The training-step and causal-prefill configurations: same JSON layout, their own stages."""
    B, H, D, bm, bn = w["B"], w["H"], w["D"], w["bm"], w["bn"]
    Hkv = w.get("Hkv", H)
    text = w.get("text", 0)
    causal = w["kind"] == "causal"
    q, k, v = make_qkv(B, H, Hkv, w["grid"], D, seed=args.seed, device=dev, text_tokens=text, text_first=causal)
    if "tokens" in w:
        q, k, v = (t[:, :, :w["tokens"]].contiguous() for t in (q, k, v))
    L = q.shape[2]
    it = max(5, min(args.steps, 30))
    stages = {}
    if causal:
        # antidiagonal estimate -> causal level map (energy bound scaled to the sparsity target) -> causal GQA forward
        base = {1: (0.0, 0.5), 2: (0.5, 0.6), 4: (0.6, 0.7), 8: (0.7, 0.8), 0: (0.8, 1.0)}
        est = ops.estimate_xattn(q, k, block_size=bm, stride=w.get("stride", 8), causal=True)
        lo, hi = 0.05, 1.25
        for _ in range(16):
            tau = 0.5 * (lo + hi)
            ratios = {lv: ((a * tau, b * tau) if lv else (0.8 * tau, 1.0)) for lv, (a, b) in base.items()}
            mp = ops.level_map_qwen(est, ratios, text, "energybound", block_size=bm, causal=True, map_dtype=torch.int8)
            dens = float(ops.density(mp, causal=True)[-1])
            lo, hi = (tau, hi) if 1 - dens > w["sparsity"] else (lo, tau)

        def step():
            e = ops.estimate_xattn(q, k, block_size=bm, stride=w.get("stride", 8), causal=True)
            m = ops.level_map_qwen(e, ratios, text, "energybound", block_size=bm, causal=True, map_dtype=torch.int8)
            return ops.sparse_attention_fwd(q, k, v, m, bm, bn, causal=True)

        stages["estimate_xattn"], _ = time_gpu(lambda: ops.estimate_xattn(q, k, block_size=bm, stride=w.get("stride", 8), causal=True), it)
        stages["level_map"], _ = time_gpu(lambda: ops.level_map_qwen(est, ratios, text, "energybound", block_size=bm, causal=True,
                                                                    map_dtype=torch.int8), it)
        kp, vp = ops.pool_kv(k, v, bn)
        stages["pool"], _ = time_gpu(lambda: ops.pool_kv(k, v, bn), it)
        t_fwd, t_fwd_avg = time_gpu(lambda: ops.sparse_attention_fwd(q, k, v, mp, bm, bn, causal=True, pools=(kp, vp)), it)
        stages["sparse_fwd"] = t_fwd
        dense_flops = 4.0 * L * L * D * H * B / 2  # lower triangle
    else:
        km, kn = bm // 4, bn // 4
        off_q = sample_offsets(B, H, bm, km, args.seed + 10, device=dev)
        off_k = sample_offsets(B, Hkv, bn, kn, args.seed + 11, device=dev)
        scores = ops.estimate_sampled(q, k, off_q, off_k, bm, bn, km, kn)
        lo, hi = 0.05, 1.25
        for _ in range(16):
            tau = 0.5 * (lo + hi)
            mp = ops.level_map(scores, scaled_ratios(tau), text, "thresholdbound", blocksize=bn, compute_tile=w["tn"], map_dtype=torch.int8)
            dens = float(ops.density(mp)[-1])
            lo, hi = (tau, hi) if 1 - dens > w["sparsity"] else (lo, tau)
        g = torch.Generator(device="cpu").manual_seed(args.seed + 5)
        dout = (torch.randn(q.shape, generator=g) * 0.02).to(torch.bfloat16).to(dev)
        out, lse, pools = ops.sparse_attention_fwd(q, k, v, mp, bm, bn, return_lse=True)

        def step():
            o, l, pl = ops.sparse_attention_fwd(q, k, v, mp, bm, bn, return_lse=True)
            return ops.sparse_attention_bwd(q, k, v, mp, o, dout, l, bm, bn, pools=pl)

        t_fwd, t_fwd_avg = time_gpu(lambda: ops.sparse_attention_fwd(q, k, v, mp, bm, bn, return_lse=True), it)
        stages["sparse_fwd_with_pooling"] = t_fwd
        stages["backward"], _ = time_gpu(lambda: ops.sparse_attention_bwd(q, k, v, mp, out, dout, lse, bm, bn, pools=pools), it)
        dense_flops = 4.0 * L * L * D * H * B * 3.5  # forward + backward of dense attention
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    marks[0].record()
    for i in range(args.steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    ms_step = marks[0].elapsed_time(marks[-1]) / args.steps
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    density = float(ops.density(mp, causal=causal)[-1])
    cpu = None if args.no_cpu else cpu_baseline_other(w, torch, q, k, v, mp, ratios if causal else None, dout if not causal else None,
                                                    dense_flops, density, causal)
    fwd_flops = 4.0 * L * L * D * H * B * density * (0.5 if causal else 1.0)
    stages = {kk: round(vv, 4) for kk, vv in stages.items()}
    stages["step"] = round(ms_step, 4)
    if args.copy_calib:
        copy_calib(torch, dev)
    return {
        "metric": METRIC, "value": round(dense_flops / (ms_step * 1e-3) / 1e12, 2),
        "unit": "effective TFLOP/s (dense-equivalent flops of the step / step time)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "ms_per_step_median": round(per_step[len(per_step) // 2], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (seeded smooth 3-D field + noise, logit std ~3; text tokens i.i.d. N(0,1))",
        "config": {"workload": w["name"], "L": L, "block_m": bm, "block_n": bn, "density": round(density, 4),
                   "sparsity": round(1 - density, 4)},
        "stages_ms": stages,
        "roofline": {"kernel": "psa_fwd_pp_kernel" if (D == 128 and bm == 128) else "psa_fwd_lds_kernel", "bound": "mfma",
                     "achieved": round(fwd_flops / (t_fwd_avg * 1e-3) / 1e12, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(fwd_flops / (t_fwd_avg * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4), "traffic": fwd_traffic_bytes(args.workload),
                     "flops_per_launch": fwd_flops, "avg_launch_ms": round(t_fwd_avg, 4)},
        "cpu_baseline": cpu,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-dense", action="store_true", help="skip the dense-attention comparison legs (keeps kernel profiles clean)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the token re-ordering and preset legs (reorder_ms, preset_ms): a profile then holds the timed layer's "
                         "kernels only")
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--copy-calib", action="store_true",
                    help="after the run, stream 1 GiB through a plain elementwise kernel (reads 1 GiB, writes 1 GiB): "
                         "under rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE its reading calibrates the counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; the path shards by (batch, head) with no exchange, "
              "but nothing here launches more than one rank. Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    if not os.path.exists(os.path.join(PKG, "psa_hip", "libpsa_hip.so")):
        import build_ext

        build_ext.build(verbose=False)
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    w = WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if w.get("kind") in ("train", "causal"):
        print(json.dumps(run_other(args, w, torch, ops, make_qkv, sample_offsets, dev)))
        return
    B, H, D, bm, bn, tn = w["B"], w["H"], w["D"], w["bm"], w["bn"], w["tn"]
    text = w.get("text", 0)
    tdtype = {"bf16": torch.bfloat16, "fp32": torch.float32}[w.get("dtype", "bf16")]
    peak = PEAK_FP32_TFLOPS if tdtype == torch.float32 else PEAK_BF16_TFLOPS
    q, k, v = make_qkv(B, H, H, w["grid"], D, seed=args.seed, device=dev, text_tokens=text, dtype=tdtype)
    L = q.shape[2]
    Mq, Nk = -(-L // bm), -(-L // bn)
    km, kn = bm // 4, bn // 4
    off_q = sample_offsets(B, H, bm, km, args.seed + 10, device=dev)
    off_k = sample_offsets(B, H, bn, kn, args.seed + 11, device=dev)

    mode = w.get("mode", "thresholdbound")
    if "ratios" in w:
        ratios, tau = w["ratios"], float("nan")  # a preset of the reference, used as it is
    else:
        # ---- calibrate tau so that sparsity ~= target (bisection on the level map, untimed) ----
        scores = ops.estimate_sampled(q, k, off_q, off_k, bm, bn, km, kn)
        lo, hi = 0.05, 1.25
        for _ in range(18):
            tau = 0.5 * (lo + hi)
            m = ops.level_map(scores, scaled_ratios(tau), text, mode, blocksize=bn, compute_tile=tn, map_dtype=torch.int8)
            dens = float(ops.density(m)[-1])
            if 1 - dens > w["sparsity"]:
                lo = tau
            else:
                hi = tau
        ratios = scaled_ratios(tau)

    state = {}

    def layer():
        # estimate -> level map -> pooling -> forward
        o, mp = ops.psa_layer_fwd(q, k, v, off_q, off_k, ratios, mode, bm, bn, tn, return_map=True, text_length=text)
        state.update(mp=mp, o=o)
        return o

    # ---- the timed region: W warm-up steps, then exactly K steps --------------------------
    for _ in range(args.warmup):
        layer()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    marks[0].record()
    for i in range(args.steps):
        layer()
        marks[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_step = marks[0].elapsed_time(marks[-1]) / args.steps
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    ms_step_median = per_step[len(per_step) // 2]

    # the same layer captured into one HIP graph (kernel nodes only) and replayed
    def layer_graph():
        return ops.psa_layer_fwd_graph(q, k, v, off_q, off_k, ratios, mode, bm, bn, tn, return_map=True, text_length=text)

    o_g, mp_g = layer_graph()
    torch.cuda.synchronize()
    graph_equal = bool(torch.equal(o_g, state["o"])) and bool(torch.equal(mp_g, state["mp"]))
    t_graph, _ = time_gpu(layer_graph, max(10, min(args.steps, 100)))

    mp = state["mp"]
    kp, vp = ops.pool_kv(k, v, bn)
    state["s"] = ops.estimate_sampled(q, k, off_q, off_k, bm, bn, km, kn)
    density = float(ops.density(mp)[-1])
    dense_flops = 4.0 * L * L * D * H * B
    exec_flops = dense_flops * density

    # ---- per-kernel timings (HIP events on the launch stream) ------------------------------
    it = max(10, min(args.steps, 100))
    t_pool, _ = time_gpu(lambda: ops.pool_kv(k, v, bn), it)
    t_est, _ = time_gpu(lambda: ops.estimate_sampled(q, k, off_q, off_k, bm, bn, km, kn), it)
    # the sampling offsets of a layer call (one device-side draw for q and k; the timed layer takes fixed offsets so
    # that every step computes the same map)
    t_draw, _ = time_gpu(lambda: ops.draw_sample_offsets(B, H, H, bm, km, bn, kn, dev), it)
    t_map, _ = time_gpu(lambda: ops.level_map(state["s"], ratios, text, mode, blocksize=bn, compute_tile=tn, map_dtype=torch.int8), it)
    out_buf = torch.empty_like(q)
    # the map's tile schedule is built once per map (by the layer, right after the map): timed as a stage of its own,
    # and the forward kernel is timed on the prebuilt schedule
    sched, t_sched = None, None
    if ops.lib.psa_schedule_bytes(B, H, H, L, D, bm, bn) > 0:
        sched = ops.build_schedule(mp, H, L, D, bm, bn)
        t_sched, _ = time_gpu(lambda: ops.build_schedule(mp, H, L, D, bm, bn, out=sched), it)
    fwd_call = lambda: ops.sparse_attention_fwd(q, k, v, mp, bm, bn, pools=(kp, vp), out=out_buf, schedule=sched)
    t_fwd_med, t_fwd_avg = time_gpu(fwd_call, it)
    exec_flops_fwd = 4.0 * L * L * D * H * B * float(ops.density(mp)[-1])
    tele = None if args.no_extras else load_telemetry(fwd_call, t_fwd_avg, exec_flops_fwd)
    sclk = tele["sclk_mhz"] if tele else None
    lib_gemm = None
    if not args.no_extras:
        # context: what the vendor library's bf16 GEMM (torch.matmul, 8192^3) sustains on this box, at which clock and power
        ga = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
        gb = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
        gemm_call = lambda: torch.matmul(ga, gb)
        _, t_gemm = time_gpu(gemm_call, 30)
        lib_gemm = {"what": "torch.matmul bf16 8192 x 8192 x 8192", "ms": round(t_gemm, 4),
                    "tflops": round(2.0 * 8192 ** 3 / (t_gemm * 1e-3) / 1e12, 1),
                    "frac_of_peak": round(2.0 * 8192 ** 3 / (t_gemm * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)}
        lib_gemm.update(load_telemetry(gemm_call, t_gemm, 2.0 * 8192 ** 3))
        del ga, gb
    t_dense = t_sdpa = None
    if not args.no_dense:
        t_dense, _ = time_gpu(lambda: ops.sparse_attention_fwd(q, k, v, None, bm, bn, out=out_buf), max(3, it // 10), warm=5)
        t_sdpa, _ = time_gpu(lambda: torch.nn.functional.scaled_dot_product_attention(q, k, v), max(3, it // 10), warm=3)

    reorder = preset = None
    if not args.no_extras:
        # ---- token re-ordering: the layer on tokens already in curve order (above), the same layer reading / writing through
        # the token index (no gather passes), and with explicit gather passes before and after; the inputs of the last two
        # are the un-gathered q, k, v, so all three compute the same layer and the outputs must agree bit for bit
        from psa_hip.utils.rearranger import GilbertRearranger

        gd, gh, gw = w["grid"]
        rr = GilbertRearranger(gw, gh, gd, text)
        idx = rr.token_index(dev)
        inv = rr._combined_index(dev, False)
        q0, k0, v0 = ops.gather_rows((q, k, v), inv)  # q0[idx[i]] = q[i]

        def layer_indexed():
            return ops.psa_layer_fwd(q0, k0, v0, off_q, off_k, ratios, mode, bm, bn, tn, text_length=text, token_index=idx)

        def layer_gathered():
            qg, kg, vg = ops.gather_rows((q0, k0, v0), idx)
            og = ops.psa_layer_fwd(qg, kg, vg, off_q, off_k, ratios, mode, bm, bn, tn, text_length=text)
            return ops.gather_rows((og,), inv)[0]

        o_ref = layer()
        reorder_equal = bool(torch.equal(layer_indexed(), layer_gathered())) and bool(torch.equal(ops.gather_rows((layer_indexed(),), idx)[0], o_ref))
        t_l0, _ = time_gpu(layer, it)
        t_l1, _ = time_gpu(layer_indexed, it)
        t_l2, _ = time_gpu(layer_gathered, it)
        reorder = {"layer_tokens_already_ordered": round(t_l0, 4), "layer_through_token_index": round(t_l1, 4),
                   "layer_with_gather_passes": round(t_l2, 4), "outputs_bit_identical": reorder_equal}
        del q0, k0, v0

        # ---- the same layer through the module API with what the reference's preset for this model turns on (Gilbert
        # re-ordering, key-similarity cap; similarity thresholds of the preset); inputs in raster order
        if args.workload == "c2":
            from psa_hip.pyramid_sparse_attention import AttentionConfig, PyramidSparseAttention

            cfg = AttentionConfig(width=gw, height=gh, depth=gd, text_length=text, use_rearrange=True, rearrange_method="Gilbert",
                                  attn_impl="old_mask_type", mask_mode=mode, warmup_steps=0, use_sim_mask=True, block_m=bm, block_n=bn,
                                  tile_n=tn, mask_ratios=ratios, sim_2x_threshold=0.7, sim_4x_threshold=0.65, sim_8x_threshold=0.6,
                                  enable_logging=False)
            mod = PyramidSparseAttention(cfg, inference_num=50, layer_num=30, model_type="wan")
            mod.sample_offsets = (off_q, off_k)
            with torch.inference_mode():
                t_mod, _ = time_gpu(lambda: mod(q, k, v, 0), it)
                t_ks, _ = time_gpu(lambda: ops.k_similarity(k, bn, 0.7, 0.65, 0.6), it)
            preset = {"module_layer": round(t_mod, 4), "k_similarity": round(t_ks, 4),
                      "what": "PyramidSparseAttention.forward, Gilbert re-ordering through the token index + similarity cap"}

    pool_bytes = 2.0 * B * H * (Nk * bn) * D * q.element_size() * (1 + 7 / 8)
    est_flops = 2.0 * (Mq * km) * (Nk * kn) * D * B * H

    roofline = {
        "kernel": ("psa_fwd_f32_kernel" if tdtype == torch.float32 else
                   "psa_fwd_pp_kernel" if (D == 128 and bm == 128) else "psa_fwd_lds_kernel"),
        "bound": "mfma",  # (the fp32 kernel computes on the vector units; its peak is the fp32 figure)
        "achieved": round(exec_flops / (t_fwd_avg * 1e-3) / 1e12, 2),
        "peak": peak,
        "unit": "TFLOP/s",
        "frac": round(exec_flops / (t_fwd_avg * 1e-3) / 1e12 / peak, 4),
        # HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command (scaled by the
        # readings of --copy-calib's 1 GiB kernel); measured for the default workload only
        "traffic": fwd_traffic_bytes(args.workload),
        "flops_per_launch": exec_flops,
        "avg_launch_ms": round(t_fwd_avg, 4),
        # context, not the fraction that counts: the shader clock under this kernel (the board's power limit holds it under
        # the 2400 MHz the peak is quoted at) and the fraction of the peak scaled to that clock
        "sclk_mhz_under_load": sclk,
        "frac_at_that_clock": None if not sclk else round(exec_flops / (t_fwd_avg * 1e-3) / 1e12 / (peak * sclk / 2400.0), 4),
        # board power while the kernel runs back to back (rocm-smi's energy counter; the board's cap is 1400 W)
        "avg_power_w_under_load": tele["avg_power_w"] if tele else None,
        "pj_per_flop": tele["pj_per_flop"] if tele else None,
        "launch_includes": ("the forward kernel alone (it walks the map's prebuilt tile schedule: stages_ms.schedule)" if sched is not None
                            else "the forward kernel and its two row-ordering launches"),
    }
    # ---- CPU baseline: the oracle on the host cores over a bounded sample -------------------
    cpu = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import psa_oracle as O

        ncores = os.cpu_count() or 1
        torch.set_num_threads(min(ncores, 32))
        def cpu_sample(heads, qblocks, reps):
            qc, kc, vc = (t[:, heads].float().cpu() for t in (q, k, v))
            mc = mp[:, heads].cpu().numpy().astype("int32")
            oqc, okc = off_q[:, heads].cpu(), off_k[:, heads].cpu()
            best, o_c = None, None
            for _ in range(reps):
                t0c = time.perf_counter()
                s_c = O.estimate_sampled(qc, kc, bm, bn, oqc, okc)
                O.level_map(s_c.numpy(), ratios, text, mode, blocksize=bn, compute_tile=tn)
                t_front = time.perf_counter() - t0c  # pooling is inside blockwalk
                t1c = time.perf_counter()
                o_c, _ = O.psa_attention_blockwalk(qc, kc, vc, mc, bm, bn, qblocks=qblocks)
                t_attn = (time.perf_counter() - t1c) * (Mq / len(qblocks))
                t_all = (t_front + t_attn) * (H / len(heads))
                best = t_all if best is None else min(best, t_all)
            # the rows the oracle computed against the GPU layer's output (same map: the GPU's)
            rows = torch.cat([torch.arange(I * bm, min((I + 1) * bm, L)) for I in qblocks])
            d = (state["o"][:, heads][:, :, rows.to(dev)].float().cpu() - o_c[:, :, rows]).abs()
            return best, float(d.max()), float(d.mean())

        # a small sample first (two heads, 32 evenly spaced q-blocks, scaled); if the whole layer fits the budget of a
        # bounded baseline (three repetitions within about 30 s), time the whole layer instead; the minimum counts
        heads = [0, 1] if H >= 2 else [0]
        qblocks = list(range(0, Mq, max(1, Mq // 32)))[:32]
        cpu_s_per_layer, cpu_max_abs, cpu_mean_abs = cpu_sample(heads, qblocks, 1)
        if cpu_s_per_layer <= 10.0:
            heads, qblocks = list(range(H)), list(range(Mq))
            cpu_s_per_layer, cpu_max_abs, cpu_mean_abs = cpu_sample(heads, qblocks, 3)
        cpu = {
            "value": round(dense_flops / cpu_s_per_layer / 1e12, 5),
            "unit": "TFLOP/s (effective)",
            "ms_per_layer": round(cpu_s_per_layer * 1e3, 1),
            "cores": torch.get_num_threads(),
            "host_cpus": ncores,
            "kind": "port",
            "repetitions": 3 if (len(heads) == H and len(qblocks) == Mq) else 1,
            # the GPU layer's output against the oracle's (run on the same tensors, in fp32) on the rows the oracle computed
            # (tolerance of the 16-bit types: 2e-2 / 2e-3)
            "max_abs": round(cpu_max_abs, 5), "mean_abs": round(cpu_mean_abs, 6),
            "sample": ("the whole layer in fp32: all %d heads, all %d q-blocks (estimate + level map + attention), minimum of 3" % (H, Mq))
            if len(heads) == H and len(qblocks) == Mq else
            ("heads %s of %d in fp32: full estimate + level map, attention on %d of %d q-blocks scaled to all; "
             "then scaled by H/%d" % (heads, H, len(qblocks), Mq, len(heads))),
        }

    if args.copy_calib:
        copy_calib(torch, dev)

    eff_tflops = dense_flops / (ms_step * 1e-3) / 1e12
    line = {
        "metric": METRIC,
        "value": round(eff_tflops, 2),
        "unit": "effective TFLOP/s (dense-equivalent 4*N^2*D*H flops per layer / layer time)",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "ms_per_step_median": round(ms_step_median, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w.get("dtype", "bf16"),
        "data": "synthetic (seeded smooth 3-D field + noise, logit std ~3)",
        "config": {"workload": w["name"], "L": L, "block_m": bm, "block_n": bn, "density": round(density, 4),
                   "sparsity": round(1 - density, 4), "mask_mode": mode, "tau": None if tau != tau else round(tau, 4)},
        "stages_ms": {"sampling_draw": round(t_draw, 4), "pool": round(t_pool, 4), "estimate": round(t_est, 4), "level_map": round(t_map, 4),
                      "schedule": None if t_sched is None else round(t_sched, 4), "sparse_fwd": round(t_fwd_med, 4), "layer": round(ms_step, 4), "wall_per_step": round(wall_ms / args.steps, 4),
                      "layer_graph": round(t_graph, 4), "layer_graph_bit_identical": graph_equal},
        "reorder_ms": reorder,
        "preset_ms": preset,
        "library_gemm": lib_gemm,
        "executed_tflops_fwd": round(exec_flops / (t_fwd_med * 1e-3) / 1e12, 2),
        "pct_bf16_peak_fwd_executed": round(100 * exec_flops / (t_fwd_med * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 2),
        "pool_gbs": round(pool_bytes / (t_pool * 1e-3) / 1e9, 1),
        "pool_pct_hbm": round(100 * pool_bytes / (t_pool * 1e-3) / 1e9 / PEAK_HBM_GBS, 2),
        "estimate_tflops": round(est_flops / (t_est * 1e-3) / 1e12, 2),
        "dense_fa": None if t_dense is None else {
            "own_kernel_ms": round(t_dense, 3), "own_kernel_tflops": round(dense_flops / (t_dense * 1e-3) / 1e12, 1),
            "torch_sdpa_ms": round(t_sdpa, 3), "layer_speedup_vs_own_dense": round(t_dense / ms_step, 2),
            "layer_speedup_vs_sdpa": round(t_sdpa / ms_step, 2)},
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
