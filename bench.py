#!/usr/bin/env python3
"""Benchmark of the Flash3D forward hot path on one MI355X.

A step = one encoder-stage forward on 4 synthetic LiDAR sweeps x 120,000 points (BASELINE config
"encoder stage"): PSH bucketing (bbox + hash + claim + scatter) -> coordinate embedding ->
LayerNorm -> QKV GEMM -> bucketed attention -> out-projection + residual -> LayerNorm + gated MLP
(256 -> 1024 -> 256) + residual, the MLP as one kernel.  C = 256, 8 heads x 32, bucket 512, scope of 1 bucket, hash 2.

Prints ONE JSON line: whole-job throughput in Mpts/s, the roofline of the dominant kernel measured
live with stream events, per-op sub-metrics (attention TFLOP/s on config 2, PSH / pooling GB/s), and
a CPU baseline (the oracle pipeline on a bounded sample, host cores stated).
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a copy kernel of known
# size, see profiles/encoder_stage_4x120k_hbm_traffic.md) at this bench's shapes
TRAFFIC_FROM = "profiles/encoder_stage_4x120k_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this bench's step; re-measure when a kernel changes)"
TRAFFIC_BYTES_PER_LAUNCH = {"ln_fc1_act": 1.613e9, "ln_qkv": 1.022e9, "attention": 1.019e9,
                            "proj_residual": 0.767e9, "fc2_residual": 1.850e9, "ln_mlp_residual": 0.848e9,
                            "proj_ln_mlp_residual": 0.876e9, "embed_ln_qkv": 0.780e9, "embed_proj_ln_mlp_residual": 0.627e9,
                            "embed_attention": 0.266e9}


def ev_time(fn, iters, warmup=3):
    """average milliseconds of fn() over `iters` launches, timed with events on the current stream"""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def ev_stats(fn, batches=20, per_batch=10, warmup=10):
    """(median, min, mean) milliseconds per launch of fn(), from `batches` event-bracketed groups of `per_batch` launches"""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(batches)]
    for a, b in evs:
        a.record()
        for _ in range(per_batch):
            fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) / per_batch for a, b in evs)
    return t[len(t) // 2], t[0], sum(t) / len(t)


def cpu_baseline(clouds, emb, blk, C, H, bs, scope, hash_op, activation):
    """the oracle pipeline on the whole batch (the same 4 sweeps), repeated for about ten seconds of CPU work,
    all host cores for the torch part"""
    from oracle import f3d_oracle as orc
    import bench_workloads as synth
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    coords, seps = synth.batch_of(clouds)
    n = coords.shape[0]
    align = bs * scope * 6
    pad_to = -(-n // align) * align
    f = lambda p: p.detach().float().cpu().to(torch.bfloat16).float()
    w = {"norm.weight": f(blk.norm.weight), "norm.bias": f(blk.norm.bias), "qkv.weight": f(blk.bwa.qkv.weight),
         "qkv.bias": f(blk.bwa.qkv.bias), "proj.weight": f(blk.bwa.proj.weight), "proj.bias": f(blk.bwa.proj.bias),
         "ln.weight": f(blk.mlp.mlp.layer_norm_weight), "ln.bias": f(blk.mlp.mlp.layer_norm_bias),
         "fc1.weight": f(blk.mlp.mlp.fc1_weight), "fc1.bias": f(blk.mlp.mlp.fc1_bias),
         "fc2.weight": f(blk.mlp.mlp.fc2_weight), "fc2.bias": f(blk.mlp.mlp.fc2_bias)}
    ew, eb = f(emb.lin.weight), f(emb.lin.bias)
    passes, t0 = 0, time.perf_counter()
    with torch.no_grad():
        while passes < 2 or (time.perf_counter() - t0 < 10.0 and passes < 8):
            scat = orc.psh_scatter_coords(coords, seps, bs, pad_to, hash_op)
            x = orc._r(orc.linear(torch.from_numpy(scat.astype(np.float32)).to(torch.bfloat16), ew, eb))
            scopes = orc.gen_scopes(pad_to, bs, scope)
            out = orc.xfmr_block(x, w, scopes, bs, H, activation)
            passes += 1
    dt = time.perf_counter() - t0
    return {"value": n * passes / dt / 1e6, "unit": "Mpts/s", "cores": cores, "kind": "port",
            "sample": f"{passes} passes of the whole stage on the same 4 sweeps ({n} points) through the oracle "
                      f"(C PSH single-threaded + torch fp32 on {cores} threads), {dt:.1f} s of CPU work"}, out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--mlp", default="swiglu", choices=["swiglu", "gelu"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-sub-metrics", action="store_true")
    ap.add_argument("--sub-metrics-only", nargs="*", default=None, metavar="GROUP",
                    help="run only the per-kernel sub-metrics (configs 1, 2, 3, 5) and print them; for profiling those "
                         "kernels.  Optional group names restrict the run: attention, psh, permute, pool, hourglass, mfma, "
                         "backward")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; the path shards by cloud without any exchange between GPUs (each cloud "
              "is bucketed, pooled and attended to on its own), and no multi-GPU figure is produced. Re-run with --gpus 1.",
              file=sys.stderr)
        sys.exit(2)

    import bench_workloads as synth
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import psh_main
    dev = "cuda:0"
    if args.sub_metrics_only is not None:
        print(json.dumps({"sub_metrics": sub_metrics(dev, set(args.sub_metrics_only) or None)}))
        return
    C, HID, H, BS, SCOPE, HASH = 256, 1024, 8, 512, 1, 2
    clouds = [synth.lidar_sweep(120_000, 1004 + i) for i in range(4)]
    coords_np, seps_np = synth.batch_of(clouds)
    coords = torch.from_numpy(coords_np).to(dev)
    seps = torch.from_numpy(seps_np.view(np.int32)).to(dev).view(torch.uint32)
    n_pts = coords.shape[0]
    import bench_workloads as configs
    emb, blk = configs.encoder_stage(args.mlp, 1004)
    emb, blk = emb.to(dev), blk.to(dev)

    @torch.no_grad()
    def step():
        # lazy: the embedding is not stored; the block forms its rows inside the attention kernel (LayerNorm + QKV of the
        # rank-4 embedding, folded) and inside the out-projection + MLP kernel
        feat = emb(coords, seps, HASH, lazy=True)
        return blk(None, feat, None)

    @torch.no_grad()
    def step_stored():
        # the same stage with the embedding stored: the kernels a block runs on ANY input (LayerNorm+QKV, attention over
        # the stored projection output, out-projection + MLP)
        return blk(None, emb(coords, seps, HASH), None)

    # Priming, before the W warm-up steps: the first process on a fresh box has been seen to stall the host once, for
    # 30-40 ms, within its first dozen steps (the stall moves when unrelated host code before the loop changes, so it
    # is tied to time since start-up, not to a call); after only a handful of warm-up steps it lands inside the timed
    # steps and doubles their average.  Half a second of untimed steps puts it behind us.
    out = None
    t_prime = time.perf_counter()
    while time.perf_counter() - t_prime < 0.5:
        for _ in range(10):
            out = step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        out = step()      # held like in the timed loop, so that the caching allocator has seen the loop's pattern
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = n_pts / (dt / args.steps) / 1e6
    for _ in range(max(3, args.warmup)):
        step_stored()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_stored()
    torch.cuda.synchronize()
    ms_per_step_stored = (time.perf_counter() - t0) / args.steps * 1e3

    # ---- per-op breakdown on the same tensors, events on the launch stream ----
    with torch.no_grad():
        feat = emb(coords, seps, HASH)
        n_pad = feat.shape[0]
        mlp = blk.mlp.mlp
        bw = lambda p: p.detach().to(torch.bfloat16).contiguous()
        scopes = blk.swin_plan.gen_scopes_from_plan(n_pad, feat.device)
        ln_out, qkv = torch.empty_like(feat), torch.empty(n_pad, 3 * C, dtype=torch.bfloat16, device=dev)
        o = torch.empty(1, n_pad, H, C // H, dtype=torch.bfloat16, device=dev)
        lse = torch.zeros(1, n_pad, H, dtype=torch.float32, device=dev)
        mid, hid, y = torch.empty_like(feat), torch.empty(n_pad, HID, dtype=torch.bfloat16, device=dev), torch.empty_like(feat)
        Wn, Bn, Wq, Bq, Wp, Bp = bw(blk.norm.weight), bw(blk.norm.bias), bw(blk.bwa.qkv.weight), bw(blk.bwa.qkv.bias), bw(blk.bwa.proj.weight), bw(blk.bwa.proj.bias)
        W1, B1, W2, B2 = bw(mlp.fc1_weight), bw(mlp.fc1_bias), bw(mlp.fc2_weight), bw(mlp.fc2_bias)
        q, k, v = (t.view(1, n_pad, H, C // H) for t in qkv.chunk(3, dim=-1))
        Wm, Bm = bw(mlp.layer_norm_weight), bw(mlp.layer_norm_bias)
        # the launches the step above makes, one by one (LayerNorm is fused into the qkv and fc1 kernels)
        scat = emb.last_scattered_coord
        We, Be = bw(emb.lin.weight), bw(emb.lin.bias)
        emb_out = torch.empty_like(feat)
        etab = pshattn.embed_table(We, Be)
        swiglu = args.mlp == "swiglu"
        # with the gated MLP the embedding is formed inside its consumers and never stored, and Q, K, V neither: the
        # attention kernel forms its rows from the coordinates
        stored = {"coord_embed": lambda: pshattn.coord_embed_bf16(scat, We, Be, emb_out),
                  "ln_qkv": lambda: pshattn.ln_linear_bf16(feat, Wn, Bn, 1e-5, Wq, Bq, None, qkv, None)}
        attention = lambda: pshattn.buck_swin_fwd(q, k, v, o, lse, scopes, BS)
        ops = {"psh_scatter": lambda: psh_main.batch_bucket_scatter(coords, seps, BS, n_pad, HASH)}
        if swiglu:
            fold = pshattn.embed_qkv_fold(We, Be, Wn, Bn, 1e-5, Wq, Bq, H)
            ops["embed_attention"] = lambda: pshattn.embed_buck_swin_fwd(scat, fold[0], fold[1], o, lse, scopes, BS)
            stored["embed_ln_qkv"] = lambda: pshattn.embed_ln_linear_bf16(scat, etab, Wn, Bn, 1e-5, Wq, Bq, qkv)
            stored["attention"] = attention
        else:
            ops.update(stored)
            ops["attention"] = attention
        # the out-projection with its residual and the gated MLP with its residual run as one kernel at this size (the
        # block's choice at inference); with gelu: the projection, LayerNorm+fc1+act, then fc2
        separate = {"proj_residual": lambda: pshattn.linear_bf16(o.view(n_pad, C), Wp, Bp, feat, mid, None),
                    "ln_mlp_residual": lambda: pshattn.ln_mlp_swiglu_bf16(mid, Wm, Bm, 1e-5, W1, B1, W2, B2, mid, y)}
        two_kernel = {"ln_fc1_act": lambda: pshattn.ln_linear_bf16(mid, Wm, Bm, 1e-5, W1, B1, None, hid, args.mlp),
                      "fc2_residual": lambda: pshattn.linear_bf16(hid, W2, B2, mid, y, None)}
        if swiglu:
            ops["embed_proj_ln_mlp_residual"] = lambda: pshattn.embed_proj_ln_mlp_swiglu_bf16(
                o.view(n_pad, C), Wp, Bp, scat, etab, Wm, Bm, 1e-5, W1, B1, W2, B2, y)
            stored["proj_ln_mlp_residual"] = lambda: pshattn.proj_ln_mlp_swiglu_bf16(o.view(n_pad, C), Wp, Bp, feat, Wm, Bm,
                                                                                     1e-5, W1, B1, W2, B2, y)
        else:
            ops["proj_residual"] = separate["proj_residual"]
            ops.update(two_kernel)
        breakdown = {name: ev_time(fn, 20) for name, fn in ops.items()}
        two_kernel_ms = {name: ev_time(fn, 20) for name, fn in two_kernel.items()}
        separate_ms = {name: ev_time(fn, 20) for name, fn in separate.items()} if swiglu else {}
        stored_ms = {name: ev_time(fn, 20) for name, fn in stored.items()} if swiglu else {}
    fc1_n = 2 * HID if args.mlp == "swiglu" else HID
    flops = {"ln_qkv": 2.0 * n_pad * C * 3 * C, "embed_ln_qkv": 2.0 * n_pad * C * 3 * C + 2.0 * n_pad * 4 * C,
             "proj_residual": 2.0 * n_pad * C * C,
             "ln_fc1_act": 2.0 * n_pad * C * fc1_n, "fc2_residual": 2.0 * n_pad * HID * C,
             "ln_mlp_residual": 2.0 * n_pad * C * fc1_n + 2.0 * n_pad * HID * C,
             "proj_ln_mlp_residual": 2.0 * n_pad * C * C + 2.0 * n_pad * C * fc1_n + 2.0 * n_pad * HID * C,
             "embed_proj_ln_mlp_residual": 2.0 * n_pad * C * C + 2.0 * n_pad * C * fc1_n + 2.0 * n_pad * HID * C + 2.0 * n_pad * 4 * C,
             "attention": 4.0 * n_pad * BS * SCOPE * C,
             "embed_attention": 4.0 * n_pad * BS * SCOPE * C + 2.0 * n_pad * 4 * 3 * C}
    # algorithmic HBM bytes per launch (bf16 activations in and out, weights negligible)
    hbm_bytes = {"ln_qkv": 2.0 * n_pad * (C + 3 * C), "embed_ln_qkv": 2.0 * n_pad * 3 * C + 6.0 * n_pad,   # coordinates in, qkv out
                 "proj_residual": 2.0 * n_pad * 3 * C,
                 "ln_fc1_act": 2.0 * n_pad * (C + HID), "fc2_residual": 2.0 * n_pad * (HID + 2 * C),
                 "ln_mlp_residual": 2.0 * n_pad * 2 * C,      # x (also the residual) in, y out
                 "proj_ln_mlp_residual": 2.0 * n_pad * 3 * C,  # attention output and block input in, y out
                 "embed_proj_ln_mlp_residual": 2.0 * n_pad * 2 * C + 6.0 * n_pad,  # attention output and coordinates in, y out
                 "attention": 2.0 * n_pad * 4 * C + 4.0 * n_pad * H,
                 "embed_attention": 6.0 * n_pad + 2.0 * n_pad * C + 4.0 * n_pad * H}   # coordinates in, O and LSE out
    kernels = {"attention": "buck_swin_fwd_scope_kernel<32,512,16>",
               "embed_attention": "buck_swin_fwd_scope_kernel<32,512,16,rows formed in the kernel>",
               "ln_qkv": "xstat_linear_kernel<256,2,8,3,LN> + ln_fold_kernel",
               "embed_ln_qkv": "xstat_linear_kernel<256,2,8,3,LN,embed> + ln_fold_kernel",
               "embed_proj_ln_mlp_residual": "ln_mlp_swiglu_kernel<256, true, true> + mlp_prep_kernel",
               "ln_fc1_act": "xstat_linear_kernel<256,2,8,3,LN,swiglu> + ln_fold_kernel",
               "proj_residual": "xstat_linear_kernel<256,2,8,3,residual>",
               "fc2_residual": "ystat_linear_kernel<256> + ys_w_prep_kernel",
               "ln_mlp_residual": "ln_mlp_swiglu_kernel<256, false> + mlp_prep_kernel",
               "proj_ln_mlp_residual": "ln_mlp_swiglu_kernel<256, true> + mlp_prep_kernel"}
    all_flops = dict(flops)
    flops = {kname: vv for kname, vv in flops.items() if kname in breakdown}
    # the two-kernel form of the MLP (what the layer runs below 60 k rows, or with fused=False), same tensors
    two_kernel_mlp = None
    if args.mlp == "swiglu":
        ms_2 = two_kernel_ms["ln_fc1_act"] + two_kernel_ms["fc2_residual"]
        two_kernel_mlp = {"kernels": kernels["ln_fc1_act"] + " ; " + kernels["fc2_residual"],
                          "ms": {kname: round(vv, 4) for kname, vv in two_kernel_ms.items()},
                          "tflops": round(all_flops["ln_mlp_residual"] / ms_2 / 1e9, 1),
                          "traffic": TRAFFIC_BYTES_PER_LAUNCH["ln_fc1_act"] + TRAFFIC_BYTES_PER_LAUNCH["fc2_residual"],
                          "hidden_activation_bytes": int(n_pad) * HID * 2}
    # the out-projection and the one-kernel MLP as two launches (what the block runs under autograd), same tensors
    separate_proj_mlp = None
    if separate_ms:
        separate_proj_mlp = {"kernels": kernels["proj_residual"] + " ; " + kernels["ln_mlp_residual"],
                             "ms": {kname: round(vv, 4) for kname, vv in separate_ms.items()},
                             "ln_mlp_tflops": round(all_flops["ln_mlp_residual"] / separate_ms["ln_mlp_residual"] / 1e9, 1),
                             "x1_bytes_written_and_read_again": int(n_pad) * C * 2 * 3}
    dominant = max(flops, key=lambda kname: breakdown[kname])
    t_dom = breakdown[dominant] * 1e-3
    ach = flops[dominant] / t_dom / 1e12
    # the binding roof is the one with the larger minimum time
    t_mfma, t_hbm = flops[dominant] / (MFMA_BF16_PEAK_TFLOPS * 1e12), hbm_bytes[dominant] / (HBM_PEAK_GBS * 1e9)
    if t_mfma >= t_hbm:
        roofline = {"kernel": kernels[dominant], "op": dominant, "bound": "mfma", "achieved": round(ach, 2),
                    "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(ach / MFMA_BF16_PEAK_TFLOPS, 4)}
    else:
        gbs = hbm_bytes[dominant] / t_dom / 1e9
        roofline = {"kernel": kernels[dominant], "op": dominant, "bound": "hbm", "achieved": round(gbs, 1),
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4)}
    roofline.update({"traffic": TRAFFIC_BYTES_PER_LAUNCH.get(dominant), "traffic_from": TRAFFIC_FROM, "avg_launch_ms": round(breakdown[dominant], 4),
                     "algorithmic_flop_per_launch": flops[dominant],
                     "algorithmic_hbm_bytes_per_launch": hbm_bytes[dominant]})
    per_op = {kname: {"ms": round(breakdown[kname], 4), "tflops": round(flops[kname] / breakdown[kname] / 1e9, 1),
                      "hbm_gbs": round(hbm_bytes[kname] / breakdown[kname] / 1e6, 1)} for kname in flops}

    sub = {}
    if not args.no_sub_metrics:
        sub = sub_metrics(dev)

    result = {
        "metric": "Flash3D encoder-stage forward throughput @ 4x120k-point LiDAR sweeps",
        "value": round(value, 3), "unit": "Mpts/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "encoder stage fwd: PSH -> embed -> LN -> QKV -> bucketed attention -> proj -> MLP "
                               f"({args.mlp}) on 4 synthetic LiDAR sweeps x 120k points",
                   "points": n_pts, "padded_rows": int(n_pad), "channels": C, "heads": H, "head_dim": C // H,
                   "mlp_hidden": HID, "bucket_size": BS, "scope_size": SCOPE, "hash_type": HASH,
                   "first_block": "the stage's input is the coordinate embedding (rank 4), as in the reference's model: LayerNorm + "
                                  "QKV projection fold into four numbers per output feature and the attention kernel forms Q, K, V "
                                  "from the rows' coordinates; the same function of the same inputs and weights (parity_vs_oracle), "
                                  "no stored embedding / LayerNorm / QKV tensors; stored_intermediates times the unfolded kernels",
                   "host_sync": "none in the timed loop: the batch is replayed, and cloud sizes / bucket geometry are cached "
                                "per separator tensor; a fresh batch pays one host synchronisation in PSH"},
        "roofline": roofline,
        "breakdown_ms": {kname: round(vv, 4) for kname, vv in breakdown.items()},
        "per_op": per_op,
        "stored_intermediates": {"ms_per_step": round(ms_per_step_stored, 4),
                                 "mpts_per_s": round(n_pts / ms_per_step_stored / 1e3, 3),
                                 "what": "the same stage with the embedding and the QKV projection stored (the kernels a "
                                         "block runs on any input); `value` is the first block as the reference's model "
                                         "feeds it: its input is the coordinate embedding (flash3d.py:162-163)",
                                 "kernels_ms": {kname: round(vv, 4) for kname, vv in stored_ms.items()} or None},
        "separate_proj_and_mlp_under_autograd": separate_proj_mlp,
        "two_kernel_mlp_on_request": two_kernel_mlp,
        "sub_metrics": sub,
    }
    if not args.no_cpu_baseline:
        cb, ref_out = cpu_baseline(clouds, emb, blk, C, H, BS, SCOPE, HASH, args.mlp)
        result["cpu_baseline"] = cb
        # the timed step's output against the oracle's on the same batch (the checker, not the thing measured)
        err = (out.float().cpu() - ref_out).abs()
        result["parity_vs_oracle"] = {"max_abs_err": round(err.max().item(), 5), "mean_abs_err": round(err.mean().item(), 6),
                                      "ref_mean_abs": round(ref_out.abs().mean().item(), 5),
                                      "ref_max_abs": round(ref_out.abs().max().item(), 4),
                                      "rows": int(ref_out.shape[0])}
    print(json.dumps(result))


def sub_metrics(dev, only=None):
    """attention TFLOP/s on config 2, PSH GB/s (config 1 latency + saturating size), pooling and
    unpooling GB/s on config 3 — each against its roofline.  `only`: a set of group names, or None for all"""
    out = {}
    groups = {"attention": sub_attention, "psh": sub_psh, "permute": sub_permute, "pool": sub_pool,
              "hourglass": sub_hourglass, "mfma": sub_mfma_rate, "issue": sub_issue, "stores": sub_store_rows,
              "backward": sub_backward}
    for name, fn in groups.items():
        if only is None or name in only:
            fn(dev, out)
    return out


def _bench_probe():
    """bench_probe.so beside this file (built by __graft_entry__.build() from bench_probe.hip): measurement aids that
    are not part of the library"""
    import ctypes
    path = os.path.join(ROOT, "bench_probe.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: run `python __graft_entry__.py` first")
    return ctypes.CDLL(path)


def issue_probe(dev, mode, iters=20000):
    """shader clocks a SIMD spends per loop trip of bench_probe_issue's mode with four waves on it, and the shader clock
    it ran at.  The SIMD's arbiter serves its oldest wave first, so the four waves of a SIMD finish one after the other:
    the last one's elapsed clocks are the time of all four (4 x trips)."""
    import ctypes
    lib = _bench_probe()
    n_cu = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    clocks = torch.zeros(n_cu * 16, 2, dtype=torch.int64, device=dev)
    for _ in range(2):
        rc = lib.bench_probe_issue(ctypes.c_uint32(mode), ctypes.c_uint32(n_cu), ctypes.c_uint32(iters),
                                   ctypes.c_void_p(sink.data_ptr()), ctypes.c_void_p(clocks.data_ptr()),
                                   ctypes.c_void_p(torch.cuda.current_stream(0).cuda_stream))
        if rc != 0:
            raise RuntimeError(f"bench_probe_issue failed with {rc}")
    torch.cuda.synchronize()
    ck = clocks.double().cpu().view(n_cu, 4, 4, 2)          # workgroup, wave / 4, SIMD (wave % 4), counter
    last = ck[..., 0].max(dim=1).values                     # the last wave of each SIMD
    ghz = (ck[..., 0] / (ck[..., 1] / 100e6) / 1e9).median().item()
    return last.median().item() / (4.0 * iters), ghz


def sub_issue(dev, out):
    """What the vector issue port of a SIMD takes for the instructions of the attention forward's inner step (one
    32 x 32 block of scores at 32-wide heads: 16 v_exp_f32, 8 v_cvt_pk_bf16_f32, four 32x32x16 and two 16x16x32 bf16
    MFMAs), each kind alone and all together with the step's dependencies, on register operands with four waves per
    SIMD and no memory instruction: the floor the attention kernels are priced against (`valu_issue_bound_ms`)."""
    exp_clk, ghz0 = issue_probe(dev, 0)
    cvt_clk, ghz1 = issue_probe(dev, 1)
    mm_clk, ghz2 = issue_probe(dev, 2)
    mix_clk, ghz3 = issue_probe(dev, 3)
    out["issue_port_probe"] = {"v_exp_f32_clocks": round(exp_clk / 16, 2),
                               "v_cvt_pk_bf16_f32_clocks": round(cvt_clk / 8, 2),
                               "six_mfma_of_a_block_clocks": round(mm_clk, 1),
                               "attention_block_mix_clocks": round(mix_clk, 1),
                               "matrix_core_clocks_per_block": 4 * 32 + 2 * 16,
                               "shader_clock_ghz": {"exp": round(ghz0, 3), "cvt": round(ghz1, 3), "mfma": round(ghz2, 3),
                                                    "mix": round(ghz3, 3)}}


def sub_hourglass(dev, out):
    out["hourglass_c5"] = hourglass_c5(dev)
    out["hourglass_c5_ref_shape"] = hourglass_c5(dev, ref_shape=True)


def sub_mfma_rate(dev, out):
    """What the matrix cores of this GPU sustain on dense bf16 products with nothing else running (register operands,
    4 waves per SIMD) and the shader clock they run at meanwhile (in-kernel shader-clock counter against the 100 MHz
    constant-rate counter): with random operands the power budget sets the clock, with a zero operand the data-sheet
    rate is reached.  Then the same question for the step's dominant kernel: the one-kernel gated MLP at the bench
    shape with N(0,1) operands and with all-zero operands (same instruction stream and addresses, nothing toggling in
    the multipliers).  Context for the `frac` figures, which are priced against the data-sheet 2.5 PFLOP/s."""
    import ctypes
    from flash3dtransformer_amd.lib import pshattn
    lib = _bench_probe()
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    wgs, iters = 1024, 100000
    clocks = torch.zeros(wgs, 2, dtype=torch.int64, device=dev)
    flop = wgs * 4 * iters * 8 * 32768.0
    u32, vp = ctypes.c_uint32, ctypes.c_void_p

    def probe(ra, rb):
        rc = lib.bench_probe_mfma_bf16(u32(wgs), u32(iters), u32(ra), u32(rb), vp(sink.data_ptr()),
                                       vp(clocks.data_ptr()), vp(torch.cuda.current_stream(0).cuda_stream))
        if rc != 0:
            raise RuntimeError(f"bench_probe_mfma_bf16 failed with {rc}")
    for name, ra, rb in (("random_operands", 1, 1), ("one_zero_operand", 0, 1)):
        ms = ev_time(lambda: probe(ra, rb), 3, warmup=1)
        ck = clocks.double().cpu()
        ghz = (ck[:, 0] / (ck[:, 1] / 100e6) / 1e9)
        out["mfma_bf16_dense_rate_" + name] = {"ms": round(ms, 3), "tflops": round(flop / ms / 1e9, 1),
                                               "frac_of_bf16_mfma_peak": round(flop / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                                               "shader_clock_ghz_median": round(ghz.median().item(), 3),
                                               "shader_clock_ghz_min": round(ghz.min().item(), 3)}
    M, C, HID = 482_304, 256, 1024
    gg = torch.Generator().manual_seed(1004)
    rnd = lambda *shape, scale=1.0: (torch.randn(*shape, generator=gg) * scale).to(torch.bfloat16).to(dev)
    y = torch.empty(M, C, dtype=torch.bfloat16, device=dev)
    fl = 6.0 * M * C * HID
    for name, zero in (("random_operands", False), ("zero_operands", True)):
        x = torch.zeros(M, C, dtype=torch.bfloat16, device=dev) if zero else rnd(M, C)
        w1 = torch.zeros(2 * HID, C, dtype=torch.bfloat16, device=dev) if zero else rnd(2 * HID, C, scale=1 / 16)
        w2 = torch.zeros(C, HID, dtype=torch.bfloat16, device=dev) if zero else rnd(C, HID, scale=1 / 32)
        b1 = torch.zeros(2 * HID, dtype=torch.bfloat16, device=dev) if zero else rnd(2 * HID)
        b2 = torch.zeros(C, dtype=torch.bfloat16, device=dev) if zero else rnd(C)
        g = torch.zeros(C, dtype=torch.bfloat16, device=dev) if zero else torch.ones(C, dtype=torch.bfloat16, device=dev)
        ms = ev_time(lambda: pshattn.ln_mlp_swiglu_bf16(x, g, b2, 1e-5, w1, b1, w2, b2, x, y), 20)
        out["ln_mlp_swiglu_256x1024_" + name] = {"ms": round(ms, 4), "tflops": round(fl / ms / 1e9, 1),
                                                 "frac_of_bf16_mfma_peak": round(fl / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4)}
        del x, w1, w2


def sub_store_rows(dev, out):
    """the write roof of the row-panel linear layers: their output (482,304 rows x 768 and x 256 bf16) written with
    their own workgroup / chunk / wave geometry and nothing else, in row pieces of 64 and of 128 bytes, back to back and
    with a pause per chunk (40 s_sleep, about the length of a chunk's products)"""
    import ctypes
    lib = _bench_probe()
    u32, vp = ctypes.c_uint32, ctypes.c_void_p
    M = 482_304
    for n in (768, 256):
        y = torch.empty(M, n, dtype=torch.bfloat16, device=dev)
        for piece in (64, 128):
            for pause in (0, 40):
                def run():
                    rc = lib.bench_probe_store_rows(vp(y.data_ptr()), u32(n), u32(M), u32(n), u32(piece), u32(pause),
                                                    vp(torch.cuda.current_stream(0).cuda_stream))
                    if rc != 0:
                        raise RuntimeError(f"bench_probe_store_rows failed with {rc}")
                ms = ev_time(run, 20)
                out[f"store_rows_{M}x{n}_piece{piece}" + ("_paced" if pause else "")] = {
                    "ms": round(ms, 4), "gbs": round(M * n * 2 / ms / 1e6, 1),
                    "frac_of_hbm_peak": round(M * n * 2 / ms / 1e6 / HBM_PEAK_GBS, 4)}
        del y


def sub_backward(dev, out):
    """backward of the dense layers at the headline workload's shapes (480,000 rows, C = 256, hidden 1024): the weight
    gradient GEMMs (2 M N K flops against the MFMA roof, M (N + K) 2 bytes against the HBM roof: the two are close for
    these shapes), LayerNorm and gate backward (one pass each, against the HBM roof), and forward + backward of the
    three dense layers of a block through the layer API"""
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd import layers as L
    M, C, HID = 480_000, 256, 1024
    gg = torch.Generator().manual_seed(1007)
    rnd = lambda *shape: torch.randn(*shape, generator=gg).to(torch.bfloat16).to(dev)
    for name, n, k in (("qkv", 3 * C, C), ("proj", C, C), ("fc1", 2 * HID, C), ("fc2", C, HID)):
        dy, x = rnd(M, n), rnd(M, k)
        dw, db = torch.empty(n, k, device=dev), torch.empty(n, device=dev)
        ms = ev_time(lambda: pshattn.linear_wgrad_bf16(dy, x, dw, db), 10)
        tf, gbs = 2.0 * M * n * k / ms / 1e9, M * (n + k) * 2.0 / ms / 1e6
        out[f"wgrad_{name}_{n}x{k}"] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_of_bf16_mfma_peak": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                                        "gbs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
        del dy, x
    x, dh = rnd(M, C), rnd(M, C)
    g16, dx = torch.ones(C, dtype=torch.bfloat16, device=dev), torch.empty(M, C, dtype=torch.bfloat16, device=dev)
    dg, dbeta = torch.empty(C, device=dev), torch.empty(C, device=dev)
    ms = ev_time(lambda: pshattn.layernorm_bwd_bf16(x, dh, g16, None, dx, dg, dbeta), 10)
    gbs = M * C * 6.0 / ms / 1e6
    out["layernorm_bwd_256"] = {"ms": round(ms, 4), "gbs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
    del x, dh, dx
    # fc1 recomputation + da = dy w2 + gate backward in one kernel: 2 M C 3 H flops, reads h and dy, writes dz and a
    hh, dyy = rnd(M, C), rnd(M, C)
    w1, w2t, b1 = rnd(2 * HID, C) / 16, rnd(HID, C) / 16, rnd(2 * HID)
    dz, aa = torch.empty(M, 2 * HID, dtype=torch.bfloat16, device=dev), torch.empty(M, HID, dtype=torch.bfloat16, device=dev)
    ms = ev_time(lambda: pshattn.mlp_gate_bwd_bf16(hh, dyy, w1, b1, w2t, dz, aa), 10)
    tf, gbs = 6.0 * M * C * HID / ms / 1e9, (2.0 * M * C * 2 + 3.0 * M * HID * 2) / ms / 1e6
    out["mlp_gate_bwd_256x1024"] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_of_bf16_mfma_peak": round(tf / MFMA_BF16_PEAK_TFLOPS, 4),
                                    "gbs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
    del hh, dyy, dz, aa
    z, da = rnd(M, 2 * HID), rnd(M, HID)
    ms = ev_time(lambda: pshattn.swiglu_bwd_bf16(z, da, z, da), 10)
    gbs = M * HID * 12.0 / ms / 1e6
    out["swiglu_bwd_1024"] = {"ms": round(ms, 4), "gbs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
    del z, da
    torch.manual_seed(1007)
    ln = L.LayerNorm(C).to(dev)
    qkv, proj, mlp = L.Linear(C, 3 * C).to(dev), L.Linear(C, C).to(dev), L.LayerNormMLP(C, HID).to(dev)
    for name, f in (("ln_qkv", lambda t: qkv(t, pre_norm=ln)), ("proj_residual", lambda t: proj(t, residual=t)),
                    ("ln_mlp_residual", lambda t: mlp(t, residual=t))):
        xin = rnd(M, C).requires_grad_(True)
        gy = torch.randn_like(f(xin))

        def step():
            f(xin).backward(gy)

        def fwd():
            with torch.no_grad():
                f(xin)
        out[f"layer_fwd_bwd_{name}"] = {"fwd_ms": round(ev_time(fwd, 5), 4), "fwd_bwd_ms": round(ev_time(step, 5), 4)}
        del xin, gy
    del qkv, proj, mlp, ln
    torch.cuda.empty_cache()
    # forward + backward of the whole 5-level hourglass (config 5: 4 sweeps x 250,000 points), training mode, fp32
    # master weights (their bf16 copies are made anew every step), loss = mean of squares; wall time per step
    import bench_workloads as configs
    model = configs.hourglass(1005).to(dev).train()
    coords_np, seps_np, _ = configs.lidar_batch(4, 250_000, 1005)
    coords, seps = configs.to_device(coords_np, seps_np, dev)

    def train_step():
        for p_ in model.parameters():
            p_.grad = None
        (model(coords, None, seps).float() ** 2).mean().backward()
    for _ in range(2):
        train_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        train_step()
    torch.cuda.synchronize()
    out["hourglass_c5_fwd_bwd"] = {"ms": round((time.perf_counter() - t0) / 3 * 1e3, 2), "points": 1_000_000}
    del model, coords, seps
    torch.cuda.empty_cache()


def sub_attention(dev, out):
    from flash3dtransformer_amd.lib import pshattn
    # ---- attention, config 2: L = 131,072, H = 8, D = 32, bucket 512, scope 1 ----
    L, H, D, BS = 131072, 8, 32, 512
    g = torch.Generator().manual_seed(1002)
    qkv = (torch.randn(1, L, 3 * H * D, generator=g) / math.sqrt(32)).to(torch.bfloat16).to(dev)
    q, k, v = [t.view(1, L, H, D) for t in qkv.chunk(3, dim=-1)]
    o = torch.empty(1, L, H, D, dtype=torch.bfloat16, device=dev)
    lse = torch.zeros(1, L, H, dtype=torch.float32, device=dev)
    sc = torch.arange(L // BS, dtype=torch.int32, device=dev).view(-1, 1).view(torch.uint32)
    med, mn, mean = ev_stats(lambda: pshattn.buck_swin_fwd(q, k, v, o, lse, sc, BS))
    fl = 4.0 * L * BS * H * D
    # What the vector issue port allows: per 32 x 32 block of scores a wave issues 16 v_exp_f32, 8 v_cvt_pk_bf16_f32 and
    # 6 MFMAs; bench_probe_issue runs exactly that mix with the step's dependencies on register operands (no LDS, no
    # memory) with four waves per SIMD, and its clocks per block at its own shader clock are the floor, next to the
    # matrix-core and HBM minimum times
    blocks = (L / 32) * (BS / 32) * H
    port_clk, port_ghz = issue_probe(dev, 3)
    out["attention_c2_unmasked"] = {"ms": round(med, 4), "ms_min": round(mn, 4), "ms_mean": round(mean, 4), "launches_timed": 200,
                                    "tflops": round(fl / med / 1e9, 2),
                                    "frac_of_bf16_mfma_peak": round(fl / med / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                                    "algorithmic_gflop": round(fl / 1e9, 2),
                                    "valu_issue_bound_ms": round(blocks * port_clk / 1024 / (port_ghz * 1e9) * 1e3, 4),
                                    "issue_probe_clocks_per_block": round(port_clk, 1),
                                    "issue_probe_shader_clock_ghz": round(port_ghz, 3),
                                    "mfma_bound_ms": round(fl / (MFMA_BF16_PEAK_TFLOPS * 1e12) * 1e3, 4),
                                    "hbm_bound_ms": round((2.0 * L * 4 * H * D + 4.0 * L * H) / (HBM_PEAK_GBS * 1e9) * 1e3, 4)}
    kl = torch.from_numpy(np.random.default_rng(1002).integers(384, 513, L // BS).astype(np.int32)).to(dev)
    med, mn, mean = ev_stats(lambda: pshattn.buck_swin_fwd(q, k, v, o, lse, sc, BS, kl))
    flm = 4.0 * float((kl.double() ** 2).sum()) * H * D
    out["attention_c2_masked"] = {"ms": round(med, 4), "ms_min": round(mn, 4), "ms_mean": round(mean, 4), "launches_timed": 200,
                                  "tflops": round(flm / med / 1e9, 2), "algorithmic_gflop": round(flm / 1e9, 2)}
    # backward on the same shape: five products of 2 T D per (query, head) (dV, dP, dS->dQ, dS->dK, and S once;
    # the kernels recompute S once more, which is not counted)
    d_o = torch.randn(1, L, H, D, generator=g).to(torch.bfloat16).to(dev)
    dq, dk, dv = [torch.zeros(1, L, H, D, dtype=torch.bfloat16, device=dev) for _ in range(3)]
    dlt = torch.zeros(1, L, H, dtype=torch.float32, device=dev)
    pshattn.buck_swin_fwd(q, k, v, o, lse, sc, BS)
    ms = ev_time(lambda: pshattn.buck_swin_bwd(q, k, v, o, d_o, lse, dlt, dq, dk, dv, sc, BS), 30)
    flb = 10.0 * L * BS * H * D
    out["attention_c2_backward"] = {"ms": round(ms, 4), "tflops": round(flb / ms / 1e9, 2),
                                    "frac_of_bf16_mfma_peak": round(flb / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                                    "algorithmic_gflop": round(flb / 1e9, 2)}
    # ---- the reference model's setting: buckets of 512 in scopes of 8 (4096 tokens per scope): the scope kernel with the
    #      key buckets streaming through LDS, then the streaming kernel for the rows it marked (none with these inputs) ----
    sc8 = torch.arange(L // BS, dtype=torch.int32, device=dev).view(-1, 8).view(torch.uint32)
    ms = ev_time(lambda: pshattn.buck_swin_fwd(q, k, v, o, lse, sc8, BS), 10)
    fl8 = 4.0 * L * BS * 8 * H * D
    out["attention_scope8_4096_tokens"] = {"kernel": "buck_swin_fwd_scope_kernel<32,512,16,key buckets streamed> + "
                                                     "buck_swin_fwd_kernel<32,64> on marked rows", "ms": round(ms, 4),
                                           "tflops": round(fl8 / ms / 1e9, 2),
                                           "frac_of_bf16_mfma_peak": round(fl8 / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                                           "algorithmic_gflop": round(fl8 / 1e9, 2)}
    ms = ev_time(lambda: pshattn.buck_swin_bwd(q, k, v, o, d_o, lse, dlt, dq, dk, dv, sc8, BS), 10)
    out["attention_scope8_4096_tokens_backward"] = {
        "kernel": "bwd_delta_kernel<32> + bwd_dkdv_stream_kernel<32> + bwd_dq_stream_kernel<32>", "ms": round(ms, 4),
        "tflops": round(2.5 * fl8 / ms / 1e9, 2),
        "frac_of_bf16_mfma_peak": round(2.5 * fl8 / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
        "algorithmic_gflop": round(2.5 * fl8 / 1e9, 2)}
    del qkv, q, k, v, o, lse, d_o, dq, dk, dv, dlt


def sub_psh(dev, out):
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import psh_main
    # ---- PSH: config 1 (latency bound) and a saturating batch, 30 B/pt three-kernel accounting ----
    for name, n_c, b in (("psh_c1_32768", 32768, 1), ("psh_saturating_64x262144", 262144, 64)):
        gg = torch.Generator().manual_seed(1001)
        coords = (torch.rand(n_c * b, 3, generator=gg) * 51.2).to(torch.float16).to(dev)
        seps = (torch.arange(1, b + 1, dtype=torch.int32) * n_c).to(dev).view(torch.uint32)
        nb, div, mx = psh_main.bucket_geometry(seps, 512)
        buf = psh_main.BucketScatterBuffers.create_buffers(coords, seps, 512, n_c * b, nb)
        bb = torch.stack([coords.min(0)[0], coords.max(0)[0]])

        def run():
            buf.bucket_cntr.zero_()
            pshattn.batch_psh_scatter_pad_hash(coords, buf.bucket_id, buf.bucket_cntr, buf.bucket_offs, seps, mx, nb,
                                               div, 512, 0xFFFF, bb[0], bb[1], buf.probe_offs, buf.bucket_cumsum,
                                               buf.scattered_coord, 0.0, 1)
        ms = ev_time(run, 30)
        byts = 26.0 * n_c * b      # K1: 6 B read + 2 B write; K3: 8 B read + 10 B write
        out[name] = {"ms": round(ms, 4), "gbs_26B_per_pt": round(byts / ms / 1e6, 1),
                     "frac_of_hbm_peak": round(byts / ms / 1e6 / HBM_PEAK_GBS, 4),
                     "mpts_per_s": round(n_c * b / ms / 1e3, 1)}
        del coords, buf


def sub_permute(dev, out):
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import psh_main
    # ---- permutation index + feature scatter and the way back: 4 x 120,000 points, 256 bf16 channels ----
    n_c, b, C = 120000, 4, 256
    gg = torch.Generator().manual_seed(1004)
    coords = (torch.rand(n_c * b, 3, generator=gg) * 51.2).to(torch.float16).to(dev)
    seps = (torch.arange(1, b + 1, dtype=torch.int32) * n_c).to(dev).view(torch.uint32)
    pad_to = -(-n_c * b // 3072) * 3072
    _, buf = psh_main.batch_bucket_scatter(coords, seps, 512, pad_to, 2)
    feat = torch.randn(n_c * b, C, generator=gg).to(torch.bfloat16).to(dev)
    index = torch.empty(pad_to, dtype=torch.uint32, device=dev)
    sfeat = torch.empty(pad_to, C, dtype=torch.bfloat16, device=dev)
    back = torch.empty_like(feat)
    ms_s = ev_time(lambda: pshattn.psh_scatter_feat_index(buf.bucket_id, buf.bucket_cntr, buf.bucket_offs, seps,
                                                          buf.bucket_cumsum, index, feat, sfeat), 30)
    ms_r = ev_time(lambda: pshattn.permute_rows(index, sfeat, back, False), 30)
    s_bytes = n_c * b * (2 + 4 + C * 2) + pad_to * (4 + C * 2)
    r_bytes = pad_to * 4 + 2 * n_c * b * C * 2
    gbs = lambda b_, ms_: round(b_ / ms_ / 1e6, 1)
    out["psh_feat_scatter_4x120k_c256"] = {"ms": round(ms_s, 4), "gbs": gbs(s_bytes, ms_s),
                                           "frac_of_hbm_peak": round(gbs(s_bytes, ms_s) / HBM_PEAK_GBS, 4)}
    out["psh_restore_order_4x120k_c256"] = {"ms": round(ms_r, 4), "gbs": gbs(r_bytes, ms_r),
                                            "frac_of_hbm_peak": round(gbs(r_bytes, ms_r) / HBM_PEAK_GBS, 4)}
    del coords, buf, feat, index, sfeat, back


def sub_pool(dev, out):
    """pooling / unpooling and their backward: config 3 (262,144 points x 128 channels, S = 8: 77 / 144 MB working
    sets, which stay inside the 256 MB Infinity Cache when a kernel is repeated, so these are latencies at the
    configuration's size) and the same kernels on 4,194,304 points (1.2 / 2.3 GB working sets: the bandwidth figures)"""
    _pool_case(dev, out, 262144, "c3", 30)
    _pool_case(dev, out, 4194304, "4m", 10)


def _pool_case(dev, out, n, tag, iters):
    from flash3dtransformer_amd.lib import pshattn
    from flash3dtransformer_amd.psh import subbuck
    C, S = 128, 8
    gg = torch.Generator().manual_seed(1003)
    coords = (torch.rand(n, 3, generator=gg) * 51.2).to(torch.float16).to(dev)
    seps = (torch.arange(1, 5, dtype=torch.int32) * (n // 4)).to(dev).view(torch.uint32)
    feat = torch.randn(n, C, generator=gg).to(torch.bfloat16).to(dev)
    res = torch.randn(n, C, generator=gg).to(torch.bfloat16).to(dev)
    sb = subbuck.SubbuckBuffers.create_subbuck_buff(coords, feat, seps, S)
    L_ = pshattn._load()
    import ctypes
    u32, vp, ci = ctypes.c_uint32, ctypes.c_void_p, ctypes.c_int
    st = vp(torch.cuda.current_stream(0).cuda_stream)

    def build():
        L_.f3d_subbuck_build(vp(coords.data_ptr()), vp(seps.data_ptr()), u32(4), u32(n), u32(n // 4), u32(S),
                             u32(0xFFFF), vp(sb.subbuck_id.data_ptr()), vp(sb.subbuck_off.data_ptr()),
                             vp(sb.reduced_sep.data_ptr()), vp(sb.reduced_coord.data_ptr()),
                             u32(sb.reduced_coord.shape[0]), vp(sb.unpool_ind.data_ptr()),
                             u32(sb.unpool_ind.shape[0]), ci(0), st)

    def reduce(op):
        L_.f3d_reduce_feat(vp(feat.data_ptr()), u32(n), u32(C), vp(sb.unpool_ind.data_ptr()),
                           u32(sb.unpool_ind.shape[0]), u32(S), u32(op), vp(sb.reduced_feat.data_ptr()),
                           u32(sb.reduced_feat.shape[0]), ci(0), st)
    up = torch.empty_like(res)
    ms_b = ev_time(build, iters)
    ms_mean = ev_time(lambda: reduce(0), iters)
    ms_max = ev_time(lambda: reduce(3), iters)
    ms_up = ev_time(lambda: pshattn.additive_unpool_fwd(res, sb.reduced_feat, up, sb.unpool_ind, S), iters)
    r = n // S
    red_bytes = n * C * 2 + r * S * 4 + r * C * 2
    up_bytes = n * C * 2 + r * C * 2 + r * S * 4 + n * C * 2
    bld_bytes = n * 6 + n * 4 + n * 2 + r * S * 4 + r * 6
    gb = lambda b_, ms_: round(b_ / ms_ / 1e6, 1)

    def put(name, ms, byts):
        key = f"{name}_{tag}" if not name.startswith("pool") else name.replace("pool", f"pool_{tag}", 1)
        if byts < 256e6:
            # the working set stays inside the 256 MB Infinity Cache when the launch is repeated: a latency at the
            # configuration's size, not HBM bandwidth
            out[key] = {"ms": round(ms, 4), "gbs_cache_resident": gb(byts, ms), "working_set_mb": round(byts / 1e6, 1)}
        else:
            out[key] = {"ms": round(ms, 4), "gbs": gb(byts, ms), "frac_of_hbm_peak": round(gb(byts, ms) / HBM_PEAK_GBS, 4),
                        "working_set_mb": round(byts / 1e6, 1)}
    put("pool_builder", ms_b, bld_bytes)
    put("pool_reduce_mean", ms_mean, red_bytes)
    put("pool_reduce_max", ms_max, red_bytes)
    put("unpool", ms_up, up_bytes)
    # backward of both (same shapes): reduce bwd reads grad R C 2 (+ input N C 2 for max) and writes N C 2;
    # unpool bwd reads N C 2, writes N C 2 + R C 2
    g_red = torch.randn(sb.reduced_feat.shape[0], C, generator=gg).to(torch.bfloat16).to(dev)
    g_in, g_res, g_down = torch.zeros_like(feat), torch.zeros_like(res), torch.zeros_like(sb.reduced_feat)
    ms_rb = ev_time(lambda: pshattn.batch_subbuck_reduce_backward(g_red, feat, sb.unpool_ind, g_in, S, 0), iters)
    ms_rbm = ev_time(lambda: pshattn.batch_subbuck_reduce_backward(g_red, feat, sb.unpool_ind, g_in, S, 3), iters)
    ms_ub = ev_time(lambda: pshattn.additive_unpool_bwd(g_res, g_down, res, sb.unpool_ind, S), iters)
    rb_bytes, rbm_bytes = r * C * 2 + n * C * 2 + r * S * 4, r * C * 2 + 2 * n * C * 2 + r * S * 4
    ub_bytes = 2 * n * C * 2 + r * C * 2 + r * S * 4
    put("pool_reduce_mean_bwd", ms_rb, rb_bytes)
    put("pool_reduce_max_bwd", ms_rbm, rbm_bytes)
    put("unpool_bwd", ms_ub, ub_bytes)
    del g_red, g_in, g_res, g_down
    del coords, feat, res, up, sb


def hourglass_c5(dev, ref_shape=False):
    """whole-model forward, config 5: 4 sweeps x 250,000 points, 5 levels C = 32/64/128/256/512, heads = C/32,
    bucket 512, scope of 1 bucket, pooling S = 2 (mean), swiglu MLP with hidden = 4C, hash 2.
    `ref_shape`: the shape of the reference's own model test instead (scopes of 8 buckets, two encoder + two decoder
    blocks per level, eval-mode BatchNorm1d + GELU around pooling / unpooling, pooled lengths aligned to bucket x scope).
    `ms`: wall time per forward, forwards queued back to back.  `host_enqueue_ms`: the time the host needs to queue
    one forward (the call returns before the GPU is done): below `ms`, the host runs ahead and per-call marshalling
    is not what the GPU waits for.  `gpu_busy_ms`: the sum of the kernel durations of one forward, from the
    profiler's kernel records (None when the profiler is not usable, e.g. under an outer tracer); `ms` minus it is
    the idle time between consecutive kernels."""
    import bench_workloads as configs
    model = (configs.hourglass_ref_shape(1005) if ref_shape else configs.hourglass(1005)).to(dev).eval()
    cfg = configs.HOURGLASS_REF_SHAPE if ref_shape else configs.HOURGLASS
    coords_np, seps_np, _ = configs.lidar_batch(4, 250_000, 1005)
    coords, seps = configs.to_device(coords_np, seps_np, dev)
    with torch.no_grad():
        for _ in range(2):
            model(coords, None, seps)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        iters = 5
        for _ in range(iters):
            out = model(coords, None, seps)
        torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / iters * 1e3
    with torch.no_grad():
        t0 = time.perf_counter()
        model(coords, None, seps)
        enqueue_ms = (time.perf_counter() - t0) * 1e3
        torch.cuda.synchronize()
    busy, n_kernels = None, None
    if not os.environ.get("ROCPROFILER_REGISTER_FORCE_LOAD") and not os.environ.get("ROCP_TOOL_LIBRARIES"):
        try:
            from torch.profiler import ProfilerActivity, profile
            with torch.no_grad(), profile(activities=[ProfilerActivity.CUDA]) as prof:
                for _ in range(iters):
                    model(coords, None, seps)
                torch.cuda.synchronize()
            ka = prof.key_averages()
            busy = sum(e.self_device_time_total for e in ka) / iters / 1e3
            n_kernels = sum(e.count for e in ka if e.self_device_time_total > 0) // iters      # device kernels only
        except Exception as exc:   # noqa: BLE001 - the timing above stands without it
            print(f"bench.py: kernel records unavailable ({type(exc).__name__}: {exc})", file=sys.stderr)
    return {"ms": round(ms, 3), "host_enqueue_ms": round(enqueue_ms, 3),
            "gpu_busy_ms": None if busy is None else round(busy, 3),
            "launches_per_forward": n_kernels, "mpts_per_s": round(coords.shape[0] / ms / 1e3, 1), "points": int(coords.shape[0]),
            "levels": list(cfg["channels"]), "subbuck_size": cfg["subbuck_size"], "scope_size": cfg["scope_size"],
            "blocks_per_level": "2 + 2" if ref_shape else "1 + 1",
            "finite": bool(torch.isfinite(out.float()).all().item())}


if __name__ == "__main__":
    main()
