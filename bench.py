"""Benchmark of the expert layer: one step = forward + backward of one ArcticMoE layer on
one batch of synthetic tokens (the headline configuration unless --config says otherwise).

    python bench.py --gpus 1 --steps 20 --warmup 5

Prints ONE JSON line: tokens/s over the whole step, the expert-GEMM TFLOP/s and its
fraction of the bf16 MFMA peak, a roofline entry for the dominant kernel (measured with
events on the launch stream), and the CPU oracle timed on a bounded sample of the same
workload as a baseline.
"""
import argparse
import json
import os
import platform
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

# name: dtype, T, H, E, K, I, make_inputs extras
CONFIGS = {
    "c1": ("float32", 2048, 512, 8, 2, 1024, {}),
    "c2": ("bfloat16", 8192, 4096, 8, 2, 14336, {}),
    "c3": ("bfloat16", 16384, 2048, 128, 8, 768, {}),
    "c5": ("bfloat16", 32768, 2048, 64, 4, 1408, dict(bias_hot=1.6, n_hot=4, n_dead=8)),
}
SEEDS = {"c1": 101, "c2": 102, "c3": 103, "c5": 105}


def time_op(fn, iters, torch):
    """average milliseconds of fn() over `iters` launches, events on the current stream"""
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def cpu_baseline(name, sample_tokens, torch):
    """The CPU oracle in reference-rounding mode (every op in the model dtype, per-expert
    matmul loop: what the reference's default path computes on a CPU), forward + backward,
    on the first `sample_tokens` tokens of the workload."""
    from oracle import moe_oracle as O

    dtype_s, T, H, E, K, I, extra = CONFIGS[name]
    dtype = getattr(torch, dtype_s)
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    x, wr, wgu, wd, dy = O.make_inputs(sample_tokens, H, E, K, I, dtype, seed=SEEDS[name], **extra)
    cfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.001)
    t0 = time.perf_counter()
    O.forward_backward(x, wr, wgu, wd, dy, cfg)
    dt = time.perf_counter() - t0
    return {
        "value": sample_tokens / dt,
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"first {sample_tokens} of {T} tokens of {name} ({dtype_s}, H={H} E={E} K={K} I={I}), "
        f"one forward+backward in {dt:.1f} s, torch-CPU on {platform.processor() or platform.machine()}",
        "tflops": 18.0 * sample_tokens * K * H * I / dt / 1e12,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c3", choices=sorted(CONFIGS))
    ap.add_argument("--tile-cfg", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-tokens", type=int, default=0)
    ap.add_argument("--kernel-iters", type=int, default=10)
    ap.add_argument("--only-kernels", action="store_true",
                    help="skip the timed layer steps and the CPU baseline: run each kernel --kernel-iters times "
                         "(for counter collection), preceded by one plain 1 GiB device copy as a traffic yardstick")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the expert layer on ONE GPU; --gpus must be 1 (no multi-GPU path in this build)")
        sys.exit(2)

    import torch
    import torch.nn.functional as F

    from arctictraining_amd import ArcticMoE, MoEConfig, ops
    from oracle import moe_oracle as O

    dtype_s, T, H, E, K, I, extra = CONFIGS[args.config]
    dtype = getattr(torch, dtype_s)
    R = T * K
    dev = torch.device("cuda:0")
    x, wr, wgu, wd, dy = O.make_inputs(T, H, E, K, I, dtype, seed=SEEDS[args.config], **extra)
    cfg = MoEConfig(
        act_fn=F.silu, input_dtype=dtype, intermediate_dim=I, model_dim=H, normalize_topk_scores=True, num_experts=E,
        top_k=K, loss_coeff=0.001,
    )
    layer = ArcticMoE(cfg).to(dev)
    layer.tile_cfg = args.tile_cfg
    with torch.no_grad():
        layer.router_gate.copy_(wr)
        layer.expert_gate_up.copy_(wgu)
        layer.expert_down.copy_(wd)
    xg = x.to(dev).requires_grad_(True)
    dyg = dy.to(dev)
    del x, wr, wgu, wd, dy

    def step():
        xg.grad = None
        for p in layer.parameters():
            p.grad = None
        y = layer(xg)
        y.backward(dyg)

    if args.only_kernels:
        args.warmup, args.steps, args.no_cpu_baseline = 1, 1, True
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)  # the yardstick: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1000.0 / args.steps

    gemm_flop = 18.0 * R * H * I
    peak = PEAK_BF16_TFLOPS if dtype == torch.bfloat16 else PEAK_F32_TFLOPS
    tflops = gemm_flop / (ms_per_step * 1e-3) / 1e12

    # ---- per-kernel timings on the stream the kernels are launched on
    layer.capture = {}
    with torch.no_grad():
        layer(xg.detach())
    cap = layer.capture
    layer.capture = None
    offsets, token_of, row_of, scores = cap["offsets"], cap["token_of"], cap["row_of"], cap["scores"]
    xd = xg.detach()
    slot_of, R_tk = cap["slot_of"], (T, K)
    s_perm = scores.t().reshape(-1)[slot_of.long()].contiguous()
    gu, inter = ops.grouped_gemm_gateup_act_fwd(
        xd, layer.expert_gate_up.detach(), offsets, a_row_map=token_of, n_rows=R, row_scale=s_perm, tile_cfg=args.tile_cfg
    )
    out = ops.grouped_gemm_nn(inter, layer.expert_down.detach(), offsets, tile_cfg=args.tile_cfg)
    d_inter = ops.grouped_gemm_nt(dyg, layer.expert_down.detach(), offsets, a_row_map=token_of, n_rows=R,
                                  tile_cfg=args.tile_cfg)
    d_gu = ops.gated_act_bwd(gu, d_inter)
    d_xp = ops.grouped_gemm_nt(d_gu, layer.expert_gate_up.detach(), offsets, tile_cfg=args.tile_cfg)
    wgu_d, wd_d = layer.expert_gate_up.detach(), layer.expert_down.detach()
    es = 2 if dtype == torch.bfloat16 else 4
    it = args.kernel_iters
    c = args.tile_cfg
    # the kernel symbol (template instance) each launch resolves to: what rocprofv3 reports
    tile = {1: "128, 128, 2, 2", 2: "256, 128, 2, 2", 3: "256, 256, 2, 2", 5: "256, 256, 4, 2"}.get(c, "256, 256, 2, 4")
    sym = {
        "gemm_gateup_act_fwd": f"grouped_gemm_bf16_kernel<{tile}, true, false, 1, 0, 0>",
        "gemm_down_fwd": f"grouped_gemm_bf16_kernel<{tile}, true, false, 0, 0, 0>",
        "gemm_dgrad_down": f"grouped_gemm_bf16_kernel<{tile}, true, true, 0, 0, 0>",
        "gemm_dgrad_gateup": f"grouped_gemm_bf16_kernel<{tile}, true, true, 0, 0, 0>",
        "gemm_wgrad_down": f"grouped_gemm_bf16_kernel<{tile}, false, false, 0, 0, 2>",
        "gemm_wgrad_gateup": f"grouped_gemm_bf16_kernel<{tile}, false, false, 0, 0, 1>",
    }
    if dtype != torch.bfloat16:
        sym = {k: "grouped_gemm_f32_kernel" for k in sym}
    # (name, callable, flops per launch, algorithmic bytes per launch)
    kernels = [
        ("gemm_gateup_act_fwd", lambda: ops.grouped_gemm_gateup_act_fwd(xd, wgu_d, offsets, a_row_map=token_of, n_rows=R,
                                                                        row_scale=s_perm, tile_cfg=c), 4.0 * R * H * I,
         (T * H + E * H * 2 * I + 3 * R * I) * es),
        ("gemm_down_fwd", lambda: ops.grouped_gemm_nn(inter, wd_d, offsets, tile_cfg=c), 2.0 * R * H * I,
         (R * I + E * I * H + R * H) * es),
        ("gemm_dgrad_down", lambda: ops.grouped_gemm_nt(dyg, wd_d, offsets, a_row_map=token_of, n_rows=R, tile_cfg=c),
         2.0 * R * H * I,
         (T * H + E * I * H + R * I) * es),
        ("gemm_wgrad_down", lambda: ops.grouped_gemm_wgrad(inter, dyg, offsets, E, tile_cfg=c, b_row_map=token_of),
         2.0 * R * H * I,
         (R * I + T * H + E * I * H) * es),
        ("gemm_dgrad_gateup", lambda: ops.grouped_gemm_nt(d_gu, wgu_d, offsets, tile_cfg=c), 4.0 * R * H * I,
         (2 * R * I + E * H * 2 * I + R * H) * es),
        ("gemm_wgrad_gateup", lambda: ops.grouped_gemm_wgrad(xd, d_gu, offsets, E, tile_cfg=c, a_row_map=token_of),
         4.0 * R * H * I,
         (T * H + 2 * R * I + E * H * 2 * I) * es),
        ("combine_fwd", lambda: ops.combine_fwd(out, row_of, None), 0.0, (R + T) * H * es + R * 4),
        ("gated_act_bwd", lambda: ops.gated_act_bwd(gu, d_inter, row_scale=s_perm, slot_of=slot_of, tk=R_tk), 0.0,
         5 * R * I * es + 12 * R),
        ("gather_rows_bwd", lambda: ops.gather_rows_bwd(d_xp, row_of, None), 0.0, (R + T) * H * es),
        ("router_topk_fwd", lambda: ops.router_topk_fwd(cap["logits"], K, True), 0.0, T * E * (es + 4) + T * K * 8),
        ("permute_plan", lambda: ops.permute_plan(cap["topk_idx"], E, scores), 0.0, R * 4 * 7),
    ]
    if dtype == torch.bfloat16 and H % 8 == 0 and I % 8 == 0:
        # checkpoint format -> expert_gate_up (not part of a step; timed as a data-format kernel)
        fused = wgu_d.view(E, 2 * I, H)  # any bits of the right size: [E, 2I, H] gate rows, then up rows
        kernels.append(("remap_pack_gate_up", lambda: ops.remap_pack(fused[:, :I, :], fused[:, I:, :]), 0.0,
                        2 * E * H * 2 * I * es))
    breakdown = []
    for name, fn, flops, nbytes in kernels:
        ms = time_op(fn, it, torch)
        entry = {"kernel": name, "ms": round(ms, 4)}
        if flops:
            entry["tflops"] = round(flops / (ms * 1e-3) / 1e12, 1)
            entry["frac_mfma_peak"] = round(flops / (ms * 1e-3) / 1e12 / peak, 4)
        else:
            entry["gbs"] = round(nbytes / (ms * 1e-3) / 1e9, 1)
            entry["frac_hbm_peak"] = round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
        entry["_flops"], entry["_bytes"] = flops, nbytes
        breakdown.append(entry)
    # Roofline of the dominant kernel SYMBOL: the template instance with the largest total time
    # per step.  The two weight-gradient GEMMs (and the two data-gradient GEMMs) share one
    # instance, so its figures are launch averages: mean flops per launch / mean duration.
    groups = {}
    for e in breakdown:
        key = sym.get(e["kernel"], e["kernel"])
        e["symbol"] = key
        if e["kernel"].startswith("remap_"):
            continue  # a load-time data-format kernel, not part of a step
        g = groups.setdefault(key, {"ms": 0.0, "flops": 0.0, "bytes": 0.0, "n": 0, "members": []})
        g["ms"] += e["ms"]
        g["flops"] += e["_flops"]
        g["bytes"] += e["_bytes"]
        g["n"] += 1
        g["members"].append(e["kernel"])
    dom_key = max(groups, key=lambda k: groups[k]["ms"])
    dg = groups[dom_key]
    avg_ms = dg["ms"] / dg["n"]
    traffic = None
    tpath = os.path.join(ROOT, "profiles", f"traffic_{args.config}.json")
    if os.path.exists(tpath):
        with open(tpath) as fh:
            traffic = json.load(fh).get(dom_key)
    if dg["flops"]:
        ach = dg["flops"] / dg["n"] / (avg_ms * 1e-3) / 1e12
        roofline = {
            "kernel": dom_key, "launches_per_step": dg["members"], "bound": "mfma", "achieved": round(ach, 1),
            "peak": peak, "unit": "TFLOP/s", "frac": round(ach / peak, 4), "traffic": traffic,
            "avg_ms": round(avg_ms, 4), "flops_per_launch": dg["flops"] / dg["n"],
            "algorithmic_bytes_per_launch": dg["bytes"] / dg["n"],
        }
    else:
        ach = dg["bytes"] / dg["n"] / (avg_ms * 1e-3) / 1e9
        roofline = {
            "kernel": dom_key, "launches_per_step": dg["members"], "bound": "hbm", "achieved": round(ach, 1),
            "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": traffic,
            "avg_ms": round(avg_ms, 4), "bytes_per_launch": dg["bytes"] / dg["n"],
        }
    gemm_ms = sum(e["ms"] for e in breakdown if e["_flops"])
    for e in breakdown:
        e.pop("_flops"), e.pop("_bytes")

    result = {
        "metric": "moe_layer_fwd_bwd_tokens_per_s",
        "value": T / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if dtype == torch.bfloat16 else "f32",
        "data": "synthetic",
        "config": {
            "workload": f"{args.config}: one MoE layer fwd+bwd, T={T} H={H} E={E} top_k={K} I={I}, seed {SEEDS[args.config]}",
            "tokens": T, "hidden": H, "experts": E, "top_k": K, "intermediate": I, "tile_cfg": args.tile_cfg,
        },
        "tflops": tflops,
        "frac_mfma_peak": tflops / peak,
        "grouped_gemm_tflops": gemm_flop / (gemm_ms * 1e-3) / 1e12,
        "grouped_gemm_frac_mfma_peak": gemm_flop / (gemm_ms * 1e-3) / 1e12 / peak,
        "roofline": roofline,
        "kernels": breakdown,
    }
    if not args.no_cpu_baseline:
        sample = args.cpu_sample_tokens or max(T // 16, 256)
        result["cpu_baseline"] = cpu_baseline(args.config, min(sample, T), torch)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
