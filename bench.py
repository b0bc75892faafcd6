"""Benchmark of the expert layer: one step = forward + backward of one ArcticMoE layer on
one batch of synthetic tokens (the headline configuration unless --config says otherwise).

    python bench.py --gpus 1 --steps 20 --warmup 5 [--config c1|c2|c3|c4|c5]

Prints ONE JSON line: tokens/s over the whole step, the expert-GEMM TFLOP/s and its
fraction of the bf16 MFMA peak, a roofline entry for the dominant kernel (measured with
events on the launch stream), the library GEMM (torch.matmul) timed on the dense
equivalents of that kernel's launches as a same-box yardstick, and the CPU oracle timed on
a bounded sample of the same workload as a baseline.

c4 is one expert-parallel rank's share of a DeepSeek-V3-like layer: 65536 routed rows that
arrive already assigned to 32 local experts (Zipf(1.2) loads), so there is no router; its
step is the grouped expert FFN forward + backward (six grouped GEMMs, the gated activation
backward being the epilogue of one of them) and its throughput is counted in routed rows.
"""
import argparse
import json
import os
import platform
import statistics
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

# name: dtype, T, H, E, K, I, input extras.  c4: T = routed rows, K = 1, no router.
CONFIGS = {
    "c1": ("float32", 2048, 512, 8, 2, 1024, {}),
    "c2": ("bfloat16", 8192, 4096, 8, 2, 14336, {}),
    "c3": ("bfloat16", 16384, 2048, 128, 8, 768, {}),
    "c4": ("bfloat16", 65536, 7168, 32, 1, 2048, dict(zipf=1.2)),
    "c5": ("bfloat16", 32768, 2048, 64, 4, 1408, dict(bias_hot=1.6, n_hot=4, n_dead=8)),
}
SEEDS = {"c1": 101, "c2": 102, "c3": 103, "c4": 104, "c5": 105}


def make_inputs(torch, T, H, E, I, dtype, seed, bias_hot=None, n_hot=0, n_dead=0):
    """Seeded inputs, generated on the CPU in float32 and then cast: x, dy ~ N(0,1), every
    weight ~ N(0, 0.02).  n_hot / n_dead bias the router through a constant input channel so
    that the first n_hot experts take about half of the assignments and the last n_dead none."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g)
    wr = torch.randn(E, H, generator=g) * 0.02
    wgu = torch.randn(E, H, 2 * I, generator=g) * 0.02
    wd = torch.randn(E, I, H, generator=g) * 0.02
    dy = torch.randn(T, H, generator=g)
    if n_hot or n_dead:
        x[:, H - 1] = 1.0
        wr[:, H - 1] = 0.0
        if n_hot:
            wr[:n_hot, H - 1] = float(bias_hot)
        if n_dead:
            wr[E - n_dead:, H - 1] = -1.0e4
    return tuple(t.to(dtype) for t in (x, wr, wgu, wd, dy))


def zipf_counts(R, E, s, seed):
    import numpy as np

    rng = np.random.Generator(np.random.PCG64(seed))
    p = np.arange(1, E + 1, dtype=np.float64) ** -s
    return rng.multinomial(R, p / p.sum())


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


def _git(*args):
    try:
        r = subprocess.run(["git", "-C", ROOT, *args], capture_output=True, text=True, timeout=10)
        return r.stdout.strip() if r.returncode == 0 else ""
    except Exception:
        return ""


def _stamp():
    """The two lines the library build left beside the library: tree commit, kernel commit."""
    try:
        with open(os.path.join(ROOT, "arctictraining_amd", "lib", "build_commit.txt")) as fh:
            lines = fh.read().split("\n")
    except OSError:
        return None, None
    head = lines[0].strip() or None
    kern = next((l.split()[1] for l in lines[1:] if l.startswith("kernels ") and len(l.split()) > 1), None)
    return head, kern


def git_head():
    """The commit of the running tree: from git when the history is here, otherwise the stamp that
    the library build left beside the library it built."""
    return _git("rev-parse", "--short=12", "HEAD") or _stamp()[0]


def kernel_commit():
    """The last commit that changed a file under arctictraining_amd/csrc (the kernels): what a
    profile of a kernel is a profile of.  From the library's build stamp (the library is what runs);
    from git only when there is no stamp."""
    return _stamp()[1] or _git("log", "-1", "--format=%h", "--abbrev=12", "--", "arctictraining_amd/csrc") or None


def cpu_baseline(name, sample_tokens, torch):
    """The CPU oracle in reference-rounding mode (every op in the model dtype, per-expert
    matmul loop: what the reference's default path computes on a CPU), forward + backward,
    on the first `sample_tokens` tokens of the workload (c4: the first rows of every expert,
    in the same proportions).  c1 is small enough for the median of five runs."""
    from oracle import moe_oracle as O

    dtype_s, T, H, E, K, I, extra = CONFIGS[name]
    dtype = getattr(torch, dtype_s)
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    reps = 5 if name == "c1" else 1
    times = []
    if name == "c4":
        counts = zipf_counts(T, E, extra["zipf"], SEEDS[name]) * sample_tokens // T
        R = int(counts.sum())
        g = torch.Generator().manual_seed(SEEDS[name])
        xp = torch.randn(R, H, generator=g).to(dtype).requires_grad_(True)
        wgu = (torch.randn(E, H, 2 * I, generator=g) * 0.02).to(dtype).requires_grad_(True)
        wd = (torch.randn(E, I, H, generator=g) * 0.02).to(dtype).requires_grad_(True)
        d_out = torch.randn(R, H, generator=g).to(dtype)
        cs = torch.from_numpy(counts).cumsum(0)
        for _ in range(reps):
            t0 = time.perf_counter()
            _, _, out = O.expert_ffn(xp, wgu, wd, cs, "silu")
            out.backward(d_out)
            times.append(time.perf_counter() - t0)
        rows = R
    else:
        x, wr, wgu, wd, dy = O.make_inputs(sample_tokens, H, E, K, I, dtype, seed=SEEDS[name],
                                           **{k: v for k, v in extra.items() if k != "zipf"})
        cfg = O.OracleConfig(model_dim=H, intermediate_dim=I, num_experts=E, top_k=K, loss_coeff=0.001)
        for _ in range(reps):
            t0 = time.perf_counter()
            O.forward_backward(x, wr, wgu, wd, dy, cfg)
            times.append(time.perf_counter() - t0)
        rows = sample_tokens
    dt = statistics.median(times)
    return {
        "value": rows / dt,
        "unit": "routed rows/s" if name == "c4" else "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"first {rows} of {T} {'routed rows' if name == 'c4' else 'tokens'} of {name} ({dtype_s}, H={H} E={E} "
        f"K={K} I={I}), forward+backward, {'median of 5 runs' if reps > 1 else 'one run'}: {dt:.2f} s, torch-CPU on "
        f"{platform.processor() or platform.machine()}",
        "tflops": 18.0 * rows * K * H * I / dt / 1e12,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c3", choices=sorted(CONFIGS))
    ap.add_argument("--tile-cfg", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--serial-weight-grads", action="store_true",
                    help="run the expert weight gradients on the main stream (the layer's default is a second stream)")
    ap.add_argument("--cpu-sample-tokens", type=int, default=0)
    ap.add_argument("--kernel-iters", type=int, default=10)
    ap.add_argument("--no-unragged", action="store_true",
                    help="skip the yardstick's run of the dominant kernel on the un-ragged problem (a kernel trace "
                         "averages per kernel symbol: this keeps its launches to the real problem)")
    ap.add_argument("--only-kernels", action="store_true",
                    help="skip the timed layer steps and the CPU baseline: run each kernel (and the library GEMM of the "
                         "yardstick) --kernel-iters times untimed, for counter collection, preceded by one plain 1 GiB "
                         "device copy as a traffic yardstick")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the expert layer on ONE GPU; --gpus must be 1 (no multi-GPU path in this build)")
        sys.exit(2)

    import torch
    import torch.nn.functional as F

    from arctictraining_amd import ArcticMoE, MoEConfig, ops

    name = args.config
    dtype_s, T, H, E, K, I, extra = CONFIGS[name]
    dtype = getattr(torch, dtype_s)
    R = T * K
    dev = torch.device("cuda:0")
    es = 2 if dtype == torch.bfloat16 else 4
    c = args.tile_cfg
    it = args.kernel_iters

    if args.only_kernels:
        args.warmup, args.steps, args.no_cpu_baseline = 1, 1, True
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)  # the yardstick of the byte counters: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # ------------------------------------------------------------------ the workload and its step
    if name == "c4":
        counts = zipf_counts(R, E, extra["zipf"], SEEDS[name])
        offsets = torch.from_numpy(counts).cumsum(0)
        offsets = torch.cat([torch.zeros(1, dtype=torch.int64), offsets]).to(torch.int32).to(dev)
        g = torch.Generator().manual_seed(SEEDS[name])
        xd = torch.randn(R, H, generator=g).to(dtype).to(dev)          # rows already grouped by expert
        dyg = torch.randn(R, H, generator=g).to(dtype).to(dev)         # upstream gradient of the rows
        s_perm = torch.rand(R, generator=g).to(dev)
        wgu_d = torch.empty(E, H, 2 * I, dtype=dtype, device=dev)
        wd_d = torch.empty(E, I, H, dtype=dtype, device=dev)
        for e in range(E):  # expert by expert: no float32 copy of the whole weight on the host
            wgu_d[e] = (torch.randn(H, 2 * I, generator=g) * 0.02).to(dtype)
            wd_d[e] = (torch.randn(I, H, generator=g) * 0.02).to(dtype)
        token_of = row_of = slot_of = None

        def step():
            ws = ops.gemm_workspace(R, E, dev)
            gu_, in_ = ops.grouped_gemm_gateup_act_fwd(xd, wgu_d, offsets, row_scale=s_perm, tile_cfg=c, workspace=ws)
            ops.grouped_gemm_nn(in_, wd_d, offsets, tile_cfg=c, workspace=ws, map_ready=True)
            if c in (0, 1, 2):
                dg_, _ = ops.grouped_gemm_nt_gated_bwd(dyg, wd_d, offsets, gu_, row_scale=s_perm, tile_cfg=c, workspace=ws,
                                                       map_ready=True)
            else:
                di_ = ops.grouped_gemm_nt(dyg, wd_d, offsets, tile_cfg=c, workspace=ws, map_ready=True)
                dg_ = ops.gated_act_bwd(gu_, di_, row_scale=s_perm)
            ops.grouped_gemm_wgrad(in_, dyg, offsets, E, tile_cfg=c)
            ops.grouped_gemm_wgrad(xd, dg_, offsets, E, tile_cfg=c)
            ops.grouped_gemm_nt(dg_, wgu_d, offsets, tile_cfg=c, workspace=ws, map_ready=True)

        workload = (f"c4: grouped expert FFN fwd+bwd on {R} routed rows pre-assigned to {E} local experts "
                    f"(Zipf(1.2) loads, largest {int(counts.max())}, smallest {int(counts.min())}), H={H} I={I}, seed {SEEDS[name]}")
    else:
        x, wr, wgu, wd, dy = make_inputs(torch, T, H, E, I, dtype, SEEDS[name], **extra)
        cfg = MoEConfig(
            act_fn=F.silu, input_dtype=dtype, intermediate_dim=I, model_dim=H, normalize_topk_scores=True, num_experts=E,
            top_k=K, loss_coeff=0.001,
        )
        layer = ArcticMoE(cfg).to(dev)
        layer.tile_cfg = c
        layer.overlap_weight_grads = not args.serial_weight_grads
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

        workload = f"{name}: one MoE layer fwd+bwd, T={T} H={H} E={E} top_k={K} I={I}, seed {SEEDS[name]}"

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

    # ------------------------------------------------------------------ per-kernel timings on the launch stream
    cap = {}
    if name != "c4":
        layer.capture = cap
        step()
        torch.cuda.synchronize()
        layer.capture = None
        offsets, token_of, row_of, scores, slot_of = (cap[k] for k in ("offsets", "token_of", "row_of", "scores", "slot_of"))
        xd = xg.detach()
        s_perm = scores.t().reshape(-1)[slot_of.long()].contiguous()
        wgu_d, wd_d = layer.expert_gate_up.detach(), layer.expert_down.detach()
    A_T = xd.shape[0]  # rows of the un-gathered activations (T, or R when the rows arrive grouped)
    gu, inter = ops.grouped_gemm_gateup_act_fwd(xd, wgu_d, offsets, a_row_map=token_of, n_rows=R, row_scale=s_perm, tile_cfg=c)
    out = ops.grouped_gemm_nn(inter, wd_d, offsets, tile_cfg=c)
    d_inter = ops.grouped_gemm_nt(dyg, wd_d, offsets, a_row_map=token_of, n_rows=R, tile_cfg=c)
    d_gu = ops.gated_act_bwd(gu, d_inter)
    d_xp = ops.grouped_gemm_nt(d_gu, wgu_d, offsets, tile_cfg=c)
    fused_bwd = dtype == torch.bfloat16 and c in (0, 1, 2)   # what the layer's backward does
    # the kernel symbol (template instance) each launch resolves to: what rocprofv3 reports
    tile = {1: "128, 128, 2, 2", 2: "256, 128, 2, 2", 3: "256, 256, 2, 2", 5: "256, 256, 4, 2"}.get(c, "256, 256, 2, 4")
    gathered = token_of is not None
    sym = {
        # grouped_gemm_rows_bf16_kernel<BM, BN, waves along M, waves along N, B K-contiguous, epilogue, activation>
        "gemm_gateup_act_fwd": f"grouped_gemm_rows_bf16_kernel<{tile}, false, 1, 0>",
        "gemm_down_fwd": f"grouped_gemm_rows_bf16_kernel<{tile}, false, 0, 0>",
        "gemm_dgrad_down": f"grouped_gemm_rows_bf16_kernel<{tile}, true, 0, 0>",
        "gemm_dgrad_down_gated_bwd": f"grouped_gemm_rows_bf16_kernel<{tile}, true, 2, 0>",
        "gemm_dgrad_gateup": f"grouped_gemm_rows_bf16_kernel<{tile}, true, 0, 0>",
        # grouped_gemm_wgrad_bf16_kernel<BM, BN, waves along M, waves along N, gathered operand>
        "gemm_wgrad_down": f"grouped_gemm_wgrad_bf16_kernel<{tile}, {2 if gathered else 0}>",
        "gemm_wgrad_gateup": f"grouped_gemm_wgrad_bf16_kernel<{tile}, {1 if gathered else 0}>",
    }
    if dtype != torch.bfloat16:
        sym = {k: "grouped_gemm_f32_kernel" for k in sym}
    # dense equivalents (M, K, N, layout) of the grouped launches, for the library yardstick
    dense = {
        "gemm_gateup_act_fwd": (R, H, 2 * I, "nn"), "gemm_down_fwd": (R, I, H, "nn"),
        "gemm_dgrad_down": (R, H, I, "nt"), "gemm_dgrad_down_gated_bwd": (R, H, I, "nt"),
        "gemm_dgrad_gateup": (R, 2 * I, H, "nt"),
        "gemm_wgrad_down": (I, R, H, "tn"), "gemm_wgrad_gateup": (H, R, 2 * I, "tn"),
    }
    # (name, callable, flops per launch, algorithmic bytes per launch)
    kernels = [
        ("gemm_gateup_act_fwd", lambda: ops.grouped_gemm_gateup_act_fwd(xd, wgu_d, offsets, a_row_map=token_of, n_rows=R,
                                                                        row_scale=s_perm, tile_cfg=c), 4.0 * R * H * I,
         (A_T * H + E * H * 2 * I + 3 * R * I) * es),
        ("gemm_down_fwd", lambda: ops.grouped_gemm_nn(inter, wd_d, offsets, tile_cfg=c), 2.0 * R * H * I,
         (R * I + E * I * H + R * H) * es),
        # bf16: the data gradient of the down projection carries the gated-activation backward as its
        # epilogue (reads gate_up, writes d_gate_up and the score-gradient partials; d_inter is never stored)
        ("gemm_dgrad_down_gated_bwd", lambda: ops.grouped_gemm_nt_gated_bwd(dyg, wd_d, offsets, gu, row_scale=s_perm,
                                                                            a_row_map=token_of, n_rows=R, tile_cfg=c),
         2.0 * R * H * I, (A_T * H + E * I * H + 4 * R * I) * es + 4 * R * ((I + 255) // 256))
        if fused_bwd else
        ("gemm_dgrad_down", lambda: ops.grouped_gemm_nt(dyg, wd_d, offsets, a_row_map=token_of, n_rows=R, tile_cfg=c),
         2.0 * R * H * I, (A_T * H + E * I * H + R * I) * es),
        ("gemm_wgrad_down", lambda: ops.grouped_gemm_wgrad(inter, dyg, offsets, E, tile_cfg=c, b_row_map=token_of),
         2.0 * R * H * I, (R * I + A_T * H + E * I * H) * es),
        ("gemm_dgrad_gateup", lambda: ops.grouped_gemm_nt(d_gu, wgu_d, offsets, tile_cfg=c), 4.0 * R * H * I,
         (2 * R * I + E * H * 2 * I + R * H) * es),
        ("gemm_wgrad_gateup", lambda: ops.grouped_gemm_wgrad(xd, d_gu, offsets, E, tile_cfg=c, a_row_map=token_of),
         4.0 * R * H * I, (A_T * H + 2 * R * I + E * H * 2 * I) * es),
    ]
    if not fused_bwd:
        kernels.append(("gated_act_bwd", lambda: ops.gated_act_bwd(gu, d_inter, row_scale=s_perm), 0.0, 5 * R * I * es + 4 * R))
    if name != "c4":
        probs, topk_idx, counts_d = cap["probs"], cap["topk_idx"], cap["counts"]
        d_scores = cap["d_scores"]
        if fused_bwd:
            parts = ops.grouped_gemm_nt_gated_bwd(dyg, wd_d, offsets, gu, row_scale=s_perm, a_row_map=token_of, n_rows=R,
                                                  tile_cfg=c)[1]
            kernels.append(("score_grad_gather", lambda: ops.score_grad_gather(parts, row_of), 0.0,
                            (parts.shape[0] + 2) * R * 4))
        else:
            kernels[-1] = ("gated_act_bwd", lambda: ops.gated_act_bwd(gu, d_inter, row_scale=s_perm, slot_of=slot_of, tk=(T, K)),
                           0.0, 5 * R * I * es + 12 * R)
        kernels += [
            ("combine_fwd", lambda: ops.combine_fwd(out, row_of, None), 0.0, (R + T) * H * es + R * 4),
            ("gather_rows_bwd", lambda: ops.gather_rows_bwd(d_xp, row_of, None), 0.0, (R + T) * H * es),
            ("router_topk_fwd", lambda: ops.router_topk_fwd(cap["logits"], K, True), 0.0, T * E * (es + 4) + T * K * 8),
            ("permute_plan", lambda: ops.permute_plan(topk_idx, E, scores), 0.0, R * 4 * 7),
            ("router_bwd", lambda: ops.router_bwd(d_scores, probs, topk_idx, counts_d, dtype, True, 0.001 / T), 0.0,
             T * E * (4 + es) + T * K * 8),
        ]
        if dtype == torch.bfloat16 and H % 8 == 0 and I % 8 == 0:
            # checkpoint format -> expert_gate_up (not part of a step; timed as a data-format kernel)
            fused = wgu_d.view(E, 2 * I, H)  # any bits of the right size: [E, 2I, H] gate rows, then up rows
            kernels.append(("remap_pack_gate_up", lambda: ops.remap_pack(fused[:, :I, :], fused[:, I:, :]), 0.0,
                            2 * E * H * 2 * I * es))
    breakdown = []
    for kname, fn, flops, nbytes in kernels:
        ms = time_op(fn, it, torch)
        entry = {"kernel": kname, "ms": round(ms, 4)}
        if flops:
            entry["tflops"] = round(flops / (ms * 1e-3) / 1e12, 1)
            entry["frac_mfma_peak"] = round(flops / (ms * 1e-3) / 1e12 / peak, 4)
        else:
            entry["gbs"] = round(nbytes / (ms * 1e-3) / 1e9, 1)
            entry["frac_hbm_peak"] = round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
        entry["_flops"], entry["_bytes"] = flops, nbytes
        breakdown.append(entry)
    # Roofline of the dominant kernel SYMBOL: the template instance with the largest total time
    # per step.  The two data-gradient GEMMs share one instance (as do the weight-gradient GEMMs
    # when no operand is gathered), so its figures are launch averages.
    groups = {}
    for e_ in breakdown:
        key = sym.get(e_["kernel"], e_["kernel"])
        e_["symbol"] = key
        if e_["kernel"].startswith("remap_"):
            continue  # a load-time data-format kernel, not part of a step
        g_ = groups.setdefault(key, {"ms": 0.0, "flops": 0.0, "bytes": 0.0, "n": 0, "members": []})
        g_["ms"] += e_["ms"]
        g_["flops"] += e_["_flops"]
        g_["bytes"] += e_["_bytes"]
        g_["n"] += 1
        g_["members"].append(e_["kernel"])
    dom_key = max(groups, key=lambda k: groups[k]["ms"])
    dg = groups[dom_key]
    avg_ms = dg["ms"] / dg["n"]
    traffic = traffic_commit = None
    tpath = os.path.join(ROOT, "profiles", f"traffic_{name}.json")
    if os.path.exists(tpath):
        with open(tpath) as fh:
            tj = json.load(fh)
        traffic, traffic_commit = tj.get("kernels", tj).get(dom_key), tj.get("commit")
    if dg["flops"]:
        ach = dg["flops"] / dg["n"] / (avg_ms * 1e-3) / 1e12
        roofline = {
            "kernel": dom_key, "launches_per_step": dg["members"], "bound": "mfma", "achieved": round(ach, 1),
            "peak": peak, "unit": "TFLOP/s", "frac": round(ach / peak, 4), "traffic": traffic,
            "traffic_measured_at_commit": traffic_commit,
            "traffic_is_of_these_kernels": traffic_commit is not None and traffic_commit == kernel_commit(),
            "avg_ms": round(avg_ms, 4), "flops_per_launch": dg["flops"] / dg["n"],
            "algorithmic_bytes_per_launch": dg["bytes"] / dg["n"],
        }
    else:
        ach = dg["bytes"] / dg["n"] / (avg_ms * 1e-3) / 1e9
        roofline = {
            "kernel": dom_key, "launches_per_step": dg["members"], "bound": "hbm", "achieved": round(ach, 1),
            "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(ach / PEAK_HBM_GBS, 4), "traffic": traffic,
            "traffic_measured_at_commit": traffic_commit,
            "traffic_is_of_these_kernels": traffic_commit is not None and traffic_commit == kernel_commit(),
            "avg_ms": round(avg_ms, 4), "bytes_per_launch": dg["bytes"] / dg["n"],
        }
    gemm_ms = sum(e_["ms"] for e_ in breakdown if e_["_flops"])
    for e_ in breakdown:
        e_.pop("_flops"), e_.pop("_bytes")

    # ------------------------------------------------------------------ same-box yardsticks
    # (1) the library GEMM (torch.matmul -> hipBLASLt) on the dense equivalents of the dominant
    # kernel's launches; (2) the dominant kernel itself on the un-ragged equivalent of its problem:
    # every expert the same number of rows, no gather.  (2) / (1) is what the tile loop and its
    # epilogue cost against the library, kernel / (2) what ragged expert loads and the gather cost.
    # With --only-kernels (1) runs --kernel-iters times untimed, so that a counter pass sees the library's kernel too.
    yardstick = None
    if dg["flops"] and dtype == torch.bfloat16:
        del gu, inter, out, d_inter, d_gu, d_xp
        torch.cuda.empty_cache()
        run = (lambda fn: [fn() for _ in range(it)] and 0.0) if args.only_kernels else (lambda fn: time_op(fn, it, torch))
        y_ms = y_flops = u_ms = 0.0
        shapes = []
        per = R // E
        offs_u = torch.arange(E + 1, dtype=torch.int64) * per
        offs_u[E] = R
        offs_u = offs_u.to(torch.int32).to(dev)
        rnd = lambda *shape: torch.randn(shape, device=dev, dtype=dtype)
        for m_ in dg["members"]:
            M_, K_, N_, lay = dense[m_]
            a_ = rnd(K_, M_) if lay == "tn" else rnd(M_, K_)
            b_ = (rnd(N_, K_) if lay == "nt" else rnd(K_, N_)) * 0.02
            fn = {"nn": lambda: torch.matmul(a_, b_), "nt": lambda: torch.matmul(a_, b_.t()),
                  "tn": lambda: torch.matmul(a_.t(), b_)}[lay]
            y_ms += run(fn)
            y_flops += 2.0 * M_ * K_ * N_
            shapes.append(f"{lay} {M_}x{K_}x{N_}")
            del a_, b_
            ufn = {
                "gemm_gateup_act_fwd": lambda a: ops.grouped_gemm_gateup_act_fwd(a[0], wgu_d, offs_u, row_scale=s_perm, tile_cfg=c),
                "gemm_down_fwd": lambda a: ops.grouped_gemm_nn(a[1], wd_d, offs_u, tile_cfg=c),
                "gemm_dgrad_down": lambda a: ops.grouped_gemm_nt(a[0], wd_d, offs_u, tile_cfg=c),
                "gemm_dgrad_down_gated_bwd": lambda a: ops.grouped_gemm_nt_gated_bwd(a[0], wd_d, offs_u, a[2], row_scale=s_perm,
                                                                                      tile_cfg=c),
                "gemm_dgrad_gateup": lambda a: ops.grouped_gemm_nt(a[2], wgu_d, offs_u, tile_cfg=c),
                "gemm_wgrad_down": lambda a: ops.grouped_gemm_wgrad(a[1], a[0], offs_u, E, tile_cfg=c),
                "gemm_wgrad_gateup": lambda a: ops.grouped_gemm_wgrad(a[0], a[2], offs_u, E, tile_cfg=c),
            }[m_]
            if not (args.only_kernels or args.no_unragged):  # (a profile averages per kernel symbol)
                bufs = (rnd(R, H), rnd(R, I), rnd(R, 2 * I))   # rows of width H, I and 2I
                u_ms += run(lambda: ufn(bufs))
                del bufs
        if not args.only_kernels:
            y_tf = y_flops / (y_ms * 1e-3) / 1e12
            u_tf = dg["flops"] / (u_ms * 1e-3) / 1e12 if u_ms else None
            yardstick = {
                "what": "torch.matmul (hipBLASLt) on the dense equivalents of the dominant kernel's launches, and that kernel "
                        "on the un-ragged equivalent of its own problem (every expert R/E rows, no gather); same event "
                        "timing, random data of the same distribution",
                "shapes": shapes, "tflops": round(y_tf, 1), "frac_mfma_peak": round(y_tf / peak, 4),
                "kernel_vs_yardstick": round(ach / y_tf, 4),
            }
            if u_tf:
                yardstick.update(kernel_unragged_tflops=round(u_tf, 1), kernel_unragged_frac_mfma_peak=round(u_tf / peak, 4),
                                 kernel_unragged_vs_yardstick=round(u_tf / y_tf, 4))

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
            "workload": workload,
            "tokens": T, "hidden": H, "experts": E, "top_k": K, "intermediate": I, "tile_cfg": c,
        },
        "commit": git_head(),
        "kernel_commit": kernel_commit(),
        "tflops": tflops,
        "frac_mfma_peak": tflops / peak,
        "grouped_gemm_tflops": gemm_flop / (gemm_ms * 1e-3) / 1e12,
        "grouped_gemm_frac_mfma_peak": gemm_flop / (gemm_ms * 1e-3) / 1e12 / peak,
        "roofline": roofline,
        "yardstick": yardstick,
        "kernels": breakdown,
        "kernels_note": "each entry is that kernel launched on its own, back to back, on the intermediates of a real "
                        "step (roofline.avg_ms comes from these launches); a kernel repeated back to back does not run "
                        "at the clocks and cache state it has inside a step, so the entries do not add up to ms_per_step",
    }
    if name == "c4":
        result["config"]["note"] = "a token of this workload is one routed row (the rows arrive already dispatched)"
    if not args.no_cpu_baseline:
        # about 0.45 TFLOP of CPU work (10-30 s on 16 host threads in bf16), at most T/8 tokens; c1 in full
        budget = int(0.45e12 / (18.0 * K * H * I)) // 256 * 256
        sample = args.cpu_sample_tokens or (T if name == "c1" else max(min(T // 8, budget), 256))
        result["cpu_baseline"] = cpu_baseline(name, min(sample, T), torch)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
