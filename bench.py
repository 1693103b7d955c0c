#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

Workload (default): the 480p video self-attention layer -- B=1, H=24, D=128, S = 31 x (30 x 52) =
48,360 tokens; hidden states ~ N(0,1) projected by random-init Wq/Wk/Wv (std 0.02), QK-RMSNorm
(eps 1e-6, unit weight), 3-axis RoPE (32/48/48, theta 1e4); non-causal, no mask.  A "step" is one
layer call through the C ABI: prologue kernels (norm + RoPE + operand layout of Q, K, V) plus the
attention kernel, inputs resident in HBM.

Prints ONE JSON line: `value` = 4*Sq*Sk*D*H / step time in TFLOP/s; `roofline` prices the attention
kernel alone (HIP events on its stream, inside the library) against the bf16 dense MFMA peak;
`cpu_baseline` times torch's CPU scaled_dot_product_attention path on a declared query-row sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "fp8": 5000.0}  # MI355X dense MFMA, published
HBM_PEAK_GBS = 8000.0
# HBM-side bytes per attention-kernel launch measured with rocprofv3 --pmc (FETCH_SIZE x 2.00 + WRITE_SIZE x 1.00,
# factors from a 1 GiB copy) in earlier profiling runs of the same command, not in this run: (bytes, file that holds
# the counter values and the commands)
MEASURED_TRAFFIC = {
    "480p": (3.96e9, "profiles/attn_fwd_kernel_480p_bf16.md"),
    "480p-fp8": (3.27e9, "profiles/attn_fwd_kernel_480p_fp8.md"),
    "480p-sparse": (3.160e10, "profiles/attn_fwd_kernel_480p_sparse_bf16.md"),
    "480p-sparse-fp8": (2.129e10, "profiles/attn_fwd_kernel_480p_sparse_fp8.md"),
    "768p": (2.09e10, "profiles/attn_fwd_kernel_768p_bf16.md"),
    "joint": (4.43e9, "profiles/attn_fwd_kernel_joint_bf16.md"),
    "cross": (6.15e8, "profiles/attn_fwd_kernel_cross_short_key.md"),
}
GEMM_TRAFFIC = (7.51e9, "profiles/gemm_kernel_480p_block.md")  # to_q/to_k/to_v launch of the 480p block


def host_cpu():
    """(model name, physical cores) of the host from /proc/cpuinfo; physical = distinct (package, core id) pairs."""
    model, cores = "unknown", set()
    try:
        phys = "0"
        for line in open("/proc/cpuinfo"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "model name":
                model = val
            elif key == "physical id":
                phys = val
            elif key == "core id":
                cores.add((phys, val))
    except OSError:
        pass
    return model, (len(cores) or os.cpu_count() or 0)


def _time_steps(step, steps, warmup):
    """(mean ms per step over the K timed steps bracketed by synchronisation, median, minimum)."""
    import torch

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    mean = (time.perf_counter() - t0) * 1e3 / steps
    per = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    return mean, per[len(per) // 2], per[0]


def bench_block(args, pk, workloads, dev) -> int:
    """The attention half of one DiT block at 480p: AdaLN modulation -> to_q/to_k/to_v (+LoRA rank 128) -> attention ->
    to_out.0 (+LoRA) with gate and residual.  A "step" is that whole sequence through the library's projection GEMMs
    (K/V written by the GEMM epilogue in the attention kernel's layout); the same block with the projections and the
    modulation as torch ops (hipBLASLt GEMMs, then the library's K/V pass and attention kernel) is timed beside it."""
    import torch
    import torch.nn.functional as F

    from pika_h3_flex_amd import projections as P

    blk = workloads.block_inputs(frames=31, rows_h=30, rows_w=52, seed=args.seed, device=dev, name="480p-block")
    S, C = blk.x.shape
    H = blk.heads
    ones = torch.ones(128, dtype=torch.float32, device=dev)
    tabs = pk.rope_tables(blk.position_ids)
    opts = dict(q_norm_weight=ones, k_norm_weight=ones, norm_eps=1e-6, rope_mode=pk.ROPE_INTERLEAVED, rope_q=tabs)
    packed = {n: P.PackedLinear.from_weights(d["weight"], d["bias"], lora_a=d["lora_a"], lora_b=d["lora_b"],
                                             lora_scale=d["lora_scale"], head_perm=(n != "v")) for n, d in blk.linears.items()}

    def fused():
        x_img = P.adaln_modulate(blk.x, shift=blk.shift, scale=blk.scale, row_index=blk.row_index, norm="layer")
        o_img = P.qkv_attention(x_img, S, packed["q"], packed["k"], packed["v"], heads=H, out_images=True, **opts)
        return P.out_proj(None, packed["out"], gate=blk.gate, row_index=blk.row_index, residual=blk.x, o_img=o_img, rows=S)

    idx = blk.row_index.long()

    def lin(x, d):
        return F.linear(x, d["weight"], d["bias"].to(x.dtype)) + d["lora_scale"] * F.linear(F.linear(x, d["lora_a"]), d["lora_b"])

    def unfused():
        xm = F.layer_norm(blk.x, (C,), eps=1e-6) * (1 + blk.scale.index_select(0, idx)) + blk.shift.index_select(0, idx)
        q, k, v = (lin(xm, blk.linears[n]).view(1, S, H, 128) for n in ("q", "k", "v"))
        o = pk.attention(q, k, v, **opts)
        return blk.x + blk.gate.index_select(0, idx) * lin(o.view(S, C), blk.linears["out"])

    def projections_only():
        x_img = P.adaln_modulate(blk.x, shift=blk.shift, scale=blk.scale, row_index=blk.row_index, norm="layer")
        return x_img

    ms, ms_median, ms_min = _time_steps(fused, args.steps, args.warmup)
    ms_unfused, _, _ = _time_steps(unfused, max(3, args.steps // 4), 2)
    # the GEMM launches alone: QKV (+ down-projections) and to_out, events on the launch stream
    x_img = P.adaln_modulate(blk.x, shift=blk.shift, scale=blk.scale, row_index=blk.row_index, norm="layer")
    o = torch.randn((S, C), device=dev).to(torch.bfloat16)
    q_scratch = torch.empty((1, S, H, 128), dtype=torch.bfloat16, device=dev)

    def qkv_only():
        import ctypes as C_

        from pika_h3_flex_amd import _lib

        a, keep = pk.ops.fill_args(q_scratch, None, None, torch.empty_like(q_scratch), kv_prepared=True, **opts)
        ws = torch.empty(pk.ops.workspace_bytes(a), dtype=torch.uint8, device=dev)
        lws = torch.empty(P.packed_bytes(S, 3 * _lib.LORA_RANK), dtype=torch.uint8, device=dev)
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
        pa = _lib.QkvArgs()
        pa.x_img, pa.S, pa.K = x_img.data_ptr(), S, C
        pa.q, pa.k, pa.v = packed["q"].c_struct(), packed["k"].c_struct(), packed["v"].c_struct()
        pa.lora_workspace, pa.lora_workspace_bytes = lws.data_ptr(), lws.numel()
        st = C_.c_void_p(torch.cuda.current_stream().cuda_stream)
        lib = _lib.load()

        def run():
            _lib.check(lib.pkh3_qkv_proj(C_.byref(pa), C_.byref(a), st))
        return run, (ws, lws, keep)

    run_qkv, _keep = qkv_only()
    ms_qkv, _, _ = _time_steps(run_qkv, 10, 3)
    o_img = P.pack_rows(o)
    ms_out, _, _ = _time_steps(lambda: P.out_proj(None, packed["out"], gate=blk.gate, row_index=blk.row_index, residual=blk.x,
                                                  o_img=o_img, rows=S), 10, 3)
    ms_mod, _, _ = _time_steps(projections_only, 10, 3)
    r = blk.linears["q"]["lora_a"].shape[0]
    flops_qkv = 3 * (2.0 * S * C * C + 2.0 * S * C * r + 2.0 * S * r * C)
    flops_out = 2.0 * S * C * C + 2.0 * S * C * r + 2.0 * S * r * C
    total = blk.attention_flops + blk.projection_flops
    value = total / (ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS["bf16"]
    gemm_tflops = flops_qkv / (ms_qkv * 1e-3) / 1e12
    line = {
        "metric": "attention-block TFLOP/s (attention 4*S*S*D*H + the four projections with LoRA; AdaLN, gate and residual included in the time)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"480p attention block: S={S}, hidden={C}, H={H}, D=128, LoRA rank {r} on to_q/to_k/to_v/to_out.0, "
                               f"AdaLN over {blk.shift.shape[0]} timestep groups, QK-RMSNorm + 3-axis RoPE, non-causal",
                   "seed": args.seed, "ms_per_step_median": round(ms_median, 4), "ms_per_step_min": round(ms_min, 4),
                   "ms_per_step_with_torch_projections": round(ms_unfused, 4),
                   "ms_adaln_modulate": round(ms_mod, 4), "ms_qkv_projection": round(ms_qkv, 4),
                   "ms_out_projection": round(ms_out, 4),
                   "out_projection_tflops": round(flops_out / (ms_out * 1e-3) / 1e12, 2)},
        "roofline": {"bound": "mfma", "achieved": round(gemm_tflops, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(gemm_tflops / peak, 4), "traffic": GEMM_TRAFFIC[0], "traffic_source": GEMM_TRAFFIC[1], "kernel": "gemm_kernel (to_q/to_k/to_v + LoRA, two launches)",
                     "kernel_ms": round(ms_qkv, 4), "flops_per_launch": flops_qkv},
        "cpu_baseline": None,
    }
    print(json.dumps(line))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="480p", choices=["plumbing", "480p", "768p", "joint", "cross", "480p-sparse", "480p-sparse-fp8", "480p-fp8", "480p-block"])
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--cpu-rows", type=int, default=32768, help="query rows of the CPU baseline sample (0 = skip)")
    ap.add_argument("--kernel-iters", type=int, default=10)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 1 GiB device-to-device copy, a kernel of known traffic for scaling profiler byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU over the full local sequence (no sequence-parallel split, "
              "no collectives); --gpus must be 1", file=sys.stderr)
        return 2

    import torch

    import __graft_entry__

    __graft_entry__.ensure_built()  # loads what is built; compiles only when there is nothing
    import pika_h3_flex_amd as pk
    from pika_h3_flex_amd import workloads

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP library is the only compute path", file=sys.stderr)
        return 2
    dev = "cuda:0"
    torch.cuda.set_device(0)

    if args.workload == "480p-block":
        return bench_block(args, pk, workloads, dev)

    base = args.workload.split("-")[0]
    inp = workloads.make(base, seed=args.seed, device=dev)
    B, Sq, H, D = inp.q.shape
    Sk = inp.k.shape[1]
    ones = torch.ones(D, dtype=torch.float32, device=dev)
    opts = dict(q_norm_weight=ones, k_norm_weight=ones, norm_eps=1e-6)
    tabs = None
    if inp.position_ids is not None:
        tabs = pk.rope_tables(inp.position_ids)
        opts.update(rope_mode=pk.ROPE_INTERLEAVED, rope_q=tabs)
    if inp.key_mask is not None:
        opts.update(key_mask=inp.key_mask)
    density = 1.0
    fp8 = args.workload.endswith("fp8")
    if "sparse" in args.workload:
        tm = pk.local_window_tile_map(Sq, inp.tokens_per_frame, window_frames=2, global_fraction=0.10, seed=args.seed)
        density = float(tm.float().mean())
        opts.update(block_mask=pk.BlockMask.from_dense(tm, device=dev))
    if fp8:
        opts.update(fp8_qk=True)
    flops = inp.flops * density

    out = torch.empty_like(inp.q)
    args_ws, _keep = pk.ops.fill_args(inp.q, inp.k, inp.v, out, **opts)
    ws = torch.empty(pk.ops.workspace_bytes(args_ws), dtype=torch.uint8, device=dev)

    def step():
        pk.attention(inp.q, inp.k, inp.v, out=out, workspace=ws, **opts)

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # the K timed steps, bracketed by synchronisation; per-step events (same stream) give median and minimum
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(args.steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    ms_median, ms_min = per_step[len(per_step) // 2], per_step[0]
    value = flops / (ms_per_step * 1e-3) / 1e12

    kernel_ms = pk.time_attention_kernel(inp.q, inp.k, inp.v, iters=args.kernel_iters, **opts)
    achieved = flops / (kernel_ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS["fp8" if fp8 else "bf16"]
    traffic = MEASURED_TRAFFIC.get(args.workload, (None, None))[0]
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                "frac": round(achieved / peak, 4), "traffic": MEASURED_TRAFFIC.get(args.workload, (None, None))[0],
                "traffic_source": MEASURED_TRAFFIC.get(args.workload, (None, None))[1], "kernel": "attn_fwd_kernel",
                "kernel_ms": round(kernel_ms, 4), "flops_per_launch": flops}

    if traffic is not None:
        # the other roof: bytes that crossed the L2 boundary per launch (profiled) over this run's kernel time
        rate = traffic / (kernel_ms * 1e-3) / 1e9
        roofline["traffic_rate_gbs"] = round(rate, 1)
        roofline["traffic_frac_of_hbm_peak"] = round(rate / HBM_PEAK_GBS, 4)
        roofline["binding_roof"] = "hbm" if rate / HBM_PEAK_GBS > achieved / peak else "mfma"

    cpu = None
    if args.cpu_rows > 0:
        from oracle import cpu_sdpa

        rows = min(args.cpu_rows, Sq)
        cpu_opts = dict(q_norm_weight=ones, k_norm_weight=ones, eps=1e-6, dtype=torch.float32)
        if tabs is not None:
            cpu_opts.update(rope_q=tabs)
        if inp.key_mask is not None:
            cpu_opts.update(key_mask=inp.key_mask.cpu())
        secs, threads = cpu_sdpa.time_cpu_baseline(inp.q, inp.k, inp.v, sample_rows=rows, **cpu_opts)
        sk_eff = Sk if inp.key_mask is None else int(inp.key_mask.sum())
        cpu_flops = 4.0 * rows * sk_eff * D * H
        cpu_model, cpu_physical = host_cpu()
        cpu = {"value": round(cpu_flops / secs / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
               "cpu_model": cpu_model, "physical_cores": cpu_physical,
               "sample": f"torch CPU F.scaled_dot_product_attention fp32 (+RMSNorm, RoPE in torch) on the first {rows} of {Sq} "
                         f"query rows x all {Sk} keys x {H} heads, dense, one call of {secs:.2f} s; rate scales linearly in rows"}

    line = {
        "metric": "attention TFLOP/s (4*Sq*Sk*D*H per layer call; prologue + attention kernel)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8-e4m3 QK^T + bf16 PV" if fp8 else "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload} attention layer: B={B}, H={H}, D={D}, Sq={Sq}, Sk={Sk}, "
                               f"QK-RMSNorm + 3-axis RoPE, non-causal" + (f", block-sparse density {density:.3f}" if density < 1 else ""),
                   "seed": args.seed, "pct_of_mfma_peak": round(100.0 * value / peak, 2),
                   "ms_per_step_median": round(ms_median, 4), "ms_per_step_min": round(ms_min, 4)},
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
