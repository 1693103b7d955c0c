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

The default run (workload 480p) then measures, outside the headline's timed region, the other
workloads of the benchmark contract -- fp8 QK^T, block-sparse, block-sparse fp8, 768p, joint
video+audio, text cross-attention, and the attention half of a 480p block through the library's
projections -- and reports them under `config.other_workloads`, and the CPU-runnable configuration 1
in full (torch CPU fp32 and bf16, and the library) under `cpu_baseline.config1`.  `--no-others` and
any other `--workload` measure just the one workload.
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
    "480p": (4.55e9, "profiles/attn_fwd_dense_kernel_480p_bf16.md"),
    "480p-fp8": (3.84e9, "profiles/attn_fwd_dense_kernel_480p_fp8.md"),
    "480p-fp8-pow2": (3.81e9, "profiles/attn_fwd_dense_kernel_480p_fp8.md"),
    "480p-sparse-fp8-pow2": (2.118e10, "profiles/attn_fwd_kernel_480p_sparse_fp8.md"),
    "480p-sparse": (3.213e10, "profiles/attn_fwd_kernel_480p_sparse_bf16.md"),
    "480p-sparse-fp8": (2.129e10, "profiles/attn_fwd_kernel_480p_sparse_fp8.md"),
    "768p": (2.33e10, "profiles/attn_fwd_dense_kernel_768p_bf16.md"),
    "joint": (4.55e9, "profiles/attn_fwd_dense_kernel_joint_bf16.md"),
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


def bench_block(args, pk, workloads, dev) -> dict:
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

    P.PackedLinear.share_adapter_buffer(packed["q"], packed["k"], packed["v"])

    def block(pl):
        x_img = P.adaln_modulate(blk.x, shift=blk.shift, scale=blk.scale, row_index=blk.row_index, norm="layer")
        o_img = P.qkv_attention(x_img, S, pl["q"], pl["k"], pl["v"], heads=H, out_images=True, **opts)
        return P.out_proj(None, pl["out"], gate=blk.gate, row_index=blk.row_index, residual=blk.x, o_img=o_img, rows=S)

    def fused():
        return block(packed)

    # the opt-in deployment form: adapters folded into the weights when they are packed (not what the reference runs)
    merged = {n: P.PackedLinear.from_weights(d["weight"], d["bias"], lora_a=d["lora_a"], lora_b=d["lora_b"],
                                             lora_scale=d["lora_scale"], head_perm=(n != "v"), merge_adapter=True)
              for n, d in blk.linears.items()}

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
    ms_merged, _, _ = _time_steps(lambda: block(merged), max(3, args.steps // 2), 2)
    del merged
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
                   "ms_per_step_with_merged_adapters": round(ms_merged, 4),
                   "ms_adaln_modulate": round(ms_mod, 4), "ms_qkv_projection": round(ms_qkv, 4),
                   "ms_out_projection": round(ms_out, 4),
                   "out_projection_tflops": round(flops_out / (ms_out * 1e-3) / 1e12, 2)},
        "roofline": {"bound": "mfma", "achieved": round(gemm_tflops, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(gemm_tflops / peak, 4), "traffic": GEMM_TRAFFIC[0], "traffic_source": GEMM_TRAFFIC[1], "kernel": "gemm_kernel (to_q/to_k/to_v + LoRA, two launches)",
                     "kernel_ms": round(ms_qkv, 4), "flops_per_launch": flops_qkv},
        "cpu_baseline": None,
    }
    return line


ATTENTION_WORKLOADS = ("plumbing", "480p", "768p", "joint", "cross", "480p-sparse", "480p-sparse-fp8", "480p-fp8",
                       "480p-fp8-pow2", "480p-sparse-fp8-pow2")
# what the default run measures beside the headline (same process, after the headline's timed region); "-pow2" is the
# opt-in fp8 rule with power-of-two block scales applied by the scaled MFMA (PKH3_FLAG_FP8_POW2_SCALES)
OTHER_WORKLOADS = ("480p-fp8", "480p-fp8-pow2", "480p-sparse", "480p-sparse-fp8", "480p-sparse-fp8-pow2", "768p", "joint",
                   "cross", "480p-block")


def algorithmic_bytes(B, Sq, Sk, H, D, fp8, density=1.0):
    """Compulsory HBM bytes of one attention-kernel launch: Q read and O written once in bf16, the K' and V operand
    images read once (K' one byte per element on the fp8 path).  Block-sparse calls still touch every K/V tile that
    any row-block keeps, i.e. all of them at these densities."""
    return float(B * H * D * (2 * Sq + 2 * Sq + (1 if fp8 else 2) * Sk + 2 * Sk))


class AttentionCase:
    """One attention workload set up on the device: inputs, options, output and workspace."""

    def __init__(self, pk, workloads, name, seed, dev, inputs=None):
        import torch

        self.pk, self.name = pk, name
        base = name.split("-")[0]
        self.inp = inputs if inputs is not None else workloads.make(base, seed=seed, device=dev)
        inp = self.inp
        self.B, self.Sq, self.H, self.D = inp.q.shape
        self.Sk = inp.k.shape[1]
        self.ones = torch.ones(self.D, dtype=torch.float32, device=dev)
        opts = dict(q_norm_weight=self.ones, k_norm_weight=self.ones, norm_eps=1e-6)
        self.tabs = None
        if inp.position_ids is not None:
            self.tabs = pk.rope_tables(inp.position_ids)
            opts.update(rope_mode=pk.ROPE_INTERLEAVED, rope_q=self.tabs)
        if inp.key_mask is not None:
            opts.update(key_mask=inp.key_mask)
        self.density = 1.0
        self.fp8 = "fp8" in name.split("-")
        self.pow2 = name.endswith("-pow2")
        if "sparse" in name:
            tm = pk.local_window_tile_map(self.Sq, inp.tokens_per_frame, window_frames=2, global_fraction=0.10, seed=seed)
            self.density = float(tm.float().mean())
            opts.update(block_mask=pk.BlockMask.from_dense(tm, device=dev))
        if self.fp8:
            opts.update(fp8_qk="pow2" if self.pow2 else True)
        self.opts = opts
        self.flops = inp.flops * self.density
        self.out = torch.empty_like(inp.q)
        args_ws, _keep = pk.ops.fill_args(inp.q, inp.k, inp.v, self.out, **opts)
        self.ws = torch.empty(pk.ops.workspace_bytes(args_ws), dtype=torch.uint8, device=dev)

    def step(self):
        self.pk.attention(self.inp.q, self.inp.k, self.inp.v, out=self.out, workspace=self.ws, **self.opts)

    def describe(self):
        return (f"{self.name} attention layer: B={self.B}, H={self.H}, D={self.D}, Sq={self.Sq}, Sk={self.Sk}, "
                f"QK-RMSNorm + 3-axis RoPE, non-causal" + (f", block-sparse density {self.density:.3f}" if self.density < 1 else "")
                + (", power-of-two fp8 block scales" if self.pow2 else ""))

    def kernel_name(self):
        if self.density < 1:
            return "attn_fwd_kernel (block-sparse, 8 waves)"
        return "attn_fwd_kernel (short-key, 4 waves)" if self.Sk <= 1024 else "attn_fwd_dense_kernel (12 waves)"

    def roofline(self, kernel_iters):
        """The attention kernel alone (HIP events on its stream, inside the library) against its MFMA peak, beside
        the bytes: algorithmic ones, and the profiled ones where a profile of this workload is committed."""
        kernel_ms = self.pk.time_attention_kernel(self.inp.q, self.inp.k, self.inp.v, iters=kernel_iters, **self.opts)
        achieved = self.flops / (kernel_ms * 1e-3) / 1e12
        peak = PEAK_TFLOPS["fp8" if self.fp8 else "bf16"]
        traffic, source = MEASURED_TRAFFIC.get(self.name, (None, None))
        alg = algorithmic_bytes(self.B, self.Sq, self.Sk if self.inp.key_mask is None else int(self.inp.key_mask.sum()),
                                self.H, self.D, self.fp8)
        r = {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
             "frac": round(achieved / peak, 4), "traffic": traffic, "traffic_source": source,
             "algorithmic_bytes": alg, "traffic_over_algorithmic": None if traffic is None else round(traffic / alg, 2),
             "kernel": self.kernel_name(), "kernel_ms": round(kernel_ms, 4), "flops_per_launch": self.flops}
        if traffic is not None:
            # the other roof: bytes that crossed the L2 boundary per launch (profiled) over this run's kernel time
            rate = traffic / (kernel_ms * 1e-3) / 1e9
            r["traffic_rate_gbs"] = round(rate, 1)
            r["traffic_frac_of_hbm_peak"] = round(rate / HBM_PEAK_GBS, 4)
            r["binding_roof"] = "hbm" if rate / HBM_PEAK_GBS > achieved / peak else "mfma"
        return r


def other_workload_record(case, steps, warmup, kernel_iters):
    ms, ms_median, ms_min = _time_steps(case.step, steps, warmup)
    r = case.roofline(kernel_iters)
    peak = r["peak"]
    tflops = case.flops / (ms * 1e-3) / 1e12
    return {"workload": case.describe(), "dtype": "fp8-e4m3 QK^T + bf16 PV" if case.fp8 else "bf16",
            "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 4), "ms_per_step_min": round(ms_min, 4),
            "tflops": round(tflops, 2), "peak_tflops": peak, "frac": round(tflops / peak, 4),
            "kernel_ms": r["kernel_ms"], "kernel_frac": r["frac"], "binding_roof": r.get("binding_roof", "mfma"),
            "algorithmic_bytes": r["algorithmic_bytes"], "traffic": r["traffic"], "traffic_source": r["traffic_source"],
            "traffic_ratio": r["traffic_over_algorithmic"], "traffic_frac_of_hbm_peak": r.get("traffic_frac_of_hbm_peak")}


def config1_baselines(pk, workloads, dev, seed):
    """The CPU-runnable configuration (B=1, H=4, S=1024, D=128, QK-RMSNorm, no mask) in full: torch CPU
    scaled_dot_product_attention in fp32 and in bf16 on the host, and the library on the card."""
    import torch

    from oracle import cpu_sdpa

    inp = workloads.make("plumbing", seed=seed, device=dev)
    ones = torch.ones(128, dtype=torch.float32, device=dev)
    flops = inp.flops
    rec = {"workload": "B=1, H=4, S=1024, D=128, QK-RMSNorm (eps 1e-6, unit weight), no mask, non-causal; whole call", "flops": flops}
    for name, dt in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
        secs, threads = cpu_sdpa.time_cpu_baseline(inp.q, inp.k, inp.v, sample_rows=inp.q.shape[1], repeats=5,
                                                   q_norm_weight=ones, k_norm_weight=ones, eps=1e-6, dtype=dt)
        rec[f"cpu_{name}_ms"] = round(secs * 1e3, 3)
        rec[f"cpu_{name}_tflops"] = round(flops / secs / 1e12, 4)
        rec["cores"] = threads
    out = torch.empty_like(inp.q)
    ms, _, ms_min = _time_steps(lambda: pk.attention(inp.q, inp.k, inp.v, out=out, q_norm_weight=ones, k_norm_weight=ones), 50, 10)
    rec["gpu_ms"] = round(ms, 4)
    rec["gpu_tflops"] = round(flops / (ms * 1e-3) / 1e12, 2)
    return rec


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="480p", choices=list(ATTENTION_WORKLOADS) + ["480p-block"])
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--cpu-rows", type=int, default=32768, help="query rows of the CPU baseline sample (0 = skip)")
    ap.add_argument("--kernel-iters", type=int, default=10)
    ap.add_argument("--no-others", action="store_true",
                    help="only the named workload: skip the other workloads and the config-1 baselines the default run adds")
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
        print(json.dumps(bench_block(args, pk, workloads, dev)))
        return 0

    case = AttentionCase(pk, workloads, args.workload, args.seed, dev)
    inp, flops, fp8 = case.inp, case.flops, case.fp8
    B, Sq, H, D, Sk = case.B, case.Sq, case.H, case.D, case.Sk

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # the K timed steps, bracketed by synchronisation; per-step events (same stream) give median and minimum
    ms_per_step, ms_median, ms_min = _time_steps(case.step, args.steps, args.warmup)
    value = flops / (ms_per_step * 1e-3) / 1e12
    roofline = case.roofline(args.kernel_iters)
    peak = roofline["peak"]

    others = None
    config1 = None
    if args.workload == "480p" and not args.no_others:
        # Everything below runs after the headline's timed region, one workload at a time, each freed before the
        # next: >= 5 warm-up and >= 10 timed layer calls each, the attention kernel alone timed beside them.
        others = {}
        o_steps, o_warm = max(10, args.steps // 2), max(5, args.warmup)
        for name in OTHER_WORKLOADS:
            if name == "480p-block":
                b_args = argparse.Namespace(**{**vars(args), "steps": o_steps, "warmup": o_warm})
                blk = bench_block(b_args, pk, workloads, dev)
                others[name] = {"workload": blk["config"]["workload"], "dtype": "bf16", "steps": o_steps, "warmup": o_warm,
                                "ms_per_step": blk["ms_per_step"], "tflops": blk["value"], "peak_tflops": PEAK_TFLOPS["bf16"],
                                "frac": round(blk["value"] / PEAK_TFLOPS["bf16"], 4),
                                "ms_per_step_with_torch_projections": blk["config"]["ms_per_step_with_torch_projections"],
                                "ms_per_step_with_merged_adapters": blk["config"]["ms_per_step_with_merged_adapters"],
                                "ms_qkv_projection": blk["config"]["ms_qkv_projection"], "qkv_projection_frac": blk["roofline"]["frac"],
                                "ms_out_projection": blk["config"]["ms_out_projection"], "ms_adaln_modulate": blk["config"]["ms_adaln_modulate"],
                                "binding_roof": "mfma", "traffic": blk["roofline"]["traffic"], "traffic_source": blk["roofline"]["traffic_source"]}
                continue
            shares_inputs = name.split("-")[0] == "480p"
            other = AttentionCase(pk, workloads, name, args.seed, dev, inputs=inp if shares_inputs else None)
            others[name] = other_workload_record(other, o_steps, o_warm, args.kernel_iters)
            del other
            torch.cuda.empty_cache()
        if args.cpu_rows > 0:
            config1 = config1_baselines(pk, workloads, dev, args.seed)

    cpu = None
    if args.cpu_rows > 0:
        from oracle import cpu_sdpa

        rows = min(args.cpu_rows, Sq)
        cpu_opts = dict(q_norm_weight=case.ones, k_norm_weight=case.ones, eps=1e-6, dtype=torch.float32)
        if case.tabs is not None:
            cpu_opts.update(rope_q=case.tabs)
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
        if config1 is not None:
            cpu["config1"] = config1

    line = {
        "metric": "attention TFLOP/s (4*Sq*Sk*D*H per layer call; prologue + attention kernel)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8-e4m3 QK^T + bf16 PV" if fp8 else "bf16", "data": "synthetic",
        "config": {"workload": case.describe(),
                   "seed": args.seed, "pct_of_mfma_peak": round(100.0 * value / peak, 2),
                   "ms_per_step_median": round(ms_median, 4), "ms_per_step_min": round(ms_min, 4)},
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    if others is not None:
        line["config"]["other_workloads"] = others
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
