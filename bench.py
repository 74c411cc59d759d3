"""Benchmark of the TTT operation on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--repeats R] [--config c1|c2|c3|c4|layer] [--no-cpu-baseline]

One step = forward + backward of block_causal_lact_swiglu over one batch of seeded synthetic input
that is resident in HBM before the timed region.  After W warm-up steps, R regions of exactly K steps are timed
(each between two device synchronisations); `value` comes from the median region.  Prints one JSON line
(metric: tokens/s, tokens = B*L); for config c1 the line also carries short runs of c2, c3 and c4 (`other_configs`).
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0

CONFIGS = {
    # name: (B, H, L, d, dh, chunk, seed, text)
    "c1": (4, 4, 4096, 384, 384, 2048, 1001,
           "config 1: block_causal_lact_swiglu fwd+bwd, 760M shape B=4 H=4 (b=16), L=4096, d=dh=384, chunk 2048, "
           "Muon NS5 + momentum 0.9, bf16 activations / fp32 fast weights"),
    "c2": (1, 4, 32768, 384, 384, 2048, 1002,
           "config 2: block_causal_lact_swiglu fwd+bwd, B=1 H=4 (b=4), L=32768, d=dh=384, chunk 2048, Muon + momentum"),
    "c4": (1, 12, 32760, 128, 256, 4680, 1004,
           "config 4: block_causal_lact_swiglu fwd+bwd, video shape b=12, L=32760, d=128, dh=256, chunk 4680, Muon + momentum"),
    # forward only: one update on 8192 tokens (8 input views), one apply on 1024 tokens (the target view)
    "c3": (1, 6, 9216, 128, 256, 8192, 1003,
           "config 3: fast_weight_swish_glu_weight_norm_mini_batch_apply forward only, NVS shape b=6, d=128, dh=256, "
           "update on 8192 tokens then apply on 1024, Muon with 5 classic Newton-Schulz steps"),
    # the layer around the operation (not a BASELINE configuration: the callers either side of the path, measured)
    "layer": (4, 4, 4096, 384, 384, 2048, 1005,
              "layer: CausalLaCTSwiGLUWithSlidingWindowAttn fwd+bwd under bf16 autocast, 760M shape (dim 1536 = 4 heads of "
              "384, 12 attention heads of 128, window 2048), B=4, L=4096, chunk 2048, Muon + momentum; projections are "
              "rocBLAS GEMMs through torch.nn.Linear, attention is torch's blocked SDPA, the rest is this library"),
}


PEAK_HBM_GBPS = 8000.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "{cfg}_fwd_bwd_hbm_traffic_pmc.txt")


def _library_label(profile_name):
    """Kernel name as rocprofv3 prints it (demangled) -> the label the library's own launch records use."""
    import re
    n = profile_name.strip()
    n = re.sub(r"^void\s+", "", n).split("(")[0].replace("lact::", "")
    n = re.sub(r"TileShape<(\d+), (\d+), \d+, \d+>\s*", r"\1x\2", n).replace(" ", "")
    m = re.match(r"k_ns_fused<(\d+x\d+),(true|false)>", n)
    if m:
        return f"k_ns_fused<{m.group(1)},{'bwd' if m.group(2) == 'true' else 'fwd'}>"
    m = re.match(r"k_row_gemm_dma<(\d+x\d+),(\d+),(\d+),(true|false)>", n)
    if m:
        epi = {"0": "store", "1": "axpby", "2": "axpby_dual"}[m.group(3)]
        return f"k_row_gemm_dma<{m.group(1)},{m.group(2)},{epi},{'Bks' if m.group(4) == 'true' else 'Bkc'}>"
    m = re.match(r"k_hidden_persist<(Apply|Update|ApplyBwd)HiddenPolicy>", n)
    if m:
        return f"k_hidden_persist<{ {'Apply': 'apply', 'Update': 'update', 'ApplyBwd': 'apply_bwd'}[m.group(1)] }>"
    m = re.match(r"(k_token_reduce(?:_rows)?_dma)<(\d+x\d+)>", n)
    if m:
        return f"{m.group(1)}<{m.group(2)}>"
    return n.split("<")[0]


def load_traffic(cfg):
    """HBM bytes per launch of every kernel and per step, read from the committed counter summary of this
    configuration (FETCH_SIZE / WRITE_SIZE of two `rocprofv3 --pmc` runs, already scaled by the copy calibration
    the file states).  Returns ({library label: bytes per launch}, bytes per step or None); empty when the file is
    missing or a line does not parse -- the bench line then carries `traffic: null`."""
    import re
    per_kernel, per_step = {}, None
    try:
        with open(TRAFFIC_PROFILE.format(cfg=cfg)) as f:
            for line in f:
                m = re.match(r"^(.*\S)\s+(\d+)\s+([0-9.]+)\s+([0-9.]+)\s*$", line)
                if m and "k_" in m.group(1):
                    per_kernel[_library_label(m.group(1))] = (float(m.group(3)) + float(m.group(4))) * 2 ** 20
                m = re.match(r"^per step.*read\s+([0-9.]+) MiB, write\s+([0-9.]+) MiB", line)
                if m:
                    per_step = (float(m.group(1)) + float(m.group(2))) * 2 ** 20
    except OSError:
        pass
    return per_kernel, per_step


def algorithmic_flops(b, L, d, dh, C, ns_steps=5):
    """Counted FLOPs of fwd+bwd (multiply-add = 2; backward = 2x forward; recompute, momentum, renorm and
    pointwise work not counted): F_apply = 6 d dh T, F_update = 12 d dh T, F_ns = 3 steps (4 r^2 c + 2 r^3)."""
    n_chunks = max(1, math.ceil(L / C))
    n_upd = n_chunks - 1
    r, c = min(d, dh), max(d, dh)
    f_apply = 6.0 * d * dh * L
    f_update = 12.0 * d * dh * (n_upd * C)
    f_ns = 3.0 * ns_steps * (4.0 * r * r * c + 2.0 * r ** 3) * n_upd
    return 3.0 * b * (f_apply + f_update + f_ns)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c1", choices=sorted(CONFIGS))
    ap.add_argument("--repeats", type=int, default=5, help="timed regions of --steps steps each; the median region is reported")
    ap.add_argument("--no-other-configs", action="store_true", help="config c1 only: skip the short runs of c2, c3 and c4")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-profile", action="store_true")
    ap.add_argument("--no-overlap", action="store_true",
                    help="keep the apply steps on the caller's stream (LACT_OPT_STREAM_OVERLAP off): kernels then run "
                         "one at a time and their durations are those of the kernel alone; used for profiles")
    ap.add_argument("--persistent-tiles", type=int, default=None,
                    help="LACT_OPT_PERSISTENT_TILES mask (bit 0 apply, 1 update, 2 apply backward hidden stage; default: the "
                         "library's, 1); 0 runs the one-tile-per-block kernels for comparison")
    ap.add_argument("--keep-preactivations", type=int, default=None,
                    help="LACT_OPT_KEEP_PREACTIVATIONS: 0 the update's backward recomputes its hidden stage, 1 the forward "
                         "keeps the rounded pre-activations and lr-scaled operands (default: the library's choice by shape)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy (three times): the known-size kernel that scales the "
                         "FETCH_SIZE / WRITE_SIZE counters of a `rocprofv3 --pmc` run of this command")
    ap.add_argument("--mfma-calibration", action="store_true",
                    help="also run the library's pure matrix-instruction kernel (three times, 1024 workgroups): the kernel "
                         "of known matrix-pipe occupancy that scales a matrix-busy counter of a `rocprofv3 --pmc` run")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the one-GPU operation only: heads (b = B*H) are independent, so N GPUs would each run "
              "a slice of b with no communication; run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import lact_amd
    from lact_amd import _lib
    from oracle import lact_oracle as O

    order = ("w0", "w1", "w2", "q", "k", "v", "lr0", "lr1", "lr2")
    names = list(order) + ["momentum"]

    def build_workload(cfg):
        """The step function of a configuration (inputs resident in HBM) and what describes it."""
        B, H, L, d, dh, C, seed, text = CONFIGS[cfg]
        b = B * H
        w = {"B": B, "H": H, "L": L, "d": d, "dh": dh, "C": C, "b": b, "seed": seed, "text": text}
        if cfg == "c3":
            import math as _m
            from lact_amd import nvs
            inp3 = O.make_inputs(b, L, d, dh, seed=seed, act_dtype=torch.bfloat16, momentum_value=None)
            for n in ("w0", "w1", "w2"):      # transposed layout and sqrt(2) gain of lact_nvs/lact_ttt.py:184-193
                inp3[n] = (inp3[n] * _m.sqrt(2.0)).transpose(1, 2).contiguous()
            dev3 = [inp3[n].to("cuda:0") for n in order]
            program = [nvs.TTTOperator(0, C, True, False), nvs.TTTOperator(C, L, False, True)]

            def step():
                with torch.no_grad():
                    return nvs.fast_weight_swish_glu_weight_norm_mini_batch_apply(*dev3, program, 5)[0]
            r_, c_ = min(d, dh), max(d, dh)   # forward only; apply on L - C tokens, one update on C tokens
            w["flops"] = b * (6.0 * d * dh * (L - C) + 12.0 * d * dh * C + 3.0 * 5 * (4.0 * r_ * r_ * c_ + 2.0 * r_ ** 3))
            w.update(step=step, inp3=inp3, program=program)
            return w
        if cfg == "layer":
            from lact_amd import layers
            torch.manual_seed(seed)
            layer = layers.CausalLaCTSwiGLUWithSlidingWindowAttn(dim=H * d, head_dim=d, attn_head_dim=128, lact_chunk_size=C,
                                                                 window_size=2048).to("cuda:0")
            xin = torch.randn(B, L, H * d, generator=torch.Generator().manual_seed(seed)).to("cuda:0").requires_grad_(True)
            gout = torch.randn(B, L, H * d, generator=torch.Generator().manual_seed(seed + 1)).bfloat16().to("cuda:0")
            no_attention = [False]
            real_attention = layers.sliding_window_attention

            def attention_or_nothing(q_, k_, v_, window):   # the TTT branch alone: attention replaced by its value input
                return v_ if no_attention[0] else real_attention(q_, k_, v_, window)
            layers.sliding_window_attention = attention_or_nothing

            def step():
                for t in layer.parameters():
                    t.grad = None
                xin.grad = None
                with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
                    out = layer(xin)
                out.backward(gout)
                return out
            w.update(step=step, no_attention=no_attention, flops=None)
            return w
        inp = O.make_inputs(b, L, d, dh, seed=seed, act_dtype=torch.bfloat16, distinct_heads=H, momentum_value=0.9)
        dev = {n: inp[n].to("cuda:0").requires_grad_(True) for n in names}
        go = torch.randn(b, L, d, generator=torch.Generator().manual_seed(seed + 1)).bfloat16().to("cuda:0")

        def step():
            for t in dev.values():
                t.grad = None
            out = lact_amd.block_causal_lact_swiglu(*[dev[n] for n in order], C, True, dev["momentum"])
            out.backward(go)
            return out
        w.update(step=step, inp=inp, go=go, flops=algorithmic_flops(b, L, d, dh, C))
        return w

    def time_steps(step, k):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(k):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / k * 1e3

    def kernel_profile(step, k):
        """Per-launch durations of k more steps (HIP events on the launch stream, kernels one at a time)."""
        Lb = _lib.lib()
        Lb.lact_set_option(_lib.OPT_STREAM_OVERLAP, 0)
        Lb.lact_profile_enable(1)
        for _ in range(k):
            step()
        buf = ctypes.create_string_buffer(1 << 20)
        _lib.check(Lb.lact_profile_report(buf, len(buf)))
        Lb.lact_profile_enable(0)
        Lb.lact_set_option(_lib.OPT_STREAM_OVERLAP, 0 if args.no_overlap else 1)
        rows = json.loads(buf.value.decode())
        by_kernel = {}
        for r in rows:
            kk = by_kernel.setdefault(r["kernel"], {"launches": 0, "ms": 0.0, "flops": 0.0})
            kk["launches"] += r["launches"]; kk["ms"] += r["ms"]; kk["flops"] += r["flops"]
        total_ms = sum(kk["ms"] for kk in by_kernel.values())
        dom_name, dom = max(((n, kk) for n, kk in by_kernel.items() if kk["flops"] > 0), key=lambda x: x[1]["ms"])
        avg_ms = dom["ms"] / dom["launches"]
        achieved = dom["flops"] / dom["launches"] / (avg_ms * 1e-3) / 1e12
        return rows, total_ms, dom_name, dom, avg_ms, achieved

    W = build_workload(args.config)
    B, H, L, d, dh, C, b, seed, text = (W[n] for n in ("B", "H", "L", "d", "dh", "C", "b", "seed", "text"))
    step = W["step"]

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.mfma_calibration:
        buf = torch.empty(1024 * 256, dtype=torch.float32, device="cuda:0")
        for _ in range(3):
            _lib.check(_lib.lib().lact_mfma_calibration(1024, 4000, ctypes.c_void_p(buf.data_ptr()),
                                                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        del buf

    if args.no_overlap:
        _lib.lib().lact_set_option(_lib.OPT_STREAM_OVERLAP, 0)
    if args.persistent_tiles is not None:
        _lib.lib().lact_set_option(_lib.OPT_PERSISTENT_TILES, args.persistent_tiles)
    if args.keep_preactivations is not None:
        _lib.lib().lact_set_option(_lib.OPT_KEEP_PREACTIVATIONS, args.keep_preactivations)
    for _ in range(args.warmup):
        step()
    # `repeats` timed regions of exactly `steps` steps each, every one bracketed by a device synchronisation; the
    # reported step time is the median region's (a region is a few tens of milliseconds: one scheduler hiccup on the
    # host would otherwise move the figure by percent).  All regions are listed in `ms_per_step_repeats`.
    reps_ms = [time_steps(step, args.steps) for _ in range(max(1, args.repeats))]
    ms_per_step = sorted(reps_ms)[len(reps_ms) // 2]
    tokens_per_s = B * L / (ms_per_step * 1e-3)
    flops = W["flops"]

    res = {
        "metric": "TTT-layer tokens/sec fwd+bwd at 760M shape, 1 GPU; MFMA util % of bf16 peak",
        "value": tokens_per_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (seeded N(0,1) q,k,v; L2-normalised q,k; random-init fast weights)",
        "config": {"workload": text, "tokens_per_step": B * L},
        "ms_per_step_repeats": reps_ms,
    }
    if flops is not None:
        op_tflops = flops / (ms_per_step * 1e-3) / 1e12
        res["config"]["algorithmic_gflop_per_step"] = flops / 1e9
        res["op_tflops"] = op_tflops
        res["op_frac_of_bf16_peak"] = op_tflops / PEAK_BF16_TFLOPS

    if args.config == "layer":
        res["metric"] = "LaCT layer tokens/sec fwd+bwd at 760M shape, 1 GPU (projections and window attention included)"
        W["no_attention"][0] = True      # the same steps without the attention branch
        for _ in range(2):
            step()
        res["ttt_branch_ms_per_step"] = time_steps(step, args.steps)
        W["no_attention"][0] = False

    traffic, step_traffic = load_traffic(args.config)
    # ---- per-kernel durations: the same K steps again with HIP events around every launch, on the stream
    #      the kernels run on (a second pass, so that the events do not perturb `value`)
    if not args.no_kernel_profile:
        rows, total_ms, dom_name, dom, avg_ms, achieved = kernel_profile(step, args.steps)
        res["roofline"] = {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                           "frac": achieved / PEAK_BF16_TFLOPS,
                           "traffic": traffic.get(dom_name),
                           "kernel": dom_name,
                           "avg_launch_ms": avg_ms, "launches_per_step": dom["launches"] / args.steps,
                           "share_of_kernel_time": dom["ms"] / total_ms}
        res["kernels"] = sorted(
            [{"kernel": r["kernel"], "site": r["site"], "launches_per_step": r["launches"] / args.steps,
              "ms_per_step": r["ms"] / args.steps,
              "tflops": (r["flops"] / (r["ms"] * 1e-3) / 1e12) if r["ms"] > 0 and r["flops"] > 0 else None}
             for r in rows], key=lambda r: -r["ms_per_step"])
        res["kernel_ms_per_step"] = total_ms / args.steps
    if step_traffic:
        gbps = step_traffic / (ms_per_step * 1e-3) / 1e9
        res["step_hbm"] = {"bytes_per_step": step_traffic, "achieved": gbps, "peak": PEAK_HBM_GBPS,
                           "unit": "GB/s", "frac": gbps / PEAK_HBM_GBPS,
                           "source": f"profiles/{args.config}_fwd_bwd_hbm_traffic_pmc.txt (FETCH_SIZE + WRITE_SIZE of every kernel of a step)"}

    # ---- CPU baseline: the oracle (a restatement of the reference's non-fused PyTorch op) on the host cores
    if not args.no_cpu_baseline and args.config != "layer":
        cb = b if args.config == "c1" else min(b, 4)   # bounded sample: the first `cb` heads, forward + backward
        if args.config != "c3":
            cpu = {n: W["inp"][n][:cb].clone().requires_grad_(True) for n in names}
            gc = W["go"][:cb].cpu()
        t0 = time.perf_counter()
        reps = 0
        while reps < 1 or (time.perf_counter() - t0 < 12.0 and reps < 40):
            if args.config == "c3":   # forward only, as the GPU leg
                with torch.no_grad():
                    O.fast_weight_swish_glu_weight_norm_mini_batch_apply(*[W["inp3"][n][:cb] for n in order], W["program"], 5,
                                                                         num=O.Numerics(autocast=True))
            else:
                for t in cpu.values():
                    t.grad = None
                o = O.block_causal_lact_swiglu(*[cpu[n] for n in order], C, True, cpu["momentum"], num=O.Numerics(autocast=True))
                o.backward(gc)
            reps += 1
        ct = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": (B * L) * (cb / b) / ct, "unit": "tokens/s", "cores": torch.get_num_threads(),
                               "kind": "port",
                               "sample": f"first {cb} of {b} heads of the same workload, {'fwd' if args.config == 'c3' else 'fwd+bwd'}, {reps} run(s), "
                                         f"{ct:.2f} s each; tokens scaled by {cb}/{b}; host has {os.cpu_count()} logical CPUs"}
    # ---- the other BASELINE configurations, timed the same way (median of three regions), each with its dominant kernel
    if args.config == "c1" and not args.no_other_configs:
        del W, step
        torch.cuda.empty_cache()
        res["other_configs"] = {}
        for cfg in ("c2", "c3", "c4"):
            Wc = build_workload(cfg)
            for _ in range(3):
                Wc["step"]()
            k = max(5, args.steps // 2)
            r3 = [time_steps(Wc["step"], k) for _ in range(3)]
            ms = sorted(r3)[1]
            tf = Wc["flops"] / (ms * 1e-3) / 1e12
            entry = {"workload": Wc["text"], "ms_per_step": ms, "tokens_per_s": Wc["B"] * Wc["L"] / (ms * 1e-3), "steps": k,
                     "ms_per_step_repeats": r3, "algorithmic_gflop_per_step": Wc["flops"] / 1e9, "op_tflops": tf,
                     "op_frac_of_bf16_peak": tf / PEAK_BF16_TFLOPS}
            if not args.no_kernel_profile:
                _, total_ms_c, dom_name_c, dom_c, avg_ms_c, achieved_c = kernel_profile(Wc["step"], k)
                entry["dominant_kernel"] = {"kernel": dom_name_c, "avg_launch_ms": avg_ms_c, "launches_per_step": dom_c["launches"] / k,
                                            "achieved_tflops": achieved_c, "frac": achieved_c / PEAK_BF16_TFLOPS,
                                            "share_of_kernel_time": dom_c["ms"] / total_ms_c}
            res["other_configs"][cfg] = entry
            del Wc
            torch.cuda.empty_cache()
    print(json.dumps(res))


if __name__ == "__main__":
    main()
