"""Benchmark of the OLMoE MoE layer (64 experts, top-8, 2048 -> 1024 -> 2048, fp16) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--tokens N] [--mode auto|gemv|gemm]
    python bench.py --sweep            # the reference's table (bench/kernels.py) for 1..4096 tokens

A step is one call of kernels.moe_layer (router GEMM, route, sort, two grouped projections,
combine) on N tokens with every input already in HBM. The default workload is decode at 8
tokens, the configuration the reference's headline is quoted on. The metric is the reference's
(bench/kernels.py:52-55): bytes of expert weights of the experts that received a token, each
counted once, over the layer time. Successive steps rotate through several layers' weights, as
a decoder does, so that no step finds its weights in the 256 MB last-level cache.

Prints ONE JSON line with the metric, a `roofline` object for the dominant kernel (the
gate/up projection: two thirds of the weight bytes), timed per launch with events on the
launch stream, a `cpu_baseline` object: the per-expert PyTorch loop on this host's cores, and (in
the default configuration) a `decode` object: tokens/s of the full 16-layer model's greedy decode
at batch 8 and 64, the second half of the reference's headline (`--decode 8,64` gives the detailed
lines with the comparison against the per-expert loop in the hook)."""

import argparse
import json
import os
import statistics
import sys
import time

import torch
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

E, TOPK, H, I = 64, 8, 2048, 1024
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, published
EXPERT_BYTES = 3 * H * I * 2   # gate + up + down of one expert, fp16
T4_WEIGHT_GBS_AT_8 = 232.98490131032196  # the reference's published figure for this metric (Tesla T4)

# HBM bytes per launch of the gate/up projection from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (scaled by a plain copy kernel of known size: 2.0 and 1.0), keyed by token count; the run is
# summarised in profiles/decode_8tok_gemv_hbm_traffic.txt (8 tokens, the weight-stream kernel) and
# profiles/prefill_4096tok_gemm.txt (4096 tokens, the 256-row MFMA tiles). Token counts not measured: None.
MEASURED_TRAFFIC_BYTES = {8: 342.1e6, 4096: 869.7e6}
SPIN_UP_MS = 50.0   # GPU kept busy this long before the warm-up steps (clock ramp of an idle GPU)


def make_layers(n_layers, seed=0):
    import cases

    layers = []
    for j in range(n_layers):
        _, router, gu, dn = cases.layer(1, seed=seed + j)
        layers.append((router, gu, dn))
    return layers


def hidden(N, seed=0):
    return torch.randn(N, H, generator=torch.Generator().manual_seed(seed + 1000 + N)).half()


def event_times(fn, reps):
    """Per-call GPU time in ms, one event pair per call on the current stream (the GPU idles
    between calls, so launch latency is included: the reference's bench/kernels.py method)."""
    out = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        out.append(a.elapsed_time(b))
    return out


def stream_times(fn, reps, group=10):
    """Per-launch GPU time in ms for back-to-back launches: an event is recorded in the stream
    after every `group` launches and all are read after one synchronize, so the queue never
    drains; an interval is `group` launches and one event (recording an event between every two
    launches adds about 2 us to each: 59.9 us where the profiler's kernel trace says 57.7)."""
    n = max(1, reps // group)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
    ev[0].record()
    for i in range(n):
        for _ in range(group):
            fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    return [ev[i].elapsed_time(ev[i + 1]) / group for i in range(n)]


def cpu_loop_baseline(h, router, gu, dn, used, reps=5):
    """The reference per-expert loop (switchyard/moe.py:34-42) restated in oracle/, fp32, on the host."""
    from oracle import moe_oracle as O

    hf, rf, gf, df = h.float(), router.float(), gu.float(), dn.float()
    idx, w = O.route(hf, rf, TOPK, False)
    O.experts_loop(hf, idx, w, gf, df)
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        O.experts_loop(hf, idx, w, gf, df)
        times.append(time.perf_counter() - t0)
    t = statistics.median(times)
    return {"value": used * EXPERT_BYTES / t / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle per-expert loop, fp32 weights, {h.shape[0]} tokens, median of {reps} passes "
                      f"({t * 1e3:.1f} ms each) after 1 warm-up; os.cpu_count()={os.cpu_count()}",
            "us_per_layer": t * 1e6}


def decode_rates(batches=(8, 64), prompt_len=512, new_tokens=128):
    """The other half of the headline metric: greedy decode of the full OLMoE-1B-7B-shaped model
    (16 layers, random fp16 weights), HIP-graph replay of the step, tokens/s per batch size."""
    from switchyard_amd import decoder as D

    s = D.OLMOE_1B_7B
    w = D.random_weights(s, device="cuda:0", seed=0)
    model = D.Decoder(s, w, max_positions=prompt_len + new_tokens + 8)
    out = {"model": "OLMoE-1B-7B shape, 16 layers, random-init fp16", "prompt_len": prompt_len,
           "new_tokens": new_tokens, "step": "HIP-graph replay of Decoder.step_fused"}
    for B in batches:
        prompts = torch.randint(3, s.vocab, (B, prompt_len), generator=torch.Generator().manual_seed(0)).tolist()
        model.generate(prompts, 4)
        torch.cuda.synchronize()
        tm = {}
        model.generate_graph(prompts, new_tokens + 1, timings=tm)
        out[f"b{B}"] = {"tok_per_s": B * tm["decode_steps"] / tm["decode_s"],
                        "ms_per_step": tm["decode_s"] * 1e3 / tm["decode_steps"],
                        "prefill_tok_per_s": B * prompt_len / tm["prefill_s"]}
    return out


def run_default(args):
    from switchyard_amd import kernels

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    N = args.tokens
    cpu_layers = make_layers(args.layers)
    layers = [tuple(t.to(dev) for t in L) for L in cpu_layers]
    h_cpu = hidden(N)
    h = h_cpu.to(dev)
    mode = args.mode

    def step(j):
        router, gu, dn = layers[j % len(layers)]
        return kernels.moe_layer(h, router, gu, dn, TOPK, False, mode)

    # experts that receive a token, per layer (the metric's numerator)
    used = []
    for router, gu, dn in layers:
        idx, _ = kernels.route(h, router, TOPK, False)
        used.append(int((torch.bincount(idx.flatten().long(), minlength=E) > 0).sum()))

    # The clocks of an idle GPU take some milliseconds of work to come up (20 launches after an
    # idle gap run several per cent slower than the same launches in a long stream), so the GPU
    # is kept busy for SPIN_UP_MS with the same layer calls before the warm-up steps; nothing of
    # it is timed.
    spin_until = time.perf_counter() + SPIN_UP_MS / 1e3
    while time.perf_counter() < spin_until:
        for j in range(10):
            step(j)
        torch.cuda.synchronize()
    for j in range(args.warmup):
        step(j)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for j in range(args.steps):
        step(j)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    used_mean = sum(used[j % len(layers)] for j in range(args.steps)) / args.steps
    value = used_mean * EXPERT_BYTES / (ms_per_step / 1e3) / 1e9

    # the same layer call timed with one event pair per call (the reference's method, median)
    ev = event_times(lambda: step(0), 20)
    ev_med = statistics.median(ev)

    # dominant kernel: the gate/up projection, one event pair per launch on the launch stream
    router, gu, dn = layers[0]
    idx, w = kernels.route(h, router, TOPK, False)
    counts, offsets, token, wsorted, pos_of = kernels.ext().sort_by_expert(idx, w, E)
    M = idx.numel()
    use_gemv = (mode if mode != "auto" else kernels._auto(N, M, E)) == "gemv"
    rot = []
    for r_, g_, d_ in layers:
        i_, w_ = kernels.route(h, r_, TOPK, False)
        s_ = kernels.ext().sort_by_expert(i_, w_, E)
        rot.append((g_, s_[1], s_[2]))
    calls = [0]
    n_layers_rot = len(layers)

    def gate_up():
        g_, off_, tok_ = rot[calls[0] % len(rot)]
        calls[0] += 1
        if use_gemv:
            return kernels.ext().grouped_gemv(h, tok_, g_, off_, M, True, None, N)
        return kernels.ext().grouped_gemm(h, tok_, g_, off_, None, 0, M, True, None)

    for _ in range(max(3, args.warmup)):
        gate_up()
    calls[0] = 0
    group = 10
    kt = stream_times(gate_up, max(args.steps, 20), group)
    k_ms = sum(kt) / len(kt)
    launches = len(kt) * group
    used_k = sum(used[j % n_layers_rot] for j in range(launches)) / launches
    if use_gemv or M // E < 300:
        alg = used_k * 2 * H * I * 2                      # gate and up rows of every used expert, once
        roof = {"bound": "hbm", "achieved": alg / (k_ms / 1e3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    else:
        alg = M * 4 * H * I                                # 2 * rows * 2I * H flops
        roof = {"bound": "mfma", "achieved": alg / (k_ms / 1e3) / 1e12, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["traffic"] = MEASURED_TRAFFIC_BYTES.get(N)
    roof["kernel"] = "gemv_kernel<swiglu> (gate/up projection)" if use_gemv else "grouped_gemm<swiglu> (gate/up projection)"
    roof["us_per_launch"] = k_ms * 1e3
    roof["algorithmic_per_launch"] = alg

    cpu = None if args.no_cpu else cpu_loop_baseline(h_cpu, *cpu_layers[0], used[0])
    n_layers = len(layers)
    decode = None
    if not args.no_cpu and N == 8 and mode == "auto":   # the default run reports the whole metric
        del layers, rot, router, gu, dn
        torch.cuda.empty_cache()
        try:
            decode = decode_rates()
        except Exception as exc:  # the layer figures above stand on their own
            decode = {"error": f"{type(exc).__name__}: {exc}"}

    line = {
        "metric": "OLMoE MoE-layer expert-weight GB/s", "value": value, "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": value / T4_WEIGHT_GBS_AT_8 if N == 8 else None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"olmoe_moe_layer_{'decode' if N <= 64 else 'prefill'}_{N}tok", "tokens": N,
                   "experts": E, "top_k": TOPK, "hidden": H, "expert_width": I, "mode": mode,
                   "layers_rotated": n_layers, "experts_used_mean": used_mean, "spin_up_ms": SPIN_UP_MS},
        "us_per_layer": ms_per_step * 1e3, "us_per_layer_event_median": ev_med * 1e3,
        "frac_of_hbm_peak": value / HBM_PEAK_GBS,
        "tflops": N * TOPK * 6 * H * I / (ms_per_step / 1e3) / 1e12,
        "vs_baseline_note": "published figure is the reference's on one Tesla T4 (320 GB/s)",
        "gpu": torch.cuda.get_device_name(0),
        "roofline": roof, "cpu_baseline": cpu, "decode": decode,
    }
    print(json.dumps(line), flush=True)


def run_sweep(args):
    """One JSON line per token count: the per-expert loop and the sorted loop in torch on the
    GPU (the reference's columns), the kernels in auto / gemv / gemm, errors, GB/s and TFLOP/s."""
    from oracle import moe_oracle as O
    from switchyard_amd import kernels

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    layers = [tuple(t.to(dev) for t in L) for L in make_layers(args.layers)]
    router, gu, dn = layers[0]
    sizes = [int(x) for x in args.sweep.split(",")] if args.sweep != "all" else [1, 8, 16, 32, 64, 128, 256, 512, 1024, 2048, 4096]

    def med(fn, reps=20, warm=3):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        return statistics.median(event_times(fn, reps))

    print(json.dumps({"bench": "moe_layer_sweep", "gpu": torch.cuda.get_device_name(0), "experts": E, "top_k": TOPK,
                      "hidden": H, "expert_width": I, "layers_rotated": len(layers)}), flush=True)
    for N in sizes:
        h = hidden(N).to(dev)
        idx, w = O.route(h, router, TOPK, False)
        j = [0]

        def rotating(mode):
            def fn():
                r_, g_, d_ = layers[j[0] % len(layers)]
                j[0] += 1
                return kernels.moe_layer(h, r_, g_, d_, TOPK, False, mode)
            return fn

        rec = {"tokens": N}
        # the clocks of a GPU that sat idle while this size was set up need work to come back up
        # (the first column measured would otherwise read several per cent slower than the others)
        spin, spin_until = rotating("auto"), time.perf_counter() + SPIN_UP_MS / 1e3
        while time.perf_counter() < spin_until:
            for _ in range(10):
                spin()
            torch.cuda.synchronize()
        rec["auto_ms"] = med(rotating("auto"))
        rec["gemv_ms"] = med(rotating("gemv")) if N <= 1024 else None
        rec["gemm_ms"] = med(rotating("gemm"))
        if not args.no_loops:
            rec["loop_ms"] = med(lambda: O.experts_loop(h, idx, w, gu, dn), reps=5, warm=1)
            rec["sorted_loop_ms"] = med(lambda: O.experts_grouped(h, idx, w, gu, dn), reps=5, warm=1)
        want = O.experts_loop(h.float(), idx, w.float(), gu.float(), dn.float())
        rec["max_err_auto"] = (kernels.moe_layer(h, router, gu, dn, TOPK, False).float() - want).abs().max().item()
        rec["max_err_fp16_loop"] = (O.experts_loop(h, idx, w, gu, dn).float() - want).abs().max().item()
        cnt = torch.bincount(idx.flatten(), minlength=E)
        used = int((cnt > 0).sum())
        rec["max_rows_per_expert"], rec["experts_used"] = int(cnt.max()), used
        best = min(x for x in (rec["auto_ms"], rec["gemv_ms"], rec["gemm_ms"]) if x)
        rec["weight_GBps_auto"] = used * EXPERT_BYTES / (rec["auto_ms"] / 1e3) / 1e9
        rec["weight_GBps_best"] = used * EXPERT_BYTES / (best / 1e3) / 1e9
        rec["tflops_auto"] = N * TOPK * 6 * H * I / (rec["auto_ms"] / 1e3) / 1e12
        rec["frac_hbm"] = rec["weight_GBps_auto"] / HBM_PEAK_GBS
        rec["frac_mfma"] = rec["tflops_auto"] / MFMA_F16_PEAK_TFLOPS
        print(json.dumps(rec), flush=True)


def run_decode(args):
    """Full OLMoE-1B-7B-shaped model (16 layers, random-init fp16, ~14 GB), greedy decode of
    `--new-tokens` tokens from random prompts of `--prompt-len` tokens; attention in PyTorch,
    MoE layers through the hook. One JSON line per batch size."""
    from oracle import moe_oracle as O
    from switchyard_amd import decoder as D

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.checkpoint:
        from switchyard_amd import checkpoint as C
        s, _ = C.shape_from_config(args.checkpoint)
        w = C.load(args.checkpoint, s, dtype=torch.float16, device=dev)
        name = f"checkpoint {args.checkpoint}, {s.layers} layers, fp16"
    else:
        s = D.OLMOE_1B_7B
        w = D.random_weights(s, device=dev, seed=0)
        name = "OLMoE-1B-7B shape, 16 layers, random-init fp16"
    model = D.Decoder(s, w, max_positions=args.prompt_len + args.new_tokens + 8)

    def loop_moe(i, h):
        L = w["layers"][i]
        return O.moe_layer(h, L["router"], L["gate_up"], L["down"], s.top_k, s.norm_topk_prob)

    loop_model = D.Decoder(s, w, moe=loop_moe, max_positions=args.prompt_len + args.new_tokens + 8)
    for B in [int(x) for x in args.decode.split(",")]:
        g = torch.Generator().manual_seed(0)
        prompts = torch.randint(3, s.vocab, (B, args.prompt_len), generator=g).tolist()
        tokens = torch.tensor(prompts, device=dev)
        # one untimed generation warms every kernel; then the decode step is captured in a HIP
        # graph and replayed once per token (prefill and replay loop timed separately)
        model.generate(prompts, 4)
        torch.cuda.synchronize()
        tm = {}
        graph_tokens, first = model.generate_graph(prompts, args.new_tokens + 1, return_first_logits=True, timings=tm)
        t_prefill, t_decode, steps = tm["prefill_s"], tm["decode_s"], tm["decode_steps"]
        if args.graph_only:   # profiling runs: nothing but the prefill and the replayed steps
            print(json.dumps({"bench": "decode", "batch": B, "prompt_len": args.prompt_len, "new_tokens": steps,
                              "decode_tok_per_s": B * steps / t_decode, "ms_per_step": t_decode * 1e3 / steps,
                              "prefill_ms": t_prefill * 1e3, "model": name}), flush=True)
            continue
        # for comparison: the step on PyTorch operators (attention side) around the MoE kernels,
        # driven from Python one launch at a time, fewer tokens
        cache = D.KVCache(s, B, args.prompt_len + 16, torch.float16, dev)
        logits = model.forward(tokens, cache)[:, -1]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(16):
            logits = model.forward(logits.argmax(-1)[:, None], cache)[:, -1]
        torch.cuda.synchronize()
        t_eager = (time.perf_counter() - t0) / 16
        # the same prompts through the per-expert loop hook: first-token logits must agree on the top-1
        ref_first = loop_model.forward(tokens)[:, -1]
        agree = first.argmax(-1) == ref_first.argmax(-1)
        top2 = ref_first.float().topk(2, dim=-1).values
        margin = (top2[:, 0] - top2[:, 1])
        rec = {"bench": "decode", "batch": B, "prompt_len": args.prompt_len, "new_tokens": steps,
               "decode_tok_per_s": B * steps / t_decode, "ms_per_step": t_decode * 1e3 / steps,
               "pytorch_attention_eager_ms_per_step": t_eager * 1e3, "pytorch_attention_eager_tok_per_s": B / t_eager,
               "prefill_tok_per_s": B * args.prompt_len / t_prefill, "prefill_ms": t_prefill * 1e3,
               "top1_rows_identical_to_loop_hook": int(agree.sum()), "rows": B,
               "largest_loop_hook_margin_where_top1_differs": float(margin[~agree].max()) if (~agree).any() else 0.0,
               "first_logits_max_abs_diff": (first.float() - ref_first.float()).abs().max().item(),
               "model": name, "gpu": torch.cuda.get_device_name(0)}
        if args.decode_loop_steps:
            cache = D.KVCache(s, B, args.prompt_len + args.decode_loop_steps, torch.float16, dev)
            logits = loop_model.forward(tokens, cache)[:, -1]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.decode_loop_steps):
                logits = loop_model.forward(logits.argmax(-1)[:, None], cache)[:, -1]
            torch.cuda.synchronize()
            rec["loop_hook_decode_tok_per_s"] = B * args.decode_loop_steps / (time.perf_counter() - t0)
        print(json.dumps(rec), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--tokens", type=int, default=8)
    ap.add_argument("--mode", default="auto", choices=["auto", "gemv", "gemm"])
    ap.add_argument("--layers", type=int, default=4, help="distinct layers' weights to rotate through")
    ap.add_argument("--sweep", default=None, help='"all" or a comma list of token counts')
    ap.add_argument("--no-loops", action="store_true", help="sweep: skip the torch per-expert loops")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run a plain 512 MiB device copy 5 times (a kernel of known traffic, to scale "
                         "rocprofv3's FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--no-cpu", action="store_true",
                    help="skip the CPU baseline and the full-model decode legs (profiling runs)")
    ap.add_argument("--decode", default=None, help='full-model greedy decode at these batch sizes, e.g. "8,64"')
    ap.add_argument("--checkpoint", default=None,
                    help="decode: an OLMoE checkpoint directory (config.json + safetensors) instead of random weights")
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--new-tokens", type=int, default=128)
    ap.add_argument("--graph-only", action="store_true",
                    help="decode: only the prefill and the graph-replayed steps (profiling runs)")
    ap.add_argument("--decode-loop-steps", type=int, default=8,
                    help="decode steps to time with the per-expert loop in the hook (0: skip)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus must be 1 (no multi-GPU figure is produced)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    with torch.no_grad():
        if args.calibrate_copy:
            src = torch.empty(512 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
            dst = torch.empty_like(src)
            for _ in range(5):
                dst.copy_(src)
            torch.cuda.synchronize()
            del src, dst
        if args.decode:
            run_decode(args)
        elif args.sweep:
            run_sweep(args)
        else:
            run_default(args)


if __name__ == "__main__":
    main()
