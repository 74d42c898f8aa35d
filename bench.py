"""Benchmark of the OLMoE MoE layer (64 experts, top-8, 2048 -> 1024 -> 2048, fp16) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--tokens N] [--mode auto|gemv|gemm]
    python bench.py --sweep            # the reference's table (bench/kernels.py) for 1..4096 tokens

A step is one call of kernels.moe_layer (router GEMM, route, sort, two grouped projections,
combine) on N tokens with every input already in HBM. The default workload is decode at 8
tokens, the configuration the reference's headline is quoted on. The metric is the reference's
(bench/kernels.py:52-55): bytes of expert weights of the experts that received a token, each
counted once, over the layer time. Successive steps rotate through several layers' weights, as
a decoder does, so that no step finds its weights in the 256 MB last-level cache.

Prints ONE JSON line. Besides the contract's fields (decode at 8 tokens, timed as a stream of
layer calls) it carries: the same figure by the reference's timing method (`*_event_median`); a
`roofline` object for the dominant kernel (the gate/up projection: two thirds of the weight
bytes) and one for the down projection, each timed per launch with events on the launch stream;
a `cpu_baseline` object: the per-expert PyTorch loop on this host's cores; `gpu_loop_fp16`: the
same loop on the GPU; and, in the default configuration, `decode_sizes` (1, 8, 16, 32 tokens),
`prefill` (4096 tokens on the MFMA tiles with its own `roofline`, bound "mfma"; 256 and 1024
tokens beside it) and `decode`: tokens/s of the full 16-layer model's greedy decode at batch 8 and
64 with the step's byte roofline, the MoE share and the top-1 check against the per-expert loop
(`--decode 8,64` prints more detail per batch)."""

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
SPIN_UP_MS = 50.0   # GPU kept busy this long before the warm-up steps (clock ramp of an idle GPU)
DECODE_SIZES = (1, 8, 16, 32)        # the decode configuration's token counts
PREFILL_SIZES = (256, 1024, 4096)    # the prefill configuration's token counts
TIMING = ("value, us_per_layer: K layer calls issued back to back between two synchronizes (a stream of layers, as a "
          "decoder issues them); *_event_median: one event pair around each single call, median of 20 after 3 "
          "warm-ups (the reference's bench/kernels.py:13-26), which adds the launch latency of an idle queue")


def measured_traffic(tokens, kernel):
    """HBM bytes per launch from a committed rocprofv3 FETCH_SIZE / WRITE_SIZE summary, or None.
    A summary under profiles/ ends with lines `bench-traffic: tokens=N kernel=NAME bytes=B file=SHA16`
    naming the kernel source it was taken from and the first 16 hex digits of its SHA-256; a figure
    whose source has changed since (or a missing summary) is not reported."""
    import glob
    import hashlib

    for path in glob.glob(os.path.join(ROOT, "profiles", "*.txt")):
        for line in open(path):
            if not line.startswith("bench-traffic:"):
                continue
            f = dict(x.split("=", 1) for x in line.split()[1:])
            if int(f["tokens"]) != tokens or f["kernel"] != kernel:
                continue
            name, sha = f["file"].split(":")
            src = os.path.join(ROOT, "switchyard_amd", "csrc", name)
            if os.path.exists(src) and hashlib.sha256(open(src, "rb").read()).hexdigest()[:16] == sha:
                return float(f["bytes"])
    return None


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


def spin_up(fn, ms=SPIN_UP_MS):
    """The clocks of an idle GPU take some milliseconds of work to come up (20 launches after an
    idle gap run several per cent slower than the same launches in a long stream), so the GPU is
    kept busy with the calls about to be timed; nothing of it is timed."""
    until = time.perf_counter() + ms / 1e3
    while time.perf_counter() < until:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()


def routed_ids(kernels, h, router):
    """Expert ids exactly as kernels.moe_layer routes them: up to OWN_ROUTER_MAX_TOKENS tokens the
    logits come from the library's own router kernel, above that from F.linear."""
    if h.shape[0] <= kernels.OWN_ROUTER_MAX_TOKENS:
        logits = kernels.ext().router_logits(h, router)
    else:
        logits = F.linear(h, router).contiguous()
    return kernels.ext().route(logits, TOPK, False)


def experts_used(kernels, h, layers):
    """Experts that receive a token, per layer (the numerator of the reference's metric)."""
    out = []
    for router, _, _ in layers:
        idx, _ = routed_ids(kernels, h, router)
        out.append(int((torch.bincount(idx.flatten().long(), minlength=E) > 0).sum()))
    return out


def time_layer(kernels, h, layers, mode, steps, warmup, spin=True):
    """One kernels.moe_layer call per step, rotating through `layers`: (ms per step of a stream
    of steps, median ms of event-timed single calls, used experts per layer)."""
    calls = [0]

    def step():
        router, gu, dn = layers[calls[0] % len(layers)]
        calls[0] += 1
        return kernels.moe_layer(h, router, gu, dn, TOPK, False, mode)

    if spin:
        spin_up(step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    calls[0] = 0
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_stream = (time.perf_counter() - t0) * 1e3 / steps
    calls[0] = 0
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    calls[0] = 0   # every event-timed call is layer 0, so its used-expert count is known exactly
    single = lambda: kernels.moe_layer(h, *layers[0], TOPK, False, mode)
    ms_event = statistics.median(event_times(single, 20))
    return ms_stream, ms_event


def layer_record(kernels, N, layers, mode, steps, warmup):
    """Layer time and both roofline fractions at N tokens."""
    h = hidden(N).to("cuda:0")
    used = experts_used(kernels, h, layers)
    ms_stream, ms_event = time_layer(kernels, h, layers, mode, steps, warmup)
    used_mean = sum(used[j % len(layers)] for j in range(steps)) / steps
    flops = N * TOPK * 6 * H * I
    gbs, gbs_ev = used_mean * EXPERT_BYTES / ms_stream / 1e6, used[0] * EXPERT_BYTES / ms_event / 1e6
    tf = flops / ms_stream / 1e9
    # the bytes a layer must move: the used experts' weights once, and per sorted row the gathered
    # row of h, act written and read, y written and read: M * (3 H + 2 I) * 2 B = M * 16 384 B here
    layer_bytes = used_mean * EXPERT_BYTES + N * TOPK * (3 * H + 2 * I) * 2
    by_bytes = {"bound": "hbm", "achieved": layer_bytes / ms_stream / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": layer_bytes / ms_stream / 1e6 / HBM_PEAK_GBS, "traffic": measured_traffic(N, "layer"),
                "kernel": "whole layer (front, sort, two projections, combine)", "us_per_launch": ms_stream * 1e3,
                "algorithmic_per_launch": layer_bytes,
                "bytes": "used experts' weights + N*k*(3H + 2I)*2 B of activations (gathered h rows, act and y written and read)"}
    return {"tokens": N, "mode": mode if mode != "auto" else kernels._auto(N, N * TOPK, E), "us_per_layer": ms_stream * 1e3,
            "roofline_bytes": by_bytes,
            "us_per_layer_event_median": ms_event * 1e3, "experts_used_mean": used_mean, "experts_used_layer0": used[0],
            "weight_GBps": gbs, "weight_GBps_event_median": gbs_ev, "frac_of_hbm_peak": gbs / HBM_PEAK_GBS,
            "frac_of_hbm_peak_event_median": gbs_ev / HBM_PEAK_GBS, "tflops": tf,
            "frac_of_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS,
            "binding_roofline": "mfma" if flops / (MFMA_F16_PEAK_TFLOPS * 1e12) > used_mean * EXPERT_BYTES / (HBM_PEAK_GBS * 1e9) else "hbm"}


def projection_times(kernels, N, layers, mode, reps, warmup):
    """The two grouped projections as the layer launches them, each timed per launch in a stream
    of launches of that kernel alone (events on the launch stream), rotating through the layers'
    weights. Returns (gate/up ms, down ms, used experts per layer, names of the two kernels).
    What moe_layer launches: on the weight-stream path up to 64 choices the gate/up stream that
    sorts the choices itself (sy_grouped_gemv_sorting) and a down projection without row scales
    (the combine applies the router weights); on the MFMA tiles sy_grouped_gemm, the down
    projection without row scales where the 256-row tile runs, with them on the smaller tiles."""
    dev = "cuda:0"
    h = hidden(N).to(dev)
    M = N * TOPK
    use_gemv = (mode if mode != "auto" else kernels._auto(N, M, E)) == "gemv"
    X = kernels.ext()
    sorting = use_gemv and M <= 64
    big_tile = not use_gemv and M >= 108 * E           # sy_gemm_rows_per_tile(M, E, K) == 256 for these shapes
    down_scaled = not use_gemv and not big_tile
    rot, used = [], []
    for router, gu, dn in layers:
        idx, w = routed_ids(kernels, h, router)
        counts, offsets, token, wsorted, pos_of = X.sort_by_expert(idx, w, E)
        used.append(int((counts > 0).sum()))
        rot.append((gu, dn, offsets, token, wsorted, idx, w))
    act = torch.randn(M, I, generator=torch.Generator().manual_seed(7)).mul_(0.3).half().to(dev)
    calls = [0]

    def gate_up():
        gu, _, off, tok, _, idx, w = rot[calls[0] % len(rot)]
        calls[0] += 1
        if sorting:
            return X.grouped_gemv_sorting(h, idx, w, gu)
        return X.grouped_gemv(h, tok, gu, off, M, True, None, N) if use_gemv else X.grouped_gemm(h, tok, gu, off, None, 0, M, True, None)

    def down():
        _, dn, off, _, ws, _, _ = rot[calls[0] % len(rot)]
        calls[0] += 1
        scale = ws if down_scaled else None
        return X.grouped_gemv(act, None, dn, off, M, False, scale, N) if use_gemv else X.grouped_gemm(act, None, dn, off, None, 0, M, False, scale)

    out = []
    for fn in (gate_up, down):
        spin_up(fn, 20.0)
        for _ in range(max(3, warmup)):
            fn()
        calls[0] = 0
        t = stream_times(fn, max(reps, 20), 10)
        out.append(sum(t) / len(t))
    if use_gemv:
        names = ("gemv_kernel<swiglu, sorts its choices> (gate/up projection, sy_grouped_gemv_sorting)" if sorting
                 else "gemv_kernel<swiglu> (gate/up projection)",
                 "gemv_kernel<no row scales> (down projection; the combine applies the router weights)"
                 + (" [up to 4 tokens the layer runs gemv_down_combine_kernel instead: down projection and combine in one launch]"
                    if N <= 4 else ""))
    else:
        tile = "gemm_stream_kernel, 256-row tile" if big_tile else "gemm_kernel, 64/128-row tile"
        names = (f"{tile} <swiglu> (gate/up projection)",
                 f"{tile} <{'row scales' if down_scaled else 'no row scales'}> (down projection"
                 + ("" if down_scaled else "; combine_kernel<weighted> applies the router weights") + ")")
    return out[0], out[1], used, use_gemv, names


def projection_rooflines(kernels, N, layers, mode, reps, warmup):
    """`roofline` objects of the gate/up projection (the dominant kernel) and of the down
    projection at N tokens, for the kernels the layer launches. Bound and algorithmic figure: below about 300 rows per expert the
    launch is a stream over the used experts' weights (bytes, against HBM peak), above it is
    bound by the MFMAs (flops, against dense fp16 peak)."""
    gu_ms, dn_ms, used, use_gemv, names = projection_times(kernels, N, layers, mode, reps, warmup)
    used_mean = sum(used) / len(used)
    M = N * TOPK
    out = []
    for name, ms, share, src in ((names[0], gu_ms, 2, "gate_up"), (names[1], dn_ms, 1, "down")):
        if use_gemv or M // E < 300:
            alg = used_mean * share * H * I * 2
            roof = {"bound": "hbm", "achieved": alg / ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s"}
        else:
            alg = M * share * 2 * H * I
            roof = {"bound": "mfma", "achieved": alg / ms / 1e9, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s"}
        roof["frac"] = roof["achieved"] / roof["peak"]
        roof["traffic"] = measured_traffic(N, ("gemv_" if use_gemv else "gemm_") + src)
        roof["kernel"] = name
        roof["us_per_launch"] = ms * 1e3
        roof["algorithmic_per_launch"] = alg
        out.append(roof)
    return out[0], out[1]


def library_batched_gemm(layers, N, reps=50):
    """What the vendor library's batched GEMM takes for the two projections of N tokens under
    perfectly even routing: torch.bmm over E problems of N*k/E rows each, every expert with its
    own weights of a rotated layer (so they stream from HBM as in the real launch), random fp16
    operands. No gather, no SwiGLU, no routing weights, no ragged experts: the same flops as
    `prefill.roofline` counts, on the easiest terms, as a measure of what this GPU sustains on
    this shape."""
    dev = layers[0][1].device
    n = N * TOPK // E
    g = torch.Generator().manual_seed(11)
    x = torch.randn(E, n, H, generator=g).half().to(dev)
    a = torch.randn(E, n, I, generator=g).mul_(0.3).half().to(dev)
    out = {"rows_per_expert": n, "what": "torch.bmm, E problems, each expert's own weights, no gather/SwiGLU/scale"}
    for name, lhs, pick, flops in (("gate_up", x, 1, 4.0), ("down", a, 2, 2.0)):
        calls = [0]

        def fn():
            w = layers[calls[0] % len(layers)][pick]
            calls[0] += 1
            return torch.bmm(lhs, w.transpose(1, 2))

        spin_up(fn, 20.0)
        t = stream_times(fn, reps, 10)
        ms = sum(t) / len(t)
        out[name + "_us"] = ms * 1e3
        out[name + "_frac_of_mfma_peak"] = E * n * flops * H * I / ms / 1e9 / MFMA_F16_PEAK_TFLOPS
    return out


def cpu_loop_baseline(h, router, gu, dn, used, reps=5, weights32=None, dtype=torch.float32):
    """The reference per-expert loop (switchyard/moe.py:34-42) restated in oracle/, on the host,
    fp32 (or fp16: weights and activations as the GPU has them), median of `reps` after 1 warm-up."""
    from oracle import moe_oracle as O

    if dtype == torch.float32:
        rf, gf, df = weights32 if weights32 is not None else (router.float(), gu.float(), dn.float())
        hf = h.float()
    else:
        hf, rf, gf, df = h, router, gu, dn
    idx, w = O.route(hf, rf, TOPK, False)
    O.experts_loop(hf, idx, w, gf, df)
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        O.experts_loop(hf, idx, w, gf, df)
        times.append(time.perf_counter() - t0)
    t = statistics.median(times)
    name = "fp32" if dtype == torch.float32 else "fp16"
    return {"value": used * EXPERT_BYTES / t / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle per-expert loop, {name} weights, {h.shape[0]} tokens, median of {reps} passes "
                      f"({t * 1e3:.1f} ms each) after 1 warm-up; os.cpu_count()={os.cpu_count()}",
            "us_per_layer": t * 1e6, "tokens": h.shape[0], "dtype": name,
            "tflops": h.shape[0] * TOPK * 6 * H * I / t / 1e12}


def cpu_baselines(cpu_layer, sizes, fp16_up_to=32):
    """The CPU loop at every token count of the metric: fp32 weights for all of them (median of 5,
    3 at 4096 tokens), fp16 too up to 32 tokens; the thread count is in every record."""
    from oracle import moe_oracle as O

    router, gu, dn = cpu_layer
    w32 = (router.float(), gu.float(), dn.float())
    out = {}
    for N in sizes:
        h = hidden(N)
        idx, _ = O.route(h.float(), w32[0], TOPK, False)
        used = int((torch.bincount(idx.flatten(), minlength=E) > 0).sum())
        out[str(N)] = cpu_loop_baseline(h, router, gu, dn, used, reps=3 if N >= 4096 else 5, weights32=w32)
        if N <= fp16_up_to:
            out[f"{N}_fp16"] = cpu_loop_baseline(h, router, gu, dn, used, reps=3, dtype=torch.float16)
    return out


def gpu_loop_baseline(layers, sizes=(1, 8, 32, 256, 1024, 4096)):
    """The reference's "loop" and "sorted loop" columns (bench/kernels.py:41-42): the per-expert
    PyTorch loop and the loop over sorted rows, in fp16 on the GPU, event-timed like the kernels
    (median of 5 after 1 warm-up), ms per layer."""
    from oracle import moe_oracle as O

    router, gu, dn = layers[0]
    out = {}
    for N in sizes:
        h = hidden(N).to("cuda:0")
        idx, w = O.route(h, router, TOPK, False)
        O.experts_loop(h, idx, w, gu, dn)
        O.experts_grouped(h, idx, w, gu, dn)
        torch.cuda.synchronize()
        out[str(N)] = {"ms_per_layer": statistics.median(event_times(lambda: O.experts_loop(h, idx, w, gu, dn), 5)),
                       "sorted_loop_ms_per_layer": statistics.median(event_times(lambda: O.experts_grouped(h, idx, w, gu, dn), 5))}
    return out


def decode_rates(batches=(8, 64), prompt_len=512, new_tokens=128):
    """The other half of the headline metric: greedy decode of the full OLMoE-1B-7B-shaped model
    (16 layers, random fp16 weights). Per batch size: tokens/s with the decode step on the
    library's kernels (HIP-graph replay of Decoder.step_fused), tokens/s of the configuration as
    written (attention in PyTorch operators, the MoE layers through the hook ->
    kernels.moe_layer; the step replayed as a graph as well), the bytes a step must read and the
    fraction of HBM peak that makes of the step time, the MoE layers' share of the step, and
    whether the first generated token is the top-1 of the same model with the per-expert
    PyTorch loop in the hook, for every row."""
    from oracle import moe_oracle as O
    from switchyard_amd import decoder as D
    from switchyard_amd import kernels

    dev = torch.device("cuda:0")
    s = D.OLMOE_1B_7B
    w = D.random_weights(s, device=dev, seed=0)
    cap = prompt_len + new_tokens + 8
    model = D.Decoder(s, w, max_positions=cap)
    as_written = D.Decoder(s, w, max_positions=cap, attention="torch")      # self.moe = the hook -> kernels.moe_layer

    def loop_moe(i, h):
        L = w["layers"][i]
        return O.moe_layer(h, L["router"], L["gate_up"], L["down"], s.top_k, s.norm_topk_prob)

    loop_model = D.Decoder(s, w, moe=loop_moe, max_positions=cap, attention="torch")
    layers = [(L["router"], L["gate_up"], L["down"]) for L in w["layers"]]
    attn_bytes = s.layers * (2 * s.heads + 2 * s.kv_heads) * s.head_dim * s.hidden * 2
    head_bytes = s.vocab * s.hidden * 2
    router_bytes = s.layers * s.experts * s.hidden * 2
    out = {"model": "OLMoE-1B-7B shape, 16 layers, random-init fp16", "prompt_len": prompt_len,
           "new_tokens": new_tokens,
           "step": "the configuration as written: attention in PyTorch operators, the MoE layers through the hook -> "
                   "kernels.moe_layer (HIP-graph replay of Decoder.step_static)",
           "fused_step": "beside it, not the stated configuration: HIP-graph replay of Decoder.step_fused, in which the "
                         "attention side runs on this library's kernels too",
           "bytes_per_step": "used experts' weights of 16 layers + attention, router and lm_head weights + the KV cache "
                             "at the mean length of the run; roofline_frac = bytes / 8 TB/s / step time"}
    for B in batches:
        prompts = torch.randint(3, s.vocab, (B, prompt_len), generator=torch.Generator().manual_seed(0)).tolist()
        tokens = torch.tensor(prompts, device=dev)
        model.generate(prompts, 4)
        torch.cuda.synchronize()
        tm = {}
        _, first = model.generate_graph(prompts, new_tokens + 1, return_first_logits=True, timings=tm)
        step_s = tm["decode_s"] / tm["decode_steps"]
        tw = {}
        _, first_w = as_written.generate_graph(prompts, new_tokens + 1, return_first_logits=True, timings=tw)
        # experts used per layer in a decode step: the routing of the first step's hidden states
        used = []

        def counting_moe(i, h):
            idx, _ = routed_ids(kernels, h, w["layers"][i]["router"])
            used.append(int((torch.bincount(idx.flatten().long(), minlength=s.experts) > 0).sum()))
            return kernels.moe_layer(h, *layers[i], s.top_k, s.norm_topk_prob)

        probe = D.Decoder(s, w, moe=counting_moe, max_positions=cap, attention="torch")
        cache = D.KVCache(s, B, prompt_len + 4, torch.float16, dev)
        nxt = probe.forward(tokens, cache)[:, -1].argmax(-1)
        del used[:]
        probe.forward(nxt[:, None], cache)
        kv_bytes = s.layers * B * 2 * s.kv_heads * s.head_dim * (prompt_len + new_tokens / 2) * 2
        step_bytes = sum(used) * EXPERT_BYTES + attn_bytes + router_bytes + head_bytes + kv_bytes
        del cache, probe
        # the MoE layers alone at this batch size: a stream of the 16 layers' calls
        hB = hidden(B).to(dev)
        moe_ms, _ = time_layer(kernels, hB, layers, "auto", 10 * s.layers, s.layers, spin=False)
        # the per-expert loop in the hook on the same prompts: the first token must be its top-1
        ref_first = loop_model.forward(tokens)[:, -1]
        agree = first.argmax(-1) == ref_first.argmax(-1)
        agree_w = first_w.argmax(-1) == ref_first.argmax(-1)
        written_s = tw["decode_s"] / tw["decode_steps"]
        out[f"b{B}"] = {"tok_per_s": B / written_s, "ms_per_step": written_s * 1e3,
                        "prefill_tok_per_s": B * prompt_len / tw["prefill_s"],
                        "experts_used_per_layer_mean": sum(used) / len(used), "bytes_per_step": step_bytes,
                        "roofline_tok_per_s": B * HBM_PEAK_GBS * 1e9 / step_bytes,
                        "roofline_frac": step_bytes / (HBM_PEAK_GBS * 1e9) / written_s,
                        "moe_ms_per_step": moe_ms * s.layers, "moe_share_of_step": moe_ms * s.layers / (written_s * 1e3),
                        "top1_rows_identical_to_loop_hook": int(agree_w.sum()), "rows": B,
                        "first_logits_max_abs_diff_vs_loop_hook": (first_w.float() - ref_first.float()).abs().max().item(),
                        "fused_step": {"tok_per_s": B / step_s, "ms_per_step": step_s * 1e3,
                                       "prefill_tok_per_s": B * prompt_len / tm["prefill_s"],
                                       "roofline_frac": step_bytes / (HBM_PEAK_GBS * 1e9) / step_s,
                                       "moe_share_of_step": moe_ms * s.layers / (step_s * 1e3),
                                       "top1_rows_identical_to_loop_hook": int(agree.sum()),
                                       "first_logits_max_abs_diff_vs_loop_hook":
                                           (first.float() - ref_first.float()).abs().max().item()}}
    return out


def run_default(args):
    from switchyard_amd import kernels

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    N = args.tokens
    cpu_layers = make_layers(args.layers)
    layers = [tuple(t.to(dev) for t in L) for L in cpu_layers]
    if args.operands == "zeros":
        # Same launches, same routing (the router keeps its values), expert weights all zero: the
        # kernels run the same instructions on operands that toggle nothing, which separates what
        # the schedule costs from what the chip's power management takes on random operands.
        layers = [(r, torch.zeros_like(g), torch.zeros_like(d)) for r, g, d in layers]
    h_cpu = hidden(N)
    h = h_cpu.to(dev)
    mode = args.mode

    # ---- the headline: exactly `steps` layer calls after `warmup`, in a stream
    used = experts_used(kernels, h, layers)
    ms_per_step, ev_med = time_layer(kernels, h, layers, mode, args.steps, args.warmup)
    used_mean = sum(used[j % len(layers)] for j in range(args.steps)) / args.steps
    value = used_mean * EXPERT_BYTES / (ms_per_step / 1e3) / 1e9
    value_ev = used[0] * EXPERT_BYTES / (ev_med / 1e3) / 1e9

    # ---- the dominant kernel of this size
    roof, roof_down = projection_rooflines(kernels, N, layers, mode, args.steps, args.warmup)

    whole = not args.no_cpu and N == 8 and mode == "auto"   # the default run reports the whole metric
    cpu = cpu_sizes = None
    if whole:
        cpu_sizes = cpu_baselines(cpu_layers[0], sorted(set(DECODE_SIZES + PREFILL_SIZES)))
        cpu = cpu_sizes[str(N)]
    elif not args.no_cpu:
        cpu = cpu_loop_baseline(h_cpu, *cpu_layers[0], used[0])
    sizes = prefill = gpu_loop = decode = None
    if whole:
        sizes = {str(n): layer_record(kernels, n, layers, "auto", 100, 10) for n in DECODE_SIZES}
        for n in DECODE_SIZES:   # the decode configuration names the weight-stream kernel: time it where "auto" prefers the tiles
            if sizes[str(n)]["mode"] != "gemv":
                sizes[f"{n}_gemv"] = layer_record(kernels, n, layers, "gemv", 100, 10)
        big = max(PREFILL_SIZES)
        prefill = layer_record(kernels, big, layers, "gemm", 50, 5)
        prefill["roofline"], prefill["down_projection"] = projection_rooflines(kernels, big, layers, "gemm", 100, 5)
        try:
            prefill["library_batched_gemm_even_routing"] = library_batched_gemm(layers, big)
        except Exception as exc:  # a comparison, not part of the metric
            prefill["library_batched_gemm_even_routing"] = {"error": f"{type(exc).__name__}: {exc}"}
        prefill["other_sizes"] = {str(n): layer_record(kernels, n, layers, "gemm", 50, 5) for n in PREFILL_SIZES if n != big}
        for rec in prefill["other_sizes"].values():   # these sizes are bound by the bytes the layer moves, not by the MFMAs
            rec["roofline"] = rec.pop("roofline_bytes")
        gpu_loop = gpu_loop_baseline(layers)
        n_layers = len(layers)
        del layers
        torch.cuda.empty_cache()
        try:
            decode = decode_rates()
        except Exception as exc:  # the layer figures above stand on their own
            decode = {"error": f"{type(exc).__name__}: {exc}"}
    else:
        n_layers = len(layers)

    line = {
        "metric": "OLMoE MoE-layer expert-weight GB/s", "value": value, "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": value / T4_WEIGHT_GBS_AT_8 if N == 8 else None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"olmoe_moe_layer_{'decode' if N <= 64 else 'prefill'}_{N}tok", "tokens": N,
                   "experts": E, "top_k": TOPK, "hidden": H, "expert_width": I, "mode": mode,
                   "layers_rotated": n_layers, "experts_used_mean": used_mean, "spin_up_ms": SPIN_UP_MS,
                   **({"operands": "zero expert weights: NOT the benchmark"} if args.operands != "random" else {})},
        "timing": TIMING,
        "us_per_layer": ms_per_step * 1e3, "frac_of_hbm_peak": value / HBM_PEAK_GBS,
        "value_event_median": value_ev, "us_per_layer_event_median": ev_med * 1e3,
        "frac_of_hbm_peak_event_median": value_ev / HBM_PEAK_GBS,
        "tflops": N * TOPK * 6 * H * I / (ms_per_step / 1e3) / 1e12,
        "vs_baseline_note": "published figure is the reference's on one Tesla T4 (320 GB/s), event-timed single calls; "
                            "`value` is the stream-of-layers figure, `value_event_median` the like-for-like one",
        "gpu": torch.cuda.get_device_name(0),
        "roofline": roof, "down_projection": roof_down, "cpu_baseline": cpu, "cpu_baseline_sizes": cpu_sizes,
        "gpu_loop_fp16": gpu_loop,
        "decode_sizes": sizes, "prefill": prefill, "decode": decode,
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
    ap.add_argument("--operands", default="random", choices=["random", "zeros"],
                    help='"zeros": expert weights of zero (a power experiment, with --no-cpu; not the benchmark)')
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
