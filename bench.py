#!/usr/bin/env python3
"""Benchmark of the BitStack compressed-linear forward on one MI355X.

Workload ("decode GEMV sweep", the second configuration of the baseline):
Llama-3.1-8B linear shapes (out x in) 4096x4096, 1024x4096, 14336x4096,
4096x14336; blocks loaded I in {1, 2, 4, 8, 16}; rank 16; fp16; seeded
synthetic signs / factors / activations.  One STEP is one pass over all 20
(shape, I) layers at one token (T = 1) through the library's fused forward
(C ABI bs_forward), each layer with its own buffers (586 MB per pass, more
than the 256 MB Infinity Cache, so every pass streams from HBM).

The headline value is the whole-pass throughput in algorithmic GB/s:
sum over layers of I * (M*N/8 + 2*k*(M+N)) + 2*T*(N+M) bytes, divided by the
wall time of the timed region (inputs resident in HBM, launches back to back,
synchronised on both sides).

Extra objects on the same JSON line:
  roofline      the packed-sign GEMV kernel pair (contraction + partial-sum
                reduce) against the 8 TB/s HBM peak: algorithmic bytes per
                forward / HIP-event time per forward, averaged over the timed
                region (events recorded on the stream the kernels run on).
  cpu_baseline  the reference's CPU path (level 0) restated in torch-CPU ops,
                timed on this host on one pass of the same sweep.
  t2, t4, t16, prefill   the same sweep at 2, 4 and 16 tokens, and the prefill configuration
                (I = 8, T in {16, 64, 128, 512, 2048}) as useful TFLOP/s.
  decode_8b     tokens/s of a random-init Llama-3.1-8B-shape decode loop built
                around the same forward (batch 1, 256 greedy tokens).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
# Time one SIMD needs per MFMA when it issues nothing else, measured on this part with a loop of independent MFMAs at
# two waves per SIMD (the shader clock settles near 1.8 GHz under such a load, so cycle counts at the 2.4 GHz peak clock
# would flatter the kernel): v_mfma_scale_f32_16x16x128_f8f6f4 (fp6 x fp4) 10.8 ns, v_mfma_f32_16x16x32_f16 8.8 ns.
MFMA_MX_NS = 10.8
MFMA_F16_NS = 8.8
SHAPES = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)]
BLOCKS = [1, 2, 4, 8, 16]
PREFILL_T = [16, 64, 128, 512, 2048]
PREFILL_WARM_MS = 60.0      # untimed load in front of every prefill timing (clock recovery after a pause)
SIDE_WARM_MS = 30.0         # the same in front of the 2-, 4- and 16-token side measurements


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the T=4 and prefill side measurements")
    ap.add_argument("--only", choices=["decode_8b", "decode_70b", "prefill", "one_layer", "scoring", "copy", "sweep_tokens"], default=None,
                    help="run just this side measurement and print its object (for profiling one path)")
    ap.add_argument("--batch", type=int, default=8, help="sequences decoded in lock step by --only decode_70b (1..48)")
    ap.add_argument("--prompt-len", type=int, default=2048, help="prompt tokens per sequence of --only decode_70b")
    ap.add_argument("--tokens", type=int, default=2, help="tokens per forward of --only sweep_tokens (the 20-layer sweep at that count)")
    ap.add_argument("--layer", default="14336x4096x16x1",
                    help="with --only one_layer: out x in x blocks x tokens of the single layer to run (counter runs)")
    ap.add_argument("--decode-kernel", choices=["auto", "f16", "mx"], default="auto",
                    help="with --only sweep_tokens / one_layer: force the fp16 or the block-scaled decode kernel (A/B timing)")
    ap.add_argument("--detail", default=None, help="write per-layer timings to this JSON file")
    return ap.parse_args()


class Layer:
    def __init__(self, M, N, I, T, seed, dev):
        import torch
        from bitstack_amd.utils.synthetic import synthetic_layer, algorithmic_bytes
        self.M, self.N, self.I, self.T = M, N, I, T
        self.q, self.u, self.vt, self.x = synthetic_layer(M, N, I, T, seed=seed, device=dev)
        self.y = torch.empty((T, M), dtype=torch.float16, device=dev)
        self.bytes = algorithmic_bytes(I, M, N, T)


def make_forward(L, lib, ws, stream):
    """Bind one bs_forward call (C ABI, ctypes) with all arguments resolved."""
    from bitstack_amd import _lib
    args = (_lib.ptr(L.q), _lib.ptr(L.u), _lib.ptr(L.vt), _lib.ptr(L.x), None, _lib.ptr(L.y),
            L.I, L.M, L.N, 16, L.T, _lib.ptr(ws), ws.numel(), stream)

    def run():
        st = lib.bs_forward(*args)
        if st != 0:
            raise RuntimeError(f"bs_forward status {st}: {_lib.error_string(st)}")
    return run


def cpu_baseline(layers_cpu, runs=5):
    """The T=1 sweep restricted to `layers_cpu` through the level-0 restatement on the host: one
    warm-up forward, then per layer the median of `runs` timed forwards."""
    import statistics
    import torch
    from oracle import torch_l0
    threads = os.cpu_count() or 1
    # the GPU box exposes 16 cores to this job whatever cpu_count() says
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    torch.set_num_threads(threads)
    tot_b, tot_t, wall0 = 0, 0.0, time.perf_counter()
    torch_l0.forward_l0(*layers_cpu[0][:4])          # warm-up
    for (q, u, vt, x, nbytes) in layers_cpu:
        ts = []
        for _ in range(runs):
            t = time.perf_counter()
            torch_l0.forward_l0(q, u, vt, x)
            ts.append(time.perf_counter() - t)
        tot_t += statistics.median(ts)
        tot_b += nbytes
    return {"value": round(tot_b / tot_t / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"the T=1 sweep restricted to blocks {{1,2}} on all four shapes ({len(layers_cpu)} layers, "
                      f"{tot_b / 1e6:.0f} MB algorithmic) through the level-0 torch-CPU restatement; per layer the median of "
                      f"{runs} forwards after one warm-up ({time.perf_counter() - wall0:.1f} s of CPU time in all)",
            "seconds_per_pass_of_the_sample": round(tot_t, 2)}


def e2e_decode_70b(torch, dev, batch=8, prompt_len=2048, new_tokens=128):
    """Random-init Llama-3.1-70B-shape model, about 30 GB of weights, `batch` sequences in
    lock step: the prompt in one pass (every linear sees batch * prompt_len tokens: rebuild +
    dense kernels; causal attention is torch's), then greedy decode (every linear sees `batch`
    tokens: from five on that is the strip kernel, weight patches rebuilt in registers and
    multiplied at once), one HIP-graph replay per step."""
    from bitstack_amd.utils.llama_decode import LLAMA_70B, SyntheticLlamaDecoder, synthetic_compression_config
    cfg, total = synthetic_compression_config(LLAMA_70B, 30e9, lo=1, hi=8)
    model = SyntheticLlamaDecoder(LLAMA_70B, cfg, prompt_len + new_tokens + 8, dev, batch=batch)
    prompt = torch.randint(0, LLAMA_70B.vocab, (batch, prompt_len), generator=torch.Generator().manual_seed(0)).to(dev)
    model.prefill(prompt[:, :min(prompt_len, 64)])          # warm-up: workspaces, kernel attributes
    model.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    model.prefill(prompt)
    torch.cuda.synchronize()
    dt_prefill = time.perf_counter() - t0
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        model.step_fused()                                  # warm-up of the decode step outside capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        model.step_fused()
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(new_tokens):
        graph.replay()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    wbytes = model.weight_bytes()
    blocks = list(cfg.values())
    s = LLAMA_70B
    per_tok = 2.0 * sum(m * n for (m, n) in (s.proj_shape(p) for p in
                        ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
                         "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj"))) * s.layers
    return {"tok_s": round(batch * new_tokens / dt, 1), "ms_per_step": round(dt / new_tokens * 1e3, 3), "batch": batch,
            "prefill_s": round(dt_prefill, 3), "prefill_tok_s": round(batch * prompt_len / dt_prefill, 1),
            "prefill_linear_tflops": round(per_tok * batch * prompt_len / dt_prefill / 1e12, 1),
            "weight_GB": round(wbytes / 1e9, 2), "blocks_per_linear_mean": round(sum(blocks) / len(blocks), 2),
            "hbm_roofline_tok_s": round(batch * 8e12 / wbytes, 1),
            "non_path_ops": "the prompt pass runs causal attention through torch SDPA and RoPE through torch ops; "
                            "the decode steps run the library's own attention kernel",
            "config": f"80 layers, hidden 8192, inter 28672, 64Q/8KV, vocab 128256, batch {batch}, {prompt_len}-token prompt in one "
                      f"pass, {new_tokens} greedy tokens per sequence, fused step, one HIP-graph replay per step"}


def scoring_eval(torch, dev, sequences=8, seqlen=2048, blocks=4):
    """One perplexity evaluation of the importance-scoring loop on the 8B shape: every linear
    with `blocks` blocks, `sequences` calibration sequences of `seqlen` random token ids through
    the one-pass forward (rebuild + dense kernels) and a cross entropy over all positions.  The
    loop itself is one such evaluation per (bit level, linear)."""
    from bitstack_amd.utils.llama_decode import LLAMA_8B, PROJ, SyntheticLlamaDecoder
    from bitstack_amd.utils import scoring
    cfg = {f"layer.{L}.{p}": blocks for L in range(LLAMA_8B.layers) for p in PROJ}
    model = SyntheticLlamaDecoder(LLAMA_8B, cfg, seqlen, dev, batch=4)
    ids = torch.randint(0, LLAMA_8B.vocab, (sequences, seqlen), generator=torch.Generator().manual_seed(0))
    scoring.eval_ppl(model, ids[:4])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ppl = scoring.eval_ppl(model, ids)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    # the loop resumes every evaluation at its linear's layer: time it for the first, the middle
    # and the last decoder layer (inputs of all layers kept from one full run per batch)
    batches = scoring._batches(model, ids)
    kept = []
    for b_ids, _ in batches:
        keep = []
        model.prefill(b_ids, keep=keep)
        kept.append(keep)
    resumed = {}
    for L in (0, LLAMA_8B.layers // 2, LLAMA_8B.layers - 1):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for b, (b_ids, real) in enumerate(batches):
            scoring._nll(model.prefill(b_ids, all_logits=True, first_layer=L, hidden=kept[b][L] if L else None), b_ids, real)
        torch.cuda.synchronize()
        resumed[f"from_layer_{L}"] = round(time.perf_counter() - t0, 3)
    mean_resumed = sum(resumed.values()) / len(resumed)
    n_lin = LLAMA_8B.layers * len(PROJ)
    return {"seconds_per_evaluation": round(dt, 3), "tokens_per_s": round(sequences * seqlen / dt, 1), "ppl_random_init": round(ppl, 1),
            "seconds_per_resumed_evaluation": resumed,
            "evaluations_per_bit_level": n_lin, "minutes_per_bit_level": round(n_lin * mean_resumed / 60, 1),
            "config": f"8B shape, {blocks} blocks per linear, {sequences} sequences x {seqlen} tokens, batch 4"}


def e2e_decode(torch, dev, prompt_len=128, new_tokens=256):
    """Random-init Llama-3.1-8B-shape decode, batch 1: all 224 decoder linears are
    BitStackLinear (level 5) with seeded per-layer block counts in [2, 12] summing
    to about 5.5 GB with the dense embed / lm_head; one decode step is captured in a
    HIP graph and replayed for `new_tokens` greedy tokens after a `prompt_len` prompt.
    Measured twice: the fused step (grouped forwards + the library's RMSNorm and
    attention kernels; the headline) and the step with one call per linear and
    torch ops in between."""
    from bitstack_amd.utils.llama_decode import LLAMA_8B, SyntheticLlamaDecoder, synthetic_compression_config
    cfg, total = synthetic_compression_config(LLAMA_8B, 5.5e9)
    model = SyntheticLlamaDecoder(LLAMA_8B, cfg, prompt_len + new_tokens + 8, dev)
    prompt = torch.randint(0, LLAMA_8B.vocab, (prompt_len,), generator=torch.Generator().manual_seed(0))

    def run(fused):
        step = model.step_fused if fused else model.step
        model.reset()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model.prefill_positions(prompt, fused=fused)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
        graph.replay()                   # the captured step also ran once during capture bookkeeping
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(new_tokens):
            graph.replay()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    dt_plain = run(False)
    dt = run(True)
    wbytes = model.weight_bytes()
    blocks = list(cfg.values())
    return {"tok_s": round(new_tokens / dt, 1), "ms_per_token": round(dt / new_tokens * 1e3, 3),
            "tok_s_one_call_per_linear_torch_ops_between": round(new_tokens / dt_plain, 1),
            "weight_GB": round(wbytes / 1e9, 3), "blocks_per_linear_mean": round(sum(blocks) / len(blocks), 2),
            "hbm_roofline_tok_s": round(8e12 / wbytes, 1), "frac_of_hbm_roofline": round(new_tokens / dt * wbytes / 8e12, 4),
            "config": f"32 layers, hidden 4096, inter 14336, 32Q/8KV, vocab 128256, batch 1, {prompt_len}-token prompt, "
                      f"{new_tokens} greedy tokens, one HIP-graph replay per token"}


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py: this build measures one GPU; --gpus {a.gpus} is not supported "
              "(every box in this run has a single MI355X)", file=sys.stderr)
        sys.exit(2)
    import torch
    from bitstack_amd import _lib
    from bitstack_amd.utils.synthetic import synthetic_layer, algorithmic_bytes
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _lib.lib()
    stream = _lib.stream_ptr(dev)

    def build_sweep(T, shapes=SHAPES, blocks=BLOCKS):
        out, seed = [], 0
        for (M, N) in shapes:
            for I in blocks:
                out.append(Layer(M, N, I, T, seed, dev))
                seed += 1
        return out

    def workspace_for(layers):
        need = max(int(lib.bs_workspace_bytes(L.I, L.M, L.N, 16, L.T)) for L in layers)
        return torch.zeros(max(need, 256), dtype=torch.uint8, device=dev)     # zeroed semaphore area

    def time_sweep_graph(layers, steps, warmup):
        """Whole-pass wall clock with one pass captured in a HIP graph and replayed:
        the 40 kernel launches of a pass then cost the host one call."""
        ws = workspace_for(layers)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fns = [make_forward(L, lib, ws, _lib.stream_ptr(dev)) for L in layers]
            for f in fns:
                f()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            cap = _lib.stream_ptr(dev)
            for L in layers:
                make_forward(L, lib, ws, cap)()
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    def time_fns(fns, steps, warmup, per_layer_events, warm_ms=0.0):
        """The callables in turn, `steps` passes after `warmup` untimed ones: wall clock of the timed
        passes and, with events around every call, the mean time of each callable (ms).  `warm_ms`: keep
        running untimed passes until that much wall time has passed (after a pause the shader clock needs
        tens of milliseconds of load to come back: a variant timed first would otherwise look 10-20 % slower
        than the same kernels timed later)."""
        for _ in range(warmup):
            for f in fns:
                f()
        torch.cuda.synchronize()
        t_warm = time.perf_counter()
        while (time.perf_counter() - t_warm) * 1e3 < warm_ms:
            for f in fns:
                f()
            torch.cuda.synchronize()
        ev = None
        if per_layer_events:
            ev = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                   for _ in fns] for _ in range(steps)]
        t0 = time.perf_counter()
        for s in range(steps):
            for j, f in enumerate(fns):
                if ev:
                    ev[s][j][0].record()
                f()
                if ev:
                    ev[s][j][1].record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        per_layer = None
        if ev:
            per_layer = [sum(ev[s][j][0].elapsed_time(ev[s][j][1]) for s in range(steps)) / steps
                         for j in range(len(fns))]          # ms per forward
        return wall, per_layer

    def time_sweep(layers, steps, warmup, per_layer_events, warm_ms=0.0):
        ws = workspace_for(layers)
        return time_fns([make_forward(L, lib, ws, stream) for L in layers], steps, warmup, per_layer_events, warm_ms)

    def prefill_side(detail):
        pre = {}
        for T in PREFILL_T:
            lp = build_sweep(T, blocks=[8])
            _, perp = time_sweep(lp, 3, 1, per_layer_events=True, warm_ms=PREFILL_WARM_MS)
            useful = sum(2.0 * L.M * L.N * L.T + 2.0 * 16 * L.I * L.M * L.N for L in lp)
            tp = sum(perp) * 1e-3
            pre[f"T{T}"] = {"useful_tflops": round(useful / tp / 1e12, 1),
                            "frac_of_f16_mfma_peak": round(useful / tp / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)}
            pre[f"T{T}"]["kernels"] = sorted({_lib.PATH_NAMES[int(lib.bs_forward_path(L.I, L.M, L.N, 16, L.T))] for L in lp})
            if T >= 512:
                # beside it, timed the same way (the four layers in turn, events around each call): the same
                # forwards with the vendor GEMM (hipBLASLt) behind the rebuild - a comparator, never the headline
                # and never what bs_forward picks by itself - and the module's level 3 = this library's rebuild
                # kernel, then torch's F.linear, as the reference's levels 2-4 are built
                import torch.nn.functional as F
                from bitstack_amd.utils.inference_utils import unpack_and_reconstruct_w_hip
                lib.bs_set_dense_kernel(_lib.DENSE_LIBRARY)
                try:
                    _, ven = time_sweep(lp, 3, 1, per_layer_events=True, warm_ms=PREFILL_WARM_MS)
                finally:
                    lib.bs_set_dense_kernel(_lib.DENSE_AUTO)
                pre[f"T{T}"]["vendor_gemm_comparator_useful_tflops"] = round(useful / (sum(ven) * 1e-3) / 1e12, 1)
                _, lvl3 = time_fns([(lambda L=L: F.linear(L.x, unpack_and_reconstruct_w_hip(L.q, L.u, L.vt))) for L in lp],
                                   3, 1, per_layer_events=True, warm_ms=PREFILL_WARM_MS)
                pre[f"T{T}"]["level3_rebuild_plus_torch_linear_useful_tflops"] = round(useful / (sum(lvl3) * 1e-3) / 1e12, 1)
                pre[f"T{T}"]["us_per_layer"] = {"layers": [f"{L.M}x{L.N}" for L in lp], "default": [round(v * 1e3, 1) for v in perp],
                                                "vendor_gemm_comparator": [round(v * 1e3, 1) for v in ven],
                                                "level3": [round(v * 1e3, 1) for v in lvl3]}
            detail += [{"M": L.M, "N": L.N, "I": L.I, "T": T, "us": round(ms * 1e3, 2),
                        "useful_tflops": round((2.0 * L.M * L.N * L.T + 32.0 * L.I * L.M * L.N) / (ms * 1e-3) / 1e12, 1)}
                       for L, ms in zip(lp, perp)]
            del lp
        return pre

    if a.only in ("one_layer", "sweep_tokens"):
        # (the setting is this thread's; the process ends with the measurement)
        _lib.check(lib.bs_set_decode_kernel({"auto": _lib.DECODE_AUTO, "f16": _lib.DECODE_F16, "mx": _lib.DECODE_MX}[a.decode_kernel]),
                   "bs_set_decode_kernel")
    if a.only == "one_layer":
        # 12 forwards of ONE layer on 3 rotating copies of its buffers (as every layer of the sweep
        # is run), nothing else on the GPU: the process to put under rocprofv3 --pmc
        M, N, I, T = (int(v) for v in a.layer.split("x"))
        copies = [Layer(M, N, I, T, seed, dev) for seed in range(3)]
        ws = workspace_for(copies)
        fns = [make_forward(L, lib, ws, stream) for L in copies]
        for r in range(2):
            fns[r % 3]()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for r in range(12):
            fns[r % 3]()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / 12 * 1e3
        print(json.dumps({"one_layer": {"M": M, "N": N, "I": I, "T": T, "algorithmic_bytes": copies[0].bytes,
                                        "us_per_forward": round(us, 2), "GBps": round(copies[0].bytes / us / 1e3, 1),
                                        "decode_plan": _lib.decode_plan(I, M, N, 16, T),
                                        "decode_kernel": {0: "none", 1: "gemv_kernel (fp16 MFMA)", 2: "gemv_mx_kernel (fp4 x fp6 MFMA)"}[
                                            lib.bs_decode_kernel(I, M, N, 16, T)]}}))
        return
    if a.only == "sweep_tokens":
        # the 20-layer sweep at --tokens tokens per forward, events around every forward: the process to trace for
        # the multi-token decode kernels
        lt = build_sweep(a.tokens)
        _, per = time_sweep(lt, max(3, a.steps // 2), 1, per_layer_events=True, warm_ms=SIDE_WARM_MS)
        bt = sum(L.bytes for L in lt)
        print(json.dumps({"sweep_tokens": {"tokens": a.tokens, "us_per_pass": round(sum(per) * 1e3, 1),
                                           "GBps": round(bt / (sum(per) * 1e-3) / 1e9, 1),
                                           "layers": [{"M": L.M, "N": L.N, "I": L.I, "us": round(ms * 1e3, 2),
                                                       "kernel": _lib.PATH_NAMES[int(lib.bs_forward_path(L.I, L.M, L.N, 16, L.T))]}
                                                      for L, ms in zip(lt, per)]}}))
        return
    if a.only == "copy":
        # a plain device-to-device copy of 256 MiB, five times: what the FETCH_SIZE / WRITE_SIZE counters read for a
        # known number of bytes (the calibration of the traffic figures under profiles/)
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 256)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy": {"bytes_read": src.numel(), "bytes_written": dst.numel(), "copies": 5}}))
        return
    if a.only == "decode_8b":
        print(json.dumps({"decode_8b": e2e_decode(torch, dev)}))
        return
    if a.only == "scoring":
        print(json.dumps({"scoring": scoring_eval(torch, dev)}))
        return
    if a.only == "decode_70b":
        print(json.dumps({"decode_70b": e2e_decode_70b(torch, dev, batch=a.batch, prompt_len=a.prompt_len)}))
        return
    if a.only == "prefill":
        print(json.dumps({"prefill": prefill_side([])}))
        return

    # ---------------------------------------------------------------- headline: T = 1 sweep
    layers = build_sweep(1)
    pass_bytes = sum(L.bytes for L in layers)
    # (a) whole-job wall clock, no events in the stream
    launch = "hip graph replay"
    try:
        wall = time_sweep_graph(layers, a.steps, a.warmup)
    except Exception as e:                      # capture unsupported: plain launches
        launch = f"eager launches (graph capture failed: {type(e).__name__})"
        wall, _ = time_sweep(layers, a.steps, a.warmup, per_layer_events=False)
    ms_per_step = wall / a.steps * 1e3
    value = pass_bytes * a.steps / wall / 1e9
    # (b) kernel time per forward from HIP events on the launch stream
    _, per_layer = time_sweep(layers, a.steps, 1, per_layer_events=True)
    ev_total_ms = sum(per_layer)
    sweep_gbs = pass_bytes / (ev_total_ms * 1e-3) / 1e9
    def kernel_name(L):
        waves, r, grid, _ = _lib.decode_plan(L.I, L.M, L.N, 16, L.T)
        path = int(lib.bs_forward_path(L.I, L.M, L.N, 16, L.T))
        if path == _lib.PATH_DECODE_MX:
            return "gemv_mx_kernel<R=%d>" % r, grid
        if path == _lib.PATH_DECODE_F16:
            return "gemv_kernel<T=%d,WAVES=%d,R=%d>" % (L.T, waves, r), grid
        return _lib.PATH_NAMES[path], 0

    detail = [{"M": L.M, "N": L.N, "I": L.I, "T": L.T, "bytes": L.bytes, "us": round(ms * 1e3, 2),
               "GBps": round(L.bytes / (ms * 1e-3) / 1e9, 1),
               "kernel": "%s x %d workgroups" % kernel_name(L)}
              for L, ms in zip(layers, per_layer)]
    best = max(detail, key=lambda d: d["GBps"])
    # dominant kernel = the instantiation that takes the most time over the pass
    by_kernel = {}
    for L, ms in zip(layers, per_layer):
        by_kernel.setdefault(kernel_name(L)[0], []).append((L, ms))
    dom, dom_runs = max(by_kernel.items(), key=lambda kv: sum(ms for _, ms in kv[1]))
    dom_bytes, dom_ms, dom_n = sum(L.bytes for L, _ in dom_runs), sum(ms for _, ms in dom_runs), len(dom_runs)
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    # HBM bytes per launch: algorithmic bytes x the (FETCH_SIZE + WRITE_SIZE) / algorithmic ratio that rocprofv3 --pmc
    # measured on one of THIS kernel's launches (profiles/decode_traffic_counters.txt, a "ratio:" line per kernel)
    traffic_ratio, traffic_note = None, "no counter run on record for this kernel"
    try:
        import hashlib
        def source_id(name):
            with open(os.path.join(ROOT, "bitstack_amd", "csrc", name), "rb") as f:
                return hashlib.sha256(f.read()).hexdigest()[:12]
        with open(os.path.join(ROOT, "profiles", "decode_traffic_counters.txt")) as f:
            lines = f.read().splitlines()
        # "source: <file> <sha256[:12]>" lines say which kernel sources the counters were collected on; a ratio is only
        # used while those files are unchanged
        stale = [p[1] for p in (l.split() for l in lines) if len(p) == 3 and p[0] == "source:" and source_id(p[1]) != p[2]]
        for line in lines:
            parts = line.split()
            if len(parts) >= 3 and parts[0] == "ratio:" and parts[1] == dom:
                if stale:
                    traffic_note = "the counter run on record was made on another version of " + ", ".join(stale) + ": not used"
                else:
                    traffic_ratio = float(parts[2])
                    traffic_note = ("HBM bytes per launch = algorithmic x %.2f, the (FETCH_SIZE + WRITE_SIZE) / algorithmic ratio of %s "
                                    "(profiles/decode_traffic_counters.txt)" % (traffic_ratio, " ".join(parts[3:])))
    except OSError:
        pass
    # What bounds it, from this run's own numbers: a least-squares line us = fixed + bytes / rate through the
    # kernel's launches separates the per-launch cost from the streaming rate; the floors are the HBM time of the
    # bytes and the matrix-core issue time of the contraction (16 MACs per sign bit; the block-scaled kernel issues
    # three 16x16x128 MFMAs per 16 x 128 signs, the fp16 kernel four 16x16x32 MFMAs, on 1024 SIMDs at the measured
    # time per MFMA).
    def mfma_floor_us(L):
        tiles = L.I * L.M * L.N / (16.0 * 128.0)
        ns = tiles * (3 * MFMA_MX_NS if "mx" in dom else 4 * MFMA_F16_NS)
        return ns / 1024.0 / 1e3
    xs, ys = [L.bytes for L, _ in dom_runs], [ms * 1e3 for _, ms in dom_runs]
    if len(xs) >= 2 and max(xs) > min(xs):
        mx_, my_ = sum(xs) / len(xs), sum(ys) / len(ys)
        slope = sum((a - mx_) * (b - my_) for a, b in zip(xs, ys)) / sum((a - mx_) ** 2 for a in xs)
        fixed_us, stream_gbs = my_ - slope * mx_, 1e-3 / slope if slope > 0 else float("inf")
    else:
        fixed_us, stream_gbs = None, None
    hbm_floor = dom_bytes / HBM_PEAK_GBS / 1e3 / dom_n
    mfma_floor = sum(mfma_floor_us(L) for L, _ in dom_runs) / dom_n
    avg_us = dom_ms * 1e3 / dom_n
    shares = {"fixed cost per forward (two launches, pipeline fill and drain)": fixed_us or 0.0,
              "matrix-core issue time of the contraction": mfma_floor, "HBM time of the bytes": hbm_floor}
    limiter = max(shares, key=shares.get)
    # the roofline this kernel is priced against: the larger of its two machine floors (HBM time of its bytes, matrix-core
    # issue time of its MFMAs); the fixed cost per forward is overhead under either
    bound = "mfma" if mfma_floor > hbm_floor else "hbm"
    if bound == "mfma":
        # issued matrix-core flops of the contraction (16 MACs per sign bit and term) against the dense peak of the
        # instruction family the kernel runs on
        terms = 3.0 if "mx" in dom else 1.0
        flops = sum(2.0 * 16 * terms * L.I * L.M * L.N for L, _ in dom_runs)
        roof_achieved, roof_peak, roof_unit = flops / (dom_ms * 1e-3) / 1e12, (10100.0 if "mx" in dom else MFMA_F16_PEAK_TFLOPS), "TFLOP/s"
    else:
        roof_achieved, roof_peak, roof_unit = achieved, HBM_PEAK_GBS, "GB/s"
    limiter_note = ("of %.1f us per forward: %.1f us fixed (intercept of the line through this kernel's launches), %.1f us MFMA "
                    "issue floor, %.1f us HBM floor; streaming rate beyond the fixed cost %s GB/s -> largest share: %s"
                    % (avg_us, fixed_us or 0.0, mfma_floor, hbm_floor,
                       "n/a" if stream_gbs is None else "%.0f" % stream_gbs, limiter))

    out = {
        "metric": "packed-sign GEMV HBM GB/s (decode sweep, Llama-3.1-8B linear shapes, T=1)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "decode GEMV sweep: (out x in) in {4096x4096, 1024x4096, 14336x4096, 4096x14336} "
                               "x blocks {1,2,4,8,16}, k=16, T=1, one fused forward per layer, distinct buffers per layer",
                   "layers_per_step": len(layers), "algorithmic_MB_per_step": round(pass_bytes / 1e6, 1),
                   "launch": launch},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "roofline": {"bound": bound, "achieved": round(roof_achieved, 1), "peak": roof_peak, "unit": roof_unit,
                     "frac": round(roof_achieved / roof_peak, 4),
                     "frac_of_hbm_peak": round(achieved / HBM_PEAK_GBS, 4),
                     "frac_of_mfma_issue_floor": round(mfma_floor / avg_us, 4),
                     "traffic": None if traffic_ratio is None else round(dom_bytes / dom_n * traffic_ratio),
                     "kernel": dom + " (+ its gemv_reduce_flat_kernel), the instantiation with the most time in the pass",
                     "launches_per_step": dom_n,
                     "avg_us_per_launch": round(dom_ms * 1e3 / dom_n, 2),
                     "avg_algorithmic_bytes_per_launch": round(dom_bytes / dom_n),
                     "traffic_note": traffic_note,
                     "limiter": limiter_note,
                     "hbm_floor_us": round(hbm_floor, 2), "mfma_issue_floor_us": round(mfma_floor, 2),
                     "fixed_us": None if fixed_us is None else round(fixed_us, 2),
                     "streaming_GBps_beyond_fixed": None if stream_gbs is None else round(stream_gbs, 1),
                     "whole_sweep_GBps_by_events": round(sweep_gbs, 1),
                     "best_layer": best},
    }

    if not a.no_extras:
        # ------------------------------------------------------------ T = 2 sweep (block-scaled kernel, 512-column units)
        l2 = build_sweep(2)
        _, per2 = time_sweep(l2, max(3, a.steps // 2), 1, per_layer_events=True, warm_ms=SIDE_WARM_MS)
        b2 = sum(L.bytes for L in l2)
        t2 = sum(per2) * 1e-3
        lib.bs_set_decode_kernel(_lib.DECODE_F16)
        try:
            _, per2f = time_sweep(l2, max(3, a.steps // 2), 1, per_layer_events=True, warm_ms=SIDE_WARM_MS)
        finally:
            lib.bs_set_decode_kernel(_lib.DECODE_AUTO)
        out["t2"] = {"GBps": round(b2 / t2 / 1e9, 1), "pct_of_hbm_peak": round(100.0 * b2 / t2 / 1e9 / HBM_PEAK_GBS, 2),
                     "kernels": sorted({kernel_name(L)[0] for L in l2}),
                     "GBps_fp16_kernel_forced": round(b2 / (sum(per2f) * 1e-3) / 1e9, 1)}
        detail += [{"M": L.M, "N": L.N, "I": L.I, "T": 2, "bytes": L.bytes, "us": round(ms * 1e3, 2),
                    "GBps": round(L.bytes / (ms * 1e-3) / 1e9, 1)} for L, ms in zip(l2, per2)]
        del l2
        # ------------------------------------------------------------ T = 4 sweep (MFMA-bound side)
        l4 = build_sweep(4)
        _, per4 = time_sweep(l4, max(3, a.steps // 2), 1, per_layer_events=True, warm_ms=SIDE_WARM_MS)
        b4 = sum(L.bytes for L in l4)
        flops4 = sum(2.0 * 16 * L.I * L.M * L.N * L.T for L in l4)
        t4 = sum(per4) * 1e-3
        out["t4"] = {"GBps": round(b4 / t4 / 1e9, 1), "kernels": sorted({kernel_name(L)[0] for L in l4}),
                     "mfma_tflops_issued": round(flops4 / t4 / 1e12, 1),
                     "frac_of_f16_mfma_peak": round(flops4 / t4 / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)}
        detail += [{"M": L.M, "N": L.N, "I": L.I, "T": 4, "bytes": L.bytes, "us": round(ms * 1e3, 2),
                    "GBps": round(L.bytes / (ms * 1e-3) / 1e9, 1)} for L, ms in zip(l4, per4)]
        del l4
        # ------------------------------------------------------------ T = 16 sweep (strip kernel: batched decode)
        l16 = build_sweep(16)
        _, per16 = time_sweep(l16, max(3, a.steps // 2), 1, per_layer_events=True, warm_ms=SIDE_WARM_MS)
        b16 = sum(L.bytes for L in l16)
        t16 = sum(per16) * 1e-3
        out["t16"] = {"GBps": round(b16 / t16 / 1e9, 1), "pct_of_hbm_peak": round(100.0 * b16 / t16 / 1e9 / HBM_PEAK_GBS, 2),
                      "kernels": sorted({kernel_name(L)[0] for L in l16}) + ["gemv_reduce_flat_kernel"]}
        detail += [{"M": L.M, "N": L.N, "I": L.I, "T": 16, "bytes": L.bytes, "us": round(ms * 1e3, 2),
                    "GBps": round(L.bytes / (ms * 1e-3) / 1e9, 1)} for L, ms in zip(l16, per16)]
        del l16
        # ------------------------------------------------------------ prefill (useful flops)
        pre = prefill_side(detail)
        out["prefill"] = pre

    if not a.no_extras:
        out["decode_8b"] = e2e_decode(torch, dev)
        torch.cuda.empty_cache()
        # 70B shape: batch 8 with 2048-token prompts (one-pass prefill, strip kernel), then batch 1 (GEMV)
        out["decode_70b"] = e2e_decode_70b(torch, dev, batch=8, prompt_len=2048)
        torch.cuda.empty_cache()
        out["decode_70b_batch1"] = e2e_decode_70b(torch, dev, batch=1, prompt_len=16)
        torch.cuda.empty_cache()

    if not a.no_cpu_baseline:
        # bounded sample of the same sweep: every shape, blocks {1, 2} (3/31 of the pass), median of 5 runs each
        cpu_layers = []
        seed = 0
        for (M, N) in SHAPES:
            for I in BLOCKS:
                if I <= 2:
                    q, u, vt, x = synthetic_layer(M, N, I, 1, seed=seed)
                    cpu_layers.append((q, u, vt, x, algorithmic_bytes(I, M, N, 1)))
                seed += 1
        out["cpu_baseline"] = cpu_baseline(cpu_layers)
    else:
        out["cpu_baseline"] = None

    if a.detail:
        os.makedirs(os.path.dirname(os.path.abspath(a.detail)), exist_ok=True)
        with open(a.detail, "w") as f:
            json.dump(detail, f, indent=1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
