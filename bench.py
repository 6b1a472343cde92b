#!/usr/bin/env python3
"""Benchmark of the split-12 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Workloads (synthetic, seeded, random-init weights of the Llama-3.1-8B shape:
32 layers, hidden 4096, FFN 14336, 32/8 heads, vocab 128256; N(0, 0.02) with
3e-4 of the entries replaced by N(0, 8) outliers so that ~0.045 % escape):

  decode (default) one step = one greedy decode step of the full engine (embedding, 32 x [RMSNorm, fused
                  QKV decode-GEMV, RoPE + INT8 KV store, GQA attention, O, add+RMSNorm, fused gate|up,
                  SiLU*mul, down, add+RMSNorm], lm_head, argmax + D2H) on a model generated and packed on
                  the GPU; prompt 128 random ids, 2048-token KV cache.  B = 1 is
                  `value`; B = 256 is measured in the same run and reported under "b256"; the
                  decode-GEMV launches of a step are also timed alone for `roofline`.

  gemm_layers     the four linear-layer shapes through the fused decode+GEMM at B = 2, 4, 8, 16, 64, 256 on three
                  rotating weight copies; `roofline` prices gate|up at B = 256 against
                  the 2.5 PFLOP/s dense bf16 MFMA peak.

  moe             one step = one Mixtral-8x7B-shaped MoE FFN layer (8 split-12 experts, top-2) over 256 tokens
                  grouped per expert through the decode+GEMM.

  attention       the attention step of one decoder layer (RoPE, INT8 KV store, GQA decode attention over the
                  INT8 cache) with every sequence on its own cache region, at several (batch, context) points;
                  `roofline` prices the cache bytes of B = 256 at 2000 positions against the HBM peak.

  codec           the standalone codec kernels on three Llama-3.1-8B tensors: t12_decompress (planes -> bf16, patched and
                  unpatched) and the GPU packer's passes (histogram, planes, escapes), in GB/s of the bytes each must move.

  convert         checkpoint ingestion end to end: a 1.4 GB bf16 safetensors checkpoint (two Llama-3.1-8B layers, embedding,
                  head) through convert() -- mmap read, packing on the GPU, model directory written -- in GB/s of checkpoint.

  tokenizer       host only: one step = encoding ~1 MB of text (150 000 words of a 4000-word list) with the engine's
                  byte-level BPE tokenizer over the ~20 000 merges that build those words; `cpu_baseline` is the reference's rule restated literally (one pass over the
                  text per merge) on a 4 KB sample of the same text.

  gemv_stack_b1   one step = every linear layer of one decode step at B = 1 through
                  the fused split-12 decode-GEMV: per layer QKV (3 segments, one
                  launch), O, gate+up (2 segments, one launch), down; then lm_head.
                  7 504 658 432 weights = 11.257 GB of compressed planes per step.

Prints ONE JSON line.  `value` is tokens per second of the step (inputs resident
in HBM), `roofline` prices the decode-GEMV kernel against the 8 TB/s HBM peak in
algorithmic bytes (1.5 B per weight + escape list + activations + outputs), and
`cpu_baseline` is the CPU oracle (fused decode + fp32 GEMV, OpenMP over the host
cores) timed on one decoder layer of the same weights and scaled to the model.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

LLAMA8B = dict(n_layer=32, n_embd=4096, n_ff=14336, n_head=32, n_head_kv=8, n_vocab=128256)
HBM_PEAK_GBS = 8000.0


def measured_traffic(key):
    """HBM bytes per launch of the named kernel, from profiles/measured_traffic.txt: the figure two rocprofv3 --pmc
    runs of this file gave (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, factors from the --calibrate copy kernel), written
    down with the first 16 hex digits of the SHA-256 of the kernel's source file at the time.  A figure whose source
    file has changed since is reported as None: counters are not read by this run."""
    import hashlib
    path = os.path.join(ROOT, "profiles", "measured_traffic.txt")
    try:
        lines = open(path).read().splitlines()
    except OSError:
        return None
    for line in lines:
        f = line.split()
        if len(f) >= 4 and not line.startswith("#") and f[0] == key:
            try:
                now = hashlib.sha256(open(os.path.join(ROOT, f[2]), "rb").read()).hexdigest()[:16]
            except OSError:
                return None
            return float(f[1]) if now == f[3] else None
    return None


def synth_weight(torch, M, K, seed, dev, sigma=0.02, p_out=3e-4, sigma_out=8.0):
    """bf16 [M, K] on the GPU: N(0, sigma) with outliers N(0, sigma_out) at rate p_out."""
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    w = torch.randn((M, K), generator=g, device=dev, dtype=torch.float32) * sigma
    m = torch.rand((M, K), generator=g, device=dev) < p_out
    o = torch.randn((M, K), generator=g, device=dev, dtype=torch.float32) * sigma_out
    w = torch.where(m, o, w).to(torch.bfloat16)
    return w


def algorithmic_bytes(t, B=1):
    """1.5*M*K + 8*P + 4*(M+1) + 2*K*B + 4*M*B  (the figure the roofline is priced in)."""
    return 1.5 * t.M * t.K + 8 * t.P + 4 * (t.M + 1) + 2 * t.K * B + 4 * t.M * B


def build_stack(t12, torch, dev, cfg, base_seed=4000):
    """Packs the model's linear layers on the GPU.  Returns the list of launches:
    each is (tensors, act_key) with act_key in {'h', 'ff'}."""
    n, ff, hd = cfg["n_embd"], cfg["n_ff"], cfg["n_embd"] // cfg["n_head"]
    kv = cfg["n_head_kv"] * hd
    launches = []
    seed = base_seed
    for _ in range(cfg["n_layer"]):
        def mk(M, K):
            nonlocal seed
            seed += 1
            return t12.pack_device(synth_weight(torch, M, K, seed, dev))
        launches.append(([mk(n, n), mk(kv, n), mk(kv, n)], "h"))      # wq | wk | wv
        launches.append(([mk(n, n)], "h"))                             # wo
        launches.append(([mk(ff, n), mk(ff, n)], "h"))                 # w_gate | w_up
        launches.append(([mk(n, ff)], "ff"))                           # w_down
    # lm_head: built in 8 row slabs to bound the fp32 staging memory, then joined
    slabs = []
    rows = cfg["n_vocab"] // 8
    for i in range(8):
        seed += 1
        slabs.append(synth_weight(torch, rows, n, seed, dev))
    w = torch.cat(slabs)
    del slabs
    launches.append(([t12.pack_device(w)], "h"))
    del w
    torch.cuda.empty_cache()
    return launches


def cpu_baseline(torch, launches, cfg, runs=3, n_weights_model=None):
    """Times the CPU oracle on the first decoder layer (7 tensors, 218 M weights) and scales
    the per-weight rate to the whole model."""
    import numpy as np
    from oracle import oracle

    packs = []
    for tensors, key in launches[:4]:
        for t in tensors:
            p = oracle.Packed(t.M, t.K, t.base_exp, t.sm.cpu().numpy(), t.gr.cpu().numpy(),
                              t.row_off.cpu().numpy(), t.cols.cpu().numpy(), t.correct.cpu().numpy(),
                              t.wrong.cpu().numpy())
            packs.append(p)
    rng = np.random.default_rng(7)
    xs = {K: oracle.f32_to_bf16_bits(rng.standard_normal(K).astype(np.float32)) for K in {p.K for p in packs}}
    w_layer = sum(p.M * p.K for p in packs)
    w_model = n_weights_model or sum(t.M * t.K for tensors, _ in launches for t in tensors)

    def leg(seconds):
        times = []
        t_begin = time.perf_counter()
        while len(times) < runs or (time.perf_counter() - t_begin < seconds and len(times) < 2000):
            t0 = time.perf_counter()
            for p in packs:
                oracle.gemv(p, xs[p.K])
            times.append(time.perf_counter() - t0)
        return sorted(times)[len(times) // 2], len(times)

    oracle.set_num_threads(0)                      # every host core the process may use
    threads = oracle.num_threads()
    t_layer, n_all = leg(10.0)                     # ~10 s of CPU work
    oracle.set_num_threads(1)
    t_one, n_one = leg(8.0)                        # ~8 s more on one thread
    oracle.set_num_threads(0)
    t_model = t_layer * w_model / w_layer
    return {
        "value": 1.0 / t_model, "unit": "tok/s", "cores": threads, "kind": "port",
        "nproc": os.cpu_count(),
        "one_thread": {"value": 1.0 / (t_one * w_model / w_layer), "unit": "tok/s", "cores": 1,
                       "GBps_compressed": 1.5 * w_layer / t_one / 1e9, "runs": n_one},
        "sample": "decoder layer 0 (wq,wk,wv,wo,gate,up,down = %d weights) x%d runs (~10 s) on %d threads, median %.4f s, "
                  "scaled by weight count to the %d-weight model; %.2f GB/s compressed; then the same layer x%d runs on "
                  "one thread (median %.4f s)" % (w_layer, n_all, threads, t_layer, w_model,
                                                  1.5 * w_layer / t_layer / 1e9, n_one, t_one),
    }


def calibration_copy(torch, dev):
    """One plain device-to-device copy kernel of exactly 1 GiB (torch's elementwise copy of an int32 tensor): the
    launch of known size that the profiler's FETCH_SIZE / WRITE_SIZE readings are scaled by."""
    src = torch.empty(2**28, dtype=torch.int32, device=dev).random_(0, 1 << 30)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def ext_stream(torch, ptr):
    return torch.cuda.ExternalStream(ptr)


def timed(torch, stream, fn, steps):
    """HIP events recorded on the stream the kernels run on, bracketed by synchronisation."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    w0 = time.perf_counter()
    e0.record(stream)
    for _ in range(steps):
        fn()
    e1.record(stream)
    torch.cuda.synchronize()
    wall = (time.perf_counter() - w0) * 1e3 / steps
    return max(e0.elapsed_time(e1) / steps, wall), e0.elapsed_time(e1) / steps


def run_decode(args, t12, torch, dev):
    """Full greedy decode on a random-init Llama-3.1-8B-shaped model generated and packed on the GPU
    prompt of 128 random ids, 2048-token KV cache, one forward + one greedy sample
    per step; B = 1 is `value`, B = 256 (256 lock-step copies sharing the cache, the reference's batched
    mode) is reported next to it."""
    import numpy as np
    cfg = dict(LLAMA8B, n_layer=args.layers, n_ctx=2048, rope_theta=500000.0, rms_norm_eps=1e-5)
    t0 = time.time()
    eng = t12.Engine.synthetic(cfg, seed=4000, max_seq=2048, batch=1)
    torch.cuda.synchronize()
    t_build = time.time() - t0
    rng = np.random.default_rng(4001)
    prompt = [int(t) for t in rng.integers(3, cfg["n_vocab"], size=args.prompt)]

    def decode_loop(e, B):
        st = ext_stream(torch, t12.lib.t12_engine_stream(e.state))
        for i, t in enumerate(prompt):                      # prefill, one token per forward (inference.cpp:721-724)
            e.set_positions([i] * B)
            e.forward([t] * B)
        # one step = sample (argmax on the device) + forward on the sampled ids, K of them inside
        # decode_greedy: the host reads token t while the GPU computes step t + 1
        e.decode(args.warmup)
        ms, ev = timed(torch, st, lambda: e.decode(args.steps), 1)
        return ms / args.steps, ev / args.steps

    ms1, _ = decode_loop(eng, 1)

    # ---- roofline of the dominant kernel: the GEMV launches of one step, alone, on the current stream
    n_l = cfg["n_layer"]
    hd = cfg["n_embd"] // cfg["n_head"]
    kvd = cfg["n_head_kv"] * hd
    g = torch.Generator(device=dev)
    g.manual_seed(99)
    acts = {cfg["n_embd"]: torch.randn(cfg["n_embd"], generator=g, device=dev).to(torch.bfloat16),
            cfg["n_ff"]: torch.randn(cfg["n_ff"], generator=g, device=dev).to(torch.bfloat16)}
    scratch = torch.empty(cfg["n_vocab"] + 2 * cfg["n_ff"], dtype=torch.float32, device=dev)
    tabs, alg_bytes, plane_bytes, n_weights, n_esc = [], 0.0, 0.0, 0, 0
    groups = [(0, 1, 2), (3,), (4, 5), (6,)]
    for layer in list(range(n_l)) + [-1]:
        for grp in (groups if layer >= 0 else [(0,)]):
            segs, off, K = [], 0, None
            for which in grp:
                seg, K, P = eng.weight(layer, which)
                seg.out = scratch.data_ptr() + 4 * off
                off += seg.M
                segs.append(seg)
                alg_bytes += 1.5 * seg.M * K + 8 * P + 4 * (seg.M + 1) + 4 * seg.M
                plane_bytes += 1.5 * seg.M * K
                n_weights += seg.M * K
                n_esc += P
            alg_bytes += 2 * K
            tabs.append((t12._seg_array(segs), len(segs), acts[K].data_ptr(), K))
    cur = torch.cuda.current_stream()

    def gemv_pass():
        for segs, n, act, K in tabs:
            rc = t12.lib.t12_gemv(segs, n, act, K, cur.cuda_stream)
            if rc:
                t12.check(rc, "t12_gemv")
    for _ in range(3):
        gemv_pass()
    _, ms_gemv = timed(torch, cur, gemv_pass, max(args.steps, 10))
    achieved = alg_bytes / (ms_gemv * 1e-3) / 1e9

    gemm_layers = gemm_layer_leg(t12, torch, dev, cfg, lambda layer, which: eng.weight(layer, which), min(3, n_l),
                                 cur, g, batches=(2, 4, 8, 16, 32, 64, 128, 256), yardstick=True)
    probe = clock_probe(t12)

    # ---- B = 256
    b256 = None
    if args.batch256:
        e256 = eng.new_state(256)
        ms256, _ = decode_loop(e256, 256)
        b256 = {"tok_s": 256e3 / ms256, "ms_per_step": ms256, "batch": 256,
                "note": "256 lock-step copies of one stream sharing one KV-cache region (the reference's batched mode)"}
        e256.close()
        # the same batch as 256 INDEPENDENT sequences: own prompt, own KV-cache region each; prompts enter
        # through the batched prefill (rows = prompt tokens), then all sequences decode together
        es = eng.new_state(256, per_sequence=2048)
        st = ext_stream(torch, t12.lib.t12_engine_stream(es.state))
        prompts = rng.integers(3, cfg["n_vocab"], size=(256, args.prompt))
        es.prefill(0, prompts[0])
        es.set_positions([0] * 256)

        def prefill_all():
            for b in range(256):
                es.prefill(b, prompts[b])
        ms_pre, _ = timed(torch, st, prefill_all, 1)
        es.decode_all(args.warmup)
        ms_ind, _ = timed(torch, st, lambda: es.decode_all(args.steps), 1)
        ms_ind /= args.steps
        b256["independent"] = {
            "tok_s": 256e3 / ms_ind, "ms_per_step": ms_ind,
            "prefill_tok_s": 256 * args.prompt / (ms_pre * 1e-3), "prefill_ms_per_sequence": ms_pre / 256,
            "note": "256 independent sequences, per-sequence INT8 KV caches of 2048 positions (34 GB), prompts of %d ids "
                    "through the batched prefill; not a mode of the reference" % args.prompt}
        es.close()

    # ---- the batch sizes between 1 and 256 that the reference publishes (docs/TECHNICAL.md:121-126), same lock-step mode
    batch_sweep = None
    if args.batch256:
        batch_sweep = {}
        for B in (4, 8, 16, 32, 64, 128):
            eb = eng.new_state(B)
            msb, _ = decode_loop(eb, B)
            batch_sweep["b%d" % B] = {"tok_s": round(B * 1e3 / msb, 1), "ms_per_step": round(msb, 4)}
            eb.close()

    result = {
        "metric": "tok/s at B=1 (Llama-3.1-8B shape), greedy decode of a split-12 model; B=256 and decode-GEMV GB/s alongside",
        "value": 1e3 / ms1, "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms1, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": (1e3 / ms1) / 57.0 if n_l == LLAMA8B["n_layer"] else None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "decode_b1: random-init Llama-3.1-8B shape (32 layers, 4096/14336, 32/8 heads, vocab 128256), "
                               "split-12 weights N(0,0.02)+3e-4 outliers, prompt %d random ids, greedy decode, 2048-token INT8 "
                               "KV cache, one forward + sample per step" % args.prompt,
                   "batch": 1, "n_layer": n_l, "weights": n_weights, "compressed_GB_per_step": plane_bytes / 1e9,
                   "escape_fraction": n_esc / max(n_weights, 1),
                   "baseline": "57.0 tok/s, Llama 3.1 8B B=1 on RTX 5070 Ti (reference README.md:46)"},
        "b256": b256,
        "batch_sweep": batch_sweep,
        "gemv_compressed_GBps": plane_bytes / (ms_gemv * 1e-3) / 1e9,
        "gemv_only_ms_per_step": ms_gemv,
        "gemm_layers": gemm_layers,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": measured_traffic("gemv_stack_b1") if n_l == LLAMA8B["n_layer"] else None,
                     "kernel": "gemv_stream_kernel", "bytes_per_launch": alg_bytes / len(tabs),
                     "us_per_launch": ms_gemv * 1e3 / len(tabs),
                     # the other target of the path: decode+GEMM at B = 256 over the four linear layers of a decoder
                     # layer, against the dense bf16 MFMA peak (median launch times of gemm_layers above)
                     "gemm_b256": {**gemm_b256_roofline(gemm_layers),
                                   "clock_ghz_mfma_only_256wg": probe["mfma_only_256wg"]["ghz"],
                                   "clock_ghz_mfma_decode_lds_256wg": probe["mfma_decode_lds_256wg"]["ghz"],
                                   "mfma_only_probe_TFLOPs": probe["mfma_only_256wg"]["TFLOPs"]}},
        "clock_probe": probe,
        "setup_s": t_build,
    }
    if not args.no_cpu_baseline:
        # the same oracle leg as the stack workload, on layer 0 of this model
        class T:
            pass
        launches = []
        for grp in groups:
            ts = []
            for which in grp:
                seg, K, P = eng.weight(0, which)
                t = T()
                t.M, t.K, t.base_exp = seg.M, K, seg.base_exp

                def pull(ptr, n, dt):
                    if n == 0 or not ptr:
                        return torch.zeros(0, dtype=dt)
                    out = torch.empty(n, dtype=dt, device=dev)
                    t12._hip_memcpy_d2d(out.data_ptr(), ptr, n * out.element_size())
                    return out.cpu()
                t.sm = pull(seg.sm, seg.M * K, torch.uint8)
                t.gr = pull(seg.gr, (seg.M * K + 1) // 2, torch.uint8)
                t.row_off = pull(seg.row_off, seg.M + 1, torch.int32) if P else torch.zeros(seg.M + 1, dtype=torch.int32)
                t.cols = pull(seg.cols, P, torch.int32)
                t.correct = pull(seg.correct, P, torch.int16)
                t.wrong = pull(seg.wrong, P, torch.int16)
                t.P = P
                ts.append(t)
            launches.append((ts, None))
        result["cpu_baseline"] = cpu_baseline(torch, launches, cfg, n_weights_model=n_weights)
    eng.close()
    return result


def run_moe(args, t12, torch, dev):
    """Mixtral-8x7B-shaped MoE FFN layer: 8 experts x (4096 -> 14336 -> 4096, SwiGLU),
    256 tokens, top-2 routing from random router logits; one step = the whole layer."""
    import importlib
    moe = importlib.import_module("turbo_lossless_amd.moe")
    E, n, ff, T = 8, 4096, 14336, 256
    t0 = time.time()
    experts = [moe.Expert(*[t12.pack_device(synth_weight(torch, M, K, 5000 + 3 * e + j, dev, p_out=5e-4))
                            for j, (M, K) in enumerate([(ff, n), (ff, n), (n, ff)])]) for e in range(E)]
    torch.cuda.synchronize()
    t_build = time.time() - t0
    g = torch.Generator(device=dev)
    g.manual_seed(5100)
    X = torch.randn((T, n), generator=g, device=dev).to(torch.bfloat16).view(torch.int16)
    ids, w = moe.route_top_k(torch.randn((T, E), generator=g, device=dev), 2)
    cur = torch.cuda.current_stream()
    layer = moe.MoeLayer(experts)
    out = torch.empty((T, n), dtype=torch.float32, device=dev)

    def step():
        layer(X, ids, w, out=out, stream=cur.cuda_stream)
    for _ in range(args.warmup):
        step()
    ms_step, ms = timed(torch, cur, step, args.steps)
    flops = 2.0 * (T * 2) * 3 * n * ff
    wbytes = 1.5 * E * 3 * n * ff
    # the same layer on the first 1 / 4 / 16 tokens (a decode step of a MoE model): only the experts those tokens name are
    # streamed; the rate is over their planes
    small = {}
    for Ts in (1, 4, 16):
        Xs, ids_s, w_s = X[:Ts].contiguous(), ids[:Ts].contiguous(), w[:Ts].contiguous()
        outs = torch.empty((Ts, n), dtype=torch.float32, device=dev)

        def step_s():
            layer(Xs, ids_s, w_s, out=outs, stream=cur.cuda_stream)
        for _ in range(args.warmup):
            step_s()
        _, ms_s = timed(torch, cur, step_s, args.steps)
        active = int(torch.unique(ids_s).numel())
        small["tokens_%d" % Ts] = {"ms": round(ms_s, 4), "experts_named": active,
                                   "weight_GBps": round(1.5 * active * 3 * n * ff / ms_s / 1e6, 1)}
    return {
        "metric": "tokens/s through one Mixtral-8x7B-shaped split-12 MoE FFN layer (8 experts, top-2), 256 tokens",
        "value": T * 1e3 / ms_step, "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "moe_mixtral_b256", "experts": E, "top_k": 2, "tokens": T,
                   "tokens_per_expert": torch.bincount(ids.reshape(-1), minlength=E).tolist()},
        "TFLOPs": flops / ms / 1e9, "weight_GBps": wbytes / ms / 1e6,
        "small_batches": small,
        "roofline": {"bound": "hbm", "achieved": wbytes / ms / 1e6, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": wbytes / ms / 1e6 / HBM_PEAK_GBS, "traffic": None, "kernel": "gemm_mfma_kernel"},
        "setup_s": t_build,
    }


def run_codec(args, t12, torch, dev):
    """The standalone codec kernels on Llama-3.1-8B tensors (three rotating copies each, so nothing is served from a
    cache): t12_decompress (split-12 planes -> bf16, patched = lossless and unpatched) and the GPU packer's three passes
    (histogram, planes, escapes).  `value` is the patched decode of gate 14336 x 4096 in GB/s of HBM traffic."""
    import ctypes as C
    cur = torch.cuda.current_stream()
    st = cur.cuda_stream
    shapes = {"gate_14336x4096": (14336, 4096), "down_4096x14336": (4096, 14336), "o_4096x4096": (4096, 4096)}
    out = {}
    t0 = time.time()
    for name, (M, K) in shapes.items():
        ws = [synth_weight(torch, M, K, 7000 + i, dev) for i in range(3)]
        ts = [t12.pack_device(w) for w in ws]
        dst = torch.empty((M, K), dtype=torch.int16, device=dev)
        n = float(M) * K
        P = sum(t.P for t in ts) / 3.0
        res = {"weights": int(n), "escapes": P / n}

        def med(fn, reps=max(args.steps, 20)):
            for _ in range(3):
                fn()
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
            for a, b in evs:
                a.record(cur)
                fn()
                b.record(cur)
            torch.cuda.synchronize()
            return sorted(a.elapsed_time(b) for a, b in evs)[reps // 2] / 3.0        # ms per tensor

        for patched in (1, 0):
            ms = med(lambda: [t12.decompress(t, patched=bool(patched), out=dst, stream=st) for t in ts])
            nbytes = 1.5 * n + 2.0 * n + (8.0 * P + 4.0 * (M + 1) if patched else 0.0)
            res["decompress_patched" if patched else "decompress_unpatched"] = {"us": ms * 1e3, "GBps": nbytes / ms / 1e6}
        hist = torch.empty(256, dtype=torch.int64, device=dev)
        ms = med(lambda: [t12.check(t12.lib.t12_pack_histogram(w.data_ptr(), w.numel(), hist.data_ptr(), st), "hist") for w in ws])
        res["pack_histogram"] = {"us": ms * 1e3, "GBps": 2.0 * n / ms / 1e6}
        sm = torch.empty(int(n), dtype=torch.uint8, device=dev)
        gr = torch.empty((int(n) + 1) // 2, dtype=torch.uint8, device=dev)
        cnt = torch.empty(M, dtype=torch.int32, device=dev)
        ms = med(lambda: [t12.check(t12.lib.t12_pack_planes(w.data_ptr(), M, K, t.base_exp, sm.data_ptr(), gr.data_ptr(),
                                                            cnt.data_ptr(), st), "planes") for w, t in zip(ws, ts)])
        res["pack_planes"] = {"us": ms * 1e3, "GBps": 3.5 * n / ms / 1e6}
        ms = med(lambda: [t12.check(t12.lib.t12_pack_escapes(w.data_ptr(), M, K, t.base_exp, t.row_off.data_ptr(), t.cols.data_ptr(),
                                                             t.correct.data_ptr(), t.wrong.data_ptr(), st), "escapes")
                          for w, t in zip(ws, ts) if t.P])
        res["pack_escapes"] = {"us": ms * 1e3, "GBps": (2.0 * n + 8.0 * P) / ms / 1e6}
        tot_us = res["pack_histogram"]["us"] + res["pack_planes"]["us"] + res["pack_escapes"]["us"]
        res["pack_total"] = {"us": tot_us, "Gweights_per_s": n / tot_us / 1e3}
        out[name] = res
        del ws, ts, dst, sm, gr
    head = out["gate_14336x4096"]["decompress_patched"]
    return {
        "metric": "GB/s of HBM traffic of the standalone split-12 decode (1.5 B read + 2 B written per weight, escapes exact), "
                  "gate 14336x4096 of Llama-3.1-8B",
        "value": head["GBps"], "unit": "GB/s", "n_gpus": 1, "steps": max(args.steps, 20), "warmup": 3,
        "ms_per_step": head["us"] / 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": "codec: t12_decompress and the GPU packer (histogram, planes, escapes) on gate 14336x4096, down "
                               "4096x14336, O 4096x4096; N(0,0.02)+3e-4 outliers; 3 rotating copies"},
        "tensors": out,
        "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["GBps"] / HBM_PEAK_GBS, "traffic": None, "kernel": "decompress_vec_kernel",
                     "bytes_per_launch": 3.5 * 14336 * 4096, "us_per_launch": head["us"]},
        "setup_s": time.time() - t0,
    }


def run_convert(args, t12, torch, dev):
    """Checkpoint ingestion end to end: a bf16 safetensors checkpoint of Llama-3.1-8B's layer shapes (2 layers, vocabulary
    32000, untied head: 1.4 GB) is written to a temporary directory, then convert() reads it (mmap), packs every matrix
    on the GPU and writes the engine's model directory.  `value` = GB of checkpoint per second of convert(); host file
    I/O and the PCIe copies are inside the timed region (this is the path's real boundary), the GPU packer's own rate is
    under --workload codec."""
    import importlib
    import shutil
    import tempfile
    conv = importlib.import_module(t12.__name__ + ".convert")
    st = importlib.import_module("safetensors.torch")
    n, ff, kv, V, nl = 4096, 14336, 1024, 32000, 2
    cfg = dict(hidden_size=n, num_attention_heads=32, num_key_value_heads=8, num_hidden_layers=nl, intermediate_size=ff,
               vocab_size=V, max_position_embeddings=8192, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
    src, dst = tempfile.mkdtemp(prefix="t12_ckpt_"), tempfile.mkdtemp(prefix="t12_model_")
    try:
        t0 = time.time()
        tensors = {"model.embed_tokens.weight": synth_weight(torch, V, n, 8000, dev, sigma=1.0, p_out=0.0).cpu(),
                   "model.norm.weight": torch.ones(n, dtype=torch.bfloat16),
                   "lm_head.weight": synth_weight(torch, V, n, 8001, dev).cpu()}
        for i in range(nl):
            pfx = "model.layers.%d." % i
            tensors[pfx + "input_layernorm.weight"] = torch.ones(n, dtype=torch.bfloat16)
            tensors[pfx + "post_attention_layernorm.weight"] = torch.ones(n, dtype=torch.bfloat16)
            for j, (name, (M, K)) in enumerate((("self_attn.q_proj", (n, n)), ("self_attn.k_proj", (kv, n)),
                                                ("self_attn.v_proj", (kv, n)), ("self_attn.o_proj", (n, n)),
                                                ("mlp.gate_proj", (ff, n)), ("mlp.up_proj", (ff, n)), ("mlp.down_proj", (n, ff)))):
                tensors[pfx + name + ".weight"] = synth_weight(torch, M, K, 8100 + 10 * i + j, dev).cpu()
        nbytes = sum(t.numel() * t.element_size() for t in tensors.values())
        st.save_file(tensors, os.path.join(src, "model.safetensors"))
        with open(os.path.join(src, "config.json"), "w") as f:
            json.dump(cfg, f)
        del tensors
        t_setup = time.time() - t0
        secs = []
        for _ in range(2):                                  # the second pass reads the checkpoint from the page cache
            shutil.rmtree(dst, ignore_errors=True)
            t1 = time.time()
            stats = conv.convert(src, dst, device=str(dev))
            torch.cuda.synchronize()
            secs.append(time.time() - t1)
        out_bytes = sum(os.path.getsize(os.path.join(dst, f)) for f in os.listdir(dst))
        # and the way back in: load_model on the directory just written (files in the page cache), derived escape
        # tables and the upload included
        os.environ["TURBO_CTX"] = "256"
        load_s = []
        for _ in range(2):
            t1 = time.time()
            eng = t12.Engine.load(dst, batch=1)
            torch.cuda.synchronize()
            load_s.append(time.time() - t1)
            eng.close()
    finally:
        shutil.rmtree(src, ignore_errors=True)
        shutil.rmtree(dst, ignore_errors=True)
    best = min(secs)
    return {
        "metric": "GB/s of bf16 checkpoint through convert(): safetensors -> GPU packer -> split-12 model directory",
        "value": nbytes / best / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": 2, "warmup": 0, "ms_per_step": best * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "convert: 2 Llama-3.1-8B layers + 32000 x 4096 embedding and head, bf16 safetensors, one shard",
                   "checkpoint_GB": nbytes / 1e9, "model_dir_GB": out_bytes / 1e9, "tensors": len(stats)},
        "seconds_per_pass": secs, "compression_ratio": out_bytes / nbytes,
        "load_model": {"seconds_per_pass": load_s, "GBps": out_bytes / min(load_s) / 1e9},
        "roofline": None, "setup_s": t_setup,
    }


def run_attention(args, t12, torch, dev):
    """The attention step of one Llama-3.1-8B decoder layer (RoPE of q and k, INT8 store of the new K / V
    row, GQA attention over the INT8 cache: launch_rope_store_attention), every sequence on its own cache
    region, at several (batch, context) points; `value` is the B = 256, 2000-position case on head-major regions (the
    layout of the engine's per-sequence caches) in GB/s of cache read; the same case in the reference's layout is among
    the cases."""
    import numpy as np
    nh, nkv, hd, theta = LLAMA8B["n_head"], LLAMA8B["n_head_kv"], LLAMA8B["n_embd"] // LLAMA8B["n_head"], 500000.0
    kv_dim = nkv * hd
    cur = torch.cuda.current_stream()
    g = torch.Generator(device=dev)
    g.manual_seed(77)
    # (batch, positions per region, context, head-major regions): the first three per-sequence cases also in the layout
    # the engine keeps its per-sequence caches in ([kv head][position][dim] instead of the reference's [position][kv head][dim])
    cases = [(256, 2048, 2000, False), (256, 2048, 150, False), (64, 8192, 8000, False), (16, 2048, 1000, False),
             (1, 8192, 8000, False), (1, 2048, 2000, False), (1, 2048, 150, False),
             (256, 2048, 2000, True), (256, 2048, 150, True), (64, 8192, 8000, True)]
    out_cases = {}
    for B, S, ctx, head_major in cases:
        kc = torch.randint(-127, 128, (B, S, kv_dim), dtype=torch.int8, device=dev, generator=g)
        vc = torch.randint(-127, 128, (B, S, kv_dim), dtype=torch.int8, device=dev, generator=g)
        ks = torch.rand((B, S, nkv), device=dev, generator=g) / 127 + 0.004
        vs = torch.rand((B, S, nkv), device=dev, generator=g) / 127 + 0.004
        q = torch.randn((B, nh * hd), device=dev, generator=g)
        k = torch.randn((B, kv_dim), device=dev, generator=g)
        v = torch.randn((B, kv_dim), device=dev, generator=g)
        out = torch.zeros((B, nh * hd), dtype=torch.int16, device=dev)
        pos = torch.full((B,), ctx - 1, dtype=torch.int32, device=dev)

        def step():
            head = (q.data_ptr(), k.data_ptr(), v.data_ptr(), kc.data_ptr(), vc.data_ptr(), ks.data_ptr(), vs.data_ptr(),
                    out.data_ptr(), pos.data_ptr() if B > 1 else None, ctx - 1, nh, nkv, hd, theta, 1.0 / np.sqrt(hd), B,
                    S * kv_dim if B > 1 else 0)
            if head_major:                       # (random contents: the same buffers serve as regions of either layout)
                t12.lib.launch_rope_store_attention_regions(*head, S, cur.cuda_stream)
            else:
                t12.lib.launch_rope_store_attention(*head, cur.cuda_stream)
        for _ in range(max(args.warmup, 1)):
            step()
        _, ms = timed(torch, cur, step, args.steps)
        nbytes = B * ctx * (2 * kv_dim + 8 * nkv)            # INT8 K and V rows + their fp32 scales
        out_cases["b%d_ctx%d%s" % (B, ctx, "_headmajor" if head_major else "")] = {
            "us": ms * 1e3, "cache_MB": nbytes / 1e6, "GBps": nbytes / ms / 1e6}
        del kc, vc, ks, vs
    head = out_cases["b256_ctx2000_headmajor"]           # the layout of the engine's per-sequence caches
    return {
        "metric": "GB/s of INT8 KV cache read by the decode-attention step of one Llama-3.1-8B layer, B=256 at 2000 positions "
                  "(head-major per-sequence regions)",
        "value": head["GBps"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["us"] / 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "attention: RoPE + INT8 KV store + GQA decode attention (32 / 8 heads, head_dim 128), "
                               "per-sequence cache regions, random INT8 caches"},
        "cases": out_cases,
        "roofline": {"bound": "hbm", "achieved": head["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": head["GBps"] / HBM_PEAK_GBS, "traffic": None, "kernel": "attn_fast_kernel<128,4> (long-context form)",
                     "bytes_per_launch": head["cache_MB"] * 1e6, "us_per_launch": head["us"]},
    }


def gemm_layer_leg(t12, torch, dev, cfg, weight_of, n_rot, cur, g, batches=(2, 4, 8, 16, 32, 64, 128, 256), iters=50,
                   yardstick=True):
    """decode+GEMM per layer shape: for each B, each of QKV (3 segments), O, gate|up
    (2 segments), down is timed over `n_rot` distinct weight copies in rotation, so that neither L2 nor
    the 256 MB last-level cache holds a tensor between launches.  weight_of(copy, which) -> (segment, K, P).
    Per case: 5 untimed rounds, then `iters` (>= 50) rounds each bracketed by its own pair of HIP events on the
    launch stream; the figure is the MEDIAN round divided by the launches in it."""
    iters = max(iters, 50)
    out = {}
    groups = [(0, 1, 2), (3,), (4, 5), (6,)]
    names = ["qkv", "o", "gate_up", "down"]

    def median_us(fn, launches):
        for _ in range(5):
            fn()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
        torch.cuda.synchronize()
        for e0, e1 in evs:
            e0.record(cur)
            fn()
            e1.record(cur)
        torch.cuda.synchronize()
        rounds = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
        return rounds[len(rounds) // 2] * 1e3 / launches

    if yardstick:
        # A yardstick off the product path: the vendor library's plain bf16 GEMM (torch.nn.functional.linear ->
        # hipBLASLt) on the same shapes with UNCOMPRESSED bf16 weights (2 bytes per weight from HBM, no decode), three
        # rotating copies, same timing.  It shows what a tuned dense kernel reaches on these skinny problems on this chip.
        for name, grp in zip(names, groups):
            M = sum(weight_of(0, w)[0].M for w in grp)
            K = weight_of(0, grp[0])[1]
            ws = [(torch.randn((M, K), generator=g, device=dev) * 0.02).to(torch.bfloat16) for _ in range(n_rot)]
            for B in batches:
                if B < 16:
                    continue
                x = torch.randn((B, K), generator=g, device=dev).to(torch.bfloat16)
                us = median_us(lambda: [torch.nn.functional.linear(x, w) for w in ws], n_rot)
                out["vendor_bf16_%s_b%d" % (name, B)] = {"us": round(us, 2), "mfma_frac": round(2.0 * M * K * B / us / 1e6 / 2500.0, 4),
                                                          "weight_GBps": round(2.0 * M * K / us / 1e3, 1)}
            del ws
        torch.cuda.empty_cache()
    for B in batches:
        xs = {K: torch.randn((B, K), generator=g, device=dev).to(torch.bfloat16) for K in (cfg["n_embd"], cfg["n_ff"])}
        obuf = torch.empty((B, 2 * cfg["n_ff"]), dtype=torch.float32, device=dev)
        for name, grp in zip(names, groups):
            calls, flops, wbytes = [], 0.0, 0.0
            for copy in range(n_rot):
                segs, off, K = [], 0, None
                for which in grp:
                    seg, K, P = weight_of(copy, which)
                    seg.out = obuf.data_ptr() + 4 * off
                    off += seg.M
                    segs.append(seg)
                flops, wbytes = 2.0 * off * K * B, 1.5 * off * K
                calls.append((t12._seg_array(segs), len(segs), xs[K].data_ptr(), K))

            def gemm_pass():
                for segs, n, act, K in calls:
                    rc = t12.lib.t12_gemm(segs, n, act, K, 2 * cfg["n_ff"], K, B, cur.cuda_stream)
                    if rc:
                        t12.check(rc, "t12_gemm")
            for _ in range(5):
                gemm_pass()
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
            torch.cuda.synchronize()
            for e0, e1 in evs:
                e0.record(cur)
                gemm_pass()
                e1.record(cur)
            torch.cuda.synchronize()
            rounds = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
            us = rounds[len(rounds) // 2] * 1e3 / n_rot
            out["%s_b%d" % (name, B)] = {"us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 1),
                                         "mfma_frac": round(flops / us / 1e6 / 2500.0, 4),
                                         "weight_GBps": round(wbytes / us / 1e3, 1), "flops": flops}
        if B > 64:
            # gate|up the way the engine's layer runs it: SiLU*mul in the GEMM's epilogue, bf16 [B, n_ff] out
            # (t12_gemm_swiglu); same flops, 14.7 MB written at B = 256 instead of 58.7 MB
            abuf = torch.empty((B, cfg["n_ff"]), dtype=torch.int16, device=dev)
            pairs = []
            for copy in range(n_rot):
                sg, K, _ = weight_of(copy, 4)
                su, _, _ = weight_of(copy, 5)
                pairs.append((t12._seg_array([sg]), t12._seg_array([su]), K))
            flops = 2.0 * 2 * cfg["n_ff"] * cfg["n_embd"] * B

            def swiglu_pass():
                for sg, su, K in pairs:
                    rc = t12.lib.t12_gemm_swiglu(sg, su, xs[K].data_ptr(), K, K, B, abuf.data_ptr(), cfg["n_ff"], cur.cuda_stream)
                    if rc:
                        t12.check(min(rc, 0), "t12_gemm_swiglu")
                        raise RuntimeError("t12_gemm_swiglu has no kernel for B = %d" % B)
            for _ in range(5):
                swiglu_pass()
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
            torch.cuda.synchronize()
            for e0, e1 in evs:
                e0.record(cur)
                swiglu_pass()
                e1.record(cur)
            torch.cuda.synchronize()
            rounds = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
            us = rounds[len(rounds) // 2] * 1e3 / n_rot
            out["gate_up_swiglu_b%d" % B] = {"us": round(us, 2), "TFLOPs": round(flops / us / 1e6, 1),
                                             "mfma_frac": round(flops / us / 1e6 / 2500.0, 4),
                                             "weight_GBps": round(1.5 * 2 * cfg["n_ff"] * cfg["n_embd"] / us / 1e3, 1),
                                             "flops": flops}
    return out


def clock_probe(t12):
    """Shader clock and MFMA rate under load (t12_probe_clock): MFMA only, and MFMA with the decode / LDS work of a
    decode+GEMM stage beside it, on 64 / 128 / 256 workgroups of eight waves.  The published 2.5 PFLOP/s is priced at
    2.4 GHz; the chip lowers its clock with the activity of the launch."""
    import ctypes as C
    out = {}
    for mix, name in ((0, "mfma_only"), (1, "mfma_decode_lds")):
        for wgs in (64, 128, 256):
            ghz, tf = C.c_double(), C.c_double()
            rc = t12.lib.t12_probe_clock(wgs, 20000, mix, C.byref(ghz), C.byref(tf), t12.current_stream())
            if rc:
                t12.check(rc, "t12_probe_clock")
            out["%s_%dwg" % (name, wgs)] = {"ghz": round(ghz.value, 3), "TFLOPs": round(tf.value, 1)}
    return out


def gemm_b256_roofline(layers):
    names = ("qkv", "o", "gate_up", "down")
    us = sum(layers["%s_b256" % k]["us"] for k in names)
    fl = sum(layers["%s_b256" % k]["flops"] for k in names)
    extra = {}
    if "vendor_bf16_gate_up_b256" in layers:
        vus = sum(layers["vendor_bf16_%s_b256" % k]["us"] for k in names)
        extra = {"vendor_bf16_frac": fl / vus / 1e6 / 2500.0, "vendor_bf16_us_per_step": vus,
                 "vendor_bf16_gate_up_frac": layers["vendor_bf16_gate_up_b256"]["mfma_frac"]}
    return {**extra, "bound": "mfma", "achieved": fl / us / 1e6, "peak": 2500.0, "unit": "TFLOP/s", "frac": fl / us / 1e6 / 2500.0,
            "traffic": None, "gate_up_traffic": measured_traffic("gemm_gate_up_b256"),
            "kernel": "gemm_mfma_kernel, QKV + O + gate|up + down at B=256", "flops_per_step": fl,
            "us_per_step": us, "gate_up_frac": layers["gate_up_b256"]["mfma_frac"],
            # the same four products as the engine's layer issues them: gate|up with SiLU*mul in its epilogue
            "gate_up_swiglu_frac": layers["gate_up_swiglu_b256"]["mfma_frac"],
            "frac_with_swiglu_epilogue": fl / (us - layers["gate_up_b256"]["us"] + layers["gate_up_swiglu_b256"]["us"]) / 1e6 / 2500.0}


def run_tokenizer(args, t12):
    """Encoding throughput of the tokenizer (host code, no GPU): seeded word list, the merge table that builds its
    words, text of those words."""
    import importlib
    import random
    import tempfile

    tf = importlib.import_module(t12.__name__ + ".tokenizer_files")
    rng = random.Random(1234)
    letters = b"etaoinshrldcumwfgypbvk"
    words = sorted({bytes(rng.choice(letters) for _ in range(rng.randint(2, 11))) for _ in range(4000)})
    merges, seen = [], set()
    for w in words:                          # a word is built left to right: (w0, w1), (w0w1, w2), ...
        for i in range(1, len(w)):
            pair = (w[:i], w[i:i + 1])
            if pair not in seen:
                seen.add(pair)
                merges.append(pair)
    rng.shuffle(merges)
    merges.sort(key=lambda m: len(m[0]))     # every merge after the one that builds its left part
    toks = [b"<unk>", b"<s>", b"</s>"] + sorted({bytes([c]) for c in letters + b" "} | {a + b for a, b in merges})
    text = b" ".join(rng.choice(words) for _ in range(150000))
    with tempfile.TemporaryDirectory() as d:
        tf.write_files(d, toks, merges, 1, 2, None)
        tok = t12.Tokenizer(d)
        steps = max(args.steps, 3)
        for _ in range(max(args.warmup, 1)):
            ids = tok.tokenize(text)
        t0 = time.time()
        for _ in range(steps):
            ids = tok.tokenize(text)
        dt = (time.time() - t0) / steps
        cpu = None
        if not args.no_cpu_baseline:
            from oracle.tokenizer_oracle import RefTokenizer
            ref = RefTokenizer(d)
            sample = text[:4096]
            t1 = time.time()
            want = ref.tokenize(sample)
            t_ref = time.time() - t1
            assert tok.tokenize(sample) == want, "tokenizer differs from the reference rule"
            cpu = {"value": len(sample) / t_ref / 1e6, "unit": "MB/s of text", "cores": 1, "kind": "port",
                   "sample": "first 4 KB of the same text, same merge table, reference rule restated in Python "
                             "(one pass over the text per merge; its cost grows with text length x merges)"}
        tok.close()
    return {"metric": "byte-level BPE encoding throughput (host)", "value": len(text) / dt / 1e6, "unit": "MB/s of text",
            "n_gpus": 1, "steps": steps, "warmup": max(args.warmup, 1), "ms_per_step": dt * 1e3, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "tokenizer: %d bytes of text, %d merges, %d ids out" % (len(text), len(merges), len(ids))},
            "roofline": None, "cpu_baseline": cpu}


def reference_named_leg(t12, torch, dev, copies_gate, cur, g, iters):
    """launch_split12_batch4/8_async (the reference's own small-batch entry points, escapes as the derived tables of its
    loader) on the gate tensor, three rotating copies, next to t12_gemm on the same tensors and batch."""
    import numpy as np
    M, K = copies_gate[0].M, copies_gate[0].K

    def tables(t):
        ro, cols, cor = t.row_off.cpu().numpy(), t.cols.cpu().numpy(), t.correct.cpu().numpy()
        rows = np.repeat(np.arange(M), np.diff(ro))
        order = np.lexsort((cols, cols % 256, rows))            # (row, col % 256, ascending col): engine/model.cpp:92-125
        return [torch.from_numpy(a).to(dev) for a in (ro[:-1].astype(np.int32).copy(), cor[order].copy())]
    tabs = [tables(t) for t in copies_gate]
    out = {}
    for NB in (4, 8):
        X = torch.randn((NB, K), device=dev, generator=g).to(torch.bfloat16).view(torch.int16)
        outs = [torch.zeros(M, device=dev) for _ in range(NB)]
        fn = t12.lib.launch_split12_batch4_async if NB == 4 else t12.lib.launch_split12_batch8_async

        def named():
            for t, (rb, vl) in zip(copies_gate, tabs):
                t12.check(fn(*([t.sm.data_ptr(), t.gr.data_ptr(), t.base_exp] + [X[j].data_ptr() for j in range(NB)] +
                               [rb.data_ptr(), None, vl.data_ptr()] + [o.data_ptr() for o in outs] + [M, K, cur.cuda_stream])))
        dense = torch.zeros((NB, M), device=dev)

        def own():
            for t in copies_gate:
                t12.gemm([t], X, outs=[dense])
        for name, fn_ in (("launch_split12_batch%d_async" % NB, named), ("t12_gemm_b%d" % NB, own)):
            for _ in range(3):
                fn_()
            _, ms = timed(torch, cur, fn_, iters)
            us = ms * 1e3 / len(copies_gate)
            out[name] = {"us": round(us, 2), "weight_GBps": round(1.5 * M * K / us / 1e3, 1)}
    return out


def run_gemm_layers(args, t12, torch, dev):
    """The four Llama-3.1-8B linear-layer shapes through the fused decode+GEMM at B = 2 .. 256 on three rotating weight
    copies, the vendor library's plain bf16 GEMM on the same shapes as a yardstick, the same launch on half and a
    quarter of its row tiles, and the shader clock under load; one step = the four layer GEMMs of one decoder layer at
    B = 256."""
    cfg = dict(LLAMA8B)
    n, ff = cfg["n_embd"], cfg["n_ff"]
    kv = cfg["n_head_kv"] * (n // cfg["n_head"])
    shapes = [(n, n), (kv, n), (kv, n), (n, n), (ff, n), (ff, n), (n, ff)]       # wq wk wv wo gate up down
    t0 = time.time()
    copies = [[t12.pack_device(synth_weight(torch, M, K, 2000 + 10 * c + i, dev)) for i, (M, K) in enumerate(shapes)]
              for c in range(3)]
    torch.cuda.synchronize()
    t_build = time.time() - t0

    def weight_of(copy, which):
        t = copies[copy][which]
        return t.segment(None), t.K, t.P
    g = torch.Generator(device=dev)
    g.manual_seed(2100)
    cur = torch.cuda.current_stream()
    if args.calibrate:
        calibration_copy(torch, dev)
    layers = gemm_layer_leg(t12, torch, dev, cfg, weight_of, 3, cur, g, iters=max(args.steps, 50))
    probe = clock_probe(t12)
    named = reference_named_leg(t12, torch, dev, [copies[c][4] for c in range(3)], cur, g, 20)
    us256 = sum(layers["%s_b256" % k]["us"] for k in ("qkv", "o", "gate_up", "down"))
    fl256 = sum(layers["%s_b256" % k]["flops"] for k in ("qkv", "o", "gate_up", "down"))
    gu = layers["gate_up_b256"]
    return {
        "metric": "decode+GEMM TFLOP/s at B=256 over the linear layers of one Llama-3.1-8B decoder layer (split-12 weights)",
        "value": fl256 / us256 / 1e6, "unit": "TFLOP/s", "n_gpus": 1, "steps": max(args.steps, 50), "warmup": 5,
        "ms_per_step": us256 / 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "gemm_layers: QKV 4096->6144 (3 segments), O 4096->4096, gate|up 4096->28672 (2 segments), "
                               "down 14336->4096; N(0,0.02)+3e-4 outliers; B in {2,4,8,16,32,64,128,256}; 3 rotating weight copies"},
        "layers": layers,
        "clock_probe": probe,
        "reference_named_launchers_gate_14336x4096": named,
        "roofline": {"bound": "mfma", "achieved": gu["TFLOPs"], "peak": 2500.0, "unit": "TFLOP/s",
                     "frac": gu["TFLOPs"] / 2500.0, "traffic": measured_traffic("gemm_gate_up_b256"),
                     "kernel": "gemm_mfma_kernel<4,2,2,2> on gate|up at B=256", "flops_per_launch": gu["flops"],
                     "us_per_launch": gu["us"],
                     "vendor_bf16_gemm_frac": layers.get("vendor_bf16_gate_up_b256", {}).get("mfma_frac"),
                     "clock_ghz_mfma_decode_lds_256wg": probe["mfma_decode_lds_256wg"]["ghz"],
                     "clock_ghz_mfma_only_256wg": probe["mfma_only_256wg"]["ghz"]},
        "setup_s": t_build,
    }


def emit(result, json_fd):
    """The ONE line of standard output.  Descriptor 1 was pointed at standard error for the whole run (the native
    library reports model and cache sizes with printf); json_fd is the original descriptor 1."""
    import ctypes
    sys.stdout.flush()
    ctypes.CDLL(None).fflush(None)           # the C library's own buffer, while descriptor 1 still points away
    os.write(json_fd, (json.dumps(result) + "\n").encode())


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="decode", choices=["decode", "gemv_stack_b1", "moe", "gemm_layers", "attention", "codec", "convert", "tokenizer"])
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--no-batch256", dest="batch256", action="store_false")
    ap.add_argument("--layers", type=int, default=LLAMA8B["n_layer"], help="debug: fewer layers (invalid as a result)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--probes", action="store_true",
                    help="gemv_stack_b1: after the timed steps also measure what could fill the time between launches (one "
                         "tensor launched repeatedly, two independent passes on two streams, a chain of idle kernels); "
                         "off by default so that a kernel trace of the workload holds the stack's launches only")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch one plain 1 GiB copy kernel (a torch tensor copy) before the steps: the known-size "
                         "yardstick for the profiler's FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no collective); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    json_fd = os.dup(1)
    os.dup2(2, 1)
    import torch
    import __graft_entry__ as ge
    t12 = ge.load_package()
    if args.workload == "tokenizer":
        emit(run_tokenizer(args, t12), json_fd)
        return
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "decode":
        emit(run_decode(args, t12, torch, dev), json_fd)
        return
    if args.workload == "gemm_layers":
        emit(run_gemm_layers(args, t12, torch, dev), json_fd)
        return
    if args.workload == "moe":
        emit(run_moe(args, t12, torch, dev), json_fd)
        return
    if args.workload == "attention":
        emit(run_attention(args, t12, torch, dev), json_fd)
        return
    if args.workload == "codec":
        emit(run_codec(args, t12, torch, dev), json_fd)
        return
    if args.workload == "convert":
        emit(run_convert(args, t12, torch, dev), json_fd)
        return
    cfg = dict(LLAMA8B, n_layer=args.layers)

    t0 = time.time()
    launches = build_stack(t12, torch, dev, cfg)
    torch.cuda.synchronize()
    t_build = time.time() - t0

    g = torch.Generator(device=dev)
    g.manual_seed(99)
    acts = {"h": torch.randn(cfg["n_embd"], generator=g, device=dev).to(torch.bfloat16),
            "ff": torch.randn(cfg["n_ff"], generator=g, device=dev).to(torch.bfloat16)}
    outs = [[torch.empty(t.M, dtype=torch.float32, device=dev) for t in tensors] for tensors, _ in launches]
    stream = t12.current_stream()
    # segment tables are built once; a step is pure launches
    seg_tabs = [(t12._seg_array([t.segment(o) for t, o in zip(tensors, out)]), len(tensors), acts[key].data_ptr(),
                 tensors[0].K) for (tensors, key), out in zip(launches, outs)]

    def step():
        for segs, n, act, K in seg_tabs:
            rc = t12.lib.t12_gemv(segs, n, act, K, stream)
            if rc:
                t12.check(rc, "t12_gemv")

    if args.calibrate:
        calibration_copy(torch, dev)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    w0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - w0) * 1e3 / args.steps
    ms = e0.elapsed_time(e1) / args.steps          # HIP events on the launch stream
    ms_step = max(ms, wall_ms)

    probes = None
    if args.probes:
        # ---- what could fill the time between two launches (about 3 us per launch, a fifth of the stack)?
        #   same_tensor: one launch repeated on ONE weight copy -- were the last-level cache to serve it, the repeat would beat
        #                the rotating stack's rate for that shape;
        #   two_streams: two independent passes of the stack interleaved on two streams -- the rate when a second, independent
        #                launch is there to run in the gaps (a decode step has none: each launch reads the previous one's output)
        def rate(fn, nbytes, reps):
            for _ in range(2):
                fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(reps):
                fn()
            b.record()
            torch.cuda.synchronize()
            return nbytes * reps / (a.elapsed_time(b) * 1e-3) / 1e9

        probes = {}
        for idx, name in ((0, "qkv"), (1, "o"), (2, "gate_up"), (3, "down")):
            segs, n, act, K = seg_tabs[idx]
            nb = sum(1.5 * t.M * t.K for t in launches[idx][0])

            def same():
                for _ in range(20):
                    t12.lib.t12_gemv(segs, n, act, K, stream)
            probes["same_tensor_%s_GBps" % name] = round(rate(same, 20 * nb, 5), 1)
        side = torch.cuda.Stream()
        outs2 = [[torch.empty(t.M, dtype=torch.float32, device=dev) for t in tensors] for tensors, _ in launches]
        seg_tabs2 = [(t12._seg_array([t.segment(o) for t, o in zip(tensors, out)]), len(tensors), acts[key].data_ptr(),
                      tensors[0].K) for (tensors, key), out in zip(launches, outs2)]
        plane_all = sum(1.5 * t.M * t.K for tensors, _ in launches for t in tensors)

        def two():
            for a_, b_ in zip(seg_tabs, seg_tabs2):
                t12.lib.t12_gemv(a_[0], a_[1], a_[2], a_[3], stream)
                t12.lib.t12_gemv(b_[0], b_[1], b_[2], b_[3], side.cuda_stream)
            torch.cuda.current_stream().wait_stream(side)
        side.wait_stream(torch.cuda.current_stream())
        probes["two_streams_two_passes_GBps"] = round(rate(two, 2 * plane_all, 3), 1)
        #   launch interval: a chain of kernels that do nothing, in stream order (what every dependent launch of a decode step
        #   pays at least) and with the ordering between them lifted (hipExtAnyOrderLaunch: no option for dependent launches)
        import ctypes as C
        for key, any_order in (("idle_kernel_chain_us_per_launch", 0), ("idle_kernel_chain_any_order_us_per_launch", 1)):
            us = C.c_double()
            rc = t12.lib.t12_probe_launch_gap(2000, any_order, C.byref(us), stream)
            if rc:
                t12.check(rc, "t12_probe_launch_gap")
            probes[key] = round(us.value, 2)

    n_launch = len(launches)
    alg_bytes = sum(algorithmic_bytes(t) for tensors, _ in launches for t in tensors)
    plane_bytes = sum(1.5 * t.M * t.K for tensors, _ in launches for t in tensors)
    n_weights = sum(t.M * t.K for tensors, _ in launches for t in tensors)
    achieved = alg_bytes / (ms * 1e-3) / 1e9       # GB/s, per-launch bytes / per-launch duration
    result = {
        "metric": "tok/s at B=1 (Llama-3.1-8B shape), split-12 decode-GEMV over every linear layer of a decode step",
        "value": 1e3 / ms_step, "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "shape": "Llama-3.1-8B", "batch": 1, "n_layer": cfg["n_layer"],
                   "weights": n_weights, "launches_per_step": n_launch,
                   "compressed_GB_per_step": plane_bytes / 1e9, "escape_fraction":
                       sum(t.P for tensors, _ in launches for t in tensors) / n_weights},
        "gemv_compressed_GBps": plane_bytes / (ms * 1e-3) / 1e9,
        "gap_probes": probes,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": measured_traffic(args.workload) if cfg["n_layer"] == LLAMA8B["n_layer"] else None,
                     "kernel": "gemv_stream_kernel", "bytes_per_launch": alg_bytes / n_launch,
                     "us_per_launch": ms * 1e3 / n_launch},
        "setup_s": t_build,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch, launches, cfg)
    emit(result, json_fd)


if __name__ == "__main__":
    main()
