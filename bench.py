#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one greedy decode step (one new token) of the Llama-2 110M-shape
decoder (dim 768, 12 layers, 12 heads x 64, FFN 2048 SwiGLU, vocab 32000, seq 1024;
random-init N(0, 0.02) fp32 weights, 128 seeded prompt ids), run by the llama2
extension library through the C ABI.  A generation forces the 128 prompt ids, runs W
untimed greedy steps and then timed greedy steps up to position 1023; the defaults
(W = 16, K = 880) are exactly one generation to 1024 tokens.  A larger K continues with
further generations (fresh seeded prompts) until exactly K steps have been timed with
HIP events on the engine's stream.

The single JSON line also carries:
  roofline      the timed unit itself: one decode step (a replay of the captured graph
                of 62 dispatches) against HBM peak, from the HIP-event time of the timed
                region, with a per-kernel-class breakdown from event pairs;
  cpu_baseline  the CPU checker (restatement of the reference's llama2 C++ forward)
                timed on this host's cores on a bounded sample of the same workload;
  also          the other named kernels at their benchmark shapes, each with its own
                roofline entry: fused prefill attention (B=8, T=1024, 12 x 64), decode
                attention over a KV cache (32 x 128, L up to 4096, batch up to 32), the
                encoder-decoder attention shapes with padding masks, the QKV / projection
                GEMMs, batch-16 and bf16-weight decode.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}

C4 = dict(dim=768, hidden_dim=2048, n_layers=12, n_heads=12, n_kv_heads=12, vocab_size=32000, seq_len=1024)
N_PROMPT = 128


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_checkpoint(cfg, seed, path):
    from mycaffe_amd import checkpoint as C
    blob = C.random_model(cfg, seed, shared_classifier=False, std=0.02)
    if not os.path.exists(path):
        C.write_v1(path, cfg, blob, False)
    return blob


def weight_bytes(cfg, es):
    L, dim, hid, V = cfg["n_layers"], cfg["dim"], cfg["hidden_dim"], cfg["vocab_size"]
    kvd = dim // cfg["n_heads"] * cfg["n_kv_heads"]
    return (L * ((dim + 2 * kvd) * dim + dim * dim + 3 * hid * dim) + V * dim) * es


def run_decode(cuda, path, bf16, batch, steps, warmup, seed=1, graph=True, kv_bf16=False):
    """Times exactly `steps` greedy decode steps (see the module docstring); returns the engine and the figures."""
    from mycaffe_amd.llm_inference import LlmInference
    inf = LlmInference(cuda)
    inf.Initialize(fTemperature=0.0)
    inf.SetOption(1, 1 if bf16 else 0)
    inf.SetOption(3, 1 if graph else 0)
    inf.SetOption(8, 1 if kv_bf16 else 0)
    inf.Load(path)
    per_gen = C4["seq_len"] - N_PROMPT - warmup
    left, ms_total, wall, gen = steps, 0.0, 0.0, 0
    first = None
    # one short untimed generation first: buffers allocated, kernels loaded, the step graph captured
    wp = np.random.default_rng(seed + 999).integers(3, C4["vocab_size"], (batch, N_PROMPT))
    inf.GenerateIds(wp[0], N_PROMPT + 4) if batch == 1 else inf.GenerateBatch(wp, N_PROMPT + 4)
    while left > 0:
        k = min(left, per_gen)
        rng = np.random.default_rng(seed + gen)
        total = N_PROMPT + warmup + k
        inf.SetOption(2, N_PROMPT + warmup)
        t0 = time.perf_counter()
        if batch == 1:
            prompt = rng.integers(3, C4["vocab_size"], N_PROMPT)
            ids = inf.GenerateIds(prompt, total)
        else:
            prompt = rng.integers(3, C4["vocab_size"], (batch, N_PROMPT))
            ids = inf.GenerateBatch(prompt, total)
        wall += time.perf_counter() - t0
        ms, nsteps = inf.QueryTiming()
        assert nsteps == k, (nsteps, k)
        ms_total += ms
        left -= k
        if first is None:
            first = (prompt, ids, inf.LastPrefill(), inf.LastRunUsedGraph())
        gen += 1
    res = {"ms_per_step": ms_total / steps, "tokens_per_s": batch * steps / (ms_total / 1e3), "wall_s_whole_generation": wall,
           "prompt": first[0], "ids": first[1], "generations": gen, "prefill_ms": first[2][0], "prefill_rows": first[2][1],
           "graph": first[3]}
    return inf, res


def bench_sampled_generation(cuda, path, steps=192):
    """Temperature 0.8, top-p 0.9 and plain multinomial, fp32 weights, one sequence: the reference samples on the host after
    a copy of the logits, at every position, the prompt's included (llm.cpp:231, llama2_sampler.cpp:126-151).  Reported
    per sampler placement: milliseconds per generated position, and the time to get through the 128 prompt positions -
    one batched pass with the device sampler (every row takes its own draw), one step per position with the host's."""
    from mycaffe_amd.llm_inference import LlmInference
    out = {}
    prompt = np.random.default_rng(17).integers(3, C4["vocab_size"], N_PROMPT)
    for topp, tag in ((0.9, "top_p_0.9"), (0.0, "multinomial")):
        for dev in (1, 0):
            inf = LlmInference(cuda)
            inf.Initialize(fTemperature=0.8, fTopp=topp, lSeed=1)
            inf.SetOption(5, 1)
            inf.SetOption(11, dev)
            inf.Load(path)
            inf.GenerateIds(prompt, N_PROMPT + 8)
            inf.SetOption(2, N_PROMPT)
            inf.GenerateIds(prompt, N_PROMPT + steps)
            ms, n = inf.QueryTiming()
            pre_ms, rows = inf.LastPrefill()
            if not rows:
                # the prompt went one step per position: time those steps
                inf.SetOption(2, 0)
                inf.GenerateIds(prompt, N_PROMPT)
                pre_ms = inf.QueryTiming()[0]
            out["%s_%s" % (tag, "device_sampler" if dev else "host_sampler")] = {
                "ms_per_position": round(ms / n, 4), "prompt_128_positions_ms": round(pre_ms, 3), "prompt_as_one_pass": bool(rows)}
            inf.CleanUp()
    return out


def prefill_summary(r, batch, es):
    """The batched prompt pass of one generation: HIP-event time, prompt tokens per second, and the model flops per second
    (2 x matrix parameters x rows, the classifier included, plus the causal half of the attention products) as a fraction
    of the peak of the matrix cores the GEMMs run on: fp32 for fp32 weights and for the few-row path, bf16 for 16-bit
    weights over more than 256 rows (where the default pass spends two bf16 products per model product)."""
    if not r["prefill_rows"]:
        return None
    rows, P = r["prefill_rows"], r["prefill_rows"] // batch
    dim, L, H = C4["dim"], C4["n_layers"], C4["n_heads"]
    flops = 2.0 * (weight_bytes(C4, 1)) * rows + L * 2.0 * batch * H * P * P * (dim // H)
    tf = flops / (r["prefill_ms"] / 1e3) / 1e12
    out = {"ms": round(r["prefill_ms"], 4), "prompt_tokens": rows, "prompt_tokens_per_s": round(rows / (r["prefill_ms"] / 1e3), 1),
           "TFLOPs": round(tf, 2)}
    if es == 2 and rows > 256:
        out["frac_mfma_bf16"] = round(tf / MFMA_PEAK_TFLOPS["bf16"], 4)
    else:
        out["frac_mfma_f32"] = round(tf / MFMA_PEAK_TFLOPS["f32"], 4)
    return out


STEADY_MS = 100.0


def timed(cuda, fn, rgf, rgl, warm, reps):
    """Mean ms of `reps` back-to-back dispatches at steady clocks.  The GPU's clocks ramp for some 40 ms after an idle gap:
    the 28 us causal attention launch measures 28.4 us over the first 2 ms after one and 24.9 us from 40 ms on, the 0.6 ms
    long-context one 0.76 against 0.61 ms.  Every section starts after host-side allocation and upload (such a gap), so
    the timed dispatches follow at least STEADY_MS milliseconds of the same dispatches, untimed."""
    if STEADY_MS <= 0:
        return cuda.TimeFunction(fn, rgf, rgl, warm, reps)
    est = cuda.TimeFunction(fn, rgf, rgl, 1, 3)
    chunk = int(min(5000, max(1, 10.0 / max(est, 1e-4))))      # about 10 ms of dispatches per library call
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < STEADY_MS:
        cuda.TimeFunction(fn, rgf, rgl, 0, chunk)
    return cuda.TimeFunction(fn, rgf, rgl, warm, reps)


def recorded_traffic(key):
    """HBM bytes per launch from the committed counter summary (FETCH_SIZE + WRITE_SIZE runs, calibrated on a
    known-size kernel); None when the summary has no entry for `key`."""
    try:
        for line in open(os.path.join(ROOT, "profiles", "hbm_traffic_counters.txt")):
            if line.startswith("traffic_bytes_per_launch:"):
                for item in line.split(":", 1)[1].split():
                    k, v = item.split("=")
                    if k == key:
                        return int(v)
    except OSError:
        pass
    return None


def timed_sets(cuda, fn, rgf, rgl_sets, warm, reps):
    """`timed` over several argument lists taken in turn (operands that do not stay in the caches between repeats)."""
    if STEADY_MS > 0:
        est = cuda.TimeFunctionSets(fn, rgf, rgl_sets, 1, 3)
        chunk = int(min(5000, max(1, 10.0 / max(est, 1e-4))))
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < STEADY_MS:
            cuda.TimeFunctionSets(fn, rgf, rgl_sets, 0, chunk)
    return cuda.TimeFunctionSets(fn, rgf, rgl_sets, warm, max(reps, 2 * len(rgl_sets)))


def step_roofline(inf, head, steps, warmup):
    """Roofline of the timed unit, one decode step (one replay of the captured graph: 62 dispatches that stream
    every weight once and the KV cache of the current length), from the HIP-event time of the timed region.
    per_class: HIP event pairs around each launch of eager steps at the first timed position; every pair also
    contains the dispatch cost that the pair around an empty kernel shows."""
    first = N_PROMPT + warmup
    n_first = min(steps, C4["seq_len"] - first)
    mean_len = first + 1 + (n_first - 1) / 2.0          # cached positions read per step, averaged over a generation
    kvd = C4["dim"] // C4["n_heads"] * C4["n_kv_heads"]
    nbytes = weight_bytes(C4, 4) + C4["n_layers"] * 2 * mean_len * kvd * 4
    us = head["ms_per_step"] * 1e3
    achieved = nbytes / (us * 1e-6) / 1e9
    prof = inf.ProfileStep(first, 16)
    pair_ms = prof.pop("_event_pair_ms")
    detail = {k: {"us_per_launch": round(v[0] / v[1] * 1e3, 3), "launches_per_step": v[1],
                  "algorithmic_MB_per_launch": round(v[2] / v[1] / 1e6, 3) if v[2] > 0 else None}
              for k, v in prof.items() if v[1] > 0}
    how = "one replay of the captured graph" if head.get("graph") else "62 eager launches (no graph: asked for, or capture failed)"
    return {"kernel": "decode step = %s (37 matvec_kernel, 12 attn_decode_fused_step_kernel, 12 matvec_merge_kernel, 1 sample_advance_kernel)" % how,
            "graph_replay": bool(head.get("graph")),
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": recorded_traffic("decode_step"),
            "traffic_note": "counter runs cover a step at position 512 (475.9 MB algorithmic there); the timed steps ran at the positions given",
            "traffic_position": 512, "traffic_algorithmic_bytes_at_that_position": 475900000,
            "timed_positions_first": first, "timed_positions_last": first + n_first - 1,
            "algorithmic_bytes_per_launch": round(nbytes), "avg_launch_us": round(us, 3), "dispatches_per_launch": 62,
            "event_pair_around_empty_kernel_us": round(pair_ms * 1e3, 3), "per_class_event_pairs": detail}


def cpu_baseline(blob, gpu_prompt, gpu_ids, budget_s=12.0):
    """The CPU checker on this host's cores: whole generations of the same workload (128 forced ids, then greedy
    to 1024 positions), repeated until about `budget_s` seconds of CPU work; every position counts as one token
    (the reference loop spends the same work on a forced position as on a sampled one)."""
    from oracle import llama2 as O
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    n = C4["seq_len"]
    tokens, dt, runs, same = 0, 0.0, 0, None
    while dt < budget_s and runs < 8:
        m = O.Llama(C4, blob, False)
        prompt = gpu_prompt if runs == 0 else np.random.default_rng(100 + runs).integers(3, C4["vocab_size"], N_PROMPT)
        t0 = time.perf_counter()
        ids = m.generate_greedy(prompt, n)
        dt += time.perf_counter() - t0
        tokens += n
        if runs == 0 and gpu_ids is not None:
            k = min(len(gpu_ids), len(ids))
            diff = np.nonzero(np.asarray(ids[:k]) != np.asarray(gpu_ids[:k]).reshape(-1)[:k])[0]
            same = {"positions_compared": int(k), "first_mismatch": int(diff[0]) if diff.size else None}
        runs += 1
        del m
    # the same loop on one thread, over a shorter sample (64 forced ids, then greedy to 96 positions)
    prev = O.set_threads(1)
    m = O.Llama(C4, blob, False)
    t0 = time.perf_counter()
    m.generate_greedy(np.asarray(gpu_prompt[:64]), 96)
    one = 96 / (time.perf_counter() - t0)
    O.set_threads(prev)
    del m
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            model = next((ln.split(":", 1)[1].strip() for ln in f if ln.startswith("model name")), "")
    except OSError:
        pass
    return {"value": round(tokens / dt, 3), "unit": "tokens/s", "cores": threads, "kind": "port",
            "cpu_model": model, "one_thread_tokens_per_s": round(one, 3), "one_thread_sample": "positions 0..95 of one generation",
            "sample": "%d whole generation(s) of the same workload (128 forced prompt ids, then greedy to 1024 positions; "
                      "fp32, batch 1), %d positions in %.1f s, every position counted" % (runs, tokens, dt),
            "ids_vs_gpu_first_generation": same}


def bench_prefill_attention(cuda, reps, warm=5, shape=(8, 12, 1024, 64), dtypes=(("bf16", True), ("f32", False)), causal=True):
    """Fused attention through ATTN_FWD (id 163): B=8, T=1024, 12 heads x 64 unless another shape is given; causal
    (the (T,T) lower-triangular mask) or without a mask."""
    from mycaffe_amd.cudadnn import CUDAFN
    B, H, T, hs = shape
    rng = np.random.default_rng(0)
    out = {}
    mask = cuda.AllocMemory(np.tril(np.ones((T, T), np.float32))) if causal else 0
    hc, ha = cuda.CreateCuDNN(), cuda.CreateAttn()
    cuda.SetAttn(hc, ha, 0, False, B, T, H, hs, 0.0)
    for name, half in dtypes:
        hs_ = [cuda.AllocMemory(rng.standard_normal(B * H * T * hs).astype(np.float32), bHalfSize=half) for _ in range(3)]
        hy = cuda.AllocMemory(B * H * T * hs, bHalfSize=half)
        rgl = [hc, ha, T, hs_[0], hs_[1], hs_[2], mask, hy, 0]
        cuda.AttnScaledDotProductForward(hc, ha, T, hs_[0], hs_[1], hs_[2], mask, hy, False)
        ms = timed(cuda, CUDAFN.CUDA_ATTN_FWD, None, rgl, warm, reps)
        useful = 2.0 * B * H * T * T * hs          # causal half of the 4*B*H*T*T*hs full-square flops
        tf = useful / (ms / 1e3) / 1e12
        if not causal:
            out[name] = {"ms": round(ms, 4), "TFLOPs": round(2 * tf, 2), "frac_mfma": round(2 * tf / MFMA_PEAK_TFLOPS[name], 4)}
            for h in hs_ + [hy]:
                cuda.FreeMemory(h)
            continue
        out[name] = {"ms": round(ms, 4), "TFLOPs_causal_useful": round(tf, 2), "TFLOPs_full_square": round(2 * tf, 2),
                     "roofline": {"kernel": "fused causal attention forward", "bound": "mfma", "achieved": round(tf, 2),
                                  "peak": MFMA_PEAK_TFLOPS[name], "unit": "TFLOP/s",
                                  "frac": round(tf / MFMA_PEAK_TFLOPS[name], 4),
                                  "traffic": recorded_traffic("flash_" + name if shape == (8, 12, 1024, 64) else
                                                               "flash_%s_B%d_T%d_%dx%d" % (name, B, T, H, hs))}}
        for h in hs_ + [hy]:
            cuda.FreeMemory(h)
    if mask:
        cuda.FreeMemory(mask)
    return out


def bench_attention_backward(cuda, reps, warm=5):
    """Gradients of the fused causal attention at B=8, T=1024, 12 heads x 64 through ATTN_BWD (id 164): the dQ kernel (which also
    produces the per-row dY.Y sums) and the dK/dV kernel of one call."""
    from mycaffe_amd.cudadnn import CUDAFN
    B, H, T, hs = 8, 12, 1024, 64
    rng = np.random.default_rng(0)
    out = {}
    mask = cuda.AllocMemory(np.tril(np.ones((T, T), np.float32)))
    hc, ha = cuda.CreateCuDNN(), cuda.CreateAttn()
    cuda.SetAttn(hc, ha, 0, True, B, T, H, hs, 0.0)
    n = B * H * T * hs
    for name, half in (("bf16", True), ("f32", False)):
        q, k, v, dy = (cuda.AllocMemory(rng.standard_normal(n).astype(np.float32), bHalfSize=half) for _ in range(4))
        y, dq, dk, dv = (cuda.AllocMemory(n, bHalfSize=half) for _ in range(4))
        cuda.AttnScaledDotProductForward(hc, ha, T, q, k, v, mask, y, False)
        rgl = [hc, ha, q, dq, k, dk, v, dv, mask, y, dy]
        cuda.AttnScaledDotProductBackward(hc, ha, q, dq, k, dk, v, dv, mask, y, dy)
        ms = timed(cuda, CUDAFN.CUDA_ATTN_BWD, None, rgl, warm, reps)
        # five T x T x hs products are the mathematical minimum (dV, dP, dQ, dK and the recomputed scores); causal half
        useful = 5.0 * B * H * T * T * hs
        tf = useful / (ms / 1e3) / 1e12
        out[name] = {"ms": round(ms, 4), "TFLOPs_causal_useful": round(tf, 2),
                     "roofline": {"kernel": "fused causal attention backward (dQ kernel + dK/dV kernel)", "bound": "mfma", "achieved": round(tf, 2),
                                  "peak": MFMA_PEAK_TFLOPS[name], "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_TFLOPS[name], 4),
                                  "traffic": recorded_traffic("attn_bwd_" + name)}}
        for h in (q, k, v, dy, y, dq, dk, dv):
            cuda.FreeMemory(h)
    cuda.FreeMemory(mask)
    return out


def bench_decode_attention(cuda, reps, warm=5, cases=None):
    """KV-cache attention, 32 heads x 128, one query token per sequence (id 2001)."""
    from mycaffe_amd.cudadnn import CUDAFN
    H, hs = 32, 128
    out = {}
    rng = np.random.default_rng(0)
    for name, half, es in (("bf16", True, 2), ("f32", False, 4)):
        for B in (1, 8, 32):
            for L in (512, 2048, 4096):
                if cases is not None and (name, B, L) not in cases:
                    continue
                n = B * H * L * hs
                kc = cuda.AllocMemory(n, bHalfSize=half)
                vc = cuda.AllocMemory(n, bHalfSize=half)
                # fill on the device: a seeded block, then doubled in place (values only matter for parity tests)
                blk = rng.standard_normal(min(n, 1 << 20)).astype(np.float32)
                src = cuda.AllocMemory(blk, bHalfSize=half)
                for dst in (kc, vc):
                    cuda.copy(blk.size, src, dst, 0, 0)
                    have = blk.size
                    while have < n:
                        c = min(have, n - have)
                        cuda.copy(c, dst, dst, 0, have)
                        have += c
                q = cuda.AllocMemory(rng.standard_normal(B * H * hs).astype(np.float32), bHalfSize=half)
                kn = cuda.AllocMemory(rng.standard_normal(B * H * hs).astype(np.float32), bHalfSize=half)
                vn = cuda.AllocMemory(rng.standard_normal(B * H * hs).astype(np.float32), bHalfSize=half)
                y = cuda.AllocMemory(B * H * hs, bHalfSize=half)
                hr = cuda.CreateRope(0, 0, B * H * hs, B, L, H, hs, 10000.0)
                # the whole step the configuration names: rotate q and the newest key at position L - 1 (theta 10000),
                # append key and value to the caches, attend over the L cached positions.  Repeats rotate q again in
                # place: its values change, its magnitude and the timing do not.
                rgl = [B, H, H, hs, L, q, kc, vc, y, H * L * hs, L * hs, hs, hr, kn, vn]
                ms = timed(cuda, CUDAFN.ATTN_DECODE_FWD, [0.0], rgl, warm, reps)
                ms_attn = timed(cuda, CUDAFN.ATTN_DECODE_FWD, [0.0], rgl[:12], warm, reps)
                nbytes = 2.0 * n * es
                gbs = nbytes / (ms / 1e3) / 1e9
                # back-to-back dispatches re-read the same cache: below the 256 MB of last-level cache the figure is
                # not an HBM rate (and the smallest cases are launch bound)
                case = {"us": round(ms * 1e3, 2), "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4),
                        "us_attention_kernel_alone": round(ms_attn * 1e3, 2), "fits_last_level_cache": bool(nbytes <= 256e6)}
                extra = []
                if nbytes < 800e6:
                    # the same step over copies of the caches taken in turn, 0.8 GB of them (more than three times the
                    # last-level cache), so that every dispatch reads its cache from HBM
                    sets = [rgl]
                    for _ in range(min(127, int(800e6 // nbytes))):
                        kc2, vc2 = cuda.AllocMemory(n, bHalfSize=half), cuda.AllocMemory(n, bHalfSize=half)
                        cuda.copy(n, kc, kc2)
                        cuda.copy(n, vc, vc2)
                        extra += [kc2, vc2]
                        sets.append(rgl[:6] + [kc2, vc2] + rgl[8:])
                    ms_cold = timed_sets(cuda, CUDAFN.ATTN_DECODE_FWD, [0.0], sets, warm, reps)
                    gbs_cold = nbytes / (ms_cold / 1e3) / 1e9
                    case.update({"us_caches_from_hbm": round(ms_cold * 1e3, 2), "GBps_caches_from_hbm": round(gbs_cold, 1),
                                 "frac_hbm_caches_from_hbm": round(gbs_cold / HBM_PEAK_GBS, 4), "cache_copies_taken_in_turn": len(sets)})
                out["%s_B%d_L%d" % (name, B, L)] = case
                cuda.FreeRope(hr)
                for h in [kc, vc, src, q, kn, vn, y] + extra:
                    cuda.FreeMemory(h)
    if "bf16_B32_L4096" not in out:
        return out
    best = out["bf16_B32_L4096"]
    out["roofline"] = {"kernel": "rope_append_kernel + attn_decode_kernel (bf16, batch 32, L 4096, 32 x 128)", "bound": "hbm", "achieved": best["GBps"],
                       "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": best["frac_hbm"],
                       "traffic": recorded_traffic("attn_decode_bf16_B32_L4096")}
    return out


def bench_encdec_attention(cuda, reps, warm=5):
    """Encoder-decoder attention shapes (d_model 512, 8 heads x 64, batch 32, source 256, target 128), bf16, through
    ATTN_FWD: encoder self attention with a (B,T) key-padding mask, decoder self attention with a (B,T,T)
    causal-and-padding mask, cross attention (T_q 128, T_k 256) with the source key-padding mask.  Valid lengths per
    sequence are uniform in [32,256] / [16,128] (seed 7).  Padded keys are computed and masked, not skipped: TFLOP/s
    is quoted on the full rectangle 4*B*H*T_q*T_k*64."""
    from mycaffe_amd.cudadnn import CUDAFN
    B, H, hs, Ts, Tt = 32, 8, 64, 256, 128
    rng = np.random.default_rng(7)
    slen, tlen = rng.integers(32, Ts + 1, B), rng.integers(16, Tt + 1, B)
    enc_mask = (np.arange(Ts)[None, :] < slen[:, None]).astype(np.float32)
    dec_mask = ((np.arange(Tt)[None, :] < tlen[:, None])[:, None, :] * np.tril(np.ones((Tt, Tt)))[None]).astype(np.float32)
    hme, hmd = cuda.AllocMemory(enc_mask), cuda.AllocMemory(dec_mask)
    out = {}
    for name, Tq, Tk, hm, code in (("encoder_self_T256_keymask", Ts, Ts, hme, 1), ("decoder_self_T128_batch_qk_mask", Tt, Tt, hmd, 2),
                                   ("cross_Tq128_Tk256_keymask", Tt, Ts, hme, 1)):
        hc, ha = cuda.CreateCuDNN(), cuda.CreateAttn()
        cuda.SetAttn(hc, ha, 0, False, B, max(Tq, Tk), H, hs, 0.0)
        hq = cuda.AllocMemory(rng.standard_normal(B * H * Tq * hs).astype(np.float32), bHalfSize=True)
        hk = cuda.AllocMemory(rng.standard_normal(B * H * Tk * hs).astype(np.float32), bHalfSize=True)
        hv = cuda.AllocMemory(rng.standard_normal(B * H * Tk * hs).astype(np.float32), bHalfSize=True)
        hy = cuda.AllocMemory(B * H * Tq * hs, bHalfSize=True)
        rgl = [hc, ha, Tq, hq, hk, hv, hm, hy, code] + ([Tk] if Tk != Tq else [])
        ms = timed(cuda, CUDAFN.CUDA_ATTN_FWD, None, rgl, warm, reps)
        tf = 4.0 * B * H * Tq * Tk * hs / (ms / 1e3) / 1e12
        out[name] = {"us": round(ms * 1e3, 2), "TFLOPs_full_rectangle": round(tf, 1), "frac_mfma": round(tf / MFMA_PEAK_TFLOPS["bf16"], 4)}
        for h in (hq, hk, hv, hy):
            cuda.FreeMemory(h)
        cuda.FreeAttn(ha)
        cuda.FreeCuDNN(hc)
    cuda.FreeMemory(hme)
    cuda.FreeMemory(hmd)
    return out


def bench_gemm(cuda, reps):
    """QKV (8192 x 2304 x 768) and output projection (8192 x 768 x 768) GEMMs of the causal self attention layer and one
    projection of the encoder-decoder attention layer (8192 x 512 x 512), weights [N, K]."""
    from mycaffe_amd.cudadnn import CUDAFN
    out = {}
    rng = np.random.default_rng(0)
    for name, half in (("bf16", True), ("f32", False)):
        for tag, (M, N, K) in (("qkv", (8192, 2304, 768)), ("proj", (8192, 768, 768)), ("mha_proj_d512", (8192, 512, 512))):
            a = cuda.AllocMemory(rng.standard_normal(M * K).astype(np.float32), bHalfSize=half)
            w = cuda.AllocMemory((rng.standard_normal(N * K) * 0.02).astype(np.float32), bHalfSize=half)
            c = cuda.AllocMemory(M * N, bHalfSize=half)
            rgl = [0, 1, M, N, K, 0, a, w, 0, c]
            ms = timed(cuda, CUDAFN.CUDA_GEMM, [1.0, 0.0], rgl, 3, reps)
            tf = 2.0 * M * N * K / (ms / 1e3) / 1e12
            out["%s_%s" % (name, tag)] = {"ms": round(ms, 4), "TFLOPs": round(tf, 2), "frac_mfma": round(tf / MFMA_PEAK_TFLOPS[name], 4),
                                          "algorithmic_bytes": (M * K + N * K + M * N) * (2 if half else 4),
                                          "traffic": recorded_traffic("gemm_%s_%s" % (tag, name))}
            for h in (a, w, c):
                cuda.FreeMemory(h)
    # InnerProductLayer backward of the QKV layer: bias update of the forward pass (K = 1), data gradient
    # dX = dY W (no transposes) and weight gradient dW += dY^T X (A transposed)
    M, N, K = 8192, 2304, 768
    for name, half in (("f32", False), ("bf16", True)):
        x = cuda.AllocMemory(rng.standard_normal(M * K).astype(np.float32), bHalfSize=half)
        w = cuda.AllocMemory((rng.standard_normal(N * K) * 0.02).astype(np.float32), bHalfSize=half)
        dy = cuda.AllocMemory(rng.standard_normal(M * N).astype(np.float32), bHalfSize=half)
        dx, dw = cuda.AllocMemory(M * K, bHalfSize=half), cuda.AllocMemory(N * K, bHalfSize=half)
        ones, bias = cuda.AllocMemory(np.ones(M, np.float32), bHalfSize=half), cuda.AllocMemory(np.zeros(N, np.float32), bHalfSize=half)
        for tag, rgf, rgl, fl in ((name + "_qkv_bias_rank1", [1.0, 1.0], [0, 0, M, N, 1, 0, ones, bias, 0, dy], None),
                                  (name + "_qkv_data_grad", [1.0, 0.0], [0, 0, M, K, N, 0, dy, w, 0, dx], 2.0 * M * N * K),
                                  (name + "_qkv_weight_grad", [1.0, 1.0], [1, 0, N, K, M, 0, dy, x, 0, dw], 2.0 * M * N * K)):
            ms = timed(cuda, CUDAFN.CUDA_GEMM, rgf, rgl, 3, reps)
            if fl is None:
                gbs = 2.0 * M * N * (2 if half else 4) / (ms / 1e3) / 1e9
                out[tag] = {"ms": round(ms, 4), "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)}
            else:
                tf = fl / (ms / 1e3) / 1e12
                out[tag] = {"ms": round(ms, 4), "TFLOPs": round(tf, 2), "frac_mfma": round(tf / MFMA_PEAK_TFLOPS[name], 4)}
        # bias gradient db += dY^T ones (InnerProductLayer.cs:473-478): a transposed mat-vec over the M rows
        ms = timed(cuda, CUDAFN.CUDA_GEMV, [1.0, 1.0], [1, M, N, 0, dy, ones, 0, bias, 0, 0, 0], 3, reps)
        gbs = M * N * (2 if half else 4) / (ms / 1e3) / 1e9
        out[name + "_qkv_bias_grad"] = {"ms": round(ms, 4), "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)}
        for h in (x, w, dy, dx, dw, ones, bias):
            cuda.FreeMemory(h)
    return out


def bench_csa_layer(cuda, reps, warm=2):
    """CausalSelfAttentionLayer.forward at B=8, T=1024, C=768, 12 heads through the layer mirror (the C# call sequence
    over the C ABI), fp32: with the fused attention handle and with the explicit MatMul / mask / softmax chain that the
    layer's default parameters select.  Wall clock around `reps` forwards, device synchronised before and after."""
    from mycaffe_amd.layers import Blob, CausalSelfAttentionLayer
    B, T, C, H = 8, 1024, 768, 12
    rng = np.random.default_rng(0)
    x = Blob(cuda, (B, T, C))
    x.mutable_cpu_data = rng.standard_normal((B, T, C)).astype(np.float32)
    wa, ba = rng.standard_normal((3 * C, C)).astype(np.float32) * 0.02, np.zeros(3 * C, np.float32)
    wp, bp = rng.standard_normal((C, C)).astype(np.float32) * 0.02, np.zeros(C, np.float32)
    out = {}
    for name, sdpa in (("fused_handle", True), ("explicit_chain", False)):
        layer = CausalSelfAttentionLayer(cuda, H, C, T, True, sdpa)
        top = Blob(cuda)
        layer.Setup(x, wa, ba, wp, bp)
        for _ in range(warm):
            layer.Forward(x, top)
        cuda.SynchronizeDevice()
        t0 = time.perf_counter()
        for _ in range(reps):
            layer.Forward(x, top)
        cuda.SynchronizeDevice()
        out[name] = {"ms_per_forward": round((time.perf_counter() - t0) / reps * 1e3, 3)}
        for b in list(layer.b.values()) + [top, layer.blobMask]:
            b.Dispose()
    x.Dispose()
    out["compiled_host"] = csa_layer_compiled_host(reps)
    return out


def csa_layer_compiled_host(reps):
    """The same layer forward issued by the compiled C++ host program (a child process with its own device context):
    per-call host cost of a compiled caller, which is what the C# layer pays, instead of the Python mirror's.
    Flops of one forward: QKV 29.0 G + causal-useful attention 25.8 G / 2 * 2 + projection 9.7 G = 51.5 G."""
    import subprocess
    from mycaffe_amd import build as B
    exe = B.host_bench_path()
    if not os.path.exists(exe):
        return {"error": "host benchmark program not built"}
    try:
        r = subprocess.run([exe, os.path.join(ROOT, "mycaffe_amd", "libmycaffe_hip.so"), str(max(reps, 20))], capture_output=True, text=True, timeout=120)
    except subprocess.TimeoutExpired:
        return {"error": "timed out"}
    if r.returncode != 0:
        return {"error": r.stderr.strip()[-300:]}
    d = json.loads(r.stdout.strip().splitlines()[-1])
    flops = 51.5e9
    for k in ("f32_fused_ms", "f32_explicit_ms", "bf16_fused_ms", "f32_4call_ms", "bf16_4call_ms", "f32_3call_ms", "bf16_3call_ms"):
        d[k.replace("_ms", "_TFLOPs_causal_useful")] = round(flops / (d[k] / 1e3) / 1e12, 1)
    return d


def bench_matmul_chain(cuda, reps, warm=3):
    """The two strided-batched MatMul calls of the explicit (not fused) attention chain at B=8, T=1024, 12 x 64, fp32
    (ids 219): Q K^T -> (B,H,T,T) and P V -> (B,H,T,hs), the route the C# layers take when the fused handle is off."""
    from mycaffe_amd.cudadnn import CUDAFN
    outer, T, hs = 96, 1024, 64
    rng = np.random.default_rng(0)
    q = cuda.AllocMemory(rng.standard_normal(outer * T * hs).astype(np.float32))
    kt = cuda.AllocMemory(rng.standard_normal(outer * T * hs).astype(np.float32))
    v = cuda.AllocMemory(rng.standard_normal(outer * T * hs).astype(np.float32))
    att = cuda.AllocMemory(outer * T * T)
    y = cuda.AllocMemory(outer * T * hs)
    out = {}
    # matmul(outer, m, n, k, A, B, C) = gemm2(false, false, n, m, k, 1, B, A, 0, C, n, k, n, k*n, m*k, m*n, outer)
    for name, (m, n, k, hA, hB, hC) in (("qk_t", (T, T, hs, q, kt, att)), ("p_v", (T, hs, T, att, v, y))):
        rgl = [0, 0, n, m, k, 0, hB, hA, 0, hC, n, k, n, k * n, m * k, m * n, outer]
        ms = timed(cuda, CUDAFN.CUDA_GEMM2, [1.0, 0.0], rgl, warm, reps)
        fl = 2.0 * outer * m * n * k
        nbytes = 4.0 * outer * (m * k + k * n + m * n)
        tf = fl / (ms / 1e3) / 1e12
        out[name] = {"ms": round(ms, 4), "TFLOPs": round(tf, 2), "frac_mfma_f32": round(tf / MFMA_PEAK_TFLOPS["f32"], 4),
                     "GBps": round(nbytes / (ms / 1e3) / 1e9, 1), "frac_hbm": round(nbytes / (ms / 1e3) / 1e9 / HBM_PEAK_GBS, 4)}
    for h in (q, kt, v, att, y):
        cuda.FreeMemory(h)
    return out


def bench_block_ops(cuda, reps, warm=3):
    """The per-block elementwise ops at the GPT-2 shape of the prefill benchmark (8192 rows x 768, MLP width 3072):
    LayerNorm handle forward / backward, GELU forward / backward, and the softmax (forward, gradient) of the explicit
    attention chain.  HBM bound: algorithmic bytes = tensors read + written."""
    from mycaffe_amd.cudadnn import CUDAFN
    rows, C = 8192, 768
    out = {}
    rng = np.random.default_rng(0)
    for name, half, es in (("bf16", True, 2), ("f32", False, 4)):
        n = rows * C
        x = cuda.AllocMemory(rng.standard_normal(n).astype(np.float32), bHalfSize=half)
        y, dy, dx = (cuda.AllocMemory(n, bHalfSize=half) for _ in range(3))
        h = cuda.CreateLayerNorm(0, n, 8, 1024, C, 1e-5)
        cuda.LayerNormForward(h, x, y)
        res = {}
        for key, fn, rgl, tensors in (("layernorm_fwd", CUDAFN.CUDA_LAYERNORM_FWD, [h, x, y], 2),
                                      ("layernorm_bwd", CUDAFN.CUDA_LAYERNORM_BWD, [h, y, dy, dx], 3)):
            ms = timed(cuda, fn, None, rgl, warm, reps)
            gbs = tensors * n * es / (ms / 1e3) / 1e9
            res[key] = {"us": round(ms * 1e3, 2), "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)}
        cuda.FreeLayerNorm(h)
        for hh in (x, y, dy, dx):
            cuda.FreeMemory(hh)
        n = rows * 4 * C
        x = cuda.AllocMemory(rng.standard_normal(n).astype(np.float32), bHalfSize=half)
        y, dy, dx = (cuda.AllocMemory(n, bHalfSize=half) for _ in range(3))
        for key, fn, rgl, tensors in (("gelu_tanh_fwd", CUDAFN.CUDA_GELU_FWD, [n, x, y, 1], 2),
                                      ("gelu_tanh_bwd", CUDAFN.CUDA_GELU_BWD, [n, dy, y, dx, x, 1], 3)):
            ms = timed(cuda, fn, None, rgl, warm, reps)
            gbs = tensors * n * es / (ms / 1e3) / 1e9
            res[key] = {"us": round(ms * 1e3, 2), "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)}
        for hh in (x, y, dy, dx):
            cuda.FreeMemory(hh)
        # softmax of the explicit attention chain's score tensor (B*H*T rows of T = 1024 values) and its gradient
        srows, slen = 8 * 12 * 1024, 1024
        n = srows * slen
        x, y, dy = (cuda.AllocMemory(n, bHalfSize=half) for _ in range(3))
        hc, d = cuda.CreateCuDNN(), cuda.CreateTensorDesc()
        cuda.SetTensorDesc(d, srows, slen, 1, 1, half)
        for key, fn, rgl, tensors in (("softmax_fwd_98304x1024", CUDAFN.SOFTMAX_FWD, [hc, 0, d, x, 0, d, y, 1, 0], 2),
                                      ("softmax_bwd_98304x1024", CUDAFN.SOFTMAX_BWD, [hc, 0, d, y, d, dy, 0, d, x, 1, 0], 3)):
            ms = timed(cuda, fn, [1.0, 0.0], rgl, warm, max(4, reps // 4))
            gbs = tensors * n * es / (ms / 1e3) / 1e9
            res[key] = {"us": round(ms * 1e3, 2), "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)}
        cuda.FreeTensorDesc(d)
        cuda.FreeCuDNN(hc)
        for hh in (x, y, dy):
            cuda.FreeMemory(hh)
        out[name] = res
    return out


def bench_copy(cuda, reps, warm=2):
    """Plain streaming kernel of known size (y = 1.0 * x over 64 Mi floats: reads 256 MiB, writes 256 MiB): the kernel
    that the FETCH_SIZE / WRITE_SIZE counter readings of the other kernels are scaled by."""
    from mycaffe_amd.cudadnn import CUDAFN
    n = 64 << 20
    a = cuda.AllocMemory(n)
    b = cuda.AllocMemory(n)
    ms = timed(cuda, CUDAFN.CUDA_SCALE, [1.0], [n, 0, a, b, 0, 0], warm, reps)
    cuda.FreeMemory(a)
    cuda.FreeMemory(b)
    return {"kernel": "map_kernel<float, false, ScaleF>", "bytes_read": n * 4, "bytes_written": n * 4, "ms": round(ms, 4),
            "GBps": round(2 * n * 4 / (ms / 1e3) / 1e9, 1)}


COUNTER_SECTIONS = ("decode_step", "copy", "prefill", "prefill_7b", "decode_attn", "backward", "gemm", "matmul_chain")


def counter_pass(cuda, path, sections):
    """A short run for hardware-counter collection (rocprofv3 --pmc serialises and slows every dispatch): a few
    dispatches of the kernels of the named sections only, so that one counter run stays within seconds.
    decode_step: two eager decode steps at position 512; copy: the 256 MiB streaming kernel that calibrates the traffic
    counters; prefill / prefill_7b: fused causal attention at B=8 T=1024 12x64 (bf16, fp32) / B=4 T=4096 32x128 (bf16);
    decode_attn: decode attention at batch 32, L 4096 (bf16, fp32); backward: attention backward; gemm: the layer
    GEMMs; matmul_chain: the two batched MatMul calls of the explicit attention chain."""
    out = {}
    for sec in sections:
        log("counter pass:", sec)
        if sec == "decode_step":
            from mycaffe_amd.llm_inference import LlmInference
            inf = LlmInference(cuda)
            inf.Initialize(fTemperature=0.0)
            inf.SetOption(3, 0)
            inf.Load(path)
            inf.ProfileStep(512, 2)
            inf.CleanUp()
            out[sec] = "2 eager steps at position 512"
        elif sec == "copy":
            out[sec] = bench_copy(cuda, 2, 0)
        elif sec == "prefill":
            out[sec] = bench_prefill_attention(cuda, 2, 0)
        elif sec == "prefill_7b":
            out[sec] = bench_prefill_attention(cuda, 2, 0, (4, 32, 4096, 128), (("bf16", True),))
        elif sec == "decode_attn":
            out[sec] = bench_decode_attention(cuda, 2, 0, cases=(("bf16", 32, 4096), ("f32", 32, 4096)))
        elif sec == "backward":
            out[sec] = bench_attention_backward(cuda, 2, 0)
        elif sec == "gemm":
            out[sec] = bench_gemm(cuda, 2)
        elif sec == "matmul_chain":
            out[sec] = bench_matmul_chain(cuda, 2, 0)
        else:
            raise SystemExit("unknown counter-pass section %r (known: %s)" % (sec, ", ".join(COUNTER_SECTIONS)))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=880)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-also", action="store_true", help="only the headline workload")
    ap.add_argument("--no-steady", action="store_true", help="time each section right away instead of after 100 ms of the same "
                    "dispatches (for traced runs, whose output would otherwise hold thousands of warm-up dispatches)")
    ap.add_argument("--no-graph", action="store_true", help="launch every decode kernel eagerly instead of replaying a HIP graph "
                    "(kernel tracing tools see the individual kernels this way)")
    ap.add_argument("--counter-pass", nargs="?", const="all", default=None, metavar="SECTIONS",
                    help="few dispatches of the kernels of the named sections (comma list of %s; default all), for rocprofv3 "
                         "--pmc runs; prints what ran instead of the benchmark line" % ", ".join(COUNTER_SECTIONS))
    ap.add_argument("--only", default="", help="comma list of 'also' sections to run: decode,sampled,prefill,backward,csa_layer,matmul_chain,block_ops,decode_attn,encdec,gemm "
                    "(and copy, the counter-calibration kernel, which only runs when named)")
    args = ap.parse_args()
    if args.no_steady:
        global STEADY_MS
        STEADY_MS = 0.0
    if args.gpus != 1:
        log("bench.py measures one GPU: every box of this build has one MI355X and the path has no multi-GPU part; "
            "run with --gpus 1")
        sys.exit(2)
    if args.steps < 1 or args.warmup < 0 or N_PROMPT + args.warmup >= C4["seq_len"]:
        log("need steps >= 1 and prompt (128) + warmup < 1024")
        sys.exit(2)

    from mycaffe_amd.cudadnn import CudaDnn
    cuda = CudaDnn(0)
    dev_name = cuda.GetDeviceName(0)
    log("device:", dev_name)
    path = os.path.join(os.environ.get("TMPDIR", "/tmp"), "mycaffe_amd_llama110m_seed1234.bin")
    t0 = time.perf_counter()
    blob = make_checkpoint(C4, 1234, path)
    log("checkpoint ready in %.1f s" % (time.perf_counter() - t0))

    if args.counter_pass:
        secs = COUNTER_SECTIONS if args.counter_pass == "all" else tuple(x for x in args.counter_pass.split(",") if x)
        print(json.dumps({"counter_pass": counter_pass(cuda, path, secs)}), flush=True)
        cuda.Dispose()
        return
    inf, head = run_decode(cuda, path, False, 1, args.steps, args.warmup, graph=not args.no_graph)
    log("fp32 batch 1: %.1f tokens/s (%.4f ms/step)" % (head["tokens_per_s"], head["ms_per_step"]))
    roof = step_roofline(inf, head, args.steps, args.warmup)
    inf.CleanUp()

    also = {}
    only = set(x for x in args.only.split(",") if x)
    want = lambda name: not args.no_also and (not only or name in only)
    also["decode_fp32_b1_wall_s_incl_id_transfers"] = round(head["wall_s_whole_generation"], 4)
    # the 128-token prompt of the same generation: one batched pass before the timed decode steps
    also["prefill_128_tokens_fp32_b1"] = prefill_summary(head, 1, 4)
    log("prompt pass, batch 1:", json.dumps(also["prefill_128_tokens_fp32_b1"]))
    if want("decode"):
        for tag, bf16, batch, kv16 in (("bf16_weights_b1", True, 1, False), ("fp32_b16", False, 16, False),
                                       ("bf16_weights_b16", True, 16, False), ("bf16_weights_and_cache_b16", True, 16, True)):
            i2, r = run_decode(cuda, path, bf16, batch, args.steps, args.warmup, graph=not args.no_graph, kv_bf16=kv16)
            # algorithmic bytes of one step: every weight once, plus each sequence's cache at the mean timed length
            first = N_PROMPT + args.warmup
            mean_len = first + 1 + (min(args.steps, C4["seq_len"] - first) - 1) / 2.0
            kvd = C4["dim"] // C4["n_heads"] * C4["n_kv_heads"]
            step_bytes = weight_bytes(C4, 2 if bf16 else 4) + batch * C4["n_layers"] * 2 * mean_len * kvd * (2 if kv16 else 4)
            gbps = step_bytes / (r["ms_per_step"] * 1e-3) / 1e9
            also["decode_" + tag] = {"tokens_per_s": round(r["tokens_per_s"], 1), "ms_per_step": round(r["ms_per_step"], 4),
                                     "algorithmic_bytes_per_step": round(step_bytes), "GBps": round(gbps, 1),
                                     "frac_hbm": round(gbps / HBM_PEAK_GBS, 4),
                                     "graph_replay": bool(r["graph"]), "prefill_128_tokens": prefill_summary(r, batch, 2 if bf16 else 4)}
            log("decode %s: %.1f tokens/s, prompt pass %s" % (tag, r["tokens_per_s"], json.dumps(also["decode_" + tag]["prefill_128_tokens"])))
            if bf16 and batch > 1:
                # the same prompt pass with option 10: activations rounded to bf16, attention in bf16 (logits to the 16-bit bar)
                i2.SetOption(10, 1)
                pr = np.random.default_rng(5).integers(3, C4["vocab_size"], (batch, N_PROMPT))
                best = None
                for _ in range(3):
                    i2.GenerateBatch(pr, N_PROMPT + 1)
                    ms, rows = i2.LastPrefill()
                    best = ms if best is None else min(best, ms)
                also["decode_" + tag]["prefill_128_tokens_bf16_activations"] = prefill_summary({"prefill_ms": best, "prefill_rows": rows}, batch, 2)
                log("  with bf16 activations (option 10):", json.dumps(also["decode_" + tag]["prefill_128_tokens_bf16_activations"]))
            i2.CleanUp()
    if want("sampled"):
        also["sampled_generation_fp32_b1"] = bench_sampled_generation(cuda, path)
        log("sampled generation:", json.dumps(also["sampled_generation_fp32_b1"]))
    if want("prefill"):
        also["prefill_attention_B8_T1024_H12x64"] = bench_prefill_attention(cuda, 50)
        log("prefill attention:", json.dumps(also["prefill_attention_B8_T1024_H12x64"]))
        # the Llama-2 7B head shape at its full context: long enough that launch and tail effects no longer count
        also["prefill_attention_B4_T4096_H32x128"] = bench_prefill_attention(cuda, 10, 2, (4, 32, 4096, 128), (("bf16", True),))
        log("prefill attention, 32 x 128 heads, T = 4096:", json.dumps(also["prefill_attention_B4_T4096_H32x128"]))
        also["prefill_attention_unmasked_bf16"] = {
            "B%d_T%d_H%dx%d" % (sh[0], sh[2], sh[1], sh[3]): bench_prefill_attention(cuda, r, 2, sh, (("bf16", True),), causal=False)["bf16"]
            for sh, r in (((8, 12, 1024, 64), 50), ((4, 32, 4096, 64), 10), ((4, 32, 4096, 128), 10))}
        log("prefill attention without a mask:", json.dumps(also["prefill_attention_unmasked_bf16"]))
    if want("decode_attn"):
        also["decode_attention_H32x128"] = bench_decode_attention(cuda, 20)
        log("decode attention roofline:", json.dumps(also["decode_attention_H32x128"]["roofline"]))
    if want("backward"):
        also["attention_backward_B8_T1024_H12x64"] = bench_attention_backward(cuda, 30)
        log("attention backward:", json.dumps(also["attention_backward_B8_T1024_H12x64"]))
    if want("csa_layer"):
        also["csa_layer_B8_T1024_C768_f32"] = bench_csa_layer(cuda, 5)
        log("csa layer:", json.dumps(also["csa_layer_B8_T1024_C768_f32"]))
    if want("matmul_chain"):
        also["matmul_chain_B8_T1024_H12x64_f32"] = bench_matmul_chain(cuda, 10)
        log("matmul chain:", json.dumps(also["matmul_chain_B8_T1024_H12x64_f32"]))
    if want("block_ops"):
        also["block_ops_8192x768"] = bench_block_ops(cuda, 20)
        log("block ops:", json.dumps(also["block_ops_8192x768"]))
    if want("encdec"):
        also["encdec_attention_B32_H8x64_bf16"] = bench_encdec_attention(cuda, 50)
        log("enc-dec attention:", json.dumps(also["encdec_attention_B32_H8x64_bf16"]))
    if "copy" in only:
        also["copy_256MiB"] = bench_copy(cuda, 10)
    if want("gemm"):
        also["gemm_inner_product"] = bench_gemm(cuda, 10)
        log("gemm:", json.dumps(also["gemm_inner_product"]))

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(blob, head["prompt"], head["ids"])
        log("cpu baseline:", json.dumps(cpu))

    # the kernels the targets are set on (fused prefill attention >= 50 % of the bf16 MFMA peak, decode attention
    # >= 70 % of HBM peak, the 16-bit QKV GEMM >= 40 %), inside the roofline object so that they travel with it
    targets = {}
    pa = also.get("prefill_attention_B8_T1024_H12x64", {}).get("bf16")
    if pa:
        targets["prefill_attention_bf16_causal_B8_T1024_H12x64"] = dict(pa["roofline"], target_frac=0.5, avg_launch_us=round(pa["ms"] * 1e3, 2))
    pa = also.get("prefill_attention_B4_T4096_H32x128", {}).get("bf16")
    if pa:
        targets["prefill_attention_bf16_causal_B4_T4096_H32x128"] = dict(pa["roofline"], target_frac=0.5, avg_launch_us=round(pa["ms"] * 1e3, 2))
    da = also.get("decode_attention_H32x128", {})
    if "roofline" in da:
        targets["decode_attention_bf16_B32_L4096_H32x128"] = dict(da["roofline"], target_frac=0.7, avg_launch_us=da["bf16_B32_L4096"]["us"])
    gq = also.get("gemm_inner_product", {}).get("bf16_qkv")
    if gq:
        targets["gemm_bf16_8192x2304x768"] = {"kernel": "QKV projection GEMM, 16-bit storage", "bound": "mfma", "achieved": gq["TFLOPs"],
                                              "peak": MFMA_PEAK_TFLOPS["bf16"], "unit": "TFLOP/s", "frac": gq["frac_mfma"], "traffic": gq["traffic"],
                                              "algorithmic_bytes": gq["algorithmic_bytes"], "target_frac": 0.4, "avg_launch_us": round(gq["ms"] * 1e3, 2)}
    roof["targets"] = targets
    # The same figures once more as flat scalars of the roofline object (a consumer that keeps only scalar keys still
    # gets them), fractions of the MI355X peak (2.5 PFLOP/s bf16 MFMA, 8 TB/s HBM).
    flat = {}
    for key, tag in (("prefill_attention_bf16_causal_B8_T1024_H12x64", "prefill_bf16_causal_B8_T1024"),
                     ("prefill_attention_bf16_causal_B4_T4096_H32x128", "prefill_bf16_causal_B4_T4096")):
        if key in targets:
            flat[tag + "_frac"] = targets[key]["frac"]
            flat[tag + "_us"] = targets[key]["avg_launch_us"]
    if "decode_attention_bf16_B32_L4096_H32x128" in targets:
        t = targets["decode_attention_bf16_B32_L4096_H32x128"]
        flat["decode_attn_bf16_B32_L4096_frac"] = t["frac"]
        flat["decode_attn_bf16_B32_L4096_GBps"] = t["achieved"]
    if "gemm_bf16_8192x2304x768" in targets:
        flat["gemm_bf16_qkv_frac"] = targets["gemm_bf16_8192x2304x768"]["frac"]
    for tag, short in (("fp32_b16", "decode_fp32_b16"), ("bf16_weights_b16", "decode_bf16w_b16"),
                       ("bf16_weights_and_cache_b16", "decode_bf16w_bf16kv_b16"), ("bf16_weights_b1", "decode_bf16w_b1")):
        d = also.get("decode_" + tag)
        if d:
            flat[short + "_frac_hbm"] = d["frac_hbm"]
            flat[short + "_tokens_per_s"] = d["tokens_per_s"]
            if d.get("prefill_128_tokens"):
                flat[short + "_prefill_ms"] = d["prefill_128_tokens"]["ms"]
            if d.get("prefill_128_tokens_bf16_activations"):
                flat[short + "_prefill_bf16_activations_ms"] = d["prefill_128_tokens_bf16_activations"]["ms"]
    sg = also.get("sampled_generation_fp32_b1")
    if sg:
        flat["sampled_top_p_device_ms_per_position"] = sg["top_p_0.9_device_sampler"]["ms_per_position"]
        flat["sampled_top_p_host_ms_per_position"] = sg["top_p_0.9_host_sampler"]["ms_per_position"]
        flat["sampled_top_p_device_prompt_128_ms"] = sg["top_p_0.9_device_sampler"]["prompt_128_positions_ms"]
        flat["sampled_top_p_host_prompt_128_ms"] = sg["top_p_0.9_host_sampler"]["prompt_128_positions_ms"]
    roof.update(flat)

    line = {
        "metric": "decode tokens/sec", "value": round(head["tokens_per_s"], 2), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(head["ms_per_step"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "Llama-2 110M-shape greedy decode (dim 768, 12 layers, 12 heads x 64, ffn 2048, vocab 32000, "
                               "seq 1024), batch 1, fp32 weights N(0,0.02), 128-id seeded prompt then greedy decode to 1024 tokens",
                   "prompt_tokens": N_PROMPT, "batch": 1, "device": dev_name},
        "roofline": roof, "cpu_baseline": cpu, "also": also,
    }
    # the north-star figures once more, last on stderr
    for k in sorted(flat):
        log("%s = %s" % (k, flat[k]))
    log("decode fp32 batch 1: %.1f tokens/s, %.4f ms/step, %.4f of HBM peak; cpu baseline %s tokens/s"
        % (head["tokens_per_s"], head["ms_per_step"], roof["frac"], cpu["value"] if cpu else "not run"))
    print(json.dumps(line), flush=True)
    cuda.Dispose()


if __name__ == "__main__":
    main()
