#!/usr/bin/env python3
"""Benchmark: greedy decode tok/s at the Llama-2-7B shape (W8A32, batch 1) on one MI355X.

A step is one token: one launch of the whole-token kernel (embedding row, 32 layers of rmsnorm+QKV+RoPE /
attention / Wo / rmsnorm+W1,W3+SwiGLU / W2, final rmsnorm + fp32 classifier + first-maximum argmax + the
token-loop step), 32 of them per replay of a captured hipGraph.  Weights are seeded N(0, 0.02)-like values
quantized with the reference's group-int8 encoder on the GPU; the prompt is 32 seeded ids; everything is
resident in HBM before the clock starts.  One JSON line is printed.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

WORKLOADS = {
    # name: (dim, hidden, layers, heads, kv_heads, vocab, seq_len, shared), seed, prompt ids
    "llama2-7b-shape": ((4096, 11008, 32, 32, 32, 32000, 4096, 0), 103, 32),
    "llama2-13b-shape": ((5120, 13824, 40, 40, 40, 32000, 4096, 0), 105, 32),
    # grouped-query attention (8 kv heads), 72 GB of weights and scales: one GPU's HBM holds it whole
    "llama2-70b-shape": ((8192, 28672, 80, 64, 8, 32000, 4096, 0), 107, 32),
    # 3584 forced prompt ids, then 512 generated: the timed region is positions 3584..4095 only
    "llama2-7b-long-context": ((4096, 11008, 32, 32, 32, 32000, 4096, 0), 104, 3584),
    "stories110m-shape": ((768, 2048, 12, 12, 12, 32000, 1024, 1), 102, 16),
    "stories15m-shape": ((288, 768, 6, 6, 6, 32000, 256, 1), 101, 8),
}
# steps of a workload when --steps is not given: its prompt ids + the generated tokens BASELINE.json's configuration names
DEFAULT_STEPS = {"llama2-7b-shape": 32 + 256, "llama2-13b-shape": 32 + 256, "llama2-70b-shape": 32 + 128,
                 "llama2-7b-long-context": 4096, "stories110m-shape": 16 + 512, "stories15m-shape": 8 + 248}
HBM_PEAK_GBS = 8000.0


def synth_prompt(seed, n, vocab):
    """ids uniform in [3, vocab) from the same counter-based generator the weights use (stream 0xFFFF)."""
    M = (1 << 64) - 1
    base = (seed * 0x9E3779B97F4A7C15 + 0xFFFF * 0xD1B54A32D192ED03) & M
    out = []
    for i in range(n):
        z = (base + i + 0x9E3779B97F4A7C15) & M
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        z ^= z >> 31
        out.append(3 + (z >> 33) % (vocab - 3))
    return np.array(out, dtype=np.int32)


# HBM bytes per launch of k_token from hardware counters.  bench.py cannot read counters itself (they need a profiler
# around the process), so this is a labelled constant from the two `rocprofv3 --pmc` runs summarised in
# profiles/hbm_traffic_llama2-7b.md (FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for a
# 256 MiB copy kernel); it is reported with its source and only for the workload and kernel it was collected on.
COUNTER_TRAFFIC = {
    "llama2-7b-shape": {"hbm_bytes_per_launch": 7460859757, "positions": "0-287 (median launch: 144)",
                        "algorithmic_bytes_at_those_positions": 7356051584,
                        "source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs), profiles/hbm_traffic_llama2-7b.md",
                        "collected": "2026-11-25"},
}


def cpu_baseline(shape, seed, prompt, gpu_tokens, budget_steps):
    """The CPU oracle (a C restatement of llama2j's CPU mode, same row/head-parallel decomposition,
    OpenMP over the host cores) timed on a bounded sample of the same workload, by the reference's
    own rule: clock starts after the first forward, tok/s = (forwards - 1) / elapsed."""
    from oracle import binding as orc
    t0 = time.time()
    m = orc.Model(dim=shape[0], hidden_dim=shape[1], n_layers=shape[2], n_heads=shape[3], n_kv_heads=shape[4],
                  vocab_size=shape[5], seq_len=shape[6], shared_weights=shape[7])
    m.fill_synth(seed, 0.02)
    fill_s = time.time() - t0
    toks, _, sec = m.generate_greedy(prompt, budget_steps)
    # only tokens past the prompt are generated (the prompt ids are forced outputs on both sides, J/Run.java:635-642)
    n_gen = max(0, min(len(toks), len(gpu_tokens)) - len(prompt))
    same = bool(np.array_equal(toks[len(prompt):len(prompt) + n_gen], gpu_tokens[len(prompt):len(prompt) + n_gen])) if n_gen > 0 else None
    cores = orc.lib().orc_num_threads()
    m.close()
    return {
        "value": round((len(toks) - 1) / sec, 4) if sec > 0 else None,
        "unit": "tok/s",
        "cores": cores,
        "kind": "port",
        "sample": "first %d forwards of the same workload (same seeded weights and prompt); C restatement of "
                  "llama2j CPU mode, reference never executed (no JVM); weights generated in %.1f s" % (len(toks), fill_s),
        "generated_tokens_compared": n_gen,
        "tokens_match_gpu": same,
    }


def cpu_baseline_long_context(shape, seed, g, gpu_tokens, positions):
    """The long-context workload cannot be prefilled on the CPU within the bench's time, so the GPU's KV cache (rows
    written by its own decode) is copied into the oracle, which then runs single forwards at a few positions deep in
    the context: their mean time is the CPU rate there, and their logits are compared with the GPU's at the same
    positions (max |delta| / max |logit|), the argmax with the token the GPU's decode emitted."""
    from oracle import binding as orc
    from llama2j_amd import BUFFER
    L, S, kvd = shape[2], shape[6], shape[0] * shape[4] // shape[3]
    m = orc.Model(dim=shape[0], hidden_dim=shape[1], n_layers=shape[2], n_heads=shape[3], n_kv_heads=shape[4],
                  vocab_size=shape[5], seq_len=shape[6], shared_weights=shape[7])
    m.fill_synth(seed, 0.02)
    kc, vc = m.buffer(orc.B_KCACHE).reshape(L, S, kvd), m.buffer(orc.B_VCACHE).reshape(L, S, kvd)
    for l in range(L):
        kc[l] = g.read(BUFFER.KCACHE, layer=l).reshape(S, kvd)
        vc[l] = g.read(BUFFER.VCACHE, layer=l).reshape(S, kvd)
    worst, same, sec = 0.0, True, 0.0
    for pos in positions:
        tok = int(gpu_tokens[pos - 1])
        t0 = time.perf_counter()
        want = m.forward(tok, pos).copy()
        sec += time.perf_counter() - t0
        got = g.forward(tok, pos)
        worst = max(worst, float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max()))
        same = same and int(np.argmax(want)) == int(np.argmax(got)) == int(gpu_tokens[pos])
    cores = orc.lib().orc_num_threads()
    m.close()
    return {
        "value": round(len(positions) / sec, 4), "unit": "tok/s", "cores": cores, "kind": "port",
        "sample": "single forwards at positions %s on the GPU's own KV cache copied to the host; C restatement of llama2j "
                  "CPU mode, reference never executed (no JVM)" % (list(positions),),
        "worst_rel_logit_err_vs_gpu": worst, "generated_tokens_compared": len(positions), "tokens_match_gpu": same,
    }


def load_test(workload, directory):
    """Not the metric: the load path (l2j_load_checkpoint = the TransformerWeights constructor,
    J/TransformerWeights.java:43-144,191-356) at the workload's shape.  Writes a llama2.c v0 checkpoint of random floats
    (27 GB at the 7B shape) into `directory` (memory-backed storage such as /dev/shm keeps the disk out of the figures),
    loads it once without caches (quantizing on the GPU, writing the .quant caches) and twice from the caches, and removes
    the files.  Prints one JSON line of its own."""
    import shutil
    import struct
    import llama2j_amd as l2j
    shape, seed, _ = WORKLOADS[workload]
    dim, hidden, L, H, kvH, vocab, seq, shared = shape
    d = os.path.join(directory, "l2j_load_test")
    shutil.rmtree(d, ignore_errors=True)
    os.makedirs(d)
    try:
        kvd = dim * kvH // H
        sizes = [vocab * dim, L * dim, L * dim * dim, L * dim * kvd, L * dim * kvd, L * dim * dim, L * dim, L * dim * hidden,
                 L * hidden * dim, L * dim * hidden, dim, seq * (dim // H) // 2 * 2] + ([] if shared else [vocab * dim])
        block = (np.random.default_rng(seed).standard_normal(16 << 20) * 0.02).astype("<f4")
        path = os.path.join(d, "model.bin")
        with open(path, "wb") as f:                      # J/Run.java:561-573: seven ints, then the tensors in file order
            f.write(struct.pack("<7i", dim, hidden, L, H, kvH, vocab if shared else -vocab, seq))
            for n in sizes:
                for o in range(0, n, block.size):
                    f.write(block[:min(block.size, n - o)].data)
        out = {"load_test": workload, "bin_bytes": os.path.getsize(path), "directory": directory}
        tokens, same = None, True
        for name, write in (("first_load_s", True), ("cached_load_s", False), ("cached_load_again_s", False)):
            t0 = time.perf_counter()
            g = l2j.Transformer.from_checkpoint(path, write_caches=write)
            g.sync()
            out[name] = round(time.perf_counter() - t0, 3)
            toks, sec = g.decode_greedy(np.array([5, 9, 13], dtype=np.int32), 24)
            same = same and (tokens is None or bool(np.array_equal(tokens, toks)))
            tokens = toks
            g.close()
        out["same_tokens_after_every_load"] = same
        out["cache_bytes"] = sum(os.path.getsize(os.path.join(d, x)) for x in os.listdir(d) if x.endswith(".quant"))
        print(json.dumps(out))
    finally:
        shutil.rmtree(d, ignore_errors=True)
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=0,
                    help="tokens decoded in the timed region (default: the configuration's own length, e.g. 32 prompt + 256 greedy = 288)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--workload", default="llama2-7b-shape", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-steps", type=int, default=97, help="forwards of the CPU baseline sample (0 = skip)")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel timing")
    ap.add_argument("--no-sampled", action="store_true", help="skip the extra decode with the device sampler")
    ap.add_argument("--no-batched", action="store_true", help="skip the extra decodes of 32 and 16 sequences at once (and the prefill)")
    ap.add_argument("--prefill-only", action="store_true", help="of those extras only the prefill (its kernels are launched one by one, "
                                                                  "which a profiler can follow; the batched decode replays a graph)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="also run a plain copy kernel of this size (scales rocprofv3 byte counters)")
    ap.add_argument("--load-test", metavar="DIR", default=None,
                    help="instead of the decode: time l2j_load_checkpoint on a synthetic checkpoint of the workload's shape written into DIR "
                         "(e.g. /dev/shm; 27 GB + 7 GB of caches at the 7B shape, removed afterwards)")
    a = ap.parse_args()
    if a.load_test:
        return load_test(a.workload, a.load_test)
    if a.gpus != 1:
        print("bench.py: this path runs on ONE GPU (batch-1 decode, no multi-GPU split); --gpus %d is not supported" % a.gpus,
              file=sys.stderr)
        return 2

    import llama2j_amd as l2j
    from llama2j_amd import KERNEL

    shape, seed, n_prompt = WORKLOADS[a.workload]
    steps = min(a.steps if a.steps > 0 else DEFAULT_STEPS[a.workload], shape[6])
    if not a.workload.endswith("long-context") and steps <= n_prompt:
        # a short run (the driver's --steps 20): half of it forced prompt ids, half generated tokens, so that the timed
        # run and the CPU leg share generated positions
        n_prompt = steps // 2
    g = l2j.Transformer(l2j.Config(*shape))
    t0 = time.time()
    g.fill_synthetic(seed, 0.02)
    g.finalize()
    load_s = time.time() - t0
    prompt = synth_prompt(seed, n_prompt, shape[5])

    long_context = a.workload.endswith("long-context")
    if long_context:
        # the decode loop always starts at position 0: time the prompt alone, then prompt + 512, and subtract
        steps = shape[6]
        a.no_sampled = True
        g.decode_greedy(prompt, 64)
        g.reset()
        g.sync()
        t0 = time.perf_counter()
        g.decode_greedy(prompt, n_prompt)
        g.sync()
        prefix_wall = time.perf_counter() - t0
        g.reset()
    elif a.warmup > 0:
        g.decode_greedy(prompt, min(a.warmup, shape[6]))
        g.reset()
    g.sync()
    t0 = time.perf_counter()
    tokens, sec_after_first = g.decode_greedy(prompt, steps)
    g.sync()
    wall = time.perf_counter() - t0
    done = len(tokens)
    if done != steps:
        print("bench.py: decode stopped after %d of %d steps (token 1 emitted)" % (done, steps), file=sys.stderr)

    lc_cpu = None
    if long_context and a.cpu_steps > 1 and done == steps:  # (before anything else touches the KV cache)
        lc_cpu = cpu_baseline_long_context(shape, seed, g, tokens, (3584, 3840, 4095))
    mean_pos = (done - 1) / 2.0
    if long_context:
        if done != steps:
            return 1
        wall -= prefix_wall
        done = steps - n_prompt
        mean_pos = (n_prompt + steps - 1) / 2.0
        sec_after_first = 0.0
    bytes_tok = g.bytes_per_token(int(round(mean_pos)))
    tok_s = done / wall
    out = {
        "metric": "decode tok/s at Llama-2-7B shape W8A32; matvec HBM GB/s vs 8 TB/s peak",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": done,
        "warmup": a.warmup,
        "ms_per_step": round(wall / done * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8 weights x f32 activations (W8A32), f32 accumulate",
        "data": "synthetic: seeded N(0,0.02)-like weights quantized by the reference's group-int8 encoder, seeded prompt ids",
        "config": {"workload": "%s: dim %d, hidden %d, %d layers, %d heads, vocab %d, seq_len %d; batch 1 greedy, "
                               "%d forced prompt positions + %d generated%s" % ((a.workload,) + shape[:4] + shape[5:7] +
                                                                 (min(n_prompt, steps), max(0, steps - n_prompt),
                                                                  "; timed: the generated positions only" if long_context else "")),
                   "forced_steps": 0 if long_context else min(n_prompt, done), "generated_steps": max(0, steps - n_prompt),
                   "weights_load_s": round(load_s, 2)},
        "tok_s_reference_rule": round((done - 1) / sec_after_first, 2) if sec_after_first > 0 else None,
        "bytes_per_token": bytes_tok,
        "stream_roofline_tok_s": round(HBM_PEAK_GBS * 1e9 / bytes_tok, 1),
        "frac_of_stream_roofline": round(tok_s * bytes_tok / (HBM_PEAK_GBS * 1e9), 4),
    }

    if not a.no_sampled:
        # Not the metric: the same decode with the reference's default sampling (temperature 0.9, top-p 0.9,
        # J/CommandLine.java:24-25) done on the device, for the cost of sampling beside the greedy figure.
        try:
            g.reset()
            g.sync()
            t0 = time.perf_counter()
            stoks, _ = g.decode_sample(prompt, steps, 0.9, 0.9, 12345)
            g.sync()
            swall = time.perf_counter() - t0
            n_sampled = max(0, int(len(stoks)) - n_prompt)   # forced positions run no sampler
            if n_sampled > 0:
                out["sampled_decode"] = {"temperature": 0.9, "topp": 0.9, "rng_seed": 12345, "steps": int(len(stoks)),
                                         "sampled_positions": n_sampled, "forced_positions": int(len(stoks)) - n_sampled,
                                         "tok_s": round(len(stoks) / swall, 2), "ms_per_step": round(swall / len(stoks) * 1e3, 4)}
        except l2j.L2JError as e:  # a vocabulary above the device sampler's limit
            out["sampled_decode"] = {"error": str(e)}
        g.reset()

    if (not a.no_batched or a.prefill_only) and not long_context:
        # Not the metric either: 32 (and 16) sequences decoded at once (every weight read once per step for all of them, the
        # products on the bf16 matrix cores); sequence 0 has the prompt of the timed run and must repeat its tokens.
        try:
            bsteps = min(steps, 288)
            n0 = min(bsteps, len(tokens))
            bmean = (bsteps - 1) / 2.0 + 0.5   # mean position of the timed steps 1 .. bsteps - 1
            wbytes = g.bytes_per_token(0)      # the weights, read once per step for all sequences
            kvbytes = g.bytes_per_token(int(round(bmean))) - wbytes   # one sequence's cache rows at the mean position
            runs = {}
            for n_seq in (() if a.prefill_only else (32, 16)):
                prompts = [prompt] + [synth_prompt(seed + 1000 + b, n_prompt, shape[5]) for b in range(1, n_seq)]
                if n_seq == 32:
                    prompts32 = prompts
                g.decode_greedy_batch(prompts, min(bsteps, 8), n_seq=n_seq)          # warm
                btoks, bsec = g.decode_greedy_batch(prompts, bsteps, n_seq=n_seq)
                per = bsec / (bsteps - 1)
                runs[n_seq] = {"sequences": n_seq, "steps": bsteps, "tok_s": round(n_seq * (bsteps - 1) / bsec, 1), "ms_per_step": round(per * 1e3, 4),
                               "roofline": {"bound": "hbm", "achieved": round((wbytes + n_seq * kvbytes) / per / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                                            "frac": round((wbytes + n_seq * kvbytes) / per / 8e12, 4),
                                            "bytes_per_step": int(wbytes + n_seq * kvbytes),
                                            "note": "weights once + every sequence's KV cache rows at the mean position, over the whole step time"},
                               "sequence_0_equals_the_single_decode": bool(np.array_equal(btoks[0, :n0], tokens[:n0]))}
            if runs:
                try:   # the same 32 loops with a sampler each, at the reference's default temperature and top-p (J/CommandLine.java:24-25)
                    stoks32, ssec32 = g.decode_sample_batch(prompts32, bsteps, 0.9, 0.9, np.arange(32, dtype=np.int64) + seed, n_seq=32)
                    runs[32]["sampled"] = {"temperature": 0.9, "topp": 0.9, "tok_s": round(32 * (bsteps - 1) / ssec32, 1),
                                           "ms_per_step": round(ssec32 / (bsteps - 1) * 1e3, 4)}
                except l2j.L2JError as e:   # a vocabulary above the one-launch sampling step's
                    runs[32]["sampled"] = {"error": str(e)}
                out["batched_decode"] = runs[32]
                out["batched_decode"]["sixteen_sequences"] = {k: runs[16][k] for k in ("tok_s", "ms_per_step", "sequence_0_equals_the_single_decode")}
        except l2j.L2JError as e:  # shapes the batched path does not take (rows that are not whole groups of 256)
            out["batched_decode"] = {"error": str(e)}
        # Nor this: the forward passes of 1024 consecutive positions of one sequence, 32 at a time through the same products
        # (l2j_prefill), as a prompt of that length would be taken instead of one position per launch.
        try:
            n_pre = min(1024, shape[6] - 1)
            ptoks = np.concatenate([[1], tokens[:min(len(tokens), n_pre - 1)],
                                    synth_prompt(seed + 77, max(0, n_pre - 1 - len(tokens)), shape[5])]).astype(np.int32)[:n_pre]
            g.reset()
            g.prefill(ptoks[:32], want_logits=False)     # warm
            g.reset()
            _, psec = g.prefill(ptoks, want_logits=False)
            out["prefill"] = {"positions": int(n_pre), "positions_per_s": round(n_pre / psec, 1), "ms": round(psec * 1e3, 3),
                              "ms_per_32_positions": round(psec * 1e3 / ((n_pre + 31) // 32), 4),
                              "note": "l2j_prefill: the forward passes of consecutive positions of one sequence, 32 per step on the "
                                      "matrix cores, into the KV cache of the single-sequence path (device time)"}
            g.reset()
        except l2j.L2JError as e:
            out["prefill"] = {"error": str(e)}

    if a.calibrate_copy > 0:
        g.calibration_copy(a.calibrate_copy << 20, 3)
    if not a.no_kernels:
        pos = int(round(mean_pos))
        kern = {}
        for k in range(7):
            try:
                us, b = g.time_kernel(k, pos, rounds=32 if k == KERNEL.TOKEN else 3)
            except l2j.L2JError:
                if k != KERNEL.TOKEN:
                    raise
                continue  # small models run one launch per phase: there is no whole-token kernel to time
            kern[KERNEL.NAMES[k]] = {"us": round(us, 3), "bytes": b, "GBps": round(b / us * 1e-3, 1),
                                     "frac": round(b / us * 1e-3 / HBM_PEAK_GBS, 4)}
        # "token" is the kernel the forward pass runs; the six others are its phases launched as kernels of
        # their own (once per layer), for orientation
        out["kernels"] = kern
        dom_name = "token" if "token" in kern else "w13"
        dom = dict(kern[dom_name])
        measured = ("start/stop events of single launches (hipExtLaunchKernelGGL), %d launches at position %d" %
                    (32 if dom_name == "token" else 3, pos))
        if dom_name == "token" and sec_after_first > 0 and done > 1:
            # The timed decode itself: its stream holds nothing but one k_token launch per token, back to back (32 per graph
            # replay); the workgroup that ends a token stores the device's wall clock in its loop step, and
            # l2j_decode_greedy returns the difference between the stamps of the first and the last token.  (An event pair
            # around every single launch, as in "kernels" above, adds about 2 % to each.)
            us = sec_after_first / (done - 1) * 1e6
            dom = {"us": round(us, 3), "bytes": bytes_tok, "GBps": round(bytes_tok / us * 1e-3, 1),
                   "frac": round(bytes_tok / us * 1e-3 / HBM_PEAK_GBS, 4)}
            measured = ("device wall-clock stamps (s_memrealtime at %d kHz, hipDeviceAttributeWallClockRate) stored by the last "
                        "workgroup of each k_token launch in its loop step: (stamp of position %d - stamp of position 0) / %d, the "
                        "launch-to-launch period of the %d launches that follow the first token's (nothing else is on the "
                        "stream); bytes at the mean position %d" % (g.get_option("wall_clock_khz"), done - 1, done - 1, done - 1, pos))
        ct = COUNTER_TRAFFIC.get(a.workload) if dom_name == "token" else None
        out["roofline"] = {"bound": "hbm",
                           "kernel": "k_token (all phases of all layers + classifier), one launch per token" if dom_name == "token"
                           else "k_matvec<PH_W13> (rmsnorm + W1,W3 matvec + SwiGLU), one launch per layer",
                           "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac"],
                           "algorithmic_bytes_per_launch": dom["bytes"], "us_per_launch": dom["us"], "measured": measured,
                           "position": pos, "traffic": ct["hbm_bytes_per_launch"] if ct else None,
                           "traffic_source": ("not measured by this run: %s, positions %s (algorithmic bytes there: %d), collected %s" %
                                              (ct["source"], ct["positions"], ct["algorithmic_bytes_at_those_positions"], ct["collected"]))
                           if ct else None}
    else:
        out["roofline"] = None

    g_tokens = tokens.copy()
    g.close()  # graph, events, buffers and stream are released here, before anything of the CPU leg or of exit runs
    if long_context:
        out["cpu_baseline"] = lc_cpu
    elif a.cpu_steps > 1:
        # (a bounded sample of its own length, about 10-30 s of CPU work: it does not shrink with a short timed run; the
        # tokens compared are the generated positions both runs have)
        out["cpu_baseline"] = cpu_baseline(shape, seed, prompt, g_tokens, min(a.cpu_steps, shape[6]))
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
