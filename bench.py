#!/usr/bin/env python3
"""Benchmark of the catgrad `Backend` hot path on one MI355X.

Workload (BASELINE.json configs[4], the configuration the metric is quoted on):
Llama-3.2-1B-shaped decoder, random-init f32 (matrices ~ N(0, 0.02), norm gains 1),
batch 4, prefill 2048 uniform-random tokens each, then 256 greedy decode steps with KV
cache — run through the host driver (the C++ mirror of catgrad's interpreter and
`LlamaModel` graph) over HipBackend.  One "step" is one full prefill + decode pass.
Timing follows `llama --bench` (catgrad-llm/examples/llama/main.rs:914-917): prefill time
is the first run including the read-back of its tokens, decode time is the remaining runs.

Prints ONE JSON line: whole-job tok/s (prefill + decode tokens over their wall time, model
and prompt resident in HBM), with
  roofline      dominant kernel of the prefill (MFMA GEMM), timed live with HIP events on
                the backend's stream around every launch of the timed region
  decode_roofline  the HBM-bound skinny GEMM of the decode loop, every 8th launch timed
  cpu_baseline  the CPU oracle (NdArrayBackend restated, 1 thread) on a bounded sample of
                the same workload
  micro         BASELINE.json configs[1] op micro-benchmarks (device time per launch)
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12       # B/s, MI355X HBM3E
MFMA_F32_PEAK = 157.3e12  # flop/s, MI355X dense f32 matrix


def profiled_traffic():
    """HBM bytes per launch of the dominant kernel (mfma_gemm_kernel) on the config-5 prefill, as the rocprofv3
    FETCH_SIZE / WRITE_SIZE passes measured them: read from the committed summary (its line
    `traffic_bytes_per_launch: <n>`), not measured by this process (counters need the profiler)."""
    path = os.path.join(ROOT, "profiles", "mfma_gemm_llama1b_prefill_pmc.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


def micro_bench(iters=20):
    """configs[1]: device time per launch from HIP events, algorithmic bytes / flop."""
    from catgrad_amd import HipBackend, _abi as A

    be = HipBackend(0)
    rng = np.random.default_rng(0)
    out = {}

    def run(name, cls, fn, unit, launches_per_call=1, mfma_peak=MFMA_F32_PEAK):
        # warm up to steady clocks: the uploads before a line leave the card idle long enough for it to clock down, and
        # the first few milliseconds of launches after that run up to 15 % slow
        t_warm = time.perf_counter()
        while True:
            for _ in range(3):
                fn()
            be.sync()
            if time.perf_counter() - t_warm >= 0.05:
                break
        be.profile_enable(cls, 1)
        be.profile_read(cls, reset=True)
        for _ in range(iters):
            fn()
        n, ms, work = be.profile_read(cls, reset=True)
        be.profile_enable(cls, 0)
        n = n / launches_per_call      # an op of several launches (the two halves of a concat): time and bytes of all
        per = max(ms / max(n, 1) * 1e-3, 1e-12)
        rate = work / max(n, 1) / per
        peak = mfma_peak if unit == "TFLOP/s" else HBM_PEAK
        out[name] = {"us": round(per * 1e6, 2), "achieved": round(rate / (1e12 if unit == "TFLOP/s" else 1e9), 2),
                     "unit": unit, "frac": round(rate / peak, 4)}

    n = 8192
    a = be.from_numpy(rng.standard_normal((n, n), dtype=np.float32))
    b = be.from_numpy(rng.standard_normal((n, n), dtype=np.float32))
    run("add_f32_8192x8192", A.K_ELEMENTWISE, lambda: be.realize(be.add(a, b)), "GB/s")
    run("mul_f32_8192x8192", A.K_ELEMENTWISE, lambda: be.realize(be.mul(a, b)), "GB/s")
    run("exp_f32_8192x8192", A.K_ELEMENTWISE, lambda: be.realize(be.exp(a)), "GB/s")
    del a, b
    r = be.from_numpy(rng.standard_normal((4096, n), dtype=np.float32))
    run("sum_last_4096x8192", A.K_REDUCE, lambda: be.realize(be.sum(r)), "GB/s")
    run("max_last_4096x8192", A.K_REDUCE, lambda: be.realize(be.max(r)), "GB/s")
    del r
    row = be.from_numpy(rng.standard_normal((1, n), dtype=np.float32))
    run("broadcast_1x8192_to_4096x8192_materialised", A.K_ELEMENTWISE,
        lambda: be.realize(be.reshape(be.broadcast(row, (4096, n)), (4096 * n,))), "GB/s")
    x = be.from_numpy(rng.standard_normal((16, 1024, 1024), dtype=np.float32))
    y = be.from_numpy(rng.standard_normal((16, 1024, 1024), dtype=np.float32))
    run("bmm_f32_16x1024x1024x1024", A.K_GEMM_MFMA, lambda: be.matmul(x, y), "TFLOP/s")
    del x, y
    # a linear layer of the 1B-shape prefill on the narrow dtypes (the reduced-precision row of the path): both operands lie
    # in memory as 2-byte / 1-byte patterns (the weight cast once, the activations by a cast per launch, which is an
    # element-wise launch of its own) and are multiplied as they lie on the 16-bit / fp8 matrix instructions, the result
    # rounded to the dtype in the product's store; against the dense peaks of those instructions
    x32 = be.from_numpy(rng.standard_normal((1, 8192, 2048), dtype=np.float32) * np.float32(0.25))
    w32 = be.from_numpy(rng.standard_normal((8192, 2048), dtype=np.float32) * np.float32(0.25))
    for dt, tag, peak in ((A.BF16, "bf16", 2.5e15), (A.F8, "fp8", 5.0e15)):
        wn = be.cast(w32, dt)
        be.realize(wn)
        wv = be.broadcast(be.transpose(wn, 0, 1), (1, 2048, 8192))
        run(f"linear_{tag}_8192x2048x8192", A.K_GEMM_MFMA, lambda: be.matmul(be.cast(x32, dt), wv), "TFLOP/s", mfma_peak=peak)
        del wn, wv
    del x32, w32
    # the same kernels on tensors that lie in memory as 2-byte patterns (bf16): 2 bytes per element read and written
    ab = be.cast(be.from_numpy(rng.standard_normal((n, n), dtype=np.float32)), A.BF16)
    bb = be.cast(be.from_numpy(rng.standard_normal((n, n), dtype=np.float32)), A.BF16)
    be.realize(ab), be.realize(bb)
    run("add_bf16_8192x8192", A.K_ELEMENTWISE, lambda: be.realize(be.add(ab, bb)), "GB/s")
    run("sum_last_bf16_8192x8192", A.K_REDUCE, lambda: be.realize(be.sum(ab)), "GB/s")
    run("transpose_bf16_8192x8192_materialised", A.K_ELEMENTWISE,
        lambda: be.realize(be.reshape(be.transpose(ab, 0, 1), (n * n,))), "GB/s")
    del ab, bb
    # the strided / indexing kernels of the path: a materialised transpose, concat along the outermost and the innermost
    # axis, the embedding gather of the 1B-shape prefill and a sum over a non-last axis (8 bytes per element moved,
    # 4 per element reduced)
    a = be.from_numpy(rng.standard_normal((n, n), dtype=np.float32))
    run("transpose_8192x8192_materialised", A.K_ELEMENTWISE,
        lambda: be.realize(be.reshape(be.transpose(a, 0, 1), (n * n,))), "GB/s")
    run("sum_axis0_8192x8192", A.K_REDUCE, lambda: be.realize(be.sum(be.transpose(a, 0, 1))), "GB/s")
    h = be.from_numpy(rng.standard_normal((n // 2, n), dtype=np.float32))
    g = be.from_numpy(rng.standard_normal((n // 2, n), dtype=np.float32))
    hv, gv = be.slice(h, 1, 0, n // 2), be.slice(g, 1, 0, n // 2)     # [4096, 4096] views of row pitch 8192
    run("concat_dim0_2x4096x8192", A.K_ELEMENTWISE, lambda: be.concat(h, g, 0), "GB/s", launches_per_call=2)
    # along the last axis the result stays a deferred two-part view until something needs memory; then two strided copies
    run("concat_dim1_2x4096x4096", A.K_ELEMENTWISE, lambda: be.realize(be.concat(hv, gv, 1)), "GB/s", launches_per_call=2)
    del a, h, g, hv, gv
    wte = be.from_numpy(rng.standard_normal((128256, 2048), dtype=np.float32))
    ids = be.from_numpy(rng.integers(0, 128256, size=(8192,), dtype=np.uint32))
    run("index_embedding_128256x2048_8192ids", A.K_GATHER, lambda: be.index(wte, 0, ids), "GB/s")
    del wte, ids
    be.pool_trim()
    return out


def cpu_baseline(cfg, params, B, sample_prefill, sample_decode, seed, gpu_tokens=None):
    """The oracle on this box's host cores (it is single-threaded, like NdArrayBackend) on a bounded sample of the
    workload: the same model at the measured batch size, a short prompt and few steps.  A forward pass of the oracle
    costs about the same whatever its token count (most of it is materialising the batch-broadcast weight views, as
    ndarray.rs:553-559 does), so the per-token rates of the sample overstate what the full 2048 + 256 run would
    reach per token of prefill and understate nothing: they are reported as measured, with the sample named.
    gpu_tokens: what HipBackend generated for the same sample prompt; compared token for token."""
    from catgrad_amd.runner import Session

    lib = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(lib):
        return None
    s = Session(lib)
    s.load_model(cfg, params=params)
    prompt = sample_prompt(cfg, B, sample_prefill, seed)
    t0 = time.perf_counter()
    toks, st = s.generate(prompt, steps=sample_decode, max_positions=sample_prefill + sample_decode)
    wall = time.perf_counter() - t0
    s.close()
    tokens = B * (sample_prefill + sample_decode)
    out = {
        "value": round(tokens / (st["prefill_s"] + st["decode_s"]), 3), "unit": "tok/s", "cores": 1,
        "host_cores": os.cpu_count(), "kind": "port",
        "sample": f"same model, batch {B}; prefill {sample_prefill} tokens/seq + {sample_decode} decode steps "
                  f"({wall:.1f} s of CPU work); prefill {B * sample_prefill / st['prefill_s']:.2f} tok/s, "
                  f"decode {B * sample_decode / max(st['decode_s'], 1e-9):.3f} tok/s; a pass costs about the same for any "
                  f"token count, so the full-size run would be about {st['prefill_s']:.0f} s of prefill per "
                  f"{B * sample_prefill} tokens scaled by the GEMM work, and {st['decode_s'] / max(sample_decode, 1):.0f} s per decode step",
    }
    if gpu_tokens is not None:
        out["tokens_equal_gpu"] = bool((toks == gpu_tokens).all())
    return out


def sample_prompt(cfg, B, S, seed):
    return np.random.default_rng(seed + 1).integers(0, cfg.vocab_size, size=(B, S), dtype=np.uint32)


CONFIGS = {
    5: (4, 2048, 256, "Llama-3.2-1B-shape decoder (hidden 2048, 16 layers, 32/8 heads, MLP 8192, vocab 128256, "
                      "rope theta 500000, tied lm_head)"),
    4: (1, 1024, 128, "Qwen3-0.6B-shape decoder (hidden 1024, 28 layers, 16/8 heads of 128, QK-norm, MLP 3072, "
                      "vocab 151936, tied lm_head)"),
    3: (1, 512, 16, "SmolLM2-135M-shape decoder (hidden 576, 30 layers, 9/3 heads, MLP 1536, vocab 49152, "
                    "tied lm_head)"),
}


def measure(config, steps, warmup, batch=None, prefill=None, decode=None, seed=0):
    """One BASELINE configuration through HipBackend: `warmup` untimed passes, then `steps` timed passes of prefill +
    greedy decode.  Returns (result dict, the open session, config, params, batch)."""
    import torch

    from catgrad_amd import _abi as A
    from catgrad_amd.runner import LLAMA_3_2_1B, QWEN3_0_6B, SMOLLM2_135M, Session, random_params

    cfg = {5: LLAMA_3_2_1B, 4: QWEN3_0_6B, 3: SMOLLM2_135M}[config]
    dB, dS, dT, cfg_name = CONFIGS[config]
    B = batch if batch is not None else dB
    S = prefill if prefill is not None else dS
    T = decode if decode is not None else dT
    params = list(random_params(cfg, seed))
    sess = Session()
    t_up = time.perf_counter()
    sess.load_model(cfg, params=params)
    sess.sync()
    t_up = time.perf_counter() - t_up
    weight_bytes = sum(int(w.size) * 4 for _, w in params)
    prompt = np.random.default_rng(seed).integers(0, cfg.vocab_size, size=(B, S), dtype=np.uint32)

    for _ in range(warmup):
        sess.generate(prompt, steps=T, max_positions=S + T)
    # The launch timings of the decode-time kernels (skinny products, attention) are taken in an untimed pass of their own:
    # two event records around 26 launches of every decode step cost the step 0.065 ms (4 %).  The timed region below
    # carries events only around the dominant kernel, the prefill's GEMM launches (its roofline figure).
    sess.profile_enable(A.K_GEMM_SKINNY, 8)
    sess.profile_enable(A.K_ATTENTION, 1)
    sess.profile_read(A.K_GEMM_SKINNY, reset=True)
    sess.profile_read(A.K_ATTENTION, reset=True)
    sess.generate(prompt, steps=T, max_positions=S + T)
    sess.sync()
    n_s, ms_s, bytes_s = sess.profile_read(A.K_GEMM_SKINNY)
    n_a, ms_a, flop_a = sess.profile_read(A.K_ATTENTION)
    sess.profile_enable(A.K_GEMM_SKINNY, 0)
    sess.profile_enable(A.K_ATTENTION, 0)
    sess.profile_enable(A.K_GEMM_MFMA, 1)
    sess.profile_read(A.K_GEMM_MFMA, reset=True)

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    pp_s = tg_s = 0.0
    calls = (0, 0)
    tokens = None
    for _ in range(steps):
        tokens, st = sess.generate(prompt, steps=T, max_positions=S + T)
        pp_s += st["prefill_s"]
        tg_s += st["decode_s"]
        calls = (st["prefill_calls"], st["decode_calls"])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    n_m, ms_m, flop_m = sess.profile_read(A.K_GEMM_MFMA)
    sess.profile_enable(A.K_GEMM_MFMA, 0)
    attn_rate = flop_a / (ms_a * 1e-3) if ms_a else 0.0
    mfma_rate = flop_m / (ms_m * 1e-3) if ms_m else 0.0
    skinny_rate = bytes_s / (ms_s * 1e-3) if ms_s else 0.0

    K = steps
    total_tokens = K * B * (S + T)
    # algorithmic bytes of a decode step: the matmul weights (lm_head included) once, plus K and V
    # of every layer at the mean cache length of the decode phase
    hd = cfg.head_dim or cfg.hidden_size // cfg.num_attention_heads
    weight_elems = cfg.num_hidden_layers * (
        2 * cfg.hidden_size * cfg.num_attention_heads * hd + 2 * cfg.hidden_size * cfg.num_key_value_heads * hd
        + 3 * cfg.hidden_size * cfg.intermediate_size) + cfg.vocab_size * cfg.hidden_size
    kv_elems = 2 * cfg.num_hidden_layers * B * cfg.num_key_value_heads * (S + T / 2.0) * hd
    step_bytes = int(4 * (weight_elems + kv_elems))
    step_rate = step_bytes / (tg_s / K / T) if T and tg_s else 0.0
    # algorithmic flop of the prefill: every linear layer over all positions (lm_head included) + dense attention
    prefill_flop = 2.0 * B * S * weight_elems + cfg.num_hidden_layers * 4.0 * B * cfg.num_attention_heads * S * S * hd
    result = {
        "metric": "tok/s prefill+decode, Llama-3.2-1B-shape f32; % HBM & MFMA roofline",
        "value": round(total_tokens / (pp_s + tg_s), 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": warmup,
        "ms_per_step": round(wall / K * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"{cfg_name}, random-init f32, batch {B}, prefill {S} random tokens, "
                        f"{T} greedy decode steps with KV cache",
            "baseline_config": config,
            "global_batch": B, "seq_len": S, "decode_steps": T, "parallelism": "single GPU",
        },
        "prefill_tok_s": round(K * B * S / pp_s, 2),
        "decode_tok_s": round(K * B * T / tg_s, 2),
        "prefill_ms": round(pp_s / K * 1e3, 3),
        "decode_ms_per_step": round(tg_s / K / T * 1e3, 4),
        # the whole prefill against the matrix peak: algorithmic flop (all linear layers + dense attention) / prefill time
        "prefill_flop": prefill_flop,
        "prefill_mfma_frac": round(prefill_flop / (pp_s / K) / MFMA_F32_PEAK, 4),
        "backend_calls": {"prefill": calls[0], "per_decode_step": round(calls[1] / max(T, 1), 1)},
        "backend": sess.backend_name,
        "roofline": {
            "kernel": "mfma_gemm_kernel (f32 v_mfma_f32_32x32x2; 128x128x32 tiles, two workgroups per compute unit; 128x64 and "
                      "split-k variants for products that do not fill the device)",
            "bound": "mfma", "achieved": round(mfma_rate / 1e12, 3), "peak": MFMA_F32_PEAK / 1e12, "unit": "TFLOP/s",
            "frac": round(mfma_rate / MFMA_F32_PEAK, 4),
            # from the committed rocprofv3 counter summary of this very workload (null for any other)
            "traffic": profiled_traffic() if (config, B, S) == (5, 4, 2048) else None,
            "traffic_source": "profiles/mfma_gemm_llama1b_prefill_pmc.txt" if (config, B, S) == (5, 4, 2048) else None,
            "launches_timed": n_m, "avg_launch_ms": round(ms_m / max(n_m, 1), 4),
            "flop_per_launch_avg": flop_m / max(n_m, 1),
        },
        # the one-pass causal attention of the prefill (q.K^T, soft-max, p.V): flop of the visible half only
        "prefill_attention": {
            "kernel": "prefill_attention_kernel (f32 v_mfma_f32_32x32x2, 128 query rows x 64 keys per step)",
            "bound": "mfma", "achieved": round(attn_rate / 1e12, 3), "peak": MFMA_F32_PEAK / 1e12, "unit": "TFLOP/s",
            "frac": round(attn_rate / MFMA_F32_PEAK, 4), "launches_timed": n_a,
            "avg_launch_ms": round(ms_a / max(n_a, 1), 4), "timed_in": "an untimed pass of its own, before the timed region",
        },
        "decode_roofline": {
            "scope": "one decode step, all kernels: every weight matrix and the KV cache are read once",
            "bound": "hbm", "bytes_per_step": step_bytes, "achieved": round(step_rate / 1e9, 2), "peak": HBM_PEAK / 1e9,
            "unit": "GB/s", "frac": round(step_rate / HBM_PEAK, 4),
            "skinny_gemm_kernels": {
                "kernels": "skinny_kt_wide / skinny_kt_mfma_xreg / skinny_kt_narrow / skinny_nn (M <= 8)",
                "achieved": round(skinny_rate / 1e9, 2), "unit": "GB/s", "frac": round(skinny_rate / HBM_PEAK, 4),
                "launches_timed": n_s, "avg_launch_us": round(ms_s / max(n_s, 1) * 1e3, 3),
                "timed_in": "an untimed pass of its own, before the timed region (every 8th launch)",
            },
        },
        # the first decoded tokens of the timed run, for eyeballing across builds; what checks tokens is the CPU sample
        # below (cpu_baseline.tokens_equal_gpu) and the full-size parity tests (tests/test_hip_config5.py)
        "first_tokens": tokens[:2].tolist() if tokens is not None else None,
        # not part of `value`: the one-off upload of the weights from pageable host memory through the
        # backend's pinned staging buffers (the PCIe-inclusive cost of a cold start)
        "weights_upload": {"bytes": weight_bytes, "seconds": round(t_up, 3), "GB_per_s": round(weight_bytes / t_up / 1e9, 2)},
    }
    return result, sess, cfg, params, B


def other_config_line(config, steps=2, warmup=1):
    """BASELINE configs 3 and 4 beside the headline line: the same measurement in a few seconds, the figures that
    matter for them (prefill against the matrix peak, decode step against HBM) only."""
    r, sess, _, _, _ = measure(config, steps, warmup)
    sess.close()
    return {
        "workload": r["config"]["workload"], "steps": steps, "warmup": warmup,
        "tok_s": r["value"], "prefill_ms": r["prefill_ms"], "prefill_tok_s": r["prefill_tok_s"],
        "decode_ms_per_step": r["decode_ms_per_step"], "decode_tok_s": r["decode_tok_s"],
        "prefill_mfma_frac": r["prefill_mfma_frac"], "gemm_kernel_mfma_frac": r["roofline"]["frac"],
        "prefill_attention_mfma_frac": r["prefill_attention"]["frac"], "decode_hbm_frac": r["decode_roofline"]["frac"],
        "backend_calls_per_decode_step": r["backend_calls"]["per_decode_step"], "first_tokens": r["first_tokens"],
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", type=int, default=5, choices=[3, 4, 5],
                    help="BASELINE.json configs index + 1: 5 = Llama-3.2-1B shape, batch 4, 2048 + 256 (the metric's "
                         "configuration, default); 4 = Qwen3-0.6B shape, batch 1, 1024 + 128; 3 = SmolLM2-135M shape, "
                         "batch 1, prefill 512 (+ 16 decode steps so that the decode figures exist)")
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--prefill", type=int, default=None)
    ap.add_argument("--decode", type=int, default=None)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-micro", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short runs of BASELINE configs 3 and 4 that the default line carries as `other_configs`")
    ap.add_argument("--cpu-sample", type=int, nargs=3, default=None, metavar=("BATCH", "PREFILL", "DECODE"),
                    help="the CPU baseline's sample (default: the measured batch, prefill 8, 1 decode step)")
    ap.add_argument("--micro-only", action="store_true", help="only the op micro-benchmarks (one JSON line of their own)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a strided copy of known size (268435456 B read + 268435456 B written per launch), "
                         "the yardstick for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this backend runs on ONE GPU; every box in this build has one GPU and the path has no "
              "collective step. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    if args.calibrate_copy:
        from catgrad_amd import HipBackend

        be = HipBackend(0)
        x = be.from_numpy(np.zeros((8192, 8192 + 4), dtype=np.float32))
        for _ in range(10):
            be.realize(be.reshape(be.slice(x, 1, 0, 8192), (8192 * 8192,)))
        be.sync()
        print(json.dumps({"calibration": "ew_kernel<copy> 10 launches", "read_bytes": 8192 * 8192 * 4,
                          "write_bytes": 8192 * 8192 * 4}))
        return

    if args.micro_only:
        print(json.dumps({"micro": micro_bench()}))
        return

    import torch  # device-wide synchronisation around the timed region

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; HipBackend has no CPU fallback.", file=sys.stderr)
        sys.exit(1)

    result, sess, cfg, params, B = measure(args.config, args.steps, args.warmup, args.batch, args.prefill, args.decode, args.seed)
    cpu_sample = args.cpu_sample or [B, 8, 1]
    gpu_sample_tokens = None
    if not args.no_cpu_baseline:   # the CPU sample's prompt through the GPU path too: its tokens are compared below
        gpu_sample_tokens, _ = sess.generate(sample_prompt(cfg, cpu_sample[0], cpu_sample[1], args.seed), steps=cpu_sample[2],
                                             max_positions=cpu_sample[1] + cpu_sample[2])
    sess.close()
    if args.config == 5 and not args.no_other_configs:
        result["other_configs"] = {f"config{c}": other_config_line(c) for c in (3, 4)}
    if not args.no_micro:
        result["micro"] = micro_bench()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg, params, *cpu_sample, args.seed, gpu_tokens=gpu_sample_tokens)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
