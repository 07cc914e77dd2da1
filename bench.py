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


# HBM bytes per mfma_gemm_kernel launch of this workload's prefill, from rocprofv3 FETCH_SIZE / WRITE_SIZE passes
# scaled by a copy kernel of known size (profiles/mfma_gemm_llama1b_prefill_pmc.txt); counters cannot be read
# from inside this process, so the figure is carried here and only reported for the profiled shape.
MFMA_GEMM_TRAFFIC_PER_LAUNCH = 0.691e9


def micro_bench(iters=20):
    """configs[1]: device time per launch from HIP events, algorithmic bytes / flop."""
    from catgrad_amd import HipBackend, _abi as A

    be = HipBackend(0)
    rng = np.random.default_rng(0)
    out = {}

    def run(name, cls, fn, unit):
        for _ in range(3):
            fn()
        be.sync()
        be.profile_enable(cls, 1)
        be.profile_read(cls, reset=True)
        for _ in range(iters):
            fn()
        n, ms, work = be.profile_read(cls, reset=True)
        be.profile_enable(cls, 0)
        per = max(ms / max(n, 1) * 1e-3, 1e-12)
        rate = work / max(n, 1) / per
        peak = MFMA_F32_PEAK if unit == "TFLOP/s" else HBM_PEAK
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
    be.pool_trim()
    return out


def cpu_baseline(cfg, params, B, sample_prefill, sample_decode, seed):
    """The oracle on this box's host cores (it is single-threaded, like NdArrayBackend) on a
    bounded sample of the workload: same model, a short prompt and few steps, at the
    batch size the reference's own CLI uses (1; catgrad-llm/examples/llama/main.rs:947-951).
    With batch 4 one forward pass alone takes about a minute of CPU time, most of it
    materialising the batch-broadcast weight views."""
    from catgrad_amd.runner import Session

    lib = os.path.join(ROOT, "oracle", "liboracle.so")
    if not os.path.exists(lib):
        return None
    s = Session(lib)
    s.load_model(cfg, params=params)
    prompt = np.random.default_rng(seed).integers(0, cfg.vocab_size, size=(B, sample_prefill), dtype=np.uint32)
    t0 = time.perf_counter()
    _, st = s.generate(prompt, steps=sample_decode, max_positions=sample_prefill + sample_decode)
    wall = time.perf_counter() - t0
    s.close()
    tokens = B * (sample_prefill + sample_decode)
    return {
        "value": round(tokens / (st["prefill_s"] + st["decode_s"]), 3), "unit": "tok/s", "cores": 1,
        "host_cores": os.cpu_count(), "kind": "port",
        "sample": f"same model, batch {B}; prefill {sample_prefill} tokens/seq + {sample_decode} decode steps "
                  f"({wall:.1f} s of CPU work); prefill {B * sample_prefill / st['prefill_s']:.2f} tok/s, "
                  f"decode {B * sample_decode / max(st['decode_s'], 1e-9):.3f} tok/s",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--prefill", type=int, default=2048)
    ap.add_argument("--decode", type=int, default=256)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-micro", action="store_true")
    ap.add_argument("--cpu-sample", type=int, nargs=3, default=[1, 4, 1], metavar=("BATCH", "PREFILL", "DECODE"))
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

    import torch  # device-wide synchronisation around the timed region

    from catgrad_amd import _abi as A
    from catgrad_amd.runner import LLAMA_3_2_1B, Session, random_params

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; HipBackend has no CPU fallback.", file=sys.stderr)
        sys.exit(1)

    cfg = LLAMA_3_2_1B
    B, S, T = args.batch, args.prefill, args.decode
    params = list(random_params(cfg, args.seed))
    sess = Session()
    t_up = time.perf_counter()
    sess.load_model(cfg, params=params)
    sess.sync()
    t_up = time.perf_counter() - t_up
    weight_bytes = sum(int(w.size) * 4 for _, w in params)
    prompt = np.random.default_rng(args.seed).integers(0, cfg.vocab_size, size=(B, S), dtype=np.uint32)

    for _ in range(args.warmup):
        sess.generate(prompt, steps=T, max_positions=S + T)
    sess.profile_enable(A.K_GEMM_MFMA, 1)
    sess.profile_enable(A.K_GEMM_SKINNY, 8)
    sess.profile_enable(A.K_ATTENTION, 1)
    sess.profile_read(A.K_GEMM_MFMA, reset=True)
    sess.profile_read(A.K_GEMM_SKINNY, reset=True)
    sess.profile_read(A.K_ATTENTION, reset=True)

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    pp_s = tg_s = 0.0
    calls = (0, 0)
    tokens = None
    for _ in range(args.steps):
        tokens, st = sess.generate(prompt, steps=T, max_positions=S + T)
        pp_s += st["prefill_s"]
        tg_s += st["decode_s"]
        calls = (st["prefill_calls"], st["decode_calls"])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    n_m, ms_m, flop_m = sess.profile_read(A.K_GEMM_MFMA)
    n_s, ms_s, bytes_s = sess.profile_read(A.K_GEMM_SKINNY)
    n_a, ms_a, flop_a = sess.profile_read(A.K_ATTENTION)
    sess.profile_enable(A.K_GEMM_MFMA, 0)
    sess.profile_enable(A.K_GEMM_SKINNY, 0)
    sess.profile_enable(A.K_ATTENTION, 0)
    attn_rate = flop_a / (ms_a * 1e-3) if ms_a else 0.0
    mfma_rate = flop_m / (ms_m * 1e-3) if ms_m else 0.0
    skinny_rate = bytes_s / (ms_s * 1e-3) if ms_s else 0.0

    K = args.steps
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
    result = {
        "metric": "tok/s prefill+decode, Llama-3.2-1B-shape f32; % HBM & MFMA roofline",
        "value": round(total_tokens / (pp_s + tg_s), 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": round(wall / K * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"Llama-3.2-1B-shape decoder (hidden 2048, 16 layers, 32/8 heads, MLP 8192, vocab 128256, "
                        f"rope theta 500000, tied lm_head), random-init f32, batch {B}, prefill {S} random tokens, "
                        f"{T} greedy decode steps with KV cache",
            "global_batch": B, "seq_len": S, "decode_steps": T, "parallelism": "single GPU",
        },
        "prefill_tok_s": round(K * B * S / pp_s, 2),
        "decode_tok_s": round(K * B * T / tg_s, 2),
        "prefill_ms": round(pp_s / K * 1e3, 3),
        "decode_ms_per_step": round(tg_s / K / T * 1e3, 4),
        "backend_calls": {"prefill": calls[0], "per_decode_step": round(calls[1] / max(T, 1), 1)},
        "backend": sess.backend_name,
        "roofline": {
            "kernel": "mfma_gemm_kernel (f32 v_mfma_f32_32x32x2; 256x256x32 tiles, 128x128 and 128x64 for small N)",
            "bound": "mfma", "achieved": round(mfma_rate / 1e12, 3), "peak": MFMA_F32_PEAK / 1e12, "unit": "TFLOP/s",
            "frac": round(mfma_rate / MFMA_F32_PEAK, 4),
            "traffic": MFMA_GEMM_TRAFFIC_PER_LAUNCH if (B, S) == (4, 2048) else None,
            "launches_timed": n_m, "avg_launch_ms": round(ms_m / max(n_m, 1), 4),
            "flop_per_launch_avg": flop_m / max(n_m, 1),
        },
        # the one-pass causal attention of the prefill (q.K^T, soft-max, p.V): flop of the visible half only
        "prefill_attention": {
            "kernel": "prefill_attention_kernel (f32 v_mfma_f32_32x32x2, 128 query rows x 64 keys per step)",
            "bound": "mfma", "achieved": round(attn_rate / 1e12, 3), "peak": MFMA_F32_PEAK / 1e12, "unit": "TFLOP/s",
            "frac": round(attn_rate / MFMA_F32_PEAK, 4), "launches_timed": n_a,
            "avg_launch_ms": round(ms_a / max(n_a, 1), 4),
        },
        "decode_roofline": {
            "scope": "one decode step, all kernels: every weight matrix and the KV cache are read once",
            "bound": "hbm", "bytes_per_step": step_bytes, "achieved": round(step_rate / 1e9, 2), "peak": HBM_PEAK / 1e9,
            "unit": "GB/s", "frac": round(step_rate / HBM_PEAK, 4),
            "skinny_gemm_kernels": {
                "kernels": "skinny_kt_wide / skinny_kt_mfma_xreg / skinny_kt_narrow / skinny_nn (M <= 8)",
                "achieved": round(skinny_rate / 1e9, 2), "unit": "GB/s", "frac": round(skinny_rate / HBM_PEAK, 4),
                "launches_timed": n_s, "avg_launch_us": round(ms_s / max(n_s, 1) * 1e3, 3),
            },
        },
        "first_tokens": tokens[:2].tolist() if tokens is not None else None,
        # not part of `value`: the one-off upload of the weights from pageable host memory through the
        # backend's pinned staging buffers (the PCIe-inclusive cost of a cold start)
        "weights_upload": {"bytes": weight_bytes, "seconds": round(t_up, 3), "GB_per_s": round(weight_bytes / t_up / 1e9, 2)},
    }
    sess.close()
    if not args.no_micro:
        result["micro"] = micro_bench()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg, params, *args.cpu_sample, args.seed)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
