"""BASELINE config 5 (Llama-3.2-1B shape, f32, batch 4, prefill 2048 + greedy decode), config 4 (Qwen3-0.6B shape,
batch 1, prefill 1024 + greedy decode) and config 3 (SmolLM2-135M shape, batch 1, prefill 512) on the GPU.

* depth-reduced, full-width models against the CPU oracle: every width of the benchmarked model (hidden 2048, 32 / 8
  heads of 64, MLP 8192, vocabulary 128256, theta 500000, tied head; resp. hidden 1024, 16 / 8 heads of 128, QK norm,
  MLP 3072, vocabulary 151936) with 2 layers — the kernels a layer launches do not depend on the depth;
* the full 16-layer config-5 model and the full 28-layer config-4 model at the benchmark's full size through properties
  that need no CPU recomputation: the fused path against every-op-its-own-kernel (`CG_FUSE=0`) and against the
  interpreter kernels (`CG_AOT=0`), KV-cached decoding against a fresh prefill of the longer sequence, and one
  sequence against an independent float64 model;
* the full 30-layer config-3 model, prefill 512 + 16 greedy decode steps, against the CPU oracle.

Tolerances: logits within 1e-3 of their scale (north star: 1e-3 relative for matmul and reductions); greedy tokens
identical except where the float64 top1-top2 gap is inside twice the measured logit error (a near-tie that another
summation order may legitimately resolve the other way)."""
import os

import numpy as np
import pytest

import np_models
from catgrad_amd.runner import LLAMA_3_2_1B, QWEN3_0_6B, SMOLLM2_135M, LlmConfig, Session, random_params
from model_cases import prompt_of
from oracle_loader import ORACLE_LIB, oracle_library

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]


def _session_with(env):
    old = {k: os.environ.get(k) for k in env}
    os.environ.update(env)
    try:
        return Session()
    finally:
        for k, v in old.items():
            if v is None:
                del os.environ[k]
            else:
                os.environ[k] = v


def _first_real_mismatch(got, ref, gaps, floor):
    """Index of the first differing choice whose float64 gap is above `floor`, or None.  Rows are compared up to their
    first difference only: afterwards the sequences legitimately diverge."""
    for b in range(got.shape[1]):
        d = np.flatnonzero(got[:, b] != ref[:, b])
        if d.size and gaps[d[0], b] > floor:
            return int(d[0]), b
    return None


def _argmax_last(x):
    return (x.shape[-1] - 1 - np.argmax(x[..., ::-1], axis=-1)).astype(np.uint32)


def _reduced(cfg, layers):
    return LlmConfig(cfg.arch, cfg.hidden_size, layers, cfg.num_attention_heads, cfg.num_key_value_heads,
                     cfg.intermediate_size, cfg.vocab_size, head_dim=cfg.head_dim, rms_norm_eps=cfg.rms_norm_eps,
                     rope_theta=cfg.rope_theta, tie_word_embeddings=cfg.tie_word_embeddings)


@pytest.mark.parametrize("name,full,B,S,steps", [("config5_llama1b_widths", LLAMA_3_2_1B, 4, 256, 8),
                                                  ("config4_qwen3_widths", QWEN3_0_6B, 1, 1024, 8)])
def test_depth_reduced_full_width_against_oracle(name, full, B, S, steps):
    cfg = _reduced(full, 2)
    params = dict(random_params(cfg, seed=0))
    prompt = prompt_of(cfg, B, S, seed=0)
    print(f"{name}: hip", flush=True)
    hip = Session()
    hip.load_model(cfg, params=params.items())
    g_h, st, l_h = hip.generate(prompt, steps=steps, max_positions=S + steps, want_logits=True)
    hip.close()
    print(f"{name}: oracle", flush=True)
    oracle_library()
    cpu = Session(ORACLE_LIB)
    cpu.load_model(cfg, params=params.items())
    g_c, _, l_c = cpu.generate(prompt, steps=steps, max_positions=S + steps, want_logits=True)
    cpu.close()
    t_h, t_c = _argmax_last(l_h), _argmax_last(l_c)     # the graph's own arg-max rule (last of equal maxima)
    assert (t_h[:, -1] == g_h[0]).all() and (t_c[:, -1] == g_c[0]).all()
    scale = float(np.abs(l_c).max())
    err = float(np.abs(l_h - l_c).max())
    # prefill choices at every position, gaps from the oracle's own logits
    part = np.partition(l_c, -2, axis=-1)
    gaps_pf = part[..., -1] - part[..., -2]
    flips = t_h != t_c
    # decode choices: float64 gaps of the oracle's sequence, teacher-forced
    print(f"{name}: float64 gaps", flush=True)
    seq = np.concatenate([prompt, g_c[:-1].T], axis=1)
    l64 = np_models.llm_logits(cfg, params, seq, positions=range(S - 1, S + steps))
    srt = np.sort(l64, -1)
    gaps = (srt[..., -1] - srt[..., -2]).T                      # [steps + 1, B]
    err64 = float(np.abs(l_c[:, -1, :] - l64[:, 0, :]).max())
    print(f"{name}: max |dlogit| hip-oracle {err:.3e}, oracle-float64 {err64:.3e} (scale {scale:.3e}); prefill flips "
          f"{int(flips.sum())}/{flips.size} (min gap {gaps_pf.min():.3e}); decode calls/step {st['decode_calls'] / steps:.0f}; "
          f"decode mismatches {int((g_h != g_c).sum())}", flush=True)
    assert err <= 1e-3 * scale
    assert err64 <= 1e-3 * scale
    assert not (flips & (gaps_pf > 2 * err)).any()
    assert _first_real_mismatch(g_h, g_c, gaps, 2 * max(err, err64)) is None


FULL = {"config5": (LLAMA_3_2_1B, 4, 2048, [0, 1, 511, 1024, 2047]),   # config, batch, prefill, positions whose logits are read back
        "config4": (QWEN3_0_6B, 1, 1024, [0, 1, 255, 511, 1023])}


@pytest.fixture(scope="module", params=list(FULL))
def full_model(request):
    cfg, B, S, sampled = FULL[request.param]
    params = dict(random_params(cfg, seed=0))
    prompt = prompt_of(cfg, B, S, seed=0)
    return request.param, cfg, params, prompt, sampled


def _rows(B, S, positions):
    return np.array([b * S + s for b in range(B) for s in positions], np.uint32)


def test_full_size_fused_against_unfused_and_interpreted(full_model):
    """Configs 5 and 4 at full size: the default path against `CG_FUSE=0` (every op its own kernel, no lazy products, no
    one-pass attention) and `CG_AOT=0` (fused programs through the interpreter kernels)."""
    name, cfg, params, prompt, SAMPLED = full_model
    (B, S), T = prompt.shape, 8
    outs = {}
    for tag, env in (("default", {}), ("unfused", {"CG_FUSE": "0"}), ("interpreted", {"CG_AOT": "0"})):
        print(f"{name} full size: {tag}", flush=True)
        s = _session_with(env)
        s.load_model(cfg, params=params.items())
        toks, lg = s.forward_rows(prompt, _rows(B, S, SAMPLED), max_positions=S + T)
        gen, st = s.generate(prompt, steps=T, max_positions=S + T)
        outs[tag] = (toks, lg, gen)
        s.close()
    t_d, l_d, g_d = outs["default"]
    scale = float(np.abs(l_d).max())
    srt = np.sort(l_d, -1)
    for tag in ("unfused", "interpreted"):
        t_o, l_o, g_o = outs[tag]
        err = float(np.abs(l_d - l_o).max())
        flips = int((t_d != t_o).sum())
        print(f"{name} full size: default vs {tag}: max |dlogit| {err:.3e} (scale {scale:.3e}); prefill argmax flips "
              f"{flips}/{t_d.size}; decode mismatches {int((g_d != g_o).sum())}", flush=True)
        assert err <= 1e-3 * scale
        # sampled positions: a flip only where the two best logits are within twice the error
        best_d, best_o = l_d.argmax(-1), l_o.argmax(-1)
        gap = srt[:, -1] - srt[:, -2]
        assert not ((best_d != best_o) & (gap > 2 * err)).any()
        assert flips <= max(t_d.size // 200, 2)      # all positions: flips are near-ties, rare at N(0, 0.02) logits
    outs.clear()


def test_full_size_cached_decode_against_fresh_prefill_and_float64(full_model):
    """Greedy decoding with the KV cache equals the argmax of a fresh prefill of prompt + generated tokens at the same
    positions; sequence 0 is also recomputed by the independent float64 model (logits of the sampled positions)."""
    name, cfg, params, prompt, _ = full_model
    (B, S), T = prompt.shape, 8
    s = Session()
    s.load_model(cfg, params=params.items())
    gen, _ = s.generate(prompt, steps=T, max_positions=S + T)          # [T + 1, B]
    seq = np.concatenate([prompt, gen[:-1].T], axis=1)                   # [B, S + T]
    pos = list(range(S - 1, S + T))
    toks, lg = s.forward_rows(seq, _rows(B, S + T, pos), max_positions=S + T)
    s.close()
    lg = lg.reshape(B, len(pos), -1)
    srt = np.sort(lg, -1)
    gaps = (srt[..., -1] - srt[..., -2]).T                               # [T + 1, B]
    fresh = toks[:, S - 1:].T                                             # [T + 1, B]
    scale = float(np.abs(lg).max())
    print(f"{name} full size: cached vs fresh prefill: mismatches {int((gen != fresh).sum())}/{gen.size}, "
          f"min gap {gaps.min():.3e} (scale {scale:.3e})", flush=True)
    assert _first_real_mismatch(gen, fresh, gaps, 2e-3 * scale) is None
    # sequence 0 in float64 (weights widened layer by layer)
    print(f"{name} full size: float64 model of sequence 0", flush=True)
    l64 = np_models.llm_logits(cfg, params, seq[:1], positions=pos)[0]   # [T + 1, V]
    err = float(np.abs(lg[0] - l64).max())
    s64 = np.sort(l64, -1)
    gap64 = s64[:, -1] - s64[:, -2]
    best64 = l64.argmax(-1)
    print(f"{name} full size: hip vs float64, sequence 0: max |dlogit| {err:.3e} (scale {scale:.3e}); "
          f"argmax differs at {int((lg[0].argmax(-1) != best64).sum())}/{len(pos)}", flush=True)
    assert err <= 1e-3 * scale
    assert not ((lg[0].argmax(-1) != best64) & (gap64 > 2 * err)).any()


def test_config3_full_model_prefill_and_decode_against_oracle():
    """BASELINE config 3 at full size (SmolLM2-135M shape: hidden 576, 30 layers, 9 / 3 heads of 64, MLP 1536,
    vocabulary 49152): prefill 512 tokens, then 16 greedy decode steps with the KV cache, logits and tokens against the
    CPU oracle with the gap rule (float64 gaps of the oracle's own sequence)."""
    cfg = SMOLLM2_135M
    B, S, steps = 1, 512, 16
    params = dict(random_params(cfg, seed=0))
    prompt = prompt_of(cfg, B, S, seed=0)
    print("config3: hip", flush=True)
    hip = Session()
    hip.load_model(cfg, params=params.items())
    g_h, st, l_h = hip.generate(prompt, steps=steps, max_positions=S + steps, want_logits=True)
    hip.close()
    print("config3: oracle", flush=True)
    oracle_library()
    cpu = Session(ORACLE_LIB)
    cpu.load_model(cfg, params=params.items())
    g_c, _, l_c = cpu.generate(prompt, steps=steps, max_positions=S + steps, want_logits=True)
    cpu.close()
    scale = float(np.abs(l_c).max())
    err = float(np.abs(l_h - l_c).max())
    t_h, t_c = _argmax_last(l_h), _argmax_last(l_c)
    part = np.partition(l_c, -2, axis=-1)
    gaps_pf = part[..., -1] - part[..., -2]
    flips = t_h != t_c
    print("config3: float64 gaps", flush=True)
    seq = np.concatenate([prompt, g_c[:-1].T], axis=1)
    l64 = np_models.llm_logits(cfg, params, seq, positions=range(S - 1, S + steps))
    srt = np.sort(l64, -1)
    gaps = (srt[..., -1] - srt[..., -2]).T
    err64 = float(np.abs(l_c[:, -1, :] - l64[:, 0, :]).max())
    print(f"config3: max |dlogit| hip-oracle {err:.3e}, oracle-float64 {err64:.3e} (scale {scale:.3e}); prefill flips "
          f"{int(flips.sum())}/{flips.size}; decode calls/step {st['decode_calls'] / steps:.0f}; decode mismatches "
          f"{int((g_h != g_c).sum())}/{g_h.size}", flush=True)
    assert err <= 1e-3 * scale
    assert err64 <= 1e-3 * scale
    assert not (flips & (gaps_pf > 2 * err)).any()
    assert _first_real_mismatch(g_h, g_c, gaps, 2 * max(err, err64)) is None
