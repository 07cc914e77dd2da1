"""Small model configurations shared by the CPU and GPU model tests."""
import numpy as np

from catgrad_amd.runner import LlmConfig, random_params

TINY_LLAMA = LlmConfig("llama", 64, 3, 4, 2, 160, 211, rope_theta=500000.0, tie_word_embeddings=True)
TINY_LLAMA_UNTIED = LlmConfig("llama", 48, 2, 6, 6, 96, 130, rope_theta=10000.0, tie_word_embeddings=False)
TINY_QWEN3 = LlmConfig("qwen3", 64, 3, 4, 2, 128, 257, head_dim=32, rms_norm_eps=1e-6, rope_theta=1000000.0,
                       tie_word_embeddings=True)
TINY = {"tiny_llama": TINY_LLAMA, "tiny_llama_untied": TINY_LLAMA_UNTIED, "tiny_qwen3": TINY_QWEN3}


def params_of(cfg, seed=0, scale=1.0):
    """Weights as a dict.  `scale` > 1 spreads the logits of these tiny models so that
    greedy choices are not near-ties."""
    out = {}
    for name, w in random_params(cfg, seed):
        out[name] = w * np.float32(scale) if w.ndim == 2 else w
    return out


def prompt_of(cfg, B, S, seed=1):
    return np.random.default_rng(seed).integers(0, cfg.vocab_size, size=(B, S), dtype=np.uint32)


def mlp_case(seed=0):
    """BASELINE config 1: x f32[64,256] ~ N(0,1), Linear(256->512, W ~ N(0,0.02), b=0) ->
    Sigmoid -> Linear(512->10), seed 0."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    w1 = (rng.standard_normal((512, 256)) * 0.02).astype(np.float32)
    w2 = (rng.standard_normal((10, 512)) * 0.02).astype(np.float32)
    return x, w1, np.zeros(512, np.float32), w2, np.zeros(10, np.float32)


def load_mlp(session, case):
    x, w1, b1, w2, b2 = case
    session.clear_params()
    session.set_param("mlp.l1.weight", w1)
    session.set_param("mlp.l1.bias", b1)
    session.set_param("mlp.l2.weight", w2)
    session.set_param("mlp.l2.bias", b2)
