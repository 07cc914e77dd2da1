"""Independent float64 numpy statements of the model mathematics (textbook formulas,
not a transcription of the op trace): RMSNorm, RoPE (rotate-half), grouped-query causal
attention, SwiGLU, greedy decoding by full recomputation.  They pin the host driver +
oracle end to end."""
import numpy as np


def rmsnorm(x, g, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * g


def rope(x, theta, positions):
    # x: [B, h, S, hd]; rotate-half convention
    hd = x.shape[-1]
    inv = 1.0 / (theta ** (np.arange(hd // 2, dtype=np.float64) * 2.0 / hd))
    ang = positions[:, None].astype(np.float64) * inv[None, :]
    cos, sin = np.cos(ang), np.sin(ang)
    cos, sin = np.concatenate([cos, cos], -1), np.concatenate([sin, sin], -1)
    x1, x2 = x[..., : hd // 2], x[..., hd // 2:]
    rot = np.concatenate([-x2, x1], -1)
    return x * cos + rot * sin


class _Wide:
    """Parameters widened to float64 one at a time, on use (the full-size models do not fit twice)."""

    def __init__(self, params):
        self.p = params

    def __getitem__(self, k):
        return self.p[k].astype(np.float64)


def llm_logits(cfg, params, tokens, positions=None):
    """Logits [B, S, V] for token ids [B, S] (no cache: full causal recomputation); with `positions`
    (indices along S) only those rows go through the vocabulary projection: [B, len(positions), V]."""
    P = _Wide(params)
    r = cfg.arch
    B, S = tokens.shape
    h, kv, hd = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.hd
    x = P[f"{r}.model.embed_tokens.weight"][tokens]
    pos = np.arange(S)
    causal = np.triu(np.ones((S, S), dtype=bool), 1)
    for l in range(cfg.num_hidden_layers):
        p = f"{r}.model.layers.{l}"
        hn = rmsnorm(x, P[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps)
        q = (hn @ P[f"{p}.self_attn.q_proj.weight"].T).reshape(B, S, h, hd).transpose(0, 2, 1, 3)
        k = (hn @ P[f"{p}.self_attn.k_proj.weight"].T).reshape(B, S, kv, hd).transpose(0, 2, 1, 3)
        v = (hn @ P[f"{p}.self_attn.v_proj.weight"].T).reshape(B, S, kv, hd).transpose(0, 2, 1, 3)
        if r == "qwen3":
            q = rmsnorm(q, P[f"{p}.self_attn.q_norm.weight"], cfg.rms_norm_eps)
            k = rmsnorm(k, P[f"{p}.self_attn.k_norm.weight"], cfg.rms_norm_eps)
        q, k = rope(q, cfg.rope_theta, pos), rope(k, cfg.rope_theta, pos)
        k, v = np.repeat(k, h // kv, axis=1), np.repeat(v, h // kv, axis=1)
        sc = q @ k.transpose(0, 1, 3, 2) / np.sqrt(hd)
        sc = np.where(causal, -np.inf, sc)
        sc = np.exp(sc - sc.max(-1, keepdims=True))
        att = (sc / sc.sum(-1, keepdims=True)) @ v
        att = att.transpose(0, 2, 1, 3).reshape(B, S, h * hd)
        x = x + att @ P[f"{p}.self_attn.o_proj.weight"].T
        hn = rmsnorm(x, P[f"{p}.post_attention_layernorm.weight"], cfg.rms_norm_eps)
        g = hn @ P[f"{p}.mlp.gate_proj.weight"].T
        u = hn @ P[f"{p}.mlp.up_proj.weight"].T
        x = x + ((g / (1.0 + np.exp(-g))) * u) @ P[f"{p}.mlp.down_proj.weight"].T
    if positions is not None:
        x = x[:, list(positions), :]
    x = rmsnorm(x, P[f"{r}.model.norm.weight"], cfg.rms_norm_eps)
    head = f"{r}.model.embed_tokens.weight" if cfg.tie_word_embeddings else f"{r}.lm_head.weight"
    return x @ P[head].T


def greedy(cfg, params, prompt, steps):
    """Tokens [(steps+1), B] and the top1-top2 logit gap of every choice."""
    toks = prompt.copy()
    out, gaps = [], []
    for _ in range(steps + 1):
        lg = llm_logits(cfg, params, toks)[:, -1, :]
        nxt = lg.argmax(-1).astype(np.uint32)
        srt = np.sort(lg, -1)
        gaps.append(srt[:, -1] - srt[:, -2])
        out.append(nxt)
        toks = np.concatenate([toks, nxt[:, None]], 1)
    return np.stack(out), np.stack(gaps)


def mlp(x, w1, b1, w2, b2):
    h = x.astype(np.float64) @ w1.astype(np.float64).T + b1
    h = 1.0 / (1.0 + np.exp(-h))
    return h @ w2.astype(np.float64).T + b2
