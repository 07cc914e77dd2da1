"""ctypes binding of the host driver (catgrad_amd/host/libcatgrad_host.so): the C++
mirror of catgrad's interpreter and model graphs that drives the backend library.

`Session()` drives the HIP backend — the product path; a missing HIP library is an
error.  Tests and the CPU-baseline leg of the benchmark pass another library that
exports the same C ABI (the CPU oracle) as `backend_library`."""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass

import numpy as np

from .backend import HIP_LIBRARY, load_hip_library

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIBRARY = os.path.join(_HERE, "host", "libcatgrad_host.so")

_lib = None


def _host():
    global _lib
    if _lib is None:
        if not os.path.exists(HOST_LIBRARY):
            raise RuntimeError(f"{HOST_LIBRARY} is missing: run `make -C {os.path.dirname(HOST_LIBRARY)}`")
        lib = C.CDLL(HOST_LIBRARY, mode=C.RTLD_LOCAL)
        P, SZ, SZP = C.c_void_p, C.c_size_t, C.POINTER(C.c_size_t)
        sig = {
            "cgm_open": (C.c_int, [C.c_char_p, C.c_int, C.POINTER(P)]),
            "cgm_close": (None, [P]),
            "cgm_last_error": (C.c_char_p, []),
            "cgm_backend_name": (C.c_char_p, [P]),
            "cgm_set_param": (C.c_int, [P, C.c_char_p, P, SZP, SZ]),
            "cgm_clear_params": (C.c_int, [P]),
            "cgm_load_safetensors": (C.c_int, [P, C.POINTER(C.c_char_p), SZ, C.POINTER(C.c_double)]),
            "cgm_set_config": (C.c_int, [P, C.c_int] + [SZ] * 7 + [C.c_float, C.c_float, C.c_int]),
            "cgm_set_schedule": (C.c_int, [P, C.c_int]),
            "cgm_cond_kat": (C.c_int, [P, C.c_float, C.c_float, C.POINTER(C.c_float)]),
            "cgm_cond_mismatch": (C.c_int, [P]),
            "cgm_helper": (C.c_int, [P, C.c_int, P, SZP, SZ, SZ, SZ, C.c_char_p, P, SZ, SZP, SZP]),
            "cgm_generate": (C.c_int, [P, P, SZ, SZ, SZ, SZ, P, C.POINTER(C.c_double)]),
            "cgm_generate_with_logits": (C.c_int, [P, P, SZ, SZ, SZ, SZ, P, C.POINTER(C.c_double), P]),
            "cgm_forward": (C.c_int, [P, P, SZ, SZ, SZ, P, P]),
            "cgm_forward_rows": (C.c_int, [P, P, SZ, SZ, SZ, P, P, SZ, P]),
            "cgm_mlp": (C.c_int, [P, P, SZ, SZ, SZ, SZ, P]),
            "cgm_pool_stats": (C.c_int, [P, SZP, SZP]),
            "cgm_sync": (C.c_int, [P]),
            "cgm_program_stats": (C.c_int, [P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.c_int]),
            "cgm_profile_enable": (C.c_int, [P, C.c_int, C.c_uint]),
            "cgm_profile_read": (C.c_int, [P, C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_double),
                                           C.POINTER(C.c_double), C.c_int]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


@dataclass(frozen=True)
class LlmConfig:
    """The config fields the dense Llama / Qwen3 graphs read
    (catgrad-llm-models/src/models/llama.rs:13-60, qwen3.rs:14-60)."""

    arch: str  # "llama" | "qwen3"
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    intermediate_size: int
    vocab_size: int
    head_dim: int = 0  # 0: hidden_size // num_attention_heads (Llama)
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False

    @property
    def hd(self) -> int:
        return self.head_dim or self.hidden_size // self.num_attention_heads

    def param_shapes(self):
        """Parameter paths in load order with their shapes (weights are stored [out, in])."""
        r, c = self.arch, self
        out = [(f"{r}.model.embed_tokens.weight", (c.vocab_size, c.hidden_size))]
        for l in range(c.num_hidden_layers):
            p = f"{r}.model.layers.{l}"
            out += [
                (f"{p}.input_layernorm.weight", (c.hidden_size,)),
                (f"{p}.self_attn.q_proj.weight", (c.num_attention_heads * c.hd, c.hidden_size)),
                (f"{p}.self_attn.k_proj.weight", (c.num_key_value_heads * c.hd, c.hidden_size)),
                (f"{p}.self_attn.v_proj.weight", (c.num_key_value_heads * c.hd, c.hidden_size)),
                (f"{p}.self_attn.o_proj.weight", (c.hidden_size, c.num_attention_heads * c.hd)),
            ]
            if c.arch == "qwen3":
                out += [(f"{p}.self_attn.q_norm.weight", (c.hd,)), (f"{p}.self_attn.k_norm.weight", (c.hd,))]
            out += [
                (f"{p}.post_attention_layernorm.weight", (c.hidden_size,)),
                (f"{p}.mlp.gate_proj.weight", (c.intermediate_size, c.hidden_size)),
                (f"{p}.mlp.up_proj.weight", (c.intermediate_size, c.hidden_size)),
                (f"{p}.mlp.down_proj.weight", (c.hidden_size, c.intermediate_size)),
            ]
        out.append((f"{r}.model.norm.weight", (c.hidden_size,)))
        if not c.tie_word_embeddings:
            out.append((f"{r}.lm_head.weight", (c.vocab_size, c.hidden_size)))
        return out

    def matmul_params(self) -> int:
        return sum(int(np.prod(s)) for n, s in self.param_shapes() if len(s) == 2 and "embed_tokens" not in n) + (
            self.vocab_size * self.hidden_size if self.tie_word_embeddings else 0)


def random_params(config: LlmConfig, seed: int = 0):
    """Random-init weights: matrices ~ N(0, 0.02), norm gains = 1; numpy default_rng(seed),
    drawn in `param_shapes()` order.  Yields (path, float32 array)."""
    rng = np.random.default_rng(seed)
    for name, shape in config.param_shapes():
        if len(shape) == 1:
            yield name, np.ones(shape, dtype=np.float32)
        else:
            w = rng.standard_normal(shape, dtype=np.float32)
            w *= np.float32(0.02)
            yield name, w


class Session:
    """`Interpreter<B>` + `Parameters<B>` + one model config, behind the host driver."""

    def __init__(self, backend_library: str | None = None, device: int = 0):
        if backend_library is None:
            load_hip_library()  # loud failure if the product library is not built
            backend_library = HIP_LIBRARY
        self._lib = _host()
        out = C.c_void_p()
        if self._lib.cgm_open(backend_library.encode(), device, C.byref(out)) != 0:
            raise RuntimeError(self._lib.cgm_last_error().decode())
        self._s = out.value

    def close(self):
        if self._s is not None:
            self._lib.cgm_close(self._s)
            self._s = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc):
        if rc != 0:
            raise RuntimeError(self._lib.cgm_last_error().decode())

    @property
    def backend_name(self) -> str:
        return self._lib.cgm_backend_name(self._s).decode()

    def set_param(self, path: str, arr: np.ndarray):
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        dims = (C.c_size_t * max(arr.ndim, 1))(*arr.shape)
        self._check(self._lib.cgm_set_param(self._s, path.encode(), arr.ctypes.data_as(C.c_void_p), dims, arr.ndim))

    def clear_params(self):
        self._check(self._lib.cgm_clear_params(self._s))

    def set_config(self, config: LlmConfig):
        self._check(self._lib.cgm_set_config(
            self._s, 0 if config.arch == "llama" else 1, config.hidden_size, config.num_hidden_layers,
            config.num_attention_heads, config.num_key_value_heads, config.hd, config.intermediate_size,
            config.vocab_size, config.rms_norm_eps, config.rope_theta, int(config.tie_word_embeddings)))
        self.config = config

    def load_safetensors(self, paths, config: LlmConfig = None):
        """Parameters from safetensors files (F32 and BF16 tensors become f32, I64 is skipped), as
        `load_model` of the reference does (catgrad-llm/src/utils/mod.rs:321-449).  Returns
        {tensors, params, bytes, seconds}."""
        if isinstance(paths, (str, os.PathLike)):
            paths = [paths]
        arr = (C.c_char_p * len(paths))(*[os.fspath(p).encode() for p in paths])
        st = (C.c_double * 4)()
        self.clear_params()
        self._check(self._lib.cgm_load_safetensors(self._s, arr, len(paths), st))
        if config is not None:
            self.set_config(config)
        return {"tensors": int(st[0]), "params": int(st[1]), "bytes": int(st[2]), "seconds": float(st[3])}

    def load_model(self, config: LlmConfig, params=None, seed: int = 0):
        self.clear_params()
        for name, w in (params if params is not None else random_params(config, seed)):
            self.set_param(name, w)
        self._check(self._lib.cgm_set_config(
            self._s, 0 if config.arch == "llama" else 1, config.hidden_size, config.num_hidden_layers,
            config.num_attention_heads, config.num_key_value_heads, config.hd, config.intermediate_size,
            config.vocab_size, config.rms_norm_eps, config.rope_theta, int(config.tie_word_embeddings)))
        self.config = config

    def set_schedule(self, schedule: int):
        """0: operations run as the graph builder issues them (default); 1: every model run is recorded as a term and
        evaluated in the layers of the reference's evaluator (eval.rs:38-66, ssa/mod.rs:24-76) with its move / clone
        value map; 2: recorded, evaluated in the order of recording."""
        self._check(self._lib.cgm_set_schedule(self._s, schedule))

    def cond_kat(self, x: float, c: float) -> float:
        """cond(c, then: x + x, else: x, [x]) on rank-0 tensors (catgrad/tests/test_if.rs)."""
        out = C.c_float()
        self._check(self._lib.cgm_cond_kat(self._s, x, c, C.byref(out)))
        return float(out.value)

    def cond_mismatch(self):
        """Records a term whose If branches disagree in their result types; raises under schedules 1 and 2."""
        self._check(self._lib.cgm_cond_mismatch(self._s))

    HELPERS = {"repeat_kv": 0, "repeat_interleave": 1, "cumsum": 2, "probe": 3}

    def helper(self, which: str, x: np.ndarray, a0: int = 0, a1: int = 0, label: str = "", out_cap: int | None = None) -> np.ndarray:
        """One helper composition of catgrad-llm-models/src/helpers/tensors.rs on an f32 tensor, through the
        interpreter mirror and the backend, under the session's schedule: repeat_kv(rep=a0), repeat_interleave(dim=a0,
        rep=a1), cumsum (last axis), probe(label) (prints when CATGRAD_PROBE is set; hands x back)."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        dims = (C.c_size_t * max(x.ndim, 1))(*x.shape)
        cap = out_cap or max(x.size * max(a0, a1, 1), 1)
        out = np.zeros(cap, dtype=np.float32)
        od, orank = (C.c_size_t * 8)(), C.c_size_t()
        self._check(self._lib.cgm_helper(self._s, self.HELPERS[which], x.ctypes.data_as(C.c_void_p), dims, x.ndim, a0, a1,
                                         label.encode(), out.ctypes.data_as(C.c_void_p), cap, od, C.byref(orank)))
        shape = tuple(od[i] for i in range(orank.value))
        return out[: int(np.prod(shape, dtype=np.int64))].reshape(shape)

    def generate(self, prompt: np.ndarray, steps: int, max_positions: int | None = None, want_logits: bool = False):
        """Prefill + `steps` greedy decode runs.  Returns (tokens [(steps+1), B], stats dict); with `want_logits`
        also the prefill run's logits [B, S, vocab] as a third value."""
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        B, S = prompt.shape
        max_positions = max_positions or (S + steps)
        out = np.zeros((steps + 1, B), dtype=np.uint32)
        stats = (C.c_double * 4)()
        logits = None
        if want_logits:
            logits = np.zeros((B, S, self.config.vocab_size), dtype=np.float32)
            self._check(self._lib.cgm_generate_with_logits(self._s, prompt.ctypes.data_as(C.c_void_p), B, S, steps,
                                                           max_positions, out.ctypes.data_as(C.c_void_p), stats,
                                                           logits.ctypes.data_as(C.c_void_p)))
        else:
            self._check(self._lib.cgm_generate(self._s, prompt.ctypes.data_as(C.c_void_p), B, S, steps, max_positions,
                                               out.ctypes.data_as(C.c_void_p), stats))
        st = {"prefill_s": stats[0], "decode_s": stats[1], "prefill_calls": int(stats[2]), "decode_calls": int(stats[3])}
        return (out, st, logits) if want_logits else (out, st)

    def forward(self, tokens: np.ndarray, max_positions: int | None = None, want_logits: bool = True):
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        B, S = tokens.shape
        out = np.zeros((B, S), dtype=np.uint32)
        logits = np.zeros((B, S, self.config.vocab_size), dtype=np.float32) if want_logits else None
        self._check(self._lib.cgm_forward(self._s, tokens.ctypes.data_as(C.c_void_p), B, S, max_positions or S,
                                          out.ctypes.data_as(C.c_void_p),
                                          logits.ctypes.data_as(C.c_void_p) if want_logits else None))
        return out, logits

    def forward_rows(self, tokens: np.ndarray, rows, max_positions: int | None = None):
        """One run on an empty cache; returns the argmax ids [B, S] and the logits [len(rows), vocab] of the chosen
        positions only (rows[i] = b * S + s), gathered on the device."""
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        rows = np.ascontiguousarray(rows, dtype=np.uint32)
        B, S = tokens.shape
        out = np.zeros((B, S), dtype=np.uint32)
        logits = np.zeros((rows.size, self.config.vocab_size), dtype=np.float32)
        self._check(self._lib.cgm_forward_rows(self._s, tokens.ctypes.data_as(C.c_void_p), B, S, max_positions or S,
                                               out.ctypes.data_as(C.c_void_p), rows.ctypes.data_as(C.c_void_p), rows.size,
                                               logits.ctypes.data_as(C.c_void_p)))
        return out, logits

    def mlp(self, x: np.ndarray, hidden: int, out_dim: int) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, in_dim = x.shape
        y = np.zeros((1, rows, out_dim), dtype=np.float32)
        self._check(self._lib.cgm_mlp(self._s, x.ctypes.data_as(C.c_void_p), rows, in_dim, hidden, out_dim,
                                      y.ctypes.data_as(C.c_void_p)))
        return y

    def profile_enable(self, cls: int, sample_every: int = 1):
        self._check(self._lib.cgm_profile_enable(self._s, cls, sample_every))

    def profile_read(self, cls: int, reset: bool = True):
        n, ms, w = C.c_uint64(), C.c_double(), C.c_double()
        self._check(self._lib.cgm_profile_read(self._s, cls, C.byref(n), C.byref(ms), C.byref(w), int(reset)))
        return int(n.value), float(ms.value), float(w.value)

    def sync(self):
        self._check(self._lib.cgm_sync(self._s))

    def program_stats(self, reset: bool = True):
        """(compiled, interpreted) launches of fused programs since the last reset."""
        c, i = C.c_uint64(), C.c_uint64()
        self._check(self._lib.cgm_program_stats(self._s, C.byref(c), C.byref(i), int(reset)))
        return int(c.value), int(i.value)

    def pool_stats(self):
        u, c = C.c_size_t(), C.c_size_t()
        self._check(self._lib.cgm_pool_stats(self._s, C.byref(u), C.byref(c)))
        return int(u.value), int(c.value)


# The benchmark configurations (BASELINE.json `configs`).
SMOLLM2_135M = LlmConfig("llama", 576, 30, 9, 3, 1536, 49152, rope_theta=10000.0, tie_word_embeddings=True)
QWEN3_0_6B = LlmConfig("qwen3", 1024, 28, 16, 8, 3072, 151936, head_dim=128, rms_norm_eps=1e-6, rope_theta=1000000.0,
                       tie_word_embeddings=True)
LLAMA_3_2_1B = LlmConfig("llama", 2048, 16, 32, 8, 8192, 128256, rope_theta=500000.0, tie_word_embeddings=True)
