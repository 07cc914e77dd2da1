// Model graphs of the benchmark configurations as eager interpreter programs:
//   LlamaModel  catgrad-llm-models/src/models/llama.rs:144-386
//   Qwen3Model  catgrad-llm-models/src/models/qwen3.rs:100-123,196-434 (dense path)
//   HiddenMlp   catgrad/examples/hidden.rs:103-132 with nn::linear + nn::Sigmoid
// plus the greedy generate loop and its timing protocol
// (catgrad-llm/examples/llama/main.rs:876-940,955-1037; catgrad-llm/src/utils/mod.rs:528-583).
#pragma once

#include <chrono>

#include "graph.hpp"
#include "nn.hpp"

namespace cgh {

struct LlmConfig { // the fields of LlamaConfig / Qwen3Config that the dense graphs read
    int arch = 0; // 0 llama, 1 qwen3
    size_t hidden_size = 0, num_hidden_layers = 0, num_attention_heads = 0, num_key_value_heads = 0;
    size_t head_dim = 0, intermediate_size = 0, vocab_size = 0;
    float rms_norm_eps = 1e-5f, rope_theta = 10000.0f;
    int tie_word_embeddings = 0;
};

struct ForwardOut {
    Tensor tokens, out_k, out_v;
};

class LlmModel {
  public:
    LlmModel(Interpreter &i, const LlmConfig &c) : i_(i), c_(c) {}
    const LlmConfig &config() const { return c_; }
    std::string root() const { return c_.arch == 0 ? "llama" : "qwen3"; }

    // `Interpreter::run(term, inputs)` for the model's term.  With Interpreter::schedule 0 the operations run as the
    // graph builder issues them; with 1 the pass is first recorded as a term and then evaluated in the layers of the
    // reference's evaluator, with its value map (graph.hpp); with 2 recorded and evaluated in the order of recording.
    ForwardOut forward(Tensor x, Tensor in_k, Tensor in_v, size_t max_positions, Tensor *logits = nullptr) {
        if (i_.schedule == 0 || i_.recorder) return def(std::move(x), std::move(in_k), std::move(in_v), max_positions, logits);
        Term term;
        Tensor sx = term.source(x.shape(), x.dtype()), sk = term.source(in_k.shape(), in_k.dtype()),
               sv = term.source(in_v.shape(), in_v.dtype());
        ForwardOut o;
        Tensor lg;
        i_.recorder = &term;
        try {
            o = def(std::move(sx), std::move(sk), std::move(sv), max_positions, logits ? &lg : nullptr);
        } catch (...) {
            i_.recorder = nullptr;
            throw;
        }
        i_.recorder = nullptr;
        std::vector<Tensor> outs;
        outs.push_back(std::move(o.tokens));
        outs.push_back(std::move(o.out_k));
        outs.push_back(std::move(o.out_v));
        if (logits) outs.push_back(std::move(lg));
        term.finish(std::move(outs));
        std::vector<Tensor> in;
        in.push_back(std::move(x));
        in.push_back(std::move(in_k));
        in.push_back(std::move(in_v));
        std::vector<Tensor> r = term.run(i_, std::move(in), i_.schedule == 2);
        if (logits) *logits = std::move(r[3]);
        return {std::move(r[0]), std::move(r[1]), std::move(r[2])};
    }

    // `DynModule::def` for inputs [x u32[B,S], in_k, in_v f32[L,B,kvH,P,hd], Nat(max_positions)]
    // `logits`, when given, receives a clone of the lm_head output (for parity checks).
    ForwardOut def(Tensor x, Tensor in_k, Tensor in_v, size_t max_positions, Tensor *logits = nullptr) {
        using namespace nn;
        I &i = i_;
        const std::string model = root() + ".model";
        // rope tables + per-layer cache views: Cache::init (helpers/cache.rs:86-103)
        auto tables = rope_tables_default(i, c_.rope_theta, max_positions, c_.head_dim, 1.0f);
        KVCache cache(i, c_.num_hidden_layers, in_k, in_v);
        size_t pos = shape(in_k)[3];
        in_k = Tensor();
        in_v = Tensor();
        x = embeddings(i, model + ".embed_tokens", std::move(x));
        size_t s = shape(x)[1];
        Tensor mask = causal_mask(i, s, pos);
        for (size_t l = 0; l < c_.num_hidden_layers; l++)
            x = layer(l, mask, cache, tables.first, tables.second, pos, model + ".layers." + std::to_string(l), std::move(x));
        mask = Tensor();
        x = rmsnorm(i, c_.rms_norm_eps, model + ".norm", std::move(x));
        const std::string lm_head = c_.tie_word_embeddings ? model + ".embed_tokens" : root() + ".lm_head";
        x = linear_no_bias(i, c_.hidden_size, c_.vocab_size, lm_head, std::move(x));
        if (logits) *logits = x;
        x = argmax(i, std::move(x));
        auto kv = cache.output(i);
        return {std::move(x), std::move(kv.first), std::move(kv.second)};
    }

  private:
    // llama.rs:349-386 / qwen3.rs:330-372
    Tensor layer(size_t l, const Tensor &mask, nn::KVCache &cache, const Tensor &cos_t, const Tensor &sin_t, size_t pos,
                 const std::string &p, Tensor x) {
        using namespace nn;
        I &i = i_;
        Tensor res = x;
        x = rmsnorm(i, c_.rms_norm_eps, p + ".input_layernorm", std::move(x));
        x = attention(l, mask, cache, cos_t, sin_t, pos, p + ".self_attn", std::move(x));
        x = add(i, std::move(res), std::move(x));
        res = x;
        x = rmsnorm(i, c_.rms_norm_eps, p + ".post_attention_layernorm", std::move(x));
        x = mlp(p + ".mlp", std::move(x));
        return add(i, std::move(x), std::move(res));
    }

    // llama.rs:230-253 / qwen3.rs:100-123
    Tensor mlp(const std::string &p, Tensor x) {
        using namespace nn;
        I &i = i_;
        Tensor gate = linear_no_bias(i, c_.hidden_size, c_.intermediate_size, p + ".gate_proj", x);
        Tensor up = linear_no_bias(i, c_.hidden_size, c_.intermediate_size, p + ".up_proj", std::move(x));
        x = mul(i, silu(i, std::move(gate)), std::move(up));
        return linear_no_bias(i, c_.intermediate_size, c_.hidden_size, p + ".down_proj", std::move(x));
    }

    // llama.rs:255-347 / qwen3.rs:196-328
    Tensor attention(size_t l, const Tensor &mask, nn::KVCache &cache, const Tensor &cos_t, const Tensor &sin_t,
                     size_t pos, const std::string &p, Tensor x) {
        using namespace nn;
        I &i = i_;
        const size_t dim = c_.hidden_size, nh = c_.num_attention_heads, nkv = c_.num_key_value_heads;
        const size_t hd = c_.head_dim, rep = nh / nkv;
        Shape xs = shape(x);
        const size_t b = xs[0], s = xs[1];
        Tensor q = linear_no_bias(i, dim, nh * hd, p + ".q_proj", x);
        Tensor k = linear_no_bias(i, dim, nkv * hd, p + ".k_proj", x);
        Tensor v = linear_no_bias(i, dim, nkv * hd, p + ".v_proj", std::move(x));
        q = reshape(i, Shape{b, s, nh, hd}, std::move(q));
        k = reshape(i, Shape{b, s, nkv, hd}, std::move(k));
        v = reshape(i, Shape{b, s, nkv, hd}, std::move(v));
        q = transpose(i, 1, 2, std::move(q));
        k = transpose(i, 1, 2, std::move(k));
        v = transpose(i, 1, 2, std::move(v));
        if (c_.arch == 1) { // Qwen3 QK-norm over head_dim (qwen3.rs:249-279)
            q = reshape(i, Shape{b * s * nh, hd}, std::move(q));
            k = reshape(i, Shape{b * s * nkv, hd}, std::move(k));
            q = rmsnorm(i, c_.rms_norm_eps, p + ".q_norm", std::move(q));
            k = rmsnorm(i, c_.rms_norm_eps, p + ".k_norm", std::move(k));
            q = reshape(i, Shape{b, nh, s, hd}, std::move(q));
            k = reshape(i, Shape{b, nkv, s, hd}, std::move(k));
        }
        q = apply_rope_embedding(i, pos, hd, cos_t, sin_t, std::move(q));
        k = apply_rope_embedding(i, pos, hd, cos_t, sin_t, std::move(k));
        auto kv = cache.update(i, l, std::move(k), std::move(v));
        k = repeat_kv(i, rep, std::move(kv.first));
        v = repeat_kv(i, rep, std::move(kv.second));
        Tensor tk = transpose(i, 2, 3, std::move(k));
        Tensor attn = matmul(i, std::move(q), std::move(tk));
        Shape sh = shape(attn);
        Tensor denom = constant(i, std::sqrt((float)hd), sh);
        denom = cast(i, std::move(denom), dtype(attn));
        attn = div(i, std::move(attn), std::move(denom));
        Tensor am = cast(i, mask, dtype(attn));
        am = broadcast(i, sh, std::move(am));
        attn = add(i, std::move(attn), std::move(am));
        attn = softmax(i, std::move(attn));
        attn = matmul(i, std::move(attn), std::move(v));
        attn = transpose(i, 1, 2, std::move(attn));
        attn = reshape(i, Shape{b, s, nh * hd}, std::move(attn));
        return linear_no_bias(i, nh * hd, dim, p + ".o_proj", std::move(attn));
    }

    Interpreter &i_;
    LlmConfig c_;
};

// hidden.rs:103-132 shaped MLP: Linear(in, hidden) -> nn::Sigmoid -> Linear(hidden, out).
inline Tensor hidden_mlp(Interpreter &i, size_t in_dim, size_t hidden, size_t out_dim, Tensor x) {
    x = nn::linear(i, in_dim, hidden, "mlp.l1", std::move(x));
    x = nn::sigmoid_module(i, std::move(x));
    return nn::linear(i, hidden, out_dim, "mlp.l2", std::move(x));
}

struct GenerateStats {
    double prefill_s = 0, decode_s = 0;
    uint64_t prefill_calls = 0, decode_calls = 0;
};

// Greedy generation with KV cache for a batch of B equal-length prompts.  One prefill
// run, then `steps` decode runs; each run ends with the only device-to-host read of
// the step, `to_vec` of the argmax tokens, of which the last position of every sequence
// is the next input (main.rs:1031-1037 generalised from batch 1 to B rows).
// out_tokens receives (steps + 1) x B ids: the token produced by the prefill, then one
// per decode run.  Prefill time includes the first read-back, as in main.rs:914-917.
// prefill_logits, when given, receives the lm_head output [B, S, vocab] of the prefill run (read back after the
// timed part of that run; for parity checks).
inline void generate(LlmModel &m, Interpreter &i, const uint32_t *prompt, size_t B, size_t S, size_t steps,
                     size_t max_positions, uint32_t *out_tokens, GenerateStats *st, std::vector<uint32_t> *prefill_logits = nullptr) {
    const LlmConfig &c = m.config();
    // empty_state_cache (utils/mod.rs:570-583) with the batch axis set to B
    Shape kv{c.num_hidden_layers, B, c.num_key_value_heads, 0, c.head_dim};
    Tensor state_k = i.backend.zeros(kv, CG_F32), state_v = i.backend.zeros(kv, CG_F32);
    std::vector<uint32_t> ids(prompt, prompt + B * S);
    size_t cur = S;
    auto t0 = std::chrono::steady_clock::now();
    uint64_t calls0 = i.backend.calls;
    for (size_t it = 0; it <= steps; it++) {
        Tensor x = i.backend.ndarray_from_vec_u32(ids.data(), ids.size(), Shape{B, cur});
        // the run's inputs are clones of the caller's state (main.rs:1007)
        Tensor logits;
        ForwardOut o = m.forward(std::move(x), state_k, state_v, max_positions, it == 0 && prefill_logits ? &logits : nullptr);
        std::vector<uint32_t> tok = i.backend.to_vec_bits(std::move(o.tokens));
        ids.resize(B);
        for (size_t b = 0; b < B; b++) {
            ids[b] = tok[b * cur + (cur - 1)];
            out_tokens[it * B + b] = ids[b];
        }
        state_k = std::move(o.out_k);
        state_v = std::move(o.out_v);
        cur = 1;
        if (it == 0) {
            auto t1 = std::chrono::steady_clock::now();
            st->prefill_s = std::chrono::duration<double>(t1 - t0).count();
            st->prefill_calls = i.backend.calls - calls0;
            if (prefill_logits) *prefill_logits = i.backend.to_vec_bits(std::move(logits));
            calls0 = i.backend.calls;
            t0 = std::chrono::steady_clock::now();
        }
    }
    st->decode_s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    st->decode_calls = i.backend.calls - calls0;
}

} // namespace cgh
