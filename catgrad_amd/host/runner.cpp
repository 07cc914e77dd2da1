// C entry points of the host driver; see runner.h.
#include "runner.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>

#include "models.hpp"
#include "weights.hpp"

using namespace cgh;

struct cgm_session {
    std::unique_ptr<Interpreter> interp;
    LlmConfig config;
    std::string name;
};

static thread_local std::string g_err;

template <class F> static int guarded(F &&f) {
    try {
        f();
        return 0;
    } catch (const std::exception &e) {
        g_err = e.what();
        return 1;
    }
}

// Runs `body` over `inputs` under the session's schedule: directly (0), or recorded as a term first and evaluated in
// the reference evaluator's layers (1) or in the order of recording (2).
template <class F> static std::vector<Tensor> run_scheduled(Interpreter &i, std::vector<Tensor> inputs, F &&body) {
    if (i.schedule == 0) return body(std::move(inputs));
    Term term;
    std::vector<Tensor> src;
    for (Tensor &t : inputs) src.push_back(term.source(t.shape(), t.dtype()));
    i.recorder = &term;
    std::vector<Tensor> r;
    try {
        r = body(std::move(src));
    } catch (...) {
        i.recorder = nullptr;
        throw;
    }
    i.recorder = nullptr;
    term.finish(std::move(r));
    return term.run(i, std::move(inputs), i.schedule == 2);
}

extern "C" {

const char *cgm_last_error(void) { return g_err.c_str(); }

int cgm_open(const char *backend_library, int device, cgm_session **out) {
    return guarded([&] {
        auto s = std::make_unique<cgm_session>();
        s->interp = std::make_unique<Interpreter>(backend_library, device);
        s->name = s->interp->backend.name();
        *out = s.release();
    });
}

void cgm_close(cgm_session *s) {
    if (!s) return;
    s->interp->parameters.clear();
    delete s;
}

const char *cgm_backend_name(cgm_session *s) { return s->name.c_str(); }

int cgm_set_param(cgm_session *s, const char *path, const float *data, const size_t *dims, size_t rank) {
    return guarded([&] {
        Shape shape(dims, dims + rank);
        size_t n = 1;
        for (size_t d : shape) n *= d;
        s->interp->parameters[path] = s->interp->backend.ndarray_from_vec_f32(data, n, shape);
    });
}

int cgm_load_safetensors(cgm_session *s, const char *const *paths, size_t npaths, double *stats4) {
    return guarded([&] {
        std::vector<std::string> files(paths, paths + npaths);
        LoadStats st = load_safetensors(*s->interp, files);
        stats4[0] = (double)st.tensors;
        stats4[1] = (double)st.params;
        stats4[2] = (double)st.bytes;
        stats4[3] = st.seconds;
    });
}

int cgm_clear_params(cgm_session *s) {
    return guarded([&] { s->interp->parameters.clear(); });
}

int cgm_set_config(cgm_session *s, int arch, size_t hidden_size, size_t num_hidden_layers, size_t num_attention_heads,
                   size_t num_key_value_heads, size_t head_dim, size_t intermediate_size, size_t vocab_size,
                   float rms_norm_eps, float rope_theta, int tie_word_embeddings) {
    return guarded([&] {
        LlmConfig &c = s->config;
        c.arch = arch;
        c.hidden_size = hidden_size;
        c.num_hidden_layers = num_hidden_layers;
        c.num_attention_heads = num_attention_heads;
        c.num_key_value_heads = num_key_value_heads;
        c.head_dim = head_dim;
        c.intermediate_size = intermediate_size;
        c.vocab_size = vocab_size;
        c.rms_norm_eps = rms_norm_eps;
        c.rope_theta = rope_theta;
        c.tie_word_embeddings = tie_word_embeddings;
    });
}

int cgm_set_schedule(cgm_session *s, int schedule) {
    return guarded([&] {
        if (schedule < 0 || schedule > 2) throw InterpreterError("unknown schedule");
        s->interp->schedule = schedule;
    });
}

int cgm_cond_kat(cgm_session *s, float x, float c, float *out) {
    return guarded([&] {
        Interpreter &i = *s->interp;
        std::vector<Tensor> in;
        in.push_back(i.backend.ndarray_from_vec_f32(&x, 1, Shape{}));
        in.push_back(i.backend.ndarray_from_vec_f32(&c, 1, Shape{}));
        std::vector<Tensor> res = run_scheduled(i, std::move(in), [&](std::vector<Tensor> a) {
            Tensor keep = a[0]; // `x.clone()`: the term also returns x itself in the reference's test
            (void)keep;
            return ops::cond(
                i, std::move(a[1]),
                [&](std::vector<Tensor> b) { return std::vector<Tensor>{ops::add(i, b[0], b[0])}; },
                [&](std::vector<Tensor> b) { return std::vector<Tensor>{std::move(b[0])}; },
                std::vector<Tensor>{std::move(a[0])});
        });
        std::vector<uint32_t> v = i.backend.to_vec_bits(std::move(res[0]));
        memcpy(out, v.data(), 4);
    });
}

int cgm_cond_mismatch(cgm_session *s) {
    return guarded([&] {
        Interpreter &i = *s->interp;
        const float one = 1.0f;
        std::vector<Tensor> in;
        in.push_back(i.backend.ndarray_from_vec_f32(&one, 1, Shape{}));
        in.push_back(i.backend.ndarray_from_vec_f32(&one, 1, Shape{}));
        run_scheduled(i, std::move(in), [&](std::vector<Tensor> a) {
            return ops::cond(
                i, std::move(a[1]),
                [&](std::vector<Tensor> b) { return std::vector<Tensor>{ops::cast(i, std::move(b[0]), CG_U32)}; },
                [&](std::vector<Tensor> b) { return std::vector<Tensor>{std::move(b[0])}; },
                std::vector<Tensor>{std::move(a[0])});
        });
    });
}

int cgm_helper(cgm_session *s, int which, const float *x, const size_t *dims, size_t rank, size_t a0, size_t a1,
               const char *label, float *out, size_t out_cap, size_t *out_dims, size_t *out_rank) {
    return guarded([&] {
        Interpreter &i = *s->interp;
        Shape shape(dims, dims + rank);
        size_t n = 1;
        for (size_t d : shape) n *= d;
        std::vector<Tensor> in;
        in.push_back(i.backend.ndarray_from_vec_f32(x, n, shape));
        std::vector<Tensor> res = run_scheduled(i, std::move(in), [&](std::vector<Tensor> a) {
            std::vector<Tensor> r;
            switch (which) {
            case 0: r.push_back(nn::repeat_kv(i, a0, std::move(a[0]))); break;
            case 1: r.push_back(nn::repeat_interleave(i, a0, a1, std::move(a[0]))); break;
            case 2: r.push_back(nn::cumsum(i, std::move(a[0]))); break;
            case 3:
                ops::probe(i, label ? label : "", a[0]);
                r.push_back(std::move(a[0]));
                break;
            default: throw InterpreterError("unknown helper");
            }
            return r;
        });
        Shape rs = res[0].shape();
        *out_rank = rs.size();
        for (size_t d = 0; d < rs.size(); d++) out_dims[d] = rs[d];
        std::vector<uint32_t> v = i.backend.to_vec_bits(std::move(res[0]));
        if (v.size() > out_cap) throw InterpreterError("helper result larger than the caller's buffer");
        memcpy(out, v.data(), v.size() * 4);
    });
}

int cgm_generate(cgm_session *s, const uint32_t *prompt, size_t B, size_t S, size_t steps, size_t max_positions,
                 uint32_t *out_tokens, double *stats4) {
    return guarded([&] {
        LlmModel m(*s->interp, s->config);
        GenerateStats st;
        const char *tc = getenv("CGH_TIME_CALLS");
        s->interp->backend.time_calls = tc && tc[0] == '1';
        s->interp->backend.seconds_in_backend = 0;
        generate(m, *s->interp, prompt, B, S, steps, max_positions, out_tokens, &st);
        if (s->interp->backend.time_calls)
            fprintf(stderr, "[host] generate: %.3f ms inside backend calls (those that return tensors), %.3f ms total\n",
                    s->interp->backend.seconds_in_backend * 1e3, (st.prefill_s + st.decode_s) * 1e3);
        stats4[0] = st.prefill_s;
        stats4[1] = st.decode_s;
        stats4[2] = (double)st.prefill_calls;
        stats4[3] = (double)st.decode_calls;
    });
}

int cgm_generate_with_logits(cgm_session *s, const uint32_t *prompt, size_t B, size_t S, size_t steps, size_t max_positions,
                             uint32_t *out_tokens, double *stats4, float *prefill_logits) {
    return guarded([&] {
        LlmModel m(*s->interp, s->config);
        GenerateStats st;
        std::vector<uint32_t> lg;
        generate(m, *s->interp, prompt, B, S, steps, max_positions, out_tokens, &st, &lg);
        memcpy(prefill_logits, lg.data(), lg.size() * 4);
        stats4[0] = st.prefill_s;
        stats4[1] = st.decode_s;
        stats4[2] = (double)st.prefill_calls;
        stats4[3] = (double)st.decode_calls;
    });
}

int cgm_forward(cgm_session *s, const uint32_t *tokens, size_t B, size_t S, size_t max_positions, uint32_t *out_tokens,
                float *out_logits) {
    return guarded([&] {
        Interpreter &i = *s->interp;
        LlmModel m(i, s->config);
        const LlmConfig &c = s->config;
        Shape kv{c.num_hidden_layers, B, c.num_key_value_heads, 0, c.head_dim};
        Tensor x = i.backend.ndarray_from_vec_u32(tokens, B * S, Shape{B, S});
        Tensor logits;
        ForwardOut o = m.forward(std::move(x), i.backend.zeros(kv, CG_F32), i.backend.zeros(kv, CG_F32), max_positions,
                                 out_logits ? &logits : nullptr);
        std::vector<uint32_t> tok = i.backend.to_vec_bits(std::move(o.tokens));
        memcpy(out_tokens, tok.data(), tok.size() * 4);
        if (out_logits) {
            std::vector<uint32_t> lg = i.backend.to_vec_bits(std::move(logits));
            memcpy(out_logits, lg.data(), lg.size() * 4);
        }
    });
}

int cgm_forward_rows(cgm_session *s, const uint32_t *tokens, size_t B, size_t S, size_t max_positions, uint32_t *out_tokens,
                     const uint32_t *rows, size_t nrows, float *out_logits) {
    return guarded([&] {
        Interpreter &i = *s->interp;
        LlmModel m(i, s->config);
        const LlmConfig &c = s->config;
        Shape kv{c.num_hidden_layers, B, c.num_key_value_heads, 0, c.head_dim};
        Tensor x = i.backend.ndarray_from_vec_u32(tokens, B * S, Shape{B, S});
        Tensor logits;
        ForwardOut o = m.forward(std::move(x), i.backend.zeros(kv, CG_F32), i.backend.zeros(kv, CG_F32), max_positions, &logits);
        std::vector<uint32_t> tok = i.backend.to_vec_bits(std::move(o.tokens));
        memcpy(out_tokens, tok.data(), tok.size() * 4);
        Tensor flat = i.backend.reshape(std::move(logits), Shape{B * S, c.vocab_size});
        Tensor idx = i.backend.ndarray_from_vec_u32(rows, nrows, Shape{nrows});
        Tensor picked = i.backend.index(std::move(flat), 0, std::move(idx));
        std::vector<uint32_t> lg = i.backend.to_vec_bits(std::move(picked));
        memcpy(out_logits, lg.data(), lg.size() * 4);
    });
}

int cgm_mlp(cgm_session *s, const float *x, size_t rows, size_t in_dim, size_t hidden, size_t out_dim, float *y) {
    return guarded([&] {
        Interpreter &i = *s->interp;
        std::vector<Tensor> in;
        in.push_back(i.backend.ndarray_from_vec_f32(x, rows * in_dim, Shape{1, rows, in_dim}));
        std::vector<Tensor> r = run_scheduled(i, std::move(in), [&](std::vector<Tensor> a) {
            std::vector<Tensor> o;
            o.push_back(hidden_mlp(i, in_dim, hidden, out_dim, std::move(a[0])));
            return o;
        });
        std::vector<uint32_t> v = i.backend.to_vec_bits(std::move(r[0]));
        memcpy(y, v.data(), v.size() * 4);
    });
}

int cgm_profile_enable(cgm_session *s, int kernel_class, unsigned sample_every) {
    return guarded([&] { s->interp->backend.profile_enable(kernel_class, sample_every); });
}

int cgm_profile_read(cgm_session *s, int kernel_class, uint64_t *launches, double *milliseconds, double *work, int reset) {
    return guarded([&] { s->interp->backend.profile_read(kernel_class, launches, milliseconds, work, reset); });
}

int cgm_sync(cgm_session *s) {
    return guarded([&] { s->interp->backend.sync(); });
}

int cgm_pool_stats(cgm_session *s, size_t *in_use, size_t *cached) {
    return guarded([&] { s->interp->backend.pool_stats(in_use, cached); });
}

int cgm_program_stats(cgm_session *s, uint64_t *compiled, uint64_t *interpreted, int reset) {
    return guarded([&] { s->interp->backend.program_stats(compiled, interpreted, reset); });
}

} // extern "C"
