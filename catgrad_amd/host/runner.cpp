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
        auto body = [&](Tensor tx, Tensor tc) {
            Tensor keep = tx; // `x.clone()`: the term also returns x itself in the reference's test
            (void)keep;
            return ops::cond(
                i, std::move(tc),
                [&](std::vector<Tensor> a) { return std::vector<Tensor>{ops::add(i, a[0], a[0])}; },
                [&](std::vector<Tensor> a) { return std::vector<Tensor>{std::move(a[0])}; },
                std::vector<Tensor>{std::move(tx)});
        };
        Tensor tx = i.backend.ndarray_from_vec_f32(&x, 1, Shape{}), tc = i.backend.ndarray_from_vec_f32(&c, 1, Shape{});
        Tensor res;
        if (i.schedule == 0) {
            res = std::move(body(std::move(tx), std::move(tc))[0]);
        } else {
            Term term;
            Tensor sx = term.source(Shape{}, CG_F32), sc = term.source(Shape{}, CG_F32);
            i.recorder = &term;
            std::vector<Tensor> r;
            try {
                r = body(std::move(sx), std::move(sc));
            } catch (...) {
                i.recorder = nullptr;
                throw;
            }
            i.recorder = nullptr;
            term.finish(std::move(r));
            std::vector<Tensor> in;
            in.push_back(std::move(tx));
            in.push_back(std::move(tc));
            res = std::move(term.run(i, std::move(in), i.schedule == 2)[0]);
        }
        std::vector<uint32_t> v = i.backend.to_vec_bits(std::move(res));
        memcpy(out, v.data(), 4);
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
        Tensor t = i.backend.ndarray_from_vec_f32(x, rows * in_dim, Shape{1, rows, in_dim});
        Tensor r = hidden_mlp(i, in_dim, hidden, out_dim, std::move(t));
        std::vector<uint32_t> v = i.backend.to_vec_bits(std::move(r));
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
