/* runner.h — C entry points of the host driver (libcatgrad_host.so): the C++ mirror of
 * catgrad's interpreter and model graphs, driving any library that exports the backend
 * C ABI (include/catgrad_hip.h).  Used by bench.py and the tests through ctypes. */
#ifndef CATGRAD_HOST_RUNNER_H
#define CATGRAD_HOST_RUNNER_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct cgm_session cgm_session; /* Interpreter<B> + Parameters + model config */

int cgm_open(const char *backend_library, int device, cgm_session **out);
void cgm_close(cgm_session *s);
const char *cgm_last_error(void);
const char *cgm_backend_name(cgm_session *s);

/* Parameters::insert(path, interpreter::tensor(backend, shape, data)) */
int cgm_set_param(cgm_session *s, const char *path, const float *data, const size_t *dims, size_t rank);
int cgm_clear_params(cgm_session *s);
/* Parameters from safetensors files (catgrad-llm/src/utils/mod.rs:321-449, dense tensors, f32 target):
 * F32 and BF16 tensors become f32 parameters named as in the file, I64 tensors are skipped.
 * stats4: [tensors loaded, parameters, bytes read, seconds]. */
int cgm_load_safetensors(cgm_session *s, const char *const *paths, size_t npaths, double *stats4);

/* arch: 0 = llama, 1 = qwen3 (dense). */
int cgm_set_config(cgm_session *s, int arch, size_t hidden_size, size_t num_hidden_layers, size_t num_attention_heads,
                   size_t num_key_value_heads, size_t head_dim, size_t intermediate_size, size_t vocab_size,
                   float rms_norm_eps, float rope_theta, int tie_word_embeddings);

/* Order of evaluation of the model runs and of cgm_cond_kat: 0 = the operations run as the graph builder issues
 * them; 1 = every run is first recorded as a term and evaluated in the layers of the reference's evaluator
 * (catgrad/src/abstract_interpreter/eval.rs:38-66, catgrad/src/ssa/mod.rs:24-76) with its move / clone value map;
 * 2 = recorded and evaluated in the order of recording. */
int cgm_set_schedule(cgm_session *s, int schedule);

/* The term of catgrad/tests/test_if.rs: cond(c, then: x + x, else: x, [x]) on rank-0 f32 tensors; *out receives
 * the result's value. */
int cgm_cond_kat(cgm_session *s, float x, float c, float *out);

/* A term whose If branches disagree in their result types (f32 against u32): under schedules 1 and 2 recording it
 * fails with a TypeError, as the reference's type checker would; returns nonzero then. */
int cgm_cond_mismatch(cgm_session *s);

/* One helper composition of catgrad-llm-models/src/helpers/tensors.rs on an f32 tensor x[dims], under the session's
 * schedule: which 0 = repeat_kv(rep = a0, x); 1 = repeat_interleave(dim = a0, rep = a1, x); 2 = cumsum(x) along the
 * last axis; 3 = probe(label, x) (catgrad/src/interpreter/tensor_op.rs:121-136: prints "[probe:label] ..." to stdout
 * when CATGRAD_PROBE is set) and hands x back.  out receives the result (at most out_cap elements), out_dims /
 * out_rank its shape (out_dims has room for 8 extents). */
int cgm_helper(cgm_session *s, int which, const float *x, const size_t *dims, size_t rank, size_t a0, size_t a1,
               const char *label, float *out, size_t out_cap, size_t *out_dims, size_t *out_rank);

/* Prefill + `steps` greedy decode runs.  out_tokens: (steps+1) x B ids.  stats:
 * [prefill_s, decode_s, backend calls in prefill, backend calls in decode]. */
int cgm_generate(cgm_session *s, const uint32_t *prompt, size_t B, size_t S, size_t steps, size_t max_positions,
                 uint32_t *out_tokens, double *stats4);
/* The same, also returning the prefill run's logits [B, S, vocab] (read back outside the timed parts). */
int cgm_generate_with_logits(cgm_session *s, const uint32_t *prompt, size_t B, size_t S, size_t steps, size_t max_positions,
                             uint32_t *out_tokens, double *stats4, float *prefill_logits);

/* One run on an empty cache.  out_tokens: B x S argmax ids.  out_logits (may be null):
 * B x S x vocab logits, read from the same run just before `argmax`. */
int cgm_forward(cgm_session *s, const uint32_t *tokens, size_t B, size_t S, size_t max_positions, uint32_t *out_tokens,
                float *out_logits);

/* As cgm_forward, but only the logits of `nrows` chosen positions are read back: rows[i] = b * S + s selects
 * sequence b, position s; out_logits: nrows x vocab.  (The [B, S, vocab] logits of a full-size run are gigabytes;
 * the rows are gathered on the device with `index` before `to_vec`.) */
int cgm_forward_rows(cgm_session *s, const uint32_t *tokens, size_t B, size_t S, size_t max_positions, uint32_t *out_tokens,
                     const uint32_t *rows, size_t nrows, float *out_logits);

/* Config-1 MLP: x f32[1, rows, in] -> Linear(in, hidden)+b -> Sigmoid -> Linear(hidden, out)+b.
 * Parameters: mlp.l1.weight [hidden,in], mlp.l1.bias [hidden], mlp.l2.weight [out,hidden], mlp.l2.bias [out]. */
int cgm_mlp(cgm_session *s, const float *x, size_t rows, size_t in_dim, size_t hidden, size_t out_dim, float *y);

/* Pass-through of the backend's launch-timing hooks (cg_profile_enable / cg_profile_read). */
int cgm_profile_enable(cgm_session *s, int kernel_class, unsigned sample_every);
int cgm_profile_read(cgm_session *s, int kernel_class, uint64_t *launches, double *milliseconds, double *work, int reset);

/* Waits for everything queued on the backend's stream (cg_sync). */
int cgm_sync(cgm_session *s);

/* Bytes the backend's device pool has handed out / holds cached. */
int cgm_pool_stats(cgm_session *s, size_t *in_use, size_t *cached);

/* Launches of fused programs since the last reset: compiled ahead of time / interpreted. */
int cgm_program_stats(cgm_session *s, uint64_t *compiled, uint64_t *interpreted, int reset);

#ifdef __cplusplus
}
#endif
#endif
