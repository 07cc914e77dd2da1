// The stdlib / LLM-helper compositions that the model graphs are made of, restated as
// eager sequences of interpreter operations.  Each function issues exactly the backend
// calls, in the order and with the operand order, of the reference definition it cites;
// `x.clone()` in the reference is a `Tensor` copy here, the last use is a move.
#pragma once

#include <cmath>
#include <limits>

#include "graph.hpp"

namespace cgh {
namespace nn {
using namespace ops;

// catgrad/src/stdlib/nn/mod.rs:117-122
inline Tensor sqrt(I &i, Tensor x) {
    Shape sh = shape(x);
    Tensor e = constant(i, 0.5f, sh);
    e = cast(i, std::move(e), dtype(x));
    return pow(i, std::move(x), std::move(e));
}

// catgrad/src/stdlib/nn/mod.rs:124-130
inline Tensor sigmoid(I &i, Tensor x) {
    Shape sh = shape(x);
    Tensor one = constant(i, 1.0f, sh);
    one = cast(i, std::move(one), dtype(x));
    Tensor e = exp(i, neg(i, std::move(x)));
    Tensor d = add(i, one, std::move(e)); // one.clone() feeds the division below
    return div(i, std::move(one), std::move(d));
}

// catgrad/src/stdlib/nn/mod.rs:36-47 with 13-33: `nn::Sigmoid.call(builder, [x])` is a Definition operation at path
// nn.sigmoid whose body is `sigmoid` (interpreter.rs:61-74 evaluates the body as a term of its own).
inline Tensor sigmoid_module(I &i, Tensor x) {
    std::vector<Tensor> args;
    args.push_back(std::move(x));
    std::vector<Tensor> r = definition(
        i, "nn.sigmoid",
        [&](std::vector<Tensor> a) {
            std::vector<Tensor> out;
            out.push_back(sigmoid(i, std::move(a[0])));
            return out;
        },
        std::move(args));
    return std::move(r[0]);
}

// catgrad/src/stdlib/nn/mod.rs:143-148
inline Tensor silu(I &i, Tensor x) {
    cg_dtype dt = dtype(x);
    x = cast(i, std::move(x), CG_F32);
    Tensor s = sigmoid(i, x);
    x = mul(i, std::move(x), std::move(s));
    return cast(i, std::move(x), dt);
}

// catgrad/src/stdlib/nn/mod.rs:168-179
inline Tensor softmax(I &i, Tensor x) {
    cg_dtype dt = dtype(x);
    x = cast(i, std::move(x), CG_F32);
    Shape sh = shape(x);
    Tensor m = max(i, x);
    Tensor bmax = broadcast(i, sh, std::move(m));
    x = sub(i, std::move(x), std::move(bmax));
    Tensor ex = exp(i, std::move(x));
    Tensor s = sum(i, ex);
    Tensor bsum = broadcast(i, sh, std::move(s));
    return cast(i, div(i, std::move(ex), std::move(bsum)), dt);
}

// catgrad/src/stdlib/nn/mod.rs:182-204 — x must be rank 3 (`unpack::<3>`).
inline Tensor linear_b_param(I &i, size_t in_dim, size_t out_dim, Tensor weight, Tensor *bias, Tensor x) {
    Tensor w_t = transpose(i, 0, 1, std::move(weight));
    Shape sh = shape(x);
    if (sh.size() != 3) throw InterpreterError("linear: input must be rank 3");
    w_t = broadcast(i, Shape{sh[0], in_dim, out_dim}, std::move(w_t));
    Tensor m = matmul(i, std::move(x), std::move(w_t));
    if (bias) {
        Tensor bb = broadcast(i, shape(m), *bias);
        return add(i, std::move(m), std::move(bb));
    }
    return m;
}
// catgrad/src/stdlib/nn/mod.rs:244-267
inline Tensor linear_no_bias(I &i, size_t in_dim, size_t out_dim, const std::string &p, Tensor x) {
    return linear_b_param(i, in_dim, out_dim, i.param(p + ".weight"), nullptr, std::move(x));
}
inline Tensor linear(I &i, size_t in_dim, size_t out_dim, const std::string &p, Tensor x) {
    Tensor w = i.param(p + ".weight");
    Tensor b = i.param(p + ".bias");
    return linear_b_param(i, in_dim, out_dim, std::move(w), &b, std::move(x));
}

// catgrad-llm-models/src/helpers/tensors.rs:27-43
inline Tensor squeeze(I &i, size_t dim, Tensor x) {
    Shape s = shape(x);
    s.erase(s.begin() + dim);
    return reshape(i, s, std::move(x));
}
inline Tensor unsqueeze(I &i, size_t dim, Tensor x) {
    Shape s = shape(x);
    s.insert(s.begin() + dim, 1);
    return reshape(i, s, std::move(x));
}

// catgrad-llm-models/src/helpers/tensors.rs:82-101
inline Tensor rmsnorm_raw(I &i, float eps, Tensor x) {
    cg_dtype dt = dtype(x);
    Shape x_shape = shape(x);
    size_t n = x_shape.back();
    x = cast(i, std::move(x), CG_F32);
    Tensor s = sum(i, mul(i, x, x));
    Tensor constn = nat_to_u32(i, n);
    constn = cast(i, std::move(constn), CG_F32);
    Shape sh = shape(s);
    constn = broadcast(i, sh, std::move(constn));
    Tensor mean = div(i, std::move(s), std::move(constn));
    Tensor epsilon = constant(i, eps, shape(mean));
    epsilon = cast(i, std::move(epsilon), CG_F32);
    Tensor rms = sqrt(i, add(i, std::move(mean), std::move(epsilon)));
    Tensor denom = broadcast(i, x_shape, std::move(rms));
    return cast(i, div(i, std::move(x), std::move(denom)), dt);
}
// catgrad-llm-models/src/helpers/tensors.rs:104-111
inline Tensor rmsnorm(I &i, float eps, const std::string &p, Tensor x) {
    Tensor gamma = i.param(p + ".weight");
    Tensor lr = rmsnorm_raw(i, eps, std::move(x));
    gamma = broadcast(i, shape(lr), std::move(gamma));
    return mul(i, std::move(lr), std::move(gamma));
}

// catgrad-llm-models/src/helpers/tensors.rs:128-151
inline Tensor repeat_interleave(I &i, size_t dim, size_t rep, Tensor x) {
    x = unsqueeze(i, dim + 1, std::move(x));
    Shape sh = shape(x);
    sh[dim + 1] = rep;
    size_t orig = sh[dim];
    x = broadcast(i, sh, std::move(x));
    sh.erase(sh.begin() + dim + 1);
    sh[dim] = orig * rep;
    return reshape(i, sh, std::move(x));
}
inline Tensor repeat_kv(I &i, size_t rep, Tensor x) { return repeat_interleave(i, 1, rep, std::move(x)); }

// catgrad-llm-models/src/helpers/tensors.rs:305-334: 1.0 where col <= row + diagonal (lower) / col >= row + diagonal (upper)
inline Tensor tri_mask(I &i, size_t size, uint32_t diagonal, bool triu) {
    Shape sh{size, size};
    Tensor diag = broadcast(i, sh, lit(i, diagonal));
    Tensor idx = arange(i, size);
    Tensor row = reshape(i, Shape{size, 1}, idx);
    Tensor col = reshape(i, Shape{1, size}, std::move(idx));
    row = broadcast(i, sh, std::move(row));
    col = broadcast(i, sh, std::move(col));
    row = add(i, std::move(row), std::move(diag));
    Tensor mask = triu ? gte(i, std::move(col), std::move(row)) : lte(i, std::move(col), std::move(row));
    return cast(i, std::move(mask), CG_F32);
}
inline Tensor tril_mask(I &i, size_t size, uint32_t diagonal) { return tri_mask(i, size, diagonal, false); }

// catgrad-llm-models/src/helpers/tensors.rs:337-351: cumulative sum along the last axis as a product with the
// transposed lower-triangular mask
inline Tensor cumsum(I &i, Tensor x) {
    Shape sh = shape(x);
    const size_t ldim = sh.back();
    sh[sh.size() - 2] = ldim;
    Tensor lower = tril_mask(i, ldim, 0);
    lower = transpose(i, 0, 1, std::move(lower));
    lower = broadcast(i, sh, std::move(lower));
    return matmul(i, std::move(x), std::move(lower));
}

// catgrad-llm-models/src/helpers/tensors.rs:207-224
inline Tensor causal_mask(I &i, size_t seq_len, size_t pos) {
    size_t size = seq_len + pos;
    Tensor ci = arange(i, size);
    Shape sh{size, size};
    ci = broadcast(i, sh, std::move(ci));
    Tensor cj = arange(i, size);
    cj = reshape(i, Shape{size, 1}, std::move(cj));
    cj = broadcast(i, sh, std::move(cj));
    Tensor mask = lt(i, std::move(cj), std::move(ci));
    mask = cast(i, std::move(mask), CG_F32);
    Tensor ninf = constant(i, std::numeric_limits<float>::lowest(), sh); // f32::MIN
    mask = mul(i, std::move(mask), std::move(ninf));
    return slice(i, 0, pos, seq_len, std::move(mask));
}

// catgrad-llm-models/src/helpers/tensors.rs:255-272
inline Tensor embeddings(I &i, const std::string &p, Tensor x) {
    Tensor wte = i.param(p + ".weight");
    Shape xs = shape(x);
    x = reshape(i, Shape{xs[0] * xs[1]}, std::move(x));
    size_t hidden = shape(wte)[1];
    Tensor te = index(i, 0, std::move(x), std::move(wte));
    return reshape(i, Shape{xs[0], xs[1], hidden}, std::move(te));
}

// catgrad-llm-models/src/helpers/rope.rs:65-104
inline std::pair<Tensor, Tensor> rope_tables_default(I &i, float theta, size_t seq_len, size_t head_dim, float factor) {
    size_t half = head_dim / 2;
    Tensor f = arange(i, half);
    f = cast(i, std::move(f), CG_F32);
    Shape sh = shape(f);
    Tensor two = constant(i, 2.0f / (float)head_dim, sh);
    f = mul(i, std::move(f), std::move(two));
    Tensor th = constant(i, theta, sh);
    Tensor freq = pow(i, std::move(th), std::move(f));
    Tensor inv_freq = inverse(i, std::move(freq));
    Shape sh2{seq_len, half};
    inv_freq = broadcast(i, sh2, std::move(inv_freq));
    Tensor fac = constant(i, factor, sh2);
    inv_freq = div(i, std::move(inv_freq), std::move(fac));
    Tensor pos = arange(i, seq_len);
    pos = cast(i, std::move(pos), CG_F32);
    pos = reshape(i, Shape{seq_len, 1}, std::move(pos));
    pos = broadcast(i, shape(inv_freq), std::move(pos));
    pos = mul(i, std::move(pos), std::move(inv_freq));
    Tensor c = cos(i, pos);
    Tensor s = sin(i, std::move(pos));
    Tensor cc = concat(i, 1, c, c);
    Tensor ss = concat(i, 1, s, s);
    return {std::move(cc), std::move(ss)};
}

// catgrad-llm-models/src/helpers/rope.rs:423-427 with `chunk` (helpers/tensors.rs:5-13)
inline Tensor rotate_half(I &i, size_t head_dim, Tensor x) {
    size_t h = head_dim / 2;
    Tensor v0 = slice(i, 3, 0, h, x);
    Tensor v1 = slice(i, 3, h, h, std::move(x));
    return concat(i, 3, neg(i, std::move(v1)), std::move(v0));
}

// catgrad-llm-models/src/helpers/rope.rs:430-451
inline Tensor apply_rope_embedding(I &i, size_t pos, size_t head_dim, Tensor cos_t, Tensor sin_t, Tensor x) {
    Shape sh = shape(x);
    size_t seq_len = sh[2];
    cos_t = slice(i, 0, pos, seq_len, std::move(cos_t));
    sin_t = slice(i, 0, pos, seq_len, std::move(sin_t));
    cos_t = broadcast(i, sh, std::move(cos_t));
    sin_t = broadcast(i, sh, std::move(sin_t));
    cg_dtype dt = dtype(x);
    x = cast(i, std::move(x), CG_F32);
    Tensor rotated = rotate_half(i, head_dim, x);
    Tensor a = mul(i, std::move(cos_t), std::move(x));
    Tensor b = mul(i, std::move(sin_t), std::move(rotated));
    return cast(i, add(i, std::move(a), std::move(b)), dt);
}

// catgrad-llm-models/src/helpers/cache.rs:7-75
struct KVCache {
    std::vector<std::pair<Tensor, Tensor>> out_kv_cache;

    KVCache(I &i, size_t num_layers, const Tensor &in_k, const Tensor &in_v) {
        for (size_t l = 0; l < num_layers; l++) {
            Tensor k = slice(i, 0, l, 1, in_k);
            Tensor v = slice(i, 0, l, 1, in_v);
            k = squeeze(i, 0, std::move(k));
            v = squeeze(i, 0, std::move(v));
            out_kv_cache.emplace_back(std::move(k), std::move(v));
        }
    }
    std::pair<Tensor, Tensor> update(I &i, size_t layer, Tensor k, Tensor v) {
        Tensor ck = out_kv_cache[layer].first, cv = out_kv_cache[layer].second;
        out_kv_cache[layer] = {Tensor(), Tensor()}; // the graph holds no other use of the old entries
        k = concat(i, 2, std::move(ck), std::move(k));
        v = concat(i, 2, std::move(cv), std::move(v));
        out_kv_cache[layer] = {k, v};
        return {std::move(k), std::move(v)};
    }
    std::pair<Tensor, Tensor> output(I &i) {
        Tensor out_k = unsqueeze(i, 0, std::move(out_kv_cache[0].first));
        Tensor out_v = unsqueeze(i, 0, std::move(out_kv_cache[0].second));
        for (size_t l = 1; l < out_kv_cache.size(); l++) {
            Tensor k = unsqueeze(i, 0, std::move(out_kv_cache[l].first));
            Tensor v = unsqueeze(i, 0, std::move(out_kv_cache[l].second));
            out_k = concat(i, 0, std::move(out_k), std::move(k));
            out_v = concat(i, 0, std::move(out_v), std::move(v));
        }
        return {std::move(out_k), std::move(out_v)};
    }
};

} // namespace nn
} // namespace cgh
