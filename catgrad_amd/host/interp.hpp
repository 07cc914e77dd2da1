// C++ mirror of the tensor interpreter that drives a `Backend`:
//   * `Value`, `TensorOp`, `tensor_op()` follow catgrad/src/interpreter/tensor_op.rs —
//     same argument order per op, same arity / dtype checks, scalars and `NatToU32`
//     become rank-0 tensors through `ndarray_from_vec_*` (tensor_op.rs:64-87).
//   * `Interpreter` owns the backend and the `Parameters` map; `param()` is the `Load`
//     operation, which clones the stored tensor (interpreter/interpreter.rs:56-59).
//   * namespace `ops` gives the DSL spellings of catgrad/src/category/lang/ops.rs and
//     catgrad/src/stdlib/ops.rs; every call goes through `tensor_op()`.
// Values are moved into operations and cloned on fan-out, which is the evaluator's
// lifetime model (catgrad/src/abstract_interpreter/eval.rs:44-49,107-116).  Shape, Nat
// and Dtype computations run on the host and issue no backend call (eval.rs:122-187).
#pragma once

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <string>
#include <vector>

#include "backend.hpp"

namespace cgh {

struct Value {
    enum Kind { TENSOR, NAT, SHAPE, DTYPE } kind = NAT;
    Tensor tensor;
    size_t nat = 0;
    Shape shape;
    cg_dtype dtype = CG_F32;

    Value() = default;
    Value(Tensor t) : kind(TENSOR), tensor(std::move(t)) {}
    Value(size_t n) : kind(NAT), nat(n) {}
    Value(int n) : kind(NAT), nat((size_t)n) {}
    Value(Shape s) : kind(SHAPE), shape(std::move(s)) {}
    Value(cg_dtype d) : kind(DTYPE), dtype(d) {}
};

struct InterpreterError : std::runtime_error { // abstract_interpreter/types.rs:104-123
    using std::runtime_error::runtime_error;
};

// `core::TensorOp` (catgrad/src/category/core.rs:170-239) with `Map(ScalarOp)` flattened.
enum class TensorOp {
    Add, Sub, Mul, Div, Neg, Pow, LT, GT, GTE, LTE, EQ, Cos, Sin, Exp, Log, Floor, Round, Where,
    NatToU32, Cast, MatMul, ScalarF32, ScalarU32, Sum, Max, Argmax, TopK, Broadcast, Reshape, Transpose,
    Slice, Concat, Arange, Index, Probe
};

struct Op {
    TensorOp op;
    float f32 = 0.0f;   // payload of ScalarF32
    uint32_t u32 = 0;   // payload of ScalarU32
    std::string label;  // payload of Probe
    Op(TensorOp o) : op(o) {}
    static Op scalar(float v) { Op o(TensorOp::ScalarF32); o.f32 = v; return o; }
    static Op scalar(uint32_t v) { Op o(TensorOp::ScalarU32); o.u32 = v; return o; }
    static Op probe(std::string l) { Op o(TensorOp::Probe); o.label = std::move(l); return o; }
};

// Builds an argument / result list by MOVING its items (a braced list would copy,
// i.e. clone, every tensor and hide uniquely owned operands from the backend).
template <class... A> std::vector<Value> vals(A &&...a) {
    std::vector<Value> v;
    v.reserve(sizeof...(a));
    (v.emplace_back(std::forward<A>(a)), ...);
    return v;
}

namespace detail {
inline void arity(const std::vector<Value> &a, size_t n) { // get_exact_arity
    if (a.size() != n) throw InterpreterError("ApplyError: wrong number of arguments");
}
inline Tensor to_tensor(Value &v) {
    if (v.kind != Value::TENSOR) throw InterpreterError("TypeError: expected a tensor");
    return std::move(v.tensor);
}
inline size_t to_nat(const Value &v) {
    if (v.kind != Value::NAT) throw InterpreterError("TypeError: expected a nat");
    return v.nat;
}
inline const Shape &to_shape(const Value &v) {
    if (v.kind != Value::SHAPE) throw InterpreterError("TypeError: expected a shape");
    return v.shape;
}
inline cg_dtype to_dtype(const Value &v) {
    if (v.kind != Value::DTYPE) throw InterpreterError("TypeError: expected a dtype");
    return v.dtype;
}
// try_into_tagged_ndarrays (tensor_op.rs:231-275): all operands must share a dtype.
inline void same_dtype(const std::vector<Value> &a) {
    for (const Value &v : a) {
        if (v.kind != Value::TENSOR) throw InterpreterError("TypeError: expected a tensor");
        if (v.tensor.dtype() != a[0].tensor.dtype()) throw InterpreterError("TypeError: mixed dtypes");
    }
}
} // namespace detail

// interpreter/tensor_op.rs:9-51
inline std::vector<Value> tensor_op(Backend &b, const Op &op, std::vector<Value> args) {
    using namespace detail;
    auto binop = [&](Tensor (Backend::*f)(Tensor, Tensor)) -> std::vector<Value> {
        arity(args, 2);
        same_dtype(args);
        return vals(Value((b.*f)(to_tensor(args[0]), to_tensor(args[1]))));
    };
    auto unop = [&](Tensor (Backend::*f)(Tensor)) -> std::vector<Value> {
        arity(args, 1);
        return vals(Value((b.*f)(to_tensor(args[0]))));
    };
    switch (op.op) {
    case TensorOp::Add: return binop(&Backend::add);
    case TensorOp::Sub: return binop(&Backend::sub);
    case TensorOp::Pow: return binop(&Backend::pow);
    case TensorOp::Sin: return unop(&Backend::sin);
    case TensorOp::Cos: return unop(&Backend::cos);
    case TensorOp::Exp: return unop(&Backend::exp);
    case TensorOp::Log: return unop(&Backend::log);
    case TensorOp::Floor: return unop(&Backend::floor);
    case TensorOp::Round: return unop(&Backend::round);
    case TensorOp::Neg: return unop(&Backend::neg);
    case TensorOp::Mul: return binop(&Backend::mul);
    case TensorOp::Div: return binop(&Backend::div);
    case TensorOp::LT: return binop(&Backend::lt);
    case TensorOp::GT: return binop(&Backend::gt);
    case TensorOp::GTE: return binop(&Backend::gte);
    case TensorOp::LTE: return binop(&Backend::lte);
    case TensorOp::EQ: return binop(&Backend::eq);
    case TensorOp::Where: {
        arity(args, 3);
        same_dtype(args);
        return vals(Value(b.where_cond(to_tensor(args[0]), to_tensor(args[1]), to_tensor(args[2]))));
    }
    case TensorOp::NatToU32: { // tensor_op.rs:77-87
        arity(args, 1);
        size_t n = to_nat(args[0]);
        if (n > 0xFFFFFFFFull) throw InterpreterError("ApplyError: nat does not fit u32");
        uint32_t v = (uint32_t)n;
        return vals(Value(b.ndarray_from_vec_u32(&v, 1, Shape{})));
    }
    case TensorOp::Cast: { // [tensor, dtype]
        arity(args, 2);
        return vals(Value(b.cast(to_tensor(args[0]), to_dtype(args[1]))));
    }
    case TensorOp::MatMul: return binop(&Backend::matmul);
    case TensorOp::ScalarF32: arity(args, 0); return vals(Value(b.ndarray_from_vec_f32(&op.f32, 1, Shape{})));
    case TensorOp::ScalarU32: arity(args, 0); return vals(Value(b.ndarray_from_vec_u32(&op.u32, 1, Shape{})));
    case TensorOp::Sum: return unop(&Backend::sum);
    case TensorOp::Max: return unop(&Backend::max);
    case TensorOp::Argmax: return unop(&Backend::argmax);
    case TensorOp::TopK: { // [x, k]
        arity(args, 2);
        auto r = b.topk(to_tensor(args[0]), to_nat(args[1]));
        return vals(Value(std::move(r.first)), Value(std::move(r.second)));
    }
    case TensorOp::Broadcast: { // [x, shape]  (tensor_op.rs:143)
        arity(args, 2);
        return vals(Value(b.broadcast(to_tensor(args[0]), to_shape(args[1]))));
    }
    case TensorOp::Reshape: { // [shape, x]  (tensor_op.rs:149)
        arity(args, 2);
        return vals(Value(b.reshape(to_tensor(args[1]), to_shape(args[0]))));
    }
    case TensorOp::Transpose: { // [x, dim0, dim1]
        arity(args, 3);
        return vals(Value(b.transpose(to_tensor(args[0]), to_nat(args[1]), to_nat(args[2]))));
    }
    case TensorOp::Slice: { // [x, dim, start, len]
        arity(args, 4);
        return vals(Value(b.slice(to_tensor(args[0]), to_nat(args[1]), to_nat(args[2]), to_nat(args[3]))));
    }
    case TensorOp::Concat: { // [a, b, dim]
        arity(args, 3);
        Tensor x = to_tensor(args[0]), y = to_tensor(args[1]);
        return vals(Value(b.concat(std::move(x), std::move(y), to_nat(args[2]))));
    }
    case TensorOp::Arange: arity(args, 1); return vals(Value(b.arange(to_nat(args[0]))));
    case TensorOp::Index: { // [x, dim, indices]
        arity(args, 3);
        Tensor x = to_tensor(args[0]), ix = to_tensor(args[2]);
        return vals(Value(b.index(std::move(x), to_nat(args[1]), std::move(ix))));
    }
    case TensorOp::Probe: { // tensor_op.rs:121-136: a debugging aid with no results; silent unless CATGRAD_PROBE is set
        if (std::getenv("CATGRAD_PROBE")) {
            arity(args, 1);
            Tensor x = to_tensor(args[0]);
            std::printf("[probe:%s] %s\n", op.label.c_str(), b.format_tensor(x).c_str());
            std::fflush(stdout);
        }
        return {};
    }
    }
    throw InterpreterError("unknown tensor op");
}

// What the interpreter hands operations to while a term is being recorded instead of run (graph.hpp).
struct OpRecorder {
    virtual ~OpRecorder() = default;
    virtual std::vector<Value> record_op(const Op &op, std::vector<Value> args) = 0;
    virtual Tensor record_param(const std::string &path, const Tensor &stored) = 0;
};

// `Interpreter<B>` (interpreter/interpreter.rs:13-59): backend + parameters.
class Interpreter {
  public:
    Interpreter(const std::string &library, int device) : backend(library, device) {}
    Backend backend;
    std::map<std::string, Tensor> parameters; // `Parameters<B>`
    OpRecorder *recorder = nullptr; // set: operations are recorded as a term, not run
    // 0: operations run as the DSL issues them; 1: a forward pass is recorded and run in the layers of the reference's
    // evaluator (graph.hpp); 2: recorded, then run in the order of recording (the lifetime model of 1, the order of 0)
    int schedule = 0;

    // `Load`: parameters.get(path).clone()
    Tensor param(const std::string &path) {
        auto it = parameters.find(path);
        if (it == parameters.end()) throw InterpreterError("MissingParameter: " + path);
        if (recorder) return recorder->record_param(path, it->second);
        return it->second;
    }
    std::vector<Value> run(const Op &op, std::vector<Value> args) {
        if (recorder) return recorder->record_op(op, std::move(args));
        return tensor_op(backend, op, std::move(args));
    }
    Tensor run1(const Op &op, std::vector<Value> args) {
        auto r = run(op, std::move(args));
        return std::move(r[0].tensor);
    }
};

// DSL spellings.  `I` plays the role of the `Builder`; argument orders are those of
// catgrad/src/category/lang/ops.rs:165-218 (e.g. `broadcast(builder, shape, x)` emits
// the operands [x, shape]; `reshape(builder, shape, x)` emits [shape, x]).
namespace ops {
using I = Interpreter;
inline Tensor add(I &i, Tensor x, Tensor y) { return i.run1(TensorOp::Add, vals(std::move(x), std::move(y))); }
inline Tensor sub(I &i, Tensor x, Tensor y) { return i.run1(TensorOp::Sub, vals(std::move(x), std::move(y))); }
inline Tensor mul(I &i, Tensor x, Tensor y) { return i.run1(TensorOp::Mul, vals(std::move(x), std::move(y))); }
inline Tensor div(I &i, Tensor x, Tensor y) { return i.run1(TensorOp::Div, vals(std::move(x), std::move(y))); }
inline Tensor pow(I &i, Tensor x, Tensor y) { return i.run1(TensorOp::Pow, vals(std::move(x), std::move(y))); }
inline Tensor lt(I &i, Tensor x, Tensor y) { return i.run1(TensorOp::LT, vals(std::move(x), std::move(y))); }
inline Tensor lte(I &i, Tensor x, Tensor y) { return i.run1(TensorOp::LTE, vals(std::move(x), std::move(y))); }
inline Tensor gte(I &i, Tensor x, Tensor y) { return i.run1(TensorOp::GTE, vals(std::move(x), std::move(y))); }
// lang/ops.rs:241-249: the operand is borrowed (`&Var`), so the operation reads a clone; it has no result
inline void probe(I &i, const std::string &label, const Tensor &x) { i.run(Op::probe(label), vals(Tensor(x))); }
inline Tensor neg(I &i, Tensor x) { return i.run1(TensorOp::Neg, vals(std::move(x))); }
inline Tensor exp(I &i, Tensor x) { return i.run1(TensorOp::Exp, vals(std::move(x))); }
inline Tensor sin(I &i, Tensor x) { return i.run1(TensorOp::Sin, vals(std::move(x))); }
inline Tensor cos(I &i, Tensor x) { return i.run1(TensorOp::Cos, vals(std::move(x))); }
inline Tensor sum(I &i, Tensor x) { return i.run1(TensorOp::Sum, vals(std::move(x))); }
inline Tensor max(I &i, Tensor x) { return i.run1(TensorOp::Max, vals(std::move(x))); }
inline Tensor argmax(I &i, Tensor x) { return i.run1(TensorOp::Argmax, vals(std::move(x))); }
inline Tensor matmul(I &i, Tensor x, Tensor y) { return i.run1(TensorOp::MatMul, vals(std::move(x), std::move(y))); }
inline Tensor cast(I &i, Tensor x, cg_dtype d) { return i.run1(TensorOp::Cast, vals(std::move(x), d)); }
inline Tensor nat_to_u32(I &i, size_t n) { return i.run1(TensorOp::NatToU32, vals(n)); }
inline Tensor arange(I &i, size_t end) { return i.run1(TensorOp::Arange, vals(end)); }
inline Tensor broadcast(I &i, const Shape &s, Tensor x) { return i.run1(TensorOp::Broadcast, vals(std::move(x), s)); }
inline Tensor reshape(I &i, const Shape &s, Tensor x) { return i.run1(TensorOp::Reshape, vals(s, std::move(x))); }
inline Tensor transpose(I &i, size_t d0, size_t d1, Tensor x) {
    return i.run1(TensorOp::Transpose, vals(std::move(x), d0, d1));
}
inline Tensor index(I &i, size_t dim, Tensor idx, Tensor x) {
    return i.run1(TensorOp::Index, vals(std::move(x), dim, std::move(idx)));
}
inline Tensor slice(I &i, size_t dim, size_t start, size_t len, Tensor x) {
    return i.run1(TensorOp::Slice, vals(std::move(x), dim, start, len));
}
inline Tensor concat(I &i, size_t dim, Tensor x, Tensor y) {
    return i.run1(TensorOp::Concat, vals(std::move(x), std::move(y), dim));
}
inline Shape shape(const Tensor &x) { return x.shape(); }
inline cg_dtype dtype(const Tensor &x) { return x.dtype(); }
// stdlib/ops.rs:16-24: lit + broadcast
inline Tensor lit(I &i, float v) { return i.run1(Op::scalar(v), vals()); }
inline Tensor lit(I &i, uint32_t v) { return i.run1(Op::scalar(v), vals()); }
inline Tensor constant(I &i, float v, const Shape &s) { return broadcast(i, s, lit(i, v)); }
// stdlib/ops.rs:26-30
inline Tensor inverse(I &i, Tensor x) {
    Tensor one = constant(i, 1.0f, shape(x));
    return div(i, std::move(one), std::move(x));
}
} // namespace ops

} // namespace cgh
