// A recorded term and its evaluation in the order of the reference's evaluator.
//
// The reference does not run a model's operations in the order the DSL issued them: `eval_with`
// (catgrad/src/abstract_interpreter/eval.rs:18-77) walks `parallel_ssa` (catgrad/src/ssa/mod.rs:24-76), the layers of
// a topological sort in which every operation sits in the earliest layer its operands allow, and within a layer
// follows the numbering of the operations.  Values live in a map from wire to value: an operation takes its operands
// OUT of the map (they are moved into the backend call, eval.rs:41-49), a Copy operation clones its operand once per
// extra target (eval.rs:107-116), a Load clones the parameter (interpreter.rs:56-59), and a wire nobody reads keeps
// its value until the run ends.
//
// While an `Interpreter` records (Interpreter::recorder set), every `tensor_op`, `param` and tensor copy of the model
// code is entered here as an operation between numbered wires instead of being run; `Term::run` then executes the
// operations layer by layer through the same `tensor_op()` dispatcher.  Differences from the reference, which change
// the schedule only: shapes, nats and dtypes are computed while recording (the reference evaluates them as
// operations of the same graph, so an operation that depends on a tensor only through its shape may come later
// there).
//
// A definition (`Module::call`, e.g. nn.sigmoid) is ONE operation of the enclosing term whose body is a term of its
// own, evaluated with its own layers when the operation's turn comes (interpreter.rs:61-74 `handle_definition`).
//
// `If` (core.rs `Operation::If`, interpreter.rs:86-107): the condition tensor is read with `to_bool`, the branch that
// is taken is a term of its own, evaluated with the remaining operands.
#pragma once

#include <algorithm>
#include <functional>
#include <memory>

#include "interp.hpp"

namespace cgh {

struct Term : WireTable, OpRecorder {
    enum Kind { OP, COPY, LOAD, IF, DEFINITION };
    struct Arg { // an operand: a wire, or a value that was known while recording
        int wire = -1;
        Value host;
    };
    struct Operation {
        Kind kind = OP;
        Op op{TensorOp::Add};
        std::string path;              // LOAD, DEFINITION
        std::vector<Arg> args;         // OP / IF / DEFINITION: in the operation's own operand order; COPY: one wire
        std::vector<int> targets;
        std::shared_ptr<Term> then_branch, else_branch; // IF; DEFINITION: then_branch is the definition's term
    };
    struct Wire {
        Shape shape;
        cg_dtype dtype = CG_F32;
        int producer = -1; // operation that writes it; -1: a source of the term
    };
    std::vector<Operation> ops;
    std::vector<Wire> wires;
    std::vector<int> sources;
    std::vector<Tensor> source_values; // concrete tensors the recorded code brought in itself (taken at the start of a run)
    std::vector<int> captured;         // their wires

    int new_wire(const Shape &s, cg_dtype dt, int producer) {
        wires.push_back({s, dt, producer});
        return (int)wires.size() - 1;
    }
    // a source of the term, to be given a value at `run`
    Tensor source(const Shape &s, cg_dtype dt) {
        const int w = new_wire(s, dt, -1);
        sources.push_back(w);
        return Tensor(this, w);
    }
    std::pair<int, int> copy(int wire) override {
        Operation o;
        o.kind = COPY;
        Arg a;
        a.wire = wire;
        o.args.push_back(a);
        const int id = (int)ops.size();
        const int w1 = new_wire(wires[wire].shape, wires[wire].dtype, id), w2 = new_wire(wires[wire].shape, wires[wire].dtype, id);
        o.targets = {w1, w2};
        ops.push_back(std::move(o));
        return {w1, w2};
    }
    Shape shape_of(int wire) const override { return wires[wire].shape; }
    cg_dtype dtype_of(int wire) const override { return wires[wire].dtype; }

    int wire_of(Tensor &t) { // the operand's wire; a concrete tensor becomes a source that already has its value
        if (t.is_wire()) return t.take_wire();
        const int w = new_wire(t.shape(), t.dtype(), -1);
        captured.push_back(w);
        source_values.push_back(std::move(t));
        return w;
    }

    // typecheck/tensor_op.rs: the result types of an operation
    static std::vector<std::pair<Shape, cg_dtype>> result_types(const Op &op, const std::vector<Value> &a) {
        auto sh = [&](size_t i) { return a[i].tensor.shape(); };
        auto dt = [&](size_t i) { return a[i].tensor.dtype(); };
        switch (op.op) {
        case TensorOp::Probe: return {};
        case TensorOp::Where: return {{sh(1), dt(1)}}; // [mask, x, y]: the type of the values, not of the mask
        case TensorOp::NatToU32: return {{Shape{}, CG_U32}};
        case TensorOp::ScalarF32: return {{Shape{}, CG_F32}};
        case TensorOp::ScalarU32: return {{Shape{}, CG_U32}};
        case TensorOp::Cast: return {{sh(0), a[1].dtype}};
        case TensorOp::MatMul: {
            Shape s = sh(0);
            s.back() = sh(1).back();
            return {{s, dt(0)}};
        }
        case TensorOp::Sum:
        case TensorOp::Max: {
            Shape s = sh(0);
            s.back() = 1;
            return {{s, dt(0)}};
        }
        case TensorOp::Argmax: {
            Shape s = sh(0);
            s.back() = 1;
            return {{s, CG_U32}};
        }
        case TensorOp::TopK: {
            Shape s = sh(0);
            s.back() = a[1].nat;
            return {{s, dt(0)}, {s, CG_U32}};
        }
        case TensorOp::Broadcast: return {{a[1].shape, dt(0)}};
        case TensorOp::Reshape: return {{a[0].shape, dt(1)}};
        case TensorOp::Transpose: {
            Shape s = sh(0);
            std::swap(s.at(a[1].nat), s.at(a[2].nat));
            return {{s, dt(0)}};
        }
        case TensorOp::Slice: {
            Shape s = sh(0);
            s.at(a[1].nat) = a[3].nat;
            return {{s, dt(0)}};
        }
        case TensorOp::Concat: {
            Shape s = sh(0);
            s.at(a[2].nat) += sh(1).at(a[2].nat);
            return {{s, dt(0)}};
        }
        case TensorOp::Arange: return {{Shape{a[0].nat}, CG_U32}};
        case TensorOp::Index: {
            Shape s = sh(0);
            s.at(a[1].nat) = a[2].tensor.numel();
            return {{s, dt(0)}};
        }
        default: return {{sh(0), dt(0)}}; // element-wise maps and comparisons: the operands' common type
        }
    }

    std::vector<Value> record_op(const Op &op, std::vector<Value> args) override {
        Operation o;
        o.op = op;
        const auto types = result_types(op, args);
        for (Value &v : args) {
            Arg a;
            if (v.kind == Value::TENSOR) a.wire = wire_of(v.tensor);
            else a.host = v;
            o.args.push_back(std::move(a));
        }
        const int id = (int)ops.size();
        std::vector<Value> out;
        for (const auto &t : types) {
            const int w = new_wire(t.first, t.second, id);
            o.targets.push_back(w);
            out.emplace_back(Tensor(this, w));
        }
        ops.push_back(std::move(o));
        return out;
    }
    Tensor record_param(const std::string &path, const Tensor &stored) override {
        Operation o;
        o.kind = LOAD;
        o.path = path;
        const int w = new_wire(stored.shape(), stored.dtype(), (int)ops.size());
        o.targets = {w};
        ops.push_back(std::move(o));
        return Tensor(this, w);
    }
    // cond(builder, c, then, else, args): both branches are recorded as terms over sources typed like `args`
    template <class F, class G>
    std::vector<Tensor> record_if(Interpreter &i, Tensor cond, std::vector<Tensor> args, F &&then_fn, G &&else_fn) {
        Operation o;
        o.kind = IF;
        std::vector<std::pair<Shape, cg_dtype>> types;
        for (Tensor &t : args) types.emplace_back(t.shape(), t.dtype());
        Arg c;
        c.wire = wire_of(cond);
        o.args.push_back(std::move(c));
        for (Tensor &t : args) {
            Arg a;
            a.wire = wire_of(t);
            o.args.push_back(std::move(a));
        }
        std::vector<std::pair<Shape, cg_dtype>> result_t;
        auto branch = [&](auto &&fn) { return record_subterm(i, types, fn, &result_t); };
        o.then_branch = branch(then_fn);
        const std::vector<std::pair<Shape, cg_dtype>> then_t = result_t;
        o.else_branch = branch(else_fn);
        // both branches have the type of the operation (the reference's type checker rejects anything else)
        if (then_t != result_t) throw InterpreterError("TypeError: the branches of If disagree in their result types");
        const int id = (int)ops.size();
        std::vector<Tensor> out;
        for (const auto &t : result_t) {
            const int w = new_wire(t.first, t.second, id);
            o.targets.push_back(w);
            out.emplace_back(this, w);
        }
        ops.push_back(std::move(o));
        return out;
    }
    // `Module::call` (a Definition operation): `fn` is the definition's body, recorded as a term over sources typed
    // like `args`.
    template <class F> std::vector<Tensor> record_definition(Interpreter &i, const std::string &path, std::vector<Tensor> args, F &&fn) {
        Operation o;
        o.kind = DEFINITION;
        o.path = path;
        std::vector<std::pair<Shape, cg_dtype>> types;
        for (Tensor &t : args) types.emplace_back(t.shape(), t.dtype());
        for (Tensor &t : args) {
            Arg a;
            a.wire = wire_of(t);
            o.args.push_back(std::move(a));
        }
        std::vector<std::pair<Shape, cg_dtype>> result_t;
        o.then_branch = record_subterm(i, types, fn, &result_t);
        const int id = (int)ops.size();
        std::vector<Tensor> out;
        for (const auto &t : result_t) {
            const int w = new_wire(t.first, t.second, id);
            o.targets.push_back(w);
            out.emplace_back(this, w);
        }
        ops.push_back(std::move(o));
        return out;
    }
    // a term of its own for a branch or a definition: `fn` runs over fresh sources while `i` records into the new term
    template <class F>
    static std::shared_ptr<Term> record_subterm(Interpreter &i, const std::vector<std::pair<Shape, cg_dtype>> &types, F &&fn,
                                                std::vector<std::pair<Shape, cg_dtype>> *result_types_out) {
        std::vector<std::pair<Shape, cg_dtype>> &result_t = *result_types_out;
        auto branch = [&](auto &&fn) {
            auto term = std::make_shared<Term>();
            std::vector<Tensor> src;
            for (const auto &t : types) src.push_back(term->source(t.first, t.second));
            OpRecorder *outer = i.recorder;
            i.recorder = term.get();
            std::vector<Tensor> res;
            try {
                res = fn(std::move(src));
            } catch (...) {
                i.recorder = outer;
                throw;
            }
            i.recorder = outer;
            result_t.clear();
            for (Tensor &r : res) {
                result_t.emplace_back(r.shape(), r.dtype());
                term->results.push_back(term->wire_of(r));
            }
            return term;
        };
        return branch(fn);
    }
    std::vector<int> results; // wires handed back by `run` (set by finish / record_if)
    void finish(std::vector<Tensor> outs) {
        for (Tensor &t : outs) results.push_back(wire_of(t));
    }

    // The layers of `layered_operations`: an operation's layer is one more than the latest layer among the operations
    // that write its operands (0 when all operands are sources); inside a layer, in the order of recording.
    std::vector<int> schedule() const {
        std::vector<int> layer(ops.size(), 0);
        for (size_t e = 0; e < ops.size(); e++) // operands are always recorded before their readers
            for (const Arg &a : ops[e].args)
                if (a.wire >= 0 && wires[a.wire].producer >= 0) layer[e] = std::max(layer[e], layer[wires[a.wire].producer] + 1);
        std::vector<int> order(ops.size());
        for (size_t e = 0; e < ops.size(); e++) order[e] = (int)e;
        std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return layer[x] < layer[y]; });
        return order;
    }

    // eval_with: `inputs` are moved into the sources' wires.  in_order: run in the order of recording instead (the
    // order of the DSL), with the same value map.
    std::vector<Tensor> run(Interpreter &i, std::vector<Tensor> inputs, bool in_order = false) {
        if (inputs.size() != sources.size()) throw InterpreterError("ApplyError: wrong number of term inputs");
        std::vector<Tensor> state(wires.size());
        std::vector<char> present(wires.size(), 0);
        auto put = [&](int w, Tensor t) {
            if (present[w]) throw InterpreterError("MultipleWrite");
            state[w] = std::move(t);
            present[w] = 1;
        };
        auto take = [&](int w) {
            if (!present[w]) throw InterpreterError("MultipleRead");
            present[w] = 0;
            return std::move(state[w]);
        };
        for (size_t k = 0; k < sources.size(); k++) put(sources[k], std::move(inputs[k]));
        for (size_t k = 0; k < captured.size(); k++) put(captured[k], source_values[k]); // a clone: the term can run again
        std::vector<int> order = schedule();
        if (in_order)
            for (size_t e = 0; e < order.size(); e++) order[e] = (int)e;
        for (int e : order) {
            Operation &o = ops[e];
            switch (o.kind) {
            case COPY: { // apply_copy: the value, then one clone per further target
                Tensor v = take(o.args[0].wire);
                for (size_t k = 1; k < o.targets.size(); k++) put(o.targets[k], v);
                put(o.targets[0], std::move(v));
                break;
            }
            case LOAD: put(o.targets[0], i.param(o.path)); break;
            case OP: {
                std::vector<Value> args;
                for (Arg &a : o.args) {
                    if (a.wire >= 0) args.emplace_back(take(a.wire));
                    else args.push_back(a.host);
                }
                std::vector<Value> res = tensor_op(i.backend, o.op, std::move(args));
                if (res.size() != o.targets.size()) throw InterpreterError("ApplyError: wrong number of results");
                for (size_t k = 0; k < res.size(); k++) put(o.targets[k], std::move(res[k].tensor));
                break;
            }
            case DEFINITION: { // handle_definition: the definition's term, evaluated with the operation's operands
                std::vector<Tensor> in;
                for (Arg &a : o.args) in.push_back(take(a.wire));
                std::vector<Tensor> res = o.then_branch->run(i, std::move(in), in_order);
                if (res.size() != o.targets.size()) throw InterpreterError("ApplyError: wrong number of results");
                for (size_t k = 0; k < res.size(); k++) put(o.targets[k], std::move(res[k]));
                break;
            }
            case IF: { // handle_if: to_bool of (a clone of) the condition, then the branch's own evaluation
                Tensor cond = take(o.args[0].wire);
                std::vector<Tensor> rest;
                for (size_t k = 1; k < o.args.size(); k++) rest.push_back(take(o.args[k].wire));
                Term &branch = i.backend.to_bool(cond) ? *o.then_branch : *o.else_branch;
                std::vector<Tensor> res = branch.run(i, std::move(rest), in_order);
                if (res.size() != o.targets.size()) throw InterpreterError("ApplyError: wrong number of results");
                for (size_t k = 0; k < res.size(); k++) put(o.targets[k], std::move(res[k]));
                break;
            }
            }
        }
        std::vector<Tensor> out;
        for (int w : results) out.push_back(take(w));
        return out; // what is left in `state` (wires nobody read) is dropped here, at the end of the run
    }
};

} // namespace cgh

namespace cgh {
namespace ops {
// `cond(builder, c, then, else, args)` (catgrad/src/category/lang/ops.rs): the operation `If`.  Run directly it is
// handle_if (interpreter.rs:86-107): to_bool of the condition, then the branch that is taken; recorded, both branches
// become terms of their own.
template <class F, class G>
inline std::vector<Tensor> cond(I &i, Tensor c, F &&then_fn, G &&else_fn, std::vector<Tensor> args) {
    if (Term *t = dynamic_cast<Term *>(i.recorder)) return t->record_if(i, std::move(c), std::move(args), then_fn, else_fn);
    return i.backend.to_bool(c) ? then_fn(std::move(args)) : else_fn(std::move(args));
}
// `Module::call(builder, args)`: a Definition operation named `path` whose body is `fn`.  Run directly, the body's
// operations are issued where the call stands, which is the order handle_definition gives them too.
template <class F> inline std::vector<Tensor> definition(I &i, const std::string &path, F &&fn, std::vector<Tensor> args) {
    if (Term *t = dynamic_cast<Term *>(i.recorder)) return t->record_definition(i, path, std::move(args), fn);
    return fn(std::move(args));
}
} // namespace ops
} // namespace cgh
