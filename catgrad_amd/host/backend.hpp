// C++ mirror of catgrad's interpreter `Backend` trait over the C ABI
// (include/catgrad_hip.h).  Method names, argument order and move semantics follow
// catgrad/src/interpreter/backend/mod.rs:24-122: tensors are passed BY VALUE and are
// consumed by the call, `Tensor`'s copy constructor is `BackendTensor::clone` (a
// reference-count bump), failures that the reference reports by panicking are thrown
// as `Panic`.
//
// The backend library is chosen by path at construction and bound with dlopen, the
// way a Rust binding links the same symbols.
#pragma once

#include <dlfcn.h>

#include <cstdint>
#include <stdexcept>
#include <chrono>
#include <string>
#include <utility>
#include <vector>

#include "../../include/catgrad_hip.h"

namespace cgh {

using Shape = std::vector<size_t>; // `Shape(Vec<usize>)` (catgrad/src/category/core.rs:48)

struct Panic : std::runtime_error {
    int status;
    Panic(int status, const std::string &msg) : std::runtime_error(msg), status(status) {}
};
struct ShapeError : Panic { // BackendError::ShapeError (backend/mod.rs:129-132)
    ShapeError() : Panic(CG_ERR_SHAPE, "ShapeError") {}
};

struct Abi {
#define CGH_FN(name) decltype(&::name) name = nullptr;
    CGH_FN(cg_backend_create) CGH_FN(cg_backend_destroy) CGH_FN(cg_last_error) CGH_FN(cg_backend_name) CGH_FN(cg_sync)
    CGH_FN(cg_pool_stats) CGH_FN(cg_program_stats) CGH_FN(cg_pool_trim) CGH_FN(cg_tensor_retain) CGH_FN(cg_tensor_release)
    CGH_FN(cg_tensor_rank) CGH_FN(cg_tensor_shape) CGH_FN(cg_tensor_dtype) CGH_FN(cg_tensor_numel)
    CGH_FN(cg_tensor_is_contiguous) CGH_FN(cg_zeros) CGH_FN(cg_from_host) CGH_FN(cg_from_host_bf16_as_f32) CGH_FN(cg_arange) CGH_FN(cg_to_host)
    CGH_FN(cg_to_bool) CGH_FN(cg_compare) CGH_FN(cg_format_tensor) CGH_FN(cg_cast) CGH_FN(cg_unary)
    CGH_FN(cg_binary) CGH_FN(cg_where) CGH_FN(cg_matmul) CGH_FN(cg_sum) CGH_FN(cg_max) CGH_FN(cg_argmax)
    CGH_FN(cg_topk) CGH_FN(cg_broadcast) CGH_FN(cg_reshape) CGH_FN(cg_transpose) CGH_FN(cg_slice)
    CGH_FN(cg_concat) CGH_FN(cg_index) CGH_FN(cg_profile_enable) CGH_FN(cg_profile_read)
#undef CGH_FN
    void *handle = nullptr;

    explicit Abi(const std::string &path) {
        handle = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
        if (!handle) throw std::runtime_error(std::string("dlopen failed: ") + dlerror());
#define CGH_LOAD(name)                                                                   \
    name = reinterpret_cast<decltype(name)>(dlsym(handle, #name));                       \
    if (!name) throw std::runtime_error(std::string("missing symbol ") + #name + " in " + path);
        CGH_LOAD(cg_backend_create) CGH_LOAD(cg_backend_destroy) CGH_LOAD(cg_last_error) CGH_LOAD(cg_backend_name)
        CGH_LOAD(cg_sync) CGH_LOAD(cg_pool_stats) CGH_LOAD(cg_program_stats) CGH_LOAD(cg_pool_trim) CGH_LOAD(cg_tensor_retain)
        CGH_LOAD(cg_tensor_release) CGH_LOAD(cg_tensor_rank) CGH_LOAD(cg_tensor_shape) CGH_LOAD(cg_tensor_dtype)
        CGH_LOAD(cg_tensor_numel) CGH_LOAD(cg_tensor_is_contiguous) CGH_LOAD(cg_zeros) CGH_LOAD(cg_from_host) CGH_LOAD(cg_from_host_bf16_as_f32)
        CGH_LOAD(cg_arange) CGH_LOAD(cg_to_host) CGH_LOAD(cg_to_bool) CGH_LOAD(cg_compare) CGH_LOAD(cg_format_tensor)
        CGH_LOAD(cg_cast) CGH_LOAD(cg_unary) CGH_LOAD(cg_binary) CGH_LOAD(cg_where) CGH_LOAD(cg_matmul) CGH_LOAD(cg_sum)
        CGH_LOAD(cg_max) CGH_LOAD(cg_argmax) CGH_LOAD(cg_topk) CGH_LOAD(cg_broadcast) CGH_LOAD(cg_reshape)
        CGH_LOAD(cg_transpose) CGH_LOAD(cg_slice) CGH_LOAD(cg_concat) CGH_LOAD(cg_index)
        CGH_LOAD(cg_profile_enable) CGH_LOAD(cg_profile_read)
#undef CGH_LOAD
    }
    Abi(const Abi &) = delete;
    ~Abi() {
        if (handle) dlclose(handle);
    }
};

// What a `Tensor` needs from a term that is being recorded (graph.hpp): a tensor that stands for a wire of such a
// term has no handle, only the wire's number.
struct WireTable {
    virtual ~WireTable() = default;
    // `x.clone()` in the DSL: a Copy operation with one source and two targets (the numbers of the two new wires)
    virtual std::pair<int, int> copy(int wire) = 0;
    virtual Shape shape_of(int wire) const = 0;
    virtual cg_dtype dtype_of(int wire) const = 0;
};

// `Backend::BackendTensor`: Clone = retain, Drop = release.  While a term is being recorded (graph.hpp) a Tensor can
// also stand for a wire of that term: copying it then records a Copy operation, as `Var::clone` does in the DSL.
class Tensor {
  public:
    Tensor() = default;
    Tensor(const Abi *abi, cg_tensor *h) : abi_(abi), h_(h) {}
    Tensor(WireTable *wires, int wire) : wires_(wires), wire_(wire) {}
    Tensor(const Tensor &o) : abi_(o.abi_), h_(o.h_), wires_(o.wires_) {
        if (h_) abi_->cg_tensor_retain(h_);
        if (wires_ && o.wire_ >= 0) {
            const std::pair<int, int> two = wires_->copy(o.wire_);
            o.wire_ = two.first;
            wire_ = two.second;
        }
    }
    Tensor(Tensor &&o) noexcept : abi_(o.abi_), h_(o.h_), wires_(o.wires_), wire_(o.wire_) {
        o.h_ = nullptr;
        o.wire_ = -1;
    }
    Tensor &operator=(Tensor o) noexcept {
        std::swap(abi_, o.abi_);
        std::swap(h_, o.h_);
        std::swap(wires_, o.wires_);
        std::swap(wire_, o.wire_);
        return *this;
    }
    ~Tensor() {
        if (h_) abi_->cg_tensor_release(h_);
    }
    explicit operator bool() const { return h_ != nullptr || wire_ >= 0; }
    cg_tensor *get() const { return h_; }
    cg_tensor *into_raw() { // hands the reference to a consuming ABI call
        cg_tensor *h = h_;
        h_ = nullptr;
        return h;
    }
    bool is_wire() const { return wire_ >= 0; }
    int take_wire() { // the wire is consumed by the operation being recorded
        const int w = wire_;
        wire_ = -1;
        return w;
    }
    Shape shape() const { // BackendTensorOps::shape
        if (wire_ >= 0) return wires_->shape_of(wire_);
        Shape s(abi_->cg_tensor_rank(h_));
        if (!s.empty()) abi_->cg_tensor_shape(h_, s.data());
        return s;
    }
    cg_dtype dtype() const { return wire_ >= 0 ? wires_->dtype_of(wire_) : abi_->cg_tensor_dtype(h_); }
    size_t numel() const {
        if (wire_ >= 0) {
            size_t n = 1;
            for (size_t d : wires_->shape_of(wire_)) n *= d;
            return n;
        }
        return abi_->cg_tensor_numel(h_);
    }

  private:
    const Abi *abi_ = nullptr;
    cg_tensor *h_ = nullptr;
    WireTable *wires_ = nullptr;
    mutable int wire_ = -1;
};

class Backend {
  public:
    Backend(const std::string &library, int device) : abi_(library) {
        if (abi_.cg_backend_create(device, &b_) != CG_OK) throw Panic(CG_ERR_DEVICE, abi_.cg_last_error());
    }
    Backend(const Backend &) = delete;
    ~Backend() {
        if (b_) abi_.cg_backend_destroy(b_);
    }
    std::string name() const { return abi_.cg_backend_name(b_); }
    uint64_t calls = 0; // backend method calls issued (for the launch-count statistics)
    bool time_calls = false;
    double seconds_in_backend = 0;

    Tensor zeros(const Shape &shape, cg_dtype dt) {
        return out([&](cg_tensor **o) { return abi_.cg_zeros(b_, dt, shape.data(), shape.size(), o); });
    }
    Tensor ndarray_from_vec_f32(const float *data, size_t len, const Shape &shape) {
        return from_vec(CG_F32, data, len, shape);
    }
    Tensor ndarray_from_vec_u32(const uint32_t *data, size_t len, const Shape &shape) {
        return from_vec(CG_U32, data, len, shape);
    }
    // mod.rs:36-46: the 16-bit floats cross the boundary as their bit patterns (2 bytes per element).
    Tensor ndarray_from_vec_f16(const uint16_t *bits, size_t len, const Shape &shape) {
        return from_vec(CG_F16, bits, len, shape);
    }
    Tensor ndarray_from_vec_bf16(const uint16_t *bits, size_t len, const Shape &shape) {
        return from_vec(CG_BF16, bits, len, shape);
    }
    // mod.rs:48-52: fp8 (float8::F8E4M3) as its bit patterns, one byte per element.
    Tensor ndarray_from_vec_fp8(const uint8_t *bits, size_t len, const Shape &shape) {
        return from_vec(CG_F8, bits, len, shape);
    }
    // Weight ingest (catgrad-llm/src/utils/mod.rs:158-168): f32 tensor from bfloat16 bit patterns.
    Tensor from_bf16_bits(const uint16_t *bits, size_t len, const Shape &shape) {
        return out([&](cg_tensor **o) {
            return abi_.cg_from_host_bf16_as_f32(b_, bits, len, shape.data(), shape.size(), o);
        });
    }
    Tensor cast(Tensor x, cg_dtype dt) {
        return out([&](cg_tensor **o) { return abi_.cg_cast(b_, x.into_raw(), dt, o); });
    }
    Tensor matmul(Tensor x, Tensor y) {
        return out([&](cg_tensor **o) { return abi_.cg_matmul(b_, x.into_raw(), y.into_raw(), o); });
    }
    Tensor binary(cg_binary_op op, Tensor x, Tensor y) {
        return out([&](cg_tensor **o) { return abi_.cg_binary(b_, op, x.into_raw(), y.into_raw(), o); });
    }
    Tensor add(Tensor x, Tensor y) { return binary(CG_ADD, std::move(x), std::move(y)); }
    Tensor sub(Tensor x, Tensor y) { return binary(CG_SUB, std::move(x), std::move(y)); }
    Tensor mul(Tensor x, Tensor y) { return binary(CG_MUL, std::move(x), std::move(y)); }
    Tensor div(Tensor x, Tensor y) { return binary(CG_DIV, std::move(x), std::move(y)); }
    Tensor pow(Tensor x, Tensor y) { return binary(CG_POW, std::move(x), std::move(y)); }
    Tensor lt(Tensor x, Tensor y) { return binary(CG_LT, std::move(x), std::move(y)); }
    Tensor gt(Tensor x, Tensor y) { return binary(CG_GT, std::move(x), std::move(y)); }
    Tensor gte(Tensor x, Tensor y) { return binary(CG_GTE, std::move(x), std::move(y)); }
    Tensor lte(Tensor x, Tensor y) { return binary(CG_LTE, std::move(x), std::move(y)); }
    Tensor eq(Tensor x, Tensor y) { return binary(CG_EQ, std::move(x), std::move(y)); }
    Tensor where_cond(Tensor m, Tensor x, Tensor y) {
        return out([&](cg_tensor **o) { return abi_.cg_where(b_, m.into_raw(), x.into_raw(), y.into_raw(), o); });
    }
    Tensor unary(cg_unary_op op, Tensor x) {
        return out([&](cg_tensor **o) { return abi_.cg_unary(b_, op, x.into_raw(), o); });
    }
    Tensor sin(Tensor x) { return unary(CG_SIN, std::move(x)); }
    Tensor cos(Tensor x) { return unary(CG_COS, std::move(x)); }
    Tensor exp(Tensor x) { return unary(CG_EXP, std::move(x)); }
    Tensor log(Tensor x) { return unary(CG_LOG, std::move(x)); }
    Tensor floor(Tensor x) { return unary(CG_FLOOR, std::move(x)); }
    Tensor round(Tensor x) { return unary(CG_ROUND, std::move(x)); }
    Tensor neg(Tensor x) { return unary(CG_NEG, std::move(x)); }
    Tensor broadcast(Tensor x, const Shape &s) {
        return out([&](cg_tensor **o) { return abi_.cg_broadcast(b_, x.into_raw(), s.data(), s.size(), o); });
    }
    Tensor reshape(Tensor x, const Shape &s) {
        return out([&](cg_tensor **o) { return abi_.cg_reshape(b_, x.into_raw(), s.data(), s.size(), o); });
    }
    Tensor transpose(Tensor x, size_t d0, size_t d1) {
        return out([&](cg_tensor **o) { return abi_.cg_transpose(b_, x.into_raw(), d0, d1, o); });
    }
    Tensor max(Tensor x) {
        return out([&](cg_tensor **o) { return abi_.cg_max(b_, x.into_raw(), o); });
    }
    Tensor sum(Tensor x) {
        return out([&](cg_tensor **o) { return abi_.cg_sum(b_, x.into_raw(), o); });
    }
    Tensor argmax(Tensor x) {
        return out([&](cg_tensor **o) { return abi_.cg_argmax(b_, x.into_raw(), o); });
    }
    std::pair<Tensor, Tensor> topk(Tensor x, size_t k) {
        calls++;
        cg_tensor *v = nullptr, *i = nullptr;
        check(abi_.cg_topk(b_, x.into_raw(), k, &v, &i));
        return {Tensor(&abi_, v), Tensor(&abi_, i)};
    }
    bool compare(const Tensor &x, const Tensor &y) {
        calls++;
        int r = 0;
        check(abi_.cg_compare(b_, x.get(), y.get(), &r));
        return r != 0;
    }
    Tensor concat(Tensor x, Tensor y, size_t dim) {
        return out([&](cg_tensor **o) { return abi_.cg_concat(b_, x.into_raw(), y.into_raw(), dim, o); });
    }
    Tensor index(Tensor x, size_t dim, Tensor indices) {
        return out([&](cg_tensor **o) { return abi_.cg_index(b_, x.into_raw(), dim, indices.into_raw(), o); });
    }
    Tensor slice(Tensor x, size_t dim, size_t start, size_t len) {
        return out([&](cg_tensor **o) { return abi_.cg_slice(b_, x.into_raw(), dim, start, len, o); });
    }
    Tensor arange(size_t end) {
        return out([&](cg_tensor **o) { return abi_.cg_arange(b_, end, o); });
    }
    bool to_bool(const Tensor &x) {
        calls++;
        int r = 0;
        check(abi_.cg_to_bool(b_, x.get(), &r));
        return r != 0;
    }
    // `to_vec`: the tensor is taken by value as in the trait and dropped afterwards.
    std::vector<uint32_t> to_vec_bits(Tensor x) {
        calls++;
        std::vector<uint32_t> v(x.numel());
        check(abi_.cg_to_host(b_, x.get(), v.data(), v.size()));
        return v;
    }
    // `to_vec` of an f16 / bf16 tensor: its 16-bit patterns.
    std::vector<uint16_t> to_vec_bits16(Tensor x) {
        calls++;
        std::vector<uint16_t> v(x.numel());
        check(abi_.cg_to_host(b_, x.get(), v.data(), v.size()));
        return v;
    }
    // `to_vec` of an fp8 tensor: its 8-bit patterns.
    std::vector<uint8_t> to_vec_bits8(Tensor x) {
        calls++;
        std::vector<uint8_t> v(x.numel());
        check(abi_.cg_to_host(b_, x.get(), v.data(), v.size()));
        return v;
    }
    std::string format_tensor(const Tensor &x) {
        std::string s(4096, '\0');
        check(abi_.cg_format_tensor(b_, x.get(), s.data(), s.size()));
        s.resize(std::char_traits<char>::length(s.c_str()));
        return s;
    }
    void sync() { check(abi_.cg_sync(b_)); }
    void profile_enable(int cls, unsigned every) { check(abi_.cg_profile_enable(b_, (cg_kernel_class)cls, every)); }
    void profile_read(int cls, uint64_t *n, double *ms, double *work, int reset) {
        check(abi_.cg_profile_read(b_, (cg_kernel_class)cls, n, ms, work, reset));
    }
    void pool_stats(size_t *in_use, size_t *cached) { check(abi_.cg_pool_stats(b_, in_use, cached)); }
    void program_stats(uint64_t *compiled, uint64_t *interpreted, int reset) {
        check(abi_.cg_program_stats(b_, compiled, interpreted, reset));
    }

  private:
    template <class F> Tensor out(F &&f) {
        calls++;
        cg_tensor *o = nullptr;
        if (time_calls) { // diagnostic: how much of a run is spent inside the backend library
            const auto t0 = std::chrono::steady_clock::now();
            const int rc = f(&o);
            seconds_in_backend += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
            check(rc);
        } else {
            check(f(&o));
        }
        return Tensor(&abi_, o);
    }
    Tensor from_vec(cg_dtype dt, const void *data, size_t len, const Shape &shape) {
        calls++;
        cg_tensor *o = nullptr;
        int st = abi_.cg_from_host(b_, dt, data, len, shape.data(), shape.size(), &o);
        if (st == CG_ERR_SHAPE) throw ShapeError();
        check(st);
        return Tensor(&abi_, o);
    }
    void check(int st) {
        if (st != CG_OK) throw Panic(st, abi_.cg_last_error());
    }
    Abi abi_;
    cg_backend *b_ = nullptr;
};

} // namespace cgh
