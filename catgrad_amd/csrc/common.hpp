// Internal declarations shared by the host runtime and the kernel launchers of
// libcatgrad_hip.so.  Nothing here is part of the C ABI (include/catgrad_hip.h).
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "../../include/catgrad_hip.h"

namespace cg {

constexpr int kMaxRank = CG_MAX_RANK;

int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char *what);

#define CG_HIP(expr)                                          \
    do {                                                      \
        hipError_t _e = (expr);                               \
        if (_e != hipSuccess) return cg::hip_fail(_e, #expr); \
    } while (0)

// Bits the kernels set in the backend's host-mapped fault word; reported by the next
// call that waits for the device.
enum : uint32_t { kFaultIndexRange = 1u, kFaultDivZero = 2u };

// Device memory pool: size-class free lists on one stream.  A block freed while
// kernels that use it are still queued may be handed out again at once, because every
// later user is ordered behind them on the same stream.
class Pool {
  public:
    int alloc(size_t bytes, void **ptr, size_t *cls);
    void free(void *ptr, size_t cls);
    void trim();
    void stats(size_t *in_use, size_t *cached);
    static size_t size_class(size_t bytes);

  private:
    std::mutex mu_;
    std::multimap<size_t, void *> free_;
    size_t in_use_ = 0, cached_ = 0;
};

struct ProfClass {
    unsigned every = 0;
    uint64_t seen = 0, timed = 0;
    double ms = 0.0, work = 0.0;
};
struct ProfPending {
    hipEvent_t a, b;
    int cls;
    double work;
};

} // namespace cg

namespace cg {
// Objects that every backend call makes and drops (tensor handles, deferred programs, lazy products, buffer records) come
// from free lists of their own instead of the C library's heap, whose arena lock the runtime's own threads contend for: a
// sampling profile of a launch-bound decode step had a fifth of the host's time in malloc / free and their lock.
template <class T> struct Pooled {
    // one list per type for the whole process, behind a flag that is almost never contended (a backend's calls are
    // serialised by its own lock); it is never destroyed, so handles dropped while the process exits still find it
    struct List {
        std::atomic_flag busy = ATOMIC_FLAG_INIT;
        std::vector<void *> free;
    };
    static List &list() {
        static List *l = new List;
        return *l;
    }
    static void *operator new(size_t n) {
        if (n == sizeof(T)) {
            List &l = list();
            while (l.busy.test_and_set(std::memory_order_acquire)) {
            }
            void *p = nullptr;
            if (!l.free.empty()) {
                p = l.free.back();
                l.free.pop_back();
            }
            l.busy.clear(std::memory_order_release);
            if (p) return p;
        }
        return ::operator new(n);
    }
    static void operator delete(void *p, size_t n) {
        if (!p) return;
        if (n == sizeof(T)) {
            List &l = list();
            while (l.busy.test_and_set(std::memory_order_acquire)) {
            }
            const bool keep = l.free.size() < 1024;
            if (keep) l.free.push_back(p);
            l.busy.clear(std::memory_order_release);
            if (keep) return;
        }
        ::operator delete(p);
    }
};

struct LazyMm;
struct DeferredWrite;
struct Buffer;
}

struct cg_backend {
    std::recursive_mutex mu; // held by every entry point for the duration of the call
    std::atomic<long> live_tensors{0}; // heap handles that name this backend (see alloc_tensor)
    bool owner_gone = false;           // cg_backend_destroy has been called; the last handle released tears down
    int device = 0;
    hipStream_t stream = nullptr;
    cg::Pool pool;
    uint32_t *fault_host = nullptr; // pinned, device-visible
    uint32_t *fault_dev = nullptr;
    uint32_t *flag_dev = nullptr;   // 4-byte scratch for to_bool / compare
    uint32_t *flag_host = nullptr;  // pinned landing zone for it
    // small read-backs (the tokens of a decode step): a kernel copies the words into pinned, device-visible memory and
    // writes a sequence number behind them; the host polls it instead of waiting for the stream (CG_FAST_READBACK=0: never)
    uint32_t *rb_host = nullptr, *rb_dev = nullptr;
    uint32_t rb_seq = 0;
    bool fast_readback = true;
    // host-to-device staging: two pinned buffers used in turn, each guarded by an event
    void *stage[2] = {nullptr, nullptr};
    hipEvent_t stage_ev[2] = {nullptr, nullptr};
    bool stage_busy[2] = {false, false};
    unsigned stage_next = 0;
    std::string name;
    std::vector<cg::LazyMm *> lazy_open; // groupable lazy products not yet computed (not retained)
    std::vector<cg::DeferredWrite> deferred; // writes waiting to share a launch (see flush_deferred)
    // Results that depend on constants only (the rotary tables every forward pass rebuilds from iota and
    // scalars) are kept, keyed by the program and its leaves, and handed out again instead of recomputed.
    // Buffers are retained here; the oldest entries go when the limits are reached.
    std::map<std::string, cg::Buffer *> const_memo;
    std::vector<std::string> const_order; // keys, oldest first
    size_t const_bytes = 0;
    cg::Buffer *iota = nullptr; // 0, 1, 2, ... : every arange is a view of it
    int64_t iota_len = 0;
    bool fuse = true; // defer element-wise ops and fuse them (CG_FUSE=0 switches it off)
    bool aot = true;  // use the compiled kernels for listed programs (CG_AOT=0: interpreter only)
    uint64_t programs_compiled = 0, programs_interpreted = 0; // launches of fused programs, by kernel kind
    // decode-time attention over a cache of at least this many positions runs a workgroup per (KV head, segment of the
    // cache) (CG_ATTN_SEG_FROM, read when the backend is created; 0: never)
    int64_t attn_seg_from = 6001;
    bool narrow_storage = true;  // tensors of the narrow float dtypes keep 2- / 1-byte elements in memory (CG_NARROW_STORAGE=0: 32-bit words)
    int64_t narrow_from = 65536; // ... from this many elements on (CG_NARROW_FROM); smaller tensors stay 32-bit words: the kernels of a
                                 // decode step, which address words, never meet a narrow operand that way
    int compute_units = 256;     // of the device (a persistent kernel launches one workgroup for each)
    bool trace_programs = false; // CG_TRACE_PROGRAMS=1: print each distinct deferred program once, to stderr
    cg::ProfClass prof[CG_K_CLASSES];
    std::vector<cg::ProfPending> prof_pending;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> prof_free;
};

namespace cg {

constexpr size_t kStageBytes = 16u << 20; // size of each pinned host-to-device staging buffer

// Row-block structure of a buffer that grows by appended rows (a KV cache): the buffer is
// [nblocks][C][R] elements, block b holds fill[b] valid rows of R elements, rows at and
// beyond fill[b] are free and no view covers them.  `concat` along the row axis appends
// in place at that frontier.
struct RowStore {
    int64_t R = 0, C = 0, nblocks = 0;
    int64_t src_C = 0; // block capacity of the buffer whose blocks migrate here: block ids are numbered in its units
    std::vector<int64_t> fill;
};

// How the elements of a buffer lie in memory.  32-bit words (f32 and u32 values; also values of the narrow float dtypes,
// each held exactly in an f32 word), or the narrow dtypes' own patterns: 2 bytes per element for bfloat16 / binary16, 1 for
// fp8 (E4M3).  A format is a property of the BUFFER, not of the dtype tag of a tensor that views it: what a narrow buffer
// holds are exactly representable values, so a tensor of any floating-point dtype may view it.  Kernels either take the
// format from their operand descriptors (element-wise kernels, fused programs, copies, gathers, the narrow-operand matrix
// products) or ask for words (device_ptr), which a narrow buffer answers with a widened copy that it makes once and keeps.
enum : int { kFmtWords = 0, kFmtBF16 = 1, kFmtF16 = 2, kFmtF8 = 3 };
inline int fmt_of(cg_dtype d) { return d == CG_BF16 ? kFmtBF16 : d == CG_F16 ? kFmtF16 : d == CG_F8 ? kFmtF8 : kFmtWords; }
inline size_t fmt_bytes(int fmt) { return fmt == kFmtWords ? 4 : fmt == kFmtF8 ? 1 : 2; }

inline uint64_t next_buffer_id() {
    static std::atomic<uint64_t> n{1};
    return n.fetch_add(1);
}

struct Buffer : Pooled<Buffer> {
    std::atomic<long> rc{1};
    const uint64_t id = next_buffer_id(); // never reused, unlike the address: what keys of kept results name
    void *ptr = nullptr;
    size_t cls = 0;
    int64_t elems = 0;           // elements in use from the start of the buffer (grows with in-place appends); <= cls / 4
    int fmt = kFmtWords;         // element format (see above); a narrow buffer is never appended to or written in place
    Buffer *wide = nullptr;      // retained: this narrow buffer's elements as 32-bit words, made when a kernel that only
                                 // reads words first needed them (device_ptr)
    cg_backend *be = nullptr;
    RowStore *rs = nullptr;      // owned
    bool constant = false;       // the contents depend on constants only (iota, programs over such buffers)
    Buffer *successor = nullptr; // retained: the roomier buffer that blocks of this one migrate to on append
    // Set by the product kernels that store a residual stream [rows <= 4, N]: per workgroup (4 columns) and row
    // the sum of squares of what it stored, [side_blocks][4] floats.  An RMS norm over these rows that feeds
    // decode-time products needs no pass of its own then (see NormFuse).  Owned (pool memory).
    void *side = nullptr;
    size_t side_cls = 0;
    uint32_t side_blocks = 0;
    // Narrow copies of 2-D views of this buffer for the matrix instructions of its dtype (launch_matmul): [rows][k] of
    // 2-byte (f16 / bf16) or 1-byte (fp8) patterns, k contiguous, one entry per view (several slices of one weight buffer
    // each keep theirs; the oldest goes when the list is full).  A weight matrix is narrowed once and the copy kept while
    // the buffer lives.  Every path that writes into an existing buffer drops the list first (drop_packed), so an entry
    // always describes what its view shows.  Owned (pool memory).
    struct Packed {
        void *ptr = nullptr;
        size_t cls = 0;
        int kind = 0; // 1 bf16, 2 f16, 3 fp8
        int64_t off = 0, rows = 0, k = 0, sr = 0, sk = 0;
    };
    std::vector<Packed> packed;
};
constexpr size_t kMaxPackedPerBuffer = 4;
// Frees the narrow copies kept with `b` (to be called before anything is written into a buffer that existed before).
void drop_packed(Buffer *b);

} // namespace cg

namespace cg {
struct Pending;
}

// A strided view of a device buffer.  Strides and offset are in elements; a stride of
// 0 is a broadcast axis.  `uniform` marks a tensor all of whose elements equal `ubits`
// (rank-0 constants, zeros, and every view of them): such tensors own no memory until a
// kernel needs to address them, and kernels take their value as an immediate.
struct cg_tensor : cg::Pooled<cg_tensor> {
    std::atomic<long> rc{1};
    cg_backend *be = nullptr;
    cg::Buffer *buf = nullptr;
    cg_dtype dt = CG_F32;
    int rank = 0;
    int64_t dims[cg::kMaxRank] = {0};
    int64_t strides[cg::kMaxRank] = {0};
    int64_t offset = 0;
    bool uniform = false;
    uint32_t ubits = 0;
    // A deferred element-wise result: no buffer yet, `pend` says how to compute it.
    cg::Pending *pend = nullptr;
    // Split axis: logical axis `split` (extent outer * split_inner) is addressed as
    // (i / split_inner) * split_os + (i % split_inner) * strides[split].  This is what
    // `reshape` makes of two adjacent axes that cannot share one stride — the merged
    // [kvH, rep] axis of repeat_kv, whose `rep` part has stride 0 — so that the batched
    // GEMM can walk the two parts as separate batch axes instead of reading a 4x copy.
    // Only transpose / slice (other axes) / broadcast / matmul understand it; every
    // other consumer first turns the tensor into a plain dense one.
    int split = -1;
    int64_t split_inner = 0, split_os = 0;
};

namespace cg {

// Floating-point dtypes: the arithmetic is f32 on 32-bit words; CG_F16 / CG_BF16 / CG_F8 results are rounded
// to their format after every op (the words always hold exactly representable values).
inline bool is_f(cg_dtype d) { return d == CG_F32 || d == CG_F16 || d == CG_BF16 || d == CG_F8; }
inline bool is_half(cg_dtype d) { return d == CG_F16 || d == CG_BF16; }
// dtypes narrower than their 32-bit words: results are rounded after every op
inline bool is_narrow(cg_dtype d) { return is_half(d) || d == CG_F8; }

inline int64_t numel(const cg_tensor *t) {
    int64_t n = 1;
    for (int i = 0; i < t->rank; i++) n *= t->dims[i];
    return n;
}
bool is_contiguous(const cg_tensor *t);
void release(cg_tensor *t);
inline void retain(cg_tensor *t) { t->rc.fetch_add(1, std::memory_order_relaxed); }
// Fresh row-major tensor with pool memory (none when numel == 0).
// `reserve_elems` asks for a buffer with room for at least that many elements.
// `fmt`: the element format of the new buffer (a narrow one only for results whose producer stores that format).
int new_dense(cg_backend *be, cg_dtype dt, const int64_t *dims, int rank, cg_tensor **out, int64_t reserve_elems = 0,
              int fmt = kFmtWords);
// The narrowest format that results of dtype dt with n elements are stored in (small results stay words: the kernels of a
// decode step address words).
int result_fmt(const cg_backend *be, cg_dtype dt, int64_t n);
// Fresh uniform tensor (no memory).
cg_tensor *new_uniform(cg_backend *be, cg_dtype dt, const int64_t *dims, int rank, uint32_t bits);
// New handle sharing t's buffer and metadata.
cg_tensor *new_view(const cg_tensor *t);
// Device address of element 0 of the view, for kernels that READ 32-bit words; allocates the 4-byte backing word of a
// uniform tensor on first use.  A view of a narrow buffer is answered from the buffer's widened copy (made on first
// use, kept with the buffer).  Never for a destination: a kernel that writes takes device_ptr_fmt.
int device_ptr(const cg_tensor *t, const void **ptr);
// The same in the buffer's own format: *fmt says how the elements behind *ptr lie in memory.
int device_ptr_fmt(const cg_tensor *t, const void **ptr, int *fmt);
inline bool is_narrow_buf(const Buffer *b) { return b && b->fmt != kFmtWords; }

// ---- magic-number division for 32-bit indices (Granlund-Montgomery round-up) ----
struct FastDiv {
    uint32_t d, m, s1, s2;
};
FastDiv make_fastdiv(uint32_t d);

// ---- launch descriptors ------------------------------------------------------------
constexpr int kMaxOuter = kMaxRank - 1;

struct Operand {
    const char *ptr;           // byte address of the view's first element (null if uniform)
    int64_t os[kMaxOuter];     // element strides of the outer axes, innermost first
    int64_t is;                // element stride of the inner axis
    uint32_t uniform;          // 1: take `ubits`, never dereference ptr
    uint32_t ubits;
    uint32_t fmt;              // element format of the memory behind ptr (kFmtWords, ...): loads widen, stores narrow
};

struct EwGeom {
    uint32_t nouter;           // collapsed rank - 1
    uint32_t inner;            // extent of the inner axis
    uint32_t ipr;              // work items per row (inner / VEC)
    uint32_t vec;              // 1 or 4 elements per work item
    FastDiv ipr_div;
    uint32_t od[kMaxOuter];    // outer extents, innermost first
    FastDiv odiv[kMaxOuter];
    uint64_t total;            // work items
};

// ---- deferred element-wise expressions ------------------------------------------------
// Element-wise results are not computed when the op is issued: the handle carries a small
// program over "leaf" views (concrete strided views or constants, all of the result's
// shape).  A consumer that is itself element-wise splices the program into its own; a
// reduction evaluates it while reading; anything else (matmul, concat, gather, read-back)
// materialises it with ONE launch of the interpreter kernel.  Each element goes through
// exactly the operations, in the order, that the separate ops would have applied, so
// results are bit-identical to unfused execution.
//
// `sum` and `max` over the last axis are deferred too, as row-reduce instructions: the
// value of such an instruction is the reduction of its operand over the row (the last axis
// of the program's iteration space) and is the same for every element of the row.  The
// tensor a reduction returns has last extent 1 while its program still iterates over rows
// of `rowlen` elements (`reduced`); broadcasting it back to the row shape yields an
// ordinary full-shape program again, so max -> sub -> exp -> sum -> div (softmax) or
// square -> sum -> scale -> sqrt -> div (RMS norm) collapse into ONE kernel in which a
// workgroup walks its row once per reduction and once more to produce the output.
constexpr int kMaxLeaves = 8, kMaxInstr = 24, kMaxViews = kMaxLeaves + 1, kMaxRowReduce = 3;

struct Instr {
    uint8_t op;      // EwOp code, | kInstrU32 when the operands are u32
    uint8_t a, b, c; // registers: < kMaxLeaves = leaf, else kMaxLeaves + instruction index
};
constexpr uint8_t kInstrU32 = 0x80;

// A decode-time attention score product q.K^T (at most 8 rows, K = head_dim) whose execution is
// put off: if the soft-max over it ends up as the left operand of p.V, the three are run as one
// fused attention kernel and the scores never exist in memory; any other use computes the
// product once (`result`) and reads it like any buffer.
// A small element-wise result whose destination is known but which nobody has read yet: the rows a
// decode step appends to the KV cache.  Put off until the next launch, which it then shares with
// its neighbours (at most three per launch).
struct DeferredWrite {
    cg_tensor *dst = nullptr; // a view of the destination; its buffer is retained
    Pending *prog = nullptr;  // owned
};

// x / pow(sum(x*x) / n + eps, e) * gamma applied to the left operand while a decode-time product loads it:
// the row sums come from the per-workgroup partial sums that the kernel which stored x left behind.
struct NormFuse {
    const float *partials; // [blocks][4]
    uint32_t blocks;
    const uint32_t *gamma; // [K]
    uint32_t n_bits, eps_bits, exp_bits;
};

struct LazyMm : Pooled<LazyMm> {
    std::atomic<long> rc{1};
    // retained operands; y is concrete, x is concrete or (groupable products only) still the deferred RMS norm
    // of a residual stream with partial sums, see norm_fuse_of
    cg_tensor *x = nullptr, *y = nullptr;
    Buffer *result = nullptr;             // retained once computed
    int64_t dims[kMaxRank] = {0};
    int rank = 0;
    // A decode-time linear layer (few rows times a weight matrix): products of this kind that
    // share their left operand and are still open when one of them is needed (q / k / v, gate / up)
    // are computed by one grouped launch.  `be` is set while the product is listed as open.
    bool groupable = false;
    cg_backend *be = nullptr;
    // A product whose value is x . y with an RMS norm over every run of hn_hd columns applied to it (see RopeStore::hgamma):
    // what became of `rmsnorm(reshape(x . y, [rows * heads, hd]))` when the product was still open.  Computed either by the
    // kernel that also embeds and stores the heads (try_rope_stores), or, when something else needs it first, as the
    // product followed by the kept program hn_prog (whose leaf 0 then reads the plain product).
    bool head_norm = false;
    Buffer *hn_gamma = nullptr; // retained
    int64_t hn_gamma_off = 0;
    uint32_t hn_hd = 0, hn_n_bits = 0, hn_eps_bits = 0, hn_exp_bits = 0;
    Pending *hn_prog = nullptr; // owned
    int64_t hn_dims[kMaxRank] = {0};
    int hn_rank = 0;
};
void lazy_mm_release(LazyMm *m);
// Computes the product if it has not been yet.
int lazy_mm_force(cg_backend *be, LazyMm *m);

// (No default member initialisers: a Pending holds eight of these and most programs use one or two, so its leaf table
// starts out uninitialised and only leaf[0 .. nleaf) is ever read.  `LeafView lv{};` gives an empty one: everything zero.)
struct LeafView {
    Buffer *buf; // retained; null for uniform leaves (and for a lazy product not yet computed)
    LazyMm *lazy; // retained: the leaf is the (row-major) result of this product
    int64_t strides[kMaxRank];
    int64_t offset;
    bool uniform;
    uint32_t ubits;
    // Piecewise leaf (the deferred form of `concat` along the last axis): positions below
    // `pw_split` of the last axis read the view above, the others read (buf2, strides2,
    // offset2) at position - pw_split; a part may be negated on load (f32 sign flip), which
    // is how rotate_half = concat(-x2, x1) of the rotary embedding stays a leaf.
    bool pw;
    Buffer *buf2; // retained
    LazyMm *lazy2; // retained: the second part is a view of this product's result (buf2 null until it is computed)
    int64_t strides2[kMaxRank];
    int64_t offset2;
    int64_t pw_split;
    bool neg1, neg2;
};

struct Pending : Pooled<Pending> {
    int nleaf = 0, ninstr = 0;
    bool expensive = false; // holds pow / exp / log / sin / cos
    int nred = 0;           // row-reduce instructions in the program
    int64_t rowlen = 0;     // extent of the last axis of the iteration space (set when nred > 0)
    bool reduced = false;   // the tensor's own last extent is 1: its value is the row-uniform result
    bool overflow = false;  // set while building when the leaf or instruction table ran out
    LeafView leaf[kMaxLeaves];
    Instr ins[kMaxInstr];
    Pending() = default;
    Pending(const Pending &o);
    Pending &operator=(const Pending &) = delete;
    ~Pending();
};

struct ViewDesc {
    const int64_t *strides;
    bool uniform;
    uint32_t ubits;
    const char *ptr; // device address of the view's first element (unused when uniform)
    int64_t vec_period = 0; // > 0: 16-byte vectors are only allowed if this divides by 4 (a piecewise leaf's split)
    int fmt = kFmtWords;    // element format of the memory behind ptr
};
// Collapses the iteration space shared by `n` views of shape `dims` (v[0] is the output)
// and fills geometry + operands.  keep_last_axis: never merge the last axis into the one
// before it (reductions need it on its own).
// allow_vec8: work items of 8 elements when some operand lies in memory in a narrow format (its 16-byte access) and the
// extents and every operand's alignment allow it (the caller's kernel must have that instantiation).
int plan_views(const int64_t *dims, int rank, const ViewDesc *v, int n, bool keep_last_axis, EwGeom *g, Operand *ops,
               bool allow_vec4 = true, bool allow_vec8 = false);

// Collapses the iteration space shared by `n` views of identical shape (views[0] is
// the output) and fills geometry + operands.  Returns CG_ERR_UNSUPPORTED when the
// space exceeds 2^32-1 work items.
int plan_elementwise(const cg_tensor *const *views, int n, EwGeom *g, Operand *ops, bool allow_vec8 = false);

// Times one launch with a pair of events on the backend's stream when the kernel class
// is being sampled; the pair is resolved by the next call that waits for the device.
class ProfScope {
  public:
    ProfScope(cg_backend *be, int cls, double work);
    ~ProfScope();

  private:
    cg_backend *be_;
    int slot_ = -1;
};
// Algorithmic bytes of a view: 4 B per distinct element (broadcast axes count once).
double distinct_bytes(const cg_tensor *t);
void prof_drain(cg_backend *be);

// ---- kernel launchers (ew.hip, reduce.hip, matmul.hip) -------------------------------
enum EwOp : int {
    // unary (CG_NEG.. order of cg_unary_op)
    kNeg = 0, kSin, kCos, kExp, kLog, kFloor, kRound,
    // f32 -> nearest bfloat16 / binary16 value (ties to even), still held as f32: how results of the
    // 16-bit float dtypes are rounded (every tensor is stored as 32-bit words)
    kRoundBF16, kRoundF16,
    // f32 -> nearest fp8 (E4M3) value, ties to even, +-448 beyond the largest finite value; still held as f32
    kRoundF8,
    // binary (order of cg_binary_op) offset by 16
    kAdd = 16, kSub, kMul, kDiv, kPow, kLt, kGt, kGte, kLte, kEq,
    kWhere = 32,
    kCastF2U = 40, kCastU2F, kCopy,
    // row reductions inside deferred programs (operand a; the result is uniform along the row)
    kRowSum = 48, kRowMax
};
constexpr bool is_row_reduce(int op) { return (op & ~0x80) == kRowSum || (op & ~0x80) == kRowMax; }

// out = op(ins...) element-wise; all views have out's shape.  `out` may be a strided view.
// round_op: kRoundBF16 / kRoundF16 / kRoundF8 applied to the (f32) result before it is stored, 0: none.
int launch_elementwise(cg_backend *be, int op, cg_dtype dt, const cg_tensor *out, const cg_tensor *const *ins, int nin, int round_op = 0);
// True when the program of `p` can be register-allocated for the interpreter kernels.
bool fused_program_fits(const Pending &p);
// Evaluates `p` for every element of shape `dims` into `out` (a dense or strided view of that shape).
int launch_fused(cg_backend *be, const cg_tensor *out, const Pending &p);
// Last-axis reduction of the value of the first `ninstr` instructions of `p` (shape dims/rank)
// into the dense tensor `out`.
int launch_fused_reduce(cg_backend *be, int kind, bool f32, const Pending &p, int ninstr, const int64_t *dims, int rank,
                        cg_tensor *out);
// Evaluates a program with row-reduce instructions over the iteration space `dims` (last axis = row).
// reduced: `out` is dense with one element per row; else `out` is a (strided) view of shape `dims`.
int launch_fused_rows(cg_backend *be, const cg_tensor *out, const Pending &p, const int64_t *dims, int rank);
int launch_arange(cg_backend *be, cg_tensor *out);
// Copies n <= kReadbackWords words to be->rb_dev and then stores `seq` at word kReadbackWords of it, visible to the host.
constexpr uint32_t kReadbackWords = 1024;
int launch_small_readback(cg_backend *be, const uint32_t *src, uint32_t n, uint32_t seq);
// A few words from the host travel with the launch, as kernel arguments: n <= kUploadWords words to dst.
constexpr uint32_t kUploadWords = 64;
int launch_small_upload(cg_backend *be, uint32_t *dst, const uint32_t *host_words, uint32_t n);
int launch_fill_word(cg_backend *be, void *ptr, uint32_t bits);
// dst[i] = (uint32_t)src[i] << 16 : bfloat16 bit patterns widened to f32
int launch_bf16_widen(cg_backend *be, const void *src, void *dst, uint64_t n);
// binary16 bit patterns widened to f32
int launch_f16_widen(cg_backend *be, const void *src, void *dst, uint64_t n);
// n elements of format `fmt` widened to 32-bit words
int launch_widen(cg_backend *be, int fmt, const void *src, void *dst, uint64_t n);
// f32 words holding bfloat16 / binary16 values -> their 16-bit patterns (exact)
int launch_narrow16(cg_backend *be, cg_dtype dt, const void *src, void *dst, uint64_t n);
// fp8 (E4M3) bytes <-> 32-bit words holding the same values
int launch_f8_widen(cg_backend *be, const void *src, void *dst, uint64_t n);
int launch_narrow8(cg_backend *be, const void *src, void *dst, uint64_t n);
// out[outer, j, inner] = x[outer, idx[j], inner]
int launch_gather(cg_backend *be, const cg_tensor *x, int dim, const cg_tensor *idx, cg_tensor *out);

enum ReduceKind : int { kSum = 0, kMax = 1, kArgmax = 2 };
int launch_reduce(cg_backend *be, int kind, const cg_tensor *x, cg_tensor *out);
// Asks for the device address of the fixed scratch array of cg_argmax_rows_noalloc on `device` (once per device).
int noalloc_setup(int device);
int launch_topk(cg_backend *be, const cg_tensor *x, int64_t k, cg_tensor *vals, cg_tensor *idxs);
// *flag_dev = any(x > 0) / any(x != y)
int launch_any_positive(cg_backend *be, const cg_tensor *x);
int launch_any_diff(cg_backend *be, const cg_tensor *x, const cg_tensor *y);

// out == nullptr: nothing is launched; CG_OK if this product would run on the kernel that can round a narrow dtype's
// result in its store (then `out` may hold that dtype's format), kDeclined if not.
int launch_matmul(cg_backend *be, const cg_tensor *x, const cg_tensor *y, cg_tensor *out);

// The batch structure of x . y after collapsing: batch axes that both operands walk as one run
// are merged, a split axis contributes its two parts, and the innermost batch axis is folded
// into M when y ignores it and x walks it as more rows.  Reads shapes and strides only, so x
// may be a descriptor without memory.
constexpr int kDeclined = -1000; // "not my case": the caller takes the ordinary route
constexpr int kMaxBatchAxes = 6;
struct MmFold {
    int64_t M = 0, N = 0, K = 0, batch = 0;
    int64_t a_sm = 0, a_sk = 0, b_sk = 0, b_sn = 0;
    int nb = 0;                                  // collapsed batch axes
    int64_t bd[kMaxBatchAxes] = {0};             // extents, innermost first
    int64_t a_bs[kMaxBatchAxes] = {0}, b_bs[kMaxBatchAxes] = {0};
};
int fold_matmul(const cg_tensor *x, const cg_tensor *y, MmFold *f);
// Several skinny products x . ys[i] -> outs[i] (n of them, the same x) in one launch; kDeclined (declared
// below) when the shapes do not allow it.
// nf != null: x is the residual stream and the kernel applies the RMS norm to it on load (needs M <= 4 and K a
// multiple of 2048; kDeclined otherwise, before anything is launched).
int launch_matmul_gated(cg_backend *be, const cg_tensor *x, const cg_tensor *yg, const cg_tensor *yu, uint32_t one,
                        cg_tensor *out, const NormFuse *nf = nullptr);
int launch_prefill_attention(cg_backend *be, const Pending &p, const int64_t *pdims, int prank, const cg_tensor *q,
                             const cg_tensor *kt, const cg_tensor *v, cg_tensor *out);
int launch_fused_group(cg_backend *be, const cg_tensor *const *outs, const Pending *const *ps, int n);
// Writes that were put off so that they can share a launch (see DeferredWrite); every function
// that launches a kernel or copies device memory calls this first.
int flush_deferred(cg_backend *be, const Pending *also = nullptr);
// nterms: 2 (out = t0 + t1) or 4.  out is a contiguous view (any offset).  keep_sums: out is the whole of its buffer, which
// may then receive the partial sums of squares of the stored rows (Buffer::side).
int launch_matmul_residual(cg_backend *be, const cg_tensor *x, const cg_tensor *y, const uint32_t *const *terms, int nterms,
                           int slot, int order, cg_tensor *out, bool keep_sums);
int launch_matmul_group(cg_backend *be, const cg_tensor *x, const cg_tensor *const *ys, cg_tensor *const *outs, int n,
                        const NormFuse *nf = nullptr);
// Where the columns of a decode-time product go when the rotary embedding and the write into a KV cache (or into q's own
// buffer) run in the product's store: column n = head * hd + d of row b goes to dst[b * sb + head * sh + d], after
// out[d] = cos[d] * x[d] + sin[d] * rot[d], rot = concat(-x[hd/2..], x[..hd/2]) when `rope` (cos, sin: hd words each).
// hgamma: when set, every head of a row (hd columns) first goes through an RMS norm of its own, x / pow(sum(x * x) / n +
// eps, e) * hgamma[d] (the q / k norm of Qwen3, qwen3.rs:249-279): a workgroup then owns a whole head.
struct RopeStore {
    uint32_t *dst;
    int64_t sb, sh;
    const uint32_t *cos, *sin;
    uint32_t hd, rope;
    const uint32_t *hgamma;
    uint32_t hn_n_bits, hn_eps_bits, hn_exp_bits;
};
// The products x . ys[i] (one row per batch entry, the same x) with such a store each; kDeclined when the shapes are not
// the grouped kernel's.  nf as in launch_matmul_group.
int launch_matmul_group_rope(cg_backend *be, const cg_tensor *x, const cg_tensor *const *ys, const RopeStore *stores, int n,
                             const NormFuse *nf);

// Decode-time attention in one pass: out = softmax-program(q . kT) . v, where `p` is the deferred
// soft-max program whose leaf 0 is the (never computed) lazy product q . kT and (pdims, prank) its
// shape.  Returns kDeclined when the shapes or the program are not what the kernel handles; the
// caller then takes the ordinary route.
int launch_decode_attention(cg_backend *be, const Pending &p, const int64_t *pdims, int prank, const cg_tensor *q,
                            const cg_tensor *kt, const cg_tensor *v, cg_tensor *out);

} // namespace cg
