// Host runtime of libcatgrad_hip.so: backend lifetime, device pool, tensor handles,
// zero-copy view algebra, argument checking and the C ABI entry points.  Arithmetic
// lives in the kernel files (ew.hip, reduce.hip, matmul.hip).
//
// The semantics implemented here follow catgrad's NdArrayBackend
// (reference: catgrad/src/interpreter/backend/ndarray.rs); each entry point cites the
// lines it replaces.  Unlike that backend, transpose / slice / broadcast / reshape are
// views whenever strides allow, constants never touch device memory, and nothing
// copies a shared buffer before using it.
#include "common.hpp"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <vector>

namespace cg {

static thread_local std::string g_err;
static std::recursive_mutex g_lazy_mu; // guards lazy backing of uniform tensors and of deferred ones (computing one may compute another)
static int ensure_concrete(cg_tensor *t);
static int run_pending(cg_backend *be, const cg_tensor *dst, const Pending &p, bool fresh);

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

int hip_fail(hipError_t e, const char *what) {
    return fail(CG_ERR_DEVICE, "HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
}

// ---- pool -------------------------------------------------------------------------
size_t Pool::size_class(size_t bytes) {
    // 512 B minimum, then eight classes per octave: at most 12.5 % slack and few enough
    // distinct sizes that the growing shapes of a decode loop keep hitting the lists.
    if (bytes <= 512) return 512;
    int e = 63 - __builtin_clzll(bytes);
    size_t step = (size_t)1 << (e - 3);
    return (bytes + step - 1) & ~(step - 1);
}

int Pool::alloc(size_t bytes, void **ptr, size_t *cls) {
    size_t c = size_class(bytes);
    {
        std::lock_guard<std::mutex> lk(mu_);
        auto it = free_.lower_bound(c);
        if (it != free_.end() && it->first <= c + c / 4) {
            *ptr = it->second;
            *cls = it->first;
            cached_ -= it->first;
            in_use_ += it->first;
            free_.erase(it);
            return CG_OK;
        }
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, c);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        trim();
        e = hipMalloc(&p, c);
        if (e != hipSuccess) return hip_fail(e, "hipMalloc");
    }
    std::lock_guard<std::mutex> lk(mu_);
    in_use_ += c;
    *ptr = p;
    *cls = c;
    return CG_OK;
}

void Pool::free(void *ptr, size_t cls) {
    std::lock_guard<std::mutex> lk(mu_);
    free_.emplace(cls, ptr);
    in_use_ -= cls;
    cached_ += cls;
}

void Pool::trim() {
    std::multimap<size_t, void *> take;
    {
        std::lock_guard<std::mutex> lk(mu_);
        take.swap(free_);
        cached_ = 0;
    }
    for (auto &kv : take) (void)hipFree(kv.second);
}

void Pool::stats(size_t *in_use, size_t *cached) {
    std::lock_guard<std::mutex> lk(mu_);
    if (in_use) *in_use = in_use_;
    if (cached) *cached = cached_;
}

// ---- tensors ----------------------------------------------------------------------
bool is_contiguous(const cg_tensor *t) {
    if (numel(t) == 0) return true;
    if (t->split >= 0) return false;
    int64_t s = 1;
    for (int i = t->rank - 1; i >= 0; i--) {
        if (t->dims[i] != 1 && t->strides[i] != s) return false;
        s *= t->dims[i];
    }
    return true;
}

void drop_packed(Buffer *b) {
    if (!b) return;
    for (Buffer::Packed &p : b->packed) b->be->pool.free(p.ptr, p.cls); // stream-ordered: queued readers come first
    b->packed.clear();
}

static void buffer_release(Buffer *b) {
    while (b && b->rc.fetch_sub(1) == 1) {
        if (b->ptr) b->be->pool.free(b->ptr, b->cls);
        if (b->side) b->be->pool.free(b->side, b->side_cls);
        drop_packed(b);
        buffer_release(b->wide); // (a widened copy has none of its own: one level deep)
        Buffer *next = b->successor;
        delete b->rs;
        delete b;
        b = next; // drop the reference this buffer held on its successor
    }
}

Pending::Pending(const Pending &o)
    : nleaf(o.nleaf), ninstr(o.ninstr), expensive(o.expensive), nred(o.nred), rowlen(o.rowlen), reduced(o.reduced) {
    for (int l = 0; l < nleaf; l++) {
        leaf[l] = o.leaf[l];
        if (leaf[l].buf) leaf[l].buf->rc.fetch_add(1);
        if (leaf[l].buf2) leaf[l].buf2->rc.fetch_add(1);
        if (leaf[l].lazy) leaf[l].lazy->rc.fetch_add(1);
        if (leaf[l].lazy2) leaf[l].lazy2->rc.fetch_add(1);
    }
    for (int i = 0; i < ninstr; i++) ins[i] = o.ins[i];
}

Pending::~Pending() {
    for (int l = 0; l < nleaf; l++) {
        buffer_release(leaf[l].buf);
        buffer_release(leaf[l].buf2);
        lazy_mm_release(leaf[l].lazy);
        lazy_mm_release(leaf[l].lazy2);
    }
}

// Is x (still) the deferred program  h / pow(sum(h * h) / n + eps, e) * gamma  over the rows of a residual stream h
// [1..4 rows, K] whose kernel left the partial sums of squares (Buffer::side)?  Then a decode-time product can apply
// the norm while it loads h (K a multiple of 4 above 256) and the norm needs no launch.  Fills nf and the stand-in tensor
// h (a borrowed view of the leaf's buffer: set h->buf to null before it goes out of scope).
static bool norm_fuse_of(const cg_tensor *x, NormFuse *nf, cg_tensor *h) {
    static const uint8_t code[7][4] = {{kMul, 0, 0, 0},   {kRowSum, 8, 8, 8}, {kDiv, 9, 1, 9},  {kAdd, 10, 2, 10},
                                       {kPow, 11, 3, 11}, {kDiv, 0, 12, 0},   {kMul, 13, 4, 13}};
    const Pending *p = x->pend;
    if (!p || !x->be->aot || x->dt != CG_F32 || x->rank < 2 || x->split >= 0) return false;
    if (p->nleaf != 5 || p->ninstr != 7 || p->nred != 1 || p->reduced) return false;
    for (int i = 0; i < 7; i++)
        if (p->ins[i].op != code[i][0] || p->ins[i].a != code[i][1] || p->ins[i].b != code[i][2] || p->ins[i].c != code[i][3]) return false;
    const int r = x->rank;
    const int64_t K = x->dims[r - 1], rows = K > 0 ? numel(x) / K : 0;
    if (K <= 256 || K % 4 != 0 || rows < 1 || rows > 4 || p->rowlen != K) return false;
    const LeafView &lh = p->leaf[0], &lg = p->leaf[4];
    if (lh.uniform || lh.pw || lh.lazy || !lh.buf || !lh.buf->side || lh.offset != 0 || (int64_t)lh.buf->side_blocks * 4 != K) return false;
    if (is_narrow_buf(lh.buf) || is_narrow_buf(lg.buf)) return false; // (the kernels read 32-bit words)
    if (!p->leaf[1].uniform || !p->leaf[2].uniform || !p->leaf[3].uniform) return false;
    if (lg.uniform || lg.pw || lg.lazy || !lg.buf || lg.offset % 4 != 0) return false;
    int64_t st = 1;
    for (int d = r - 1; d >= 0; d--) { // h dense in the program's space, gamma along the last axis only
        if (x->dims[d] != 1 && lh.strides[d] != st) return false;
        if (x->dims[d] != 1 && lg.strides[d] != (d == r - 1 ? 1 : 0)) return false;
        st *= x->dims[d];
    }
    nf->partials = static_cast<const float *>(lh.buf->side);
    nf->blocks = lh.buf->side_blocks;
    nf->gamma = static_cast<const uint32_t *>(lg.buf->ptr) + lg.offset;
    nf->n_bits = p->leaf[1].ubits;
    nf->eps_bits = p->leaf[2].ubits;
    nf->exp_bits = p->leaf[3].ubits;
    h->be = x->be;
    h->buf = lh.buf;
    h->dt = CG_F32;
    h->rank = r;
    memcpy(h->dims, x->dims, sizeof h->dims);
    int64_t s2 = 1;
    for (int d = r - 1; d >= 0; d--) {
        h->strides[d] = s2;
        s2 *= x->dims[d];
    }
    h->offset = 0;
    return true;
}

// t0 + t1 with one term a decode-time product nobody has needed yet and of the extent that the products' residual
// store takes (the residual stream after an o or down projection): worth computing where it stands — the add runs
// in the product's store and the row sums of squares come with it — rather than carrying it into a longer program.
static bool residual_sum_open(const cg_tensor *x) {
    const Pending *p = x->pend;
    if (!p || !x->be->aot || x->dt != CG_F32 || p->nleaf != 2 || p->ninstr != 1 || p->nred != 0) return false;
    if (p->ins[0].op != kAdd || p->ins[0].a + p->ins[0].b != 1) return false;
    int open = 0;
    for (int l = 0; l < 2; l++) {
        const LeafView &lv = p->leaf[l];
        if (lv.uniform || lv.pw) return false;
        if (lv.lazy && !lv.lazy->result) {
            const LazyMm *m = lv.lazy;
            const int64_t N = m->rank > 0 ? m->dims[m->rank - 1] : 0;
            if (!m->groupable || m->head_norm || m->rc.load() != 1 || m->rank != x->rank || N < 512 || N >= 8192) return false;
            open++;
        } else if (!lv.lazy && !lv.buf) {
            return false;
        }
    }
    return open == 1;
}

static void lazy_mm_close(LazyMm *m) { // no longer open for grouping
    if (!m->be) return;
    auto &v = m->be->lazy_open;
    for (size_t i = 0; i < v.size(); i++)
        if (v[i] == m) {
            v[i] = v.back();
            v.pop_back();
            break;
        }
    m->be = nullptr;
}

void lazy_mm_release(LazyMm *m) {
    if (!m) return;
    if (m->rc.fetch_sub(1) == 1) {
        lazy_mm_close(m);
        release(m->x);
        release(m->y);
        buffer_release(m->result);
        buffer_release(m->hn_gamma);
        delete m->hn_prog;
        delete m;
    }
}

int lazy_mm_force(cg_backend *be, LazyMm *m) {
    if (m->result) return CG_OK;
    if (m->head_norm) {
        // nobody took it with the norm in the store: the plain product, then the kept norm program over it
        lazy_mm_close(m);
        if (m->x->pend) {
            int xrc = ensure_concrete(m->x);
            if (xrc) return xrc;
        }
        cg_tensor *raw = nullptr, *o = nullptr;
        int rc = new_dense(be, CG_F32, m->dims, m->rank, &raw);
        if (!rc) rc = launch_matmul(be, m->x, m->y, raw);
        if (!rc) rc = new_dense(be, CG_F32, m->hn_dims, m->hn_rank, &o);
        if (!rc) {
            LeafView &l0 = m->hn_prog->leaf[0];
            buffer_release(l0.buf);
            l0.buf = raw->buf;
            l0.buf->rc.fetch_add(1);
            rc = run_pending(be, o, *m->hn_prog, true);
        }
        if (!rc) {
            m->result = o->buf;
            o->buf = nullptr;
        }
        release(o);
        release(raw);
        return rc;
    }
    if (m->groupable && m->be) {
        // the other open products with the same left operand go along in the same launch
        LazyMm *grp[4] = {m};
        int n = 1;
        for (LazyMm *o : be->lazy_open)
            if (o != m && !o->result && !o->head_norm && o->x == m->x && n < 4) grp[n++] = o;
        NormFuse nf;
        cg_tensor h;
        const bool normed = m->x->pend && norm_fuse_of(m->x, &nf, &h);
        if (n > 1 || normed) {
            cg_tensor *outs[4] = {nullptr, nullptr, nullptr, nullptr};
            const cg_tensor *ys[4];
            int rc = CG_OK;
            for (int i = 0; i < n && !rc; i++) {
                ys[i] = grp[i]->y;
                rc = new_dense(be, CG_F32, grp[i]->dims, grp[i]->rank, &outs[i]);
            }
            if (!rc && normed) rc = launch_matmul_group(be, &h, ys, outs, n, &nf); // the norm runs in the products' loads
            h.buf = nullptr;
            if (!rc && normed) be->programs_compiled++;
            if ((!rc && !normed) || (normed && rc == kDeclined)) {
                rc = m->x->pend ? ensure_concrete(m->x) : CG_OK;
                if (!rc) rc = n > 1 ? launch_matmul_group(be, m->x, ys, outs, n) : kDeclined;
            }
            if (rc == CG_OK)
                for (int i = 0; i < n; i++) {
                    grp[i]->result = outs[i]->buf;
                    outs[i]->buf = nullptr;
                    lazy_mm_close(grp[i]);
                }
            for (int i = 0; i < n; i++) release(outs[i]);
            if (rc != kDeclined) return rc;
        }
    }
    lazy_mm_close(m);
    if (m->x->pend) { // a left operand still deferred (see norm_fuse_of): this launch takes it from memory
        int xrc = ensure_concrete(m->x);
        if (xrc) return xrc;
    }
    cg_tensor *o;
    int rc = new_dense(be, CG_F32, m->dims, m->rank, &o);
    if (rc) return rc;
    rc = launch_matmul(be, m->x, m->y, o);
    if (!rc) {
        m->result = o->buf;
        o->buf = nullptr;
    }
    release(o);
    return rc;
}

// Every handle that can leave the library is counted in its backend: the backend's memory pool, stream and lock
// outlive cg_backend_destroy for as long as such a handle exists (see there).
static cg_tensor *alloc_tensor(cg_backend *be) {
    cg_tensor *t = new cg_tensor;
    t->be = be;
    be->live_tensors.fetch_add(1, std::memory_order_relaxed);
    return t;
}

void release(cg_tensor *t) {
    if (!t) return;
    if (t->rc.fetch_sub(1) == 1) {
        cg_backend *be = t->be;
        buffer_release(t->buf);
        delete t->pend;
        delete t;
        be->live_tensors.fetch_sub(1, std::memory_order_relaxed);
    }
}

static void set_row_major(cg_tensor *t) {
    int64_t s = 1;
    for (int i = t->rank - 1; i >= 0; i--) {
        t->strides[i] = s;
        s *= t->dims[i];
    }
}

int new_dense(cg_backend *be, cg_dtype dt, const int64_t *dims, int rank, cg_tensor **out, int64_t reserve_elems, int fmt) {
    cg_tensor *t = alloc_tensor(be);
    t->be = be;
    t->dt = dt;
    t->rank = rank;
    for (int i = 0; i < rank; i++) t->dims[i] = dims[i];
    set_row_major(t);
    int64_t n = numel(t);
    if (n > 0) {
        Buffer *b = new Buffer;
        b->be = be;
        int rc = be->pool.alloc((size_t)(n > reserve_elems ? n : reserve_elems) * fmt_bytes(fmt), &b->ptr, &b->cls);
        if (rc) {
            delete b;
            delete t;
            be->live_tensors.fetch_sub(1, std::memory_order_relaxed);
            return rc;
        }
        b->elems = n;
        b->fmt = fmt;
        t->buf = b;
    }
    *out = t;
    return CG_OK;
}

cg_tensor *new_uniform(cg_backend *be, cg_dtype dt, const int64_t *dims, int rank, uint32_t bits) {
    cg_tensor *t = alloc_tensor(be);
    t->be = be;
    t->dt = dt;
    t->rank = rank;
    for (int i = 0; i < rank; i++) {
        t->dims[i] = dims[i];
        t->strides[i] = 0;
    }
    t->uniform = true;
    t->ubits = bits;
    return t;
}

cg_tensor *new_view(const cg_tensor *t) {
    cg_tensor *v = alloc_tensor(t->be);
    v->be = t->be;
    v->buf = t->buf;
    if (v->buf) v->buf->rc.fetch_add(1);
    v->dt = t->dt;
    v->rank = t->rank;
    memcpy(v->dims, t->dims, sizeof v->dims);
    memcpy(v->strides, t->strides, sizeof v->strides);
    v->offset = t->offset;
    v->uniform = t->uniform;
    v->ubits = t->ubits;
    v->split = t->split;
    v->split_inner = t->split_inner;
    v->split_os = t->split_os;
    return v;
}

int result_fmt(const cg_backend *be, cg_dtype dt, int64_t n) {
    return be->narrow_storage && is_narrow(dt) && n >= be->narrow_from ? fmt_of(dt) : kFmtWords;
}

// The words of a narrow buffer: its widened copy, made now if nobody needed it before.
static int wide_of(Buffer *b, Buffer **out) {
    std::lock_guard<std::recursive_mutex> lk(g_lazy_mu);
    if (!b->wide) {
        Buffer *w = new Buffer;
        w->be = b->be;
        int rc = b->be->pool.alloc((size_t)b->elems * 4, &w->ptr, &w->cls);
        if (!rc) rc = launch_widen(b->be, b->fmt, b->ptr, w->ptr, (uint64_t)b->elems);
        if (rc) {
            buffer_release(w);
            return rc;
        }
        w->elems = b->elems;
        w->constant = b->constant;
        b->wide = w;
    }
    *out = b->wide;
    return CG_OK;
}

// The handle's view moves from a narrow buffer to that buffer's widened copy (the values stay; every holder of the handle
// sees it).  For the paths that go on writing into the buffer behind a tensor.
static int make_words(cg_tensor *t) {
    if (t->pend || !is_narrow_buf(t->buf)) return CG_OK;
    std::lock_guard<std::recursive_mutex> lk(g_lazy_mu);
    Buffer *w;
    int rc = wide_of(t->buf, &w);
    if (rc) return rc;
    w->rc.fetch_add(1);
    Buffer *old = t->buf;
    t->buf = w;
    if (old->rc.load() == 1) { // nobody else sees the narrow buffer: the copy is the handle's alone from here on
        old->wide = nullptr;
        w->rc.fetch_sub(1);
    }
    buffer_release(old);
    return CG_OK;
}

int device_ptr_fmt(const cg_tensor *t, const void **ptr, int *fmt) {
    if (t->buf && !t->pend && t->buf->fmt != kFmtWords) {
        *fmt = t->buf->fmt;
        *ptr = static_cast<const char *>(t->buf->ptr) + t->offset * (int64_t)fmt_bytes(t->buf->fmt);
        return CG_OK;
    }
    *fmt = kFmtWords;
    return device_ptr(t, ptr);
}

int device_ptr(const cg_tensor *t, const void **ptr) {
    if (t->pend) return fail(CG_ERR_ARG, "internal error: address of a deferred tensor requested");
    if (t->buf && t->buf->fmt != kFmtWords) {
        Buffer *w;
        int rc = wide_of(t->buf, &w);
        if (rc) return rc;
        *ptr = static_cast<const char *>(w->ptr) + t->offset * 4;
        return CG_OK;
    }
    if (!t->buf) {
        if (!t->uniform || numel(t) == 0) {
            *ptr = nullptr;
            return CG_OK;
        }
        std::lock_guard<std::recursive_mutex> lk(g_lazy_mu);
        if (!t->buf) {
            Buffer *b = new Buffer;
            b->be = t->be;
            int rc = t->be->pool.alloc(4, &b->ptr, &b->cls);
            if (rc) {
                delete b;
                return rc;
            }
            rc = launch_fill_word(t->be, b->ptr, t->ubits);
            if (rc) {
                buffer_release(b);
                return rc;
            }
            const_cast<cg_tensor *>(t)->buf = b;
        }
    }
    *ptr = static_cast<const char *>(t->buf->ptr) + t->offset * 4;
    return CG_OK;
}

FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    uint32_t l = 0;
    while (l < 32 && ((uint64_t)1 << l) < d) l++;
    f.m = (uint32_t)((((uint64_t)1 << 32) * (((uint64_t)1 << l) - d)) / d + 1);
    f.s1 = l < 1 ? l : 1;
    f.s2 = l > 0 ? l - 1 : 0;
    return f;
}

int plan_views(const int64_t *vdims, int vrank, const ViewDesc *v, int n, bool keep_last_axis, EwGeom *g,
               Operand *ops, bool allow_vec4, bool allow_vec8) {
    int r = 0;
    int64_t dims[kMaxRank];
    int64_t st[kMaxViews + 1][kMaxRank];
    bool last_kept = false;
    for (int i = 0; i < vrank; i++) {
        const bool is_last = i == vrank - 1;
        if (vdims[i] == 1 && !(keep_last_axis && is_last)) continue;
        dims[r] = vdims[i];
        for (int k = 0; k < n; k++) st[k][r] = v[k].uniform ? 0 : v[k].strides[i];
        if (is_last) last_kept = true;
        r++;
    }
    (void)last_kept;
    // merge axis i+1 into axis i when every operand steps through them as one run
    int w = 0;
    for (int i = 0; i < r; i++) {
        const bool protect = keep_last_axis && i == r - 1;
        if (w > 0 && !protect) {
            bool ok = true;
            for (int k = 0; k < n && ok; k++) ok = st[k][w - 1] == st[k][i] * dims[i];
            if (ok) {
                dims[w - 1] *= dims[i];
                for (int k = 0; k < n; k++) st[k][w - 1] = st[k][i];
                continue;
            }
        }
        dims[w] = dims[i];
        for (int k = 0; k < n; k++) st[k][w] = st[k][i];
        w++;
    }
    r = w;
    if (r == 0) {
        r = 1;
        dims[0] = 1;
        for (int k = 0; k < n; k++) st[k][0] = 1;
    }
    for (int i = 0; i < r; i++)
        if (dims[i] > 0xFFFFFFFFll) return fail(CG_ERR_UNSUPPORTED, "axis extent above 2^32-1 elements");
    int64_t inner = dims[r - 1];
    bool vec4 = allow_vec4 && inner % 4 == 0;
    bool vec8 = allow_vec4 && allow_vec8 && inner % 8 == 0, any_narrow = false;
    for (int k = 0; k < n; k++) {
        Operand &o = ops[k];
        memset(&o, 0, sizeof o);
        o.uniform = v[k].uniform ? 1u : 0u;
        o.ubits = v[k].ubits;
        o.ptr = v[k].uniform ? nullptr : v[k].ptr;
        o.is = st[k][r - 1];
        o.fmt = v[k].uniform ? (uint32_t)kFmtWords : (uint32_t)v[k].fmt;
        for (int d = 0; d < r - 1; d++) o.os[d] = st[k][r - 2 - d];
        if (v[k].vec_period > 0 && v[k].vec_period % 4) vec4 = false;
        if (v[k].vec_period > 0 && v[k].vec_period % 8) vec8 = false;
        if (!o.uniform && o.is == 1) {
            const size_t eb = fmt_bytes((int)o.fmt);
            any_narrow = any_narrow || o.fmt != kFmtWords;
            if (reinterpret_cast<uintptr_t>(o.ptr) % (4 * eb)) vec4 = false; // four elements per access
            // eight: one access of 16 (16-bit formats) or 8 bytes (fp8), two of 16 bytes for words
            if (reinterpret_cast<uintptr_t>(o.ptr) % (eb == 4 ? 16 : 8 * eb)) vec8 = false;
            for (int d = 0; d < r - 1; d++) {
                if (o.os[d] % 4) vec4 = false;
                if (o.os[d] % (eb == 4 ? 4 : 8)) vec8 = false;
            }
        }
    }
    vec8 = vec8 && vec4 && any_narrow;
    g->nouter = (uint32_t)(r - 1);
    g->inner = (uint32_t)inner;
    g->vec = vec8 ? 8 : vec4 ? 4 : 1;
    g->ipr = (uint32_t)(inner / g->vec);
    g->ipr_div = make_fastdiv(g->ipr ? g->ipr : 1);
    uint64_t total = g->ipr;
    for (int d = 0; d < r - 1; d++) {
        g->od[d] = (uint32_t)dims[r - 2 - d];
        g->odiv[d] = make_fastdiv(g->od[d]);
        total *= g->od[d];
    }
    if (total > 0xFFFFFFFFull) return fail(CG_ERR_UNSUPPORTED, "element-wise launch above 2^32-1 work items");
    g->total = total;
    return CG_OK;
}

int plan_elementwise(const cg_tensor *const *views, int n, EwGeom *g, Operand *ops, bool allow_vec8) {
    ViewDesc v[kMaxViews];
    for (int k = 0; k < n; k++) {
        v[k].strides = views[k]->strides;
        v[k].uniform = views[k]->uniform;
        v[k].ubits = views[k]->ubits;
        v[k].ptr = nullptr;
        v[k].fmt = kFmtWords;
        if (!views[k]->uniform) {
            const void *p;
            int rc = device_ptr_fmt(views[k], &p, &v[k].fmt);
            if (rc) return rc;
            v[k].ptr = static_cast<const char *>(p);
        }
    }
    return plan_views(views[0]->dims, views[0]->rank, v, n, false, g, ops, true, allow_vec8);
}

// ---- launch timing ---------------------------------------------------------------------
constexpr size_t kProfMaxPending = 16384;

ProfScope::ProfScope(cg_backend *be, int cls, double work) : be_(be) {
    ProfClass &c = be->prof[cls];
    if (!c.every) return;
    if (c.seen++ % c.every) return;
    if (be->prof_pending.size() >= kProfMaxPending) return;
    ProfPending p;
    if (!be->prof_free.empty()) {
        p.a = be->prof_free.back().first;
        p.b = be->prof_free.back().second;
        be->prof_free.pop_back();
    } else {
        if (hipEventCreate(&p.a) != hipSuccess) return;
        if (hipEventCreate(&p.b) != hipSuccess) {
            (void)hipEventDestroy(p.a);
            return;
        }
    }
    p.cls = cls;
    p.work = work;
    (void)hipEventRecord(p.a, be->stream);
    be->prof_pending.push_back(p);
    slot_ = (int)be->prof_pending.size() - 1;
}

ProfScope::~ProfScope() {
    if (slot_ >= 0) (void)hipEventRecord(be_->prof_pending[slot_].b, be_->stream);
}

// Call only after the stream has been synchronised.
void prof_drain(cg_backend *be) {
    for (ProfPending &p : be->prof_pending) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, p.a, p.b) == hipSuccess) {
            ProfClass &c = be->prof[p.cls];
            c.timed++;
            c.ms += ms;
            c.work += p.work;
        } else {
            (void)hipGetLastError();
        }
        be->prof_free.emplace_back(p.a, p.b);
    }
    be->prof_pending.clear();
}

double distinct_bytes(const cg_tensor *t) {
    if (t->uniform) return 0.0;
    double n = 1.0;
    for (int i = 0; i < t->rank; i++)
        if (t->strides[i] != 0 || t->dims[i] <= 1) n *= (double)t->dims[i];
    return (double)fmt_bytes(t->buf && !t->pend ? t->buf->fmt : kFmtWords) * n;
}

// ---- helpers for the entry points -------------------------------------------------------
struct Consume { // the consumed reference of a tensor argument (move semantics of the ABI)
    cg_tensor *t;
    explicit Consume(cg_tensor *t) : t(t) {}
    ~Consume() { release(t); }
};

static const char *kTodo = "unknown dtype";
static bool supported(cg_dtype d) { return d == CG_F32 || d == CG_U32 || d == CG_F16 || d == CG_BF16 || d == CG_F8; }
// bytes of one element at the boundary (from_vec / to_vec)
static size_t host_bytes(cg_dtype d) { return d == CG_F8 ? 1 : is_half(d) ? 2 : 4; }

// The 16-bit float dtypes on the host (constants that never reach the device): widening of a bit pattern
// and rounding of an f32 to the nearest representable value (ties to even), both as f32 bits.
static uint32_t widen16_host(cg_dtype dt, uint16_t h) {
    if (dt == CG_BF16) return (uint32_t)h << 16;
    _Float16 v;
    memcpy(&v, &h, 2);
    float f = (float)v;
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static uint32_t round16_host(cg_dtype dt, uint32_t u) {
    if (dt == CG_BF16) {
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u | 0x00400000u) & 0xFFFF0000u;
        return (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
    }
    float f;
    memcpy(&f, &u, 4);
    f = (float)(_Float16)f;
    memcpy(&u, &f, 4);
    return u;
}
static uint16_t narrow16_host(cg_dtype dt, uint32_t u) {
    if (dt == CG_BF16) return (uint16_t)(u >> 16);
    float f;
    memcpy(&f, &u, 4);
    _Float16 v = (_Float16)f;
    uint16_t h;
    memcpy(&h, &v, 2);
    return h;
}

// fp8 = E4M3 on the host, as round_f8_bits / f8_byte_of / f8_word_of do it on the device
static uint32_t round8_host(uint32_t u) {
    const uint32_t sign = u & 0x80000000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7FC00000u;
    if (a >= 0x43E00000u) return sign | 0x43E00000u;
    if (a < 0x3C800000u) {
        float f;
        memcpy(&f, &a, 4);
        f = nearbyintf(f * 512.0f) * (1.0f / 512.0f);
        uint32_t r;
        memcpy(&r, &f, 4);
        return sign | r;
    }
    const uint32_t r = (a + 0x7FFFFu + ((a >> 20) & 1u)) & 0xFFF00000u;
    return sign | (r > 0x43E00000u ? 0x43E00000u : r);
}
static uint32_t widen8_host(uint8_t b) {
    const uint32_t sign = (uint32_t)(b & 0x80u) << 24, e = (b >> 3) & 0xFu, m = b & 7u;
    if (e == 0xFu && m == 7u) return sign | 0x7FC00000u;
    if (e != 0) return sign | ((e + 120u) << 23) | (m << 20);
    const float f = (float)m * (1.0f / 512.0f);
    uint32_t r;
    memcpy(&r, &f, 4);
    return sign | r;
}
static uint8_t narrow8_host(uint32_t u) {
    const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7Fu;
    if (a >= 0x3C800000u) return sign | (uint8_t)((((a >> 23) - 120u) << 3) | ((a >> 20) & 7u));
    float f;
    memcpy(&f, &a, 4);
    return sign | (uint8_t)(uint32_t)(f * 512.0f);
}
// a constant's value rounded to a narrow dtype
static uint32_t round_host(cg_dtype dt, uint32_t u) { return dt == CG_F8 ? round8_host(u) : is_half(dt) ? round16_host(dt, u) : u; }

static bool same_shape(const cg_tensor *a, const cg_tensor *b) {
    if (a->rank != b->rank) return false;
    for (int i = 0; i < a->rank; i++)
        if (a->dims[i] != b->dims[i]) return false;
    return true;
}

static int wait_and_check(cg_backend *be) {
    CG_HIP(hipStreamSynchronize(be->stream));
    if (!be->prof_pending.empty()) prof_drain(be);
    uint32_t f = *reinterpret_cast<volatile uint32_t *>(be->fault_host);
    if (f) {
        *reinterpret_cast<volatile uint32_t *>(be->fault_host) = 0;
        if (f & kFaultIndexRange) return fail(CG_ERR_RANGE, "index: index out of bounds (detected on device)");
        if (f & kFaultDivZero) return fail(CG_ERR_RANGE, "attempt to divide by zero (detected on device)");
    }
    return CG_OK;
}

// The read-back kernel with sequence number `seq` has run (and with it everything before it on the stream): polls the word
// it writes last.  Launch timings that wait to be read need the stream itself; so does a device that does not answer
// within a tenth of a second (a fault: the stream's own wait reports it).
static int wait_for_readback(cg_backend *be, uint32_t seq) {
    if (be->prof_pending.size() > 2048) return wait_and_check(be);
    volatile uint32_t *word = be->rb_host + kReadbackWords;
    const auto t0 = std::chrono::steady_clock::now();
    for (uint32_t spins = 0; *word != seq; spins++) {
        if ((spins & 1023) == 1023 && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(100)) return wait_and_check(be);
        __builtin_ia32_pause();
    }
    std::atomic_thread_fence(std::memory_order_acquire);
    uint32_t f = *reinterpret_cast<volatile uint32_t *>(be->fault_host);
    if (f) {
        *reinterpret_cast<volatile uint32_t *>(be->fault_host) = 0;
        if (f & kFaultIndexRange) return fail(CG_ERR_RANGE, "index: index out of bounds (detected on device)");
        if (f & kFaultDivZero) return fail(CG_ERR_RANGE, "attempt to divide by zero (detected on device)");
    }
    return CG_OK;
}

// fresh: dst is the whole of a buffer allocated for this very result (nothing else lives in it).
static int run_pending(cg_backend *be, const cg_tensor *dst, const Pending &p, bool fresh);
static int run_pending(cg_backend *be, const cg_tensor *dst, const Pending &p) { return run_pending(be, dst, p, false); }

// Row-major copy of a view (the materialising half of reshape / to_vec).
static int materialize(cg_backend *be, const cg_tensor *x, cg_tensor **out) {
    cg_tensor *o;
    // a copy of a view of a narrow buffer keeps the buffer's format (whatever dtype tags the view); a program without row
    // reductions stores the format of its dtype
    int fmt = kFmtWords;
    if (x->pend) fmt = x->pend->nred == 0 ? result_fmt(be, x->dt, numel(x)) : kFmtWords;
    else if (is_narrow_buf(x->buf) && be->narrow_storage && numel(x) >= be->narrow_from) fmt = x->buf->fmt;
    else if (x->buf) fmt = result_fmt(be, x->dt, numel(x));
    int rc = new_dense(be, x->dt, x->dims, x->rank, &o, 0, fmt);
    if (rc) return rc;
    if (numel(x) > 0 && x->split >= 0) {
        // copy through the physical (rank + 1) shape: the split axis becomes two axes on both sides
        cg_tensor src, dst;
        const int a = x->split, r = x->rank;
        src.be = dst.be = be;
        src.buf = x->buf;
        dst.buf = o->buf;
        src.dt = dst.dt = x->dt;
        src.rank = dst.rank = r + 1;
        src.offset = x->offset;
        for (int i = 0, j = 0; i < r; i++) {
            if (i == a) {
                src.dims[j] = dst.dims[j] = x->dims[i] / x->split_inner;
                src.strides[j] = x->split_os;
                dst.strides[j] = o->strides[i] * x->split_inner;
                j++;
                src.dims[j] = dst.dims[j] = x->split_inner;
                src.strides[j] = x->strides[i];
                dst.strides[j] = o->strides[i];
                j++;
            } else {
                src.dims[j] = dst.dims[j] = x->dims[i];
                src.strides[j] = x->strides[i];
                dst.strides[j] = o->strides[i];
                j++;
            }
        }
        const cg_tensor *ins[1] = {&src};
        rc = launch_elementwise(be, kCopy, x->dt, &dst, ins, 1);
        src.buf = dst.buf = nullptr;
        if (rc) {
            release(o);
            return rc;
        }
    } else if (numel(x) > 0) {
        const cg_tensor *ins[1] = {x};
        rc = x->pend ? run_pending(be, o, *x->pend, true) : launch_elementwise(be, kCopy, x->dt, o, ins, 1);
        if (rc) {
            release(o);
            return rc;
        }
    }
    *out = o;
    return CG_OK;
}

// numpy-style "reshape without copying": new strides for `dims` if the view allows it.
static bool try_view_reshape(const int64_t *xdims, const int64_t *xstrides, int xrank, const int64_t *dims, int rank,
                             int64_t *strides) {
    int64_t od[kMaxRank], os[kMaxRank];
    int on = 0;
    for (int i = 0; i < xrank; i++)
        if (xdims[i] != 1) {
            od[on] = xdims[i];
            os[on] = xstrides[i];
            on++;
        }
    int oi = 0, ni = 0;
    while (ni < rank && oi < on) {
        int64_t np = dims[ni], op = od[oi];
        int oj = oi + 1, nj = ni + 1;
        while (np != op) {
            if (np < op) {
                if (nj >= rank) return false;
                np *= dims[nj++];
            } else {
                if (oj >= on) return false;
                op *= od[oj++];
            }
        }
        for (int k = oi; k < oj - 1; k++)
            if (os[k] != os[k + 1] * od[k + 1]) return false;
        int64_t s = os[oj - 1];
        for (int k = nj - 1; k >= ni; k--) {
            strides[k] = s;
            s *= dims[k];
        }
        oi = oj;
        ni = nj;
    }
    if (oi < on) return false;
    for (; ni < rank; ni++) {
        if (dims[ni] != 1) return false;
        strides[ni] = 0;
    }
    return true;
}

// ---- deferred element-wise expressions (see common.hpp) ---------------------------------
static bool is_expensive(int op) { return op == kPow || op == kExp || op == kLog || op == kSin || op == kCos; }
// Cheap enough to evaluate once per consumer instead of being written out and re-read.
static bool cheap(const Pending *p) { return !p->expensive && p->nred == 0 && p->ninstr <= 4 && p->nleaf <= 3; }

static void leaf_as_tensor(const Pending &p, int l, const cg_tensor *shape_of, cg_dtype dt, cg_tensor *t) {
    const LeafView &lv = p.leaf[l];
    t->be = shape_of->be;
    t->buf = lv.buf;
    t->dt = dt;
    t->rank = shape_of->rank;
    memcpy(t->dims, shape_of->dims, sizeof t->dims);
    memcpy(t->strides, lv.strides, sizeof t->strides);
    t->offset = lv.offset;
    t->uniform = lv.uniform;
    t->ubits = lv.ubits;
}

// Runs the program of `p` into `dst` (a dense or strided view of p's shape).  A single
// instruction goes to the specialised single-op kernel.
// Lazy products among the leaves are computed now and become ordinary buffer leaves.
static int resolve_lazy_leaves(cg_backend *be, const Pending &cp) {
    Pending &p = const_cast<Pending &>(cp); // a cache fill: the value of the program does not change
    for (int l = 0; l < p.nleaf; l++) {
        LeafView &lv = p.leaf[l];
        if (lv.lazy) {
            int rc = lazy_mm_force(be, lv.lazy);
            if (rc) return rc;
            lv.buf = lv.lazy->result;
            lv.buf->rc.fetch_add(1);
            lazy_mm_release(lv.lazy);
            lv.lazy = nullptr;
        }
        if (lv.lazy2) {
            int rc = lazy_mm_force(be, lv.lazy2);
            if (rc) return rc;
            lv.buf2 = lv.lazy2->result;
            lv.buf2->rc.fetch_add(1);
            lazy_mm_release(lv.lazy2);
            lv.lazy2 = nullptr;
        }
    }
    return CG_OK;
}

// g * (1 / (c + exp(-g))) * u where g and u are open products of the same left operand that nobody
// else holds (gate and up projection of an MLP block): one launch that never writes g and u.
static int try_gated_pair(cg_backend *be, const cg_tensor *dst, const Pending &p) {
    static const uint8_t code[6][3] = {{kNeg, 0, 0}, {kExp, 8, 8}, {kAdd, 1, 9}, {kDiv, 1, 10}, {kMul, 0, 11}, {kMul, 12, 2}};
    if (p.nleaf != 3 || p.ninstr != 6 || p.nred != 0 || !is_contiguous(dst) || dst->dt != CG_F32) return kDeclined;
    for (int i = 0; i < 6; i++) {
        const Instr &in = p.ins[i];
        if (in.op != code[i][0] || in.a != code[i][1] || (i >= 2 && in.b != code[i][2])) return kDeclined;
    }
    const LeafView &lg = p.leaf[0], &lc = p.leaf[1], &lu = p.leaf[2];
    if (!lc.uniform || lg.uniform || lu.uniform || lg.pw || lu.pw || !lg.lazy || !lu.lazy || lg.lazy == lu.lazy) return kDeclined;
    LazyMm *mg = lg.lazy, *mu = lu.lazy;
    if (mg->result || mu->result || mg->head_norm || mu->head_norm || !mg->groupable || !mu->groupable || mg->x != mu->x || mg->rc.load() != 1 ||
        mu->rc.load() != 1 || mg->rank != dst->rank || mu->rank != dst->rank)
        return kDeclined;
    // both leaves are the whole products, read in place
    int64_t st = 1;
    for (int d = dst->rank - 1; d >= 0; d--) {
        if (mg->dims[d] != dst->dims[d] || mu->dims[d] != dst->dims[d]) return kDeclined;
        if (dst->dims[d] != 1 && (lg.strides[d] != st || lu.strides[d] != st)) return kDeclined;
        st *= dst->dims[d];
    }
    if (lg.offset != 0 || lu.offset != 0) return kDeclined;
    int rc = kDeclined;
    {
        NormFuse nf;
        cg_tensor h;
        if (mg->x->pend && norm_fuse_of(mg->x, &nf, &h)) { // the norm runs in the products' loads
            rc = launch_matmul_gated(be, &h, mg->y, mu->y, lc.ubits, const_cast<cg_tensor *>(dst), &nf);
            if (rc == CG_OK) be->programs_compiled++;
        }
        h.buf = nullptr;
    }
    if (rc == kDeclined) {
        if (mg->x->pend) {
            int xrc = ensure_concrete(mg->x);
            if (xrc) return xrc;
        }
        rc = launch_matmul_gated(be, mg->x, mg->y, mu->y, lc.ubits, const_cast<cg_tensor *>(dst));
    }
    if (rc == CG_OK) {
        lazy_mm_close(mg);
        lazy_mm_close(mu);
        be->programs_compiled++;
    }
    return rc;
}

// A sum of four dense terms, one of them a product nobody has needed yet (the residual stream after the
// o or down projection): the adds run in the product's store.
// fresh: dst is a whole new buffer, so the row sums of squares of what is stored may be kept with it.
static int try_residual_store(cg_backend *be, const cg_tensor *dst, const Pending &p, bool fresh) {
    static const uint8_t orders[2][3][2] = {{{1, 2}, {0, 8}, {9, 3}}, {{1, 2}, {8, 3}, {0, 9}}};
    if (p.nred != 0 || !is_contiguous(dst) || dst->dt != CG_F32) return kDeclined;
    int order = -1;
    const int nterms = p.nleaf;
    if (p.nleaf == 2 && p.ninstr == 1) { // t0 + t1, either way round
        if (p.ins[0].op != kAdd || p.ins[0].a + p.ins[0].b != 1) return kDeclined;
        order = 0;
    } else if (p.nleaf == 4 && p.ninstr == 3) {
        for (int o = 0; o < 2 && order < 0; o++) {
            bool same = true;
            for (int i = 0; i < 3; i++) same = same && p.ins[i].op == kAdd && p.ins[i].a == orders[o][i][0] && p.ins[i].b == orders[o][i][1];
            if (same) order = o;
        }
    }
    if (order < 0) return kDeclined;
    int slot = -1;
    const uint32_t *terms[4] = {nullptr, nullptr, nullptr, nullptr};
    for (int l = 0; l < nterms; l++) {
        const LeafView &lv = p.leaf[l];
        if (lv.uniform || lv.pw || lv.offset % 4 != 0) return kDeclined;
        int64_t st = 1;
        for (int d = dst->rank - 1; d >= 0; d--) { // the term is read in place, element for element
            if (dst->dims[d] != 1 && lv.strides[d] != st) return kDeclined;
            st *= dst->dims[d];
        }
        if (lv.lazy && !lv.lazy->result) {
            LazyMm *m = lv.lazy;
            if (slot >= 0 || !m->groupable || m->head_norm || m->rc.load() != 1 || lv.offset != 0 || m->rank != dst->rank) return kDeclined;
            for (int d = 0; d < dst->rank; d++)
                if (m->dims[d] != dst->dims[d]) return kDeclined;
            for (LazyMm *o : be->lazy_open)
                if (o != m && !o->result && o->x == m->x) return kDeclined; // it belongs to a group
            slot = l;
        } else {
            const Buffer *b = lv.lazy ? lv.lazy->result : lv.buf;
            if (!b || is_narrow_buf(b)) return kDeclined;
            terms[l] = static_cast<const uint32_t *>(b->ptr) + lv.offset;
        }
    }
    if (slot < 0) return kDeclined;
    LazyMm *m = p.leaf[slot].lazy;
    if (m->x->pend) { // a left operand still deferred (see norm_fuse_of): this launch takes it from memory
        int xrc = ensure_concrete(m->x);
        if (xrc) return xrc;
    }
    int rc = launch_matmul_residual(be, m->x, m->y, terms, nterms, slot, order, const_cast<cg_tensor *>(dst), fresh && dst->offset == 0);
    if (rc == CG_OK) {
        lazy_mm_close(m);
        be->programs_compiled++;
    }
    return rc;
}

static int run_pending(cg_backend *be, const cg_tensor *dst, const Pending &p, bool fresh) {
    if (!fresh) drop_packed(dst->buf); // a part of a buffer that may have been multiplied before is about to change
    const bool narrow_dst = is_narrow_buf(dst->buf);
    if (narrow_dst && p.nred > 0) return fail(CG_ERR_ARG, "internal error: a narrow buffer written by a kernel that stores words");
    if (be->aot && !narrow_dst) {
        int grc = try_gated_pair(be, dst, p);
        if (grc == kDeclined) grc = try_residual_store(be, dst, p, fresh);
        if (grc != kDeclined) return grc;
    }
    {
        int lrc = resolve_lazy_leaves(be, p);
        if (lrc) return lrc;
    }
    if (p.nred > 0) {
        // the iteration space: dst's shape, with the row restored when dst holds one value per row
        cg_tensor space;
        space.rank = dst->rank;
        memcpy(space.dims, dst->dims, sizeof space.dims);
        if (p.reduced) space.dims[space.rank - 1] = p.rowlen;
        const Instr last = p.ins[p.ninstr - 1];
        if (p.reduced && p.nred == 1 && is_row_reduce(last.op) && is_contiguous(dst)) {
            // a lone reduction: the dedicated reduction kernels
            const int kind = (last.op & ~kInstrU32) == kRowMax ? kMax : kSum;
            const bool f32 = !(last.op & kInstrU32);
            cg_tensor *out = const_cast<cg_tensor *>(dst);
            if (p.ninstr == 1 && !p.leaf[last.a].uniform && !p.leaf[last.a].pw) { // (a plain view: a two-part leaf is not one tensor)
                cg_tensor leaf;
                leaf_as_tensor(p, last.a, &space, f32 ? CG_F32 : CG_U32, &leaf);
                leaf.be = be;
                int rc = launch_reduce(be, kind, &leaf, out);
                leaf.buf = nullptr;
                return rc;
            }
            if (p.ninstr > 1 && last.a == kMaxLeaves + p.ninstr - 2)
                return launch_fused_reduce(be, kind, f32, p, p.ninstr - 1, space.dims, space.rank, out);
        }
        // the same of a narrow dtype, whose result is rounded to the dtype: the reduction kernels, then the rounding of
        // the few results where they stand
        const Instr first = p.ins[0];
        if (p.reduced && p.nred == 1 && p.ninstr == 2 && is_row_reduce(first.op) && !(first.op & kInstrU32) && first.a < kMaxLeaves &&
            !p.leaf[first.a].uniform && !p.leaf[first.a].pw && last.a == kMaxLeaves &&
            (last.op == kRoundBF16 || last.op == kRoundF16 || last.op == kRoundF8) &&
            is_contiguous(dst)) {
            cg_tensor *out = const_cast<cg_tensor *>(dst);
            cg_tensor leaf;
            leaf_as_tensor(p, first.a, &space, CG_F32, &leaf);
            leaf.be = be;
            int rc = launch_reduce(be, first.op == kRowMax ? kMax : kSum, &leaf, out);
            leaf.buf = nullptr;
            const cg_tensor *ins[1] = {out};
            if (!rc) rc = launch_elementwise(be, last.op, CG_F32, out, ins, 1);
            return rc;
        }
        return launch_fused_rows(be, dst, p, space.dims, space.rank);
    }
    bool piecewise = false;
    for (int l = 0; l < p.nleaf; l++) piecewise = piecewise || p.leaf[l].pw;
    if (p.ninstr == 1 && p.nleaf == 1 && piecewise && (p.ins[0].op & ~kInstrU32) == kCopy && !p.leaf[0].neg1 && !p.leaf[0].neg2 &&
        numel(dst) >= (1 << 20)) {
        // a large concat along the last axis that somebody wants in memory after all: two strided copies at streaming
        // speed (the program kernels walk a two-part leaf element by element)
        const LeafView &lv = p.leaf[0];
        const int last = dst->rank - 1;
        int rc = CG_OK;
        for (int part = 0; part < 2 && !rc; part++) {
            cg_tensor src, half;
            src.be = half.be = be;
            src.buf = part ? lv.buf2 : lv.buf;
            half.buf = dst->buf;
            src.dt = half.dt = dst->dt;
            src.rank = half.rank = dst->rank;
            memcpy(src.dims, dst->dims, sizeof src.dims);
            src.dims[last] = part ? dst->dims[last] - lv.pw_split : lv.pw_split;
            memcpy(half.dims, src.dims, sizeof half.dims);
            memcpy(src.strides, part ? lv.strides2 : lv.strides, sizeof src.strides);
            memcpy(half.strides, dst->strides, sizeof half.strides);
            src.offset = part ? lv.offset2 : lv.offset;
            half.offset = dst->offset + (part ? lv.pw_split * dst->strides[last] : 0);
            const cg_tensor *ins[1] = {&src};
            if (numel(&src) > 0) rc = launch_elementwise(be, kCopy, dst->dt, &half, ins, 1);
            src.buf = half.buf = nullptr;
        }
        return rc;
    }
    // one operation, or one operation of a narrow dtype with the rounding of its result behind it: the single-op kernel
    const bool op_and_round = p.ninstr == 2 && !(p.ins[0].op & kInstrU32) && p.ins[1].a == kMaxLeaves &&
                              (p.ins[1].op == kRoundBF16 || p.ins[1].op == kRoundF16 || p.ins[1].op == kRoundF8) &&
                              p.ins[0].a < kMaxLeaves && p.ins[0].b < kMaxLeaves && p.ins[0].c < kMaxLeaves;
    if ((p.ninstr == 1 || op_and_round) && !piecewise) {
        const Instr in = p.ins[0];
        const int op = in.op & ~kInstrU32;
        const cg_dtype dt = (in.op & kInstrU32) ? CG_U32 : CG_F32;
        const int nin = op == kWhere ? 3 : (op >= kAdd && op <= kEq) ? 2 : 1;
        cg_tensor tmp[3];
        const cg_tensor *ins[3];
        const uint8_t regs[3] = {in.a, in.b, in.c};
        for (int k = 0; k < nin; k++) {
            leaf_as_tensor(p, regs[k], dst, dt, &tmp[k]);
            ins[k] = &tmp[k];
        }
        int rc = launch_elementwise(be, op, dt, dst, ins, nin, op_and_round ? p.ins[1].op : 0);
        for (int k = 0; k < nin; k++) tmp[k].buf = nullptr;
        return rc;
    }
    return launch_fused(be, dst, p);
}

// ---- results of constant programs -------------------------------------------------------------------------
constexpr size_t kConstEntryBytes = 64u << 20, kConstTotalBytes = 512u << 20, kConstEntries = 256;

// The identity of a program whose leaves are constants or constant buffers, as a byte string; false
// when some leaf is neither.
static bool const_key(const Pending &p, const int64_t *dims, int rank, std::string *key) {
    if (p.overflow) return false;
    std::string k;
    auto put = [&](const void *v, size_t n) { k.append(static_cast<const char *>(v), n); };
    const int32_t head[5] = {rank, p.nleaf, p.ninstr, p.nred, p.reduced ? 1 : 0};
    put(head, sizeof head);
    put(dims, sizeof(int64_t) * (size_t)rank);
    put(&p.rowlen, sizeof p.rowlen);
    for (int i = 0; i < p.ninstr; i++) put(&p.ins[i], sizeof(Instr));
    for (int l = 0; l < p.nleaf; l++) {
        const LeafView &lv = p.leaf[l];
        if (lv.lazy || lv.lazy2) return false;
        const char kind = lv.uniform ? 'u' : lv.pw ? 'p' : 'v';
        put(&kind, 1);
        if (lv.uniform) {
            put(&lv.ubits, sizeof lv.ubits);
            continue;
        }
        if (!lv.buf || !lv.buf->constant) return false;
        put(&lv.buf->id, sizeof lv.buf->id);
        put(&lv.offset, sizeof lv.offset);
        for (int d = 0; d < rank; d++) {
            const int64_t st = dims[d] > 1 ? lv.strides[d] : 0;
            put(&st, sizeof st);
        }
        if (lv.pw) {
            if (!lv.buf2 || !lv.buf2->constant) return false;
            put(&lv.buf2->id, sizeof lv.buf2->id);
            put(&lv.offset2, sizeof lv.offset2);
            put(&lv.pw_split, sizeof lv.pw_split);
            const char neg[2] = {(char)lv.neg1, (char)lv.neg2};
            put(neg, 2);
            for (int d = 0; d < rank; d++) {
                const int64_t st = dims[d] > 1 ? lv.strides2[d] : 0;
                put(&st, sizeof st);
            }
        }
    }
    *key = std::move(k);
    return true;
}

// The same for a tensor: deferred (its program), a constant, or a view of a constant buffer.
static bool const_tensor_key(const cg_tensor *t, std::string *key) {
    if (t->split >= 0) return false;
    if (t->pend) return const_key(*t->pend, t->dims, t->rank, key);
    std::string k(t->uniform ? "U" : "V");
    auto put = [&](const void *v, size_t n) { k.append(static_cast<const char *>(v), n); };
    put(&t->rank, sizeof t->rank);
    put(t->dims, sizeof(int64_t) * (size_t)t->rank);
    if (t->uniform) {
        put(&t->ubits, sizeof t->ubits);
    } else {
        if (!t->buf || !t->buf->constant) return false;
        put(&t->buf->id, sizeof t->buf->id);
        put(&t->offset, sizeof t->offset);
        for (int d = 0; d < t->rank; d++) {
            const int64_t st = t->dims[d] > 1 ? t->strides[d] : 0;
            put(&st, sizeof st);
        }
    }
    *key = std::move(k);
    return true;
}

static void const_memo_clear(cg_backend *be) {
    for (auto &kv : be->const_memo) buffer_release(kv.second);
    be->const_memo.clear();
    be->const_order.clear();
    be->const_bytes = 0;
    buffer_release(be->iota);
    be->iota = nullptr;
    be->iota_len = 0;
}

static void const_memo_insert(cg_backend *be, const std::string &key, Buffer *b) {
    if (b->cls > kConstEntryBytes) return;
    while (!be->const_order.empty() && (be->const_memo.size() >= kConstEntries || be->const_bytes + b->cls > kConstTotalBytes)) {
        auto it = be->const_memo.find(be->const_order.front());
        if (it != be->const_memo.end()) {
            be->const_bytes -= it->second->cls;
            buffer_release(it->second);
            be->const_memo.erase(it);
        }
        be->const_order.erase(be->const_order.begin());
    }
    b->constant = true;
    b->rc.fetch_add(1);
    be->const_memo[key] = b;
    be->const_order.push_back(key);
    be->const_bytes += b->cls;
}

static void drop_deferred(DeferredWrite &w) {
    delete w.prog;
    if (w.dst) {
        buffer_release(w.dst->buf);
        w.dst->buf = nullptr;
        delete w.dst;
    }
    w.prog = nullptr;
    w.dst = nullptr;
}

// The waiting writes of a decode step's attention block: the rotary embedding of q and of k (k's destination the
// new row of the KV cache, helpers/rope.rs:423-447 and helpers/cache.rs:64-74) and the copy of v into its cache row,
// each over a product that nobody has computed yet (q / k / v share their left operand).  Then the products
// themselves store roped values straight to those destinations, in one launch: the three products never reach
// memory un-roped and the launch that would read them back goes away.  `also`: a program that refers to the same
// products and goes away with the caller (the handle that is being made concrete).  kDeclined: not that shape.
static int try_rope_stores(cg_backend *be, std::vector<DeferredWrite> &w, const Pending *also) {
    const int n = (int)w.size();
    if (!be->aot || !be->fuse || n < 1 || n > 4) return kDeclined;
    LazyMm *ms[4];
    RopeStore st[4];
    for (int i = 0; i < n; i++) {
        const Pending &p = *w[i].prog;
        const cg_tensor *dst = w[i].dst;
        if (p.reduced || p.nred || p.overflow || dst->dt != CG_F32 || dst->rank != 4 || dst->dims[2] != 1 || dst->split >= 0 || is_narrow_buf(dst->buf))
            return kDeclined;
        const int64_t B = dst->dims[0], H = dst->dims[1], hd = dst->dims[3];
        if (hd < 8 || hd % 8 || dst->strides[3] != 1) return kDeclined;
        const LeafView *lx = nullptr, *lc = nullptr, *ls = nullptr, *lr = nullptr;
        if (p.nleaf == 1 && p.ninstr == 1 && p.ins[0].op == kCopy) {
            lx = &p.leaf[0];
        } else if (p.nleaf == 4 && p.ninstr == 3 && p.ins[0].op == kMul && p.ins[1].op == kMul && p.ins[2].op == kAdd &&
                   p.ins[0].a + p.ins[0].b == 1 && p.ins[1].a + p.ins[1].b == 5 && p.ins[2].a + p.ins[2].b == 2 * kMaxLeaves + 1) {
            // cos * x + sin * rotate_half(x), the factors of each product in either order
            const bool x_first = p.leaf[0].lazy != nullptr, r_first = p.leaf[2].pw;
            lx = &p.leaf[x_first ? 0 : 1];
            lc = &p.leaf[x_first ? 1 : 0];
            lr = &p.leaf[r_first ? 2 : 3];
            ls = &p.leaf[r_first ? 3 : 2];
        } else {
            return kDeclined;
        }
        LazyMm *m = lx->lazy;
        if (lx->uniform || lx->pw || !m || m->result || !m->groupable || !m->be || m->rank < 1) return kDeclined;
        const int64_t N = m->dims[m->rank - 1];
        int64_t rows = 1;
        for (int d = 0; d + 1 < m->rank; d++) rows *= m->dims[d];
        if (H * hd != N || rows != B || B > 4 || (m->head_norm && m->hn_hd != (uint32_t)hd)) return kDeclined;
        auto whole = [&](const int64_t *s, int64_t off, int64_t want_off) { // the view [B, H, 1, hd] of the product's rows, from `want_off`
            return (B == 1 || s[0] == N) && (H == 1 || s[1] == hd) && s[3] == 1 && off == want_off;
        };
        auto row_table = [&](const LeafView *l) { // one row of hd factors, the same for every batch entry and head
            return l->buf && !is_narrow_buf(l->buf) && !l->uniform && !l->pw && !l->lazy && (B == 1 || l->strides[0] == 0) && (H == 1 || l->strides[1] == 0) &&
                   l->strides[3] == 1;
        };
        if (!whole(lx->strides, lx->offset, 0)) return kDeclined;
        memset(&st[i], 0, sizeof st[i]);
        if (lr) {
            if (!lr->pw || lr->uniform || lr->lazy != m || lr->lazy2 != m || !lr->neg1 || lr->neg2 || lr->pw_split * 2 != hd) return kDeclined;
            if (!whole(lr->strides, lr->offset, hd / 2) || !whole(lr->strides2, lr->offset2, 0)) return kDeclined;
            if (!row_table(lc) || !row_table(ls)) return kDeclined;
            st[i].cos = static_cast<const uint32_t *>(lc->buf->ptr) + lc->offset;
            st[i].sin = static_cast<const uint32_t *>(ls->buf->ptr) + ls->offset;
            st[i].rope = 1;
        }
        if (m->head_norm) { // the heads' own RMS norm ahead of the embedding
            st[i].hgamma = static_cast<const uint32_t *>(m->hn_gamma->ptr) + m->hn_gamma_off;
            st[i].hn_n_bits = m->hn_n_bits;
            st[i].hn_eps_bits = m->hn_eps_bits;
            st[i].hn_exp_bits = m->hn_exp_bits;
        }
        st[i].dst = static_cast<uint32_t *>(dst->buf->ptr) + dst->offset;
        st[i].sb = B > 1 ? dst->strides[0] : 0;
        st[i].sh = H > 1 ? dst->strides[1] : 0;
        st[i].hd = (uint32_t)hd;
        if (st[i].sb < 0 || st[i].sh < 0) return kDeclined;
        for (int k = 0; k < i; k++)
            if (ms[k] == m) return kDeclined; // one destination per product
        if (i > 0 && m->x != ms[0]->x) return kDeclined;
        ms[i] = m;
    }
    // nobody else may want the products as they are: every reference to them is held by these programs
    for (int i = 0; i < n; i++) {
        long held = 0;
        auto count = [&](const Pending *p) {
            for (int l = 0; p && l < p->nleaf; l++) held += (p->leaf[l].lazy == ms[i]) + (p->leaf[l].lazy2 == ms[i]);
        };
        for (int k = 0; k < n; k++) count(w[k].prog);
        count(also);
        if (ms[i]->rc.load() != held) return kDeclined;
    }
    cg_tensor *x = ms[0]->x;
    NormFuse nf;
    cg_tensor h;
    const bool normed = x->pend && norm_fuse_of(x, &nf, &h);
    const cg_tensor *ys[4];
    for (int i = 0; i < n; i++) ys[i] = ms[i]->y;
    int rc = CG_OK;
    if (x->pend && !normed) rc = ensure_concrete(x);
    if (!rc) rc = launch_matmul_group_rope(be, normed ? &h : x, ys, st, n, normed ? &nf : nullptr);
    h.buf = nullptr;
    if (rc) return rc;
    be->programs_compiled++;
    for (int i = 0; i < n; i++) lazy_mm_close(ms[i]); // they go away with the programs, never computed on their own
    return CG_OK;
}

int flush_deferred(cg_backend *be, const Pending *also) {
    if (be->deferred.empty()) return CG_OK;
    std::vector<DeferredWrite> w;
    w.swap(be->deferred); // the launches below come back here and find nothing to do
    int rc = try_rope_stores(be, w, also);
    if (rc != kDeclined) {
        for (DeferredWrite &d : w) drop_deferred(d);
        return rc;
    }
    rc = CG_OK;
    const int n = (int)w.size();
    for (int i = 0; i < n && !rc; i++) rc = resolve_lazy_leaves(be, *w[i].prog);
    bool done = false;
    if (!rc && n >= 2) {
        const cg_tensor *outs[4];
        const Pending *ps[4];
        for (int i = 0; i < n && i < 4; i++) {
            outs[i] = w[i].dst;
            ps[i] = w[i].prog;
        }
        rc = n <= 4 ? launch_fused_group(be, outs, ps, n) : kDeclined;
        done = rc == CG_OK;
        if (rc == kDeclined) rc = CG_OK;
    }
    for (int i = 0; i < n && !rc && !done; i++) rc = run_pending(be, w[i].dst, *w[i].prog);
    for (DeferredWrite &d : w) drop_deferred(d);
    return rc;
}

// Puts off the write of `prog`'s value (or, prog == null, of a copy of `src`) into the view `dst`.
// At most three writes wait at a time.
static int defer_write(cg_backend *be, const cg_tensor *dst, const Pending *prog) {
    if (be->deferred.size() >= 3) {
        int rc = flush_deferred(be);
        if (rc) return rc;
    }
    drop_packed(dst->buf);
    DeferredWrite w;
    w.dst = new cg_tensor;
    w.dst->be = be;
    w.dst->buf = dst->buf;
    w.dst->buf->rc.fetch_add(1);
    w.dst->dt = dst->dt;
    w.dst->rank = dst->rank;
    memcpy(w.dst->dims, dst->dims, sizeof dst->dims);
    memcpy(w.dst->strides, dst->strides, sizeof dst->strides);
    w.dst->offset = dst->offset;
    w.prog = new Pending(*prog);
    be->deferred.push_back(w);
    return CG_OK;
}

// A program small enough to wait for company: no row reduces, at most 16 K elements.
static bool may_wait(const cg_backend *be, const cg_tensor *dst, const Pending *p) {
    return be->fuse && be->aot && p && p->nred == 0 && !p->reduced && numel(dst) > 0 && numel(dst) <= 16384;
}

// Turns a deferred tensor into a concrete one, in place (every holder of the handle sees it).
static int ensure_concrete(cg_tensor *t) {
    if (t->split >= 0) { // a split-axis view becomes a plain dense tensor, in place
        std::lock_guard<std::recursive_mutex> lk(g_lazy_mu);
        if (t->split < 0) return CG_OK;
        const hipError_t she = hipSetDevice(t->be->device);
        if (she != hipSuccess) return hip_fail(she, "hipSetDevice");
        cg_tensor *m;
        int rc = materialize(t->be, t, &m);
        if (rc) return rc;
        buffer_release(t->buf);
        t->buf = m->buf;
        m->buf = nullptr;
        t->offset = 0;
        t->split = -1;
        set_row_major(t);
        release(m);
        return CG_OK;
    }
    if (!t->pend) return CG_OK;
    std::lock_guard<std::recursive_mutex> lk(g_lazy_mu);
    if (!t->pend) return CG_OK;
    cg_backend *be = t->be;
    hipError_t he = hipSetDevice(be->device);
    if (he != hipSuccess) return hip_fail(he, "hipSetDevice");
    if (t->pend->nleaf == 1 && t->pend->ninstr == 1 && (t->pend->ins[0].op & ~kInstrU32) == kCopy && !t->pend->leaf[0].pw &&
        !t->pend->leaf[0].uniform) {
        // nothing but a view of one buffer (possibly the result of a lazy product, computed now):
        // the handle becomes that view
        int lrc = resolve_lazy_leaves(be, *t->pend);
        if (lrc) return lrc;
        const LeafView &lv = t->pend->leaf[0];
        lv.buf->rc.fetch_add(1);
        t->buf = lv.buf;
        t->offset = lv.offset;
        memcpy(t->strides, lv.strides, sizeof t->strides);
        Pending *old = t->pend;
        t->pend = nullptr;
        delete old;
        return CG_OK;
    }
    std::string ckey;
    const bool constant = be->fuse && numel(t) > 0 && const_key(*t->pend, t->dims, t->rank, &ckey);
    if (constant) {
        auto hit = be->const_memo.find(ckey);
        if (hit != be->const_memo.end()) { // computed before from the same constants: the handle takes that buffer
            hit->second->rc.fetch_add(1);
            Pending *old = t->pend;
            t->buf = hit->second;
            t->offset = 0;
            set_row_major(t);
            t->pend = nullptr;
            delete old;
            return CG_OK;
        }
    }
    Buffer *b = new Buffer;
    b->be = be;
    // a big result of a narrow dtype is stored as that dtype's patterns by the program kernels (not by the row-reduce and
    // product-store paths, which write words)
    bool plain = t->pend->nred == 0 && !t->pend->reduced;
    for (int l = 0; l < t->pend->nleaf; l++) plain = plain && !t->pend->leaf[l].lazy && !t->pend->leaf[l].lazy2;
    b->fmt = plain ? result_fmt(be, t->dt, numel(t)) : kFmtWords;
    int rc = be->pool.alloc((size_t)numel(t) * fmt_bytes(b->fmt), &b->ptr, &b->cls);
    if (rc) {
        delete b;
        return rc;
    }
    b->elems = numel(t);
    cg_tensor dst;
    dst.be = be;
    dst.buf = b;
    dst.dt = t->dt;
    dst.rank = t->rank;
    memcpy(dst.dims, t->dims, sizeof dst.dims);
    set_row_major(&dst);
    if (constant) const_memo_insert(be, ckey, b); // before the leaves go away with the program
    if (!be->deferred.empty() && may_wait(be, &dst, t->pend)) {
        // writes are waiting for a launch: this one goes along
        rc = defer_write(be, &dst, t->pend);
        if (!rc) rc = flush_deferred(be, t->pend);
    } else {
        rc = run_pending(be, &dst, *t->pend, true);
    }
    dst.buf = nullptr;
    if (rc) {
        if (constant) const_memo_clear(be); // it holds a buffer that was never filled
        buffer_release(b);
        return rc;
    }
    Pending *old = t->pend;
    t->buf = b;
    t->offset = 0;
    set_row_major(t);
    t->pend = nullptr;
    delete old;
    return CG_OK;
}

static bool same_leaf(const LeafView &a, const LeafView &b, const int64_t *dims, int rank) {
    if (a.uniform != b.uniform || a.pw != b.pw || a.lazy != b.lazy || a.lazy2 != b.lazy2) return false;
    if (a.uniform) return a.ubits == b.ubits;
    if (a.buf != b.buf || a.offset != b.offset) return false;
    for (int i = 0; i < rank; i++)
        if (dims[i] > 1 && a.strides[i] != b.strides[i]) return false;
    if (a.pw) {
        if (a.buf2 != b.buf2 || a.offset2 != b.offset2 || a.pw_split != b.pw_split || a.neg1 != b.neg1 || a.neg2 != b.neg2)
            return false;
        for (int i = 0; i < rank; i++)
            if (dims[i] > 1 && a.strides2[i] != b.strides2[i]) return false;
    }
    return true;
}

static int add_leaf(Pending *p, const LeafView &lv, const int64_t *dims, int rank) {
    for (int l = 0; l < p->nleaf; l++)
        if (same_leaf(p->leaf[l], lv, dims, rank)) return l;
    bool second_pw = false; // the kernels address one piecewise leaf per program
    for (int l = 0; l < p->nleaf; l++) second_pw = second_pw || (lv.pw && p->leaf[l].pw);
    if (p->nleaf == kMaxLeaves || second_pw) {
        p->overflow = true;
        return 0;
    }
    p->leaf[p->nleaf] = lv;
    if (lv.buf) lv.buf->rc.fetch_add(1);
    if (lv.buf2) lv.buf2->rc.fetch_add(1);
    if (lv.lazy) lv.lazy->rc.fetch_add(1);
    if (lv.lazy2) lv.lazy2->rc.fetch_add(1);
    return p->nleaf++;
}

static int instr_arity(int op) {
    op &= ~kInstrU32;
    return op == kWhere ? 3 : (op >= kAdd && op <= kEq) ? 2 : 1;
}

// Appends `in` unless the program already computes the very same thing; returns its register.
static uint8_t emit_instr(Pending *p, Instr in) {
    const int n = instr_arity(in.op);
    if (n < 2) in.b = in.a;
    if (n < 3) in.c = in.a;
    for (int i = 0; i < p->ninstr; i++) {
        const Instr &o = p->ins[i];
        if (o.op == in.op && o.a == in.a && o.b == in.b && o.c == in.c) return (uint8_t)(kMaxLeaves + i);
    }
    if (p->ninstr == kMaxInstr) {
        p->overflow = true;
        return (uint8_t)kMaxLeaves;
    }
    p->ins[p->ninstr] = in;
    if (is_row_reduce(in.op)) p->nred++;
    p->expensive = p->expensive || is_expensive(in.op & ~kInstrU32);
    return (uint8_t)(kMaxLeaves + p->ninstr++);
}

// Copies the program of `src` into `p` (leaves merged, repeated work shared); returns the
// register of its result.  zero_last: src is a plain program over [.., 1] entering a space
// whose last axis is a row, so its leaves do not move along that axis.
static uint8_t splice_program(Pending *p, const Pending *src, const int64_t *dims, int rank, bool zero_last) {
    uint8_t lmap[kMaxLeaves], rmap[kMaxInstr];
    for (int l = 0; l < src->nleaf; l++) {
        LeafView lv = src->leaf[l];
        if (zero_last) lv.strides[rank - 1] = 0;
        lmap[l] = (uint8_t)add_leaf(p, lv, dims, rank);
    }
    auto remap = [&](uint8_t r) -> uint8_t { return r < kMaxLeaves ? lmap[r] : rmap[r - kMaxLeaves]; };
    uint8_t last = 0;
    for (int i = 0; i < src->ninstr; i++) {
        Instr in = src->ins[i];
        const int n = instr_arity(in.op);
        in.a = remap(in.a);
        in.b = n > 1 ? remap(in.b) : in.a;
        in.c = n > 2 ? remap(in.c) : in.a;
        if ((in.op & ~kInstrU32) == kCopy) { // inside a larger program a copy is just its operand
            last = rmap[i] = in.a;
            continue;
        }
        last = rmap[i] = emit_instr(p, in);
    }
    return last;
}

// The result of applying `op` element-wise to `ins` (all of ins[0]'s shape) as a deferred
// tensor.  Deferred inputs that this call owns alone, or that are cheap, are spliced in;
// other deferred inputs are made concrete first so that their value is computed once.
static int defer_elementwise(cg_backend *be, int op, cg_dtype in_dt, cg_dtype out_dt, cg_tensor *const *ins, int nin,
                             cg_tensor **out) {
    const cg_tensor *shape_of = ins[0];
    if (numel(shape_of) == 0) return new_dense(be, out_dt, shape_of->dims, shape_of->rank, out);
    const int rank = shape_of->rank;
    bool splice[3] = {false, false, false};
    int64_t rowlen = 0; // > 0: the operands hold one value per row of this length
    for (int k = 0; k < nin; k++) {
        cg_tensor *x = ins[k];
        if (x->split >= 0) {
            int rc = ensure_concrete(x);
            if (rc) return rc;
        }
        if (op != kAdd && x->pend && residual_sum_open(x)) { // see there; a further add may still join the sum
            int rc = ensure_concrete(x);
            if (rc) return rc;
        }
        if (!x->pend) continue;
        long mine = 0; // references to x that this very call consumes
        for (int j = 0; j < nin; j++) mine += ins[j] == x;
        bool ok = x->rc.load() <= mine || cheap(x->pend);
        if (ok && x->pend->reduced) { // row results of different row lengths do not mix
            if (rowlen == 0) rowlen = x->pend->rowlen;
            else ok = rowlen == x->pend->rowlen;
        }
        if (ok) {
            splice[k] = true;
        } else {
            int rc = ensure_concrete(x);
            if (rc) return rc;
        }
    }
    // a full-shape row program over rows of length 1 cannot join a space whose rows are longer
    for (int k = 0; k < nin && rowlen > 0; k++) {
        cg_tensor *x = ins[k];
        if (splice[k] && x->pend->nred > 0 && !x->pend->reduced) {
            int rc = ensure_concrete(x);
            if (rc) return rc;
            for (int j = 0; j < nin; j++)
                if (ins[j] == x) splice[j] = false;
        }
    }
    Pending *p = nullptr;
    for (;;) { // build; while the program does not fit, compute the largest deferred input first and rebuild
        int64_t rl = 0;
        for (int k = 0; k < nin; k++)
            if (splice[k] && ins[k]->pend->reduced) rl = ins[k]->pend->rowlen;
        int64_t sdims[kMaxRank]; // the program's iteration space
        memcpy(sdims, shape_of->dims, sizeof sdims);
        if (rl > 0) sdims[rank - 1] = rl;
        p = new Pending;
        uint8_t reg[3] = {0, 0, 0};
        for (int k = 0; k < nin; k++) {
            cg_tensor *x = ins[k];
            bool done = false;
            for (int j = 0; j < k && !done; j++)
                if (ins[j] == x) {
                    reg[k] = reg[j];
                    done = true;
                }
            if (done) continue;
            if (splice[k]) {
                reg[k] = splice_program(p, x->pend, sdims, rank, rl > 0 && !x->pend->reduced);
            } else {
                LeafView lv{};
                lv.uniform = x->uniform;
                lv.ubits = x->ubits;
                if (!x->uniform) {
                    lv.buf = x->buf;
                    memcpy(lv.strides, x->strides, sizeof lv.strides);
                    if (rl > 0) lv.strides[rank - 1] = 0;
                    lv.offset = x->offset;
                }
                reg[k] = (uint8_t)add_leaf(p, lv, sdims, rank);
            }
        }
        Instr in;
        in.op = (uint8_t)(op | (in_dt == CG_U32 ? kInstrU32 : 0));
        in.a = reg[0];
        in.b = nin > 1 ? reg[1] : reg[0];
        in.c = nin > 2 ? reg[2] : reg[0];
        emit_instr(p, in);
        if (p->nred > 0) {
            p->rowlen = sdims[rank - 1];
            p->reduced = rl > 0;
        }
        if (!p->overflow && p->nred <= kMaxRowReduce && fused_program_fits(*p)) break;
        delete p;
        int worst = -1;
        for (int k = 0; k < nin; k++)
            if (splice[k] && (worst < 0 || ins[k]->pend->ninstr > ins[worst]->pend->ninstr)) worst = k;
        if (worst < 0) return fail(CG_ERR_ARG, "internal error: single instruction does not fit");
        cg_tensor *w = ins[worst];
        int rc = ensure_concrete(w);
        if (rc) return rc;
        for (int k = 0; k < nin; k++)
            if (ins[k] == w) splice[k] = false;
    }
    cg_tensor *t = alloc_tensor(be);
    t->be = be;
    t->dt = out_dt;
    t->rank = rank;
    memcpy(t->dims, shape_of->dims, sizeof t->dims);
    set_row_major(t);
    t->pend = p;
    *out = t;
    return CG_OK;
}

// The deferred sum / max of x over its last axis (extent >= 1): x's program, or x as a leaf,
// plus one row-reduce instruction.  *out stays null when the program would not fit.
static int defer_reduce(cg_backend *be, int kind, cg_tensor *x, const int64_t *odims, cg_tensor **out) {
    *out = nullptr;
    const int rank = x->rank;
    if (x->split >= 0 || (x->pend && x->pend->reduced)) {
        int rc = ensure_concrete(x);
        if (rc) return rc;
    }
    Pending *p;
    uint8_t src;
    if (x->pend) {
        if (x->pend->nred >= kMaxRowReduce || x->pend->ninstr >= kMaxInstr) return CG_OK;
        p = new Pending(*x->pend);
        src = (uint8_t)(kMaxLeaves + p->ninstr - 1);
    } else {
        p = new Pending;
        LeafView lv{};
        lv.uniform = x->uniform;
        lv.ubits = x->ubits;
        if (!x->uniform) {
            lv.buf = x->buf;
            memcpy(lv.strides, x->strides, sizeof lv.strides);
            lv.offset = x->offset;
        }
        src = (uint8_t)add_leaf(p, lv, x->dims, rank);
    }
    Instr in;
    in.op = (uint8_t)((kind == kMax ? kRowMax : kRowSum) | (x->dt == CG_U32 ? kInstrU32 : 0));
    in.a = in.b = in.c = src;
    emit_instr(p, in);
    p->rowlen = x->dims[rank - 1];
    p->reduced = true;
    if (!fused_program_fits(*p)) {
        delete p;
        return CG_OK;
    }
    cg_tensor *t = alloc_tensor(be);
    t->be = be;
    t->dt = x->dt;
    t->rank = rank;
    memcpy(t->dims, odims, sizeof t->dims);
    set_row_major(t);
    t->pend = p;
    *out = t;
    return CG_OK;
}

// x: the deferred RMS norm  v / pow(sum(v * v) / n + eps, e) * gamma  over the rows of [R, hd], v the whole of a decode-time
// product [rows <= 4, N = heads * hd] that nobody has needed yet (the q / k norm of Qwen3, qwen3.rs:249-279).  Then x
// becomes a plain view of a NEW open product that carries the norm (LazyMm::head_norm): the views, the rotary embedding and
// the cache write that follow treat it like any open product, and the kernel that stores the embedded heads norms them on
// the way (try_rope_stores).  False: not that shape; x is untouched.
static bool head_norm_lazy(cg_tensor *x) {
    static const uint8_t code[7][4] = {{kMul, 0, 0, 0},   {kRowSum, 8, 8, 8}, {kDiv, 9, 1, 9},  {kAdd, 10, 2, 10},
                                       {kPow, 11, 3, 11}, {kDiv, 0, 12, 0},   {kMul, 13, 4, 13}};
    const Pending *p = x->pend;
    cg_backend *be = x->be;
    if (!p || !be->aot || !be->fuse || x->dt != CG_F32 || x->rank != 2 || x->split >= 0) return false;
    if (p->nleaf != 5 || p->ninstr != 7 || p->nred != 1 || p->reduced || p->overflow) return false;
    for (int i = 0; i < 7; i++)
        if (p->ins[i].op != code[i][0] || p->ins[i].a != code[i][1] || p->ins[i].b != code[i][2] || p->ins[i].c != code[i][3]) return false;
    const int64_t R = x->dims[0], hd = x->dims[1];
    if (hd < 16 || hd > 128 || hd % 16 || p->rowlen != hd || R < 1) return false;
    const LeafView &lx = p->leaf[0], &lg = p->leaf[4];
    if (lx.uniform || lx.pw || !lx.lazy || lx.lazy->result || lx.offset != 0 || lx.strides[1] != 1 || (R > 1 && lx.strides[0] != hd)) return false;
    LazyMm *m = lx.lazy;
    if (!m->groupable || !m->be || m->head_norm || m->rc.load() != 1 || m->rank < 1) return false;
    int64_t n = 1;
    for (int d = 0; d < m->rank; d++) n *= m->dims[d];
    const int64_t N = m->dims[m->rank - 1], K = m->x->rank > 0 ? m->x->dims[m->x->rank - 1] : 0;
    if (n != R * hd || N % hd || n / N > 4 || K <= 256 || K % 4) return false; // (what the kernels of launch_matmul_group_rope take)
    if (!p->leaf[1].uniform || !p->leaf[2].uniform || !p->leaf[3].uniform) return false;
    if (lg.uniform || lg.pw || lg.lazy || !lg.buf || is_narrow_buf(lg.buf) || lg.strides[1] != 1 || (R > 1 && lg.strides[0] != 0)) return false;
    LazyMm *m2 = new LazyMm;
    m2->x = m->x;
    retain(m2->x);
    m2->y = m->y;
    retain(m2->y);
    memcpy(m2->dims, m->dims, sizeof m2->dims);
    m2->rank = m->rank;
    m2->groupable = true;
    m2->be = be;
    be->lazy_open.push_back(m2);
    m2->head_norm = true;
    m2->hn_gamma = lg.buf;
    m2->hn_gamma->rc.fetch_add(1);
    m2->hn_gamma_off = lg.offset;
    m2->hn_hd = (uint32_t)hd;
    m2->hn_n_bits = p->leaf[1].ubits;
    m2->hn_eps_bits = p->leaf[2].ubits;
    m2->hn_exp_bits = p->leaf[3].ubits;
    m2->hn_prog = new Pending(*p); // for whoever needs the value without the fused store: leaf 0 will read the plain product
    lazy_mm_release(m2->hn_prog->leaf[0].lazy);
    m2->hn_prog->leaf[0].lazy = nullptr;
    m2->hn_prog->leaf[0].buf = nullptr;
    memcpy(m2->hn_dims, x->dims, sizeof m2->hn_dims);
    m2->hn_rank = x->rank;
    Pending *np = new Pending;
    LeafView lv{};
    lv.lazy = m2;
    lv.strides[0] = hd;
    lv.strides[1] = 1;
    add_leaf(np, lv, x->dims, x->rank);
    lazy_mm_release(m2); // the leaf holds it now
    Instr in;
    in.op = (uint8_t)kCopy;
    in.a = in.b = in.c = 0;
    emit_instr(np, in);
    Pending *old = x->pend;
    x->pend = np;
    delete old; // the plain product goes with it, never computed
    return true;
}

// A view of a deferred tensor is the same program over re-strided leaves.  `fn` rewrites
// one leaf (strides/offset) for the new shape; returns false when that leaf cannot be
// viewed that way (then the tensor is made concrete and the caller takes the normal path).
template <class F>
static int pending_view(cg_tensor *x, const int64_t *dims, int rank, F &&fn, cg_tensor **out, bool *handled) {
    *handled = false;
    if (!x->pend) return CG_OK;
    if (x->pend->nred > 0 && !head_norm_lazy(x)) return ensure_concrete(x); // rows do not survive re-striding
    for (int l = 0; l < x->pend->nleaf; l++)
        if (x->pend->leaf[l].pw) return ensure_concrete(x); // nor does a split of the last axis
    int64_t n = 1;
    for (int i = 0; i < rank; i++) n *= dims[i];
    const bool grows = n > numel(x);
    if ((x->rc.load() > 1 && !cheap(x->pend)) || (grows && x->pend->expensive && n > 65536) || n == 0) {
        return ensure_concrete(x); // compute once, then view the buffer
    }
    Pending *p = new Pending(*x->pend);
    for (int l = 0; l < p->nleaf; l++) {
        if (p->leaf[l].uniform) continue;
        if (!fn(p->leaf[l])) {
            delete p;
            return ensure_concrete(x);
        }
    }
    cg_tensor *t = alloc_tensor(x->be);
    t->be = x->be;
    t->dt = x->dt;
    t->rank = rank;
    for (int i = 0; i < rank; i++) t->dims[i] = dims[i];
    set_row_major(t);
    t->pend = p;
    *out = t;
    *handled = true;
    return CG_OK;
}

static uint32_t f32_as_u32_host(float v) { // Rust `as`: saturating, NaN -> 0
    if (!(v == v) || v <= 0.0f) return 0;
    if (v >= 4294967296.0f) return 0xFFFFFFFFu;
    return (uint32_t)v;
}
static float bits_f(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static uint32_t f_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

// Exactly-rounded scalar ops are folded on the host when every operand is uniform
// (IEEE add/sub/mul/div and comparisons give the same bits on host and device).
static bool fold_binary(int op, cg_dtype dt, uint32_t a, uint32_t b, uint32_t *r, bool *divzero) {
    if (is_f(dt)) {
        float x = bits_f(a), y = bits_f(b);
        switch (op) {
        case CG_ADD: *r = f_bits(x + y); return true;
        case CG_SUB: *r = f_bits(x - y); return true;
        case CG_MUL: *r = f_bits(x * y); return true;
        case CG_DIV: *r = f_bits(x / y); return true;
        case CG_LT: *r = f_bits(x < y ? 1.0f : 0.0f); return true;
        case CG_GT: *r = f_bits(x > y ? 1.0f : 0.0f); return true;
        case CG_GTE: *r = f_bits(x >= y ? 1.0f : 0.0f); return true;
        case CG_LTE: *r = f_bits(x <= y ? 1.0f : 0.0f); return true;
        case CG_EQ: *r = f_bits(x == y ? 1.0f : 0.0f); return true;
        default: return false; // pow goes to the device so that one libm serves all elements
        }
    }
    switch (op) {
    case CG_ADD: *r = a + b; return true;
    case CG_SUB: *r = a - b; return true;
    case CG_MUL: *r = a * b; return true;
    case CG_DIV:
        if (b == 0) {
            *divzero = true;
            return true;
        }
        *r = a / b;
        return true;
    case CG_POW: {
        uint32_t acc = 1, base = a, e = b;
        while (e) {
            if (e & 1) acc *= base;
            base *= base;
            e >>= 1;
        }
        *r = acc;
        return true;
    }
    case CG_LT: *r = a < b; return true;
    case CG_GT: *r = a > b; return true;
    case CG_GTE: *r = a >= b; return true;
    case CG_LTE: *r = a <= b; return true;
    case CG_EQ: *r = a == b; return true;
    default: return false;
    }
}


// ---- zero-copy concat: adjacent views, and appended rows -----------------------------------
// concat(x, y, dim) of two views of ONE buffer where y starts exactly where x ends along `dim`
// and all other axes are laid out alike is just the wider view.  (This is how the per-layer KV
// entries, once they live in one row store, restack into the [L, B, kvH, T, hd] cache for free.)
static bool try_adjacent_merge(cg_tensor *x, cg_tensor *y, size_t dim, cg_tensor **out) {
    if (!x->buf || x->buf != y->buf || x->uniform || y->uniform || x->split >= 0 || y->split >= 0) return false;
    const int64_t xd = x->dims[dim], yd = y->dims[dim];
    for (int i = 0; i < x->rank; i++) {
        if ((size_t)i == dim) continue;
        if (x->dims[i] > 1 && x->strides[i] != y->strides[i]) return false;
    }
    const int64_t gap = y->offset - x->offset;
    int64_t sd;
    if (xd > 1) sd = x->strides[dim];
    else if (yd > 1) sd = y->strides[dim];
    else sd = gap;
    if (sd <= 0 || gap != xd * sd) return false;
    if (xd > 1 && x->strides[dim] != sd) return false;
    if (yd > 1 && y->strides[dim] != sd) return false;
    cg_tensor *v = new_view(x);
    v->dims[dim] = xd + yd;
    v->strides[dim] = sd;
    *out = v;
    return true;
}

// concat(x, y, dim) that appends a few rows to every block of a blocked tensor (the KV update
// `concat(cached [B, kvH, T, hd], new [B, kvH, s, hd], 2)`, helpers/cache.rs:30-39).  With a row
// store behind x and x at its frontier the rows are written in place; otherwise x's blocks
// migrate, together with the new rows, into the buffer's roomier successor (one copy per 256+
// appended rows instead of one per append).  Returns false when the pattern does not apply.
static bool try_row_append(cg_backend *b, cg_tensor *x, cg_tensor *y, size_t dim, cg_tensor **out, int *status) {
    *status = CG_OK;
    if (!x->buf || x->pend || x->uniform || x->split >= 0 || y->split >= 0 || y->uniform) return false;
    const int r = x->rank;
    const int64_t xd = x->dims[dim], yd = y->dims[dim];
    if (xd <= 0 || yd <= 0 || yd * 4 > xd) return false; // append-like only
    int64_t R = 1;
    for (int j = r - 1; j > (int)dim; j--) { // inner axes dense row-major
        if (x->dims[j] > 1 && x->strides[j] != R) return false;
        R *= x->dims[j];
    }
    if (xd > 1 && x->strides[dim] != R) return false;
    int64_t outer = 1, min_os = 0;
    for (int i = 0; i < (int)dim; i++) {
        if (x->dims[i] <= 1) continue;
        outer *= x->dims[i];
        if (x->strides[i] <= 0) return false;
        if (min_os == 0 || x->strides[i] < min_os) min_os = x->strides[i];
    }
    if (outer <= 1 || outer > 65536 || min_os % R) return false;
    if (numel(x) * 4 < 65536) return false; // not worth the bookkeeping
    if (is_narrow_buf(x->buf)) { // rows are appended to 32-bit words
        hipError_t she = hipSetDevice(b->device);
        *status = she == hipSuccess ? make_words(x) : hip_fail(she, "hipSetDevice");
        if (*status) return true;
    }
    Buffer *src = x->buf;
    RowStore *rs = src->rs;
    const int64_t C = rs ? rs->C : min_os / R;
    if (rs && rs->R != R) return false;
    if (C < xd || x->offset % (C * R)) return false;
    for (int i = 0; i < (int)dim; i++)
        if (x->dims[i] > 1 && x->strides[i] % (C * R)) return false;
    if (!rs && xd != C) return false; // a partial view of a plain buffer: its "slack" is someone's data
    // blocks of a plain buffer: what has been written of it, not the size class it was rounded up to
    const int64_t src_elems = src->elems > 0 ? src->elems : (int64_t)(src->cls / 4);
    const int64_t src_blocks = (src_elems + C * R - 1) / (C * R);
    // blocks touched, in row-major order of the outer index
    std::vector<int64_t> blocks((size_t)outer);
    {
        int64_t idx[kMaxRank] = {0};
        for (int64_t o = 0; o < outer; o++) {
            int64_t off = x->offset;
            for (int i = 0; i < (int)dim; i++) off += idx[i] * x->strides[i];
            blocks[(size_t)o] = off / (C * R);
            if (blocks[(size_t)o] >= (rs ? rs->nblocks : src_blocks)) return false;
            for (int i = (int)dim - 1; i >= 0; i--) {
                if (x->dims[i] <= 1) continue;
                if (++idx[i] < x->dims[i]) break;
                idx[i] = 0;
            }
        }
    }
    hipError_t he = hipSetDevice(b->device);
    if (he != hipSuccess) {
        *status = hip_fail(he, "hipSetDevice");
        return true;
    }
    if (y->pend && ((y->rc.load() > 1 && !cheap(y->pend)) || y->pend->reduced)) {
        *status = ensure_concrete(y);
        if (*status) return true;
    }
    auto write_rows = [&](Buffer *dstbuf, int64_t dC, int64_t row0, const cg_tensor *src_t) -> int {
        // destination: the rows [row0, row0 + rows) of x's blocks inside dstbuf (block capacity dC)
        cg_tensor dst;
        dst.be = b;
        dst.buf = dstbuf;
        dst.dt = x->dt;
        dst.rank = r;
        memcpy(dst.dims, src_t->dims, sizeof dst.dims);
        for (int i = 0; i < r; i++) {
            if (i < (int)dim) dst.strides[i] = x->dims[i] > 1 ? x->strides[i] / (C * R) * (dC * R) : 0;
            else dst.strides[i] = i == (int)dim ? R : x->strides[i];
        }
        dst.offset = x->offset / (C * R) * (dC * R) + row0 * R;
        const cg_tensor *ins[1] = {src_t};
        int rc;
        drop_packed(dstbuf);
        if (src_t->pend && may_wait(b, &dst, src_t->pend))
            rc = defer_write(b, &dst, src_t->pend); // the rows are written with the next launch
        else
            rc = src_t->pend ? run_pending(b, &dst, *src_t->pend) : launch_elementwise(b, kCopy, x->dt, &dst, ins, 1);
        dst.buf = nullptr;
        return rc;
    };
    bool at_frontier = rs != nullptr && xd + yd <= C;
    for (int64_t o = 0; o < outer && at_frontier; o++) at_frontier = rs->fill[(size_t)blocks[(size_t)o]] == xd;
    Buffer *dstbuf = src;
    int64_t dC = C;
    if (at_frontier) {
        *status = write_rows(src, C, xd, y);
        if (*status) return true;
        for (int64_t o = 0; o < outer; o++) rs->fill[(size_t)blocks[(size_t)o]] = xd + yd;
    } else {
        if (!src->successor) {
            const int64_t nb = rs ? rs->nblocks : src_blocks;
            int64_t grow = (xd + yd) / 8;
            if (grow < 256) grow = 256;
            Buffer *nbuf = new Buffer;
            nbuf->be = b;
            nbuf->rs = new RowStore;
            nbuf->rs->R = R;
            nbuf->rs->C = xd + yd + grow;
            nbuf->rs->src_C = C;
            nbuf->rs->nblocks = nb;
            nbuf->rs->fill.assign((size_t)nb, 0);
            int rc = b->pool.alloc((size_t)(nb * nbuf->rs->C * R) * 4, &nbuf->ptr, &nbuf->cls);
            if (rc) {
                delete nbuf->rs;
                delete nbuf;
                *status = rc;
                return true;
            }
            nbuf->elems = nb * nbuf->rs->C * R;
            src->successor = nbuf;
        }
        dstbuf = src->successor;
        RowStore *ds = dstbuf->rs;
        // the successor numbers its blocks as the view that created it saw this buffer: another blocking does not fit
        if (ds->R != R || ds->src_C != C || ds->C < xd + yd) return false;
        for (int64_t o = 0; o < outer; o++) {
            if (blocks[(size_t)o] >= ds->nblocks) return false;
            if (ds->fill[(size_t)blocks[(size_t)o]] != 0) return false; // somebody already migrated these blocks
        }
        dC = ds->C;
        *status = write_rows(dstbuf, dC, 0, x);
        if (!*status) *status = write_rows(dstbuf, dC, xd, y);
        if (*status) return true;
        for (int64_t o = 0; o < outer; o++) ds->fill[(size_t)blocks[(size_t)o]] = xd + yd;
    }
    cg_tensor *v = alloc_tensor(b);
    v->be = b;
    v->buf = dstbuf;
    dstbuf->rc.fetch_add(1);
    v->dt = x->dt;
    v->rank = r;
    memcpy(v->dims, x->dims, sizeof v->dims);
    v->dims[dim] = xd + yd;
    for (int i = 0; i < r; i++) {
        if (i < (int)dim) v->strides[i] = x->dims[i] > 1 ? x->strides[i] / (C * R) * (dC * R) : x->strides[i];
        else v->strides[i] = i == (int)dim ? R : x->strides[i];
    }
    v->offset = x->offset / (C * R) * (dC * R);
    *out = v;
    return true;
}

} // namespace cg

using namespace cg;

extern "C" {

// ---- backend lifetime ----------------------------------------------------------------
// Every entry point that touches a backend's state holds the backend's lock for its whole duration
// (declared first, so the tensor arguments it consumes are released under the lock too): handles may be
// cloned, moved between threads and used from several threads; calls on one backend then run one at a time.
struct Enter {
    explicit Enter(cg_backend *b) : b_(b) {
        if (b_) b_->mu.lock();
    }
    ~Enter() {
        if (b_) b_->mu.unlock();
    }
    Enter(const Enter &) = delete;
    Enter &operator=(const Enter &) = delete;
    cg_backend *b_;
};

int cg_backend_create(int device, cg_backend **out) {
    if (!out) return fail(CG_ERR_ARG, "null out");
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(CG_ERR_DEVICE, "no HIP device available (hipGetDeviceCount: %s); HipBackend has no CPU fallback",
                    hipGetErrorString(e));
    }
    if (device < 0 || device >= count) return fail(CG_ERR_ARG, "device %d out of range (%d devices)", device, count);
    CG_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    CG_HIP(hipGetDeviceProperties(&prop, device));
    if (int nrc = noalloc_setup(device)) return nrc; // set-up of the entry point that may not allocate later
    cg_backend *b = new cg_backend;
    b->device = device;
    CG_HIP(hipStreamCreateWithFlags(&b->stream, hipStreamNonBlocking));
    CG_HIP(hipHostMalloc((void **)&b->fault_host, 64, hipHostMallocMapped));
    memset(b->fault_host, 0, 64);
    CG_HIP(hipHostGetDevicePointer((void **)&b->fault_dev, b->fault_host, 0));
    CG_HIP(hipHostMalloc((void **)&b->rb_host, (kReadbackWords + 16) * 4, hipHostMallocMapped));
    memset(b->rb_host, 0, (kReadbackWords + 16) * 4);
    CG_HIP(hipHostGetDevicePointer((void **)&b->rb_dev, b->rb_host, 0));
    if (const char *fr = getenv("CG_FAST_READBACK")) b->fast_readback = fr[0] != '0';
    CG_HIP(hipHostMalloc((void **)&b->flag_host, 64, hipHostMallocDefault));
    CG_HIP(hipMalloc((void **)&b->flag_dev, 64));
    const char *fuse = getenv("CG_FUSE"); // CG_FUSE=0: run every element-wise op as its own kernel
    b->fuse = !(fuse && fuse[0] == '0');
    const char *aot = getenv("CG_AOT");
    b->aot = !(aot && aot[0] == '0');
    if (const char *seg = getenv("CG_ATTN_SEG_FROM")) b->attn_seg_from = atoll(seg);
    if (const char *ns = getenv("CG_NARROW_STORAGE")) b->narrow_storage = ns[0] != '0';
    if (const char *nf = getenv("CG_NARROW_FROM")) b->narrow_from = std::max<int64_t>(atoll(nf), 2);
    const char *trace = getenv("CG_TRACE_PROGRAMS");
    b->trace_programs = trace && trace[0] == '1';
    b->compute_units = std::max(prop.multiProcessorCount, 1);
    char name[256];
    snprintf(name, sizeof name, "hip:%s (%s, %d CUs)%s", prop.gcnArchName, prop.name, prop.multiProcessorCount,
             b->fuse ? "" : " [unfused]");
    b->name = name;
    *out = b;
    return CG_OK;
}

// What is left of a backend once nothing refers to it any more.
static void backend_teardown(cg_backend *b) {
    (void)hipSetDevice(b->device);
    (void)hipStreamSynchronize(b->stream);
    b->pool.trim();
    (void)hipFree(b->flag_dev);
    for (int i = 0; i < 2; i++) {
        if (b->stage[i]) (void)hipHostFree(b->stage[i]);
        if (b->stage_ev[i]) (void)hipEventDestroy(b->stage_ev[i]);
    }
    (void)hipHostFree(b->flag_host);
    (void)hipHostFree(b->fault_host);
    (void)hipHostFree(b->rb_host);
    (void)hipStreamDestroy(b->stream);
    delete b;
}

// The reference's tensors own their data and may outlive the backend value that made them
// (`BackendTensorOps: Send + Sync + Clone`, backend/mod.rs:124-126, no lifetime ties them to a `Backend`).  So
// destroying a backend only gives up the owner's hold on it: everything that needs no tensor goes now, and the pool,
// the stream and the lock stay until the last tensor handle has been released (cg_tensor_release then finishes the
// job).  Such surviving handles can be cloned, queried for their shape and released, nothing else.
void cg_backend_destroy(cg_backend *b) {
    if (!b) return;
    bool last;
    {
        Enter entered(b);
        (void)hipSetDevice(b->device);
        for (DeferredWrite &d : b->deferred) drop_deferred(d); // nobody can read them any more
        b->deferred.clear();
        const_memo_clear(b);
        (void)hipStreamSynchronize(b->stream);
        prof_drain(b);
        for (auto &ev : b->prof_free) {
            (void)hipEventDestroy(ev.first);
            (void)hipEventDestroy(ev.second);
        }
        b->prof_free.clear();
        b->pool.trim();
        b->owner_gone = true;
        last = b->live_tensors.load() == 0;
    }
    if (last) backend_teardown(b);
}

const char *cg_last_error(void) { return g_err.c_str(); }
const char *cg_backend_name(cg_backend *b) { return b ? b->name.c_str() : ""; }

int cg_sync(cg_backend *b) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b) return fail(CG_ERR_ARG, "null backend");
    if (int frc = flush_deferred(b)) return frc;
    return wait_and_check(b);
}

int cg_pool_stats(cg_backend *b, size_t *bytes_in_use, size_t *bytes_cached) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b) return fail(CG_ERR_ARG, "null backend");
    b->pool.stats(bytes_in_use, bytes_cached);
    // what the backend keeps for itself (iota, results of constant programs) counts as cached
    size_t kept = b->const_bytes + (b->iota ? b->iota->cls : 0);
    if (bytes_in_use) *bytes_in_use -= kept < *bytes_in_use ? kept : *bytes_in_use;
    if (bytes_cached) *bytes_cached += kept;
    return CG_OK;
}

int cg_pool_trim(cg_backend *b) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b) return fail(CG_ERR_ARG, "null backend");
    CG_HIP(hipStreamSynchronize(b->stream));
    const_memo_clear(b);
    b->pool.trim();
    return CG_OK;
}

int cg_profile_enable(cg_backend *b, cg_kernel_class cls, unsigned sample_every) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || (int)cls < 0 || (int)cls >= CG_K_CLASSES) return fail(CG_ERR_ARG, "bad profile class");
    b->prof[cls].every = sample_every;
    return CG_OK;
}

int cg_program_stats(cg_backend *b, uint64_t *compiled, uint64_t *interpreted, int reset) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b) return fail(CG_ERR_ARG, "null backend");
    if (compiled) *compiled = b->programs_compiled;
    if (interpreted) *interpreted = b->programs_interpreted;
    if (reset) b->programs_compiled = b->programs_interpreted = 0;
    return CG_OK;
}

int cg_realize(cg_backend *b, cg_tensor *t) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !t) return fail(CG_ERR_ARG, "null argument");
    return ensure_concrete(t);
}

int cg_profile_read(cg_backend *b, cg_kernel_class cls, uint64_t *launches, double *milliseconds, double *work,
                    int reset) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || (int)cls < 0 || (int)cls >= CG_K_CLASSES) return fail(CG_ERR_ARG, "bad profile class");
    int rc = wait_and_check(b);
    if (rc) return rc;
    ProfClass &c = b->prof[cls];
    if (launches) *launches = c.timed;
    if (milliseconds) *milliseconds = c.ms;
    if (work) *work = c.work;
    if (reset) {
        c.seen = c.timed = 0;
        c.ms = c.work = 0.0;
    }
    return CG_OK;
}

// ---- handles -------------------------------------------------------------------------
void cg_tensor_retain(cg_tensor *t) {
    if (t) retain(t);
}
void cg_tensor_release(cg_tensor *t) {
    if (!t) return;
    cg_backend *be = t->be;
    bool last;
    {
        Enter entered(be); // the last holder of a deferred tensor also closes what it had open in the backend
        release(t);
        last = be->owner_gone && be->live_tensors.load() == 0;
    }
    if (last) backend_teardown(be); // the backend was destroyed while handles were still out: this was the last one
}
size_t cg_tensor_rank(const cg_tensor *t) { return (size_t)t->rank; }
void cg_tensor_shape(const cg_tensor *t, size_t *dims) {
    for (int i = 0; i < t->rank; i++) dims[i] = (size_t)t->dims[i];
}
cg_dtype cg_tensor_dtype(const cg_tensor *t) { return t->dt; }
size_t cg_tensor_numel(const cg_tensor *t) { return (size_t)numel(t); }
int cg_tensor_is_contiguous(const cg_tensor *t) {
    Enter entered(t->be); // a deferred tensor may be being computed, in place, by another thread
    if (t->pend) return 1; // a deferred result is row-major once computed
    return (t->uniform && numel(t) > 1) ? 0 : (is_contiguous(t) ? 1 : 0);
}

// ---- creation --------------------------------------------------------------------------
static int check_dims(const size_t *dims, size_t rank, int64_t *d64) {
    if (rank > CG_MAX_RANK) return fail(CG_ERR_ARG, "rank %zu above CG_MAX_RANK", rank);
    if (rank && !dims) return fail(CG_ERR_ARG, "null dims");
    for (size_t i = 0; i < rank; i++) d64[i] = (int64_t)dims[i];
    return CG_OK;
}

// ndarray.rs:71-84 — a zero tensor is a uniform constant: no memory, no memset.
int cg_zeros(cg_backend *b, cg_dtype dtype, const size_t *dims, size_t rank, cg_tensor **out) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(dtype)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    int64_t d[kMaxRank];
    int rc = check_dims(dims, rank, d);
    if (rc) return rc;
    *out = new_uniform(b, dtype, d, (int)rank, 0);
    return CG_OK;
}

// ndarray.rs:86-96,122-132 and interpreter/mod.rs:28-30.  One-element tensors (the
// `Scalar` / `NatToU32` constants of tensor_op.rs:64-87) stay on the host as uniforms.
// Host memory to device memory through the backend's two pinned staging buffers: the host
// copy into one buffer overlaps the DMA out of the other, nothing waits for the device unless
// a buffer is still in flight, and `src` may be freed on return.
static int staged_upload(cg_backend *b, void *dst, const void *src, size_t bytes) {
    // (a few words — the tokens of a decode step — go as the arguments of a small kernel: no staging buffer, no event)
    if (b->fast_readback && bytes % 4 == 0 && bytes <= kUploadWords * 4 && reinterpret_cast<uintptr_t>(dst) % 4 == 0)
        return launch_small_upload(b, static_cast<uint32_t *>(dst), static_cast<const uint32_t *>(src), (uint32_t)(bytes / 4));
    const char *s = static_cast<const char *>(src);
    char *d = static_cast<char *>(dst);
    for (size_t off = 0; off < bytes; off += kStageBytes) {
        const size_t chunk = std::min(kStageBytes, bytes - off);
        const unsigned i = b->stage_next;
        b->stage_next ^= 1u;
        if (!b->stage[i]) {
            CG_HIP(hipHostMalloc(&b->stage[i], kStageBytes, hipHostMallocDefault));
            CG_HIP(hipEventCreateWithFlags(&b->stage_ev[i], hipEventDisableTiming));
        }
        if (b->stage_busy[i]) CG_HIP(hipEventSynchronize(b->stage_ev[i]));
        memcpy(b->stage[i], s + off, chunk);
        CG_HIP(hipMemcpyAsync(d + off, b->stage[i], chunk, hipMemcpyHostToDevice, b->stream));
        CG_HIP(hipEventRecord(b->stage_ev[i], b->stream));
        b->stage_busy[i] = true;
    }
    return CG_OK;
}

int cg_from_host(cg_backend *b, cg_dtype dtype, const void *data, size_t len, const size_t *dims, size_t rank,
                 cg_tensor **out) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(dtype)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    int64_t d[kMaxRank];
    int rc = check_dims(dims, rank, d);
    if (rc) return rc;
    size_t n = 1;
    for (size_t i = 0; i < rank; i++) n *= dims[i];
    if (n != len) return fail(CG_ERR_SHAPE, "ShapeError");
    if (n && !data) return fail(CG_ERR_ARG, "null data");
    if (n == 1) {
        uint32_t bits;
        if (is_half(dtype)) {
            uint16_t h;
            memcpy(&h, data, 2);
            bits = widen16_host(dtype, h);
        } else if (dtype == CG_F8) {
            bits = widen8_host(*static_cast<const uint8_t *>(data));
        } else {
            memcpy(&bits, data, 4);
        }
        *out = new_uniform(b, dtype, d, (int)rank, bits);
        return CG_OK;
    }
    cg_tensor *t;
    const int fmt = result_fmt(b, dtype, (int64_t)n);
    rc = new_dense(b, dtype, d, (int)rank, &t, 0, fmt);
    if (rc) return rc;
    if (n) {
        CG_HIP(hipSetDevice(b->device));
        if (fmt != kFmtWords) { // kept as they come: 2 or 1 bytes per element
            rc = staged_upload(b, t->buf->ptr, data, n * host_bytes(dtype));
        } else if (is_narrow(dtype)) { // a small tensor: uploaded as it is, widened to 32-bit words on the device
            void *tmp = nullptr;
            size_t cls = 0;
            const size_t eb = host_bytes(dtype);
            rc = b->pool.alloc(n * eb, &tmp, &cls);
            if (!rc) {
                rc = staged_upload(b, tmp, data, n * eb);
                if (!rc)
                    rc = dtype == CG_BF16  ? launch_bf16_widen(b, tmp, t->buf->ptr, n)
                         : dtype == CG_F16 ? launch_f16_widen(b, tmp, t->buf->ptr, n)
                                           : launch_f8_widen(b, tmp, t->buf->ptr, n);
                b->pool.free(tmp, cls); // stream-ordered: later users queue behind the widening kernel
            }
        } else {
            rc = staged_upload(b, t->buf->ptr, data, n * 4);
        }
        if (rc) {
            release(t);
            return rc;
        }
    }
    *out = t;
    return CG_OK;
}

int cg_from_host_bf16_as_f32(cg_backend *b, const uint16_t *bits, size_t len, const size_t *dims, size_t rank,
                             cg_tensor **out) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !out) return fail(CG_ERR_ARG, "null argument");
    int64_t d[kMaxRank];
    int rc = check_dims(dims, rank, d);
    if (rc) return rc;
    size_t n = 1;
    for (size_t i = 0; i < rank; i++) n *= dims[i];
    if (n != len) return fail(CG_ERR_SHAPE, "ShapeError");
    if (n && !bits) return fail(CG_ERR_ARG, "null data");
    if (n == 1) {
        *out = new_uniform(b, CG_F32, d, (int)rank, (uint32_t)bits[0] << 16);
        return CG_OK;
    }
    cg_tensor *t;
    rc = new_dense(b, CG_F32, d, (int)rank, &t);
    if (rc) return rc;
    if (n) {
        CG_HIP(hipSetDevice(b->device));
        void *tmp = nullptr;
        size_t cls = 0;
        rc = b->pool.alloc(n * 2, &tmp, &cls);
        if (!rc) {
            rc = staged_upload(b, tmp, bits, n * 2);
            if (!rc) rc = launch_bf16_widen(b, tmp, t->buf->ptr, n);
            b->pool.free(tmp, cls); // stream-ordered: later users queue behind the widening kernel
        }
        if (rc) {
            release(t);
            return rc;
        }
    }
    *out = t;
    return CG_OK;
}

// ndarray.rs:134-138.  The reference builds the range in f32 and casts; for
// end <= 2^24 that is the integer iota produced here.  Larger ends are rejected
// rather than reproducing the reference's rounding artefacts.
int cg_arange(cg_backend *b, size_t end, cg_tensor **out) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !out) return fail(CG_ERR_ARG, "null argument");
    if (end > (1u << 24)) return fail(CG_ERR_UNSUPPORTED, "arange: end above 2^24 is inexact in the reference");
    int64_t d[1] = {(int64_t)end};
    cg_tensor *t;
    if (b->fuse && end > 0) {
        // a view of the backend's one iota buffer, which grows in powers of two
        if ((int64_t)end > b->iota_len) {
            int64_t cap = 4096;
            while (cap < (int64_t)end) cap *= 2;
            cg_tensor *full;
            int64_t fd[1] = {cap};
            CG_HIP(hipSetDevice(b->device));
            int rc = new_dense(b, CG_U32, fd, 1, &full);
            if (!rc) rc = launch_arange(b, full);
            if (rc) {
                release(full);
                return rc;
            }
            buffer_release(b->iota);
            b->iota = full->buf;
            b->iota->constant = true;
            b->iota->rc.fetch_add(1);
            b->iota_len = cap;
            release(full);
        }
        t = alloc_tensor(b);
        t->be = b;
        t->dt = CG_U32;
        t->rank = 1;
        t->dims[0] = d[0];
        t->strides[0] = 1;
        t->buf = b->iota;
        t->buf->rc.fetch_add(1);
        *out = t;
        return CG_OK;
    }
    int rc = new_dense(b, CG_U32, d, 1, &t);
    if (rc) return rc;
    if (end) {
        rc = launch_arange(b, t);
        if (rc) {
            release(t);
            return rc;
        }
    }
    *out = t;
    return CG_OK;
}

// ---- read-back -----------------------------------------------------------------------------
static int copy_out(cg_backend *b, const cg_tensor *t, void *dst, size_t len) {
    if (int frc = flush_deferred(b)) return frc;
    if (len == 0) return wait_and_check(b);
    if (t->pend) {
        int rc = ensure_concrete(const_cast<cg_tensor *>(t));
        if (rc) return rc;
    }
    if (t->uniform) {
        uint32_t *d = static_cast<uint32_t *>(dst);
        for (size_t i = 0; i < len; i++) d[i] = t->ubits;
        return wait_and_check(b);
    }
    cg_tensor *tmp = nullptr;
    const cg_tensor *src = t;
    if (!is_contiguous(t)) {
        int rc = materialize(b, t, &tmp);
        if (rc) return rc;
        src = tmp;
    }
    const void *p;
    int rc = device_ptr(src, &p);
    if (!rc && b->fast_readback && len <= kReadbackWords) {
        // a few words (the tokens of a decode step): copied by a kernel into pinned memory that the host polls — neither
        // the runtime's staged copy nor its wake-up stands between the last kernel of a step and the first of the next
        const uint32_t seq = ++b->rb_seq;
        rc = launch_small_readback(b, static_cast<const uint32_t *>(p), (uint32_t)len, seq);
        if (!rc) rc = wait_for_readback(b, seq);
        if (!rc) memcpy(dst, b->rb_host, len * 4);
    } else if (!rc) {
        hipError_t e = hipMemcpyAsync(dst, p, len * 4, hipMemcpyDeviceToHost, b->stream);
        rc = e == hipSuccess ? wait_and_check(b) : hip_fail(e, "device to host copy");
    }
    release(tmp);
    return rc;
}

// ndarray.rs:50-58.  Non-contiguous views are materialised first (the reference panics).
int cg_to_host(cg_backend *b, const cg_tensor *t, void *dst, size_t len) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !t || (!dst && len)) return fail(CG_ERR_ARG, "null argument");
    if ((int64_t)len != numel(t)) return fail(CG_ERR_SHAPE, "to_vec: length mismatch");
    CG_HIP(hipSetDevice(b->device));
    if (is_narrow(t->dt) && len > 0) {
        // 2- or 1-byte elements out: the words are narrowed on the device (exact), then copied
        const size_t eb = host_bytes(t->dt);
        if (t->uniform) {
            if (t->dt == CG_F8) {
                memset(dst, narrow8_host(t->ubits), len);
            } else {
                uint16_t *d16 = static_cast<uint16_t *>(dst);
                const uint16_t h = narrow16_host(t->dt, t->ubits);
                for (size_t i = 0; i < len; i++) d16[i] = h;
            }
            return wait_and_check(b);
        }
        int rc = ensure_concrete(const_cast<cg_tensor *>(t));
        if (rc) return rc;
        cg_tensor *tmp = nullptr;
        const cg_tensor *src = t;
        if (!is_contiguous(t)) {
            rc = materialize(b, t, &tmp);
            if (rc) return rc;
            src = tmp;
        }
        const void *p;
        void *half = nullptr;
        size_t cls = 0;
        if (src->buf && src->buf->fmt == fmt_of(t->dt)) { // the patterns are in memory as they are wanted
            int sf;
            rc = flush_deferred(b);
            if (!rc) rc = device_ptr_fmt(src, &p, &sf);
            if (!rc) {
                hipError_t e = hipMemcpyAsync(dst, p, len * eb, hipMemcpyDeviceToHost, b->stream);
                rc = e == hipSuccess ? wait_and_check(b) : hip_fail(e, "device to host copy");
            }
            release(tmp);
            return rc;
        }
        rc = device_ptr(src, &p);
        if (!rc) rc = b->pool.alloc(len * eb, &half, &cls);
        if (!rc) {
            rc = t->dt == CG_F8 ? launch_narrow8(b, p, half, len) : launch_narrow16(b, t->dt, p, half, len);
            if (!rc) {
                hipError_t e = hipMemcpyAsync(dst, half, len * eb, hipMemcpyDeviceToHost, b->stream);
                rc = e == hipSuccess ? wait_and_check(b) : hip_fail(e, "device to host copy");
            }
            b->pool.free(half, cls);
        }
        release(tmp);
        return rc;
    }
    return copy_out(b, t, dst, len);
}

static int read_flag(cg_backend *b, int *out) {
    CG_HIP(hipMemcpyAsync(b->flag_host, b->flag_dev, 4, hipMemcpyDeviceToHost, b->stream));
    int rc = wait_and_check(b);
    if (rc) return rc;
    *out = *b->flag_host != 0;
    return CG_OK;
}

// ndarray.rs:140-149
int cg_to_bool(cg_backend *b, const cg_tensor *t, int *out) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !t || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(t->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    CG_HIP(hipSetDevice(b->device));
    if (numel(t) == 0) {
        *out = 0;
        return wait_and_check(b);
    }
    if (t->uniform) {
        *out = is_f(t->dt) ? bits_f(t->ubits) > 0.0f : t->ubits != 0;
        return wait_and_check(b);
    }
    int rc = ensure_concrete(const_cast<cg_tensor *>(t));
    if (rc) return rc;
    rc = launch_any_positive(b, t);
    if (rc) return rc;
    return read_flag(b, out);
}

// ndarray.rs:534-541
int cg_compare(cg_backend *b, const cg_tensor *x, const cg_tensor *y, int *out) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt) || !supported(y->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (x->dt != y->dt) return fail(CG_ERR_DTYPE, "compare: dtype mismatch");
    CG_HIP(hipSetDevice(b->device));
    if (!same_shape(x, y)) {
        *out = 0;
        return wait_and_check(b);
    }
    if (numel(x) == 0) {
        *out = 1;
        return wait_and_check(b);
    }
    int rc = ensure_concrete(const_cast<cg_tensor *>(x));
    if (!rc) rc = ensure_concrete(const_cast<cg_tensor *>(y));
    if (!rc) rc = launch_any_diff(b, x, y);
    if (rc) return rc;
    int diff = 0;
    rc = read_flag(b, &diff);
    *out = !diff;
    return rc;
}

// ndarray.rs:60-69 — free-form debug rendering: dtype, shape and the first 16 elements.
int cg_format_tensor(cg_backend *b, const cg_tensor *t, char *buf, size_t cap) {
    Enter entered(b);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !t || !buf || !cap) return fail(CG_ERR_ARG, "null argument");
    CG_HIP(hipSetDevice(b->device));
    size_t n = (size_t)numel(t);
    std::vector<uint32_t> host(n);
    int rc = copy_out(b, t, host.data(), n); // the 32-bit words, whatever the dtype
    if (rc) return rc;
    std::string s = t->dt == CG_F32 ? "f32[" : t->dt == CG_F16 ? "f16[" : t->dt == CG_BF16 ? "bf16[" : t->dt == CG_F8 ? "fp8[" : "u32[";
    for (int i = 0; i < t->rank; i++) s += (i ? "," : "") + std::to_string(t->dims[i]);
    s += "] [";
    size_t shown = std::min<size_t>(n, 16);
    char tmp[48];
    for (size_t i = 0; i < shown; i++) {
        if (is_f(t->dt))
            snprintf(tmp, sizeof tmp, "%s%.9g", i ? ", " : "", bits_f(host[i]));
        else
            snprintf(tmp, sizeof tmp, "%s%u", i ? ", " : "", host[i]);
        s += tmp;
    }
    s += n > shown ? ", ...]" : "]";
    snprintf(buf, cap, "%s", s.c_str());
    return CG_OK;
}

// ---- element-wise ------------------------------------------------------------------------------
static int ew_result(cg_backend *b, int op, cg_dtype compute_dt, cg_dtype out_dt, const cg_tensor *shape_of,
                     const cg_tensor *const *ins, int nin, cg_tensor **out) {
    if (b->fuse) return defer_elementwise(b, op, compute_dt, out_dt, const_cast<cg_tensor *const *>(ins), nin, out);
    for (int k = 0; k < nin; k++) {
        int erc = ensure_concrete(const_cast<cg_tensor *>(ins[k]));
        if (erc) return erc;
    }
    cg_tensor *o;
    int rc = new_dense(b, out_dt, shape_of->dims, shape_of->rank, &o);
    if (rc) return rc;
    if (numel(o) > 0) {
        rc = launch_elementwise(b, op, compute_dt, o, ins, nin);
        if (rc) {
            release(o);
            return rc;
        }
    }
    *out = o;
    return CG_OK;
}

// Results of the 16-bit float dtypes and of fp8: the f32 value just computed is rounded to the dtype (one more
// deferred instruction, or on the host for a constant).  Takes over the reference in *io.
static int round_result(cg_backend *b, cg_dtype dt, cg_tensor **io) {
    if (!is_narrow(dt)) return CG_OK;
    cg_tensor *x = *io;
    *io = nullptr;
    int rc = CG_OK;
    if (x->uniform) {
        *io = new_uniform(b, dt, x->dims, x->rank, round_host(dt, x->ubits));
    } else {
        const cg_tensor *ins[1] = {x};
        rc = ew_result(b, dt == CG_BF16 ? kRoundBF16 : dt == CG_F16 ? kRoundF16 : kRoundF8, dt, dt, x, ins, 1, io);
    }
    release(x);
    return rc;
}

// The same tensor under another floating-point dtype tag (its words already hold values of that dtype).
static int retag(cg_backend *b, cg_tensor *x, cg_dtype target, cg_tensor **out) {
    if (x->uniform) {
        *out = new_uniform(b, target, x->dims, x->rank, x->ubits);
        return CG_OK;
    }
    const cg_tensor *ins[1] = {x};
    return ew_result(b, kCopy, CG_F32, target, x, ins, 1, out); // deferred: a view once it is needed
}

// ndarray.rs:151-174; the 16-bit float dtypes as candle.rs:575-599 (`to_dtype`): widening is exact,
// narrowing rounds to nearest even, u32 goes through f32 on the way.
int cg_cast(cg_backend *b, cg_tensor *x, cg_dtype target, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(target) || !supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (target == x->dt) { // identity: hand the same handle back
        retain(x);
        *out = x;
        return CG_OK;
    }
    if (!b->fuse) CG_HIP(hipSetDevice(b->device)); // (deferred results: whoever computes them makes the device current)
    if (is_f(x->dt) && is_f(target)) {
        // between floating-point dtypes: the words stay, a narrower target rounds them
        int rc = retag(b, x, target, out);
        const bool exact = target == CG_F32; // f16 <-> bf16 round too: neither contains the other
        return rc || exact ? rc : round_result(b, target, out);
    }
    if (x->uniform) {
        uint32_t r = target == CG_U32 ? f32_as_u32_host(bits_f(x->ubits)) : f_bits((float)x->ubits);
        *out = new_uniform(b, target, x->dims, x->rank, r);
        return round_result(b, target, out);
    }
    const cg_tensor *ins[1] = {x};
    int rc = ew_result(b, target == CG_U32 ? kCastF2U : kCastU2F, x->dt, target, x, ins, 1, out);
    return rc ? rc : round_result(b, target, out);
}

// ndarray.rs:352-407, 630-648
int cg_unary(cg_backend *b, cg_unary_op op, cg_tensor *x, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if ((int)op < CG_NEG || (int)op > CG_ROUND) return fail(CG_ERR_ARG, "unknown unary op %d", (int)op);
    if (x->dt == CG_U32 && op != CG_NEG) {
        static const char *names[] = {"neg", "sin", "cos", "exp", "log", "floor", "round"};
        return fail(CG_ERR_DTYPE, "Invalid input types for %s", names[op]);
    }
    if (x->uniform && op == CG_NEG) {
        uint32_t r = is_f(x->dt) ? (x->ubits ^ 0x80000000u) : (0u - x->ubits);
        *out = new_uniform(b, x->dt, x->dims, x->rank, r);
        return CG_OK;
    }
    if (!b->fuse) CG_HIP(hipSetDevice(b->device)); // (deferred results: whoever computes them makes the device current)
    const cg_tensor *ins[1] = {x};
    const cg_dtype dt = x->dt;
    int rc = ew_result(b, kNeg + (int)op, dt, dt, x, ins, 1, out);
    // neg, floor and round of a representable value are representable; the others round
    const bool exact = op == CG_NEG || op == CG_FLOOR || op == CG_ROUND;
    return rc || exact ? rc : round_result(b, dt, out);
}

// ndarray.rs:185-323, 598-654
int cg_binary(cg_backend *b, cg_binary_op op, cg_tensor *x, cg_tensor *y, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x), cy(y);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt) || !supported(y->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if ((int)op < CG_ADD || (int)op > CG_EQ) return fail(CG_ERR_ARG, "unknown binary op %d", (int)op);
    if (x->dt != y->dt) return fail(CG_ERR_DTYPE, "TypeError: mixed dtypes in a binary operation");
    if (!same_shape(x, y)) return fail(CG_ERR_SHAPE, "Shape mismatch in operation");
    if (x->uniform && y->uniform && numel(x) > 0) {
        uint32_t r = 0;
        bool divzero = false;
        if (fold_binary(op, x->dt, x->ubits, y->ubits, &r, &divzero)) {
            if (divzero) return fail(CG_ERR_RANGE, "attempt to divide by zero");
            *out = new_uniform(b, x->dt, x->dims, x->rank, round_host(x->dt, r));
            return CG_OK;
        }
    }
    if (!b->fuse) CG_HIP(hipSetDevice(b->device)); // (deferred results: whoever computes them makes the device current)
    const cg_tensor *ins[2] = {x, y};
    const cg_dtype dt = x->dt;
    int rc = ew_result(b, kAdd + (int)op, dt, dt, x, ins, 2, out);
    const bool exact = op >= CG_LT; // comparisons give 0 or 1
    return rc || exact ? rc : round_result(b, dt, out);
}

// ndarray.rs:325-350
int cg_where(cg_backend *b, cg_tensor *mask, cg_tensor *x, cg_tensor *y, cg_tensor **out) {
    Enter entered(b);
    Consume cm(mask), cx(x), cy(y);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !mask || !x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (mask->dt != x->dt || y->dt != x->dt) return fail(CG_ERR_DTYPE, "TypeError: mixed dtypes in where");
    if (!same_shape(mask, x) || !same_shape(x, y)) return fail(CG_ERR_SHAPE, "Shape mismatch in operation");
    if (!b->fuse) CG_HIP(hipSetDevice(b->device)); // (deferred results: whoever computes them makes the device current)
    const cg_tensor *ins[3] = {mask, x, y};
    return ew_result(b, kWhere, x->dt, x->dt, x, ins, 3, out);
}

// ---- contraction / reductions ---------------------------------------------------------------------
// ndarray.rs:176-183, 750-816
static int matmul_entry(cg_backend *b, cg_tensor *x, cg_tensor *y, cg_tensor **out, bool *rounded);
// The 16-bit float dtypes: products of exactly held values, summed in f32, rounded once.
int cg_matmul(cg_backend *b, cg_tensor *x, cg_tensor *y, cg_tensor **out) {
    Enter entered(b);
    const cg_dtype dt = x ? x->dt : CG_F32;
    bool rounded = false; // (by the product's own store)
    int rc = matmul_entry(b, x, y, out, &rounded);
    return rc || rounded ? rc : round_result(b, dt, out);
}
static int matmul_entry(cg_backend *b, cg_tensor *x, cg_tensor *y, cg_tensor **out, bool *rounded) {
    Consume cx(x), cy(y);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt) || !supported(y->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (x->dt != y->dt) return fail(CG_ERR_DTYPE, "TypeError: mixed dtypes in matmul");
    if (x->rank < 2) return fail(CG_ERR_SHAPE, "batched_matmul: lhs must be at least rank 2");
    if (y->rank < 2) return fail(CG_ERR_SHAPE, "batched_matmul: rhs must be at least rank 2");
    int r = x->rank;
    if (x->dims[r - 1] != y->dims[y->rank - 2])
        return fail(CG_ERR_SHAPE, "batched_matmul: incompatible matrix dimensions");
    if (x->rank != y->rank) return fail(CG_ERR_SHAPE, "batched_matmul: batch dimensions must match");
    for (int i = 0; i < r - 2; i++)
        if (x->dims[i] != y->dims[i]) return fail(CG_ERR_SHAPE, "batched_matmul: batch dimensions must match");
    int64_t od[kMaxRank];
    for (int i = 0; i < r - 2; i++) od[i] = x->dims[i];
    od[r - 2] = x->dims[r - 2];
    od[r - 1] = y->dims[r - 1];
    // deferred operands are computed now; a split axis may stay if it is a batch axis (the GEMM walks
    // its two parts as separate batch axes) and the two operands do not disagree about it
    int rc = CG_OK;
    if (b->fuse && x->pend && x->rc.load() == 1 && x->pend->nleaf > 0 && x->pend->leaf[0].lazy &&
        !x->pend->leaf[0].lazy->result && !y->pend && !y->uniform && (y->split < 0 || y->split < r - 2)) {
        // soft-max over a lazy q.K^T, times V: one fused attention pass if the kernel takes the shapes
        CG_HIP(hipSetDevice(b->device));
        LazyMm *m = x->pend->leaf[0].lazy;
        cg_tensor *o;
        rc = new_dense(b, x->dt, od, r, &o);
        if (rc) return rc;
        rc = numel(o) > 0 ? launch_decode_attention(b, *x->pend, x->dims, x->rank, m->x, m->y, y, o) : kDeclined;
        if (rc == kDeclined && numel(o) > 0) rc = launch_prefill_attention(b, *x->pend, x->dims, x->rank, m->x, m->y, y, o);
        if (rc == CG_OK) {
            *out = o;
            return CG_OK;
        }
        release(o);
        if (rc != kDeclined) return rc;
        rc = CG_OK;
    }
    // the RMS norm of a residual stream stays deferred when decode-time products can apply it on load (norm_fuse_of)
    bool norm_x = false;
    if (b->fuse && x->pend && r == 3) {
        NormFuse nfx;
        cg_tensor hx;
        norm_x = norm_fuse_of(x, &nfx, &hx);
        hx.buf = nullptr;
    }
    if (!norm_x && (x->pend || x->split >= r - 2)) rc = ensure_concrete(x);
    if (!rc && (y->pend || y->split >= r - 2)) rc = ensure_concrete(y);
    if (!rc && x->split >= 0 && y->split >= 0 && (x->split != y->split || x->split_inner != y->split_inner))
        rc = ensure_concrete(y);
    if (rc) return rc;
    {
        // decode-time q.K^T: put off, so that soft-max and p.V can absorb it (see LazyMm)
        int64_t n_out = 1;
        for (int i = 0; i < r; i++) n_out *= od[i];
        const int64_t K = x->dims[r - 1];
        // (few rows: a decode step; many rows: a prefill, whose one-pass kernel takes head_dim 64 and 128)
        const bool scores = r == 4 && K > 0 && K <= 256 && od[r - 1] > 1 && (x->dims[r - 2] <= 8 || ((K == 64 || K == 128) && b->aot));
        // a decode-time linear layer: at most 8 rows in all, the weight shared by the batch
        const bool linear = r == 3 && x->dims[0] * x->dims[1] <= 8 && K > 256 && od[r - 1] >= 64 && y->strides[0] == 0 &&
                            y->split < 0 && is_contiguous(x);
        const bool lazy = b->fuse && x->dt == CG_F32 && n_out > 0 && (scores || linear) && K % 4 == 0 && !x->uniform && !y->uniform &&
                          x->split < 0 && y->strides[r - 2] == 1;
        if (norm_x && !(lazy && linear)) { // not a product that could apply the norm: the norm runs now
            rc = ensure_concrete(x);
            if (rc) return rc;
        }
        if (lazy) {
            LazyMm *m = new LazyMm;
            if (linear) {
                m->groupable = true;
                m->be = b;
                b->lazy_open.push_back(m);
            }
            retain(x);
            retain(y);
            m->x = x;
            m->y = y;
            m->rank = r;
            memcpy(m->dims, od, sizeof m->dims);
            cg_tensor *t = alloc_tensor(b);
            t->be = b;
            t->dt = CG_F32;
            t->rank = r;
            memcpy(t->dims, od, sizeof t->dims);
            set_row_major(t);
            Pending *p = new Pending;
            LeafView lv{};
            lv.lazy = m;
            memcpy(lv.strides, t->strides, sizeof lv.strides);
            add_leaf(p, lv, od, r);
            lazy_mm_release(m); // the leaf holds it now
            Instr in;
            in.op = (uint8_t)kCopy;
            in.a = in.b = in.c = 0;
            emit_instr(p, in);
            t->pend = p;
            *out = t;
            return CG_OK;
        }
    }
    CG_HIP(hipSetDevice(b->device));
    // A big product of a narrow dtype whose result is stored narrow rounds in its own store when the kernel it runs on can
    // (asked first: launch_matmul without a result), and leaves the patterns; otherwise f32 words, rounded by the caller.
    int64_t n_res = 1;
    for (int i = 0; i < r; i++) n_res *= od[i];
    int fmt = is_narrow(x->dt) && n_res > 0 ? result_fmt(b, x->dt, n_res) : kFmtWords;
    if (fmt != kFmtWords) {
        rc = launch_matmul(b, x, y, nullptr);
        if (rc == kDeclined) fmt = kFmtWords;
        else if (rc) return rc;
    }
    cg_tensor *o;
    rc = new_dense(b, x->dt, od, r, &o, 0, fmt);
    if (rc) return rc;
    if (numel(o) > 0) {
        rc = launch_matmul(b, x, y, o);
        if (rc) {
            release(o);
            return rc;
        }
    }
    *rounded = fmt != kFmtWords;
    *out = o;
    return CG_OK;
}

static int reduce_entry(cg_backend *b, int kind, const char *what, cg_tensor *x, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (x->rank == 0) return fail(CG_ERR_SHAPE, "%s: rank-0 tensor has no last axis", what);
    if (kind == kArgmax && x->dims[x->rank - 1] == 0)
        return fail(CG_ERR_SHAPE, "argmax: called `Option::unwrap()` on a `None` value (empty axis)");
    int64_t od[kMaxRank];
    memcpy(od, x->dims, sizeof od);
    od[x->rank - 1] = 1;
    cg_tensor *o;
    int rc;
    if (b->fuse && kind != kArgmax && numel(x) > 0) {
        rc = defer_reduce(b, kind, x, od, out);
        if (rc || *out) return rc;
    }
    CG_HIP(hipSetDevice(b->device));
    rc = new_dense(b, kind == kArgmax ? CG_U32 : x->dt, od, x->rank, &o);
    if (rc) return rc;
    if (numel(o) > 0) {
        const bool only_a_view = x->pend && x->pend->nleaf == 1 && x->pend->ninstr == 1 &&
                                 (x->pend->ins[0].op & ~kInstrU32) == kCopy && !x->pend->leaf[0].pw && !x->pend->leaf[0].uniform;
        if (x->pend && !only_a_view && x->pend->nred == 0 && (x->rc.load() == 1 || cheap(x->pend))) {
            rc = resolve_lazy_leaves(b, *x->pend);
            if (!rc) rc = launch_fused_reduce(b, kind, is_f(x->dt), *x->pend, x->pend->ninstr, x->dims, x->rank, o);
        } else {
            rc = ensure_concrete(x);
            if (!rc) rc = launch_reduce(b, kind, x, o);
        }
        if (rc) {
            release(o);
            return rc;
        }
    }
    *out = o;
    return CG_OK;
}

// ndarray.rs:418-425, 723-730.  The 16-bit float dtypes: summed in f32, rounded once.
int cg_sum(cg_backend *b, cg_tensor *x, cg_tensor **out) {
    Enter entered(b);
    const cg_dtype dt = x ? x->dt : CG_F32;
    int rc = reduce_entry(b, kSum, "sum", x, out);
    return rc ? rc : round_result(b, dt, out);
}
// ndarray.rs:409-416, 656-668
int cg_max(cg_backend *b, cg_tensor *x, cg_tensor **out) {
    Enter entered(b);
    const cg_dtype dt = x ? x->dt : CG_F32;
    int rc = reduce_entry(b, kMax, "max", x, out);
    // exact, except that the seed f32::MIN of an empty or all-NaN row is not a value of the 16-bit dtypes
    return rc ? rc : round_result(b, dt, out);
}
// ndarray.rs:427-434, 670-694
int cg_argmax(cg_backend *b, cg_tensor *x, cg_tensor **out) { return reduce_entry(b, kArgmax, "argmax", x, out); }

// ndarray.rs:436-446, 696-721
int cg_topk(cg_backend *b, cg_tensor *x, size_t k, cg_tensor **values, cg_tensor **indices) {
    Enter entered(b);
    Consume cx(x);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !values || !indices) return fail(CG_ERR_ARG, "null argument");
    if (x->dt == CG_U32) return fail(CG_ERR_DTYPE, "Unsupported type for topk");
    if (!is_f(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (x->rank == 0) return fail(CG_ERR_SHAPE, "topk: rank-0 tensor has no last axis");
    int64_t n = x->dims[x->rank - 1];
    if (n == 0) return fail(CG_ERR_SHAPE, "topk: attempt to divide by zero (empty last axis)");
    if ((int64_t)k > n) return fail(CG_ERR_SHAPE, "topk: k larger than the last axis");
    int64_t od[kMaxRank];
    memcpy(od, x->dims, sizeof od);
    od[x->rank - 1] = (int64_t)k;
    CG_HIP(hipSetDevice(b->device));
    cg_tensor *v, *i;
    int rc = ensure_concrete(x);
    if (rc) return rc;
    rc = new_dense(b, x->dt, od, x->rank, &v);
    if (rc) return rc;
    rc = new_dense(b, CG_U32, od, x->rank, &i);
    if (rc) {
        release(v);
        return rc;
    }
    if (numel(v) > 0) {
        rc = launch_topk(b, x, (int64_t)k, v, i);
        if (rc) {
            release(v);
            release(i);
            return rc;
        }
    }
    *values = v;
    *indices = i;
    return CG_OK;
}

// ---- shape and indexing ---------------------------------------------------------------------------
// ndarray.rs:448-455, 553-559 — a stride-0 view; the reference materialises.
int cg_broadcast(cg_backend *b, cg_tensor *x, const size_t *dims, size_t rank, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    int64_t d[kMaxRank];
    int rc = check_dims(dims, rank, d);
    if (rc) return rc;
    if ((size_t)x->rank > rank) return fail(CG_ERR_SHAPE, "broadcast: incompatible shape (rank)");
    int shift = (int)rank - x->rank;
    for (int i = 0; i < x->rank; i++)
        if (x->dims[i] != d[i + shift] && x->dims[i] != 1)
            return fail(CG_ERR_SHAPE, "broadcast: incompatible shape (axis %d: %lld -> %lld)", i, (long long)x->dims[i],
                        (long long)d[i + shift]);
    if (x->pend && x->pend->reduced && x->rc.load() == 1 && (int)rank == x->rank && d[rank - 1] == x->pend->rowlen) {
        // row results broadcast back over their rows: the same program, seen at full shape
        bool same = true;
        for (int i = 0; i + 1 < (int)rank; i++) same = same && d[i] == x->dims[i];
        if (same) {
            Pending *p = new Pending(*x->pend);
            p->reduced = false;
            cg_tensor *t = alloc_tensor(b);
            t->be = b;
            t->dt = x->dt;
            t->rank = (int)rank;
            memcpy(t->dims, d, sizeof(int64_t) * rank);
            set_row_major(t);
            t->pend = p;
            *out = t;
            return CG_OK;
        }
    }
    if (x->pend) {
        bool handled;
        rc = pending_view(x, d, (int)rank, [&](LeafView &lv) {
            int64_t ns[kMaxRank];
            for (int i = 0; i < (int)rank; i++) {
                int j = i - shift;
                ns[i] = (j >= 0 && x->dims[j] == d[i]) ? lv.strides[j] : 0;
            }
            memcpy(lv.strides, ns, sizeof(int64_t) * rank);
            return true;
        }, out, &handled);
        if (rc || handled) return rc;
    }
    cg_tensor *v = new_view(x);
    v->rank = (int)rank;
    for (int i = 0; i < (int)rank; i++) {
        int j = i - shift;
        v->dims[i] = d[i];
        v->strides[i] = (j >= 0 && x->dims[j] == d[i] && !x->uniform) ? x->strides[j] : 0;
    }
    if (v->split >= 0) v->split += shift;
    *out = v;
    return CG_OK;
}

// ndarray.rs:504-511, 545-551 — a view when the strides allow it, else one row-major copy.
int cg_reshape(cg_backend *b, cg_tensor *x, const size_t *dims, size_t rank, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    int64_t d[kMaxRank];
    int rc = check_dims(dims, rank, d);
    if (rc) return rc;
    int64_t n = 1;
    for (size_t i = 0; i < rank; i++) n *= d[i];
    if (n != numel(x)) return fail(CG_ERR_SHAPE, "reshape: element count mismatch");
    if (x->pend) {
        bool handled;
        rc = pending_view(x, d, (int)rank, [&](LeafView &lv) {
            int64_t ns[kMaxRank];
            if (!try_view_reshape(x->dims, lv.strides, x->rank, d, (int)rank, ns)) return false;
            memset(lv.strides, 0, sizeof lv.strides);
            memcpy(lv.strides, ns, sizeof(int64_t) * rank);
            return true;
        }, out, &handled);
        if (rc || handled) return rc;
    }
    if (x->split >= 0) {
        rc = ensure_concrete(x);
        if (rc) return rc;
    }
    if (n == 0 || x->uniform) {
        cg_tensor *v = new_view(x);
        v->rank = (int)rank;
        for (size_t i = 0; i < rank; i++) {
            v->dims[i] = d[i];
            v->strides[i] = 0;
        }
        if (n == 0 && !x->uniform) set_row_major(v);
        *out = v;
        return CG_OK;
    }
    int64_t st[kMaxRank];
    if (try_view_reshape(x->dims, x->strides, x->rank, d, (int)rank, st)) {
        cg_tensor *v = new_view(x);
        v->rank = (int)rank;
        for (size_t i = 0; i < rank; i++) {
            v->dims[i] = d[i];
            v->strides[i] = st[i];
        }
        *out = v;
        return CG_OK;
    }
    // Two adjacent axes that cannot share a stride but are merged by the new shape (everything else
    // unchanged) stay a view with a split axis; this is repeat_kv's [kvH, rep] -> [kvH * rep]
    // (catgrad-llm-models/src/helpers/tensors.rs:128-151), which then costs no copy.
    if ((int)rank == x->rank - 1 && !x->pend) {
        for (int a = 0; a + 1 < x->rank; a++) {
            bool ok = d[a] == x->dims[a] * x->dims[a + 1];
            for (int i = 0; i < a && ok; i++) ok = d[i] == x->dims[i];
            for (int i = a + 2; i < x->rank && ok; i++) ok = d[i - 1] == x->dims[i];
            if (!ok) continue;
            cg_tensor *v = new_view(x);
            v->rank = (int)rank;
            for (int i = 0; i < (int)rank; i++) {
                v->dims[i] = d[i];
                v->strides[i] = i < a ? x->strides[i] : x->strides[i + 1];
            }
            v->split = a;
            v->split_inner = x->dims[a + 1];
            v->split_os = x->strides[a];
            *out = v;
            return CG_OK;
        }
    }
    CG_HIP(hipSetDevice(b->device));
    cg_tensor *m;
    rc = materialize(b, x, &m);
    if (rc) return rc;
    m->rank = (int)rank;
    for (size_t i = 0; i < rank; i++) m->dims[i] = d[i];
    set_row_major(m);
    *out = m;
    return CG_OK;
}

// ndarray.rs:457-464, 561-569
int cg_transpose(cg_backend *b, cg_tensor *x, size_t dim0, size_t dim1, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (dim0 >= (size_t)x->rank || dim1 >= (size_t)x->rank) return fail(CG_ERR_RANGE, "transpose: axis out of range");
    if (x->pend) {
        int64_t nd[kMaxRank];
        memcpy(nd, x->dims, sizeof nd);
        std::swap(nd[dim0], nd[dim1]);
        bool handled;
        int rc = pending_view(x, nd, x->rank, [&](LeafView &lv) {
            std::swap(lv.strides[dim0], lv.strides[dim1]);
            return true;
        }, out, &handled);
        if (rc || handled) return rc;
    }
    cg_tensor *v = new_view(x);
    std::swap(v->dims[dim0], v->dims[dim1]);
    std::swap(v->strides[dim0], v->strides[dim1]);
    if (v->split == (int)dim0) v->split = (int)dim1;
    else if (v->split == (int)dim1) v->split = (int)dim0;
    *out = v;
    return CG_OK;
}

// ndarray.rs:489-502, 581-588
int cg_slice(cg_backend *b, cg_tensor *x, size_t dim, size_t start, size_t len, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (dim >= (size_t)x->rank) return fail(CG_ERR_RANGE, "slice: axis out of range");
    if ((int64_t)start > x->dims[dim] || (int64_t)len > x->dims[dim] - (int64_t)start)
        return fail(CG_ERR_RANGE, "slice: range out of bounds");
    if (x->pend) {
        int64_t nd[kMaxRank];
        memcpy(nd, x->dims, sizeof nd);
        nd[dim] = (int64_t)len;
        bool handled;
        int rc = pending_view(x, nd, x->rank, [&](LeafView &lv) {
            lv.offset += (int64_t)start * lv.strides[dim];
            return true;
        }, out, &handled);
        if (rc || handled) return rc;
    }
    if (x->split == (int)dim) {
        int rc = ensure_concrete(x);
        if (rc) return rc;
    }
    cg_tensor *v = new_view(x);
    v->dims[dim] = (int64_t)len;
    v->offset += (int64_t)start * x->strides[dim];
    *out = v;
    return CG_OK;
}

// ndarray.rs:513-532, 590-596 — two strided copies into the halves of a fresh tensor.
int cg_concat(cg_backend *b, cg_tensor *x, cg_tensor *y, size_t dim, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x), cy(y);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !y || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt) || !supported(y->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (x->dt != y->dt) return fail(CG_ERR_DTYPE, "Incompatible types for concatenation");
    if (x->rank != y->rank || dim >= (size_t)x->rank) return fail(CG_ERR_SHAPE, "concat: incompatible shapes");
    for (int i = 0; i < x->rank; i++)
        if ((size_t)i != dim && x->dims[i] != y->dims[i]) return fail(CG_ERR_SHAPE, "concat: incompatible shapes");
    if (x->split >= 0 || y->split >= 0) {
        int erc = x->split >= 0 ? ensure_concrete(x) : CG_OK;
        if (!erc && y->split >= 0) erc = ensure_concrete(y);
        if (erc) return erc;
    }
    int64_t od[kMaxRank];
    memcpy(od, x->dims, sizeof od);
    od[dim] = x->dims[dim] + y->dims[dim];
    // an empty operand contributes nothing: the other operand IS the result (tensors are
    // immutable, so handing the same handle back is indistinguishable from a copy)
    if (x->dims[dim] == 0) {
        retain(y);
        *out = y;
        return CG_OK;
    }
    if (y->dims[dim] == 0) {
        retain(x);
        *out = x;
        return CG_OK;
    }
    if (try_adjacent_merge(x, y, dim, out)) return CG_OK;
    {
        int arc;
        if (try_row_append(b, x, y, dim, out, &arc)) return arc;
    }
    if (b->fuse && dim == (size_t)x->rank - 1 && numel(x) > 0 && numel(y) > 0) {
        // Along the last axis the result can stay deferred as one piecewise leaf when each
        // operand is a plain view, or the negation of one (rotate_half of the rotary embedding,
        // helpers/rope.rs:423-427): its consumer then reads both halves in place.
        LeafView lv{};
        // a part may also be a view of a decode-time product that has not been computed yet: it stays open, so that a
        // rotary embedding over it can still run in the product's own store (see try_rope_stores)
        auto part = [&](cg_tensor *t, Buffer **buf, LazyMm **lazy, int64_t *strides, int64_t *offset, bool *neg) {
            if (t->uniform || t->split >= 0) return false;
            const int64_t *st;
            if (!t->pend) {
                if (!t->buf) return false;
                *buf = t->buf;
                st = t->strides;
                *offset = t->offset;
                *neg = false;
            } else {
                const Pending *p = t->pend;
                if (p->nleaf != 1 || p->ninstr != 1 || p->nred || p->leaf[0].uniform || p->leaf[0].pw) return false;
                const int pop = p->ins[0].op & ~kInstrU32;
                if (p->ins[0].op != kNeg && pop != kCopy) return false; // a view, or the f32 negation of one
                const LeafView &src = p->leaf[0];
                if (src.lazy && src.lazy->result) { // computed in the meantime: an ordinary buffer
                    *buf = src.lazy->result;
                } else {
                    *buf = src.buf;
                    *lazy = src.lazy;
                }
                st = src.strides;
                *offset = src.offset;
                *neg = pop != kCopy;
            }
            memcpy(strides, st, sizeof(int64_t) * kMaxRank);
            return true;
        };
        if (part(x, &lv.buf, &lv.lazy, lv.strides, &lv.offset, &lv.neg1) && part(y, &lv.buf2, &lv.lazy2, lv.strides2, &lv.offset2, &lv.neg2)) {
            lv.pw = true;
            lv.pw_split = x->dims[dim];
            Pending *p = new Pending;
            add_leaf(p, lv, od, x->rank);
            Instr in;
            in.op = (uint8_t)(kCopy | (x->dt == CG_U32 ? kInstrU32 : 0));
            in.a = in.b = in.c = 0;
            emit_instr(p, in);
            cg_tensor *t = alloc_tensor(b);
            t->be = b;
            t->dt = x->dt;
            t->rank = x->rank;
            memcpy(t->dims, od, sizeof t->dims);
            set_row_major(t);
            t->pend = p;
            *out = t;
            return CG_OK;
        }
    }
    CG_HIP(hipSetDevice(b->device));
    int64_t nx = numel(x), ny = numel(y);
    bool outermost = true; // `dim` is the outermost axis with extent > 1: y lands right after x in memory
    for (size_t i = 0; i < dim; i++) outermost = outermost && od[i] == 1;
    // Growing a stack along its outermost axis (the per-layer restack of the KV cache,
    // helpers/cache.rs:64-74): when this call holds the only reference to x and x's buffer
    // has room behind it, y is appended in place and x's handle is returned with the larger
    // extent — one copy of y instead of a copy of everything accumulated so far.
    if (outermost && nx > 0 && ny > 0 && !x->uniform && x->rc.load() == 1 && x->buf && x->buf->rc.load() == 1 &&
        x->offset == 0 && is_contiguous(x) && !is_narrow_buf(x->buf) && (size_t)(nx + ny) * 4 <= x->buf->cls) {
        cg_tensor tail;
        tail.be = b;
        tail.buf = x->buf;
        tail.dt = x->dt;
        tail.rank = y->rank;
        memcpy(tail.dims, y->dims, sizeof tail.dims);
        int64_t st = 1;
        for (int i = y->rank - 1; i >= 0; i--) {
            tail.strides[i] = st;
            st *= y->dims[i];
        }
        tail.offset = nx;
        const cg_tensor *ins[1] = {y};
        int rc = CG_OK;
        if (y->pend && ((y->rc.load() > 1 && !cheap(y->pend)) || y->pend->reduced)) rc = ensure_concrete(y);
        if (!rc) rc = y->pend ? run_pending(b, &tail, *y->pend) : launch_elementwise(b, kCopy, x->dt, &tail, ins, 1);
        tail.buf = nullptr;
        if (rc) return rc;
        x->buf->elems = nx + ny;
        drop_packed(x->buf);
        if (x->buf->side) { // row sums kept for the rows this buffer held so far do not describe the grown tensor
            b->pool.free(x->buf->side, x->buf->side_cls);
            x->buf->side = nullptr;
            x->buf->side_blocks = 0;
        }
        x->dims[dim] = od[dim];
        set_row_major(x);
        retain(x);
        *out = x;
        return CG_OK;
    }
    cg_tensor *o;
    // both operands constants (the halves of a rotary table): the result is kept and handed out again
    std::string ckey;
    bool constant = false;
    if (b->fuse && nx > 0 && ny > 0) {
        std::string kx, ky;
        if (const_tensor_key(x, &kx) && const_tensor_key(y, &ky)) {
            constant = true;
            const int64_t d = (int64_t)dim, lx = (int64_t)kx.size();
            ckey.assign("concat");
            ckey.append(reinterpret_cast<const char *>(&d), sizeof d);
            ckey.append(reinterpret_cast<const char *>(&lx), sizeof lx);
            ckey += kx;
            ckey += ky;
            auto hit = b->const_memo.find(ckey);
            if (hit != b->const_memo.end()) {
                o = alloc_tensor(b);
                o->be = b;
                o->dt = x->dt;
                o->rank = x->rank;
                memcpy(o->dims, od, sizeof o->dims);
                set_row_major(o);
                o->buf = hit->second;
                o->buf->rc.fetch_add(1);
                *out = o;
                return CG_OK;
            }
        }
    }
    // a stack that starts growing gets room for as much again, so later appends stay in place
    // (a stack that may grow in place holds words; other big results of a narrow dtype are stored narrow, written by the
    // copy / program kernels of the two halves)
    const bool growing = outermost && !constant;
    const bool by_rows = (x->pend && (x->pend->nred > 0 || x->pend->reduced)) || (y->pend && (y->pend->nred > 0 || y->pend->reduced));
    int rc = new_dense(b, x->dt, od, x->rank, &o, growing ? 2 * (nx + ny) : 0, growing || by_rows ? kFmtWords : result_fmt(b, x->dt, nx + ny));
    if (rc) return rc;
    if (constant) const_memo_insert(b, ckey, o->buf);
    const cg_tensor *parts[2] = {x, y};
    int64_t at = 0;
    for (int p = 0; p < 2 && !rc; p++) {
        const cg_tensor *src = parts[p];
        if (numel(src) > 0) {
            cg_tensor half; // stack view of the output's slice; never released
            half.be = b;
            half.buf = o->buf;
            half.dt = o->dt;
            half.rank = o->rank;
            memcpy(half.dims, src->dims, sizeof half.dims);
            memcpy(half.strides, o->strides, sizeof half.strides);
            half.offset = at * o->strides[dim];
            const cg_tensor *ins[1] = {src};
            if (src->pend && ((src->rc.load() > 1 && !cheap(src->pend)) || src->pend->reduced)) rc = ensure_concrete(const_cast<cg_tensor *>(src));
            // a deferred operand is evaluated straight into its half of the result
            if (!rc) rc = src->pend ? run_pending(b, &half, *src->pend) : launch_elementwise(b, kCopy, o->dt, &half, ins, 1);
        }
        at += src->dims[dim];
    }
    if (rc) {
        if (constant) const_memo_clear(b); // it holds a buffer that was never filled
        release(o);
        return rc;
    }
    *out = o;
    return CG_OK;
}

// ndarray.rs:466-487, 571-579 — gather; out-of-range indices are detected by the kernel
// and reported by the next call that waits for the device.
int cg_index(cg_backend *b, cg_tensor *x, size_t dim, cg_tensor *indices, cg_tensor **out) {
    Enter entered(b);
    Consume cx(x), ci(indices);
    if (b && b->owner_gone) return fail(CG_ERR_ARG, "backend used after cg_backend_destroy");
    if (!b || !x || !indices || !out) return fail(CG_ERR_ARG, "null argument");
    if (!supported(x->dt)) return fail(CG_ERR_UNSUPPORTED, "%s", kTodo);
    if (indices->dt != CG_U32) return fail(CG_ERR_DTYPE, "Invalid input types for indexing");
    if (dim >= (size_t)x->rank) return fail(CG_ERR_RANGE, "index: axis out of range");
    CG_HIP(hipSetDevice(b->device));
    int64_t J = numel(indices);
    int64_t od[kMaxRank];
    memcpy(od, x->dims, sizeof od);
    od[dim] = J;
    cg_tensor *o = nullptr;
    int64_t on = 1;
    for (int i = 0; i < x->rank; i++) on *= od[i];
    int rc = CG_OK;
    if (on > 0) {
        if (x->dims[dim] == 0) return fail(CG_ERR_RANGE, "index: index out of bounds for an axis of length 0");
        // the gather kernel wants a row-major source and a 1-D index vector
        cg_tensor *xs = nullptr, *is = nullptr;
        const cg_tensor *src = x, *idx = indices;
        rc = ensure_concrete(x);
        if (!rc) rc = ensure_concrete(indices);
        if (!rc && (!is_contiguous(x) || x->uniform)) {
            rc = materialize(b, x, &xs);
            src = xs;
        }
        if (!rc && indices->rank != 1) {
            rc = materialize(b, indices, &is);
            idx = is;
        }
        // rows of a narrow source are gathered as they lie in memory; a big result keeps the source's format
        if (!rc) {
            int ofmt = kFmtWords;
            if (is_narrow_buf(src->buf) && b->narrow_storage && on >= b->narrow_from) {
                int64_t inner = 1;
                for (int i = (int)dim + 1; i < x->rank; i++) inner *= x->dims[i];
                const int64_t eb = (int64_t)fmt_bytes(src->buf->fmt);
                if (inner * eb % 4 == 0 && src->offset * eb % 4 == 0) ofmt = src->buf->fmt; // (whole 32-bit words per row: see launch_gather)
            }
            rc = new_dense(b, x->dt, od, x->rank, &o, 0, ofmt);
        }
        if (!rc) rc = launch_gather(b, src, (int)dim, idx, o);
        release(xs);
        release(is);
        if (rc) {
            release(o);
            return rc;
        }
    } else {
        rc = new_dense(b, x->dt, od, x->rank, &o);
        if (rc) return rc;
    }
    *out = o;
    return CG_OK;
}

} // extern "C"
