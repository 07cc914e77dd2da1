/*
 * catgrad_hip.h — C ABI of the MI355X (gfx950) tensor backend for catgrad.
 *
 * One entry point per method of catgrad's interpreter `Backend` trait
 * (reference: catgrad/src/interpreter/backend/mod.rs:24-122).  A Rust
 * `impl Backend for HipBackend` binds exactly these symbols; nothing in the
 * signatures depends on PyTorch, C++ or HIP types.
 *
 * Conventions
 *  - Every function returns a cg_status (0 = CG_OK).  On failure the message
 *    is available from cg_last_error() (thread local).  The reference's
 *    failures on this path are Rust panics except for
 *    BackendError::ShapeError (mod.rs:129-132); a binding turns a non-zero
 *    status into the same panic / Err.
 *  - Tensors are opaque, atomically reference-counted handles to a strided
 *    view of a device buffer.  cg_tensor_retain is the trait's
 *    `BackendTensor::clone` (O(1)); cg_tensor_release is `Drop`.
 *  - MOVE SEMANTICS: every function that takes tensors and RETURNS a tensor
 *    consumes one reference of each tensor argument, whether it succeeds or
 *    fails — exactly as the trait takes `TaggedTensor<Self>` by value
 *    (mod.rs:60-107) and the evaluator moves values into ops
 *    (catgrad/src/abstract_interpreter/eval.rs:44-49).  A caller that wants
 *    to keep using an argument retains it first.  Query functions
 *    (cg_tensor_*, cg_to_host, cg_to_bool, cg_compare, cg_format_tensor)
 *    borrow their arguments.
 *  - Kernels never broadcast implicitly: element-wise operands must have the
 *    same shape and dtype (mod.rs:20-22); reductions keep rank (mod.rs:23).
 *  - All work is queued on the backend's single HIP stream; only
 *    cg_to_host, cg_to_bool, cg_compare, cg_format_tensor and cg_sync wait
 *    for the device.  Device-detected faults (gather index out of range,
 *    u32 division by zero) are reported by the next waiting call.
 *  - Threads: handles may be cloned, sent to and used from any thread
 *    (`BackendTensorOps: Send + Sync`, mod.rs:124); calls on one backend are
 *    serialised by a lock inside the library, so concurrent callers are
 *    safe but do not overlap.  cg_backend_destroy must not race with
 *    another call on the same backend.
 *  - Lifetime: a tensor handle may outlive its backend, as the reference's
 *    tensors may (they own their data; nothing in mod.rs:124-126 ties a
 *    tensor to a `Backend` value).  cg_backend_destroy gives up the owner's
 *    hold: work in flight is waited for and cached memory freed at once, and
 *    the pool, stream and lock go with the last cg_tensor_release.  After
 *    cg_backend_destroy a surviving handle may only be retained, queried
 *    (cg_tensor_rank / shape / dtype / numel) and released.
 *  - dims/shape arrays are row-major extents as size_t; rank 0 and zero
 *    extents are legal.  Maximum rank: CG_MAX_RANK.
 */
#ifndef CATGRAD_HIP_H
#define CATGRAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CG_MAX_RANK 8

typedef struct cg_backend cg_backend; /* `HipBackend` instance: device, stream, pool */
typedef struct cg_tensor cg_tensor;   /* `HipBackend::BackendTensor` */

/* Order follows `enum Dtype` (catgrad/src/category/core.rs:23-29). */
typedef enum cg_dtype {
    CG_F32 = 0,
    CG_F16 = 1,  /* IEEE binary16; NdArrayBackend has todo!() here (ndarray.rs:7-9), CandleBackend implements it */
    CG_BF16 = 2, /* bfloat16; idem.  Both: 2-byte elements at the boundary (cg_from_host / cg_to_host) and in device memory
                    (tensors of 65536 elements and more: uploads, element-wise results, copies, gathers, concats; smaller
                    tensors and the results of products and row reductions are held as 32-bit words, each holding its value
                    exactly); every op computes in f32 on exactly held values and rounds its result to the dtype (nearest,
                    ties to even); sums and products accumulate in f32 and round once */
    CG_F8 = 3,   /* float8::F8E4M3 (candle.rs:9,382): 4 exponent bits (bias 7), 3 mantissa bits, no infinities, largest
                    finite value 448; same model: 1-byte elements at the boundary and in device memory (same rule), every
                    result rounded to nearest even and saturated to +-448.  NdArrayBackend has todo!() here too.
                    (CG_NARROW_STORAGE=0 in the environment when a backend is created keeps every tensor as 32-bit words;
                    CG_NARROW_FROM=n moves the limit of 65536 elements.) */
    CG_U32 = 4
} cg_dtype;

typedef enum cg_status {
    CG_OK = 0,
    CG_ERR_SHAPE = 1,       /* BackendError::ShapeError and "Shape mismatch in operation" */
    CG_ERR_DTYPE = 2,       /* unsupported dtype / mixed dtypes / "Invalid input types for .." */
    CG_ERR_RANGE = 3,       /* dim / slice / index out of range, u32 division by zero */
    CG_ERR_DEVICE = 4,      /* HIP runtime error */
    CG_ERR_UNSUPPORTED = 5, /* reduced-precision floats (todo!() in the reference) */
    CG_ERR_ARG = 6          /* null pointer, rank > CG_MAX_RANK */
} cg_status;

/* `ScalarOp` unary cases (core.rs:245-264), dispatched at
 * catgrad/src/interpreter/tensor_op.rs:19-25. */
typedef enum cg_unary_op {
    CG_NEG = 0,
    CG_SIN = 1,
    CG_COS = 2,
    CG_EXP = 3,
    CG_LOG = 4,
    CG_FLOOR = 5,
    CG_ROUND = 6 /* ties to even (ndarray.rs:646-648) */
} cg_unary_op;

/* `ScalarOp` binary cases, dispatched at tensor_op.rs:16-18,26-32. */
typedef enum cg_binary_op {
    CG_ADD = 0,
    CG_SUB = 1,
    CG_MUL = 2,
    CG_DIV = 3,
    CG_POW = 4,
    CG_LT = 5,
    CG_GT = 6,
    CG_GTE = 7,
    CG_LTE = 8,
    CG_EQ = 9
} cg_binary_op;

/* ---- backend lifetime ---------------------------------------------------
 * `HipBackend::new(device)`; the reference constructs its backends as plain
 * values (`NdArrayBackend`, ndarray.rs:11-12; `CandleBackend::new_accel`,
 * candle.rs:399-410). */
int cg_backend_create(int device, cg_backend **out);
void cg_backend_destroy(cg_backend *b);
const char *cg_last_error(void);
/* Human-readable name of the implementation ("hip:gfx950 ..." / "oracle:cpu"). */
const char *cg_backend_name(cg_backend *b);
/* Wait for all queued work; reports deferred device-detected faults. */
int cg_sync(cg_backend *b);
/* Bytes currently handed out by / cached in the device pool (lifetime tests).  Memory the backend keeps for
 * itself (its iota buffer, kept results of constant programs) counts as cached. */
int cg_pool_stats(cg_backend *b, size_t *bytes_in_use, size_t *bytes_cached);
/* Return cached blocks to the driver; also drops the kept results of constant programs. */
int cg_pool_trim(cg_backend *b);

/* ---- measurement hooks (no counterpart in the reference; used by the benchmark) ----
 * Per-kernel-class device timing with HIP events recorded on the backend's stream
 * around every `sample_every`-th launch of the class (0 switches the class off).
 * cg_profile_read returns the launches timed so far, their summed device time and their
 * summed algorithmic work (flop for the GEMM classes, bytes for the others) and
 * optionally resets the counters; it waits for the device. */
typedef enum cg_kernel_class {
    CG_K_GEMM_MFMA = 0,   /* work = 2*M*N*K flop per batch entry */
    CG_K_GEMM_SKINNY = 1, /* work = bytes of A, B and C */
    CG_K_GEMM_SIMPLE = 2, /* work = flop */
    CG_K_ELEMENTWISE = 3, /* work = bytes of distinct operand elements + output */
    CG_K_REDUCE = 4,      /* work = bytes of the input + output */
    CG_K_GATHER = 5,      /* work = bytes gathered + written */
    CG_K_ATTENTION = 6,   /* one-pass causal attention of a prefill; work = flop of the visible scores and sums */
    CG_K_PACK = 7,        /* an operand narrowed to 2- / 1-byte patterns in memory for a product; work = bytes read + written */
    CG_K_CLASSES = 8
} cg_kernel_class;
int cg_profile_enable(cg_backend *b, cg_kernel_class cls, unsigned sample_every);
/* Element-wise results are computed lazily (fused into their consumer); cg_realize queues
 * the computation of `t` now, as any non-element-wise consumer or read-back would.
 * Borrows `t`.  Used by the op micro-benchmarks to time a single op. */
int cg_realize(cg_backend *b, cg_tensor *t);
int cg_profile_read(cg_backend *b, cg_kernel_class cls, uint64_t *launches, double *milliseconds, double *work,
                    int reset);
/* Launches of fused (deferred) programs since the last reset: through a kernel compiled
 * ahead of time for that very program, and through the interpreter kernels.  No counterpart
 * in the reference (it has no fusion); the conformance tests use it to check that the
 * programs of the decoder graphs still match the compiled ones. */
int cg_program_stats(cg_backend *b, uint64_t *compiled, uint64_t *interpreted, int reset);

/* ---- tensor handles -------------------------------------------------------
 * `BackendTensorOps` (mod.rs:124-126): Clone + shape(). */
void cg_tensor_retain(cg_tensor *t);
void cg_tensor_release(cg_tensor *t);
size_t cg_tensor_rank(const cg_tensor *t);
/* Writes rank extents into dims (capacity >= rank). `BackendTensorOps::shape`. */
void cg_tensor_shape(const cg_tensor *t, size_t *dims);
cg_dtype cg_tensor_dtype(const cg_tensor *t);
size_t cg_tensor_numel(const cg_tensor *t);
/* 1 when the view is row-major contiguous (what ndarray calls standard layout). */
int cg_tensor_is_contiguous(const cg_tensor *t);

/* ---- creation --------------------------------------------------------------*/
/* `Backend::zeros` (mod.rs:28; ndarray.rs:71-84). */
int cg_zeros(cg_backend *b, cg_dtype dtype, const size_t *dims, size_t rank, cg_tensor **out);
/* `Backend::ndarray_from_vec_{f32,f16,bf16,fp8,u32}` (mod.rs:30-58; ndarray.rs:86-96,122-132;
 * candle.rs:530-562 for the 16-bit floats and fp8): row-major host data of `len` elements, 4 bytes each
 * for f32/u32, 2 bytes each for f16/bf16, 1 byte each for fp8; CG_ERR_SHAPE iff len != prod(dims). */
int cg_from_host(cg_backend *b, cg_dtype dtype, const void *data, size_t len,
                 const size_t *dims, size_t rank, cg_tensor **out);
/* Weight ingest (catgrad-llm/src/utils/mod.rs:158-168 `decode_bf16_to_f32_into` followed by
 * `interpreter::tensor`, utils/mod.rs:303-318): an f32 tensor from `len` bfloat16 bit patterns.
 * The reference widens on the host with rayon and hands the backend f32; here the 2-byte
 * values cross PCIe and are widened (bits << 16, exact) on the device. */
int cg_from_host_bf16_as_f32(cg_backend *b, const uint16_t *bits, size_t len, const size_t *dims, size_t rank,
                             cg_tensor **out);
/* `Backend::arange` (mod.rs:107; ndarray.rs:134-138): u32 [0, end). */
int cg_arange(cg_backend *b, size_t end, cg_tensor **out);

/* ---- read-back (borrowing) --------------------------------------------------*/
/* `Backend::to_vec` (mod.rs:111; ndarray.rs:50-58; candle.rs:463-470): row-major copy of the
 * logical contents into `dst` (capacity `len` elements of the tensor's dtype, 2 bytes each for
 * f16/bf16, 1 byte each for fp8; must equal numel). */
int cg_to_host(cg_backend *b, const cg_tensor *t, void *dst, size_t len);
/* `Backend::to_bool` (mod.rs:109; ndarray.rs:140-149): any element > 0 (f32) / != 0 (u32). */
int cg_to_bool(cg_backend *b, const cg_tensor *t, int *out);
/* `Backend::compare` (mod.rs:87; ndarray.rs:534-541): same shape and all elements ==. */
int cg_compare(cg_backend *b, const cg_tensor *x, const cg_tensor *y, int *out);
/* `Backend::format_tensor` (mod.rs:113-121; ndarray.rs:60-69): writes a NUL-terminated
 * debug rendering into buf (truncated to cap). */
int cg_format_tensor(cg_backend *b, const cg_tensor *t, char *buf, size_t cap);

/* ---- element-wise (consuming) -----------------------------------------------*/
/* `Backend::cast` (mod.rs:60; ndarray.rs:151-174). */
int cg_cast(cg_backend *b, cg_tensor *x, cg_dtype target, cg_tensor **out);
/* `Backend::{neg,sin,cos,exp,log,floor,round}` (mod.rs:73-79; ndarray.rs:352-407). */
int cg_unary(cg_backend *b, cg_unary_op op, cg_tensor *x, cg_tensor **out);
/* `Backend::{add,sub,mul,div,pow,lt,gt,gte,lte,eq}` (mod.rs:62-71; ndarray.rs:185-323). */
int cg_binary(cg_backend *b, cg_binary_op op, cg_tensor *x, cg_tensor *y, cg_tensor **out);
/* `Backend::where_cond` (mod.rs:72; ndarray.rs:325-350): mask > 0 ? x : y. */
int cg_where(cg_backend *b, cg_tensor *mask, cg_tensor *x, cg_tensor *y, cg_tensor **out);

/* ---- contraction and reductions (consuming) ----------------------------------*/
/* `Backend::matmul` (mod.rs:61; ndarray.rs:176-183,750-816): [..,M,K] x [..,K,N]. */
int cg_matmul(cg_backend *b, cg_tensor *x, cg_tensor *y, cg_tensor **out);
/* `Backend::sum` / `max` / `argmax` over the last axis, rank kept
 * (mod.rs:83-85; ndarray.rs:409-434,656-694,723-730). */
int cg_sum(cg_backend *b, cg_tensor *x, cg_tensor **out);
int cg_max(cg_backend *b, cg_tensor *x, cg_tensor **out);
int cg_argmax(cg_backend *b, cg_tensor *x, cg_tensor **out);
/* No counterpart in the reference.  For callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the arg-max of cg_argmax over the rows of a dense
 * [rows, n] array of `dtype` words (4 bytes each, also for the narrow float dtypes) that already lies in device
 * memory at `x`, written as u32 to `out` (device memory, `rows` entries).  The two kernels are queued on `stream`
 * (a hipStream_t; null = the default stream) of `device`; the call allocates nothing, frees nothing and does not
 * wait.  Per-segment partial results go to a fixed 128 KiB array that each GPU holds until the process ends:
 * rows * min(256, ceil(n / 1024)) must not exceed 16384 (and rows 65535), else CG_ERR_UNSUPPORTED.  All calls on one
 * GPU share that array: calls that overlap in time on one GPU race; order them on one stream or with events.
 * Precondition: cg_noalloc_setup(device) — or cg_backend_create on that device, which includes it — has returned
 * CG_OK in this process; otherwise CG_ERR_ARG (the call itself never resolves the array's address: that would load
 * code, which is not allowed under stream capture).  The calling thread's current device is left as it was. */
int cg_noalloc_setup(int device);
int cg_argmax_rows_noalloc(int device, cg_dtype dtype, const void *x, size_t rows, size_t n, uint32_t *out,
                           void *stream);
/* `Backend::topk` (mod.rs:86; ndarray.rs:436-446,696-721). */
int cg_topk(cg_backend *b, cg_tensor *x, size_t k, cg_tensor **values, cg_tensor **indices);

/* ---- shape and indexing (consuming) -------------------------------------------*/
/* `Backend::broadcast` (mod.rs:80; ndarray.rs:448-455,553-559). */
int cg_broadcast(cg_backend *b, cg_tensor *x, const size_t *dims, size_t rank, cg_tensor **out);
/* `Backend::reshape` (mod.rs:81; ndarray.rs:504-511,545-551). */
int cg_reshape(cg_backend *b, cg_tensor *x, const size_t *dims, size_t rank, cg_tensor **out);
/* `Backend::transpose` (mod.rs:82; ndarray.rs:457-464,561-569). */
int cg_transpose(cg_backend *b, cg_tensor *x, size_t dim0, size_t dim1, cg_tensor **out);
/* `Backend::slice` (mod.rs:100-106; ndarray.rs:489-502,581-588). */
int cg_slice(cg_backend *b, cg_tensor *x, size_t dim, size_t start, size_t len, cg_tensor **out);
/* `Backend::concat` (mod.rs:88-93; ndarray.rs:513-532,590-596). */
int cg_concat(cg_backend *b, cg_tensor *x, cg_tensor *y, size_t dim, cg_tensor **out);
/* `Backend::index` (mod.rs:94-99; ndarray.rs:466-487,571-579): gather along dim. */
int cg_index(cg_backend *b, cg_tensor *x, size_t dim, cg_tensor *indices, cg_tensor **out);

#ifdef __cplusplus
}
#endif
#endif /* CATGRAD_HIP_H */
