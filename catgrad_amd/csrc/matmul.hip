// Batched matrix multiply for gfx950: C[b, M, N] = A[b, M, K] * B[b, K, N], f32.
//
// Operands are consumed through their strides: row/column strides of A and B are
// arbitrary (transposed views cost nothing), every batch axis has its own stride per
// operand (0 = shared), so `linear`'s transposed, batch-broadcast weight view
// (catgrad/src/stdlib/nn/mod.rs:182-204) and attention's [B, h, S, hd] head views
// (catgrad-llm-models/src/models/llama.rs:285-345) are multiplied in place.  When the
// right-hand side is shared by the whole batch and the left-hand side's batch and row
// axes form one run, the batch is folded into M (one tall GEMM instead of B small ones).
//
// Kernels
//   mfma_gemm_kernel   256 threads = 2x2 waves, one template for three macro tiles: 128x128x32 (2x2
//                      v_mfma_f32_32x32x2_f32 accumulators per wave, two workgroups per compute unit) for
//                      f32 products, 128x64x32 when N is a small multiple of 64 or the product has at
//                      most one 128x128 tile per compute unit, 256x256x32 (each wave a 128x128 block as
//                      4x4 accumulators, all 256 accumulation registers, 144 KiB of LDS) for the 16-bit
//                      and fp8 products and for x.y with a row-contiguous right operand when there is at
//                      least one such tile per compute unit; HALF variants
//                      narrow the tiles to bf16 / f16 on their way into LDS, or read operands that
//                      pack_operand_kernel narrowed in memory (bf16 / f16 / fp8), and issue
//                      v_mfma_f32_32x32x16_{bf16,f16} / v_mfma_scale_f32_32x32x64_f8f6f4.  Tiles of
//                      k-contiguous operands are staged K-fastest in LDS (pitch 36 words: 128-bit fragment
//                      reads and tile stores are both free of bank conflicts), those of row-contiguous f32
//                      operands rows-fastest; whole tiles are loaded at fixed per-lane offsets without
//                      tests; two LDS buffers, next tile's global loads in flight during
//                      the MFMAs, XCD-aware tile order.  MFMA-bound: 2*M*N*K flop.
//   skinny_kt_*        M <= 8 with K-contiguous B rows (decode-time linear layers and q.K^T),
//                      HBM-bound streams of B (4*K*N bytes):
//                      skinny_kt_wide / _narrow: a wave per output column (or per 4 columns, or a
//                      column per 16/32 lanes for short K), 16-byte loads along K, wave shuffle
//                      reduction;
//                      skinny_kt_mfma_xreg_*: M <= 4 on the 4x4x1 matrix instruction with the
//                      activations held in registers, in the variants the decode step needs:
//                      _group (products that share their left operand in one launch), _group_rope
//                      (the same with the rotary embedding and the KV-cache row writes in the
//                      store), _gated / _cols_gated (two products and SiLU(g)*u in one launch),
//                      _residual (the residual adds in the store, row sums of squares left
//                      behind), _norm (an RMS norm applied to the left operand while it loads).
//   skinny_nn_kernel   M <= 8 with N-contiguous B rows (p.V of a decode step), split over K
//                      with a second pass that adds the partial sums.
//   simple_gemm_kernel u32 (wrapping) and any shape the others decline.
//
// Accumulation is f32 with fused multiply-add; the summation order differs from the
// reference's `matrixmultiply::sgemm`, which is why the contract for matmul is 1e-3
// relative (ndarray.rs:750-816 makes no promise on order either).
#include "common.hpp"
#include "device_utils.hpp"

#include <algorithm>
#include <type_traits>

namespace cg {

namespace {

struct MmArgs {
    const uint32_t *A;
    const uint32_t *B;
    uint32_t *C;
    uint32_t M, N, K;
    int64_t a_sm, a_sk, b_sk, b_sn;
    uint32_t nb;                    // collapsed batch axes
    uint32_t bd[kMaxBatchAxes];     // extents, innermost first
    FastDiv bdiv[kMaxBatchAxes];
    int64_t a_bs[kMaxBatchAxes], b_bs[kMaxBatchAxes];
    uint32_t batch;
    uint32_t a_vec, b_vec;          // 16-byte loads along the unit-stride axis are legal
    uint32_t ksplit;                // mfma_gemm_kernel: values of k per workgroup along grid.z (a multiple of 32), 0 = all of K
    uint32_t c_fmt;                 // mfma_gemm_dlds_kernel: kFmtWords, or the operands' narrow format: C holds its patterns, rounded in the store
};

__device__ __forceinline__ void batch_offsets(const MmArgs &a, uint32_t b, int64_t &oa, int64_t &ob) {
    oa = 0;
    ob = 0;
    for (uint32_t d = 0; d < a.nb; d++) {
        uint32_t q = fastdiv(b, a.bdiv[d]);
        int64_t i = (int64_t)(b - q * a.bd[d]);
        b = q;
        oa += i * a.a_bs[d];
        ob += i * a.b_bs[d];
    }
}

// ------------------------------------------------------------------------------------------
// MFMA kernel
// ------------------------------------------------------------------------------------------
constexpr int BM = 128, BK = 32; // (the kernels shadow BM and define BN from their tile parameters)
constexpr int PITCH = BK + 4; // words per LDS row: row r starts at bank 4r mod 32
constexpr size_t gemm_lds_bytes(int bn, int bm = BM, bool half = false) {
    return 2 * (size_t)(bm + bn) * (half ? BK / 2 + 4 : PITCH) * sizeof(float);
}
constexpr int kThreads = 256;
constexpr uint32_t kXcds = 8, kGroupM = 8;

typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));

// Loads one TR x BK tile (rows along `R` with stride s_r, k with stride s_k) into
// registers: TR*BK/4/256 float4 slots per thread.  Layout of the float4 slots of a tile:
//   K-contiguous source (s_k == 1): slot = row*(BK/4) + kq  (float4 along k; 8 lanes read
//                                                            128 contiguous bytes of a row)
//   R-contiguous source (s_r == 1): float4 along rows; a wave's 64 slots are 16 row-quads x 4 values of k
//                                   (rows_fast_slot), so that its LDS stores spread over all banks
//   otherwise                      : as K-contiguous, element by element
template <int TR> struct TileRegs {
    static constexpr int slots = TR * BK / 4 / 256;
    float4v v[slots];
};

__device__ __forceinline__ float ld_guard(const uint32_t *p, bool ok) { return ok ? asf(*p) : 0.0f; }

// Slot -> (first of four rows, k) of a tile whose rows are the unit-stride axis in memory: 16 row-quads x 4 consecutive k
// per wave, global loads of 256 contiguous bytes per k.  An f32 tile keeps that order in LDS (store_tile).  A tile that is
// narrowed to 16 bits is staged K-fastest (pairs of k share a word), so a lane's four values go to four different LDS
// rows, one store each; with each lane writing its four rows in an order rotated by its row-quad (rows_fast_order), a
// wave's store covers all 32 banks twice, which is the best 64 lanes can do (a whole wave on one k would hit 2 banks).
template <int TR> __device__ __forceinline__ void rows_fast_slot(uint32_t slot, uint32_t &row, uint32_t &k) {
    const uint32_t group = slot / 64, in = slot % 64;
    row = (group % (TR / 64)) * 64 + (in % 16) * 4;
    k = (group / (TR / 64)) * 4 + in / 16;
}
__device__ __forceinline__ uint32_t rows_fast_order(uint32_t slot, int i) { return ((uint32_t)i + ((slot % 16) >> 1)) & 3u; }
__device__ __forceinline__ float pick4(const float4v &v, uint32_t j) { return j == 0 ? v[0] : j == 1 ? v[1] : j == 2 ? v[2] : v[3]; }

template <bool ROWS_FAST, int TR>
__device__ __forceinline__ void load_tile(TileRegs<TR> &t, const uint32_t *base, int64_t s_r, int64_t s_k, uint32_t r0,
                                          uint32_t k0, uint32_t R, uint32_t K, bool vec_ok) {
#pragma unroll
    for (int h = 0; h < TileRegs<TR>::slots; h++) {
        uint32_t slot = threadIdx.x + h * kThreads;
        if (!ROWS_FAST) {
            uint32_t row = r0 + slot / (BK / 4), k = k0 + (slot % (BK / 4)) * 4;
            const uint32_t *p = base + (int64_t)row * s_r + (int64_t)k * s_k;
            if (vec_ok && row < R && k + 3 < K) {
                t.v[h] = *reinterpret_cast<const float4v *>(p);
            } else {
                bool rok = row < R;
                t.v[h][0] = ld_guard(p, rok && k < K);
                t.v[h][1] = ld_guard(p + s_k, rok && k + 1 < K);
                t.v[h][2] = ld_guard(p + 2 * s_k, rok && k + 2 < K);
                t.v[h][3] = ld_guard(p + 3 * s_k, rok && k + 3 < K);
            }
        } else {
            uint32_t row, k;
            rows_fast_slot<TR>(slot, row, k);
            row += r0;
            k += k0;
            const uint32_t *p = base + (int64_t)row * s_r + (int64_t)k * s_k;
            if (vec_ok && k < K && row + 3 < R) {
                t.v[h] = *reinterpret_cast<const float4v *>(p);
            } else {
                bool kok = k < K;
                t.v[h][0] = ld_guard(p, kok && row < R);
                t.v[h][1] = ld_guard(p + s_r, kok && row + 1 < R);
                t.v[h][2] = ld_guard(p + 2 * s_r, kok && row + 2 < R);
                t.v[h][3] = ld_guard(p + 3 * s_r, kok && row + 3 < R);
            }
        }
    }
}

// Stores the registers into an LDS tile: K-fastest, [TR][PITCH], for k-contiguous operands; rows-fastest, [BK][TR], for
// row-contiguous ones.
template <bool ROWS_FAST, int TR> __device__ __forceinline__ void store_tile(const TileRegs<TR> &t, float *lds) {
#pragma unroll
    for (int h = 0; h < TileRegs<TR>::slots; h++) {
        uint32_t slot = threadIdx.x + h * kThreads;
        if (!ROWS_FAST) {
            uint32_t row = slot / (BK / 4), k = (slot % (BK / 4)) * 4;
            *reinterpret_cast<float4v *>(lds + row * PITCH + k) = t.v[h];
        } else {
            // rows stay the fastest axis in LDS too, [BK][TR]: one 16-byte store, no transposition (eight lanes cover 32
            // consecutive words); the fragments are then read a word at a time, 32 consecutive words per half wave
            uint32_t row, k;
            rows_fast_slot<TR>(slot, row, k);
            *reinterpret_cast<float4v *>(lds + k * TR + row) = t.v[h];
        }
    }
}

// ---- the 16-bit float dtypes on their own matrix instructions ------------------------------------------------
// Tensors of these dtypes hold f32 words with exactly representable values, so a tile is narrowed to its 16-bit
// patterns on the way into LDS (exact: the upper half of the word for bfloat16, v_cvt_f16_f32 for binary16) and the
// products run on v_mfma_f32_32x32x16_{bf16,f16}: 16 k per instruction instead of 2, f32 accumulation as before.
// LDS rows hold BK/2 words + 4 of padding (a row starts 20 banks after the one before: 8 lanes of a 128-bit
// read cover all 32 banks); a lane's 128-bit read is its 8 consecutive k of one 16-deep chunk.
constexpr int PITCH_H = BK / 2 + 4;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef long long2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int8v __attribute__((ext_vector_type(8)));

// HALF: 1 bfloat16, 2 binary16
template <int HALF> __device__ __forceinline__ uint32_t pack_halves(float lo, float hi) {
    if constexpr (HALF == 1) return (asu(lo) >> 16) | (asu(hi) & 0xFFFF0000u);
    return (uint32_t)__half_as_ushort(__float2half_rn(lo)) | ((uint32_t)__half_as_ushort(__float2half_rn(hi)) << 16);
}
template <int HALF> __device__ __forceinline__ uint16_t narrow_half(float v) {
    if constexpr (HALF == 1) return (uint16_t)(asu(v) >> 16);
    return __half_as_ushort(__float2half_rn(v));
}

// Stores the registers K-fastest into an LDS tile [TR][PITCH_H] of 16-bit patterns.
template <bool ROWS_FAST, int HALF, int TR> __device__ __forceinline__ void store_tile_half(const TileRegs<TR> &t, uint32_t *lds) {
#pragma unroll
    for (int h = 0; h < TileRegs<TR>::slots; h++) {
        uint32_t slot = threadIdx.x + h * kThreads;
        if (!ROWS_FAST) {
            uint32_t row = slot / (BK / 4), k = (slot % (BK / 4)) * 4;
            uint2 w;
            w.x = pack_halves<HALF>(t.v[h][0], t.v[h][1]);
            w.y = pack_halves<HALF>(t.v[h][2], t.v[h][3]);
            *reinterpret_cast<uint2 *>(lds + row * PITCH_H + k / 2) = w;
        } else {
            uint32_t row, k;
            rows_fast_slot<TR>(slot, row, k);
            uint16_t *l16 = reinterpret_cast<uint16_t *>(lds);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t j = rows_fast_order(slot, i);
                l16[(row + j) * (PITCH_H * 2) + k] = narrow_half<HALF>(pick4(t.v[h], j));
            }
        }
    }
}

// NT / MT: 32-wide MFMA tiles per wave along N / M (the block is 2 x 2 waves).  NT = 2, MT = 2: the
// 128 x 128 macro tile; NT = 1: 128 x 64 (each wave a 64 x 32 strip) for products whose N is a small
// multiple of 64, such as p.V with head_dim 64; NT = MT = 4: 256 x 256, each wave a 128 x 128 block in
// 256 accumulation registers, one wave per SIMD: four times the matrix instructions between two
// barriers and half the LDS traffic per flop, for products with enough tiles to fill the chip.
// HALF: 0 f32 operands (v_mfma_f32_32x32x2_f32); 1 / 2: bfloat16 / binary16 operands (see above).
// 3 / 4 / 5: operands that are ALREADY narrow in memory — bfloat16 / binary16 / fp8 (E4M3) patterns, k contiguous,
// addressed as 32-bit words of 2 or 4 values (a.K counts words; see pack_operand).  The tile pipeline is the f32 one
// word for word (16-byte global loads, K-fastest LDS rows of 32 words + 4, one 128-bit LDS read per fragment); a
// fragment then is 8 (16) consecutive k of a row and feeds one v_mfma_f32_32x32x16_{bf16,f16} (two
// v_mfma_f32_32x32x16_fp8_fp8): a tile is 64 (128) deep in k, and half (a quarter) of the bytes move per flop.
template <bool A_MFAST, bool B_NFAST, int NT, int MT = 2, int HALF = 0>
__global__ __launch_bounds__(kThreads) void mfma_gemm_kernel(const MmArgs a) {
    constexpr int BN = 64 * NT, BM = 64 * MT; // shadow the defaults
    constexpr bool WIDEN = HALF == 1 || HALF == 2; // f32 words narrowed on their way into LDS
    constexpr bool PACKED = HALF >= 3;             // narrow in memory already
    static_assert(!PACKED || (!A_MFAST && !B_NFAST), "packed operands are k-contiguous");
    constexpr int LP = WIDEN ? PITCH_H : PITCH; // words per LDS row
    extern __shared__ float lds_dyn[]; // [2][BM][LP] for A, then [2][BN][LP] for B
    auto lds_a = [&](uint32_t buf) { return lds_dyn + buf * (BM * LP); };
    auto lds_b = [&](uint32_t buf) { return lds_dyn + 2 * BM * LP + buf * (BN * LP); };
    auto stage = [&](const TileRegs<BM> &ta, const TileRegs<BN> &tb, uint32_t buf) {
        if constexpr (WIDEN) {
            store_tile_half<A_MFAST, HALF>(ta, reinterpret_cast<uint32_t *>(lds_a(buf)));
            store_tile_half<B_NFAST, HALF>(tb, reinterpret_cast<uint32_t *>(lds_b(buf)));
        } else {
            store_tile<A_MFAST>(ta, lds_a(buf));
            store_tile<B_NFAST>(tb, lds_b(buf));
        }
    };

    // Tile order.  Workgroups are dealt round-robin to the 8 XCDs, each with its own L2, so
    // the linear id is first regrouped to give every XCD one contiguous run of tiles; inside
    // the run tiles advance down a column of kGroupM row-tiles before moving to the next
    // column-tile, so that the tiles in flight on one XCD share A and B panels in its L2
    // instead of each streaming its own from HBM.
    const uint32_t tiles_n = (a.N + BN - 1) / BN, tiles_m = (a.M + BM - 1) / BM;
    const uint32_t ntiles = tiles_m * tiles_n;
    uint32_t lin;
    {
        const uint32_t xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
        const uint32_t q = ntiles / kXcds, r = ntiles % kXcds;
        lin = xcd * q + (xcd < r ? xcd : r) + slot;
    }
    const uint32_t per_group = kGroupM * tiles_n;
    const uint32_t group = lin / per_group, in_group = lin % per_group;
    const uint32_t first_m = group * kGroupM;
    const uint32_t gsize = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
    const uint32_t tile_m = first_m + in_group % gsize, tile_n = in_group / gsize;
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    int64_t oa, ob;
    batch_offsets(a, blockIdx.y, oa, ob);
    // A product with too few tiles for the device is cut along k over grid.z: this workgroup multiplies k0 .. k0 + Kk and
    // leaves its tile in slot (batch entry, split) of a.C, which then is scratch memory that splitk_reduce_kernel sums up
    // in a fixed order.
    const uint32_t k0 = blockIdx.z * a.ksplit;
    const uint32_t Kk = a.ksplit ? min(a.K - k0, a.ksplit) : a.K;
    const uint32_t *A = a.A + oa + (int64_t)k0 * a.a_sk;
    const uint32_t *B = a.B + ob + (int64_t)k0 * a.b_sk;
    uint32_t *C = a.C + ((uint64_t)blockIdx.y * gridDim.z + blockIdx.z) * a.M * a.N;

    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t wm = (wave / 2) * (32 * MT), wn = (wave % 2) * (32 * NT); // wave quadrant
    const uint32_t li = lane % 32, lg = lane / 32;

    float16v acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    TileRegs<BM> ra;
    TileRegs<BN> rb;
    const uint32_t nk = (Kk + BK - 1) / BK;
    load_tile<A_MFAST>(ra, A, a.a_sm, a.a_sk, m0, 0, a.M, Kk, a.a_vec);
    load_tile<B_NFAST>(rb, B, a.b_sn, a.b_sk, n0, 0, a.N, Kk, a.b_vec);
    stage(ra, rb, 0);
    __syncthreads();

    if constexpr (PACKED) {
        // A tile's burst of matrix instructions is an eighth (a sixteenth) as long as the f32 tile's, about as long as a
        // trip to memory: the next tile is staged into the other LDS buffer in the middle of the burst and the loads of
        // the tile after it are asked for right there, a whole burst before they are needed (two sets of tile registers
        // for loads two tiles ahead spill: the accumulators take every accumulation register).
        // a 128-bit fragment is the lane's 8 (fp8: 16) consecutive k of its row: lane group g supplies the second half
        // of each 16-deep step (fp8: bytes 0..7 of both groups form one step, bytes 8..15 the next — A and B agree)
        float4v fa[2][MT], fb[2][NT]; // the fragments of the next 16-deep step are read while the current one multiplies
        int8v fa8[2], fb8[NT];        // fp8: the 32 bytes a lane feeds to one 64-deep instruction; a ring of two A rows, all of B
        // Whole tiles (every tile but a ragged last one) are loaded without a test: a lane's slots sit 32 rows apart at the
        // same k, so its byte offsets into the operands are fixed (rows beyond the edge are clamped: what they contribute
        // lands in accumulator rows that are never stored) and a tile is 16 + 16 loads at a base that moves by one tile.
        uint32_t offa[TileRegs<BM>::slots], offb[TileRegs<BN>::slots];
#pragma unroll
        for (int h = 0; h < TileRegs<BM>::slots; h++) {
            const uint32_t slot = threadIdx.x + h * kThreads, row = min(m0 + slot / (BK / 4), a.M - 1);
            offa[h] = (uint32_t)(((uint64_t)row * (uint64_t)a.a_sm + (slot % (BK / 4)) * 4) * 4);
        }
#pragma unroll
        for (int h = 0; h < TileRegs<BN>::slots; h++) {
            const uint32_t slot = threadIdx.x + h * kThreads, row = min(n0 + slot / (BK / 4), a.N - 1);
            offb[h] = (uint32_t)(((uint64_t)row * (uint64_t)a.b_sn + (slot % (BK / 4)) * 4) * 4);
        }
        const bool lean = (uint64_t)a.M * (uint64_t)a.a_sm < (1ull << 30) && (uint64_t)a.N * (uint64_t)a.b_sn < (1ull << 30); // offsets fit 32 bits
        auto ask = [&](TileRegs<BM> &ta, TileRegs<BN> &tb, uint32_t kt) {
            if (lean && (kt + 1) * BK <= Kk) {
                const char *pa = reinterpret_cast<const char *>(A + (uint64_t)kt * BK), *pb = reinterpret_cast<const char *>(B + (uint64_t)kt * BK);
#pragma unroll
                for (int h = 0; h < TileRegs<BM>::slots; h++) ta.v[h] = *reinterpret_cast<const float4v *>(pa + offa[h]);
#pragma unroll
                for (int h = 0; h < TileRegs<BN>::slots; h++) tb.v[h] = *reinterpret_cast<const float4v *>(pb + offb[h]);
            } else {
                load_tile<false>(ta, A, a.a_sm, a.a_sk, m0, kt * BK, a.M, Kk, a.a_vec);
                load_tile<false>(tb, B, a.b_sn, a.b_sk, n0, kt * BK, a.N, Kk, a.b_vec);
            }
        };
        // One tile: S steps of 16 (fp8: 32) k.  Set 0 holds the fragments of step 0 when a tile begins; every step reads the
        // fragments of the next one while it multiplies.  The barrier stands before the LAST step: by then every wave has
        // read all of this tile's fragments and has staged its share of the next tile into the other buffer, so the first
        // fragments of the next tile are read behind the barrier, under the last step's matrix instructions, and the matrix
        // pipe never drains at a tile border.
        // In the steady state (whole tiles, offsets that fit) the 16 slots of the next tile (one 16-byte LDS store each) and
        // the 16 loads of the tile after it are dealt out between groups of four matrix instructions of the first S - 1 steps:
        // a burst of 16 loads (a KB each) blocks the wave's instruction issue for as long as the texture path takes them.
        constexpr int S = BK / 8;
        auto frag_a = [&](const float *la, const int set, const int kc, const int i) {
            fa[set][i] = *reinterpret_cast<const float4v *>(la + (wm + i * 32 + li) * PITCH + kc * 8 + lg * 4);
        };
        auto frag8 = [&](const float *l, const int d, const uint32_t row0) { // the two fragments of double step d of a row
            const float *p = l + (row0 + li) * PITCH + d * 16 + lg * 4;
            const int4v lo = __builtin_bit_cast(int4v, *reinterpret_cast<const float4v *>(p));
            const int4v hi = __builtin_bit_cast(int4v, *reinterpret_cast<const float4v *>(p + 8));
            return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        };
        auto frag_b = [&](const float *lb, const int set, const int kc, const int j) {
            fb[set][j] = *reinterpret_cast<const float4v *>(lb + (wn + j * 32 + li) * PITCH + kc * 8 + lg * 4);
        };
        auto mma_row = [&](const int set, const int i) {
#pragma unroll
            for (int j = 0; j < NT; j++) {
                if constexpr (HALF == 3) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[set][i]),
                                                                        __builtin_bit_cast(bf16x8, fb[set][j]), acc[i][j], 0, 0, 0);
                } else if constexpr (HALF == 4) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fa[set][i]),
                                                                       __builtin_bit_cast(f16x8, fb[set][j]), acc[i][j], 0, 0, 0);
                } else {
                    const long2v pa = __builtin_bit_cast(long2v, fa[set][i]), pb = __builtin_bit_cast(long2v, fb[set][j]);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(pa[0], pb[0], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(pa[1], pb[1], acc[i][j], 0, 0, 0);
                }
            }
        };
        static_assert(MT == NT && TileRegs<BM>::slots == 8 && TileRegs<BN>::slots == 8, "the slot schedule below is for the 256 x 256 tile");
        auto iteration = [&](const uint32_t kt, auto steady) {
            constexpr bool STEADY = decltype(steady)::value;
            const uint32_t cur = kt & 1;
            const bool next = STEADY || kt + 1 < nk;
            const float *la = lds_a(cur), *lb = lds_b(cur);
            float *na = lds_a(cur ^ 1), *nb = lds_b(cur ^ 1);
            const char *pa = reinterpret_cast<const char *>(A + (uint64_t)(kt + 2) * BK), *pb = reinterpret_cast<const char *>(B + (uint64_t)(kt + 2) * BK);
            auto slot = [&](const int q) { // stage slot q of tile kt + 1, then ask for slot q of tile kt + 2
                const uint32_t sl = threadIdx.x + (q % 8) * kThreads, row = sl / (BK / 4), k = (sl % (BK / 4)) * 4;
                if (q < 8) {
                    *reinterpret_cast<float4v *>(na + row * PITCH + k) = ra.v[q % 8];
                    ra.v[q % 8] = *reinterpret_cast<const float4v *>(pa + offa[q % 8]);
                } else {
                    *reinterpret_cast<float4v *>(nb + row * PITCH + k) = rb.v[q % 8];
                    rb.v[q % 8] = *reinterpret_cast<const float4v *>(pb + offb[q % 8]);
                }
            };
            if constexpr (HALF == 5) {
                // fp8 runs at twice the 16-bit rate only on the 64-deep instruction (v_mfma_scale_f32_32x32x64_f8f6f4 with
                // both scales 2^0; the 16-deep fp8 instruction takes the cycles of the 16-bit one): a lane feeds it 32 bytes
                // of its row, two fragments.  A tile is two such double steps; B's four blocks stay in registers for a double
                // step and are replaced one by one behind the last row's instructions, A rows go through a ring of two.  The
                // barrier stands before the last row of the second double step; 16 slots over the 7 rows before it.
                if constexpr (!STEADY) {
                    // the first and the last tiles: nothing is carried in registers from one tile to the next (the guarded
                    // loads need the registers): stage and ask first, then read this tile's fragments as they are needed
                    if (next) {
                        stage(ra, rb, cur ^ 1);
                        if (kt + 2 < nk) ask(ra, rb, kt + 2);
                    }
                    fa8[0] = frag8(la, 0, wm);
#pragma unroll
                    for (int j = 0; j < NT; j++) fb8[j] = frag8(lb, 0, wn + j * 32);
                }
#pragma unroll
                for (int d = 0; d < 2; d++) {
#pragma unroll
                    for (int i = 0; i < MT; i++) {
                        const bool last = d == 1 && i == MT - 1;
                        if (last) {
                            if constexpr (STEADY) {
                                asm volatile("" ::: "memory");
                                __builtin_amdgcn_s_waitcnt(0xc07f);
                                __builtin_amdgcn_s_barrier();
                                asm volatile("" ::: "memory");
                                fa8[0] = frag8(na, 0, wm);
                            }
                        } else if (i == MT - 1) {
                            fa8[0] = frag8(la, 1, wm);
                        } else {
                            fa8[(i + 1) & 1] = frag8(la, d, wm + (i + 1) * 32);
                        }
#pragma unroll
                        for (int j = 0; j < NT; j++) {
                            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa8[i & 1], fb8[j], acc[i][j], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
                            if (i == MT - 1) {
                                if (d == 0) fb8[j] = frag8(lb, 1, wn + j * 32);
                                else if constexpr (STEADY) fb8[j] = frag8(nb, 0, wn + j * 32);
                            }
                        }
                        if constexpr (STEADY) {
                            const int g = d * MT + i; // 0..6 before the barrier: 3, 2, 2, 2, 3, 2, 2 slots
                            if (g < 7) {
                                const int first = g < 1 ? 0 : g < 5 ? 3 + (g - 1) * 2 : 12 + (g - 5) * 2;
                                const int count = (g == 0 || g == 4) ? 3 : 2;
#pragma unroll
                                for (int c = 0; c < count; c++) slot(first + c);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
                if constexpr (!STEADY) __syncthreads();
                return;
            }
#pragma unroll
            for (int kc = 0; kc < S - 1; kc++) {
#pragma unroll
                for (int i = 0; i < MT; i++) {
                    frag_a(la, (kc + 1) & 1, kc + 1, i);
                    frag_b(lb, (kc + 1) & 1, kc + 1, i);
                    mma_row(kc & 1, i);
                    if constexpr (STEADY) {
                        // 16 slots over 12 groups: every third group takes two
                        const int g = kc * MT + i, first = g + (g + 2) / 3;
                        slot(first);
                        if (g % 3 == 0) slot(first + 1);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                if constexpr (!STEADY) {
                    if (kc == S / 2 - 1 && next) {
                        stage(ra, rb, cur ^ 1);
                        if (kt + 2 < nk) ask(ra, rb, kt + 2);
                    }
                }
            }
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): this wave's LDS stores have landed (loads in flight stay in flight)
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
#pragma unroll
            for (int i = 0; i < MT; i++) {
                if (next) {
                    frag_a(na, 0, 0, i);
                    frag_b(nb, 0, 0, i);
                }
                mma_row((S - 1) & 1, i);
                if constexpr (STEADY) __builtin_amdgcn_sched_barrier(0);
            }
        };
        static_assert(S % 2 == 0, "the last step multiplies from set 1 while set 0 is refilled");
        auto first_fragments = [&]() {
            if constexpr (HALF == 5) {
                fa8[0] = frag8(lds_a(0), 0, wm);
#pragma unroll
                for (int j = 0; j < NT; j++) fb8[j] = frag8(lds_b(0), 0, wn + j * 32);
            } else {
#pragma unroll
                for (int i = 0; i < MT; i++) {
                    frag_a(lds_a(0), 0, 0, i);
                    frag_b(lds_b(0), 0, 0, i);
                }
            }
        };
        uint32_t kt = 0;
        if (lean && 3 * BK <= Kk) {
            // tile 1 is asked for slot by slot in the order the loop consumes the slots: only then does the compiler's count
            // of loads in flight at the loop's head match the one at its end, and each LDS store waits for its own load
            // (all but the 15 younger ones) instead of for every load
            const char *pa = reinterpret_cast<const char *>(A + (uint64_t)BK), *pb = reinterpret_cast<const char *>(B + (uint64_t)BK);
#pragma unroll
            for (int h = 0; h < 8; h++) {
                ra.v[h] = *reinterpret_cast<const float4v *>(pa + offa[h]);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int h = 0; h < 8; h++) {
                rb.v[h] = *reinterpret_cast<const float4v *>(pb + offb[h]);
                __builtin_amdgcn_sched_barrier(0);
            }
            first_fragments();
            for (; (kt + 3) * BK <= Kk; kt++) iteration(kt, std::true_type{});
        } else {
            if (nk > 1) ask(ra, rb, 1); // (tile 0 is in LDS buffer 0 by now)
            if constexpr (HALF != 5) first_fragments();
        }
        for (; kt < nk; kt++) iteration(kt, std::false_type{});
    }
    // Operands whose 16-byte loads are legal everywhere (aligned, unit stride along k or along the rows): a lane's slots keep
    // their place in every tile, so its byte offsets into the operands are fixed (rows beyond the edge clamped: their values
    // land in accumulator rows that are never stored) and a whole tile is loaded without a test per slot, at a base that
    // moves by one tile.  (The generic loader's tests and fallbacks cost the 256 x 256 tile 4 % of its time.)
    uint32_t offa_kk[TileRegs<BM>::slots], offb_kk[TileRegs<BN>::slots];
    bool lean_kk = false;
    // (The 256 x 256 tile with both operands row-contiguous, or with one such operand narrowed to bfloat16, has no registers
    // left for the offsets.)
    constexpr bool LEAN = !PACKED && (MT != 4 || (!(A_MFAST && B_NFAST) && !((A_MFAST || B_NFAST) && HALF == 1)));
    if constexpr (LEAN) {
        const bool a_ok = A_MFAST ? (a.a_vec && a.a_sm == 1 && a.M % 4 == 0 && a.M >= 4) : (a.a_vec && a.a_sk == 1 && a.a_sm > 0);
        const bool b_ok = B_NFAST ? (a.b_vec && a.b_sn == 1 && a.N % 4 == 0 && a.N >= 4) : (a.b_vec && a.b_sk == 1 && a.b_sn > 0);
        const uint64_t a_span = A_MFAST ? (uint64_t)Kk * (uint64_t)a.a_sk : (uint64_t)a.M * (uint64_t)a.a_sm;
        const uint64_t b_span = B_NFAST ? (uint64_t)Kk * (uint64_t)a.b_sk : (uint64_t)a.N * (uint64_t)a.b_sn;
        lean_kk = a_ok && b_ok && a.a_sk > 0 && a.b_sk > 0 && a_span < (1ull << 30) && b_span < (1ull << 30); // offsets fit 32 bits
#pragma unroll
        for (int h = 0; h < TileRegs<BM>::slots; h++) {
            const uint32_t slot = threadIdx.x + h * kThreads;
            if constexpr (A_MFAST) {
                uint32_t row, k;
                rows_fast_slot<BM>(slot, row, k);
                offa_kk[h] = (uint32_t)(((uint64_t)k * (uint64_t)a.a_sk + min(m0 + row, a.M - 4)) * 4);
            } else {
                offa_kk[h] = (uint32_t)(((uint64_t)min(m0 + slot / (BK / 4), a.M - 1) * (uint64_t)a.a_sm + (slot % (BK / 4)) * 4) * 4);
            }
        }
#pragma unroll
        for (int h = 0; h < TileRegs<BN>::slots; h++) {
            const uint32_t slot = threadIdx.x + h * kThreads;
            if constexpr (B_NFAST) {
                uint32_t row, k;
                rows_fast_slot<BN>(slot, row, k);
                offb_kk[h] = (uint32_t)(((uint64_t)k * (uint64_t)a.b_sk + min(n0 + row, a.N - 4)) * 4);
            } else {
                offb_kk[h] = (uint32_t)(((uint64_t)min(n0 + slot / (BK / 4), a.N - 1) * (uint64_t)a.b_sn + (slot % (BK / 4)) * 4) * 4);
            }
        }
    }
    auto iterate = [&](const uint32_t kt, auto whole_next) {
        const uint32_t cur = kt & 1;
        const bool more = decltype(whole_next)::value || kt + 1 < nk;
        const float *la = lds_a(cur), *lb = lds_b(cur);
        // One 8-deep chunk of the tile: lane group g supplies k = 8*kc + 4*g + t to the t-th MFMA,
        // for A and B alike, so one 128-bit LDS read feeds four MFMAs.
        auto chunk = [&](const int kc) {
            float4v fa[MT], fb[NT];
#pragma unroll
            for (int i = 0; i < MT; i++) {
                if constexpr (A_MFAST) {
#pragma unroll
                    for (int t = 0; t < 4; t++) fa[i][t] = la[(kc * 8 + lg * 4 + t) * BM + wm + i * 32 + li];
                } else {
                    fa[i] = *reinterpret_cast<const float4v *>(la + (wm + i * 32 + li) * PITCH + kc * 8 + lg * 4);
                }
            }
#pragma unroll
            for (int j = 0; j < NT; j++) {
                if constexpr (B_NFAST) {
#pragma unroll
                    for (int t = 0; t < 4; t++) fb[j][t] = lb[(kc * 8 + lg * 4 + t) * BN + wn + j * 32 + li];
                } else {
                    fb[j] = *reinterpret_cast<const float4v *>(lb + (wn + j * 32 + li) * PITCH + kc * 8 + lg * 4);
                }
            }
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int j = 0; j < NT; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][t], fb[j][t], acc[i][j], 0, 0, 0);
        };
        // While a wave is in its burst of matrix instructions it wins issue arbitration against the other
        // wave of its SIMD (which is loading or storing a tile): the two stop advancing in lock-step and
        // their stalls at the barrier no longer coincide.
        if constexpr (decltype(whole_next)::value) {
            // the next tile is a whole tile of k-contiguous, aligned operands: no test per slot
            const char *pa = reinterpret_cast<const char *>(A + (uint64_t)(kt + 1) * BK * (A_MFAST ? (uint64_t)a.a_sk : 1ull));
            const char *pb = reinterpret_cast<const char *>(B + (uint64_t)(kt + 1) * BK * (B_NFAST ? (uint64_t)a.b_sk : 1ull));
#pragma unroll
            for (int h = 0; h < TileRegs<BM>::slots; h++) ra.v[h] = *reinterpret_cast<const float4v *>(pa + offa_kk[h]);
#pragma unroll
            for (int h = 0; h < TileRegs<BN>::slots; h++) rb.v[h] = *reinterpret_cast<const float4v *>(pb + offb_kk[h]);
        } else if (more) {
            load_tile<A_MFAST>(ra, A, a.a_sm, a.a_sk, m0, (kt + 1) * BK, a.M, Kk, a.a_vec);
            load_tile<B_NFAST>(rb, B, a.b_sn, a.b_sk, n0, (kt + 1) * BK, a.N, Kk, a.b_vec);
        }
        __builtin_amdgcn_s_setprio(1);
        if constexpr (WIDEN) {
            // 16-deep chunks: lane group g supplies k = 16*kc + 8*g .. + 7, one 128-bit LDS read per operand block
#pragma unroll
            for (int kc = 0; kc < BK / 16; kc++) {
                float4v fa[MT], fb[NT];
#pragma unroll
                for (int i = 0; i < MT; i++)
                    fa[i] = *reinterpret_cast<const float4v *>(la + (wm + i * 32 + li) * PITCH_H + kc * 8 + lg * 4);
#pragma unroll
                for (int j = 0; j < NT; j++)
                    fb[j] = *reinterpret_cast<const float4v *>(lb + (wn + j * 32 + li) * PITCH_H + kc * 8 + lg * 4);
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int j = 0; j < NT; j++) {
                        if constexpr (HALF == 1)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[i]),
                                                                                __builtin_bit_cast(bf16x8, fb[j]), acc[i][j], 0, 0, 0);
                        else
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fa[i]),
                                                                               __builtin_bit_cast(f16x8, fb[j]), acc[i][j], 0, 0, 0);
                    }
            }
        } else if constexpr (MT == 4) {
            // one wave per SIMD: nobody else fills the time the staging of the next tile takes (for a row-contiguous
            // operand 4-byte LDS stores and their addresses), so it goes between the two halves of the burst, by when
            // the tile's global loads have long arrived; the other LDS buffer is written, the current one read
#pragma unroll
            for (int kc = 0; kc < BK / 16; kc++) chunk(kc);
            if (more) stage(ra, rb, cur ^ 1);
#pragma unroll
            for (int kc = BK / 16; kc < BK / 8; kc++) chunk(kc);
        } else {
#pragma unroll
            for (int kc = 0; kc < BK / 8; kc++) chunk(kc);
        }
        __builtin_amdgcn_s_setprio(0);
        if (more && (HALF || MT != 4)) stage(ra, rb, cur ^ 1);
        __syncthreads();
        };
    {
        uint32_t kt = 0;
        if constexpr (LEAN) {
            if (lean_kk)
                for (; (kt + 2) * BK <= Kk; kt++) iterate(kt, std::true_type{});
        }
        for (; kt < (PACKED ? 0u : nk); kt++) iterate(kt, std::false_type{});
    }

    // D layout of v_mfma_f32_32x32x2_f32: lane (li, lg), register v -> row 8*(v/4) + 4*lg + v%4, col li
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++) {
            uint32_t col = n0 + wn + j * 32 + li;
            if (col < a.N) {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    uint32_t row = m0 + wm + i * 32 + 8 * (v / 4) + 4 * lg + (v % 4);
                    if (row < a.M) C[(uint64_t)row * a.N + col] = asu(acc[i][j][v]);
                }
            }
        }
}

// ------------------------------------------------------------------------------------------
// The 256 x 256 tile of operands that lie narrow in memory, fed by loads that go from memory straight into LDS
// (global_load_lds_dwordx4): no tile registers, no LDS stores, so what a workgroup has in flight is bounded by LDS
// instead of by registers.  The register-staged kernel above keeps one tile step (64 KB) in flight per compute unit
// and a step lasts as long as a trip to memory (about 2 us under load, 31 GB/s per unit, whatever the matrix pipes
// could take); here a step is 64 bytes of k per row (32 values of 16 bits, 64 of fp8), a stage is 32 KB and LDS holds a
// ring of kDldsStages of them: one being multiplied, the others in flight.
// A row's 64 bytes are four 16-byte columns; column c of row r sits at column c ^ ((r >> 2) & 3) of the row's place, so
// that the sixteen lanes that a 128-bit fragment read serves at a time (sixteen consecutive rows, one logical column)
// cover all 64 banks (counted: no bank conflicts; with (r >> 1) & 3, which spreads eight rows over 32 banks, every read
// took two turns).  A load instruction of a wave fills 1 KB = 16 consecutive rows in lane order: lane l fetches row
// l / 4, logical column (l % 4) ^ ((row >> 2) & 3).
// HALF: 3 bfloat16, 4 binary16 (two 16-deep steps per stage), 5 fp8 (one 64-deep step per stage).  a.K counts 32-bit
// words and is a multiple of 64 (whole turns of the ring); rows beyond the edge are clamped as above.
// ------------------------------------------------------------------------------------------
constexpr int kDldsStages = 4;
constexpr uint32_t kDldsOperandBytes = 256 * 64, kDldsStageBytes = 2 * kDldsOperandBytes;
constexpr size_t kDldsLdsBytes = (size_t)kDldsStages * kDldsStageBytes;

template <int HALF, bool NARROW_OUT> __global__ __launch_bounds__(kThreads) void mfma_gemm_dlds_kernel(const MmArgs a) {
    constexpr int NS = kDldsStages;
    static_assert(NS == 4, "the last stages of a tile below are written out for a ring of four");
    extern __shared__ float lds_dyn[];
    typedef __attribute__((address_space(3))) char lds_char;
    lds_char *const lds = (lds_char *)lds_dyn;

    // Tile order as in mfma_gemm_kernel: a run of tiles per XCD, down a column of kGroupM row tiles first.  The grid is one
    // workgroup per compute unit (or per tile if there are fewer); workgroup b takes tiles b, b + grid, b + 2 grid, ...
    const uint32_t tiles_n = (a.N + 255) / 256, tiles_m = (a.M + 255) / 256;
    const uint32_t ntiles = tiles_m * tiles_n;
    auto tile_origin = [&](const uint32_t vb, uint32_t &m0, uint32_t &n0) {
        const uint32_t xcd = vb % kXcds, slot = vb / kXcds;
        const uint32_t q = ntiles / kXcds, r = ntiles % kXcds;
        const uint32_t lin = xcd * q + (xcd < r ? xcd : r) + slot;
        const uint32_t per_group = kGroupM * tiles_n;
        const uint32_t group = lin / per_group, in_group = lin % per_group;
        const uint32_t first_m = group * kGroupM;
        const uint32_t gsize = (tiles_m - first_m) < kGroupM ? (tiles_m - first_m) : kGroupM;
        m0 = (first_m + in_group % gsize) * 256;
        n0 = (in_group / gsize) * 256;
    };

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
    const uint32_t wm = (wave / 2) * 128, wn = (wave % 2) * 128;
    const uint32_t li = lane % 32, lg = lane / 32;

    // this lane's share of a stage: instruction q of wave w fills rows 64 w + 16 q .. + 15 of an operand's place
    uint32_t offa[4], offb[4];
    auto set_offa = [&](const uint32_t m0) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t row = wave * 64 + q * 16 + lane / 4, col = (lane % 4) ^ ((row >> 2) & 3);
            offa[q] = (uint32_t)((uint64_t)min(m0 + row, a.M - 1) * (uint64_t)a.a_sm * 4 + col * 16);
        }
    };
    auto set_offb = [&](const uint32_t n0) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t row = wave * 64 + q * 16 + lane / 4, col = (lane % 4) ^ ((row >> 2) & 3);
            offb[q] = (uint32_t)((uint64_t)min(n0 + row, a.N - 1) * (uint64_t)a.b_sn * 4 + col * 16);
        }
    };
    const char *const ga = reinterpret_cast<const char *>(a.A), *const gb = reinterpret_cast<const char *>(a.B);
    // load q of stage kt (of the tile whose offsets are set): 0..3 the four of A, 4..7 the four of B
    auto issue = [&](const uint32_t kt, const int q) {
        const char *const p = (q < 4 ? ga : gb) + (uint64_t)kt * 64 + (q < 4 ? offa[q & 3] : offb[q & 3]);
        lds_char *const l = lds + (kt % NS) * kDldsStageBytes + (q < 4 ? 0u : kDldsOperandBytes) + wave * 4096 + (q & 3) * 1024;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)p, (__attribute__((address_space(3))) void *)l, 16, 0, 0);
    };
    // fragment addresses: row li of a 32-row block, logical column c -> byte li * 64 + ((c ^ sw) * 16)
    const uint32_t sw = (li >> 2) & 3;
    auto frag = [&](const uint32_t stage_base, const uint32_t row0, const uint32_t c) {
        return *reinterpret_cast<const __attribute__((address_space(3))) float4v *>(lds + stage_base + (row0 + li) * 64 + ((c ^ sw) * 16));
    };

    float16v acc[4][4];
    auto clear = [&]() {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
    };
    // D layout of the 32 x 32 instructions: lane (li, lg), register v -> row 8 (v / 4) + 4 lg + v % 4, column li.  A whole
    // tile is stored at a per-lane 32-bit offset from addresses that are the same for every lane (M N < 2^30).
    // With NARROW_OUT the result is rounded to the operands' format here (what the separate rounding pass over the f32 result
    // would give, bit for bit) and stored as its patterns, a quarter or an eighth of the bytes of that f32 result and pass:
    // lanes exchange values so that each stores 32 bits — two columns of one row (16-bit: lanes pair up, the even lane takes
    // the first of two rows, the odd lane the second) or four (fp8: a quad transposes its 4 x 4 values).
    auto pattern = [&](const float x) -> uint32_t {
        if constexpr (HALF == 3) return round_bf16_bits(asu(x)) >> 16;
        else if constexpr (HALF == 4) return (uint32_t)__half_as_ushort(__float2half_rn(x));
        else return (uint32_t)f8_byte_of(round_f8_bits(asu(x)));
    };
    const uint32_t lane_off = ((wm + 4 * lg) * a.N + wn + li) * 4;
    const uint32_t sub = HALF == 5 ? (li & 3) : (li & 1); // this lane's row among the 4 (2) that its group exchanges
    const uint32_t lane_off_narrow = ((wm + 4 * lg + sub) * a.N + wn + li - sub) * (HALF == 5 ? 1 : 2);
    // v_perm_b32 selectors of the quad's transposition (byte values 0..3: the second source's bytes, 4..7: the first's, 12: zero)
    const uint32_t quad_sel_a = (0x0C0C0C0Cu & ~(0xFFu << (8 * sub)) & ~(0xFFu << (8 * ((sub + 1) & 3)))) | (sub << (8 * sub)) | ((4 + sub) << (8 * ((sub + 1) & 3)));
    const uint32_t quad_sel_b = (0x0C0C0C0Cu & ~(0xFFu << (8 * ((sub + 2) & 3))) & ~(0xFFu << (8 * ((sub + 3) & 3)))) | (sub << (8 * ((sub + 2) & 3))) |
                                ((4 + sub) << (8 * ((sub + 3) & 3)));
    auto store = [&](const uint32_t m0, const uint32_t n0) {
        const bool whole = m0 + 256 <= a.M && n0 + 256 <= a.N;
        if (whole && !NARROW_OUT) {
            char *const base = reinterpret_cast<char *>(a.C) + ((uint64_t)m0 * a.N + n0) * 4;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const uint32_t r = i * 32 + 8 * (v / 4) + (v % 4);
                        // (written out: the compiler would keep a 64-bit address per row in vector registers)
                        asm volatile("global_store_dword %0, %1, %2" ::"v"(lane_off), "v"(acc[i][j][v]), "s"(base + ((uint64_t)r * a.N + j * 32) * 4) : "memory");
                    }
                    __builtin_amdgcn_sched_barrier(0); // (a block at a time: its 16 values pass through 16 registers)
                }
            return;
        }
        if (whole) {
            constexpr uint32_t EB = HALF == 5 ? 1 : 2;
            char *const base = reinterpret_cast<char *>(a.C) + ((uint64_t)m0 * a.N + n0) * EB;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if constexpr (HALF != 5) {
#pragma unroll
                        for (int v = 0; v < 16; v += 2) {
                            // v_cvt_pk_{bf16,f16}_f32 round two values as the rounding pass does (all 2^32 patterns compared)
                            const float2v pair = {acc[i][j][v], acc[i][j][v + 1]};
                            uint32_t mine;
                            if constexpr (HALF == 3) mine = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
                            else mine = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, f16x2));
                            const uint32_t theirs = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0xB1, 0xF, 0xF, true); // the pair's other lane
                            // even lane: its and the other's first row; odd lane: the other's and its second row
                            const uint32_t two = __builtin_amdgcn_perm(theirs, mine, sub ? 0x03020706u : 0x05040100u);
                            const uint32_t r = i * 32 + 8 * (v / 4) + (v % 4);
                            asm volatile("global_store_dword %0, %1, %2" ::"v"(lane_off_narrow), "v"(two), "s"(base + ((uint64_t)r * a.N + j * 32) * 2) : "memory");
                        }
                    } else {
#pragma unroll
                        for (int v = 0; v < 16; v += 4) {
                            // v_cvt_pk_fp8_f32 rounds as the rounding pass does once the magnitude is clamped to 448 (it holds no
                            // infinities) and NaNs are set apart: they become the clamped pattern 0x7e, which the 0x7f below completes
                            // (all 2^32 patterns compared)
                            float xs[4];
                            uint32_t nans = 0;
#pragma unroll
                            for (int k = 0; k < 4; k++) {
                                const uint32_t u = asu(acc[i][j][v + k]), mag = u & 0x7FFFFFFFu;
                                xs[k] = asf(min(mag, 0x43E00000u) | (u & 0x80000000u));
                                nans |= mag > 0x7F800000u ? 0x7Fu << (8 * k) : 0u;
                            }
                            int packed = __builtin_amdgcn_cvt_pk_fp8_f32(xs[0], xs[1], 0, false);
                            packed = __builtin_amdgcn_cvt_pk_fp8_f32(xs[2], xs[3], packed, true);
                            const uint32_t mine = (uint32_t)packed | nans; // byte k: row k of this lane's column
                            // lane q of the quad keeps row q: byte q of every lane's word, at the place of that lane's column
                            const uint32_t r1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0x39, 0xF, 0xF, true); // of lane q + 1
                            const uint32_t r2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0x4E, 0xF, 0xF, true); // of lane q + 2
                            const uint32_t r3 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mine, 0x93, 0xF, 0xF, true); // of lane q + 3
                            const uint32_t four = __builtin_amdgcn_perm(r1, mine, quad_sel_a) | __builtin_amdgcn_perm(r3, r2, quad_sel_b);
                            const uint32_t r = i * 32 + 8 * (v / 4);
                            asm volatile("global_store_dword %0, %1, %2" ::"v"(lane_off_narrow), "v"(four), "s"(base + ((uint64_t)r * a.N + j * 32)) : "memory");
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t col = n0 + wn + j * 32 + li;
                if (col < a.N) {
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const uint32_t row = m0 + wm + i * 32 + 8 * (v / 4) + 4 * lg + (v % 4);
                        if (row < a.M) {
                            const uint64_t at = (uint64_t)row * a.N + col;
                            if constexpr (!NARROW_OUT) a.C[at] = asu(acc[i][j][v]);
                            else if constexpr (HALF == 5) reinterpret_cast<uint8_t *>(a.C)[at] = (uint8_t)pattern(acc[i][j][v]);
                            else reinterpret_cast<uint16_t *>(a.C)[at] = (uint16_t)pattern(acc[i][j][v]);
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
    };

    const uint32_t nk = a.K / 16; // a multiple of NS: stage kt of every tile sits in place kt % NS of the ring
    uint32_t vb = blockIdx.x, m0, n0;
    tile_origin(vb, m0, n0);
    set_offa(m0);
    set_offb(n0);
    // A wave's loads wait for each other in the texture path (a KB each), and while one waits the wave issues nothing:
    // they are dealt out one behind every group of matrix instructions.  The first half of stage kt asks for the second
    // half of the loads (B) of the stage 3 ahead, its second half (behind the barrier, when the place of stage kt is free) for
    // the first half (A) of the stage 4 ahead.  The stages of a workgroup's tiles form one stream: the last four stages of a
    // tile ask for the first stages of the next, and the matrix pipes pause at a tile's end only for the stores of the result.
#pragma unroll
    for (int s = 0; s < NS - 1; s++)
#pragma unroll
        for (int q = 0; q < 8; q++) issue(s, q);
#pragma unroll
    for (int q = 0; q < 4; q++) issue(NS - 1, q);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0f70 | (20 & 15) | ((20 >> 4) << 14)); // vmcnt(20): stage 0 is in LDS
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // wait until at most `stages` younger stages are in flight and every fragment read has returned, then meet the others:
    // the next stage is in LDS for everybody, and nobody reads the current stage's place any more.  (Loads finish in the
    // order asked for; the stores of a finished tile share the counter and only make the wait longer than needed.)
    auto meet = [&](auto stages) {
        constexpr uint32_t n = decltype(stages)::value * 8;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt(0x0070 | (n & 15) | ((n >> 4) << 14)); // vmcnt(n) lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    typedef std::integral_constant<int, 2> Y2;
    typedef std::true_type Ask;

    if constexpr (HALF != 5) {
        float4v fa[2][4], fb[2][4];
        auto mma_row = [&](const int set, const int i) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if constexpr (HALF == 3)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[set][i]),
                                                                        __builtin_bit_cast(bf16x8, fb[set][j]), acc[i][j], 0, 0, 0);
                else
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fa[set][i]),
                                                                       __builtin_bit_cast(f16x8, fb[set][j]), acc[i][j], 0, 0, 0);
            }
        };
        // step c of a stage: lane group g supplies the 8 values of k at 16 c + 8 g: logical column 2 c + g
        auto read = [&](const uint32_t kt, const int set, const int c, const int i) {
            const uint32_t base = (kt % NS) * kDldsStageBytes;
            fa[set][i] = frag(base, wm + i * 32, c * 2 + lg);
            fb[set][i] = frag(base + kDldsOperandBytes, wn + i * 32, c * 2 + lg);
        };
#pragma unroll
        for (int i = 0; i < 4; i++) read(0, 0, 0, i);
        // YOUNGER: stages younger than the next one that may still be in flight when this stage meets the others (-1: the
        // last stage of the last tile); FIRST / SECOND: the loads dealt out in the two halves are those of stages fkt / skt
        auto stage = [&](const uint32_t kt, auto younger, auto first, auto second, const uint32_t fkt, const uint32_t skt) {
            constexpr int YOUNGER = decltype(younger)::value;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                read(kt, 1, 1, i);
                mma_row(0, i);
                if constexpr (decltype(first)::value) issue(fkt, 4 + i);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (YOUNGER >= 0) meet(std::integral_constant<uint32_t, (uint32_t)(YOUNGER < 0 ? 0 : YOUNGER)>{});
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if constexpr (YOUNGER >= 0) read(kt + 1, 0, 0, i);
                mma_row(1, i);
                if constexpr (decltype(second)::value) issue(skt, i);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        for (;;) {
            // (a workgroup's last tile asks for its own first stages again: one way through the loop, and loads nobody reads)
            const uint32_t nvb = vb + gridDim.x;
            const bool more = nvb < ntiles;
            uint32_t nm0, nn0;
            tile_origin(more ? nvb : vb, nm0, nn0);
            clear();
            uint32_t kt = 0;
            for (; kt + NS < nk; kt++) stage(kt, Y2{}, Ask{}, Ask{}, kt + NS - 1, kt + NS);
            set_offa(nm0);
            stage(kt, Y2{}, Ask{}, Ask{}, kt + NS - 1, 0);
            set_offb(nn0);
            stage(kt + 1, Y2{}, Ask{}, Ask{}, 0, 1);
            stage(kt + 2, Y2{}, Ask{}, Ask{}, 1, 2);
            stage(kt + 3, Y2{}, Ask{}, Ask{}, 2, 3);
            store(m0, n0);
            if (!more) break;
            vb = nvb, m0 = nm0, n0 = nn0;
        }
    } else {
        // fp8: a lane feeds the 64-deep instruction 32 bytes of its row — logical columns g and 2 + g (A and B agree on
        // which bytes of the 64 they are).  The fragments of a stage sit in one of two register sets, the stage's parity;
        // the next stage's are read behind the barrier, under the second half of this stage's instructions.
        int8v fa8[2][4], fb8[2][4];
        auto read8 = [&](const uint32_t kt, const int set, const int i) {
            const uint32_t base = (kt % NS) * kDldsStageBytes;
            const int4v alo = __builtin_bit_cast(int4v, frag(base, wm + i * 32, lg)), ahi = __builtin_bit_cast(int4v, frag(base, wm + i * 32, 2 + lg));
            fa8[set][i] = __builtin_shufflevector(alo, ahi, 0, 1, 2, 3, 4, 5, 6, 7);
            const int4v blo = __builtin_bit_cast(int4v, frag(base + kDldsOperandBytes, wn + i * 32, lg)),
                        bhi = __builtin_bit_cast(int4v, frag(base + kDldsOperandBytes, wn + i * 32, 2 + lg));
            fb8[set][i] = __builtin_shufflevector(blo, bhi, 0, 1, 2, 3, 4, 5, 6, 7);
        };
        auto mma8 = [&](const int set, const int i, const int j) {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa8[set][i], fb8[set][j], acc[i][j], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
        };
#pragma unroll
        for (int i = 0; i < 4; i++) read8(0, 0, i);
        // (a load behind every second matrix instruction, which is twice as long as a 16-bit one)
        auto stage8 = [&](const uint32_t kt, const int set, auto younger, auto first, auto second, const uint32_t fkt, const uint32_t skt) {
            constexpr int YOUNGER = decltype(younger)::value;
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    mma8(set, i, 2 * h);
                    mma8(set, i, 2 * h + 1);
                    if constexpr (decltype(first)::value) issue(fkt, 4 + 2 * i + h);
                    __builtin_amdgcn_sched_barrier(0);
                }
            if constexpr (YOUNGER >= 0) meet(std::integral_constant<uint32_t, (uint32_t)(YOUNGER < 0 ? 0 : YOUNGER)>{});
#pragma unroll
            for (int i = 2; i < 4; i++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    if constexpr (YOUNGER >= 0) read8(kt + 1, set ^ 1, 2 * (i - 2) + h);
                    mma8(set, i, 2 * h);
                    mma8(set, i, 2 * h + 1);
                    if constexpr (decltype(second)::value) issue(skt, 2 * (i - 2) + h);
                    __builtin_amdgcn_sched_barrier(0);
                }
        };
        for (;;) {
            const uint32_t nvb = vb + gridDim.x;
            const bool more = nvb < ntiles;
            uint32_t nm0, nn0;
            tile_origin(more ? nvb : vb, nm0, nn0);
            clear();
            uint32_t kt = 0;
            for (; kt + NS < nk; kt += 2) {
                stage8(kt, 0, Y2{}, Ask{}, Ask{}, kt + NS - 1, kt + NS);
                stage8(kt + 1, 1, Y2{}, Ask{}, Ask{}, kt + NS, kt + NS + 1);
            }
            set_offa(nm0);
            stage8(kt, 0, Y2{}, Ask{}, Ask{}, kt + NS - 1, 0);
            set_offb(nn0);
            stage8(kt + 1, 1, Y2{}, Ask{}, Ask{}, 0, 1);
            stage8(kt + 2, 0, Y2{}, Ask{}, Ask{}, 1, 2);
            stage8(kt + 3, 1, Y2{}, Ask{}, Ask{}, 2, 3);
            store(m0, n0);
            if (!more) break;
            vb = nvb, m0 = nm0, n0 = nn0;
        }
    }
    // (loads into LDS must not outlive the workgroup: its LDS passes to the next one)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070); // vmcnt(0) lgkmcnt(0)
}

// ------------------------------------------------------------------------------------------
// Skinny kernel: M <= 8, B rows K-contiguous (b_sk == 1).  One wave per output column.
// ------------------------------------------------------------------------------------------
template <int MM> __global__ __launch_bounds__(kThreads) void skinny_kt_kernel(const MmArgs a) {
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t n = blockIdx.x * (kThreads / 64) + wave;
    if (n >= a.N) return;
    int64_t oa, ob;
    batch_offsets(a, blockIdx.y, oa, ob);
    const uint32_t *A = a.A + oa;
    const uint32_t *Brow = a.B + ob + (int64_t)n * a.b_sn;
    float acc[MM];
#pragma unroll
    for (int m = 0; m < MM; m++) acc[m] = 0.0f;
    const bool vec = a.b_vec && a.a_vec && a.a_sk == 1 && (a.K % 4 == 0);
    if (vec) {
        for (uint32_t k = lane * 4; k < a.K; k += 256) {
            float4v b = *reinterpret_cast<const float4v *>(Brow + k);
#pragma unroll
            for (int m = 0; m < MM; m++) {
                if ((uint32_t)m < a.M) {
                    float4v x = *reinterpret_cast<const float4v *>(A + (int64_t)m * a.a_sm + k);
                    acc[m] = fmaf(x[0], b[0], acc[m]);
                    acc[m] = fmaf(x[1], b[1], acc[m]);
                    acc[m] = fmaf(x[2], b[2], acc[m]);
                    acc[m] = fmaf(x[3], b[3], acc[m]);
                }
            }
        }
    } else {
        for (uint32_t k = lane; k < a.K; k += 64) {
            float b = asf(Brow[k]);
#pragma unroll
            for (int m = 0; m < MM; m++)
                if ((uint32_t)m < a.M) acc[m] = fmaf(asf(A[(int64_t)m * a.a_sm + (int64_t)k * a.a_sk]), b, acc[m]);
        }
    }
#pragma unroll
    for (int m = 0; m < MM; m++) {
        float v = acc[m];
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) v += __shfl_xor(v, s);
        if (lane == 0 && (uint32_t)m < a.M) a.C[((uint64_t)blockIdx.y * a.M + m) * a.N + n] = asu(v);
    }
}


// Vectorised skinny kernel for K > 256: a wave owns COLS output columns and walks K with
// 16-byte loads (COLS weight loads + M activation loads in flight per lane per trip; the
// activation rows stay in L1/L2).  SPLIT: the four waves of the block share the columns
// and split K, for shapes with too few columns to fill the chip.
// A sum of four terms one of which is the product: out = (t0 + (t1 + t2)) + t3 (order 0) or
// t0 + ((t1 + t2) + t3) (order 1), term[slot] being x.B^T and the others dense tensors of the
// output's shape.  The residual adds of a decoder layer run in the store of the o / down projection.
struct MmResidual {
    const uint32_t *term[4];
    uint32_t slot, order;
    uint32_t nterms;  // 4, or 2: out = t0 + t1
    float *partials;  // null, or [workgroups][4]: per row the sum of squares of the four columns stored
};
// the sum, given all its terms
__device__ __forceinline__ uint32_t residual_sum(const MmResidual &r, const uint32_t (&t)[4]) {
    if (r.nterms == 2) return apply<kAdd, true>(t[0], t[1], 0, nullptr);
    const uint32_t inner = apply<kAdd, true>(t[1], t[2], 0, nullptr);
    return r.order == 0 ? apply<kAdd, true>(apply<kAdd, true>(t[0], inner, 0, nullptr), t[3], 0, nullptr)
                        : apply<kAdd, true>(t[0], apply<kAdd, true>(inner, t[3], 0, nullptr), 0, nullptr);
}

#ifndef CG_WIDE_UNROLL
#define CG_WIDE_UNROLL 2
#endif
template <int MM, int COLS, bool SPLIT, bool RESIDUAL = false>
__device__ __forceinline__ void skinny_kt_wide_body(const MmArgs &a, const uint32_t block_x, const uint32_t block_y,
                                                    const MmResidual *res = nullptr) {
    static_assert(!RESIDUAL || (COLS == 1 && !SPLIT), "the residual store is written for one column per wave");
    constexpr int kWideUnroll = COLS == 1 ? CG_WIDE_UNROLL : 2;
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t group = SPLIT ? block_x : block_x * 4 + wave;
    const uint32_t n0 = group * COLS;
    const bool live = n0 < a.N;
    int64_t oa, ob;
    batch_offsets(a, block_y, oa, ob);
    const uint32_t *A = a.A + oa;
    const uint32_t *B = a.B + ob;
    uint32_t term[RESIDUAL ? MM : 1][4] = {};
    if constexpr (RESIDUAL) {
        // asked for before the walk along K, used after it
        if (live && lane == 0) {
#pragma unroll
            for (int m = 0; m < MM; m++)
#pragma unroll
                for (int t = 0; t < 4; t++)
                    if ((uint32_t)m < a.M && (uint32_t)t != res->slot && (uint32_t)t < res->nterms)
                        term[m][t] = res->term[t][((uint64_t)block_y * a.M + m) * a.N + n0];
        }
    }
    float acc[COLS][MM];
#pragma unroll
    for (int c = 0; c < COLS; c++)
#pragma unroll
        for (int m = 0; m < MM; m++) acc[c][m] = 0.0f;
    if (live) {
        const uint32_t kstep = SPLIT ? 1024u : 256u;
#pragma unroll kWideUnroll
        for (uint32_t k = (SPLIT ? wave * 256u : 0u) + lane * 4; k < a.K; k += kstep) {
            float4v w[COLS], x[MM];
#pragma unroll
            for (int c = 0; c < COLS; c++) {
                w[c] = (float4v){0.f, 0.f, 0.f, 0.f};
                if (n0 + c < a.N) w[c] = *reinterpret_cast<const float4v *>(B + (int64_t)(n0 + c) * a.b_sn + k);
            }
#pragma unroll
            for (int m = 0; m < MM; m++) {
                x[m] = (float4v){0.f, 0.f, 0.f, 0.f};
                if ((uint32_t)m < a.M) x[m] = *reinterpret_cast<const float4v *>(A + (int64_t)m * a.a_sm + k);
            }
#pragma unroll
            for (int c = 0; c < COLS; c++)
#pragma unroll
                for (int m = 0; m < MM; m++) {
                    acc[c][m] = fmaf(x[m][0], w[c][0], acc[c][m]);
                    acc[c][m] = fmaf(x[m][1], w[c][1], acc[c][m]);
                    acc[c][m] = fmaf(x[m][2], w[c][2], acc[c][m]);
                    acc[c][m] = fmaf(x[m][3], w[c][3], acc[c][m]);
                }
        }
    }
#pragma unroll
    for (int c = 0; c < COLS; c++)
#pragma unroll
        for (int m = 0; m < MM; m++) {
#pragma unroll
            for (int s = 32; s >= 1; s >>= 1) acc[c][m] += __shfl_xor(acc[c][m], s);
        }
    if (SPLIT) {
        __shared__ float part[4][COLS * MM];
        if (lane == 0) {
#pragma unroll
            for (int c = 0; c < COLS; c++)
#pragma unroll
                for (int m = 0; m < MM; m++) part[wave][c * MM + m] = acc[c][m];
        }
        __syncthreads();
        if (threadIdx.x < COLS * MM) {
            uint32_t c = threadIdx.x / MM, m = threadIdx.x % MM;
            float v = (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
            if (n0 + c < a.N && m < a.M) a.C[((uint64_t)block_y * a.M + m) * a.N + n0 + c] = asu(v);
        }
    } else if (live && lane == 0) {
#pragma unroll
        for (int c = 0; c < COLS; c++)
#pragma unroll
            for (int m = 0; m < MM; m++)
                if (n0 + c < a.N && (uint32_t)m < a.M) {
                    uint32_t v = asu(acc[c][m]);
                    if constexpr (RESIDUAL) {
                        uint32_t t[4];
#pragma unroll
                        for (int i = 0; i < 4; i++) t[i] = (uint32_t)i == res->slot ? v : term[m][i];
                        v = residual_sum(*res, t);
                    }
                    a.C[((uint64_t)block_y * a.M + m) * a.N + n0 + c] = v;
                }
    }
}

template <int MM, int COLS, bool SPLIT>
__global__ __launch_bounds__(kThreads) void skinny_kt_wide_kernel(const MmArgs a) {
    skinny_kt_wide_body<MM, COLS, SPLIT>(a, blockIdx.x, blockIdx.y);
}

template <int MM> __global__ __launch_bounds__(kThreads) void skinny_kt_wide_residual_kernel(const MmArgs a, const MmResidual r) {
    skinny_kt_wide_body<MM, 1, false, true>(a, blockIdx.x, blockIdx.y, &r);
}

// Several products that share their left operand (the q / k / v projections of a decode step,
// gate and up) in one launch: the workgroups are dealt to the problems in order.
// Products too narrow for eight columns per workgroup still gain from the matrix-instruction kernel at four
// columns per workgroup (one activation load per lane and trip instead of M) when its 2048-wide chunks of k are full.
// With a single row it is 0.7 us behind the one-column-per-wave kernel at K = 2048 and level with it at K = 8192;
// it is used all the same, because its residual store and its norm-applying loads save two launches per layer.
// Chunks of 2048 values of k when K is a multiple of that, of 1024 when of that (hidden sizes like 1024 or 3072); any
// other K (a multiple of 4 above 256: hidden sizes like 576 or 1536) runs with a ragged last chunk, the waves of a
// workgroup then interleaved every 64 values of k (xreg_lane_k) so that a short chunk still spreads over all four.
static inline int xreg_trips(uint32_t K) {
    return K % 2048 == 0 ? 8 : K % 1024 == 0 ? 4 : (K % 4 == 0 && K > 256) ? (K > 1024 ? 8 : 4) : 0;
}
// Column groups per workgroup of the one-chunk gated kernel: as many as leave about two workgroups per compute unit
// (env CG_XREG_ITERS=n forces n, for measurements).
static inline uint32_t xreg_cols_iters(uint64_t groups) {
    static const int forced = [] {
        const char *e = getenv("CG_XREG_ITERS");
        return e ? atoi(e) : 0;
    }();
    if (forced > 0) return (uint32_t)forced;
    const uint64_t it = groups / 512;
    return (uint32_t)(it < 1 ? 1 : it > 4 ? 4 : it);
}
static inline bool xreg_narrow(uint32_t M, uint32_t K) { return M >= 1 && M <= 4 && xreg_trips(K) != 0; }
constexpr int kMaxGroup = 4;
struct MmGroup {
    MmArgs p[kMaxGroup];
    uint32_t first[kMaxGroup + 1]; // first workgroup of each problem; first[n] = grid size
    uint32_t n;
};
__device__ __forceinline__ uint32_t group_problem(const MmGroup &g, uint32_t &block_x) {
    // every slot of the prefix table is compared (the problems are in increasing order of their first workgroup), so the
    // table is read from the argument block at once instead of one dependent scalar load per problem
    uint32_t p = 0;
#pragma unroll
    for (int i = 1; i < kMaxGroup; i++) p += (uint32_t)i < g.n && blockIdx.x >= g.first[i] ? 1u : 0u;
    block_x = blockIdx.x - g.first[p];
    return p;
}
template <int MM> __global__ __launch_bounds__(kThreads) void skinny_kt_wide_group_kernel(const MmGroup g) {
    uint32_t bx;
    const uint32_t p = group_problem(g, bx);
    skinny_kt_wide_body<MM, 1, false>(g.p[p], bx, 0);
}

// Skinny kernel on the 4x4x1 matrix instruction (16 independent 4x4 outer products per
// issue): lane (b, j) = (lane / 4, lane % 4) feeds weight W[n0 + j][k] and activation
// X[j][k] for the k values of block b, so one 16-byte weight load per lane drives four
// instructions that update all 4 (rows) x 4 (columns) partial sums of the block.  Against
// the FMA kernels this needs a quarter of the vector issue slots.  The four waves of a
// workgroup split each 2048-wide chunk of k into runs of 512 (a wave reads 2 KiB in a row of
// each weight row: measured 12 % faster on the gate / up pair than interleaving the waves
// every 256 bytes), keep their share of the chunk's activations in registers (8 x 16 bytes
// per lane and row group) and reuse it for CG groups of four columns, so the activation rows
// are fetched once per 4 * CG columns.
// RESIDUAL (CG = 1): the store adds the other terms of a four-term sum, as skinny_kt_wide_residual_kernel does.
// GATED (CG = 2): the two column groups are the same four columns of two weight matrices, a.B and
// `second` (same shape and strides), and the block writes g * (1 / (one + exp(-g))) * u for
// g = x.B^T, u = x.second^T: the SiLU-gated pair of an MLP block without writing g and u.
// pow(sum / n + eps, e): the divisor of an RMS norm from its row's sum of squares, in the program's own ops
__device__ __forceinline__ uint32_t norm_divisor(const NormFuse &nf, float sum) {
    const uint32_t mean = apply<kDiv, true>(asu(sum), nf.n_bits, 0, nullptr);
    return apply<kPow, true>(apply<kAdd, true>(mean, nf.eps_bits, 0, nullptr), nf.exp_bits, 0, nullptr);
}
// Where a lane's k values lie inside a chunk of TRIPS * 256: trip t covers k0 + kb + ks * t .. + 3.  Whole chunks: a wave
// takes a quarter of the chunk in a row (2 KiB in a row of each weight row: measured 12 % faster on the gate / up pair than
// interleaving the waves every 256 bytes).  A ragged last chunk: the waves interleaved every 64 values of k, so that what
// there is of the chunk is shared by all four.
// WHOLE: K is known to be whole chunks (the kernels branch once, at their top: loads without a test per trip).
template <int TRIPS, bool WHOLE = false> __device__ __forceinline__ void xreg_lane_k(uint32_t K, uint32_t wave, uint32_t b, uint32_t &kb, uint32_t &ks) {
    const bool ragged = !WHOLE && K % (TRIPS * 256) != 0;
    kb = (ragged ? wave * 64 : wave * (TRIPS * 64)) + b * 4;
    ks = ragged ? 256u : 64u;
}
template <bool WHOLE, int MM, int CG, bool GATED, bool RESIDUAL, bool NORM, int TRIPS>
__device__ __forceinline__ void skinny_kt_mfma_xreg_body_impl(const MmArgs &a, const uint32_t block_x, const uint32_t block_y, const uint32_t *second,
                                                              const uint32_t one, const MmResidual *res, const NormFuse *nf) {
    static_assert(!NORM || MM == 4, "the norm's row sums are kept for four rows");
    static_assert(!GATED || CG == 2, "a gated pair is two column groups");
    static_assert(!(GATED && RESIDUAL), "one epilogue at a time");
    constexpr int G = MM / 4;
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t j = lane % 4, b = lane / 4;
    const uint32_t n0 = block_x * (GATED ? 4 : 4 * CG);
    int64_t oa, ob;
    batch_offsets(a, block_y, oa, ob);
    const uint32_t *wrow[CG];
#pragma unroll
    for (int c = 0; c < CG; c++)
        wrow[c] = GATED ? (c == 0 ? a.B : second) + ob + (int64_t)min(n0 + j, a.N - 1) * a.b_sn
                        : a.B + ob + (int64_t)min(n0 + 4 * c + j, a.N - 1) * a.b_sn;
    const uint32_t *xrow[G];
#pragma unroll
    for (int g = 0; g < G; g++) xrow[g] = a.A + oa + (int64_t)min((uint32_t)(4 * g) + j, a.M - 1) * a.a_sm;
    float4v acc[CG][G];
#pragma unroll
    for (int c = 0; c < CG; c++)
#pragma unroll
        for (int g = 0; g < G; g++) acc[c][g] = (float4v){0.f, 0.f, 0.f, 0.f};
    // the sum's other terms for the value this thread will store: asked for before the walk along K
    uint32_t term[4] = {};
    if constexpr (RESIDUAL) {
        if (threadIdx.x < CG * MM * 4) {
            const uint32_t c = threadIdx.x / (MM * 4), m = threadIdx.x / 4 % MM, col = n0 + 4 * c + threadIdx.x % 4;
            if (col < a.N && m < a.M) {
#pragma unroll
                for (int t = 0; t < 4; t++)
                    if ((uint32_t)t != res->slot && (uint32_t)t < res->nterms)
                        term[t] = res->term[t][((uint64_t)block_y * a.M + m) * a.N + col];
            }
        }
    }
    // NORM: the products are taken of x * gamma and divided by d_m = pow(sum(x[m]^2) / n + eps, e) where they are stored:
    // (x / d * gamma) . w = ((x * gamma) . w) / d.  The row sums are put together from the partial sums that the kernel
    // which stored x left (always in the same order); thread t takes entries t, t + 256, ... of [blocks][4], all of row
    // t % 4.  The first eight per thread are asked for here and added up after the walk along K: nothing waits for them.
    float pv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if constexpr (NORM) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const uint32_t i = threadIdx.x + u * kThreads;
            if (i < nf->blocks * 4) pv[u] = nf->partials[i];
        }
    }
    // of every chunk of TRIPS * 256 values of k (2048 or 1024) a wave takes a quarter in a row (TRIPS trips of 64)
    static_assert(TRIPS == 8 || TRIPS == 4, "chunks of 2048 or 1024");
    uint32_t kb, ks;
    xreg_lane_k<TRIPS, WHOLE>(a.K, wave, b, kb, ks);
    for (uint32_t k0 = 0; k0 < a.K; k0 += TRIPS * 256) {
        float4v xr[G][TRIPS];
#pragma unroll
        for (int t = 0; t < TRIPS; t++) {
            const uint32_t k = k0 + kb + ks * t;
#pragma unroll
            for (int g = 0; g < G; g++) {
                xr[g][t] = (float4v){0.f, 0.f, 0.f, 0.f};
                if (WHOLE || k < a.K) xr[g][t] = *reinterpret_cast<const float4v *>(xrow[g] + k);
            }
        }
        float4v gm[NORM ? TRIPS : 1]; // asked for with the activations, multiplied in once the first weights are on their way
        if constexpr (NORM) {
#pragma unroll
            for (int t = 0; t < TRIPS; t++) {
                const uint32_t k = k0 + kb + ks * t;
                gm[t] = (float4v){0.f, 0.f, 0.f, 0.f};
                if (WHOLE || k < a.K) gm[t] = *reinterpret_cast<const float4v *>(nf->gamma + k);
            }
        }
#pragma unroll
        for (int c = 0; c < CG; c++) {
            float4v w[TRIPS];
#pragma unroll
            for (int t = 0; t < TRIPS; t++) {
                const uint32_t k = k0 + kb + ks * t;
                w[t] = (float4v){0.f, 0.f, 0.f, 0.f};
                if (WHOLE || k < a.K) w[t] = *reinterpret_cast<const float4v *>(wrow[c] + k);
            }
            if constexpr (NORM) {
                if (c == 0) {
#pragma unroll
                    for (int t = 0; t < TRIPS; t++)
#pragma unroll
                        for (int g = 0; g < G; g++)
#pragma unroll
                            for (int e = 0; e < 4; e++) xr[g][t][e] = asf(apply<kMul, true>(asu(xr[g][t][e]), asu(gm[t][e]), 0, nullptr));
                }
            }
#pragma unroll
            for (int t = 0; t < TRIPS; t++)
#pragma unroll
                for (int g = 0; g < G; g++) {
                    acc[c][g] = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[g][t][0], w[t][0], acc[c][g], 0, 0, 0);
                    acc[c][g] = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[g][t][1], w[t][1], acc[c][g], 0, 0, 0);
                    acc[c][g] = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[g][t][2], w[t][2], acc[c][g], 0, 0, 0);
                    acc[c][g] = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[g][t][3], w[t][3], acc[c][g], 0, 0, 0);
                }
        }
    }
    __shared__ float part[4][CG * MM * 4];
    __shared__ float nsum[4][4];
    if constexpr (NORM) {
        float s = 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) s += pv[u];
        for (uint32_t i = threadIdx.x + 8 * kThreads; i < nf->blocks * 4; i += kThreads) s += nf->partials[i];
#pragma unroll
        for (int sh = 32; sh >= 4; sh >>= 1) s += __shfl_xor(s, sh);
        if (lane < 4) nsum[wave][lane] = s;
    }
#pragma unroll
    for (int c = 0; c < CG; c++)
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float v = acc[c][g][i];
#pragma unroll
                for (int s = 32; s >= 4; s >>= 1) v += __shfl_xor(v, s);
                if (lane < 4) part[wave][(c * MM + 4 * g + i) * 4 + j] = v;
            }
    __syncthreads();
    if constexpr (GATED) {
        if (threadIdx.x < MM * 4) {
            const uint32_t t = threadIdx.x, u_at = MM * 4 + t, m = t / 4, col = n0 + t % 4;
            uint32_t gv = asu((part[0][t] + part[1][t]) + (part[2][t] + part[3][t]));
            uint32_t uv = asu((part[0][u_at] + part[1][u_at]) + (part[2][u_at] + part[3][u_at]));
            if constexpr (NORM) {
                const uint32_t d = norm_divisor(*nf, (nsum[0][m % 4] + nsum[1][m % 4]) + (nsum[2][m % 4] + nsum[3][m % 4]));
                gv = apply<kDiv, true>(gv, d, 0, nullptr);
                uv = apply<kDiv, true>(uv, d, 0, nullptr);
            }
            // the ops of the deferred program, in its order
            const uint32_t e = apply<kExp, true>(apply<kNeg, true>(gv, 0, 0, nullptr), 0, 0, nullptr);
            const uint32_t sg = apply<kDiv, true>(one, apply<kAdd, true>(one, e, 0, nullptr), 0, nullptr);
            const uint32_t r = apply<kMul, true>(apply<kMul, true>(gv, sg, 0, nullptr), uv, 0, nullptr);
            if (col < a.N && m < a.M) a.C[((uint64_t)block_y * a.M + m) * a.N + col] = r;
        }
    } else if (threadIdx.x < CG * MM * 4) {
        const uint32_t c = threadIdx.x / (MM * 4), m = threadIdx.x / 4 % MM, col = n0 + 4 * c + threadIdx.x % 4;
        uint32_t v = asu((part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]));
        if constexpr (NORM)
            v = apply<kDiv, true>(v, norm_divisor(*nf, (nsum[0][m % 4] + nsum[1][m % 4]) + (nsum[2][m % 4] + nsum[3][m % 4])), 0, nullptr);
        if constexpr (RESIDUAL) {
#pragma unroll
            for (int t = 0; t < 4; t++) term[t] = (uint32_t)t == res->slot ? v : term[t];
            v = residual_sum(*res, term);
        }
        const bool stored = col < a.N && m < a.M;
        if (stored) a.C[((uint64_t)block_y * a.M + m) * a.N + col] = v;
        if constexpr (RESIDUAL) {
            // threads 0..15 = (row m, column n0 + t % 4): the row's sum of squares over the block's four columns
            if (res->partials) {
                float q = stored ? asf(v) * asf(v) : 0.0f;
                q += __shfl_xor(q, 1);
                q += __shfl_xor(q, 2);
                if (threadIdx.x % 4 == 0) res->partials[(uint64_t)block_x * 4 + m] = q;
            }
        }
    }
}
template <int MM, int CG, bool GATED = false, bool RESIDUAL = false, bool NORM = false, int TRIPS = 8>
__device__ __forceinline__ void skinny_kt_mfma_xreg_body(const MmArgs &a, const uint32_t block_x, const uint32_t block_y,
                                                         const uint32_t *second = nullptr, const uint32_t one = 0,
                                                         const MmResidual *res = nullptr, const NormFuse *nf = nullptr) {
    if (a.K % (TRIPS * 256) == 0) skinny_kt_mfma_xreg_body_impl<true, MM, CG, GATED, RESIDUAL, NORM, TRIPS>(a, block_x, block_y, second, one, res, nf);
    else skinny_kt_mfma_xreg_body_impl<false, MM, CG, GATED, RESIDUAL, NORM, TRIPS>(a, block_x, block_y, second, one, res, nf);
}

template <int MM, int CG, int TRIPS = 8> __global__ __launch_bounds__(kThreads) void skinny_kt_mfma_xreg_kernel(const MmArgs a) {
    skinny_kt_mfma_xreg_body<MM, CG, false, false, false, TRIPS>(a, blockIdx.x, blockIdx.y);
}
template <int MM, int TRIPS = 8>
__global__ __launch_bounds__(kThreads) void skinny_kt_mfma_xreg_gated_kernel(const MmArgs a, const uint32_t *second, uint32_t one) {
    skinny_kt_mfma_xreg_body<MM, 2, true, false, false, TRIPS>(a, blockIdx.x, blockIdx.y, second, one);
}
template <int MM, int TRIPS = 8>
__global__ __launch_bounds__(kThreads) void skinny_kt_mfma_xreg_residual_kernel(const MmArgs a, const MmResidual r) {
    skinny_kt_mfma_xreg_body<MM, 1, false, true, false, TRIPS>(a, blockIdx.x, blockIdx.y, nullptr, 0, &r);
}
// the same with the RMS norm of the left operand applied on load
template <int TRIPS = 8>
__global__ __launch_bounds__(kThreads) void skinny_kt_mfma_xreg_gated_norm_kernel(const MmArgs a, const uint32_t *second, uint32_t one,
                                                                                  const NormFuse nf) {
    skinny_kt_mfma_xreg_body<4, 2, true, false, true, TRIPS>(a, blockIdx.x, blockIdx.y, second, one, nullptr, &nf);
}
template <int MM, int CG, int TRIPS = 8> __global__ __launch_bounds__(kThreads) void skinny_kt_mfma_xreg_group_kernel(const MmGroup g) {
    uint32_t bx;
    const uint32_t p = group_problem(g, bx);
    skinny_kt_mfma_xreg_body<MM, CG, false, false, false, TRIPS>(g.p[p], bx, 0);
}
template <int TRIPS = 8>
__global__ __launch_bounds__(kThreads) void skinny_kt_mfma_xreg_group_norm_kernel(const MmGroup g, const NormFuse nf) {
    uint32_t bx;
    const uint32_t p = group_problem(g, bx);
    skinny_kt_mfma_xreg_body<4, 1, false, false, true, TRIPS>(g.p[p], bx, 0, nullptr, 0, nullptr, &nf);
}

// The grouped products of an attention block's decode step (q, k, v: a few rows, the same left operand) with the
// rotary embedding and the move into the KV cache done where they are stored: a workgroup owns two groups of four
// columns half a head apart (the pair the embedding mixes; next to each other for a product stored as it is) and
// writes column n = head * hd + d of row m to dst[m * sb + head * sh + d] (see RopeStore).  The embedding's ops are
// those of the deferred program cos * x + sin * concat(-x2, x1), in its order.  M <= 4, K a multiple of TRIPS * 256,
// N a multiple of hd (of 8 without the embedding).
struct RopeGroup {
    RopeStore s[kMaxGroup];
};
template <bool WHOLE, bool NORM, int TRIPS>
__device__ __forceinline__ void skinny_kt_mfma_xreg_group_rope_impl(const MmGroup &g, const RopeGroup &rg, const NormFuse &nf) {
    static_assert(TRIPS == 8 || TRIPS == 4, "chunks of 2048 or 1024");
    uint32_t bx;
    const uint32_t p = group_problem(g, bx);
    const MmArgs &a = g.p[p];
    const RopeStore &rs = rg.s[p];
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t j = lane % 4, b = lane / 4;
    const uint32_t span = rs.rope ? rs.hd : 8, per = span / 8;
    const uint32_t n0 = bx / per * span + bx % per * 4;
    const uint32_t nc[2] = {n0, n0 + span / 2};
    const uint32_t *wrow[2];
#pragma unroll
    for (int c = 0; c < 2; c++) wrow[c] = a.B + (int64_t)min(nc[c] + j, a.N - 1) * a.b_sn;
    const uint32_t *xrow = a.A + (int64_t)min(j, a.M - 1) * a.a_sm;
    float4v acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    // the embedding's factors for the value this thread will store: asked for before the walk along K
    uint32_t cs = 0, sn = 0;
    if (rs.rope && threadIdx.x < 32) {
        const uint32_t d = (nc[threadIdx.x / 16] + threadIdx.x % 4) % rs.hd;
        cs = rs.cos[d];
        sn = rs.sin[d];
    }
    float pv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if constexpr (NORM) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const uint32_t i = threadIdx.x + u * kThreads;
            if (i < nf.blocks * 4) pv[u] = nf.partials[i];
        }
    }
    uint32_t kb, ks;
    xreg_lane_k<TRIPS, WHOLE>(a.K, wave, b, kb, ks);
    // (a value of k beyond K contributes zeros: only a ragged last chunk has any)
    auto at = [&](const uint32_t *row, uint32_t k) {
        float4v v = {0.f, 0.f, 0.f, 0.f};
        if (WHOLE || k < a.K) v = *reinterpret_cast<const float4v *>(row + k);
        return v;
    };
    for (uint32_t k0 = 0; k0 < a.K; k0 += TRIPS * 256) {
        float4v xr[TRIPS];
#pragma unroll
        for (int t = 0; t < TRIPS; t++) xr[t] = at(xrow, k0 + kb + ks * t);
        float4v gm[NORM ? TRIPS : 1];
        if constexpr (NORM) {
#pragma unroll
            for (int t = 0; t < TRIPS; t++) gm[t] = at(nf.gamma, k0 + kb + ks * t);
        }
#pragma unroll
        for (int c = 0; c < 2; c++) {
            float4v w[TRIPS];
#pragma unroll
            for (int t = 0; t < TRIPS; t++) w[t] = at(wrow[c], k0 + kb + ks * t);
            if constexpr (NORM) {
                if (c == 0) {
#pragma unroll
                    for (int t = 0; t < TRIPS; t++)
#pragma unroll
                        for (int e = 0; e < 4; e++) xr[t][e] = asf(apply<kMul, true>(asu(xr[t][e]), asu(gm[t][e]), 0, nullptr));
                }
            }
#pragma unroll
            for (int t = 0; t < TRIPS; t++) {
                acc[c] = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[t][0], w[t][0], acc[c], 0, 0, 0);
                acc[c] = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[t][1], w[t][1], acc[c], 0, 0, 0);
                acc[c] = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[t][2], w[t][2], acc[c], 0, 0, 0);
                acc[c] = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[t][3], w[t][3], acc[c], 0, 0, 0);
            }
        }
    }
    __shared__ float part[4][32];
    __shared__ float nsum[4][4];
    if constexpr (NORM) {
        float s = 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) s += pv[u];
        for (uint32_t i = threadIdx.x + 8 * kThreads; i < nf.blocks * 4; i += kThreads) s += nf.partials[i];
#pragma unroll
        for (int sh = 32; sh >= 4; sh >>= 1) s += __shfl_xor(s, sh);
        if (lane < 4) nsum[wave][lane] = s;
    }
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float v = acc[c][i];
#pragma unroll
            for (int s = 32; s >= 4; s >>= 1) v += __shfl_xor(v, s);
            if (lane < 4) part[wave][(c * 4 + i) * 4 + j] = v;
        }
    __syncthreads();
    if (threadIdx.x < 64) { // the first wave: lanes 0..31 hold (column group, row, column), the others idle along
        const uint32_t t = threadIdx.x % 32, c = t / 16, m = t / 4 % 4, col = nc[c] + t % 4;
        uint32_t v = asu((part[0][t] + part[1][t]) + (part[2][t] + part[3][t]));
        if constexpr (NORM) v = apply<kDiv, true>(v, norm_divisor(nf, (nsum[0][m] + nsum[1][m]) + (nsum[2][m] + nsum[3][m])), 0, nullptr);
        const uint32_t other = __shfl_xor(v, 16); // the same row's column half a head away
        if (rs.rope) {
            // lower half: rotate_half reads -x[d + hd / 2]; upper half: x[d - hd / 2]
            const uint32_t rot = c == 0 ? apply<kNeg, true>(other, 0, 0, nullptr) : other;
            v = apply<kAdd, true>(apply<kMul, true>(cs, v, 0, nullptr), apply<kMul, true>(sn, rot, 0, nullptr), 0, nullptr);
        }
        if (threadIdx.x < 32 && col < a.N && m < a.M) rs.dst[(int64_t)m * rs.sb + (int64_t)(col / rs.hd) * rs.sh + col % rs.hd] = v;
    }
}
template <bool NORM, int TRIPS>
__global__ __launch_bounds__(kThreads) void skinny_kt_mfma_xreg_group_rope_kernel(const MmGroup g, const RopeGroup rg, const NormFuse nf) {
    if (g.p[0].K % (TRIPS * 256) == 0) skinny_kt_mfma_xreg_group_rope_impl<true, NORM, TRIPS>(g, rg, nf); // (the problems of a group share k)
    else skinny_kt_mfma_xreg_group_rope_impl<false, NORM, TRIPS>(g, rg, nf);
}

// The store above for products whose heads go through an RMS norm of their own first (RopeStore::hgamma, the q / k norm of
// Qwen3): the norm needs the sum of squares over all hd columns of a head, which lie with hd / 8 workgroups of the
// eight-columns-per-workgroup kernel, and workgroups cannot exchange values inside a launch for less than a launch costs.
// So that kernel leaves those products plain (rows already divided by the input norm) in scratch memory, N columns a row,
// and this small launch finishes them: a workgroup per head of a product, a thread per (row, column) of the head; the
// head's norm, the embedding and the store, op for op as the stand-alone programs.  Measured against one launch with a
// workgroup of 1024 threads per head (a compute unit streams about 25 GB/s on its own however deep its loads are queued,
// so that launch is as slow as its heads are few: 23 to 29 us for the 32 heads of 128 x 1024 of the Qwen3-0.6B shape):
// 9 + 3 us and a hand-over, 1.94 -> 1.66 ms per decode step of that shape.
struct HeadFinish {
    RopeStore s[kMaxGroup];
    const uint32_t *src[kMaxGroup];
    uint32_t N[kMaxGroup];
    uint32_t first[kMaxGroup + 1]; // prefix sums of the products' head counts
    uint32_t n, M;
};
constexpr int kFinishThreads = 512;
__global__ __launch_bounds__(kFinishThreads) void head_norm_rope_finish_kernel(const HeadFinish f) {
    uint32_t p = 0;
    while (p + 1 < f.n && blockIdx.x >= f.first[p + 1]) p++;
    const uint32_t head = blockIdx.x - f.first[p];
    const RopeStore &rs = f.s[p];
    const uint32_t e = threadIdx.x, m = e / rs.hd, d = e % rs.hd;
    const bool mine = e < f.M * rs.hd; // (M <= 4, hd <= 128: at most 512 threads)
    uint32_t hg = 0, cs = 0, sn = 0, v = 0;
    if (mine) v = f.src[p][(int64_t)m * f.N[p] + head * rs.hd + d];
    if (mine && rs.hgamma) hg = rs.hgamma[d];
    if (mine && rs.rope) {
        cs = rs.cos[d];
        sn = rs.sin[d];
    }
    __shared__ float hv[4][128], hy[4][128];
    if (rs.hgamma) { // (the same for the whole workgroup)
        if (mine) hv[m][d] = asf(v);
        __syncthreads();
        if (mine) {
            float ss = 0.0f; // the row's sum of squares, its columns in order
            for (uint32_t c = 0; c < rs.hd; c++) ss += hv[m][c] * hv[m][c];
            const uint32_t mean = apply<kDiv, true>(asu(ss), rs.hn_n_bits, 0, nullptr);
            const uint32_t r = apply<kPow, true>(apply<kAdd, true>(mean, rs.hn_eps_bits, 0, nullptr), rs.hn_exp_bits, 0, nullptr);
            v = apply<kMul, true>(apply<kDiv, true>(v, r, 0, nullptr), hg, 0, nullptr);
        }
    }
    if (rs.rope) {
        if (mine) hy[m][d] = asf(v);
        __syncthreads();
        if (mine) {
            // lower half: rotate_half reads -x[d + hd / 2]; upper half: x[d - hd / 2]
            const bool low = d < rs.hd / 2;
            const uint32_t other = asu(hy[m][low ? d + rs.hd / 2 : d - rs.hd / 2]);
            const uint32_t rot = low ? apply<kNeg, true>(other, 0, 0, nullptr) : other;
            v = apply<kAdd, true>(apply<kMul, true>(cs, v, 0, nullptr), apply<kMul, true>(sn, rot, 0, nullptr), 0, nullptr);
        }
    }
    if (mine) rs.dst[(int64_t)m * rs.sb + (int64_t)head * rs.sh + d] = v;
}

// The gated pair when K is exactly one chunk (TRIPS * 256: the hidden size of the model): the workgroup asks for its
// share of the activations (and of gamma, and of the row sums of an RMS norm) ONCE and walks `iters` consecutive
// groups of four columns with them, the next group's weights always on their way while the current group is
// multiplied, reduced and stored.  Measured on the 1B-shape decode step: the activation, gamma and partial-sum loads
// of a workgroup that owns a single column group cost a fifth of the kernel's time although they all hit in L2 (they
// are three quarters as many bytes again as the weights); four groups per workgroup take 29.5 instead of 34.3 us for
// the 128 MiB of gate + up, more leave too few workgroups in flight.  For q / k / v and o (a quarter of the columns)
// one group per workgroup stays the fastest.  Weights are read with the non-temporal hint.
// M <= 4, batch folded away (one batch entry).  Epilogues as in skinny_kt_mfma_xreg_body.
template <bool WHOLE, bool NORM, int TRIPS>
__device__ __forceinline__ void skinny_kt_mfma_xreg_cols_gated_impl(const MmArgs &a, const uint32_t *second, uint32_t one, uint32_t iters, const NormFuse &nf) {
    static_assert(TRIPS == 8 || TRIPS == 4, "chunks of 2048 or 1024");
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t j = lane % 4, b = lane / 4;
    uint32_t kb, ks; // this lane's k: kb + ks t (beyond K, in a chunk that K does not fill: zeros)
    xreg_lane_k<TRIPS, WHOLE>(a.K, wave, b, kb, ks);
    const uint32_t *xrow = a.A + (int64_t)min(j, a.M - 1) * a.a_sm;
    float4v xr[TRIPS];
#pragma unroll
    for (int t = 0; t < TRIPS; t++) {
        xr[t] = (float4v){0.f, 0.f, 0.f, 0.f};
        if (WHOLE || kb + ks * t < a.K) xr[t] = *reinterpret_cast<const float4v *>(xrow + kb + ks * t);
    }
    float pv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float4v gm[NORM ? TRIPS : 1];
    if constexpr (NORM) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const uint32_t i = threadIdx.x + u * kThreads;
            if (i < nf.blocks * 4) pv[u] = nf.partials[i];
        }
#pragma unroll
        for (int t = 0; t < TRIPS; t++) {
            gm[t] = (float4v){0.f, 0.f, 0.f, 0.f};
            if (WHOLE || kb + ks * t < a.K) gm[t] = *reinterpret_cast<const float4v *>(nf.gamma + kb + ks * t);
        }
    }
    __shared__ float part[2][4][32];
    __shared__ float nsum[4][4];
    const uint32_t groups = (a.N + 3) / 4;
    float4v wg[TRIPS], wu[TRIPS]; // the group's four columns of the two weight matrices
    auto ask = [&](float4v (&w)[TRIPS], const uint32_t *base, uint32_t n0) {
        const uint32_t *row = base + (int64_t)min(n0 + j, a.N - 1) * a.b_sn + kb;
#pragma unroll
        for (int t = 0; t < TRIPS; t++) {
            w[t] = (float4v){0.f, 0.f, 0.f, 0.f};
            if (WHOLE || kb + ks * t < a.K) w[t] = __builtin_nontemporal_load(reinterpret_cast<const float4v *>(row + ks * t));
        }
    };
    auto multiply = [&](float4v &sum, const float4v (&w)[TRIPS]) {
#pragma unroll
        for (int t = 0; t < TRIPS; t++) {
            sum = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[t][0], w[t][0], sum, 0, 0, 0);
            sum = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[t][1], w[t][1], sum, 0, 0, 0);
            sum = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[t][2], w[t][2], sum, 0, 0, 0);
            sum = __builtin_amdgcn_mfma_f32_4x4x1f32(xr[t][3], w[t][3], sum, 0, 0, 0);
        }
    };
    const uint32_t first_grp = blockIdx.x * iters;
    if (first_grp >= groups) return; // the same for every thread of the workgroup
    ask(wg, a.B, first_grp * 4);
    if constexpr (NORM) {
        // (x / d * gamma) . w = ((x * gamma) . w) / d: gamma goes in once, while the first weights are on their way; the row
        // sums of squares are put together from the partial sums, always in the same order
#pragma unroll
        for (int t = 0; t < TRIPS; t++)
#pragma unroll
            for (int e = 0; e < 4; e++) xr[t][e] = asf(apply<kMul, true>(asu(xr[t][e]), asu(gm[t][e]), 0, nullptr));
        float s = 0.0f;
#pragma unroll
        for (int u = 0; u < 8; u++) s += pv[u];
        for (uint32_t i = threadIdx.x + 8 * kThreads; i < nf.blocks * 4; i += kThreads) s += nf.partials[i];
#pragma unroll
        for (int sh = 32; sh >= 4; sh >>= 1) s += __shfl_xor(s, sh);
        if (lane < 4) nsum[wave][lane] = s;
    }
    uint32_t divisor = 0;
    for (uint32_t it = 0; it < iters; it++) {
        const uint32_t grp = first_grp + it;
        if (grp >= groups) break;
        const uint32_t n0 = grp * 4;
        float4v acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
        ask(wu, second, n0);
        multiply(acc_g, wg);
        if (it + 1 < iters && grp + 1 < groups) ask(wg, a.B, n0 + 4); // on its way through the rest of this group
        multiply(acc_u, wu);
        float (*pt)[32] = part[it & 1];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float vg = acc_g[i], vu = acc_u[i];
#pragma unroll
            for (int s = 32; s >= 4; s >>= 1) {
                vg += __shfl_xor(vg, s);
                vu += __shfl_xor(vu, s);
            }
            if (lane < 4) {
                pt[wave][i * 4 + j] = vg;
                pt[wave][16 + i * 4 + j] = vu;
            }
        }
        __syncthreads(); // (the buffer written two groups ago was read before the barrier of the group in between)
        if (threadIdx.x < 16) {
            const uint32_t t = threadIdx.x, m = t / 4, col = n0 + t % 4;
            uint32_t gv = asu((pt[0][t] + pt[1][t]) + (pt[2][t] + pt[3][t]));
            uint32_t uv = asu((pt[0][16 + t] + pt[1][16 + t]) + (pt[2][16 + t] + pt[3][16 + t]));
            if constexpr (NORM) {
                if (it == 0) divisor = norm_divisor(nf, (nsum[0][m] + nsum[1][m]) + (nsum[2][m] + nsum[3][m]));
                gv = apply<kDiv, true>(gv, divisor, 0, nullptr);
                uv = apply<kDiv, true>(uv, divisor, 0, nullptr);
            }
            // the ops of the deferred program, in its order
            const uint32_t e = apply<kExp, true>(apply<kNeg, true>(gv, 0, 0, nullptr), 0, 0, nullptr);
            const uint32_t sg = apply<kDiv, true>(one, apply<kAdd, true>(one, e, 0, nullptr), 0, nullptr);
            const uint32_t r = apply<kMul, true>(apply<kMul, true>(gv, sg, 0, nullptr), uv, 0, nullptr);
            if (col < a.N && m < a.M) a.C[(uint64_t)m * a.N + col] = r;
        }
    }
}
template <bool NORM, int TRIPS>
__global__ __launch_bounds__(kThreads) void skinny_kt_mfma_xreg_cols_gated_kernel(const MmArgs a, const uint32_t *second, uint32_t one,
                                                                                  uint32_t iters, const NormFuse nf) {
    if (a.K % (TRIPS * 256) == 0) skinny_kt_mfma_xreg_cols_gated_impl<true, NORM, TRIPS>(a, second, one, iters, nf);
    else skinny_kt_mfma_xreg_cols_gated_impl<false, NORM, TRIPS>(a, second, one, iters, nf);
}

// Vectorised skinny kernel for short K (K <= 4*LPC, e.g. q.K^T of a decode step with
// K = head_dim): LPC lanes share a column, so a wave covers 64/LPC columns per pass and
// the activation fragment is loaded once.
template <int MM, int LPC> __global__ __launch_bounds__(kThreads) void skinny_kt_narrow_kernel(const MmArgs a) {
    constexpr uint32_t CPW = 64 / LPC, PASSES = 4;
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t sub = lane / LPC, l = lane % LPC;
    const uint32_t nblock = blockIdx.x * (4 * CPW * PASSES);
    int64_t oa, ob;
    batch_offsets(a, blockIdx.y, oa, ob);
    const uint32_t *A = a.A + oa;
    const uint32_t *B = a.B + ob;
    const uint32_t k = l * 4;
    const bool kin = k < a.K;
    float4v x[MM];
#pragma unroll
    for (int m = 0; m < MM; m++) {
        x[m] = (float4v){0.f, 0.f, 0.f, 0.f};
        if (kin && (uint32_t)m < a.M) x[m] = *reinterpret_cast<const float4v *>(A + (int64_t)m * a.a_sm + k);
    }
    float4v w[PASSES];
#pragma unroll
    for (uint32_t p = 0; p < PASSES; p++) {
        uint32_t col = nblock + (p * 4 + wave) * CPW + sub;
        w[p] = (float4v){0.f, 0.f, 0.f, 0.f};
        if (kin && col < a.N) w[p] = *reinterpret_cast<const float4v *>(B + (int64_t)col * a.b_sn + k);
    }
#pragma unroll
    for (uint32_t p = 0; p < PASSES; p++) {
        uint32_t col = nblock + (p * 4 + wave) * CPW + sub;
#pragma unroll
        for (int m = 0; m < MM; m++) {
            float v = fmaf(x[m][3], w[p][3], fmaf(x[m][2], w[p][2], fmaf(x[m][1], w[p][1], x[m][0] * w[p][0])));
#pragma unroll
            for (int s = LPC / 2; s >= 1; s >>= 1) v += __shfl_xor(v, s);
            if (l == 0 && col < a.N && (uint32_t)m < a.M) a.C[((uint64_t)blockIdx.y * a.M + m) * a.N + col] = asu(v);
        }
    }
}

// Skinny kernel for N-contiguous B (p.V of a decode step: M = 1, K = T, N = head_dim):
// a block owns 64 output columns (16 lanes x float4) and splits K over 16 lane groups,
// which an LDS exchange sums at the end.
template <int MM>
__global__ __launch_bounds__(kThreads) void skinny_nn_kernel(const MmArgs a, uint32_t *dst, uint32_t kchunk) {
    const uint32_t ng = threadIdx.x % 16, kg = threadIdx.x / 16;
    const uint32_t n = blockIdx.x * 64 + ng * 4;
    int64_t oa, ob;
    batch_offsets(a, blockIdx.y, oa, ob);
    const uint32_t *A = a.A + oa;
    const uint32_t *B = a.B + ob;
    float4v acc[MM];
#pragma unroll
    for (int m = 0; m < MM; m++) acc[m] = (float4v){0.f, 0.f, 0.f, 0.f};
    const bool vec = a.b_vec && n + 3 < a.N;
    const uint32_t kbeg = blockIdx.z * kchunk, kend = min(a.K, kbeg + kchunk);
#pragma unroll 4
    for (uint32_t k = kbeg + kg; k < kend; k += 16) {
        const uint32_t *p = B + (int64_t)k * a.b_sk + (int64_t)n * a.b_sn;
        float4v w;
        if (vec) {
            w = *reinterpret_cast<const float4v *>(p);
        } else {
            w[0] = ld_guard(p, n < a.N);
            w[1] = ld_guard(p + a.b_sn, n + 1 < a.N);
            w[2] = ld_guard(p + 2 * a.b_sn, n + 2 < a.N);
            w[3] = ld_guard(p + 3 * a.b_sn, n + 3 < a.N);
        }
#pragma unroll
        for (int m = 0; m < MM; m++) {
            if ((uint32_t)m < a.M) {
                float x = asf(A[(int64_t)m * a.a_sm + (int64_t)k * a.a_sk]);
                acc[m][0] = fmaf(x, w[0], acc[m][0]);
                acc[m][1] = fmaf(x, w[1], acc[m][1]);
                acc[m][2] = fmaf(x, w[2], acc[m][2]);
                acc[m][3] = fmaf(x, w[3], acc[m][3]);
            }
        }
    }
    __shared__ float red[16][64 * MM + 4];
#pragma unroll
    for (int m = 0; m < MM; m++)
#pragma unroll
        for (int j = 0; j < 4; j++) red[kg][m * 64 + ng * 4 + j] = acc[m][j];
    __syncthreads();
    for (uint32_t o = threadIdx.x; o < 64 * MM; o += kThreads) {
        float v = 0.0f;
#pragma unroll
        for (int g = 0; g < 16; g++) v += red[g][o];
        uint32_t m = o / 64, col = blockIdx.x * 64 + o % 64;
        // dst is C itself (gridDim.z == 1) or the [batch][gridDim.z][M][N] partial sums
        if (m < a.M && col < a.N)
            dst[(((uint64_t)blockIdx.y * gridDim.z + blockIdx.z) * a.M + m) * a.N + col] = asu(v);
    }
}

// The same four elements at a time (mn a multiple of 4, both arrays 16-byte aligned): the sums in the same fixed order.
__global__ __launch_bounds__(kThreads) void splitk_reduce4_kernel(const float4v *part, float4v *C, uint32_t splits, uint32_t mn4, uint64_t total4) {
    const uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= total4) return;
    const uint64_t b = i / mn4, e = i % mn4;
    float4v v = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t s = 0; s < splits; s++) {
        const float4v p = __builtin_nontemporal_load(part + (b * splits + s) * mn4 + e);
        v[0] += p[0];
        v[1] += p[1];
        v[2] += p[2];
        v[3] += p[3];
    }
    C[i] = v;
}

// C[b][e] = sum over s of part[b][s][e]   (e < M*N)
__global__ __launch_bounds__(kThreads) void splitk_reduce_kernel(const uint32_t *part, uint32_t *C, uint32_t splits,
                                                                 uint32_t mn, uint64_t total) {
    uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= total) return;
    uint64_t b = i / mn, e = i % mn;
    float v = 0.0f;
    for (uint32_t s = 0; s < splits; s++) v += asf(part[(b * splits + s) * mn + e]);
    C[i] = asu(v);
}

// ------------------------------------------------------------------------------------------
// Plain kernel: one thread per output element.  u32 with wrapping arithmetic
// (ndarray.rs:181) and the f32 shapes nothing else takes.
// ------------------------------------------------------------------------------------------
template <bool F> __global__ __launch_bounds__(kThreads) void simple_gemm_kernel(const MmArgs a) {
    uint64_t e = (uint64_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= (uint64_t)a.M * a.N) return;
    uint32_t m = (uint32_t)(e / a.N), n = (uint32_t)(e % a.N);
    int64_t oa, ob;
    batch_offsets(a, blockIdx.y, oa, ob);
    const uint32_t *A = a.A + oa + (int64_t)m * a.a_sm;
    const uint32_t *B = a.B + ob + (int64_t)n * a.b_sn;
    uint32_t r;
    if (F) {
        float s = 0.0f;
        for (uint32_t k = 0; k < a.K; k++) s = fmaf(asf(A[(int64_t)k * a.a_sk]), asf(B[(int64_t)k * a.b_sk]), s);
        r = asu(s);
    } else {
        uint32_t s = 0;
        for (uint32_t k = 0; k < a.K; k++) s += A[(int64_t)k * a.a_sk] * B[(int64_t)k * a.b_sk];
        r = s;
    }
    a.C[(uint64_t)blockIdx.y * a.M * a.N + e] = r;
}

} // namespace

int fold_matmul(const cg_tensor *x, const cg_tensor *y, MmFold *f) {
    const int r = x->rank;
    int64_t M = x->dims[r - 2];
    auto stride = [](const cg_tensor *t, int ax) -> int64_t { return t->uniform ? 0 : t->strides[ax]; };
    f->a_sm = stride(x, r - 2);
    f->a_sk = stride(x, r - 1);
    f->b_sk = stride(y, r - 2);
    f->b_sn = stride(y, r - 1);
    // collapse the batch axes of A and B together (C is row-major, so it follows); a split axis of
    // either operand contributes its two parts as separate axes
    int64_t bd[kMaxRank + 1], sa[kMaxRank + 1], sb[kMaxRank + 1];
    int w = 0;
    auto push_axis = [&](int64_t d, int64_t s1, int64_t s2) {
        if (d == 1) return;
        if (w > 0 && sa[w - 1] == s1 * d && sb[w - 1] == s2 * d) {
            bd[w - 1] *= d;
            sa[w - 1] = s1;
            sb[w - 1] = s2;
        } else {
            bd[w] = d;
            sa[w] = s1;
            sb[w] = s2;
            w++;
        }
    };
    for (int i = 0; i < r - 2; i++) {
        const int64_t d = x->dims[i], s1 = stride(x, i), s2 = stride(y, i);
        const bool xs = x->split == i, ys = y->split == i;
        if (xs || ys) {
            const int64_t inner = xs ? x->split_inner : y->split_inner;
            push_axis(d / inner, xs ? x->split_os : s1 * inner, ys ? y->split_os : s2 * inner);
            push_axis(inner, s1, s2);
        } else {
            push_axis(d, s1, s2);
        }
    }
    // fold the innermost batch axis into M when B ignores it and A walks it as more rows
    while (w > 0 && sb[w - 1] == 0 && (M == 1 || sa[w - 1] == f->a_sm * M)) {
        if (M == 1) f->a_sm = sa[w - 1];
        M *= bd[w - 1];
        w--;
    }
    if (w > kMaxBatchAxes) return fail(CG_ERR_UNSUPPORTED, "matmul: more than %d non-mergeable batch axes", kMaxBatchAxes);
    int64_t batch = 1;
    for (int i = 0; i < w; i++) batch *= bd[i];
    f->M = M;
    f->N = y->dims[r - 1];
    f->K = x->dims[r - 1];
    f->batch = batch;
    f->nb = w;
    for (int d = 0; d < w; d++) {
        f->bd[d] = bd[w - 1 - d];
        f->a_bs[d] = sa[w - 1 - d];
        f->b_bs[d] = sb[w - 1 - d];
    }
    return CG_OK;
}

// Kernel arguments of x . y -> c (row-major); the folded extents come back in *f.
// The geometry of x . y (everything of MmArgs but the operands' addresses and what depends on them).
static int mm_geometry(const cg_tensor *x, const cg_tensor *y, void *c, MmArgs *ap, MmFold *fp) {
    MmArgs &a = *ap;
    memset(&a, 0, sizeof a);
    a.C = static_cast<uint32_t *>(c);
    MmFold &f = *fp;
    int rc = fold_matmul(x, y, &f);
    if (rc) return rc;
    const int64_t M = f.M, N = f.N, K = f.K, batch = f.batch;
    const int w = f.nb;
    a.a_sm = f.a_sm;
    a.a_sk = f.a_sk;
    a.b_sk = f.b_sk;
    a.b_sn = f.b_sn;
    if (M > 0x7FFFFFFFll || N > 0x7FFFFFFFll || K > 0x7FFFFFFFll || batch > 65535ll * 1024)
        return fail(CG_ERR_UNSUPPORTED, "matmul: extent above 2^31-1");
    a.M = (uint32_t)M;
    a.N = (uint32_t)N;
    a.K = (uint32_t)K;
    a.nb = (uint32_t)w;
    a.batch = (uint32_t)batch;
    for (int d = 0; d < w; d++) {
        a.bd[d] = (uint32_t)f.bd[d];
        a.bdiv[d] = make_fastdiv(a.bd[d]);
        a.a_bs[d] = f.a_bs[d];
        a.b_bs[d] = f.b_bs[d];
    }
    return CG_OK;
}

// The 32-bit words of one operand (`left`: x, else y) and whether 16-byte loads may run along its unit-stride axis.  An
// operand that lies in memory in a narrow format is read through its widened copy, unless the caller takes it as it
// lies (`native`: then the address stays null and the operand counts as unaligned).
static int mm_operand(const cg_tensor *t, bool left, bool native, MmArgs *ap) {
    MmArgs &a = *ap;
    const void *p = nullptr;
    if (!native) {
        int rc = device_ptr(t, &p);
        if (rc) return rc;
    }
    bool al = !native && reinterpret_cast<uintptr_t>(p) % 16 == 0;
    for (uint32_t d = 0; d < a.nb; d++)
        if ((left ? a.a_bs[d] : a.b_bs[d]) % 4) al = false;
    // 16-byte loads run along the unit-stride axis; the other axis' stride must keep alignment
    if (left) {
        a.A = static_cast<const uint32_t *>(p);
        const bool kfast = a.a_sk == 1 || a.K == 1, mfast = !kfast && a.a_sm == 1;
        a.a_vec = al && ((a.a_sk == 1 && a.a_sm % 4 == 0) || (mfast && a.a_sk % 4 == 0));
    } else {
        a.B = static_cast<const uint32_t *>(p);
        const bool kfast = a.b_sk == 1 || a.K == 1, nfast = !kfast && a.b_sn == 1;
        a.b_vec = al && ((a.b_sk == 1 && a.b_sn % 4 == 0) || (nfast && a.b_sk % 4 == 0));
    }
    return CG_OK;
}

static int make_mm_args(const cg_tensor *x, const cg_tensor *y, void *c, MmArgs *ap, MmFold *fp) {
    int rc = mm_geometry(x, y, c, ap, fp);
    if (!rc) rc = mm_operand(x, true, false, ap);
    if (!rc) rc = mm_operand(y, false, false, ap);
    return rc;
}

// The buffer that device_ptr's address of t lies in: the widened copy for a view of a narrow buffer.
static Buffer *words_buffer(const cg_tensor *t) { return is_narrow_buf(t->buf) ? t->buf->wide : t->buf; }

// May the [rows, K] view of t (row stride s_r, k stride s_k, in elements) be multiplied as it lies in memory, by the
// kernels of narrow kind `kind` (1 bf16, 2 f16, 3 fp8)?  Its buffer holds that very format, k is contiguous and every row
// starts on a 16-byte boundary.  dense: the rows must also follow each other without gaps.
static bool native_rows(const cg_tensor *t, int kind, int64_t s_r, int64_t s_k, int64_t K, bool dense) {
    if (!t->buf || t->uniform || t->buf->fmt != kind) return false;
    const int64_t eb = (int64_t)fmt_bytes(kind);
    if (s_k != 1 || s_r * eb % 16 != 0 || t->offset * eb % 16 != 0) return false;
    return !dense || s_r == K;
}
static const void *native_ptr(const cg_tensor *t) {
    return static_cast<const char *>(t->buf->ptr) + t->offset * (int64_t)fmt_bytes(t->buf->fmt);
}

int launch_matmul_group(cg_backend *be, const cg_tensor *x, const cg_tensor *const *ys, cg_tensor *const *outs, int n,
                        const NormFuse *nf) {
    if (int frc = flush_deferred(be)) return frc;
    if (n < (nf ? 1 : 2) || n > kMaxGroup || x->dt != CG_F32) return kDeclined;
    MmGroup g;
    memset(&g, 0, sizeof g);
    double bytes = distinct_bytes(x);
    bool all_wide = true;
    for (int i = 0; i < n; i++) {
        MmFold f;
        int rc = make_mm_args(x, ys[i], outs[i]->buf->ptr, &g.p[i], &f);
        if (rc) return rc;
        const MmArgs &a = g.p[i];
        const bool vec = a.a_vec && a.b_vec && a.a_sk == 1 && a.K % 4 == 0;
        if (f.batch != 1 || a.M > 8 || a.b_sk != 1 || !vec || a.K <= 256 || a.N < 4) return kDeclined;
        if (i > 0 && (a.M != g.p[0].M || a.K != g.p[0].K || a.a_sm != g.p[0].a_sm)) return kDeclined;
        all_wide = all_wide && a.N >= 8192;
        bytes += distinct_bytes(ys[i]) + distinct_bytes(outs[i]);
    }
    const bool xreg = !nf && all_wide && g.p[0].M <= 4;
    const bool xreg1 = !xreg && xreg_narrow(g.p[0].M, g.p[0].K);
    if (nf && !xreg1) return kDeclined;
    for (int i = 0; i < n && nf; i++)
        if (g.p[i].N >= 8192) return kDeclined; // a vocabulary-sized product: the kernel with more columns per wave, the norm on its own
    uint32_t blocks = 0;
    for (int i = 0; i < n; i++) {
        g.first[i] = blocks;
        blocks += xreg ? (g.p[i].N + 7) / 8 : (g.p[i].N + 3) / 4;
    }
    g.first[n] = blocks;
    g.n = (uint32_t)n;
    ProfScope prof(be, CG_K_GEMM_SKINNY, bytes);
    if (xreg)
        hipLaunchKernelGGL((skinny_kt_mfma_xreg_group_kernel<4, 2, 8>), dim3(blocks), dim3(kThreads), 0, be->stream, g);
    else if (nf && xreg_trips(g.p[0].K) == 8)
        hipLaunchKernelGGL(skinny_kt_mfma_xreg_group_norm_kernel<8>, dim3(blocks), dim3(kThreads), 0, be->stream, g, *nf);
    else if (nf)
        hipLaunchKernelGGL(skinny_kt_mfma_xreg_group_norm_kernel<4>, dim3(blocks), dim3(kThreads), 0, be->stream, g, *nf);
    else if (xreg1 && xreg_trips(g.p[0].K) == 8)
        hipLaunchKernelGGL((skinny_kt_mfma_xreg_group_kernel<4, 1, 8>), dim3(blocks), dim3(kThreads), 0, be->stream, g);
    else if (xreg1)
        hipLaunchKernelGGL((skinny_kt_mfma_xreg_group_kernel<4, 1, 4>), dim3(blocks), dim3(kThreads), 0, be->stream, g);
    else if (g.p[0].M <= 1)
        hipLaunchKernelGGL((skinny_kt_wide_group_kernel<1>), dim3(blocks), dim3(kThreads), 0, be->stream, g);
    else if (g.p[0].M <= 4)
        hipLaunchKernelGGL((skinny_kt_wide_group_kernel<4>), dim3(blocks), dim3(kThreads), 0, be->stream, g);
    else
        hipLaunchKernelGGL((skinny_kt_wide_group_kernel<8>), dim3(blocks), dim3(kThreads), 0, be->stream, g);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "grouped matmul launch");
}

int launch_matmul_group_rope(cg_backend *be, const cg_tensor *x, const cg_tensor *const *ys, const RopeStore *stores, int n,
                             const NormFuse *nf) {
    if (n < 1 || n > kMaxGroup || x->dt != CG_F32) return kDeclined;
    MmGroup g;
    RopeGroup rg;
    memset(&g, 0, sizeof g);
    memset(&rg, 0, sizeof rg);
    double bytes = distinct_bytes(x);
    uint32_t blocks = 0;
    bool by_head = false; // some product's heads are normed: two launches (see head_norm_rope_finish_kernel)
    for (int i = 0; i < n; i++) by_head = by_head || stores[i].hgamma != nullptr;
    for (int i = 0; i < n; i++) {
        MmFold f;
        int rc = make_mm_args(x, ys[i], stores[i].dst, &g.p[i], &f);
        if (rc) return rc;
        const MmArgs &a = g.p[i];
        const RopeStore &st = stores[i];
        const bool vec = a.a_vec && a.b_vec && a.a_sk == 1 && a.K % 4 == 0;
        if (f.batch != 1 || !xreg_narrow(a.M, a.K) || a.b_sk != 1 || !vec || a.N >= 8192) return kDeclined;
        if (i > 0 && (a.M != g.p[0].M || a.K != g.p[0].K || a.a_sm != g.p[0].a_sm)) return kDeclined;
        if (st.hd < 8 || st.hd % 8 || a.N % st.hd || !st.dst || (st.rope && (!st.cos || !st.sin))) return kDeclined;
        if (by_head && (st.hd % 16 || st.hd > 128)) return kDeclined;
        rg.s[i] = st;
        g.first[i] = blocks;
        blocks += a.N / 8;
        bytes += distinct_bytes(ys[i]) + 4.0 * (double)a.M * a.N;
    }
    g.first[n] = blocks;
    g.n = (uint32_t)n;
    NormFuse none;
    memset(&none, 0, sizeof none);
    const bool wide = xreg_trips(g.p[0].K) == 8;
    ProfScope prof(be, CG_K_GEMM_SKINNY, bytes);
    HeadFinish hf;
    void *tmp = nullptr;
    size_t tmp_cls = 0;
    uint32_t finish_heads = 0;
    if (by_head) { // the normed products go to scratch memory as they are (see head_norm_rope_finish_kernel)
        memset(&hf, 0, sizeof hf);
        hf.M = g.p[0].M;
        uint64_t words = 0;
        for (int i = 0; i < n; i++)
            if (stores[i].hgamma) words += (uint64_t)g.p[i].M * g.p[i].N;
        if (int arc = be->pool.alloc(words * 4, &tmp, &tmp_cls)) return arc;
        uint32_t *at = static_cast<uint32_t *>(tmp);
        uint32_t heads = 0;
        for (int i = 0; i < n; i++) {
            if (!stores[i].hgamma) continue;
            const uint32_t k = hf.n++;
            hf.s[k] = stores[i];
            hf.src[k] = at;
            hf.N[k] = g.p[i].N;
            hf.first[k] = heads;
            heads += g.p[i].N / stores[i].hd;
            RopeStore &plain = rg.s[i]; // column n of row m to at[m * N + n]
            plain.dst = at;
            plain.sb = g.p[i].N;
            plain.sh = stores[i].hd;
            plain.rope = 0;
            plain.hgamma = nullptr;
            at += (uint64_t)g.p[i].M * g.p[i].N;
        }
        hf.first[hf.n] = heads;
        finish_heads = heads;
    }
    if (nf && wide) hipLaunchKernelGGL((skinny_kt_mfma_xreg_group_rope_kernel<true, 8>), dim3(blocks), dim3(kThreads), 0, be->stream, g, rg, *nf);
    else if (nf) hipLaunchKernelGGL((skinny_kt_mfma_xreg_group_rope_kernel<true, 4>), dim3(blocks), dim3(kThreads), 0, be->stream, g, rg, *nf);
    else if (wide) hipLaunchKernelGGL((skinny_kt_mfma_xreg_group_rope_kernel<false, 8>), dim3(blocks), dim3(kThreads), 0, be->stream, g, rg, none);
    else hipLaunchKernelGGL((skinny_kt_mfma_xreg_group_rope_kernel<false, 4>), dim3(blocks), dim3(kThreads), 0, be->stream, g, rg, none);
    if (by_head) {
        const uint32_t threads = (hf.M * 128 + 63) / 64 * 64;
        hipLaunchKernelGGL(head_norm_rope_finish_kernel, dim3(finish_heads), dim3(threads), 0, be->stream, hf);
        be->pool.free(tmp, tmp_cls); // stream-ordered: later users queue behind the finishing launch
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "grouped matmul with rotary store launch");
}

// out = g * (1 / (one + exp(-g))) * u with g = x.yg, u = x.yu: two decode-time linear layers and
// the program between them and the next product in one launch.  Declines unless the 4x4x1
// kernel takes the shapes.
int launch_matmul_gated(cg_backend *be, const cg_tensor *x, const cg_tensor *yg, const cg_tensor *yu, uint32_t one,
                        cg_tensor *out, const NormFuse *nf) {
    if (int frc = flush_deferred(be)) return frc;
    if (x->dt != CG_F32) return kDeclined;
    MmArgs ag, au;
    MmFold fg, fu;
    uint32_t *const c = static_cast<uint32_t *>(out->buf->ptr) + out->offset; // out: a contiguous view, not always at element 0
    int rc = make_mm_args(x, yg, c, &ag, &fg);
    if (!rc) rc = make_mm_args(x, yu, c, &au, &fu);
    if (rc) return rc;
    const bool vec = ag.a_vec && ag.b_vec && au.b_vec && ag.a_sk == 1 && ag.K % 4 == 0;
    if (fg.batch != 1 || fu.batch != 1 || ag.M > 4 || ag.b_sk != 1 || au.b_sk != 1 || !vec || ag.K <= 256 || ag.N < 512 ||
        au.N != ag.N || au.K != ag.K || au.M != ag.M || au.b_sn != ag.b_sn)
        return kDeclined;
    if (nf && xreg_trips(ag.K) == 0) return kDeclined;
    const bool short_chunks = xreg_trips(ag.K) == 4; // K a multiple of 1024 but not of 2048
    ProfScope prof(be, CG_K_GEMM_SKINNY, distinct_bytes(x) + distinct_bytes(yg) + distinct_bytes(yu) + distinct_bytes(out));
    const dim3 ggrid((ag.N + 3) / 4);
    if (xreg_trips(ag.K) == 0) return kDeclined;
    if ((int)ag.K <= xreg_trips(ag.K) * 256) { // one chunk of k (full or not): see skinny_kt_mfma_xreg_cols_gated_kernel
        NormFuse none;
        memset(&none, 0, sizeof none);
        const uint32_t groups = (ag.N + 3) / 4, iters = xreg_cols_iters(groups);
        const dim3 cgrid((groups + iters - 1) / iters);
        if (nf && short_chunks) hipLaunchKernelGGL((skinny_kt_mfma_xreg_cols_gated_kernel<true, 4>), cgrid, dim3(kThreads), 0, be->stream, ag, au.B, one, iters, *nf);
        else if (nf) hipLaunchKernelGGL((skinny_kt_mfma_xreg_cols_gated_kernel<true, 8>), cgrid, dim3(kThreads), 0, be->stream, ag, au.B, one, iters, *nf);
        else if (short_chunks) hipLaunchKernelGGL((skinny_kt_mfma_xreg_cols_gated_kernel<false, 4>), cgrid, dim3(kThreads), 0, be->stream, ag, au.B, one, iters, none);
        else hipLaunchKernelGGL((skinny_kt_mfma_xreg_cols_gated_kernel<false, 8>), cgrid, dim3(kThreads), 0, be->stream, ag, au.B, one, iters, none);
    } else if (nf && short_chunks)
        hipLaunchKernelGGL(skinny_kt_mfma_xreg_gated_norm_kernel<4>, ggrid, dim3(kThreads), 0, be->stream, ag, au.B, one, *nf);
    else if (nf)
        hipLaunchKernelGGL(skinny_kt_mfma_xreg_gated_norm_kernel<8>, ggrid, dim3(kThreads), 0, be->stream, ag, au.B, one, *nf);
    else if (short_chunks)
        hipLaunchKernelGGL((skinny_kt_mfma_xreg_gated_kernel<4, 4>), ggrid, dim3(kThreads), 0, be->stream, ag, au.B, one);
    else
        hipLaunchKernelGGL((skinny_kt_mfma_xreg_gated_kernel<4, 8>), ggrid, dim3(kThreads), 0, be->stream, ag, au.B, one);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "gated matmul launch");
}

// out = a sum of four terms, term[slot] = x.y, the other three dense tensors of out's shape
// (device pointers); `order` as in MmResidual.  Declines unless the one-column-per-wave kernel
// is what the product would run on anyway.
int launch_matmul_residual(cg_backend *be, const cg_tensor *x, const cg_tensor *y, const uint32_t *const *terms, int nterms,
                           int slot, int order, cg_tensor *out, bool keep_sums) {
    if (int frc = flush_deferred(be)) return frc;
    if (x->dt != CG_F32) return kDeclined;
    MmArgs a;
    MmFold f;
    int rc = make_mm_args(x, y, static_cast<uint32_t *>(out->buf->ptr) + out->offset, &a, &f);
    if (rc) return rc;
    const bool vec = a.a_vec && a.b_vec && a.a_sk == 1 && a.K % 4 == 0;
    if (f.batch != 1 || a.M > 8 || a.b_sk != 1 || !vec || a.K <= 256 || a.N < 512 || a.N >= 8192) return kDeclined;
    MmResidual r;
    for (int t = 0; t < 4; t++) r.term[t] = t == slot || t >= nterms ? nullptr : terms[t];
    r.slot = (uint32_t)slot;
    r.order = (uint32_t)order;
    r.nterms = (uint32_t)nterms;
    r.partials = nullptr;
    const uint32_t blocks = (uint32_t)((a.N + 3) / 4);
    if (keep_sums && out->offset == 0 && xreg_narrow(a.M, a.K) && !out->buf->side) {
        // the stored rows' sums of squares per workgroup, for an RMS norm that may follow (Buffer::side)
        Buffer *ob = out->buf;
        if (be->pool.alloc((size_t)blocks * 4 * sizeof(float), &ob->side, &ob->side_cls) == CG_OK) {
            ob->side_blocks = blocks;
            r.partials = static_cast<float *>(ob->side);
        } else {
            ob->side = nullptr;
        }
    }
    ProfScope prof(be, CG_K_GEMM_SKINNY, distinct_bytes(x) + distinct_bytes(y) + 4.0 * distinct_bytes(out));
    dim3 grid((uint32_t)((a.N + 3) / 4));
    if (xreg_narrow(a.M, a.K)) {
        if (xreg_trips(a.K) == 8)
            hipLaunchKernelGGL((skinny_kt_mfma_xreg_residual_kernel<4, 8>), grid, dim3(kThreads), 0, be->stream, a, r);
        else
            hipLaunchKernelGGL((skinny_kt_mfma_xreg_residual_kernel<4, 4>), grid, dim3(kThreads), 0, be->stream, a, r);
    } else if (a.M <= 1)
        hipLaunchKernelGGL((skinny_kt_wide_residual_kernel<1>), grid, dim3(kThreads), 0, be->stream, a, r);
    else if (a.M <= 4)
        hipLaunchKernelGGL((skinny_kt_wide_residual_kernel<4>), grid, dim3(kThreads), 0, be->stream, a, r);
    else
        hipLaunchKernelGGL((skinny_kt_wide_residual_kernel<8>), grid, dim3(kThreads), 0, be->stream, a, r);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "matmul with residual launch");
}

// ---- narrow operands for the 16-bit and 8-bit matrix instructions ---------------------------------------------------
// A [rows, k] view of f32 words that hold values of a narrow dtype (exactly) is written as its 2-byte (bf16 / f16) or
// 1-byte (fp8) patterns, k contiguous: half or a quarter of the bytes for the product that follows, and a tile of the
// same 32 words is 64 or 128 deep in k.  KIND 1 bf16, 2 f16, 3 fp8.  A thread narrows four consecutive k of a row.
template <int KIND>
__global__ __launch_bounds__(kThreads) void pack_operand_kernel(const uint32_t *src, int64_t s_r, int64_t s_k, uint32_t rows, uint32_t K,
                                                                void *dst) {
    const uint64_t quads = (uint64_t)rows * (K / 4);
    const uint64_t i = (uint64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= quads) return;
    const uint32_t r = (uint32_t)(i / (K / 4)), k = (uint32_t)(i % (K / 4)) * 4;
    const uint32_t *p = src + (int64_t)r * s_r + (int64_t)k * s_k;
    uint32_t w[4];
    if (s_k == 1 && ((reinterpret_cast<uintptr_t>(p) & 15) == 0)) {
        const uint4 v = *reinterpret_cast<const uint4 *>(p);
        w[0] = v.x, w[1] = v.y, w[2] = v.z, w[3] = v.w;
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = p[(int64_t)e * s_k];
    }
    if constexpr (KIND == 3) {
        static_cast<uint32_t *>(dst)[i] = (uint32_t)f8_byte_of(w[0]) | ((uint32_t)f8_byte_of(w[1]) << 8) | ((uint32_t)f8_byte_of(w[2]) << 16) |
                                          ((uint32_t)f8_byte_of(w[3]) << 24);
    } else {
        uint2 o;
        o.x = pack_halves<KIND>(asf(w[0]), asf(w[1]));
        o.y = pack_halves<KIND>(asf(w[2]), asf(w[3]));
        static_cast<uint2 *>(dst)[i] = o;
    }
}

// (env CG_GEMM_PACKED=0 keeps the products of narrow dtypes on 32-bit words)
static bool packed_narrow_ok() {
    static const bool ok = [] {
        const char *e = getenv("CG_GEMM_PACKED");
        return !(e && e[0] == '0');
    }();
    return ok;
}

// (env CG_PACKED_MFMA=0 keeps few-row products of the 16-bit dtypes on the wave-per-column kernel, for measurements)
static bool packed_mfma_ok() {
    static const bool ok = [] {
        const char *e = getenv("CG_PACKED_MFMA");
        return !(e && e[0] == '0');
    }();
    return ok;
}

// The narrow copy of the [rows, K] view (row stride s_r, k stride s_k, in words) at `ptr` inside `buf`: the copy kept with
// the buffer for this very view if there is one; else a new one, kept with the buffer when `keep` (a weight matrix is
// narrowed once, shared activations once for the products that multiply them; the oldest entry makes room when the list is
// full), else handed to the caller, who frees *tmp after its launch.
static int pack_operand(cg_backend *be, Buffer *buf, const uint32_t *ptr, int64_t s_r, int64_t s_k, int64_t rows, int64_t K, int kind,
                        bool keep, const void **packed, void **tmp, size_t *tmp_cls) {
    const int64_t off = ptr - static_cast<const uint32_t *>(buf->ptr);
    for (const Buffer::Packed &p : buf->packed)
        if (p.kind == kind && p.off == off && p.rows == rows && p.k == K && p.sr == s_r && p.sk == s_k) {
            *packed = p.ptr;
            return CG_OK;
        }
    void *dst = nullptr;
    size_t cls = 0;
    int rc = be->pool.alloc((size_t)rows * (size_t)K * (kind == 3 ? 1 : 2), &dst, &cls);
    if (rc) return rc;
    const uint64_t quads = (uint64_t)rows * (uint64_t)(K / 4);
    const dim3 grid((uint32_t)((quads + kThreads - 1) / kThreads));
    {
        ProfScope prof(be, CG_K_PACK, (double)rows * (double)K * (4.0 + (kind == 3 ? 1.0 : 2.0)));
        if (kind == 1) hipLaunchKernelGGL(pack_operand_kernel<1>, grid, dim3(kThreads), 0, be->stream, ptr, s_r, s_k, (uint32_t)rows, (uint32_t)K, dst);
        else if (kind == 2) hipLaunchKernelGGL(pack_operand_kernel<2>, grid, dim3(kThreads), 0, be->stream, ptr, s_r, s_k, (uint32_t)rows, (uint32_t)K, dst);
        else hipLaunchKernelGGL(pack_operand_kernel<3>, grid, dim3(kThreads), 0, be->stream, ptr, s_r, s_k, (uint32_t)rows, (uint32_t)K, dst);
    }
    if (keep) {
        if (buf->packed.size() >= kMaxPackedPerBuffer) { // stream-ordered free: products already queued on it come first
            be->pool.free(buf->packed.front().ptr, buf->packed.front().cls);
            buf->packed.erase(buf->packed.begin());
        }
        Buffer::Packed p;
        p.ptr = dst;
        p.cls = cls;
        p.kind = kind;
        p.off = off;
        p.rows = rows;
        p.k = K;
        p.sr = s_r;
        p.sk = s_k;
        buf->packed.push_back(p);
    } else {
        *tmp = dst;
        *tmp_cls = cls;
    }
    *packed = dst;
    return CG_OK;
}

// Few rows (M <= 8) times a weight matrix of a narrow dtype that pack_operand narrowed in memory: a wave per output
// column walks K with 16-byte loads of the narrow row (8 two-byte or 16 one-byte weights per lane and trip), widens them in
// registers (exact) and multiplies with the f32 words of the activations; HBM-bound on the narrow weights, 2 or 1 bytes
// per weight instead of 4.  f32 accumulation, lanes combined by a wave shuffle.  KIND 1 bf16, 2 f16, 3 fp8.
template <int KIND> __device__ __forceinline__ void widen_weights(const uint4v &raw, float (&w)[KIND == 3 ? 16 : 8]) {
    const uint32_t r[4] = {raw[0], raw[1], raw[2], raw[3]};
    if constexpr (KIND == 1) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[2 * i] = asf(r[i] << 16);
            w[2 * i + 1] = asf(r[i] & 0xFFFF0000u);
        }
    } else if constexpr (KIND == 2) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[2 * i] = __half2float(__ushort_as_half((unsigned short)(r[i] & 0xFFFFu)));
            w[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(r[i] >> 16)));
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int b = 0; b < 4; b++) w[4 * i + b] = asf(f8_word_of((uint8_t)(r[i] >> (8 * b))));
    }
}
// The same for at most four rows of the 16-bit dtypes on the matrix instruction v_mfma_f32_4x4x4_{bf16_1k,f16}: the layout
// of skinny_kt_mfma_xreg_body (lane (b, j) = (lane / 4, lane % 4) feeds weight row n0 + j and activation row j for the k of
// block b) with 8 k per lane and trip instead of 4: one 16-byte load of narrow weights drives two instructions.  The
// activations, which are f32 words in memory, are narrowed (exact) into registers ONCE per workgroup — all of K, 16
// registers per 2048 — and the workgroup walks `iters` consecutive groups of four columns with them, the next group's
// weights on their way while the current group is reduced: the activation traffic out of L2, twice the weights' bytes per
// column group, is paid once.  K = KCH x 1024.  KIND 1 bf16, 2 f16.
typedef short short4v __attribute__((ext_vector_type(4)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));
template <int KIND, int KCH>
__global__ __launch_bounds__(kThreads) void skinny_kt_packed_mfma_kernel(const MmArgs a, const void *weights, uint32_t iters) {
    constexpr int TRIPS = 2 * KCH; // a wave takes 128 k per trip, four waves 512: two trips per 1024
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t j = lane % 4, b = lane / 4;
    const uint32_t kb = wave * 128 + b * 8; // this lane's k: kb + 512 t .. + 7
    const uint32_t groups = (a.N + 3) / 4;
    const uint32_t first_grp = blockIdx.x * iters;
    if (first_grp >= groups) return; // the same for every thread of the workgroup
    uint4v wq[TRIPS];
    auto ask = [&](uint32_t grp) {
        const uint16_t *row = static_cast<const uint16_t *>(weights) + (size_t)min(grp * 4 + j, a.N - 1) * a.K + kb;
#pragma unroll
        for (int t = 0; t < TRIPS; t++) wq[t] = __builtin_nontemporal_load(reinterpret_cast<const uint4v *>(row + 512 * t));
    };
    ask(first_grp);
    // the activations of row j, narrowed: xq[t] = its 8 values at kb + 512 t as four words of two
    uint4v xq[TRIPS];
    {
        const uint32_t *xrow = a.A + (int64_t)min(j, a.M - 1) * a.a_sm + kb;
#pragma unroll
        for (int t = 0; t < TRIPS; t++) {
            const float4v lo = *reinterpret_cast<const float4v *>(xrow + 512 * t), hi = *reinterpret_cast<const float4v *>(xrow + 512 * t + 4);
            xq[t][0] = pack_halves<KIND>(lo[0], lo[1]);
            xq[t][1] = pack_halves<KIND>(lo[2], lo[3]);
            xq[t][2] = pack_halves<KIND>(hi[0], hi[1]);
            xq[t][3] = pack_halves<KIND>(hi[2], hi[3]);
        }
    }
    __shared__ float part[2][4][16];
    for (uint32_t it = 0; it < iters; it++) {
        const uint32_t grp = first_grp + it;
        if (grp >= groups) break;
        float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < TRIPS; t++) {
            typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
            const uint2v x0 = {xq[t][0], xq[t][1]}, x1 = {xq[t][2], xq[t][3]}, w0 = {wq[t][0], wq[t][1]}, w1 = {wq[t][2], wq[t][3]};
            if constexpr (KIND == 1) {
                acc = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(short4v, x0), __builtin_bit_cast(short4v, w0), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(short4v, x1), __builtin_bit_cast(short4v, w1), acc, 0, 0, 0);
            } else {
                acc = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4v, x0), __builtin_bit_cast(half4v, w0), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4v, x1), __builtin_bit_cast(half4v, w1), acc, 0, 0, 0);
            }
        }
        if (it + 1 < iters && grp + 1 < groups) ask(grp + 1); // on its way through the reduction of this group
        float (*pt)[16] = part[it & 1];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float v = acc[i];
#pragma unroll
            for (int s = 32; s >= 4; s >>= 1) v += __shfl_xor(v, s);
            if (lane < 4) pt[wave][i * 4 + j] = v;
        }
        __syncthreads(); // (the buffer written two groups ago was read before the barrier of the group in between)
        if (threadIdx.x < 16) {
            const uint32_t m = threadIdx.x / 4, col = grp * 4 + threadIdx.x % 4;
            const float v = (pt[0][threadIdx.x] + pt[1][threadIdx.x]) + (pt[2][threadIdx.x] + pt[3][threadIdx.x]);
            if (col < a.N && m < a.M) a.C[(uint64_t)m * a.N + col] = asu(v);
        }
    }
}

template <int MM, int KIND>
__global__ __launch_bounds__(kThreads) void skinny_kt_packed_kernel(const MmArgs a, const void *weights) {
    constexpr int PER = KIND == 3 ? 16 : 8; // weights per lane and trip
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t n = blockIdx.x * 4 + wave;
    if (n >= a.N) return;
    const uint8_t *row = static_cast<const uint8_t *>(weights) + (size_t)n * a.K * (KIND == 3 ? 1 : 2);
    float acc[MM];
#pragma unroll
    for (int m = 0; m < MM; m++) acc[m] = 0.0f;
#pragma unroll 2
    for (uint32_t k = lane * PER; k < a.K; k += 64 * PER) {
        const uint4v raw = __builtin_nontemporal_load(reinterpret_cast<const uint4v *>(row + (size_t)k * (KIND == 3 ? 1 : 2)));
        float w[PER];
        widen_weights<KIND>(raw, w);
#pragma unroll
        for (int m = 0; m < MM; m++) {
            if ((uint32_t)m < a.M) {
                const uint32_t *x = a.A + (int64_t)m * a.a_sm + k;
#pragma unroll
                for (int q = 0; q < PER / 4; q++) {
                    const float4v xv = *reinterpret_cast<const float4v *>(x + 4 * q);
                    acc[m] = fmaf(xv[0], w[4 * q], acc[m]);
                    acc[m] = fmaf(xv[1], w[4 * q + 1], acc[m]);
                    acc[m] = fmaf(xv[2], w[4 * q + 2], acc[m]);
                    acc[m] = fmaf(xv[3], w[4 * q + 3], acc[m]);
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MM; m++) {
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) acc[m] += __shfl_xor(acc[m], s);
        if (lane == 0 && (uint32_t)m < a.M) a.C[(uint64_t)m * a.N + n] = asu(acc[m]);
    }
}

int launch_matmul(cg_backend *be, const cg_tensor *x, const cg_tensor *y, cg_tensor *out) {
    if (int frc = flush_deferred(be)) return frc;
    MmArgs a;
    MmFold f;
    int rc = mm_geometry(x, y, out ? out->buf->ptr : nullptr, &a, &f);
    if (rc) return rc;
    const int64_t M = f.M, N = f.N, K = f.K, batch = f.batch;
    const bool a_mfast = !(a.a_sk == 1 || K == 1) && a.a_sm == 1;
    const bool b_nfast = !(a.b_sk == 1 || K == 1) && a.b_sn == 1;

    if (batch > 65535) return fail(CG_ERR_UNSUPPORTED, "matmul: more than 65535 batch entries after folding");
    const bool f32 = is_f(x->dt);
    const int half = x->dt == CG_BF16 ? 1 : x->dt == CG_F16 ? 2 : 0; // operands of the 16-bit matrix instructions
    const int kind = half ? half : x->dt == CG_F8 ? 3 : 0;           // the narrow kernels' operand format (0: none)
    hipStream_t s = be->stream;

    // ---- the tiled kernels' plan (used by the last branch below; here because it decides how operands are addressed) ----
    // the narrow tile when the wide one would leave over a seventh of its columns empty, and when the product has at
    // most one 128 x 128 tile per compute unit: twice the workgroups then fill the chip (4096 x 2048 x 512: 148 -> 83 us)
    // or at least put two on a unit (8192 x 2048 x 512: 148 -> 145 us); with more tiles than that the wide one wins
    // (env CG_GEMM_NARROW_BELOW=n moves the limit, for measurements)
    const int64_t cols128 = (N + 127) / 128 * 128, cols64 = (N + 63) / 64 * 64;
    static const int64_t narrow_below = [] { const char *e = getenv("CG_GEMM_NARROW_BELOW"); return e ? atoll(e) : 256ll; }();
    const int64_t tiles128 = ((M + BM - 1) / BM) * (cols128 / 128) * (int64_t)batch;
    const bool narrow = (cols128 * 7 > cols64 * 8 || (tiles128 <= narrow_below && N >= 128)) && !half; // (the 16-bit kernels come in the two square tiles)
    const int bn = narrow ? 64 : 128;
    // the 64 x 64 tile when even the narrow tile leaves most compute units without one (the linear layers of a short prompt on
    // a narrow model: 512 x 576 is 36 tiles of 128 x 64): twice the workgroups, each cut along k half as often
    // below 128 tiles of 128 x 64 — the SmolLM2-135M shape's prefill of 512 tokens 7.34 -> 6.84 ms, the Qwen3-0.6B shape's of
    // 1024 unchanged (env CG_GEMM_TINY_BELOW=n moves the limit, for measurements; 0: never)
    static const int64_t tiny_below = [] { const char *e = getenv("CG_GEMM_TINY_BELOW"); return e ? atoll(e) : 128ll; }();
    const bool tiny = narrow && !kind && ((M + BM - 1) / BM) * (cols64 / 64) * (int64_t)batch < tiny_below && M > 64;
    const int bm = tiny ? 64 : BM;
    // the 256 x 256 tile when it covers the chip at least once (env CG_GEMM_BIG=0 switches it off)
    const uint64_t tiles_big = (uint64_t)((M + 255) / 256) * ((N + 255) / 256) * batch;
    static const bool big_allowed = [] {
        const char *e = getenv("CG_GEMM_BIG");
        return !(e && e[0] == '0');
    }();
    const bool fits_big = big_allowed && !narrow && tiles_big >= 256 && M >= 256 && N >= 256;
    // f32 words: since whole tiles are loaded without tests, two workgroups of the 128 x 128 tile per compute unit (two
    // waves per SIMD covering each other's barriers) are as fast as one of the wide tile or faster — 137-138 against
    // 134-135 TFLOP/s on the 1B shape's linear layers, and a partial last round costs a quarter as much (8192 x 2048 x
    // 3072: 755 against 1015 us) — except with a k-contiguous left and a row-contiguous right operand (x.y: 1 % behind).
    // The 16-bit and fp8 paths keep the wide tile (half the L2 bytes per flop, which is what bounds them).
    const bool narrow_dtype = kind != 0;
    const bool big = fits_big && (narrow_dtype || (!a_mfast && b_nfast));
    // Operands of a narrow dtype in a product big enough for the 256 x 256 tile are multiplied from 2-byte / 1-byte
    // patterns: as they lie in memory when their buffer holds that format, else narrowed in memory first (the right
    // operand once per buffer) (env CG_GEMM_PACKED=0 switches it off).
    const bool big_packed = f32 && K != 0 && M > 8 && kind && packed_narrow_ok() && big && batch == 1 && K % (kind == 3 ? 16 : 8) == 0 && x->buf && y->buf;

    // ---- the operands' addresses -------------------------------------------------------------------------------------
    const bool x_native = big_packed && native_rows(x, kind, a.a_sm, a.a_sk, K, false);
    rc = mm_operand(x, true, x_native, &a);
    if (rc) return rc;
    // a decode-time linear layer of a narrow dtype reads its weight matrix at 2 or 1 bytes a weight (see below)
    const bool skinny_packed = f32 && K != 0 && M <= (half ? 8 : 2) && packed_narrow_ok() && kind && batch == 1 && a.a_sk == 1 && a.a_vec &&
                               a.a_sm % 4 == 0 && K % 16 == 0 && K >= 256 && N >= 64 && y->buf;
    const bool y_native = (skinny_packed && native_rows(y, kind, a.b_sn, a.b_sk, K, true)) || (big_packed && native_rows(y, kind, a.b_sn, a.b_sk, K, false));
    rc = mm_operand(y, false, y_native, &a);
    if (rc) return rc;
    // Whole stages of 64 bytes of k in whole turns of the ring, 16-byte rows, byte offsets that fit 32 bits: the wide tile
    // fed by loads straight into LDS (env CG_GEMM_DLDS=0: the register-staged one).  Only that kernel can round the result
    // to the operands' format in its store; without `out` the call just says whether this product would run on it.
    static const bool dlds_allowed = [] {
        const char *e = getenv("CG_GEMM_DLDS");
        return !(e && e[0] == '0');
    }();
    const int64_t per = kind == 3 ? 4 : 2;           // elements per 32-bit word
    const int64_t kw = kind ? K / per : 0;           // words per row
    const int64_t a_pitch = x_native ? a.a_sm / per : kw, b_pitch = y_native ? a.b_sn / per : kw; // (a view taken as it lies keeps its own row pitch)
    const bool dlds = big_packed && dlds_allowed && kw % (16 * kDldsStages) == 0 && a_pitch % 4 == 0 && b_pitch % 4 == 0 &&
                      (!x_native || reinterpret_cast<uintptr_t>(native_ptr(x)) % 16 == 0) && (!y_native || reinterpret_cast<uintptr_t>(native_ptr(y)) % 16 == 0) &&
                      (uint64_t)M * (uint64_t)a_pitch * 4 < (1ull << 32) && (uint64_t)N * (uint64_t)b_pitch * 4 < (1ull << 32) &&
                      (uint64_t)M * (uint64_t)N < (1ull << 30);
    const bool can_round = dlds && N % 4 == 0;
    if (!out) return can_round ? CG_OK : kDeclined;
    const int c_fmt = out->buf->fmt;
    if (c_fmt != kFmtWords && !can_round) return fail(CG_ERR_ARG, "matmul: a narrow result needs the kernel that rounds in its store");
    const double flop = 2.0 * (double)M * (double)N * (double)K * (double)batch;
    const double bytes = distinct_bytes(x) + distinct_bytes(y) + distinct_bytes(out);
    const bool simple = K == 0 || !f32, skinny = !simple && M <= 8 && (a.b_sk == 1 || a.b_sn == 1);
    ProfScope prof(be, simple ? CG_K_GEMM_SIMPLE : skinny ? CG_K_GEMM_SKINNY : CG_K_GEMM_MFMA, skinny ? bytes : flop);
    if (K == 0 || !f32) {
        uint64_t elems = (uint64_t)M * N;
        dim3 grid((uint32_t)((elems + kThreads - 1) / kThreads), (uint32_t)batch);
        if (f32)
            hipLaunchKernelGGL((simple_gemm_kernel<true>), grid, dim3(kThreads), 0, s, a);
        else
            hipLaunchKernelGGL((simple_gemm_kernel<false>), grid, dim3(kThreads), 0, s, a);
    } else if (skinny_packed) {
        // a decode-time linear layer of a narrow dtype: the weight matrix in memory as its dtype's patterns (as uploaded, or
        // narrowed once), read at 2 or 1 bytes a weight
        // (measured on 2048 x 8192: one row 10.7 instead of 15.6 us for the 16-bit dtypes, 13.2 instead of 15.4 for fp8; with
        // four rows the loads of the activations bound both kernels alike, and widening fp8 costs more than it saves)
        const void *pb = y_native ? native_ptr(y) : nullptr;
        void *tb = nullptr;
        size_t cb = 0;
        int prc = y_native ? CG_OK : pack_operand(be, words_buffer(y), a.B, a.b_sn, a.b_sk, N, K, kind, true, &pb, &tb, &cb);
        if (prc) return prc;
        const dim3 pgrid((uint32_t)((N + 3) / 4));
        const int kch = (int)(K / 1024);
        if (half && M <= 4 && K % 1024 == 0 && (kch == 1 || kch == 2 || kch == 4 || kch == 8) && packed_mfma_ok()) {
            // all of the activations narrowed into registers, several column groups per workgroup (see the kernel)
            const uint32_t groups = (uint32_t)((N + 3) / 4), iters = xreg_cols_iters(groups);
            const dim3 mgrid((groups + iters - 1) / iters);
#define CG_PACKED_MFMA(KCH)                                                                                              \
    if (half == 1) hipLaunchKernelGGL((skinny_kt_packed_mfma_kernel<1, KCH>), mgrid, dim3(kThreads), 0, s, a, pb, iters);      \
    else hipLaunchKernelGGL((skinny_kt_packed_mfma_kernel<2, KCH>), mgrid, dim3(kThreads), 0, s, a, pb, iters);
            if (kch == 1) { CG_PACKED_MFMA(1) }
            else if (kch == 2) { CG_PACKED_MFMA(2) }
            else if (kch == 4) { CG_PACKED_MFMA(4) }
            else { CG_PACKED_MFMA(8) }
#undef CG_PACKED_MFMA
            if (tb) be->pool.free(tb, cb);
            hipError_t me = hipGetLastError();
            return me == hipSuccess ? CG_OK : hip_fail(me, "matmul launch");
        }
#define CG_PACKED(MM)                                                                                                     \
    if (kind == 1) hipLaunchKernelGGL((skinny_kt_packed_kernel<MM, 1>), pgrid, dim3(kThreads), 0, s, a, pb);                  \
    else if (kind == 2) hipLaunchKernelGGL((skinny_kt_packed_kernel<MM, 2>), pgrid, dim3(kThreads), 0, s, a, pb);             \
    else hipLaunchKernelGGL((skinny_kt_packed_kernel<MM, 3>), pgrid, dim3(kThreads), 0, s, a, pb);
        if (M <= 1) { CG_PACKED(1) }
        else if (M <= 4) { CG_PACKED(4) }
        else { CG_PACKED(8) }
#undef CG_PACKED
        if (tb) be->pool.free(tb, cb); // stream-ordered: later users queue behind the product
    } else if (M <= 8 && a.b_sk == 1) {
        const bool vec = a.a_vec && a.b_vec && a.a_sk == 1 && K % 4 == 0;
#define CG_MM_SWITCH(CALL)        \
    if (M <= 1) { CALL(1) }       \
    else if (M <= 4) { CALL(4) }  \
    else { CALL(8) }
        if (!vec) {
            dim3 grid((uint32_t)((N + 3) / 4), (uint32_t)batch);
#define CG_CALL(MMV) hipLaunchKernelGGL((skinny_kt_kernel<MMV>), grid, dim3(kThreads), 0, s, a);
            CG_MM_SWITCH(CG_CALL)
#undef CG_CALL
        } else if (K <= 256) {
            const int lpc = K <= 64 ? 16 : K <= 128 ? 32 : 64;
            const uint32_t cols_per_block = 4 * (64 / lpc) * 4;
            dim3 grid((uint32_t)((N + cols_per_block - 1) / cols_per_block), (uint32_t)batch);
#define CG_CALL(MMV)                                                                                          \
    if (lpc == 16) hipLaunchKernelGGL((skinny_kt_narrow_kernel<MMV, 16>), grid, dim3(kThreads), 0, s, a);     \
    else if (lpc == 32) hipLaunchKernelGGL((skinny_kt_narrow_kernel<MMV, 32>), grid, dim3(kThreads), 0, s, a); \
    else hipLaunchKernelGGL((skinny_kt_narrow_kernel<MMV, 64>), grid, dim3(kThreads), 0, s, a);
            CG_MM_SWITCH(CG_CALL)
#undef CG_CALL
        } else {
            // enough waves to cover 256 CUs several times over, else split K inside the block
            const int64_t cols = N * batch;
            if (cols >= 16384) {
                dim3 grid((uint32_t)((N + 15) / 16), (uint32_t)batch);
#define CG_CALL(MMV) hipLaunchKernelGGL((skinny_kt_wide_kernel<MMV, 4, false>), grid, dim3(kThreads), 0, s, a);
                CG_MM_SWITCH(CG_CALL)
#undef CG_CALL
            } else if (cols >= 4096 && M <= 4) { // the wider projections of a decode step: activations are fetched once per 8 columns
                dim3 grid((uint32_t)((N + 7) / 8), (uint32_t)batch);
                if (xreg_trips((uint32_t)K) == 4)
                    hipLaunchKernelGGL((skinny_kt_mfma_xreg_kernel<4, 2, 4>), grid, dim3(kThreads), 0, s, a);
                else
                    hipLaunchKernelGGL((skinny_kt_mfma_xreg_kernel<4, 2, 8>), grid, dim3(kThreads), 0, s, a);
            } else if (cols >= 2048 && xreg_narrow((uint32_t)M, (uint32_t)K)) {
                dim3 grid((uint32_t)((N + 3) / 4), (uint32_t)batch);
                if (xreg_trips((uint32_t)K) == 4)
                    hipLaunchKernelGGL((skinny_kt_mfma_xreg_kernel<4, 1, 4>), grid, dim3(kThreads), 0, s, a);
                else
                    hipLaunchKernelGGL((skinny_kt_mfma_xreg_kernel<4, 1, 8>), grid, dim3(kThreads), 0, s, a);
            } else if (cols >= 2048) {
                dim3 grid((uint32_t)((N + 3) / 4), (uint32_t)batch);
#define CG_CALL(MMV) hipLaunchKernelGGL((skinny_kt_wide_kernel<MMV, 1, false>), grid, dim3(kThreads), 0, s, a);
                CG_MM_SWITCH(CG_CALL)
#undef CG_CALL
            } else {
                dim3 grid((uint32_t)N, (uint32_t)batch);
#define CG_CALL(MMV) hipLaunchKernelGGL((skinny_kt_wide_kernel<MMV, 1, true>), grid, dim3(kThreads), 0, s, a);
                CG_MM_SWITCH(CG_CALL)
#undef CG_CALL
            }
        }
    } else if (M <= 8 && a.b_sn == 1) {
        // split K over grid.z until about 2048 blocks are in flight (>= 128 k-rows each)
        const int64_t blocks_xy = ((N + 63) / 64) * batch;
        int64_t splits = std::min<int64_t>(std::min<int64_t>((2048 + blocks_xy - 1) / blocks_xy, (K + 127) / 128), 64);
        if (splits < 1) splits = 1;
        const uint32_t kchunk = (uint32_t)((((K + splits - 1) / splits) + 15) / 16 * 16);
        splits = (K + kchunk - 1) / kchunk;
        void *scratch = nullptr;
        size_t scratch_cls = 0;
        uint32_t *dst = a.C;
        if (splits > 1) {
            int prc = be->pool.alloc((size_t)batch * splits * M * N * 4, &scratch, &scratch_cls);
            if (prc) return prc;
            dst = static_cast<uint32_t *>(scratch);
        }
        dim3 grid((uint32_t)((N + 63) / 64), (uint32_t)batch, (uint32_t)splits);
#define CG_CALL(MMV) hipLaunchKernelGGL((skinny_nn_kernel<MMV>), grid, dim3(kThreads), 0, s, a, dst, kchunk);
        CG_MM_SWITCH(CG_CALL)
#undef CG_CALL
        if (splits > 1) {
            uint64_t total = (uint64_t)batch * M * N;
            hipLaunchKernelGGL(splitk_reduce_kernel, dim3((uint32_t)((total + kThreads - 1) / kThreads)), dim3(kThreads),
                               0, s, static_cast<const uint32_t *>(scratch), a.C, (uint32_t)splits, (uint32_t)(M * N),
                               total);
            be->pool.free(scratch, scratch_cls); // stream-ordered: later users queue behind the reduce
        }
#undef CG_MM_SWITCH
    } else {
        uint64_t tiles = big ? tiles_big / batch : (uint64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
        if (tiles > 0x7FFFFFFFull) return fail(CG_ERR_UNSUPPORTED, "matmul: too many tiles");
        // Too few tiles for the device (the linear layers of a short prefill on a narrow model): cut along k as well, so that
        // about two workgroups per compute unit run, each with at least 128 values of k; the partial tiles go to scratch memory
        // and are summed in a fixed order (the same shape always gets the same cut: results are identical from run to run).
        // (env CG_GEMM_SPLITK=0 switches it off)
        static const bool splitk_allowed = [] {
            const char *e = getenv("CG_GEMM_SPLITK");
            return !(e && e[0] == '0');
        }();
        static const int64_t splitk_below = [] { const char *e = getenv("CG_GEMM_SPLITK_BELOW"); return e ? atoll(e) : 256ll; }();
        static const int64_t splitk_target = [] { const char *e = getenv("CG_GEMM_SPLITK_TARGET"); return e ? atoll(e) : 512ll; }();
        int64_t splits = 1;
        uint32_t kchunk = 0;
        if (splitk_allowed && !narrow_dtype && !big && (int64_t)(tiles * (uint64_t)batch) < splitk_below && K >= 256) {
            const int64_t wgs = (int64_t)tiles * batch;
            splits = std::min<int64_t>(std::min<int64_t>((splitk_target + wgs - 1) / wgs, K / 128), 16);
            kchunk = (uint32_t)(((K + splits - 1) / splits + BK - 1) / BK * BK);
            splits = (K + kchunk - 1) / kchunk;
            if (splits < 2) {
                splits = 1;
                kchunk = 0;
            }
        }
        void *kscratch = nullptr;
        size_t kscratch_cls = 0;
        if (splits > 1) {
            int src = be->pool.alloc((size_t)batch * splits * M * N * 4, &kscratch, &kscratch_cls);
            if (src) return src;
            a.C = static_cast<uint32_t *>(kscratch);
            a.ksplit = kchunk;
        }
        dim3 grid((uint32_t)tiles, (uint32_t)batch, (uint32_t)splits);
        static const bool lds_ok = [] { // the tiles need more than the default 64 KiB of dynamic LDS
            bool ok = true;
#define CG_LDS(AF, BF)                                                                                                \
    ok &= hipFuncSetAttribute(reinterpret_cast<const void *>(&mfma_gemm_kernel<AF, BF, 2>),                           \
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes(128)) == hipSuccess;    \
    ok &= hipFuncSetAttribute(reinterpret_cast<const void *>(&mfma_gemm_kernel<AF, BF, 1>),                           \
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes(64)) == hipSuccess;     \
    ok &= hipFuncSetAttribute(reinterpret_cast<const void *>(&mfma_gemm_kernel<AF, BF, 4, 4>),                        \
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes(256, 256)) == hipSuccess; \
    ok &= hipFuncSetAttribute(reinterpret_cast<const void *>(&mfma_gemm_kernel<AF, BF, 4, 4, 1>),                     \
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes(256, 256, true)) == hipSuccess; \
    ok &= hipFuncSetAttribute(reinterpret_cast<const void *>(&mfma_gemm_kernel<AF, BF, 4, 4, 2>),                     \
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes(256, 256, true)) == hipSuccess;
            CG_LDS(true, true) CG_LDS(true, false) CG_LDS(false, true) CG_LDS(false, false)
#undef CG_LDS
            ok &= hipFuncSetAttribute(reinterpret_cast<const void *>(&mfma_gemm_kernel<false, false, 4, 4, 3>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes(256, 256)) == hipSuccess;
            ok &= hipFuncSetAttribute(reinterpret_cast<const void *>(&mfma_gemm_kernel<false, false, 4, 4, 4>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes(256, 256)) == hipSuccess;
            ok &= hipFuncSetAttribute(reinterpret_cast<const void *>(&mfma_gemm_kernel<false, false, 4, 4, 5>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes(256, 256)) == hipSuccess;
            return ok;
        }();
        if (!lds_ok) return fail(CG_ERR_DEVICE, "matmul: cannot reserve %zu bytes of LDS", gemm_lds_bytes(128));
        if (big_packed) {
            const void *pa = x_native ? native_ptr(x) : nullptr, *pb = y_native ? native_ptr(y) : nullptr;
            void *ta = nullptr, *tb = nullptr;
            size_t ca = 0, cb = 0;
            // (the left operand's narrow copy is kept with its buffer when somebody else holds the activations too — q / k / v
            // and gate / up multiply the same ones —; an operand only this product reads is narrowed for it alone)
            const bool x_shared = x->rc.load() > 1 || x->buf->rc.load() > 1;
            int prc = x_native ? CG_OK : pack_operand(be, words_buffer(x), a.A, a.a_sm, a.a_sk, M, K, kind, x_shared, &pa, &ta, &ca);
            if (!prc && !y_native) prc = pack_operand(be, words_buffer(y), a.B, a.b_sn, a.b_sk, N, K, kind, true, &pb, &tb, &cb);
            if (!prc) {
                MmArgs p = a;
                p.A = static_cast<const uint32_t *>(pa);
                p.B = static_cast<const uint32_t *>(pb);
                p.K = (uint32_t)kw;
                p.a_sm = a_pitch;
                p.b_sn = b_pitch;
                p.a_sk = p.b_sk = 1;
                p.a_vec = p.b_vec = 1;
                p.c_fmt = (uint32_t)c_fmt;
                static const bool dlds_ok = [] {
                    bool ok = true;
#define CG_DLDS_LDS(H, NARROW)                                                                                                 \
    ok &= hipFuncSetAttribute(reinterpret_cast<const void *>(&mfma_gemm_dlds_kernel<H, NARROW>), hipFuncAttributeMaxDynamicSharedMemorySize, \
                              (int)kDldsLdsBytes) == hipSuccess;
                    CG_DLDS_LDS(3, false) CG_DLDS_LDS(3, true) CG_DLDS_LDS(4, false) CG_DLDS_LDS(4, true) CG_DLDS_LDS(5, false) CG_DLDS_LDS(5, true)
#undef CG_DLDS_LDS
                    return ok;
                }();
                if (dlds && !dlds_ok) prc = fail(CG_ERR_DEVICE, "matmul: cannot reserve %zu bytes of LDS", kDldsLdsBytes);
                else if (dlds) {
                    const dim3 pgrid((uint32_t)std::min<uint64_t>(tiles, (uint64_t)be->compute_units)); // its workgroups walk the tiles
                    const bool narrow_out = c_fmt != kFmtWords;
                    if (kind == 1 && narrow_out) hipLaunchKernelGGL((mfma_gemm_dlds_kernel<3, true>), pgrid, dim3(kThreads), kDldsLdsBytes, s, p);
                    else if (kind == 1) hipLaunchKernelGGL((mfma_gemm_dlds_kernel<3, false>), pgrid, dim3(kThreads), kDldsLdsBytes, s, p);
                    else if (kind == 2 && narrow_out) hipLaunchKernelGGL((mfma_gemm_dlds_kernel<4, true>), pgrid, dim3(kThreads), kDldsLdsBytes, s, p);
                    else if (kind == 2) hipLaunchKernelGGL((mfma_gemm_dlds_kernel<4, false>), pgrid, dim3(kThreads), kDldsLdsBytes, s, p);
                    else if (narrow_out) hipLaunchKernelGGL((mfma_gemm_dlds_kernel<5, true>), pgrid, dim3(kThreads), kDldsLdsBytes, s, p);
                    else hipLaunchKernelGGL((mfma_gemm_dlds_kernel<5, false>), pgrid, dim3(kThreads), kDldsLdsBytes, s, p);
                } else if (kind == 1) hipLaunchKernelGGL((mfma_gemm_kernel<false, false, 4, 4, 3>), grid, dim3(kThreads), gemm_lds_bytes(256, 256), s, p);
                else if (kind == 2) hipLaunchKernelGGL((mfma_gemm_kernel<false, false, 4, 4, 4>), grid, dim3(kThreads), gemm_lds_bytes(256, 256), s, p);
                else hipLaunchKernelGGL((mfma_gemm_kernel<false, false, 4, 4, 5>), grid, dim3(kThreads), gemm_lds_bytes(256, 256), s, p);
            }
            if (ta) be->pool.free(ta, ca); // stream-ordered: later users queue behind the product
            if (tb) be->pool.free(tb, cb);
            if (prc) return prc;
            hipError_t pe = hipGetLastError();
            return pe == hipSuccess ? CG_OK : hip_fail(pe, "matmul launch");
        }
#define CG_GEMM_HALF(AF, BF, H)                                                                                    \
    do {                                                                                                           \
        if (big)                                                                                                   \
            hipLaunchKernelGGL((mfma_gemm_kernel<AF, BF, 4, 4, H>), grid, dim3(kThreads), gemm_lds_bytes(256, 256, true), s, a); \
        else                                                                                                       \
            hipLaunchKernelGGL((mfma_gemm_kernel<AF, BF, 2, 2, H>), grid, dim3(kThreads), gemm_lds_bytes(128, 128, true), s, a); \
    } while (0)
#define CG_GEMM(AF, BF)                                                                                            \
    do {                                                                                                           \
        if (half == 1) {                                                                                           \
            CG_GEMM_HALF(AF, BF, 1);                                                                               \
        } else if (half == 2) {                                                                                    \
            CG_GEMM_HALF(AF, BF, 2);                                                                               \
        } else if (big)                                                                                            \
            hipLaunchKernelGGL((mfma_gemm_kernel<AF, BF, 4, 4>), grid, dim3(kThreads), gemm_lds_bytes(256, 256), s, a); \
        else if (tiny)                                                                                             \
            hipLaunchKernelGGL((mfma_gemm_kernel<AF, BF, 1, 1>), grid, dim3(kThreads), gemm_lds_bytes(64, 64), s, a); \
        else if (narrow)                                                                                           \
            hipLaunchKernelGGL((mfma_gemm_kernel<AF, BF, 1>), grid, dim3(kThreads), gemm_lds_bytes(64), s, a);     \
        else                                                                                                       \
            hipLaunchKernelGGL((mfma_gemm_kernel<AF, BF, 2>), grid, dim3(kThreads), gemm_lds_bytes(128), s, a);    \
    } while (0)
        if (a_mfast) {
            if (b_nfast) CG_GEMM(true, true);
            else CG_GEMM(true, false);
        } else {
            if (b_nfast) CG_GEMM(false, true);
            else CG_GEMM(false, false);
        }
#undef CG_GEMM
#undef CG_GEMM_HALF
        if (splits > 1) {
            uint32_t *const dst = static_cast<uint32_t *>(out->buf->ptr);
            const uint64_t mn = (uint64_t)M * N, total = mn * batch;
            if (mn % 4 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0)
                hipLaunchKernelGGL(splitk_reduce4_kernel, dim3((uint32_t)((total / 4 + kThreads - 1) / kThreads)), dim3(kThreads), 0, s,
                                   static_cast<const float4v *>(kscratch), reinterpret_cast<float4v *>(dst), (uint32_t)splits,
                                   (uint32_t)(mn / 4), total / 4);
            else
                hipLaunchKernelGGL(splitk_reduce_kernel, dim3((uint32_t)((total + kThreads - 1) / kThreads)), dim3(kThreads), 0, s,
                                   static_cast<const uint32_t *>(kscratch), dst, (uint32_t)splits, (uint32_t)mn, total);
            be->pool.free(kscratch, kscratch_cls); // stream-ordered: later users queue behind the reduce
        }
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? CG_OK : hip_fail(e, "matmul launch");
}

} // namespace cg
