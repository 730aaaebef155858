// Box copies: strided <-> strided moves of rectangular sub-volumes, several
// boxes per launch.  This is the pack / unpack / self-copy work of Repartition
// (reference: backends/mpi_numpy/functional/repartition.py:158-208) and of
// HaloExchange (backends/mpi_numpy/functional/halo_exchange.py:50-74, 115-140).
//
// Host side: every box is rewritten in BYTES, unit dimensions are dropped,
// dimensions that are contiguous on both sides are merged, and the widest
// power-of-two vector (<= 16 B) that divides the innermost run, both base
// addresses and every remaining stride is chosen.  A box is then a matrix of
// R rows (the flattened outer dimensions) by C vectors (the innermost one).
//
// Device side: a workgroup moves tiles of 1024 vectors shaped TR rows x TC
// columns, TC the power of two covering C (at most 1024), so a vector's row and
// column inside its tile are bit fields of its number; only the row needs
// multiply-high divisions, and only when more than one outer dimension is left.
// Workgroups are persistent (they stride over the tile sequence of the launch),
// loads and stores are non-temporal, and nothing but the box table -- passed by
// value as kernel arguments and read with scalar loads -- is read besides the
// payload.
#include "ddl_common.h"

#include <algorithm>
#include <cmath>
#include <type_traits>
#include <vector>

namespace ddl {
namespace {

constexpr int kMaxDevDims = 5;   // outer dimensions left after merging (plus the innermost one)
constexpr int kBatch = 16;       // boxes per launch (kernel-argument budget)
constexpr int kThreads = 256;
constexpr int kUnroll = 4;
constexpr uint32_t kTileVecs = kThreads * kUnroll;
constexpr uint32_t kTileLog = 10;  // log2(kTileVecs)
static_assert((1u << kTileLog) == kTileVecs, "tile size must be 2^kTileLog");
constexpr uint32_t kPersistentBlocks = 4096;  // 16 per CU
constexpr uint64_t kMaxVecs = (1ull << 31) - kTileVecs;
constexpr uint64_t kLongRunBytes = 64 << 10;   // boxes whose innermost runs are at least this long are interleaved within a launch

enum Op { OP_COPY = 0, OP_ADD = 1, OP_ZERO = 2 };

// Multi-dword vectors are only promised dword alignment (see lower_box).
typedef unsigned int u32x4_a __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_a __attribute__((ext_vector_type(2)));
typedef u32x4_a u32x4 __attribute__((aligned(4)));
typedef u32x2_a u32x2 __attribute__((aligned(4)));

struct DevDim {
    int64_t ss;  // source stride, bytes
    int64_t ds;  // destination stride, bytes
    FastDiv fd;  // divide by the extent
};

struct DevBox {
    const char* src;
    char* dst;
    int64_t css, cds;     // column (innermost) strides, bytes
    uint32_t cols;        // C: vectors per row
    uint32_t rows;        // R: product of the outer extents
    uint32_t tc_log;      // log2(TC)
    uint32_t col_tiles;   // ceil(C / TC)
    uint32_t nd;          // outer dimensions (0 = a single row)
    uint32_t vlog;        // log2(vector bytes)
    uint32_t first_tile;  // first tile of this box in the launch
    uint32_t ct_mul, ct_shr;  // multiply-high division by col_tiles
    uint32_t pad;
    DevDim dim[kMaxDevDims];  // outer dimensions, 0 = slowest
};

struct Batch {
    DevBox box[kBatch];
    uint32_t first_tile[kBatch];  // copy of box[i].first_tile, contiguous for one wide scalar load
    uint32_t nbox;
    uint32_t ntiles;
    FastDiv rr;   // div = nbox when the launch walks its boxes round-robin (tile b belongs to box b % nbox), else 0
};

static_assert(sizeof(Batch) <= 4096, "box table must fit the kernel-argument segment");

// ---------------------------------------------------------------- device --

template <typename T>
struct AddOp;

template <>
struct AddOp<float> {
    static __device__ float apply(float a, float b) { return a + b; }
};
template <>
struct AddOp<double> {
    static __device__ double apply(double a, double b) { return a + b; }
};

struct bf16_bits {
    uint16_t u;
};
struct f16_bits {
    uint16_t u;
};

// Integers wrap around, as two's-complement sums do in NumPy and ATen.
template <>
struct AddOp<int32_t> {
    static __device__ int32_t apply(int32_t a, int32_t b) {
        return static_cast<int32_t>(static_cast<uint32_t>(a) + static_cast<uint32_t>(b));
    }
};
template <>
struct AddOp<int64_t> {
    static __device__ int64_t apply(int64_t a, int64_t b) {
        return static_cast<int64_t>(static_cast<uint64_t>(a) + static_cast<uint64_t>(b));
    }
};
// bf16 arithmetic: operands widened to fp32, one fp32 operation, the result
// rounded to nearest even by the conversion instruction (two results per
// instruction); a NaN stays a NaN.
typedef __bf16 bf16_pair __attribute__((ext_vector_type(2)));
typedef float f32_pair __attribute__((ext_vector_type(2)));

__device__ inline float bf16_low(uint32_t w) { return __uint_as_float(w << 16); }
__device__ inline float bf16_high(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
__device__ inline uint32_t bf16_rounded_pair(float low, float high) {
    f32_pair f;
    f[0] = low, f[1] = high;
    const bf16_pair r = __builtin_convertvector(f, bf16_pair);
    uint32_t w;
    __builtin_memcpy(&w, &r, 4);
    return w;
}
__device__ inline uint16_t bf16_rounded(float v) {
    const __bf16 r = static_cast<__bf16>(v);
    uint16_t u;
    __builtin_memcpy(&u, &r, 2);
    return u;
}

template <>
struct AddOp<bf16_bits> {
    static __device__ bf16_bits apply(bf16_bits a, bf16_bits b) {
        bf16_bits r;
        r.u = bf16_rounded(bf16_low(a.u) + bf16_low(b.u));
        return r;
    }
    static __device__ uint32_t apply_pair(uint32_t a, uint32_t b) {
        return bf16_rounded_pair(bf16_low(a) + bf16_low(b), bf16_high(a) + bf16_high(b));
    }
};
template <>
struct AddOp<f16_bits> {
    static __device__ f16_bits apply(f16_bits a, f16_bits b) {
        _Float16 ha, hb;
        __builtin_memcpy(&ha, &a.u, 2);
        __builtin_memcpy(&hb, &b.u, 2);
        const _Float16 hs = static_cast<_Float16>(static_cast<float>(ha) + static_cast<float>(hb));
        f16_bits r;
        __builtin_memcpy(&r.u, &hs, 2);
        return r;
    }
};

template <typename T, typename V>
__device__ inline V add_vectors(V d, V s) {
    constexpr int n = sizeof(V) / sizeof(T);
    static_assert(n >= 1, "vector narrower than the element");
    if constexpr (std::is_same<T, bf16_bits>::value && sizeof(V) >= 4) {
        constexpr int words = sizeof(V) / 4;
        uint32_t dw[words], sw[words];
        __builtin_memcpy(dw, &d, sizeof(V));
        __builtin_memcpy(sw, &s, sizeof(V));
#pragma unroll
        for (int i = 0; i < words; ++i) dw[i] = AddOp<bf16_bits>::apply_pair(dw[i], sw[i]);
        V out;
        __builtin_memcpy(&out, dw, sizeof(V));
        return out;
    }
    T dv[n], sv[n];
    __builtin_memcpy(dv, &d, sizeof(V));
    __builtin_memcpy(sv, &s, sizeof(V));
#pragma unroll
    for (int i = 0; i < n; ++i) dv[i] = AddOp<T>::apply(dv[i], sv[i]);
    V out;
    __builtin_memcpy(&out, dv, sizeof(V));
    return out;
}

// The box table lives in the kernel-argument segment and is read with scalar
// loads at compile-time offsets from the selected box; nothing of it is copied
// into registers arrays, LDS or scratch.
#if defined(__HIP_DEVICE_COMPILE__)
typedef const Batch __attribute__((address_space(4))) * BatchPtr;
typedef const DevBox __attribute__((address_space(4))) * DevBoxPtr;
#else
typedef const Batch* BatchPtr;
typedef const DevBox* DevBoxPtr;
#endif

// ND = number of outer dimensions this instantiation decomposes (the table
// entries beyond a box's own count hold extent 1 and stride 0).  Every table
// field is fetched unconditionally at the top, so the scalar loads are issued
// together and waited for once per tile.
template <int ND>
__device__ __forceinline__ void tile_offsets(DevBoxPtr bx, uint32_t tile, int64_t (&soff)[kUnroll], int64_t (&doff)[kUnroll],
                                             bool (&live)[kUnroll]) {
    const uint32_t col_tiles = bx->col_tiles;
    const uint32_t tc_log = bx->tc_log;
    const uint32_t ct_mul = bx->ct_mul, ct_shr = bx->ct_shr;
    const uint32_t rows = bx->rows, cols = bx->cols;
    const int64_t css = bx->css, cds = bx->cds;
    int64_t dss[ND > 0 ? ND : 1], dds[ND > 0 ? ND : 1];
    uint32_t ddiv[ND > 0 ? ND : 1], dmul[ND > 0 ? ND : 1], dshr[ND > 0 ? ND : 1];
#pragma unroll
    for (int d = 0; d < ND; ++d) {
        dss[d] = bx->dim[d].ss;
        dds[d] = bx->dim[d].ds;
        ddiv[d] = bx->dim[d].fd.div;
        dmul[d] = bx->dim[d].fd.mul;
        dshr[d] = bx->dim[d].fd.shr;
    }
    const uint32_t row_tile = col_tiles == 1 ? tile : (__umulhi(tile, ct_mul) >> ct_shr);  // wave-uniform
    const uint32_t col_tile = tile - row_tile * col_tiles;
    const uint32_t row0 = row_tile << (kTileLog - tc_log);
    const uint32_t col0 = col_tile << tc_log;
    const uint32_t tc = 1u << tc_log;
    const bool interior = col0 + tc <= cols && row0 + (kTileVecs >> tc_log) <= rows;   // wave-uniform
    if (ND <= 1 && interior) {
        // Whole tile inside the box and rows addressed by one stride: the four
        // vectors of a lane differ by wave-uniform steps, so one position is
        // computed and the others follow by addition.
        const uint32_t j = threadIdx.x;
        const uint32_t col = col0 + (j & (tc - 1u));
        const uint32_t r = row0 + (j >> tc_log);
        int64_t so = static_cast<int64_t>(col) * css, dof = static_cast<int64_t>(col) * cds;
        if (ND > 0) {
            so += static_cast<int64_t>(r) * dss[0];
            dof += static_cast<int64_t>(r) * dds[0];
        }
        // step of kThreads vectors: columns while they fit the tile row, rows after that
        int64_t sstep[kUnroll], dstep[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t jj = u * kThreads;                 // uniform
            const uint32_t dc = jj & (tc - 1u), dr = jj >> tc_log;
            sstep[u] = static_cast<int64_t>(dc) * css + (ND > 0 ? static_cast<int64_t>(dr) * dss[0] : 0);
            dstep[u] = static_cast<int64_t>(dc) * cds + (ND > 0 ? static_cast<int64_t>(dr) * dds[0] : 0);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            soff[u] = so + sstep[u];
            doff[u] = dof + dstep[u];
            live[u] = true;
        }
    } else {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t j = threadIdx.x + u * kThreads;   // vector number inside the tile
            uint32_t col = col0 + (j & (tc - 1u));
            uint32_t r = row0 + (j >> tc_log);
            live[u] = col < cols && r < rows;
            // Vectors past the edge of the box are clamped onto its last column /
            // row: they re-move an element another lane moves too, which keeps
            // every load and store unconditional.
            col = col < cols ? col : cols - 1;
            r = r < rows ? r : rows - 1;
            int64_t so = static_cast<int64_t>(col) * css, dof = static_cast<int64_t>(col) * cds;
#pragma unroll
            for (int d = ND - 1; d > 0; --d) {
                const uint32_t q = ddiv[d] == 1 ? r : (__umulhi(r, dmul[d]) >> dshr[d]);
                const uint32_t idx = r - q * ddiv[d];
                so += static_cast<int64_t>(idx) * dss[d];
                dof += static_cast<int64_t>(idx) * dds[d];
                r = q;
            }
            if (ND > 0) {
                so += static_cast<int64_t>(r) * dss[0];
                dof += static_cast<int64_t>(r) * dds[0];
            }
            soff[u] = so;
            doff[u] = dof;
        }
    }
}

template <int OP, typename T, typename V, int ND>
__device__ inline void move_tile(DevBoxPtr bx, uint32_t tile) {
    int64_t soff[kUnroll], doff[kUnroll];
    bool live[kUnroll];
    tile_offsets<ND>(bx, tile, soff, doff, live);
    char* const dst = bx->dst;
    if constexpr (OP == OP_ZERO) {
        V z;
        __builtin_memset(&z, 0, sizeof(V));
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) __builtin_nontemporal_store(z, reinterpret_cast<V*>(dst + doff[u]));
        return;
    }
    const char* const src = bx->src;
    V val[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) val[u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(src + soff[u]));
    if constexpr (OP == OP_ADD) {
        if constexpr (sizeof(V) >= sizeof(T)) {
            V cur[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) cur[u] = *reinterpret_cast<const V*>(dst + doff[u]);
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) val[u] = add_vectors<T, V>(cur[u], val[u]);
        }
        // An accumulation must happen exactly once per element.
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
            if (live[u]) *reinterpret_cast<V*>(dst + doff[u]) = val[u];
        return;
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) __builtin_nontemporal_store(val[u], reinterpret_cast<V*>(dst + doff[u]));
}

template <int OP, typename T, typename V>
__device__ inline void move_tile_nd(DevBoxPtr bx, uint32_t tile, uint32_t nd) {
    if (nd == 0)
        move_tile<OP, T, V, 0>(bx, tile);
    else if (nd == 1)
        move_tile<OP, T, V, 1>(bx, tile);
    else if (nd == 2)
        move_tile<OP, T, V, 2>(bx, tile);
    else
        move_tile<OP, T, V, kMaxDevDims>(bx, tile);
}

template <int OP, typename T>
__global__ __launch_bounds__(kThreads) void box_kernel(const Batch bt_by_value) {
#if defined(__HIP_DEVICE_COMPILE__)
    BatchPtr bt = (BatchPtr)__builtin_amdgcn_kernarg_segment_ptr();
#else
    BatchPtr bt = &bt_by_value;
#endif
    // Persistent workgroups: each walks the launch's tile sequence with a
    // stride of the grid, so a few thousand workgroups serve any volume.
    const uint32_t nbox = bt->nbox;
    const uint32_t ntiles = bt->ntiles;
    const uint32_t rr_div = bt->rr.div, rr_mul = bt->rr.mul, rr_shr = bt->rr.shr;
    for (uint32_t b = blockIdx.x; b < ntiles; b += gridDim.x) {
        uint32_t bi = 0, tile;
        if (rr_div != 0) {   // boxes of equal tile counts, interleaved
            tile = __umulhi(b, rr_mul) >> rr_shr;
            bi = b - tile * rr_div;
        } else {
#pragma unroll
            for (uint32_t i = 1; i < kBatch; ++i) bi += (i < nbox && b >= bt->first_tile[i]) ? 1u : 0u;
            tile = b - bt->first_tile[bi];
        }
        DevBoxPtr bx = &bt->box[bi];
        const uint32_t nd = bx->nd;
        switch (bx->vlog) {
            case 4: move_tile_nd<OP, T, u32x4>(bx, tile, nd); break;
            case 3: move_tile_nd<OP, T, u32x2>(bx, tile, nd); break;
            case 2: move_tile_nd<OP, T, uint32_t>(bx, tile, nd); break;
            case 1: move_tile_nd<OP, T, uint16_t>(bx, tile, nd); break;
            default: move_tile_nd<OP, T, uint8_t>(bx, tile, nd); break;
        }
    }
}

// Copy of a batch of boxes that all have the same geometry -- equal extents and
// strides, at most one outer dimension, 16-byte vectors, extents that are whole
// tiles -- and differ only in their two base addresses: the pack of a
// Repartition whose boxes are equal column strips, the unpack of equal slabs,
// the all-gather re-layout.  What the general kernel spends in front of its
// first load (which box a tile belongs to, then that box's geometry, then the
// addresses: three rounds of dependent scalar loads, paid at full latency by
// every workgroup of a launch that has just one tile per workgroup) shrinks to
// one round here: the box is a grid coordinate, so the two base addresses and
// the shared geometry are fetched together.  One tile per workgroup.
//
// ROUND_ROBIN: blockIdx.x is the box and blockIdx.y the tile (tiles of all boxes
// take turns, see launch_batches), else the other way round (box after box).
// WAVE_ROWS: the tile is one contiguous run of 16 KiB on both sides; wavefront w
// then owns bytes [4 KiB w, 4 KiB (w + 1)) of it instead of every fourth KiB, so
// that the four wavefronts' first requests go to four different 4 KiB pieces
// (measured on the unpack of eight [8,512,1024] bf16 slabs: 24.05 -> 23.48 us).
struct UniformBatch {
    const char* src[kBatch];
    char* dst[kBatch];
    int64_t srow, drow;        // strides of the outer dimension, bytes (0 without one)
    uint32_t tc_log;           // log2 of the vectors a tile covers along the columns
    uint32_t col_tiles;        // tiles side by side along the columns
    uint32_t ct_mul, ct_shr;   // multiply-high division by col_tiles
};

#if defined(__HIP_DEVICE_COMPILE__)
typedef const UniformBatch __attribute__((address_space(4))) * UniformPtr;
#else
typedef const UniformBatch* UniformPtr;
#endif

template <bool ROUND_ROBIN, bool WAVE_ROWS>
__global__ __launch_bounds__(kThreads) void uniform_copy_kernel(const UniformBatch ub_by_value) {
#if defined(__HIP_DEVICE_COMPILE__)
    UniformPtr ub = (UniformPtr)__builtin_amdgcn_kernarg_segment_ptr();
#else
    UniformPtr ub = &ub_by_value;
#endif
    const uint32_t box = ROUND_ROBIN ? blockIdx.x : blockIdx.y;
    const uint32_t tile = ROUND_ROBIN ? blockIdx.y : blockIdx.x;
    const char* const src = ub->src[box];
    char* const dst = ub->dst[box];
    const int64_t srow = ub->srow, drow = ub->drow;
    const uint32_t tc_log = ub->tc_log, col_tiles = ub->col_tiles, ct_mul = ub->ct_mul, ct_shr = ub->ct_shr;
    const uint32_t row_tile = col_tiles == 1 ? tile : (__umulhi(tile, ct_mul) >> ct_shr);
    const uint32_t col_tile = tile - row_tile * col_tiles;
    u32x4 val[kUnroll];
    if (WAVE_ROWS) {
        // tc_log == kTileLog: the tile is vectors [col_tile 1024, +1024) of row row_tile
        const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
        const int64_t within = static_cast<int64_t>((col_tile << kTileLog) + wave * (kTileVecs / 4) + lane) * 16;
        const char* const s = src + static_cast<int64_t>(row_tile) * srow + within;
        char* const d = dst + static_cast<int64_t>(row_tile) * drow + within;
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) val[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + u * 1024));
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) __builtin_nontemporal_store(val[u], reinterpret_cast<u32x4*>(d + u * 1024));
    } else {
        const uint32_t tc = 1u << tc_log;
        const uint32_t j = threadIdx.x;
        const uint32_t col = (col_tile << tc_log) + (j & (tc - 1u));
        const uint32_t r = (row_tile << (kTileLog - tc_log)) + (j >> tc_log);
        const char* const s = src + static_cast<int64_t>(col) * 16 + static_cast<int64_t>(r) * srow;
        char* const d = dst + static_cast<int64_t>(col) * 16 + static_cast<int64_t>(r) * drow;
        int64_t sstep[kUnroll], dstep[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t jj = u * kThreads;                 // uniform: columns while they fit the tile row, rows after that
            const uint32_t dc = jj & (tc - 1u), dr = jj >> tc_log;
            sstep[u] = static_cast<int64_t>(dc) * 16 + static_cast<int64_t>(dr) * srow;
            dstep[u] = static_cast<int64_t>(dc) * 16 + static_cast<int64_t>(dr) * drow;
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) val[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + sstep[u]));
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) __builtin_nontemporal_store(val[u], reinterpret_cast<u32x4*>(d + dstep[u]));
    }
}

// Sum of several sources into one destination, each source divided first.
//
// The quotient and every partial sum are rounded to the element type, in the
// order of the sources: bit for bit what a chain of element-wise divisions and
// accumulating box copies gives, in one pass that reads every source once and
// writes the destination once.
// How the sources are divided (SumArgs::divide).
constexpr uint32_t kDivNone = 0;        // divisor 1: summed as they are
constexpr uint32_t kDivDivide = 1;      // a / d
constexpr uint32_t kDivReciprocal = 2;  // d is a power of two: a * (1/d), the same bits as a / d for every a

// The quotient by a divisor d with reciprocal r.  (A third way -- a * r
// corrected twice with fused multiply-adds, the tail of the usual division
// sequence with r computed once on the host, guarded by a range test on a --
// is exact as well but measured slower than the division itself: eight bf16
// slabs divided by 3 and summed in 57 us against 37 us.)
template <uint32_t MODE>
__device__ inline float quotient(float a, float d, float r) {
    return MODE == kDivReciprocal ? a * r : a / d;
}
template <uint32_t MODE>
__device__ inline double quotient(double a, double d, double r) {
    return MODE == kDivReciprocal ? a * r : a / d;
}

// One element (or, for bf16, one 32-bit word holding two) divided; the quotient
// is computed in fp32 for the 16-bit types and rounded once to the element type.
template <typename T>
struct DivOp;
template <>
struct DivOp<float> {
    template <uint32_t MODE>
    static __device__ float apply(float a, double d, double r) { return quotient<MODE>(a, static_cast<float>(d), static_cast<float>(r)); }
};
template <>
struct DivOp<double> {
    template <uint32_t MODE>
    static __device__ double apply(double a, double d, double r) { return quotient<MODE>(a, d, r); }
};
template <>
struct DivOp<bf16_bits> {
    template <uint32_t MODE>
    static __device__ bf16_bits apply(bf16_bits a, double d, double r) {
        bf16_bits out;
        out.u = bf16_rounded(quotient<MODE>(bf16_low(a.u), static_cast<float>(d), static_cast<float>(r)));
        return out;
    }
    template <uint32_t MODE>
    static __device__ uint32_t apply_pair(uint32_t a, double d, double r) {
        const float df = static_cast<float>(d), rf = static_cast<float>(r);
        return bf16_rounded_pair(quotient<MODE>(bf16_low(a), df, rf), quotient<MODE>(bf16_high(a), df, rf));
    }
};
template <>
struct DivOp<f16_bits> {
    template <uint32_t MODE>
    static __device__ f16_bits apply(f16_bits a, double d, double r) {
        _Float16 ha;
        __builtin_memcpy(&ha, &a.u, 2);
        const _Float16 hq = static_cast<_Float16>(quotient<MODE>(static_cast<float>(ha), static_cast<float>(d), static_cast<float>(r)));
        f16_bits out;
        __builtin_memcpy(&out.u, &hq, 2);
        return out;
    }
};
// Integers are only ever summed (the host refuses a divisor other than 1 for them).
template <>
struct DivOp<int32_t> {
    template <uint32_t MODE>
    static __device__ int32_t apply(int32_t a, double, double) { return a; }
};
template <>
struct DivOp<int64_t> {
    template <uint32_t MODE>
    static __device__ int64_t apply(int64_t a, double, double) { return a; }
};

template <typename T, typename V, uint32_t MODE>
__device__ inline V div_vector(V s, double d, double r) {
    if constexpr (MODE == kDivNone) return s;
    constexpr int n = sizeof(V) / sizeof(T);
    if constexpr (std::is_same<T, bf16_bits>::value && sizeof(V) >= 4) {
        constexpr int words = sizeof(V) / 4;
        uint32_t w[words];
        __builtin_memcpy(w, &s, sizeof(V));
#pragma unroll
        for (int i = 0; i < words; ++i) w[i] = DivOp<bf16_bits>::apply_pair<MODE>(w[i], d, r);
        V out;
        __builtin_memcpy(&out, w, sizeof(V));
        return out;
    }
    T sv[n];
    __builtin_memcpy(sv, &s, sizeof(V));
#pragma unroll
    for (int i = 0; i < n; ++i) sv[i] = DivOp<T>::template apply<MODE>(sv[i], d, r);
    V out;
    __builtin_memcpy(&out, sv, sizeof(V));
    return out;
}

constexpr int kMaxSumSources = 64;
constexpr int kSumPiecesSources = 5;        // from this many sources on, whole-tile boxes take sum_pieces_kernel
constexpr uint32_t kSumGroup = 2;   // 2: 27.6 us for eight [4,2048,1024] bf16 slabs, 1: 29.5 us, 4: 31.0 us (registers cost more wavefronts than the loads gain)

struct SumArgs {
    DevBox box;                        // src: the box in source 0
    int64_t delta[kMaxSumSources];     // bytes from source 0 to source q (delta[0] = 0)
    double divisor, reciprocal;
    uint32_t nsrc;
    uint32_t ntiles;
    uint32_t divide;                   // kDivNone, kDivDivide or kDivReciprocal (host side: which instantiation is launched)
    uint32_t pad;
};

#if defined(__HIP_DEVICE_COMPILE__)
typedef const SumArgs __attribute__((address_space(4))) * SumArgsPtr;
#else
typedef const SumArgs* SumArgsPtr;
#endif

template <typename T, typename V, int ND, uint32_t MODE>
__device__ inline void sum_tile(SumArgsPtr sa, uint32_t tile) {
    DevBoxPtr bx = &sa->box;
    int64_t soff[kUnroll], doff[kUnroll];
    bool live[kUnroll];
    tile_offsets<ND>(bx, tile, soff, doff, live);
    const char* const src = bx->src;
    const uint32_t nsrc = sa->nsrc;
    const double divisor = sa->divisor, reciprocal = sa->reciprocal;
    // Sources are fetched kSumGroup at a time (all their loads issued before the first addition) and added in order.
    V acc[kUnroll];
    for (uint32_t q0 = 0; q0 < nsrc; q0 += kSumGroup) {
        V val[kSumGroup][kUnroll];
#pragma unroll
        for (uint32_t g = 0; g < kSumGroup; ++g) {
            const uint32_t q = q0 + g < nsrc ? q0 + g : nsrc - 1;   // past the end: the last source again, fetched and not added
            const char* const sq = src + sa->delta[q];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) val[g][u] = __builtin_nontemporal_load(reinterpret_cast<const V*>(sq + soff[u]));
        }
#pragma unroll
        for (uint32_t g = 0; g < kSumGroup; ++g) {
            if (q0 + g >= nsrc) break;
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) val[g][u] = div_vector<T, V, MODE>(val[g][u], divisor, reciprocal);
            if (q0 + g == 0) {
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) acc[u] = val[g][u];
            } else {
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) acc[u] = add_vectors<T, V>(acc[u], val[g][u]);
            }
        }
    }
    // The destination may be one of the sources: an element is written by the one lane that owns it.
    char* const dst = bx->dst;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
        if (live[u]) __builtin_nontemporal_store(acc[u], reinterpret_cast<V*>(dst + doff[u]));
}

template <typename T, typename V, uint32_t MODE>
__device__ inline void sum_tile_nd(SumArgsPtr sa, uint32_t tile, uint32_t nd) {
    if (nd == 0)
        sum_tile<T, V, 0, MODE>(sa, tile);
    else if (nd == 1)
        sum_tile<T, V, 1, MODE>(sa, tile);
    else if (nd == 2)
        sum_tile<T, V, 2, MODE>(sa, tile);
    else
        sum_tile<T, V, kMaxDevDims, MODE>(sa, tile);
}

template <typename T, uint32_t MODE>
__global__ __launch_bounds__(kThreads) void sum_kernel(const SumArgs args_by_value) {
#if defined(__HIP_DEVICE_COMPILE__)
    SumArgsPtr sa = (SumArgsPtr)__builtin_amdgcn_kernarg_segment_ptr();
#else
    SumArgsPtr sa = &args_by_value;
#endif
    const uint32_t ntiles = sa->ntiles;
    const uint32_t nd = sa->box.nd, vlog = sa->box.vlog;
    for (uint32_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        // A vector holds whole elements: the host lowers the box with the element size as the narrowest vector.
        if (vlog == 4)
            sum_tile_nd<T, u32x4, MODE>(sa, tile, nd);
        else if (vlog == 3) {
            if constexpr (sizeof(T) <= 8) sum_tile_nd<T, u32x2, MODE>(sa, tile, nd);
        } else if (vlog == 2) {
            if constexpr (sizeof(T) <= 4) sum_tile_nd<T, uint32_t, MODE>(sa, tile, nd);
        } else {
            if constexpr (sizeof(T) <= 2) sum_tile_nd<T, uint16_t, MODE>(sa, tile, nd);
        }
    }
}

// The addend that leaves every partial sum as it is, bit for bit: -0.0 for the
// floating-point types (x + -0.0 is x for every x, -0.0 included), 0 for integers.
template <typename T, typename V>
__device__ inline V sum_identity() {
    constexpr int n = sizeof(V) / sizeof(T);
    T e[n];
    for (int i = 0; i < n; ++i) {
        if constexpr (std::is_same<T, float>::value) e[i] = -0.0f;
        else if constexpr (std::is_same<T, double>::value) e[i] = -0.0;
        else if constexpr (std::is_integral<T>::value) e[i] = 0;
        else e[i].u = 0x8000;
    }
    V out;
    __builtin_memcpy(&out, e, sizeof(V));
    return out;
}

// The same sum for many sources (five and more) over a box of whole tiles with
// 16-byte vectors and at most one outer dimension: a workgroup takes a quarter
// tile -- one vector per lane -- and has eight sources in flight, where
// sum_kernel has four vectors of two.  Measured on the slab [4,2048,1024] of
// eight [4,2048,8192] bf16 tensors (rows of 2 KiB, 16 KiB apart): 28.4 us in
// sum_kernel's shape, 26.2 us in this one.  What the figures of a stand-alone
// harness say about why: a workgroup that touches few rows of many tensors
// does better than one that touches many rows of two, as long as the rows are
// shorter than 4 KiB; from 4 KiB on the shapes are within 2 % of each other.
//
// Workgroups go to the eight XCDs in turn, so the three low bits of the
// workgroup number name the XCD, and which address bits they coincide with
// matters too: in the harness, with one row of 2 KiB per 128 threads, the sum
// takes 25.9-26.4 us when they are address bits 14-16 or 15-17 (the natural
// order of quarter tiles here), 32.6 at 16-18, 28.2 at 17-19 (whole tiles of
// eight such rows: sum_kernel's order) and 18-20, 29.9 when every XCD has a
// contiguous eighth.  Orders that move them to bit 19 and above measured
// 25.2 us in one process and 26.5-29 us in the next -- above the page size the
// bits that matter are physical -- so the natural order stays.
//
// The geometry arrives as scalar arguments -- the first sixteen dwords of the
// argument segment are in scalar registers when a wavefront starts -- and the
// table of the sources follows as a structure read with one wide scalar load
// per eight sources: a workgroup that lives for one round of loads cannot
// afford the five rounds of dependent scalar loads a structure read field by
// field costs it.
struct SumSources {
    double divisor, reciprocal;
    int64_t delta[kMaxSumSources];     // bytes from source 0 to source q, padded to a multiple of eight with the last source
};
constexpr int kSumPiecesScalarBytes = 64;   // what precedes the SumSources argument of sum_pieces_kernel

#if defined(__HIP_DEVICE_COMPILE__)
typedef const SumSources __attribute__((address_space(4))) * SumSourcesPtr;
typedef const char __attribute__((address_space(4))) * KernargBytes;
#else
typedef const SumSources* SumSourcesPtr;
#endif

template <typename T, uint32_t MODE>
__global__ __launch_bounds__(kThreads) void sum_pieces_kernel(const char* src0, char* dst0, int64_t srow, int64_t drow, uint32_t col_tiles,
                                                              uint32_t ct_mul, uint32_t ct_shr, uint32_t tc_log, uint32_t nsrc,
                                                              uint32_t unused0, uint32_t unused1, uint32_t unused2,
                                                              const SumSources sources_by_value) {
#if defined(__HIP_DEVICE_COMPILE__)
    SumSourcesPtr ss = (SumSourcesPtr)((KernargBytes)__builtin_amdgcn_kernarg_segment_ptr() + kSumPiecesScalarBytes);
#else
    SumSourcesPtr ss = &sources_by_value;
#endif
    typedef u32x4 V;
    const uint32_t tile = blockIdx.x / kUnroll, part = blockIdx.x % kUnroll;
    const uint32_t row_tile = col_tiles == 1 ? tile : (__umulhi(tile, ct_mul) >> ct_shr);
    const uint32_t col_tile = tile - row_tile * col_tiles;
    const uint32_t v = threadIdx.x + part * kThreads;              // vector number inside the tile
    const uint32_t col = (col_tile << tc_log) + (v & ((1u << tc_log) - 1u));
    const uint32_t r = (row_tile << (kTileLog - tc_log)) + (v >> tc_log);
    const char* const src = src0 + static_cast<int64_t>(col) * 16 + static_cast<int64_t>(r) * srow;
    char* const dst = dst0 + static_cast<int64_t>(col) * 16 + static_cast<int64_t>(r) * drow;
    // Eight sources at a time, all requested before the first addition.  Beyond the last source the table repeats it;
    // what is fetched there is replaced by the element that changes no sum (-0.0, integer 0) rather than skipped, so
    // that no load hangs on a condition and the compiler keeps the eight together.
    constexpr uint32_t G = 8;
    const V nothing = sum_identity<T, V>();
    V acc = nothing;
    for (uint32_t q0 = 0; q0 < nsrc; q0 += G) {
        int64_t delta[G];
#pragma unroll
        for (uint32_t g = 0; g < G; ++g) delta[g] = ss->delta[q0 + g];
        V val[G];
#pragma unroll
        for (uint32_t g = 0; g < G; ++g) val[g] = __builtin_nontemporal_load(reinterpret_cast<const V*>(src + delta[g]));
#pragma unroll
        for (uint32_t g = 0; g < G; ++g) {
            const V quotient = div_vector<T, V, MODE>(val[g], ss->divisor, ss->reciprocal);
            const V sum = add_vectors<T, V>(acc, q0 + g < nsrc ? quotient : nothing);
            acc = q0 + g == 0 ? quotient : sum;              // the first source as it is: -0.0 + 0.0 would lose its sign
        }
    }
    __builtin_nontemporal_store(acc, reinterpret_cast<V*>(dst));
}

// ------------------------------------------------------------------ host --

struct HostDim {
    int64_t n, ss, ds;
};

// Rewrites one box in bytes, merges what can be merged and appends the
// resulting device boxes (more than one only when a box must be split).
int lower_box(const ddl_box_t& in, int elem_size, bool has_src, std::vector<DevBox>* out) {
    if (in.ndim < 1 || in.ndim > DDL_MAX_DIMS) return fail(DDL_E_DIMS, "box ndim %d outside [1,%d]", in.ndim, DDL_MAX_DIMS);
    std::vector<HostDim> dims;
    for (int d = 0; d < in.ndim; ++d) {
        if (in.shape[d] < 0) return fail(DDL_E_SHAPE, "negative box extent %lld in dim %d", (long long)in.shape[d], d);
        if (in.shape[d] == 0) return 0;  // zero volume: nothing to move
    }
    if (in.dst == nullptr || (has_src && in.src == nullptr)) return fail(DDL_E_ARG, "null box pointer");
    if (!aligned_to(in.dst, elem_size & -elem_size) || (has_src && !aligned_to(in.src, elem_size & -elem_size)))
        return fail(DDL_E_ALIGN, "box pointer not aligned to the element size %d", elem_size);
    for (int d = 0; d < in.ndim; ++d) {
        if (in.shape[d] == 1) continue;
        dims.push_back({in.shape[d], has_src ? in.src_stride[d] * elem_size : 0, in.dst_stride[d] * elem_size});
    }
    dims.push_back({elem_size, has_src ? 1 : 0, 1});  // the bytes of one element
    // Merge neighbours that are contiguous on both sides (inner to outer).
    std::vector<HostDim> m;
    for (int d = static_cast<int>(dims.size()) - 1; d >= 0; --d) {
        if (!m.empty()) {
            HostDim& inner = m.back();
            if (dims[d].ss == inner.ss * inner.n && dims[d].ds == inner.ds * inner.n) {
                inner.n *= dims[d].n;
                continue;
            }
        }
        m.push_back(dims[d]);
    }
    std::reverse(m.begin(), m.end());  // m[0] outermost, m.back() = innermost byte run
    // Vector width: the widest power of two (<= 16 B) dividing the innermost run.
    // Base addresses and outer strides only have to be multiples of 4 bytes for
    // the 8- and 16-byte vectors: gfx950 executes dword-aligned multi-dword
    // global accesses at nearly the speed of aligned ones (measured: a copy
    // whose destination is shifted by 4 bytes runs at 5.68 instead of 5.88 TB/s).
    uint64_t align_bits = reinterpret_cast<uintptr_t>(in.dst);
    if (has_src) align_bits |= reinterpret_cast<uintptr_t>(in.src);
    for (size_t d = 0; d + 1 < m.size(); ++d) {
        align_bits |= static_cast<uint64_t>(m[d].ds < 0 ? -m[d].ds : m[d].ds);
        if (has_src) align_bits |= static_cast<uint64_t>(m[d].ss < 0 ? -m[d].ss : m[d].ss);
    }
    uint32_t vlog = 0;
    while (vlog < 4 && ((static_cast<uint64_t>(m.back().n) >> vlog) & 1u) == 0) ++vlog;
    if ((align_bits & 3u) != 0) {
        uint32_t alog = 0;
        while (alog < 2 && ((align_bits >> alog) & 1u) == 0) ++alog;
        vlog = vlog < alog ? vlog : alog;
    }
    const int64_t vbytes = 1ll << vlog;
    m.back().n /= vbytes;
    m.back().ss = has_src ? vbytes : 0;
    m.back().ds = vbytes;
    if (m.back().n == 1 && m.size() > 1) m.pop_back();  // element == vector: the next dimension becomes the columns

    // Split until the box fits 31-bit vector indices and kMaxDevDims dimensions.
    struct Piece {
        std::vector<HostDim> d;
        int64_t so, dof;
    };
    std::vector<Piece> work{{m, 0, 0}};
    while (!work.empty()) {
        Piece p = std::move(work.back());
        work.pop_back();
        uint64_t total = 1;
        bool too_big = false;
        for (const HostDim& h : p.d) {
            if (h.n > static_cast<int64_t>(kMaxVecs) || total * static_cast<uint64_t>(h.n) > kMaxVecs) too_big = true;
            if (!too_big) total *= static_cast<uint64_t>(h.n);
        }
        if (too_big || static_cast<int>(p.d.size()) > kMaxDevDims + 1) {
            // Cut the outermost dimension: in halves when it alone is large,
            // into single slices when there are too many dimensions.
            HostDim o = p.d.front();
            if (static_cast<int>(p.d.size()) > kMaxDevDims + 1 || o.n == 1) {
                for (int64_t i = 0; i < o.n; ++i) {
                    Piece q{std::vector<HostDim>(p.d.begin() + 1, p.d.end()), p.so + i * o.ss, p.dof + i * o.ds};
                    work.push_back(std::move(q));
                }
            } else {
                const int64_t h0 = o.n / 2;
                Piece a = p, b = p;
                a.d.front().n = h0;
                b.d.front().n = o.n - h0;
                b.so += h0 * o.ss;
                b.dof += h0 * o.ds;
                work.push_back(std::move(a));
                work.push_back(std::move(b));
            }
            continue;
        }
        // Innermost dimension = columns, the rest = rows.
        DevBox db{};
        db.src = has_src ? static_cast<const char*>(in.src) + p.so : nullptr;
        db.dst = static_cast<char*>(in.dst) + p.dof;
        const HostDim inner = p.d.back();
        db.cols = static_cast<uint32_t>(inner.n);
        db.css = inner.ss;
        db.cds = inner.ds;
        db.rows = static_cast<uint32_t>(total / static_cast<uint64_t>(inner.n));
        uint32_t tc_log = 0;
        while (tc_log < kTileLog && (1u << tc_log) < db.cols) ++tc_log;
        db.tc_log = tc_log;
        db.col_tiles = (db.cols + (1u << tc_log) - 1) >> tc_log;
        const FastDiv ct = make_fastdiv(db.col_tiles);
        db.ct_mul = ct.mul;
        db.ct_shr = ct.shr;
        db.nd = static_cast<uint32_t>(p.d.size() - 1);
        db.vlog = vlog;
        for (int d = 0; d < kMaxDevDims; ++d) {
            // Unused entries (extent 1, stride 0) sit at the slow end so that the
            // general instantiation may decompose all kMaxDevDims of them.
            const int unused = kMaxDevDims - static_cast<int>(db.nd);
            const bool general = db.nd > 2;
            const int src_d = general ? d - unused : d;
            if (src_d >= 0 && src_d < static_cast<int>(db.nd)) {
                db.dim[d].ss = p.d[src_d].ss;
                db.dim[d].ds = p.d[src_d].ds;
                db.dim[d].fd = make_fastdiv(static_cast<uint32_t>(p.d[src_d].n));
            } else {
                db.dim[d].ss = 0;
                db.dim[d].ds = 0;
                db.dim[d].fd = make_fastdiv(1);
            }
        }
        out->push_back(db);
    }
    return 0;
}

// Whether the boxes of a batch differ in their base addresses only and consist
// of whole tiles, so that uniform_copy_kernel can move them.
constexpr uint64_t kUniformMaxTiles = 16384;   // 256 MiB a launch: beyond that the persistent kernel's fewer, longer-lived workgroups serve as well
inline bool uniform_batch(const Batch& bt, uint32_t n, uint64_t tiles) {
    const DevBox& a = bt.box[0];
    if (n < 1 || tiles > kUniformMaxTiles || tiles % n != 0 || tiles / n > 65535) return false;
    if (a.vlog != 4 || a.nd > 1 || a.css != 16 || a.cds != 16) return false;
    const uint32_t tc = 1u << a.tc_log, tr = kTileVecs >> a.tc_log;
    if (a.cols % tc != 0 || a.rows % tr != 0) return false;
    for (uint32_t k = 1; k < n; ++k) {
        const DevBox& b = bt.box[k];
        if (b.vlog != a.vlog || b.nd != a.nd || b.css != a.css || b.cds != a.cds || b.cols != a.cols || b.rows != a.rows) return false;
        if (a.nd == 1 && (b.dim[0].ss != a.dim[0].ss || b.dim[0].ds != a.dim[0].ds)) return false;
    }
    return true;
}

inline int launch_uniform(const Batch& bt, uint32_t n, uint32_t tiles_per_box, bool round_robin, hipStream_t stream) {
    UniformBatch ub{};
    const DevBox& a = bt.box[0];
    for (uint32_t k = 0; k < n; ++k) {
        ub.src[k] = bt.box[k].src;
        ub.dst[k] = bt.box[k].dst;
    }
    ub.srow = a.nd == 1 ? a.dim[0].ss : 0;
    ub.drow = a.nd == 1 ? a.dim[0].ds : 0;
    ub.tc_log = a.tc_log, ub.col_tiles = a.col_tiles, ub.ct_mul = a.ct_mul, ub.ct_shr = a.ct_shr;
    const bool wave_rows = a.tc_log == kTileLog;
    const dim3 grid = round_robin ? dim3(n, tiles_per_box) : dim3(tiles_per_box, n);
    if (round_robin && wave_rows)
        hipLaunchKernelGGL((uniform_copy_kernel<true, true>), grid, dim3(kThreads), 0, stream, ub);
    else if (round_robin)
        hipLaunchKernelGGL((uniform_copy_kernel<true, false>), grid, dim3(kThreads), 0, stream, ub);
    else if (wave_rows)
        hipLaunchKernelGGL((uniform_copy_kernel<false, true>), grid, dim3(kThreads), 0, stream, ub);
    else
        hipLaunchKernelGGL((uniform_copy_kernel<false, false>), grid, dim3(kThreads), 0, stream, ub);
    return check_launch("uniform_copy_kernel");
}

template <int OP, typename T>
int launch_batches(const std::vector<DevBox>& boxes, hipStream_t stream) {
    size_t i = 0;
    while (i < boxes.size()) {
        Batch bt{};
        uint64_t tiles = 0;
        uint32_t n = 0;
        while (i < boxes.size() && n < kBatch) {
            const uint64_t tr = kTileVecs >> boxes[i].tc_log;  // rows per tile
            const uint64_t t = static_cast<uint64_t>(boxes[i].col_tiles) * ((boxes[i].rows + tr - 1) / tr);
            if (n > 0 && tiles + t > 0x7FFFFFFFull) break;
            bt.box[n] = boxes[i];
            bt.box[n].first_tile = static_cast<uint32_t>(tiles);
            bt.first_tile[n] = static_cast<uint32_t>(tiles);
            tiles += t;
            ++n;
            ++i;
        }
        bt.nbox = n;
        bt.ntiles = static_cast<uint32_t>(tiles);
        // Order of the tiles.  Box after box is the default.  Boxes whose rows
        // are long contiguous runs (the 1 MiB pieces an unpack of
        // [8,4096,1024] bf16 from eight buffers writes into its output, 8 MiB
        // apart) are walked round-robin instead: the few thousand tiles in
        // flight at one moment then touch the pieces of all boxes rather than
        // those of the first few, which spreads the accesses over address bits
        // 20 and up -- measured 5 to 12 % faster for that unpack, depending on
        // the machine, while the pack of the same repartition (rows of 2 KiB)
        // loses 1 % when interleaved and stays box after box.
        // Boxes of equal size that scatter short rows into a wider tensor (the
        // pieces of an all-gather written into their column strips, the unpack of
        // a repartition towards a split of the last dimension) take turns as
        // well: the tiles in flight then complete whole rows of the destination
        // instead of one strip of every row -- 47.7 -> 44.6 us for eight
        // [4,2048,1024] bf16 pieces into [4,2048,8192].  The mirror image, strips
        // gathered into contiguous buffers, reads a strip of every row either
        // way and loses 1 % when its writes alternate between the buffers.
        bool equal = n >= 2 && tiles < 0x7FFFFFFFull, long_runs = true, scatter = true;
        for (uint32_t k = 0; k < n && equal; ++k) {
            const uint64_t own = (k + 1 < n ? bt.first_tile[k + 1] : tiles) - bt.first_tile[k];
            equal = own * n == tiles;
            long_runs = long_runs && (static_cast<uint64_t>(bt.box[k].cols) << bt.box[k].vlog) >= kLongRunBytes;
            scatter = scatter && bt.box[k].nd == 1 && bt.box[k].dim[0].ds > bt.box[k].dim[0].ss;
        }
        const bool interleave = equal && (long_runs || scatter);
        bt.rr = interleave ? make_fastdiv(n) : FastDiv{0, 0, 0, 0};
        if (OP == OP_COPY && uniform_batch(bt, n, tiles)) {
            if (int rc = launch_uniform(bt, n, static_cast<uint32_t>(tiles / n), interleave, stream)) return rc;
            continue;
        }
        const uint32_t blocks = tiles < kPersistentBlocks ? static_cast<uint32_t>(tiles) : kPersistentBlocks;
        hipLaunchKernelGGL((box_kernel<OP, T>), dim3(blocks), dim3(kThreads), 0, stream, bt);
        if (int rc = check_launch("box_kernel")) return rc;
    }
    return 0;
}

int run_boxes(const ddl_box_t* boxes, int nbox, int elem_size, int op, int dtype, bool has_src, hipStream_t stream) {
    if (nbox < 0 || (nbox > 0 && boxes == nullptr)) return fail(DDL_E_ARG, "bad box list (nbox=%d)", nbox);
    if (elem_size < 1 || elem_size > 4096) return fail(DDL_E_ARG, "element size %d outside [1,4096]", elem_size);
    static const int dt_size[] = {0, 4, 8, 2, 2, 4, 8};
    if (op == DDL_OP_ADD) {
        if (dtype < DDL_DT_F32 || dtype > DDL_DT_I64) return fail(DDL_E_ARG, "DDL_OP_ADD needs an arithmetic dtype, got %d", dtype);
        if (dt_size[dtype] != elem_size) return fail(DDL_E_ARG, "dtype %d does not have element size %d", dtype, elem_size);
    } else if (op != DDL_OP_COPY && op != OP_ZERO) {
        return fail(DDL_E_ARG, "unknown box operation %d", op);
    }
    std::vector<DevBox> dev;
    dev.reserve(nbox);
    for (int b = 0; b < nbox; ++b)
        if (int rc = lower_box(boxes[b], elem_size, has_src, &dev)) return rc;
    if (dev.empty()) return 0;
    if (op == OP_ZERO) return launch_batches<OP_ZERO, uint8_t>(dev, stream);
    if (op == DDL_OP_COPY) return launch_batches<OP_COPY, uint8_t>(dev, stream);
    switch (dtype) {
        case DDL_DT_F32: return launch_batches<OP_ADD, float>(dev, stream);
        case DDL_DT_F64: return launch_batches<OP_ADD, double>(dev, stream);
        case DDL_DT_BF16: return launch_batches<OP_ADD, bf16_bits>(dev, stream);
        case DDL_DT_I32: return launch_batches<OP_ADD, int32_t>(dev, stream);
        case DDL_DT_I64: return launch_batches<OP_ADD, int64_t>(dev, stream);
        default: return launch_batches<OP_ADD, f16_bits>(dev, stream);
    }
}

// Builds the box list of a pack / unpack / zero call: one side is a strided
// tensor addressed by (start, shape), the other a contiguous buffer.
int tensor_boxes(const void* tensor, const int64_t* tshape, const int64_t* tstrides, int ndim, int elem_size,
                 int nbox, const int64_t* start, const int64_t* shape, const void* const* bufs, bool tensor_is_src,
                 bool need_bufs, std::vector<ddl_box_t>* out) {
    if (ndim < 1 || ndim > DDL_MAX_DIMS) return fail(DDL_E_DIMS, "ndim %d outside [1,%d]", ndim, DDL_MAX_DIMS);
    if (nbox < 0) return fail(DDL_E_ARG, "negative box count");
    if (nbox == 0) return 0;
    if (!tensor || !tshape || !tstrides || !start || !shape || (need_bufs && !bufs)) return fail(DDL_E_ARG, "null argument");
    if (elem_size < 1) return fail(DDL_E_ARG, "element size %d", elem_size);
    for (int b = 0; b < nbox; ++b) {
        if (need_bufs && bufs[b] == nullptr) continue;
        ddl_box_t bx{};
        bx.ndim = ndim;
        int64_t off = 0, run = 1;
        bool empty = false;
        for (int d = ndim - 1; d >= 0; --d) {
            const int64_t s0 = start[b * ndim + d], n = shape[b * ndim + d];
            if (s0 < 0 || n < 0 || s0 + n > tshape[d])
                return fail(DDL_E_SHAPE, "box %d: [%lld,%lld) outside extent %lld of dim %d", b, (long long)s0,
                            (long long)(s0 + n), (long long)tshape[d], d);
            if (n == 0) empty = true;
            off += s0 * tstrides[d];
            bx.shape[d] = n;
            if (tensor_is_src) {
                bx.src_stride[d] = tstrides[d];
                bx.dst_stride[d] = run;
            } else {
                bx.dst_stride[d] = tstrides[d];
                bx.src_stride[d] = run;
            }
            run *= n;
        }
        if (empty) continue;
        const char* tp = static_cast<const char*>(tensor) + off * elem_size;
        if (tensor_is_src) {
            bx.src = tp;
            bx.dst = const_cast<void*>(bufs[b]);
        } else {
            bx.dst = const_cast<char*>(tp);
            bx.src = need_bufs ? bufs[b] : nullptr;
        }
        out->push_back(bx);
    }
    return 0;
}


template <typename T>
int launch_sum(const std::vector<DevBox>& pieces, const void* const* srcs, int nsrc, double divisor, hipStream_t stream) {
    for (const DevBox& db : pieces) {
        SumArgs sa{};
        sa.box = db;
        for (int q = 0; q < nsrc; ++q) sa.delta[q] = static_cast<const char*>(srcs[q]) - static_cast<const char*>(srcs[0]);
        // The 16-bit types and fp32 divide in fp32, by the divisor as fp32 shows it.
        constexpr bool in_fp32 = !std::is_integral<T>::value && sizeof(T) <= 4;
        const double shown = in_fp32 ? static_cast<double>(static_cast<float>(divisor)) : divisor;
        int exponent = 0;
        const bool power_of_two = std::fabs(std::frexp(shown, &exponent)) == 0.5;
        sa.divisor = shown;
        if (divisor == 1.0 || std::is_integral<T>::value) {
            sa.divide = kDivNone;
        } else if (power_of_two && exponent > -100 && exponent < 100) {
            // An exact reciprocal: the product is the quotient rounded once, as the division is --
            // the same bits for every input without the dozen instructions of a division
            // (eight bf16 slabs [4,2048,1024] divided by 8 and summed: 48.6 -> 28.6 us).
            sa.divide = kDivReciprocal;
            sa.reciprocal = 1.0 / shown;
        } else {
            sa.divide = kDivDivide;
        }
        sa.nsrc = static_cast<uint32_t>(nsrc);
        const uint64_t tr = kTileVecs >> db.tc_log;
        const uint64_t tiles = static_cast<uint64_t>(db.col_tiles) * ((db.rows + tr - 1) / tr);
        sa.ntiles = static_cast<uint32_t>(tiles);
        const bool whole_tiles = db.cols % (1u << db.tc_log) == 0 && db.rows % tr == 0;
        if (nsrc >= kSumPiecesSources && db.vlog == 4 && db.nd <= 1 && db.css == 16 && db.cds == 16 && whole_tiles &&
            tiles * kUnroll <= 0x7FFFFFFFull) {
            const uint32_t items = static_cast<uint32_t>(tiles * kUnroll);
            SumSources ss{};
            ss.divisor = sa.divisor, ss.reciprocal = sa.reciprocal;
            for (int q = 0; q < kMaxSumSources; ++q) ss.delta[q] = sa.delta[q < nsrc ? q : nsrc - 1];
            const int64_t srow = db.nd == 1 ? db.dim[0].ss : 0, drow = db.nd == 1 ? db.dim[0].ds : 0;
#define DDL_LAUNCH_SUM_PIECES(MODE)                                                                                              \
    hipLaunchKernelGGL((sum_pieces_kernel<T, MODE>), dim3(items), dim3(kThreads), 0, stream, db.src, db.dst, srow, drow,            \
                       db.col_tiles, db.ct_mul, db.ct_shr, db.tc_log, static_cast<uint32_t>(nsrc), 0u, 0u, 0u, ss)
            if (sa.divide == kDivNone)
                DDL_LAUNCH_SUM_PIECES(kDivNone);
            else if (sa.divide == kDivReciprocal)
                DDL_LAUNCH_SUM_PIECES(kDivReciprocal);
            else
                DDL_LAUNCH_SUM_PIECES(kDivDivide);
#undef DDL_LAUNCH_SUM_PIECES
            if (int rc = check_launch("sum_pieces_kernel")) return rc;
            continue;
        }
        const uint32_t blocks = tiles < kPersistentBlocks ? static_cast<uint32_t>(tiles) : kPersistentBlocks;
        if (sa.divide == kDivNone)
            hipLaunchKernelGGL((sum_kernel<T, kDivNone>), dim3(blocks), dim3(kThreads), 0, stream, sa);
        else if (sa.divide == kDivReciprocal)
            hipLaunchKernelGGL((sum_kernel<T, kDivReciprocal>), dim3(blocks), dim3(kThreads), 0, stream, sa);
        else
            hipLaunchKernelGGL((sum_kernel<T, kDivDivide>), dim3(blocks), dim3(kThreads), 0, stream, sa);
        if (int rc = check_launch("sum_kernel")) return rc;
    }
    return 0;
}

}  // namespace
}  // namespace ddl

extern "C" {

int ddl_sum_boxes(const ddl_box_t* box, const void* const* srcs, int nsrc, int elem_size, int dtype, double divisor, void* stream) {
    using namespace ddl;
    if (!box || !srcs) return fail(DDL_E_ARG, "sum_boxes: null argument");
    if (nsrc < 1 || nsrc > kMaxSumSources) return fail(DDL_E_UNSUPP, "sum_boxes: %d sources outside [1,%d]", nsrc, kMaxSumSources);
    static const int dt_size[] = {0, 4, 8, 2, 2, 4, 8};
    if (dtype < DDL_DT_F32 || dtype > DDL_DT_I64) return fail(DDL_E_ARG, "sum_boxes needs an arithmetic dtype, got %d", dtype);
    if (dt_size[dtype] != elem_size) return fail(DDL_E_ARG, "dtype %d does not have element size %d", dtype, elem_size);
    if (!(divisor == divisor) || divisor == 0.0) return fail(DDL_E_ARG, "sum_boxes: divisor %g", divisor);
    if ((dtype == DDL_DT_I32 || dtype == DDL_DT_I64) && divisor != 1.0) return fail(DDL_E_UNSUPP, "sum_boxes: integers are summed, not divided");
    for (int q = 0; q < nsrc; ++q) {
        if (!srcs[q]) return fail(DDL_E_ARG, "sum_boxes: source %d is null", q);
        // One vector width serves all sources: they must sit at the same offset from a 16-byte boundary.
        if ((reinterpret_cast<uintptr_t>(srcs[q]) - reinterpret_cast<uintptr_t>(srcs[0])) % 16 != 0)
            return fail(DDL_E_ALIGN, "sum_boxes: source %d is not a multiple of 16 bytes from source 0", q);
    }
    ddl_box_t in = *box;
    in.src = srcs[0];
    std::vector<DevBox> pieces;
    if (int rc = lower_box(in, elem_size, true, &pieces)) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case DDL_DT_F32: return launch_sum<float>(pieces, srcs, nsrc, divisor, s);
        case DDL_DT_F64: return launch_sum<double>(pieces, srcs, nsrc, divisor, s);
        case DDL_DT_BF16: return launch_sum<bf16_bits>(pieces, srcs, nsrc, divisor, s);
        case DDL_DT_I32: return launch_sum<int32_t>(pieces, srcs, nsrc, divisor, s);
        case DDL_DT_I64: return launch_sum<int64_t>(pieces, srcs, nsrc, divisor, s);
        default: return launch_sum<f16_bits>(pieces, srcs, nsrc, divisor, s);
    }
}

int ddl_copy_boxes(const ddl_box_t* boxes, int nbox, int elem_size, int op, int dtype, void* stream) {
    if (op != DDL_OP_COPY && op != DDL_OP_ADD) return ddl::fail(DDL_E_ARG, "unknown box operation %d", op);
    return ddl::run_boxes(boxes, nbox, elem_size, op, dtype, true, static_cast<hipStream_t>(stream));
}

int ddl_pack_boxes(const void* tensor, const int64_t* tensor_shape, const int64_t* tensor_strides, int ndim,
                   int elem_size, int nbox, const int64_t* box_start, const int64_t* box_shape, void* const* bufs,
                   void* stream) {
    std::vector<ddl_box_t> boxes;
    if (int rc = ddl::tensor_boxes(tensor, tensor_shape, tensor_strides, ndim, elem_size, nbox, box_start, box_shape,
                                   const_cast<const void* const*>(bufs), true, true, &boxes))
        return rc;
    return ddl::run_boxes(boxes.data(), static_cast<int>(boxes.size()), elem_size, DDL_OP_COPY, DDL_DT_BITS, true,
                          static_cast<hipStream_t>(stream));
}

int ddl_unpack_boxes(void* tensor, const int64_t* tensor_shape, const int64_t* tensor_strides, int ndim, int elem_size,
                     int nbox, const int64_t* box_start, const int64_t* box_shape, const void* const* bufs, int op,
                     int dtype, void* stream) {
    if (op != DDL_OP_COPY && op != DDL_OP_ADD) return ddl::fail(DDL_E_ARG, "unknown box operation %d", op);
    std::vector<ddl_box_t> boxes;
    if (int rc = ddl::tensor_boxes(tensor, tensor_shape, tensor_strides, ndim, elem_size, nbox, box_start, box_shape,
                                   bufs, false, true, &boxes))
        return rc;
    return ddl::run_boxes(boxes.data(), static_cast<int>(boxes.size()), elem_size, op, dtype, true,
                          static_cast<hipStream_t>(stream));
}

int ddl_zero_boxes(void* tensor, const int64_t* tensor_shape, const int64_t* tensor_strides, int ndim, int elem_size,
                   int nbox, const int64_t* box_start, const int64_t* box_shape, void* stream) {
    std::vector<ddl_box_t> boxes;
    if (int rc = ddl::tensor_boxes(tensor, tensor_shape, tensor_strides, ndim, elem_size, nbox, box_start, box_shape,
                                   nullptr, false, false, &boxes))
        return rc;
    return ddl::run_boxes(boxes.data(), static_cast<int>(boxes.size()), elem_size, ddl::OP_ZERO, DDL_DT_BITS, false,
                          static_cast<hipStream_t>(stream));
}

}  // extern "C"
