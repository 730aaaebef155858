// Box copies: strided <-> strided moves of rectangular sub-volumes, several
// boxes per launch.  This is the pack / unpack / self-copy work of Repartition
// (reference: backends/mpi_numpy/functional/repartition.py:158-208) and of
// HaloExchange (backends/mpi_numpy/functional/halo_exchange.py:50-74, 115-140).
//
// Host side: every box is rewritten in BYTES, unit dimensions are dropped,
// dimensions that are contiguous on both sides are merged, and the widest
// power-of-two vector (<= 16 B) that divides the innermost run, both base
// addresses and every remaining stride is chosen.  Device side: one workgroup
// moves a tile of 256 x 4 vectors of one box; a vector's position is recovered
// from its linear index with multiply-high divisions, so nothing but the box
// table (passed by value as kernel arguments) is read besides the payload.
#include "ddl_common.h"

#include <algorithm>
#include <vector>

namespace ddl {
namespace {

constexpr int kMaxDevDims = 6;   // dimensions left after merging
constexpr int kBatch = 16;       // boxes per launch (kernel-argument budget)
constexpr int kThreads = 256;
constexpr int kUnroll = 4;
constexpr uint32_t kTileVecs = kThreads * kUnroll;
constexpr uint64_t kMaxVecs = (1ull << 31) - kTileVecs;

enum Op { OP_COPY = 0, OP_ADD = 1, OP_ZERO = 2 };

struct DevDim {
    int64_t ss;  // source stride, bytes
    int64_t ds;  // destination stride, bytes
    FastDiv fd;  // divide by the extent (in vectors for the innermost one)
};

struct DevBox {
    const char* src;
    char* dst;
    uint32_t total;       // vectors in the box
    uint32_t nd;          // dimensions used
    uint32_t vlog;        // log2(vector bytes)
    uint32_t first_tile;  // first workgroup of this box in the launch
    DevDim dim[kMaxDevDims];
};

struct Batch {
    DevBox box[kBatch];
    uint32_t nbox;
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

template <>
struct AddOp<bf16_bits> {
    // fp32 add, round to nearest even, quiet NaN: the arithmetic ATen uses for
    // a bf16 add.
    static __device__ bf16_bits apply(bf16_bits a, bf16_bits b) {
        const float fa = __uint_as_float(static_cast<uint32_t>(a.u) << 16);
        const float fb = __uint_as_float(static_cast<uint32_t>(b.u) << 16);
        const float s = fa + fb;
        uint32_t u = __float_as_uint(s);
        bf16_bits r;
        if (s != s) {
            r.u = 0x7FC0;
        } else {
            u += 0x7FFFu + ((u >> 16) & 1u);
            r.u = static_cast<uint16_t>(u >> 16);
        }
        return r;
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
    T dv[n], sv[n];
    __builtin_memcpy(dv, &d, sizeof(V));
    __builtin_memcpy(sv, &s, sizeof(V));
#pragma unroll
    for (int i = 0; i < n; ++i) dv[i] = AddOp<T>::apply(dv[i], sv[i]);
    V out;
    __builtin_memcpy(&out, dv, sizeof(V));
    return out;
}

template <int OP, typename T, typename V>
__device__ inline void move_tile(const DevBox& bx, uint32_t tile) {
    const uint32_t v0 = tile * kTileVecs + threadIdx.x;
    int64_t soff[kUnroll], doff[kUnroll];
    bool live[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        uint32_t r = v0 + u * kThreads;
        live[u] = r < bx.total;
        int64_t so = 0, dof = 0;
        for (int d = static_cast<int>(bx.nd) - 1; d > 0; --d) {
            const uint32_t q = fd_div(r, bx.dim[d].fd);
            const uint32_t idx = r - q * bx.dim[d].fd.div;
            so += static_cast<int64_t>(idx) * bx.dim[d].ss;
            dof += static_cast<int64_t>(idx) * bx.dim[d].ds;
            r = q;
        }
        so += static_cast<int64_t>(r) * bx.dim[0].ss;
        dof += static_cast<int64_t>(r) * bx.dim[0].ds;
        soff[u] = so;
        doff[u] = dof;
    }
    if constexpr (OP == OP_ZERO) {
        V z;
        __builtin_memset(&z, 0, sizeof(V));
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
            if (live[u]) *reinterpret_cast<V*>(bx.dst + doff[u]) = z;
        return;
    }
    V val[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
        if (live[u]) val[u] = *reinterpret_cast<const V*>(bx.src + soff[u]);
    if constexpr (OP == OP_ADD) {
        if constexpr (sizeof(V) >= sizeof(T)) {
            V cur[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                if (live[u]) cur[u] = *reinterpret_cast<const V*>(bx.dst + doff[u]);
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                if (live[u]) val[u] = add_vectors<T, V>(cur[u], val[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
        if (live[u]) *reinterpret_cast<V*>(bx.dst + doff[u]) = val[u];
}

template <int OP, typename T>
__global__ __launch_bounds__(kThreads) void box_kernel(const Batch bt) {
    const uint32_t b = blockIdx.x;
    uint32_t bi = 0;
    for (uint32_t i = 1; i < bt.nbox; ++i) bi = (b >= bt.box[i].first_tile) ? i : bi;
    const DevBox& bx = bt.box[bi];
    const uint32_t tile = b - bx.first_tile;
    switch (bx.vlog) {
        case 4: move_tile<OP, T, uint4>(bx, tile); break;
        case 3: move_tile<OP, T, uint2>(bx, tile); break;
        case 2: move_tile<OP, T, uint32_t>(bx, tile); break;
        case 1: move_tile<OP, T, uint16_t>(bx, tile); break;
        default: move_tile<OP, T, uint8_t>(bx, tile); break;
    }
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
    // Vector width: divides the run, the base addresses and every outer stride.
    uint64_t bits = static_cast<uint64_t>(m.back().n) | reinterpret_cast<uintptr_t>(in.dst) | 16u;
    if (has_src) bits |= reinterpret_cast<uintptr_t>(in.src);
    for (size_t d = 0; d + 1 < m.size(); ++d) {
        bits |= static_cast<uint64_t>(m[d].ds < 0 ? -m[d].ds : m[d].ds);
        if (has_src) bits |= static_cast<uint64_t>(m[d].ss < 0 ? -m[d].ss : m[d].ss);
    }
    uint32_t vlog = 0;
    while (vlog < 4 && ((bits >> vlog) & 1u) == 0) ++vlog;
    const int64_t vbytes = 1ll << vlog;
    m.back().n /= vbytes;
    m.back().ss = has_src ? vbytes : 0;
    m.back().ds = vbytes;
    if (m.back().n == 1 && m.size() > 1) m.pop_back();

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
        if (too_big || static_cast<int>(p.d.size()) > kMaxDevDims) {
            // Cut the outermost dimension: in halves when it alone is large,
            // into single slices when there are too many dimensions.
            HostDim o = p.d.front();
            if (static_cast<int>(p.d.size()) > kMaxDevDims || o.n == 1) {
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
        DevBox db{};
        db.src = has_src ? static_cast<const char*>(in.src) + p.so : nullptr;
        db.dst = static_cast<char*>(in.dst) + p.dof;
        db.total = static_cast<uint32_t>(total);
        db.nd = static_cast<uint32_t>(p.d.size());
        db.vlog = vlog;
        for (size_t d = 0; d < p.d.size(); ++d) {
            db.dim[d].ss = p.d[d].ss;
            db.dim[d].ds = p.d[d].ds;
            db.dim[d].fd = make_fastdiv(static_cast<uint32_t>(p.d[d].n));
        }
        out->push_back(db);
    }
    return 0;
}

template <int OP, typename T>
int launch_batches(const std::vector<DevBox>& boxes, hipStream_t stream) {
    size_t i = 0;
    while (i < boxes.size()) {
        Batch bt{};
        uint64_t tiles = 0;
        uint32_t n = 0;
        while (i < boxes.size() && n < kBatch) {
            const uint64_t t = (static_cast<uint64_t>(boxes[i].total) + kTileVecs - 1) / kTileVecs;
            if (n > 0 && tiles + t > 0x7FFFFFFFull) break;
            bt.box[n] = boxes[i];
            bt.box[n].first_tile = static_cast<uint32_t>(tiles);
            tiles += t;
            ++n;
            ++i;
        }
        bt.nbox = n;
        hipLaunchKernelGGL((box_kernel<OP, T>), dim3(static_cast<uint32_t>(tiles)), dim3(kThreads), 0, stream, bt);
        if (int rc = check_launch("box_kernel")) return rc;
    }
    return 0;
}

int run_boxes(const ddl_box_t* boxes, int nbox, int elem_size, int op, int dtype, bool has_src, hipStream_t stream) {
    if (nbox < 0 || (nbox > 0 && boxes == nullptr)) return fail(DDL_E_ARG, "bad box list (nbox=%d)", nbox);
    if (elem_size < 1 || elem_size > 4096) return fail(DDL_E_ARG, "element size %d outside [1,4096]", elem_size);
    static const int dt_size[] = {0, 4, 8, 2, 2};
    if (op == DDL_OP_ADD) {
        if (dtype < DDL_DT_F32 || dtype > DDL_DT_F16) return fail(DDL_E_ARG, "DDL_OP_ADD needs a floating dtype, got %d", dtype);
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

}  // namespace
}  // namespace ddl

extern "C" {

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
