// Fused halo staging: zero padding, ghost fill and send-slab pack in ONE pass
// over the padded tensor.  It produces what the reference does in three steps,
//   F.pad                       nn/conv_feature.py:400-407
//   torch.clone + per-dimension pack / unpack loop
//                               backends/mpi_numpy/functional/halo_exchange.py:30-76
// with the slab geometry of HaloExchange._assemble_slices
// (nn/halo_exchange.py:37-99), when every ghost slab is known before the call.
//
// Why the fusion is exact.  Ghost slabs of different exchange dimensions never
// overlap: slab i restricts every dimension j > i to the bulk range, so an
// element lying in ghost strips of several dimensions belongs only to the slab
// of the highest one.  A bulk (send) slab of dimension i restricts dimensions
// j > i to the bulk range too, hence contains ghosts of dimensions < i only --
// the values it must carry under the reference's dimension-ordered loop are
// the final ones.  So every element of the padded tensor has exactly one
// source (a ghost slab, the shard, or zero) and is forwarded to the bulk slabs
// that contain it.
//
// Mapping.  A wavefront owns kRows consecutive rows (all dimensions but the
// last); row geometry is wave-uniform scalar work, the lanes walk the last
// dimension, and the loads of all owned rows are issued before any store so
// that enough bytes are in flight to cover HBM latency.  The innermost face
// (a 1-element-wide slab at a 520-byte pitch in the 130^3 case) costs nothing
// extra here because every row is streamed anyway.
#include "ddl_common.h"

namespace ddl {
namespace {

constexpr int HD = 6;       // tensor dimensions supported by the fused kernel
constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kRows = 8;    // rows per wavefront

struct HaloArgs {
    const char* x;
    char* xpad;
    const char* ghost[HD][2];
    char* bulk[HD][2];
    int64_t xstride[HD];        // elements
    int64_t gstride[HD][2][HD]; // ghost slab strides of (dim, side), dims < L
    int64_t bstride[HD][2][HD];
    int64_t gbase[HD][2];       // offset correction, see slab_offset()
    int64_t bbase[HD][2];
    uint32_t xs[HD], ps[HD], padl[HD];
    uint32_t recvl[HD], recvr[HD], sendl[HD], sendr[HD];
    FastDiv fd[HD];             // division by ps[j]
    int32_t nd;
    uint32_t nrows;             // product of ps[0..nd-2]
};
static_assert(sizeof(HaloArgs) <= 3800, "halo arguments must fit the kernel-argument segment");

struct RowInfo {
    const char* mid;   // element w of the row is mid[w] for wlo <= w < whi
    uint32_t wlo, whi;
    uint32_t special;  // row touches a ghost or bulk strip of a dimension < L
};

// Coordinates of a padded row in dimensions 0..L-1 (loops are fully unrolled so
// that the coordinate array stays in registers).
__device__ inline void row_coords(const HaloArgs& a, uint32_t row, uint32_t (&c)[HD]) {
    const int L = a.nd - 1;
    uint32_t r = row;
#pragma unroll
    for (int j = HD - 2; j > 0; --j) {
        c[j] = 0;
        if (j < L) {
            const uint32_t q = fd_div(r, a.fd[j]);
            c[j] = r - q * a.ps[j];
            r = q;
        }
    }
    c[0] = r;
    c[HD - 1] = 0;
}

template <typename T>
__device__ inline RowInfo classify(const HaloArgs& a, uint32_t row) {
    const int L = a.nd - 1;
    uint32_t c[HD];
    row_coords(a, row, c);
    int gh = -1, gside = 0;
    bool inx = true;
    uint32_t special = 0;
    int64_t xoff = 0;
#pragma unroll
    for (int j = 0; j < HD - 1; ++j) {
        if (j >= L) break;
        const uint32_t lo = a.recvl[j], hi = a.ps[j] - a.recvr[j];
        if (c[j] < lo) {
            gh = j;
            gside = 0;
        } else if (c[j] >= hi) {
            gh = j;
            gside = 1;
        } else if (c[j] < lo + a.sendl[j] || c[j] >= hi - a.sendr[j]) {
            special = 1;
        }
        const uint32_t xc = c[j] - a.padl[j];  // wraps when left of the shard
        inx = inx && xc < a.xs[j];
        xoff += static_cast<int64_t>(xc) * a.xstride[j];
    }
    RowInfo ri;
    ri.special = special | (gh >= 0 ? 1u : 0u);
    if (gh >= 0) {
        int64_t off = a.gbase[gh][gside];
#pragma unroll
        for (int j = 0; j < HD - 1; ++j)
            if (j < L) off += static_cast<int64_t>(c[j]) * a.gstride[gh][gside][j];
        ri.mid = a.ghost[gh][gside] + off * static_cast<int64_t>(sizeof(T));
        ri.wlo = a.recvl[L];
        ri.whi = a.ps[L] - a.recvr[L];
    } else if (inx) {
        ri.mid = a.x + (xoff - static_cast<int64_t>(a.padl[L])) * static_cast<int64_t>(sizeof(T));
        ri.wlo = a.padl[L];
        ri.whi = a.padl[L] + a.xs[L];
    } else {
        ri.mid = nullptr;
        ri.wlo = 0;
        ri.whi = 0;
    }
    return ri;
}

// Forwards the row's values to the bulk slabs of dimensions < L containing it.
template <typename T, int KW>
__device__ inline void forward_row(const HaloArgs& a, uint32_t row, uint32_t w0, const T (&v)[KW]) {
    const int L = a.nd - 1;
    const int lane = threadIdx.x & (kWave - 1);
    uint32_t c[HD];
    row_coords(a, row, c);
    const uint32_t blo = a.recvl[L], bhi = a.ps[L] - a.recvr[L];
    bool inner_bulk = true;  // dimensions j > i (below L) inside their bulk range
#pragma unroll
    for (int i = HD - 2; i >= 0; --i) {
        if (i >= L) continue;
        const uint32_t lo = a.recvl[i], hi = a.ps[i] - a.recvr[i];
        if (inner_bulk) {
            for (int s = 0; s < 2; ++s) {
                const uint32_t s0 = s == 0 ? lo : hi - a.sendr[i];
                const uint32_t s1 = s == 0 ? lo + a.sendl[i] : hi;
                if (a.bulk[i][s] == nullptr || c[i] < s0 || c[i] >= s1) continue;
                int64_t off = a.bbase[i][s];
#pragma unroll
                for (int j = 0; j < HD - 1; ++j)
                    if (j < L) off += static_cast<int64_t>(c[j]) * a.bstride[i][s][j];
                T* dst = reinterpret_cast<T*>(a.bulk[i][s]) + off;
#pragma unroll
                for (int k = 0; k < KW; ++k) {
                    const uint32_t w = w0 + lane + k * kWave;
                    if (w >= blo && w < bhi) dst[w] = v[k];
                }
            }
        }
        inner_bulk = inner_bulk && c[i] >= lo && c[i] < hi;
    }
}

template <typename T, int KW>
__global__ __launch_bounds__(kBlock) void halo_pad_kernel(const HaloArgs a) {
    const int L = a.nd - 1;
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * kWavesPerBlock + threadIdx.x / kWave);
    const uint32_t row0 = wave * kRows;
    if (row0 >= a.nrows) return;
    const uint32_t W = a.ps[L];
    const uint32_t glo = a.recvl[L], ghi = W - a.recvr[L];
    const T* gl = reinterpret_cast<const T*>(a.ghost[L][0]);
    const T* gr = reinterpret_cast<const T*>(a.ghost[L][1]);
    T* bl = reinterpret_cast<T*>(a.bulk[L][0]);
    T* br = reinterpret_cast<T*>(a.bulk[L][1]);

    RowInfo ri[kRows];
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
        if (row0 + i < a.nrows) {
            ri[i] = classify<T>(a, row0 + i);
        } else {
            ri[i].mid = nullptr;
            ri[i].wlo = ri[i].whi = 0;
            ri[i].special = 0;
        }
    }

    for (uint32_t w0 = 0; w0 < W; w0 += kWave * KW) {
        T v[kRows][KW];
#pragma unroll
        for (int i = 0; i < kRows; ++i) {
            const uint32_t row = row0 + i;
#pragma unroll
            for (int k = 0; k < KW; ++k) {
                const uint32_t w = w0 + lane + k * kWave;
                T t = T(0);
                if (row < a.nrows && w < W) {
                    if (w < glo) {
                        t = gl[static_cast<int64_t>(row) * a.recvl[L] + w];
                    } else if (w >= ghi) {
                        t = gr[static_cast<int64_t>(row) * a.recvr[L] + (w - ghi)];
                    } else if (w >= ri[i].wlo && w < ri[i].whi) {
                        t = reinterpret_cast<const T*>(ri[i].mid)[w];
                    }
                }
                v[i][k] = t;
            }
        }
#pragma unroll
        for (int i = 0; i < kRows; ++i) {
            const uint32_t row = row0 + i;
            if (row >= a.nrows) continue;
            T* out = reinterpret_cast<T*>(a.xpad) + static_cast<int64_t>(row) * W;
#pragma unroll
            for (int k = 0; k < KW; ++k) {
                const uint32_t w = w0 + lane + k * kWave;
                if (w < W) {
                    out[w] = v[i][k];
                    if (bl && w >= glo && w < glo + a.sendl[L]) bl[static_cast<int64_t>(row) * a.sendl[L] + (w - glo)] = v[i][k];
                    if (br && w >= ghi - a.sendr[L] && w < ghi)
                        br[static_cast<int64_t>(row) * a.sendr[L] + (w - (ghi - a.sendr[L]))] = v[i][k];
                }
            }
            if (ri[i].special) forward_row<T, KW>(a, row, w0, v[i]);
        }
    }
}

template <typename T>
int launch_halo(const HaloArgs& a, hipStream_t s) {
    const uint32_t waves = (a.nrows + kRows - 1) / kRows;
    const uint32_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    const uint32_t W = a.ps[a.nd - 1];
    if (W <= 64)
        hipLaunchKernelGGL((halo_pad_kernel<T, 1>), dim3(blocks), dim3(kBlock), 0, s, a);
    else if (W <= 128)
        hipLaunchKernelGGL((halo_pad_kernel<T, 2>), dim3(blocks), dim3(kBlock), 0, s, a);
    else if (W <= 192)
        hipLaunchKernelGGL((halo_pad_kernel<T, 3>), dim3(blocks), dim3(kBlock), 0, s, a);
    else
        hipLaunchKernelGGL((halo_pad_kernel<T, 4>), dim3(blocks), dim3(kBlock), 0, s, a);
    return check_launch("halo_pad_kernel");
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_halo_pad_exchange(const void* x, void* xpad, const int64_t* x_shape, int ndim, int elem_size,
                                     const int64_t* pad, const int64_t* recv, const int64_t* send,
                                     const void* const* ghost_bufs, void* const* bulk_bufs, void* stream) {
    using namespace ddl;
    if (ndim < 1 || ndim > DDL_MAX_DIMS) return fail(DDL_E_DIMS, "halo: ndim %d outside [1,%d]", ndim, DDL_MAX_DIMS);
    if (!x_shape || !pad || !recv || !send) return fail(DDL_E_ARG, "halo: null geometry argument");
    if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8)
        return fail(DDL_E_ARG, "halo: element size %d not in {1,2,4,8}", elem_size);

    // Leading dimensions that carry no padding and no exchange are folded into
    // one (batch x channel in the convolution case).
    int64_t xs[DDL_MAX_DIMS], pl[DDL_MAX_DIMS], pr[DDL_MAX_DIMS], rl[DDL_MAX_DIMS], rr[DDL_MAX_DIMS], sl[DDL_MAX_DIMS],
        sr[DDL_MAX_DIMS];
    int src_dim[DDL_MAX_DIMS];
    int nd = 0;
    for (int d = 0; d < ndim; ++d) {
        const int64_t v[7] = {x_shape[d], pad[2 * d], pad[2 * d + 1], recv[2 * d], recv[2 * d + 1], send[2 * d], send[2 * d + 1]};
        for (int q = 0; q < 7; ++q)
            if (v[q] < 0) return fail(DDL_E_ARG, "halo: negative geometry value in dim %d", d);
        const bool plain = v[1] == 0 && v[2] == 0 && v[3] == 0 && v[4] == 0 && v[5] == 0 && v[6] == 0;
        const bool prev_plain = nd > 0 && pl[nd - 1] == 0 && pr[nd - 1] == 0 && rl[nd - 1] == 0 && rr[nd - 1] == 0 &&
                                sl[nd - 1] == 0 && sr[nd - 1] == 0;
        if (plain && prev_plain && d != ndim - 1) {
            xs[nd - 1] *= v[0];
            continue;
        }
        xs[nd] = v[0]; pl[nd] = v[1]; pr[nd] = v[2]; rl[nd] = v[3]; rr[nd] = v[4]; sl[nd] = v[5]; sr[nd] = v[6];
        src_dim[nd] = d;
        ++nd;
    }
    if (nd > HD) return fail(DDL_E_UNSUPP, "halo: %d dimensions left after folding, at most %d supported", nd, HD);

    HaloArgs a{};
    a.nd = nd;
    a.x = static_cast<const char*>(x);
    a.xpad = static_cast<char*>(xpad);
    int64_t ps[HD];
    int64_t total = 1, nrows = 1;
    for (int j = 0; j < nd; ++j) {
        ps[j] = xs[j] + pl[j] + pr[j];
        if (rl[j] + sl[j] > ps[j] - rr[j] || rr[j] + sr[j] > ps[j] - rl[j])
            return fail(DDL_E_SHAPE, "halo: ghost+bulk widths exceed the padded extent %lld in dim %d", (long long)ps[j], src_dim[j]);
        if (ps[j] >= (1ll << 31)) return fail(DDL_E_UNSUPP, "halo: padded extent too large");
        total *= ps[j];
        if (j < nd - 1) nrows *= ps[j];
    }
    if (total == 0) return 0;
    if (nrows >= (1ll << 31) - 4096) return fail(DDL_E_UNSUPP, "halo: more than 2^31 rows");
    if (!xpad) return fail(DDL_E_ARG, "halo: null output");
    int64_t xvol = 1;
    for (int j = 0; j < nd; ++j) xvol *= xs[j];
    if (xvol > 0 && !x) return fail(DDL_E_ARG, "halo: null input");
    if (!aligned_to(xpad, elem_size) || !aligned_to(x, elem_size)) return fail(DDL_E_ALIGN, "halo: tensor misaligned");
    a.nrows = static_cast<uint32_t>(nrows);
    int64_t st = 1;
    for (int j = nd - 1; j >= 0; --j) {
        a.xstride[j] = st;
        st *= xs[j];
        a.xs[j] = static_cast<uint32_t>(xs[j]);
        a.ps[j] = static_cast<uint32_t>(ps[j]);
        a.padl[j] = static_cast<uint32_t>(pl[j]);
        a.recvl[j] = static_cast<uint32_t>(rl[j]);
        a.recvr[j] = static_cast<uint32_t>(rr[j]);
        a.sendl[j] = static_cast<uint32_t>(sl[j]);
        a.sendr[j] = static_cast<uint32_t>(sr[j]);
        a.fd[j] = make_fastdiv(static_cast<uint32_t>(ps[j] > 0 ? ps[j] : 1));
    }
    const int L = nd - 1;
    for (int i = 0; i < nd; ++i) {
        for (int s = 0; s < 2; ++s) {
            const int d = src_dim[i];
            const void* gb = ghost_bufs ? ghost_bufs[2 * d + s] : nullptr;
            void* bb = bulk_bufs ? bulk_bufs[2 * d + s] : nullptr;
            const int64_t gw = s == 0 ? rl[i] : rr[i];
            const int64_t bw = s == 0 ? sl[i] : sr[i];
            if (gw > 0 && !gb) return fail(DDL_E_ARG, "halo: ghost width %lld in dim %d side %d but no slab given", (long long)gw, d, s);
            if (!aligned_to(gb, elem_size) || !aligned_to(bb, elem_size)) return fail(DDL_E_ALIGN, "halo: slab misaligned");
            a.ghost[i][s] = gw > 0 ? static_cast<const char*>(gb) : nullptr;
            a.bulk[i][s] = bw > 0 ? static_cast<char*>(bb) : nullptr;
            // Slab extents: j < i full, j == i the strip, j > i the bulk range.
            for (int kind = 0; kind < 2; ++kind) {
                const int64_t width = kind == 0 ? gw : bw;
                const int64_t strip0 = kind == 0 ? (s == 0 ? 0 : ps[i] - rr[i]) : (s == 0 ? rl[i] : ps[i] - rr[i] - sr[i]);
                int64_t ext[HD], str[HD];
                for (int j = 0; j < nd; ++j) ext[j] = j < i ? ps[j] : (j == i ? width : ps[j] - rl[j] - rr[j]);
                int64_t run = 1;
                for (int j = nd - 1; j >= 0; --j) {
                    str[j] = run;
                    run *= ext[j];
                }
                int64_t base = -strip0 * str[i];
                for (int j = i + 1; j < nd; ++j) base -= rl[j] * str[j];
                for (int j = 0; j < L; ++j) (kind == 0 ? a.gstride : a.bstride)[i][s][j] = str[j];
                (kind == 0 ? a.gbase : a.bbase)[i][s] = base;
            }
        }
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (elem_size) {
        case 1: return launch_halo<uint8_t>(a, s);
        case 2: return launch_halo<uint16_t>(a, s);
        case 4: return launch_halo<uint32_t>(a, s);
        default: return launch_halo<uint64_t>(a, s);
    }
}
