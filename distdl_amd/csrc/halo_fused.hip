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
// Two kernels.  halo_flat_kernel (further down) serves 2-, 4- and 8-byte
// elements and writes the padded tensor in whole 128-byte lines;
// halo_pad_kernel serves everything else and writes it row by row.
//
// Mapping of halo_pad_kernel.  Dimensions are named L (last, columns), M (second
// to last, rows) and "outer" (the rest, a plane index).  A workgroup owns one
// plane and a chunk of its rows: everything that depends on the outer coordinates only
// (which slab or shard plane feeds the rows, which bulk slabs take them, all
// base offsets) is wave-uniform scalar work done once per workgroup.  Each row
// is then a run [wlo, whi) copied from one source with 16-byte vectors -- the
// padded row starts are only 4-byte aligned, which gfx950 handles at nearly
// full speed -- plus a few edge elements (padding zeros, last-dimension ghosts,
// the run's remainder) handled one element per lane.  LPR lanes share a row, so
// a wavefront covers 64/LPR rows per instruction and keeps kUnroll such row
// groups in flight before the first store.
#include "ddl_common.h"

namespace ddl {
namespace {

constexpr int HD = 6;        // tensor dimensions supported by the fused kernel
constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kUnroll = 4;   // row groups in flight per wavefront (lean path)
constexpr int kGen = 1;      // row groups in flight in the general path

struct Slab {
    char* ptr;               // nullptr when the slab is absent
    int64_t base;            // element offset of padded coordinate 0 (may be negative)
    int64_t stride[HD - 1];  // element strides of dimensions 0..L-1 (dimension L has stride 1)
};

// Arguments of halo_flat_kernel are laid out for few, wide scalar loads.
struct FlatTop {
    const char* x;           // shard
    char* xpad;
    const char* gm[2];       // ghost slabs of M (nullptr when absent)
    const char* gl;          // ghost slabs of L
    const char* gr;
    int64_t xstrM;           // shard stride of M
    int64_t x_off0;          // -(padl[M] * xstrM + padl[L]): shard offset of padded (h, w) = (0, 0) in shard plane 0
    uint32_t total;          // elements of the padded tensor (< 2^31)
    uint32_t nstages;        // pieces of kStage consecutive elements
    uint32_t W, H;           // ps[L], ps[M]
    uint32_t fdW_mul, fdW_shr, fdH_mul, fdH_shr;
    uint32_t glo, ghi;       // bulk range of L
    uint32_t hlo, hhi;       // bulk range of M
    uint32_t padL, xhiL;     // shard columns [padL, xhiL)
    uint32_t padM, xsM;
    uint32_t m_l1, m_r0;     // rows [hlo, m_l1) and [m_r0, hhi) feed the bulk slabs of M (empty without a slab)
    uint32_t n_ghost;        // ghost columns of a row, recvl[L] + recvr[L]
    uint32_t fdg_mul, fdg_shr;
    uint32_t any_outer;      // some dimension below M has a bulk slab
    uint32_t n_bl, n_br;     // columns of the left / right bulk strip of L (0 without a slab)
    uint32_t sl, sr;         // sendl[L], sendr[L]
    uint32_t fds_mul, fds_shr;   // division by n_bl + n_br
};
struct FlatDim {
    uint32_t ps, fd_mul, fd_shr;
    uint32_t lo, hi;         // bulk range
    uint32_t padl, xs;
    uint32_t strip_l1, strip_r0;   // coordinates [lo, strip_l1) and [strip_r0, hi) feed this dimension's bulk slabs
    uint32_t reserved;       // keeps xstride 8-byte aligned
    int64_t xstride;
};

struct HaloArgs {
    const char* x;
    char* xpad;
    Slab ghost[HD][2];
    Slab bulk[HD][2];
    int64_t xstride[HD];
    uint32_t xs[HD], ps[HD], padl[HD];
    uint32_t recvl[HD], recvr[HD], sendl[HD], sendr[HD];
    FastDiv fd[HD];          // division by ps[j]
    int32_t nd;              // >= 2
    uint32_t nplanes;        // product of ps[0..nd-3]
    uint32_t row_chunks;     // workgroups per plane
    uint32_t rows_per_block;
    uint32_t max_vecs;       // vectors of the longest run of any row
    uint32_t max_edge;       // single-element tasks per row, upper bound
    FlatTop top;             // halo_flat_kernel: what every wavefront reads first, kept together
    FlatDim outer[HD - 2];   // halo_flat_kernel: the dimensions below M
};
static_assert(sizeof(HaloArgs) <= 3900, "halo arguments must fit the kernel-argument segment");

#if defined(__HIP_DEVICE_COMPILE__)
typedef const HaloArgs __attribute__((address_space(4))) * ArgsPtr;
typedef const Slab __attribute__((address_space(4))) * SlabPtr;
#else
typedef const HaloArgs* ArgsPtr;
typedef const Slab* SlabPtr;
#endif

template <typename T, int N>
struct VecType {
    typedef T type __attribute__((ext_vector_type(N), aligned(sizeof(T))));
};
template <typename T>
struct VecType<T, 1> {
    typedef T type;
};

// Offset of padded coordinates (c[0..M-1], h, w) inside a slab.
__device__ inline int64_t slab_offset(SlabPtr b, const uint32_t (&c)[HD], int M, uint32_t h, uint32_t w) {
    int64_t off = b->base + static_cast<int64_t>(h) * b->stride[M] + w;
#pragma unroll
    for (int j = 0; j < HD - 2; ++j)
        if (j < M) off += static_cast<int64_t>(c[j]) * b->stride[j];
    return off;
}

// Stores `val` (a vector of the row's run, or one edge element) into every
// bulk slab of a dimension below L that contains position (c, h, w).
template <typename T, typename V>
__device__ inline void forward_below_L(ArgsPtr a, const uint32_t (&c)[HD], int M, uint32_t h, uint32_t w, bool lane_on,
                                       V val) {
    const uint32_t hlo = a->recvl[M], hhi = a->ps[M] - a->recvr[M];
    // dimension M: the row's own strips; outer dimensions are unrestricted
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        SlabPtr b = &a->bulk[M][s];
        if (b->ptr == nullptr) continue;                                   // scalar test
        const uint32_t s0 = s == 0 ? hlo : hhi - a->sendr[M], s1 = s == 0 ? hlo + a->sendl[M] : hhi;
        if (lane_on && h >= s0 && h < s1) *reinterpret_cast<V*>(reinterpret_cast<T*>(b->ptr) + slab_offset(b, c, M, h, w)) = val;
    }
    // outer dimension i: decided by the plane, and the row must be in the bulk range of M
    const bool h_bulk = h >= hlo && h < hhi;
    bool inner_bulk = true;   // outer dimensions above i inside their bulk range
#pragma unroll
    for (int i = HD - 3; i >= 0; --i) {
        if (i >= M) continue;
        const uint32_t lo = a->recvl[i], hi = a->ps[i] - a->recvr[i];
        if (inner_bulk) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                SlabPtr b = &a->bulk[i][s];
                const uint32_t s0 = s == 0 ? lo : hi - a->sendr[i], s1 = s == 0 ? lo + a->sendl[i] : hi;
                if (b->ptr == nullptr || c[i] < s0 || c[i] >= s1) continue;   // scalar test
                if (lane_on && h_bulk) *reinterpret_cast<V*>(reinterpret_cast<T*>(b->ptr) + slab_offset(b, c, M, h, w)) = val;
            }
        }
        inner_bulk = inner_bulk && c[i] >= lo && c[i] < hi;
    }
}

template <typename T, int LPR>
__global__ __launch_bounds__(kBlock) void halo_pad_kernel(const HaloArgs args_by_value) {
#if defined(__HIP_DEVICE_COMPILE__)
    ArgsPtr a = (ArgsPtr)__builtin_amdgcn_kernarg_segment_ptr();
#else
    ArgsPtr a = &args_by_value;
#endif
    constexpr int EPV = sizeof(T) >= 4 ? 16 / sizeof(T) : 1;   // elements per vector
    typedef typename VecType<T, EPV>::type V;
    constexpr int RPI = kWave / LPR;                            // rows per wavefront instruction

    const int nd = a->nd;
    const int L = nd - 1, M = nd - 2;
    const uint32_t plane = blockIdx.x / a->row_chunks;          // scalar
    const uint32_t chunk = blockIdx.x - plane * a->row_chunks;
    const uint32_t W = a->ps[L], H = a->ps[M];
    const uint32_t glo = a->recvl[L], ghi = W - a->recvr[L];
    const uint32_t sl = a->sendl[L], sr = a->sendr[L];
    const uint32_t hlo = a->recvl[M], hhi = H - a->recvr[M];

    // ---- outer coordinates and what they decide (scalar) ----
    uint32_t c[HD];
    {
        uint32_t r = plane;
#pragma unroll
        for (int j = HD - 3; j > 0; --j) {
            c[j] = 0;
            if (j < M) {
                const uint32_t n = a->ps[j];
                const uint32_t q = n == 1 ? r : (__umulhi(r, a->fd[j].mul) >> a->fd[j].shr);
                c[j] = r - q * n;
                r = q;
            }
        }
        c[0] = M > 0 ? r : 0;
        c[HD - 2] = c[HD - 1] = 0;
    }
    const int64_t plane_row0 = static_cast<int64_t>(plane) * H;
    bool in_x = true;
    int64_t x_off = 0;
    int gh = -1, gside = 0;
#pragma unroll
    for (int j = 0; j < HD - 2; ++j) {
        if (j < M) {
            const uint32_t lo = a->recvl[j], hi = a->ps[j] - a->recvr[j];
            if (c[j] < lo) {
                gh = j;
                gside = 0;
            } else if (c[j] >= hi) {
                gh = j;
                gside = 1;
            }
            const uint32_t xc = c[j] - a->padl[j];               // wraps when left of the shard
            in_x = in_x && xc < a->xs[j];
            x_off += static_cast<int64_t>(xc) * a->xstride[j];
        }
    }
    // Row sources decided by the plane: an outer ghost slab, or the two ghost slabs of M.
    const char* gh_ptr = nullptr;
    int64_t gh_off = 0, gh_mstride = 0;
    if (gh >= 0) {
        SlabPtr g = &a->ghost[gh][gside];
        gh_ptr = g->ptr;
        gh_off = slab_offset(g, c, M, 0, 0);
        gh_mstride = g->stride[M];
    }
    const char* gm_ptr[2];
    int64_t gm_off[2], gm_mstride[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
        SlabPtr g = &a->ghost[M][s];
        gm_ptr[s] = g->ptr;
        gm_off[s] = slab_offset(g, c, M, 0, 0);
        gm_mstride[s] = g->stride[M];
    }
    const T* gl = reinterpret_cast<const T*>(a->ghost[L][0].ptr);
    const T* gr = reinterpret_cast<const T*>(a->ghost[L][1].ptr);
    T* bl = reinterpret_cast<T*>(a->bulk[L][0].ptr);
    T* br = reinterpret_cast<T*>(a->bulk[L][1].ptr);
    const uint32_t n_bl = bl ? sl : 0u, n_br = br ? sr : 0u;
    const uint32_t rl = a->recvl[L], rr = a->recvr[L];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const uint32_t lc = lane & (LPR - 1);                        // this lane's position inside its row
    const uint32_t sub = lane / LPR;                             // which of the wavefront's RPI rows
    const uint32_t h_begin = chunk * a->rows_per_block;
    const uint32_t h_end = h_begin + a->rows_per_block < H ? h_begin + a->rows_per_block : H;
    const uint32_t xsM = a->xs[M], padM = a->padl[M], padL = a->padl[L], xsL = a->xs[L];
    const int64_t xstrM = a->xstride[M];
    const T* xbase = reinterpret_cast<const T*>(a->x);
    T* obase = reinterpret_cast<T*>(a->xpad);
    const uint32_t max_vecs = a->max_vecs, max_edge = a->max_edge;

    // Does any bulk slab of an outer dimension take rows of this plane?  (scalar)
    bool outer_forward = false;
    {
        bool inner_bulk = true;
#pragma unroll
        for (int i = HD - 3; i >= 0; --i) {
            if (i >= M) continue;
            const uint32_t lo = a->recvl[i], hi = a->ps[i] - a->recvr[i];
            if (inner_bulk) {
                if (a->bulk[i][0].ptr != nullptr && c[i] >= lo && c[i] < lo + a->sendl[i]) outer_forward = true;
                if (a->bulk[i][1].ptr != nullptr && c[i] >= hi - a->sendr[i] && c[i] < hi) outer_forward = true;
            }
            inner_bulk = inner_bulk && c[i] >= lo && c[i] < hi;
        }
    }
    // Rows [plain_lo, plain_hi) of a plain plane are shard rows that feed no
    // slab below L: their source and destination are affine in the row number.
    const bool plane_plain = in_x && gh < 0 && !outer_forward;
    const uint32_t left_m = a->bulk[M][0].ptr ? hlo + a->sendl[M] : hlo;
    const uint32_t right_m = a->bulk[M][1].ptr ? hhi - a->sendr[M] : hhi;
    const uint32_t plain_lo = padM > left_m ? padM : left_m;
    const uint32_t plain_hi = padM + xsM < right_m ? padM + xsM : right_m;
    const uint32_t wave_s = __builtin_amdgcn_readfirstlane(wave);
    constexpr uint32_t kRowsPerWave = RPI * kUnroll;

    // The chunk's rows split into [h_begin, lean_lo) and [lean_hi, h_end), which
    // take the general path, and the plain rows [lean_lo, lean_hi) between them.
    uint32_t lean_lo = h_end, lean_hi = h_end;
    if (plane_plain) {
        lean_lo = plain_lo < h_begin ? h_begin : (plain_lo < h_end ? plain_lo : h_end);
        lean_hi = plain_hi < lean_lo ? lean_lo : (plain_hi < h_end ? plain_hi : h_end);
    }

    // ---- lean path: groups of kRowsPerWave plain rows, dealt round-robin to the wavefronts ----
    for (uint32_t wh0 = lean_lo + wave_s * kRowsPerWave; wh0 < lean_hi; wh0 += kWavesPerBlock * kRowsPerWave) {
        {
            const T* sp[kUnroll];
            T* op[kUnroll];
            int64_t rowi[kUnroll];
            bool rv[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                uint32_t h = wh0 + u * RPI + sub;
                rv[u] = h < lean_hi;
                h = rv[u] ? h : lean_hi - 1;                       // rows past the range: loads stay valid, stores are masked
                sp[u] = xbase + (x_off + static_cast<int64_t>(h - padM) * xstrM - static_cast<int64_t>(padL));
                rowi[u] = plane_row0 + h;
                op[u] = obase + rowi[u] * static_cast<int64_t>(W);
            }
            const uint32_t x_hi = padL + xsL;
            const uint32_t nvx = xsL / EPV;
            const uint32_t run_end = padL + nvx * EPV;
            const uint32_t n_edge = padL + (W - run_end);
            const uint32_t n_task = n_edge + n_bl + n_br;
            // All loads of a step -- the vectors of the run and the single
            // elements -- are issued before its first store.
            for (uint32_t it = 0; it * LPR < nvx || it * LPR < n_task; ++it) {
                V val[kUnroll];
                const uint32_t vi = it * LPR + lc;
                const bool act = vi < nvx;
                const uint32_t wv = padL + (act ? vi : 0u) * EPV;
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) val[u] = *reinterpret_cast<const V*>(sp[u] + wv);

                const uint32_t e = it * LPR + lc;
                uint32_t w = 0;
                int k = 3;
                if (e < n_edge) {
                    w = e < padL ? e : run_end + (e - padL);
                    k = 0;
                } else if (e < n_edge + n_bl) {
                    w = glo + (e - n_edge);
                    k = 1;
                } else if (e < n_task) {
                    w = ghi - sr + (e - n_edge - n_bl);
                    k = 2;
                }
                const bool in_l = w < glo, in_r = w >= ghi;
                const bool in_m = !in_l && !in_r && w >= padL && w < x_hi;
                T ev[kUnroll];
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) {
                    const T* p = xbase;
                    p = in_m ? sp[u] + w : p;
                    p = in_l ? gl + rowi[u] * rl + w : p;
                    p = in_r ? gr + rowi[u] * rr + (w - ghi) : p;
                    const T t = *p;
                    ev[u] = (in_l || in_r || in_m) ? t : T(0);
                }
#pragma unroll
                for (int u = 0; u < kUnroll; ++u)
                    if (act && rv[u]) *reinterpret_cast<V*>(op[u] + wv) = val[u];
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) {
                    if (k == 0 && rv[u]) op[u][w] = ev[u];
                    if (k == 1 && rv[u]) bl[rowi[u] * sl + (w - glo)] = ev[u];
                    if (k == 2 && rv[u]) br[rowi[u] * sr + (w - (ghi - sr))] = ev[u];
                }
            }
        }
    }

    // ---- general path: the rows before and after the plain range, RPI rows per wavefront step ----
#pragma unroll 1
    for (int part = 0; part < 2; ++part) {
        const uint32_t r0 = part == 0 ? h_begin : lean_hi;
        const uint32_t r1 = part == 0 ? lean_lo : h_end;
#pragma unroll 1
        for (uint32_t wh0 = r0 + wave_s * RPI; wh0 < r1; wh0 += kWavesPerBlock * RPI) {
            const int g = 0;
            {
            // ---- per lane: the rows it serves and the single source of each ----
            const T* src[kGen];      // element w of the run is src[w]; nullptr = zeros
            uint32_t wlo[kGen], whi[kGen], hh[kGen];
            T* out[kGen];
#pragma unroll
            for (int u = 0; u < kGen; ++u) {
                uint32_t h = wh0 + (g * kGen + u) * RPI + sub;
                // Rows past the range are clamped onto its last row: they redo it
                // with identical values, which keeps every load unconditional.
                h = h < r1 ? h : r1 - 1;
                hh[u] = h;
                const uint32_t xh = h - padM;
                const T* p = nullptr;
                uint32_t lo = glo, hi = ghi;                          // zero rows and ghost rows span the bulk range of L
                if (in_x && xh < xsM) {
                    p = xbase + (x_off + static_cast<int64_t>(xh) * xstrM - static_cast<int64_t>(padL));
                    lo = padL;
                    hi = padL + xsL;
                }
                if (gh_ptr) {
                    p = reinterpret_cast<const T*>(gh_ptr) + (gh_off + static_cast<int64_t>(h) * gh_mstride);
                    lo = glo;
                    hi = ghi;
                }
                if (h < hlo && gm_ptr[0]) {
                    p = reinterpret_cast<const T*>(gm_ptr[0]) + (gm_off[0] + static_cast<int64_t>(h) * gm_mstride[0]);
                    lo = glo;
                    hi = ghi;
                }
                if (h >= hhi && gm_ptr[1]) {
                    p = reinterpret_cast<const T*>(gm_ptr[1]) + (gm_off[1] + static_cast<int64_t>(h) * gm_mstride[1]);
                    lo = glo;
                    hi = ghi;
                }
                src[u] = p;
                wlo[u] = lo;
                whi[u] = hi;
                out[u] = obase + (plane_row0 + h) * static_cast<int64_t>(W);
            }

            // ---- the runs, one vector per lane and step ----
            for (uint32_t v0 = 0; v0 < max_vecs; v0 += LPR) {
                V val[kGen];
                bool act[kGen];
#pragma unroll
                for (int u = 0; u < kGen; ++u) {
                    const uint32_t w = wlo[u] + (v0 + lc) * EPV;
                    act[u] = w + EPV <= whi[u];
                    const bool has = act[u] && src[u] != nullptr;
                    const T* p = has ? src[u] + w : xbase;            // idle lanes read a valid dummy address
                    const V t = *reinterpret_cast<const V*>(p);
                    V z;
                    __builtin_memset(&z, 0, sizeof(V));
                    val[u] = has ? t : z;
                }
#pragma unroll
                for (int u = 0; u < kGen; ++u) {
                    const uint32_t w = wlo[u] + (v0 + lc) * EPV;
                    if (act[u]) *reinterpret_cast<V*>(out[u] + w) = val[u];
                }
#pragma unroll
                for (int u = 0; u < kGen; ++u) {
                    const uint32_t w = wlo[u] + (v0 + lc) * EPV;
                    forward_below_L<T, V>(a, c, M, hh[u], w, act[u], val[u]);
                }
            }

            // ---- edge elements and the bulk strips of L, one element per lane ----
            for (uint32_t e0 = 0; e0 < max_edge; e0 += LPR) {
                T ev[kGen];
                uint32_t ew[kGen];
                int kind[kGen];                                    // 0 edge, 1 left strip, 2 right strip, 3 nothing
#pragma unroll
                for (int u = 0; u < kGen; ++u) {
                    const int64_t row = plane_row0 + hh[u];
                    const uint32_t run_end = wlo[u] + ((whi[u] - wlo[u]) / EPV) * EPV;   // first element after the vectors
                    const uint32_t n_edge = wlo[u] + (W - run_end);                      // [0,wlo) and [run_end,W)
                    const uint32_t e = e0 + lc;
                    uint32_t w = 0;
                    int k = 3;
                    if (e < n_edge) {
                        w = e < wlo[u] ? e : run_end + (e - wlo[u]);
                        k = 0;
                    } else if (e < n_edge + n_bl) {
                        w = glo + (e - n_edge);
                        k = 1;
                    } else if (e < n_edge + n_bl + n_br) {
                        w = ghi - sr + (e - n_edge - n_bl);
                        k = 2;
                    }
                    const bool in_l = w < glo, in_r = w >= ghi;
                    const bool in_m = !in_l && !in_r && src[u] != nullptr && w >= wlo[u] && w < whi[u];
                    const T* p = xbase;
                    p = in_m ? src[u] + w : p;
                    p = in_l ? gl + row * rl + w : p;
                    p = in_r ? gr + row * rr + (w - ghi) : p;
                    const T t = *p;
                    ev[u] = (in_l || in_r || in_m) ? t : T(0);
                    ew[u] = w;
                    kind[u] = k;
                }
#pragma unroll
                for (int u = 0; u < kGen; ++u) {
                    const int64_t row = plane_row0 + hh[u];
                    const uint32_t w = ew[u];
                    if (kind[u] == 0) out[u][w] = ev[u];
                    if (kind[u] == 1) bl[row * sl + (w - glo)] = ev[u];
                    if (kind[u] == 2) br[row * sr + (w - (ghi - sr))] = ev[u];
                    // an edge element inside the bulk range of L also belongs to the slabs below L
                    forward_below_L<T, T>(a, c, M, hh[u], w, kind[u] == 0 && w >= glo && w < ghi, ev[u]);
                }
            }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// 2- and 4-byte elements, whole-line stores.  Rows of the padded tensor are seldom
// whole 128-byte lines (130 floats in the convolution case), and writing them
// row by row costs a quarter of the store rate.  The padded tensor is
// contiguous, though, so it is also a plain run of elements: a wavefront takes
// kStage consecutive elements (4 or 2 KiB, aligned in memory), assembles them in
// its own LDS area and writes the area out with aligned 16-byte vectors, 1 KiB
// per instruction.
//
// Assembly: at most 64 padded rows meet a piece, so lane k classifies row k --
// all rows at once, in vector arithmetic: plane and row number, the plane's
// coordinates, whether it is a shard row (then where it starts in the shard)
// or all zeros, whether a bulk slab below L contains it.  The few rows that come
// from a ghost slab are then settled one by one in scalar code.  The result is
// one source pointer per row, held by lane k (a row is either a shard row, whose
// run is the shard's columns, or a ghost row, whose run is the bulk range of L:
// bit 0 of the pointer says which).  The area is cleared and filled by 16
// global -> LDS loads of one element per lane: lane l of load m owns element
// 64 m + l of the piece, takes its row's pointer from lane k with a cross-lane
// read and fetches from there (or stays idle: zeros), so consecutive lanes
// fetch consecutive addresses.
// The ghost columns of L (a few elements per row) are fetched one element per
// lane for all rows of the piece at once.  The bulk slabs are served from the
// assembled area.  Wavefronts do not share data: no barriers.
constexpr uint32_t kStage = 1024;            // elements per wavefront
constexpr uint32_t kFlatMinPitch = kStage / 32;   // shortest padded row: keeps a piece within 64 rows (and a load within 3)
constexpr uint32_t kArea = kStage;

typedef const __attribute__((address_space(1))) void* global_ptr;
typedef __attribute__((address_space(3))) void* lds_ptr;

// Offset of row h of plane c inside a slab whose dimensions 0..M are the tensor's.
template <int M>
__device__ inline int64_t slab_row_offset(SlabPtr b, const uint32_t (&c)[HD], uint32_t h) {
    int64_t off = b->base + static_cast<int64_t>(h) * b->stride[M];
#pragma unroll
    for (int j = 0; j < M; ++j) off += static_cast<int64_t>(c[j]) * b->stride[j];
    return off;
}

// T: uint32_t or uint16_t.  In LDS every element has a 4-byte slot (a 2-byte
// global -> LDS load writes its lane's slot, zero-extended); 2-byte elements are
// packed when the piece is read back.
template <int ND, typename T>
__global__ __launch_bounds__(kBlock) void halo_flat_kernel(const HaloArgs args_by_value) {
#if defined(__HIP_DEVICE_COMPILE__)
    ArgsPtr a = (ArgsPtr)__builtin_amdgcn_kernarg_segment_ptr();
#else
    ArgsPtr a = &args_by_value;
#endif
    constexpr int L = ND - 1, M = ND - 2;
    __shared__ __attribute__((aligned(16))) uint32_t stage_mem[kWavesPerBlock * kArea];
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t stage = blockIdx.x * kWavesPerBlock + wave;
    if (stage >= a->top.nstages) return;
    uint32_t* const area = stage_mem + wave * kArea;             // slot of element g0 of the padded tensor
    const uint32_t g0 = stage * kStage;
    const uint32_t total = a->top.total;
    const uint32_t n_el = total - g0 < kStage ? total - g0 : kStage;

#pragma unroll
    for (uint32_t j = 0; j < kStage / 256; ++j) *reinterpret_cast<uint4*>(area + j * 256 + lane * 4) = make_uint4(0, 0, 0, 0);

    const uint32_t W = a->top.W, H = a->top.H;
    const uint32_t glo = a->top.glo, ghi = a->top.ghi, hlo = a->top.hlo, hhi = a->top.hhi;
    const uint32_t padL = a->top.padL, xhiL = a->top.xhiL, padM = a->top.padM, xsM = a->top.xsM;
    const uint32_t m_l1 = a->top.m_l1, m_r0 = a->top.m_r0;
    const int64_t xstrM = a->top.xstrM;
    const T* const xbase = reinterpret_cast<const T*>(a->top.x) + a->top.x_off0;
    const uint32_t any_outer = a->top.any_outer;

    // First row of the piece: its global row number and the (non-positive)
    // position of its column 0 relative to the piece.
    const uint32_t row0 = __umulhi(g0, a->top.fdW_mul) >> a->top.fdW_shr;
    const int rowq0 = static_cast<int>(row0 * W) - static_cast<int>(g0);
    const uint32_t nrows = (n_el - rowq0 + W - 1) / W;           // rows that meet the piece, at most 64

    // ---- lane k: row k of the piece ----
    const uint32_t vrow = row0 + lane;
    const uint32_t vplane = H == 1 ? vrow : (__umulhi(vrow, a->top.fdH_mul) >> a->top.fdH_shr);
    const uint32_t vh = vrow - vplane * H;
    uint32_t v_inx = 1, v_ghost = 0, v_fwd = 0;
    int64_t v_xoff = static_cast<int64_t>(vh) * xstrM;
    {
        uint32_t vc[HD] = {0, 0, 0, 0, 0, 0};
        uint32_t r = vplane;
#pragma unroll
        for (int j = M - 1; j > 0; --j) {
            const uint32_t n = a->outer[j].ps;
            const uint32_t q = n == 1 ? r : (__umulhi(r, a->outer[j].fd_mul) >> a->outer[j].fd_shr);
            vc[j] = r - q * n;
            r = q;
        }
        if (M > 0) vc[0] = r;
        uint32_t inner = 1;
#pragma unroll
        for (int i = M - 1; i >= 0; --i) {                        // a slab of dimension i holds the bulk range of the dimensions above i
            const uint32_t ci = vc[i], lo = a->outer[i].lo, hi = a->outer[i].hi;
            const uint32_t inb = (ci >= lo) & (ci < hi);
            const uint32_t strip = ((ci >= lo) & (ci < a->outer[i].strip_l1)) | ((ci >= a->outer[i].strip_r0) & (ci < hi));
            v_fwd |= inner & strip;
            inner &= inb;
            v_ghost |= inb ^ 1u;
            const uint32_t xc = ci - a->outer[i].padl;           // wraps when left of the shard
            v_inx &= xc < a->outer[i].xs ? 1u : 0u;
            v_xoff += static_cast<int64_t>(xc) * a->outer[i].xstride;
        }
    }
    const bool v_valid = lane < nrows;
    const bool v_hbulk = vh >= hlo && vh < hhi;
    // rows of a ghost plane or a ghost strip of M may come from a slab: settled below, one by one
    const bool v_complex = v_valid && (v_ghost != 0 || !v_hbulk);
    const bool v_shard = v_inx != 0 && vh - padM < xsM;
    const bool v_forward = v_valid && ((vh >= hlo && vh < m_l1) || (vh >= m_r0 && vh < hhi) || (any_outer != 0 && v_fwd != 0 && v_hbulk));
    // Element w of the row is vp[w] for w in its run: the shard's columns, or
    // the bulk range of L when bit 0 is set (a row from a ghost slab).
    uint64_t vp = v_shard ? reinterpret_cast<uint64_t>(xbase + v_xoff) : 0;

    // ---- what a plane decides (scalar; used for the few rows handled one by one) ----
    uint32_t c[HD] = {0, 0, 0, 0, 0, 0};
    const T* gplane = nullptr;                                    // ghost slab of an outer dimension: row h at gplane + h * gstr
    int64_t gstr = 0;
    auto setup_plane = [&](uint32_t plane) {
        uint32_t r = plane;
#pragma unroll
        for (int j = M - 1; j > 0; --j) {
            const uint32_t n = a->outer[j].ps;
            const uint32_t q = n == 1 ? r : (__umulhi(r, a->outer[j].fd_mul) >> a->outer[j].fd_shr);
            c[j] = r - q * n;
            r = q;
        }
        if (M > 0) c[0] = r;
        int gh = -1, gside = 0;
#pragma unroll
        for (int j = 0; j < M; ++j) {
            const uint32_t left = c[j] < a->outer[j].lo, right = c[j] >= a->outer[j].hi;
            gh = (left | right) ? j : gh;
            gside = right ? 1 : (left ? 0 : gside);
        }
        gplane = nullptr;
        if (gh >= 0 && a->ghost[gh][gside].ptr != nullptr) {
            SlabPtr g = &a->ghost[gh][gside];
            gplane = reinterpret_cast<const T*>(g->ptr) + slab_row_offset<M>(g, c, 0);
            gstr = g->stride[M];
        }
    };
    auto plane_and_row = [&](uint32_t k, uint32_t& plane, uint32_t& h) {
        const uint32_t row = row0 + k;
        plane = H == 1 ? row : (__umulhi(row, a->top.fdH_mul) >> a->top.fdH_shr);
        h = row - plane * H;
    };

    // ---- rows that may come from a ghost slab (scalar, few) ----
    {
        uint64_t todo = __ballot(v_complex);
        uint32_t decoded = ~0u;
        const T* const gm0 = reinterpret_cast<const T*>(a->top.gm[0]);
        const T* const gm1 = reinterpret_cast<const T*>(a->top.gm[1]);
        while (todo != 0) {
            const uint32_t k = static_cast<uint32_t>(__builtin_ctzll(todo));
            todo &= todo - 1;
            uint32_t plane, h;
            plane_and_row(k, plane, h);
            if (decoded != plane) {
                setup_plane(plane);
                decoded = plane;
            }
            const T* p = nullptr;                                 // a ghost row spans the bulk range of L; without a slab it is zeros
            if (gplane != nullptr) p = gplane + static_cast<int64_t>(h) * gstr;
            if (h < hlo && gm0 != nullptr) p = gm0 + slab_row_offset<M>(&a->ghost[M][0], c, h);
            if (h >= hhi && gm1 != nullptr) p = gm1 + slab_row_offset<M>(&a->ghost[M][1], c, h);
            if (lane == k) vp = p != nullptr ? (reinterpret_cast<uint64_t>(p) | 1u) : 0;
        }
    }
    // The zeros must be in place before a global -> LDS load can land (those do
    // not queue behind LDS instructions).
    __builtin_amdgcn_s_waitcnt(0xC07F);                          // lgkmcnt(0)

    // ---- the runs: lane l of load m fetches element 64 m + l of the piece ----
    {
        const uint32_t t0 = lane - static_cast<uint32_t>(rowq0);  // position counted from column 0 of the first row
        uint32_t k = __umulhi(t0, a->top.fdW_mul) >> a->top.fdW_shr;
        uint32_t w = t0 - k * W;
#pragma unroll 4
        for (uint32_t m = 0; m < kStage / kWave; ++m) {
            const int from = static_cast<int>((k < kWave ? k : kWave - 1) * 4);
            const uint32_t plo = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(static_cast<uint32_t>(vp))));
            const uint32_t phi = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(static_cast<uint32_t>(vp >> 32))));
            const bool ghost_row = (plo & 1u) != 0;
            const uint32_t lo = ghost_row ? glo : padL, hi = ghost_row ? ghi : xhiL;
            const T* p = reinterpret_cast<const T*>(static_cast<uint64_t>(plo & ~1u) | (static_cast<uint64_t>(phi) << 32));
            if (m * kWave + lane < n_el && p != nullptr && w >= lo && w < hi) {
                if (sizeof(T) == 4)
                    __builtin_amdgcn_global_load_lds((global_ptr)(p + w), (lds_ptr)(area + m * kWave), 4, 0, 0);
                else
                    __builtin_amdgcn_global_load_lds((global_ptr)(p + w), (lds_ptr)(area + m * kWave), 2, 0, 0);
            }
            w += kWave;
#pragma unroll
            for (int t = 0; t < 2; ++t) {                         // rows hold at least 32 elements
                const bool wrap = w >= W;
                w = wrap ? w - W : w;
                k = wrap ? k + 1 : k;
            }
        }
    }

    // ---- ghost columns of L: one element per lane, all rows of the piece ----
    const uint32_t n_ghost = a->top.n_ghost;
    if (n_ghost != 0) {
        const T* gl = reinterpret_cast<const T*>(a->top.gl);
        const T* gr = reinterpret_cast<const T*>(a->top.gr);
        const uint32_t rl = glo, rr = W - ghi;
        for (uint32_t e0 = 0; e0 < nrows * n_ghost; e0 += kWave) {
            const uint32_t e = e0 + lane;
            const uint32_t k = n_ghost == 1 ? e : (__umulhi(e, a->top.fdg_mul) >> a->top.fdg_shr);
            const uint32_t i = e - k * n_ghost;
            const uint32_t w = i < rl ? i : ghi + (i - rl);
            const uint32_t q = static_cast<uint32_t>(rowq0 + static_cast<int>(k * W + w));
            const bool on = e < nrows * n_ghost && q < n_el;
            const int64_t row = static_cast<int64_t>(row0) + k;
            const T* p = i < rl ? gl + row * rl + w : gr + row * rr + (w - ghi);
            T v = 0;
            if (on) v = *p;
            if (on) area[q] = v;
        }
    }

    __builtin_amdgcn_s_waitcnt(0x0070);                          // every load has landed, every LDS write is done
    asm volatile("" ::: "memory");

    // ---- the piece leaves in whole lines: 16 bytes per lane, 1 KiB per instruction ----
    {
        T* const out = reinterpret_cast<T*>(a->top.xpad) + g0;
        constexpr uint32_t EPV = 16 / sizeof(T);                 // elements per store
        typedef typename VecType<uint32_t, 4>::type V;           // the padded tensor is not read again here: streaming store
#pragma unroll
        for (uint32_t j = 0; j < kStage / (kWave * EPV); ++j) {
            const uint32_t o = (j * kWave + lane) * EPV;
            uint32_t e[EPV];
#pragma unroll
            for (uint32_t t = 0; t < EPV; t += 4) {
                const uint4 v = *reinterpret_cast<const uint4*>(area + o + t);
                e[t] = v.x, e[t + 1] = v.y, e[t + 2] = v.z, e[t + 3] = v.w;
            }
            if (o + EPV <= n_el) {
                V nv;
                if (sizeof(T) == 4) {
#pragma unroll
                    for (uint32_t t = 0; t < 4; ++t) nv[t] = e[t];
                } else {
#pragma unroll
                    for (uint32_t t = 0; t < 4; ++t) nv[t] = e[(2 * t) % EPV] | (e[(2 * t + 1) % EPV] << 16);
                }
                __builtin_nontemporal_store(nv, reinterpret_cast<V*>(out + o));
            } else {
#pragma unroll
                for (uint32_t t = 0; t < EPV; ++t)
                    if (o + t < n_el) out[o + t] = static_cast<T>(e[t]);
            }
        }
    }

    // ---- bulk strips of L: one element per lane ----
    const uint32_t n_bl = a->top.n_bl, n_br = a->top.n_br, n_strip = n_bl + n_br;
    if (n_strip != 0) {
        T* bl = reinterpret_cast<T*>(a->bulk[L][0].ptr);
        T* br = reinterpret_cast<T*>(a->bulk[L][1].ptr);
        const uint32_t sl = a->top.sl, sr = a->top.sr;
        for (uint32_t e0 = 0; e0 < nrows * n_strip; e0 += kWave) {
            const uint32_t e = e0 + lane;
            const uint32_t k = n_strip == 1 ? e : (__umulhi(e, a->top.fds_mul) >> a->top.fds_shr);
            const uint32_t i = e - k * n_strip;
            const uint32_t w = i < n_bl ? glo + i : ghi - sr + (i - n_bl);
            const uint32_t q = static_cast<uint32_t>(rowq0 + static_cast<int>(k * W + w));
            const int64_t row = static_cast<int64_t>(row0) + k;
            if (e < nrows * n_strip && q < n_el) {
                const T v = static_cast<T>(area[q]);
                if (i < n_bl)
                    bl[row * sl + (w - glo)] = v;
                else
                    br[row * sr + (w - (ghi - sr))] = v;
            }
        }
    }

    // ---- bulk slabs below L: the bulk range of L of the rows they contain (scalar, few) ----
    {
        uint64_t todo = __ballot(v_forward);
        uint32_t decoded = ~0u;
        while (todo != 0) {
            const uint32_t k = static_cast<uint32_t>(__builtin_ctzll(todo));
            todo &= todo - 1;
            uint32_t plane, h;
            plane_and_row(k, plane, h);
            if (decoded != plane) {
                setup_plane(plane);
                decoded = plane;
            }
            const int rowq = rowq0 + static_cast<int>(k * W);
            auto copy_row = [&](SlabPtr b) {
                T* const dst = reinterpret_cast<T*>(b->ptr) + slab_row_offset<M>(b, c, h);
                // the part of [glo, ghi) inside the piece, in 64-element steps counted from glo
                const int before = -rowq - static_cast<int>(glo);
                uint32_t w0 = glo + (before > 0 ? (static_cast<uint32_t>(before) >> 6) << 6 : 0u);
                for (; w0 < ghi && rowq + static_cast<int>(w0) < static_cast<int>(n_el); w0 += kWave) {
                    const uint32_t w = w0 + lane;
                    const uint32_t q = static_cast<uint32_t>(rowq + static_cast<int>(w));
                    if (w < ghi && q < n_el) dst[w] = static_cast<T>(area[q]);
                }
            };
            // dimension M: the row's own strips; outer dimensions are unrestricted
            if (h >= hlo && h < m_l1) copy_row(&a->bulk[M][0]);
            if (h >= m_r0 && h < hhi) copy_row(&a->bulk[M][1]);
            // outer dimension i: decided by the plane, and the row must be in the bulk range of M
            if (any_outer != 0 && h >= hlo && h < hhi) {
                bool inner_bulk = true;                           // outer dimensions above i inside their bulk range
#pragma unroll
                for (int i = M - 1; i >= 0; --i) {
                    const uint32_t blo = a->outer[i].lo, bhi = a->outer[i].hi;
                    if (inner_bulk) {
                        if (c[i] >= blo && c[i] < a->outer[i].strip_l1) copy_row(&a->bulk[i][0]);
                        if (c[i] >= a->outer[i].strip_r0 && c[i] < bhi) copy_row(&a->bulk[i][1]);
                    }
                    inner_bulk = inner_bulk && c[i] >= blo && c[i] < bhi;
                }
            }
        }
    }
}

// Rows at least this long (shard elements) take halo_flat_kernel when the
// caller leaves the choice to the library.
constexpr int64_t kFlatMinRow = 32;

template <typename T>
int launch_halo(const HaloArgs& a, uint32_t lpr, hipStream_t s) {
    const uint32_t blocks = a.nplanes * a.row_chunks;
    if (lpr <= 16)
        hipLaunchKernelGGL((halo_pad_kernel<T, 16>), dim3(blocks), dim3(kBlock), 0, s, a);
    else if (lpr <= 32)
        hipLaunchKernelGGL((halo_pad_kernel<T, 32>), dim3(blocks), dim3(kBlock), 0, s, a);
    else
        hipLaunchKernelGGL((halo_pad_kernel<T, 64>), dim3(blocks), dim3(kBlock), 0, s, a);
    return check_launch("halo_pad_kernel");
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_halo_pad_exchange(const void* x, void* xpad, const int64_t* x_shape, int ndim, int elem_size,
                                     const int64_t* pad, const int64_t* recv, const int64_t* send,
                                     const void* const* ghost_bufs, void* const* bulk_bufs, int kernel, void* stream) {
    using namespace ddl;
    if (ndim < 1 || ndim > DDL_MAX_DIMS) return fail(DDL_E_DIMS, "halo: ndim %d outside [1,%d]", ndim, DDL_MAX_DIMS);
    if (kernel != DDL_HALO_AUTO && kernel != DDL_HALO_ROWS && kernel != DDL_HALO_LINES)
        return fail(DDL_E_ARG, "halo: kernel choice %d is not DDL_HALO_AUTO, _ROWS or _LINES", kernel);
    // shortest shard row the whole-line kernel takes under this choice
    const int64_t flat_min_row = kernel == DDL_HALO_ROWS ? INT64_MAX : kernel == DDL_HALO_LINES ? 1 : kFlatMinRow;
    if (!x_shape || !pad || !recv || !send) return fail(DDL_E_ARG, "halo: null geometry argument");
    if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8)
        return fail(DDL_E_ARG, "halo: element size %d not in {1,2,4,8}", elem_size);

    // Leading dimensions that carry no padding and no exchange are folded into
    // one (batch x channel in the convolution case); a 1-D tensor gets a unit
    // row dimension in front.
    int64_t xs[DDL_MAX_DIMS + 1], pl[DDL_MAX_DIMS + 1], pr[DDL_MAX_DIMS + 1], rl[DDL_MAX_DIMS + 1], rr[DDL_MAX_DIMS + 1],
        sl[DDL_MAX_DIMS + 1], sr[DDL_MAX_DIMS + 1];
    int src_dim[DDL_MAX_DIMS + 1];
    int nd = 0;
    if (ndim == 1) {
        xs[0] = 1;
        pl[0] = pr[0] = rl[0] = rr[0] = sl[0] = sr[0] = 0;
        src_dim[0] = -1;
        nd = 1;
    }
    for (int d = 0; d < ndim; ++d) {
        const int64_t v[7] = {x_shape[d], pad[2 * d], pad[2 * d + 1], recv[2 * d], recv[2 * d + 1], send[2 * d], send[2 * d + 1]};
        for (int q = 0; q < 7; ++q)
            if (v[q] < 0) return fail(DDL_E_ARG, "halo: negative geometry value in dim %d", d);
        const bool plain = v[1] == 0 && v[2] == 0 && v[3] == 0 && v[4] == 0 && v[5] == 0 && v[6] == 0;
        const bool prev_plain = nd > 0 && src_dim[nd - 1] >= 0 && pl[nd - 1] == 0 && pr[nd - 1] == 0 && rl[nd - 1] == 0 &&
                                rr[nd - 1] == 0 && sl[nd - 1] == 0 && sr[nd - 1] == 0;
        if (plain && prev_plain && d < ndim - 2) {
            xs[nd - 1] *= v[0];
            continue;
        }
        xs[nd] = v[0]; pl[nd] = v[1]; pr[nd] = v[2]; rl[nd] = v[3]; rr[nd] = v[4]; sl[nd] = v[5]; sr[nd] = v[6];
        src_dim[nd] = d;
        ++nd;
    }
    if (nd > HD) return fail(DDL_E_UNSUPP, "halo: %d dimensions left after folding, at most %d supported", nd, HD);
    // 8-byte elements are moved as pairs of 4-byte ones: the same tensor and the
    // same slabs with every extent of the last dimension doubled.
    int es = elem_size;
    if (elem_size == 8 && aligned_to(xpad, 16)) {
        const int l = nd - 1;
        xs[l] *= 2; pl[l] *= 2; pr[l] *= 2; rl[l] *= 2; rr[l] *= 2; sl[l] *= 2; sr[l] *= 2;
        es = 4;
    }

    HaloArgs a{};
    a.nd = nd;
    a.x = static_cast<const char*>(x);
    a.xpad = static_cast<char*>(xpad);
    const int L = nd - 1, M = nd - 2;
    int64_t ps[HD];
    int64_t total = 1, nplanes = 1;
    for (int j = 0; j < nd; ++j) {
        ps[j] = xs[j] + pl[j] + pr[j];
        if (rl[j] + sl[j] > ps[j] - rr[j] || rr[j] + sr[j] > ps[j] - rl[j])
            return fail(DDL_E_SHAPE, "halo: ghost+bulk widths exceed the padded extent %lld in dim %d", (long long)ps[j], src_dim[j]);
        if (rl[j] > pl[j] || rr[j] > pr[j])
            return fail(DDL_E_SHAPE, "halo: ghost width larger than the padding in dim %d", src_dim[j]);
        if (ps[j] >= (1ll << 31)) return fail(DDL_E_UNSUPP, "halo: padded extent too large");
        total *= ps[j];
        if (j < M) nplanes *= ps[j];
    }
    if (total == 0) return 0;
    if (!xpad) return fail(DDL_E_ARG, "halo: null output");
    int64_t xvol = 1;
    for (int j = 0; j < nd; ++j) xvol *= xs[j];
    if (xvol > 0 && !x) return fail(DDL_E_ARG, "halo: null input");
    if (!aligned_to(xpad, elem_size) || !aligned_to(x, elem_size)) return fail(DDL_E_ALIGN, "halo: tensor misaligned");
    if (xvol == 0) a.x = a.xpad;   // only ever used as a readable dummy address
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
    for (int i = 0; i < nd; ++i) {
        for (int s = 0; s < 2; ++s) {
            const int d = src_dim[i];
            const void* gb = (ghost_bufs && d >= 0) ? ghost_bufs[2 * d + s] : nullptr;
            void* bb = (bulk_bufs && d >= 0) ? bulk_bufs[2 * d + s] : nullptr;
            const int64_t gw = s == 0 ? rl[i] : rr[i];
            const int64_t bw = s == 0 ? sl[i] : sr[i];
            if (gw > 0 && !gb) return fail(DDL_E_ARG, "halo: ghost width %lld in dim %d side %d but no slab given", (long long)gw, d, s);
            if (!aligned_to(gb, elem_size) || !aligned_to(bb, elem_size)) return fail(DDL_E_ALIGN, "halo: slab misaligned");
            // Slab extents: j < i full, j == i the strip, j > i the bulk range.
            for (int kind = 0; kind < 2; ++kind) {
                Slab& sb = kind == 0 ? a.ghost[i][s] : a.bulk[i][s];
                const int64_t width = kind == 0 ? gw : bw;
                sb.ptr = nullptr;
                if (width > 0) sb.ptr = kind == 0 ? const_cast<char*>(static_cast<const char*>(gb)) : static_cast<char*>(bb);
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
                for (int j = 0; j < L; ++j) sb.stride[j] = str[j];
                sb.base = base;
            }
        }
    }
    // Work split: LPR lanes per row (a power of two covering the longest run in
    // vectors, at most a wavefront); the rows of a plane are cut into about
    // 64-row chunks, one workgroup each.
    const int epv = es >= 4 ? 16 / es : 1;
    const int64_t bulk_l = ps[L] - rl[L] - rr[L];
    const int64_t longest = bulk_l > xs[L] ? bulk_l : xs[L];
    const int64_t shortest = bulk_l < xs[L] ? bulk_l : xs[L];
    a.max_vecs = static_cast<uint32_t>(longest / epv);
    // edge tasks: what whole vectors of the shortest run leave uncovered, plus the bulk strips of L
    a.max_edge = static_cast<uint32_t>(ps[L] - (shortest / epv) * epv + sl[L] + sr[L]);
    uint32_t lpr = 16;
    while (lpr < 64 && lpr < a.max_vecs) lpr *= 2;
    const int64_t rows_per_pass = (64 / lpr) * kWavesPerBlock;
    const int64_t target_rows = 64;
    int64_t chunks = (ps[M] + target_rows / 2) / target_rows;
    if (chunks < 1) chunks = 1;
    int64_t rpb = (ps[M] + chunks - 1) / chunks;
    rpb = ((rpb + rows_per_pass - 1) / rows_per_pass) * rows_per_pass;
    a.rows_per_block = static_cast<uint32_t>(rpb);
    a.row_chunks = static_cast<uint32_t>((ps[M] + rpb - 1) / rpb);
    if (nplanes * static_cast<int64_t>(a.row_chunks) >= (1ll << 31)) return fail(DDL_E_UNSUPP, "halo: too many workgroups");
    a.nplanes = static_cast<uint32_t>(nplanes);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if ((es == 4 || es == 2) && total < (1ll << 31) && xs[L] >= flat_min_row && ps[L] >= kFlatMinPitch && aligned_to(xpad, 16)) {
        const int64_t nstages = (total + kStage - 1) / kStage;
        FlatTop& t = a.top;
        t.x = a.x;
        t.xpad = a.xpad;
        t.gm[0] = a.ghost[M][0].ptr;
        t.gm[1] = a.ghost[M][1].ptr;
        t.gl = a.ghost[L][0].ptr;
        t.gr = a.ghost[L][1].ptr;
        t.xstrM = a.xstride[M];
        t.x_off0 = -(pl[M] * a.xstride[M] + pl[L]);
        t.total = static_cast<uint32_t>(total);
        t.nstages = static_cast<uint32_t>(nstages);
        t.W = a.ps[L];
        t.H = a.ps[M];
        t.fdW_mul = a.fd[L].mul;
        t.fdW_shr = a.fd[L].shr;
        t.fdH_mul = a.fd[M].mul;
        t.fdH_shr = a.fd[M].shr;
        t.glo = a.recvl[L];
        t.ghi = a.ps[L] - a.recvr[L];
        t.hlo = a.recvl[M];
        t.hhi = a.ps[M] - a.recvr[M];
        t.padL = a.padl[L];
        t.xhiL = a.padl[L] + a.xs[L];
        t.padM = a.padl[M];
        t.xsM = a.xs[M];
        t.m_l1 = a.bulk[M][0].ptr ? t.hlo + a.sendl[M] : t.hlo;
        t.m_r0 = a.bulk[M][1].ptr ? t.hhi - a.sendr[M] : t.hhi;
        t.n_ghost = a.recvl[L] + a.recvr[L];
        t.n_bl = a.bulk[L][0].ptr ? a.sendl[L] : 0u;
        t.n_br = a.bulk[L][1].ptr ? a.sendr[L] : 0u;
        t.sl = a.sendl[L];
        t.sr = a.sendr[L];
        const FastDiv fdg = make_fastdiv(t.n_ghost > 0 ? t.n_ghost : 1), fds = make_fastdiv(t.n_bl + t.n_br > 0 ? t.n_bl + t.n_br : 1);
        t.fdg_mul = fdg.mul;
        t.fdg_shr = fdg.shr;
        t.fds_mul = fds.mul;
        t.fds_shr = fds.shr;
        t.any_outer = 0;
        for (int j = 0; j < M; ++j) {
            FlatDim& o = a.outer[j];
            o.ps = a.ps[j];
            o.fd_mul = a.fd[j].mul;
            o.fd_shr = a.fd[j].shr;
            o.lo = a.recvl[j];
            o.hi = a.ps[j] - a.recvr[j];
            o.padl = a.padl[j];
            o.xs = a.xs[j];
            o.strip_l1 = a.bulk[j][0].ptr ? o.lo + a.sendl[j] : o.lo;
            o.strip_r0 = a.bulk[j][1].ptr ? o.hi - a.sendr[j] : o.hi;
            o.xstride = a.xstride[j];
            if (a.bulk[j][0].ptr || a.bulk[j][1].ptr) t.any_outer = 1;
        }
        const dim3 grid(static_cast<uint32_t>((nstages + kWavesPerBlock - 1) / kWavesPerBlock));
        if (es == 4) {
            switch (nd) {
                case 2: hipLaunchKernelGGL((halo_flat_kernel<2, uint32_t>), grid, dim3(kBlock), 0, s, a); break;
                case 3: hipLaunchKernelGGL((halo_flat_kernel<3, uint32_t>), grid, dim3(kBlock), 0, s, a); break;
                case 4: hipLaunchKernelGGL((halo_flat_kernel<4, uint32_t>), grid, dim3(kBlock), 0, s, a); break;
                case 5: hipLaunchKernelGGL((halo_flat_kernel<5, uint32_t>), grid, dim3(kBlock), 0, s, a); break;
                default: hipLaunchKernelGGL((halo_flat_kernel<6, uint32_t>), grid, dim3(kBlock), 0, s, a); break;
            }
        } else {
            switch (nd) {
                case 2: hipLaunchKernelGGL((halo_flat_kernel<2, uint16_t>), grid, dim3(kBlock), 0, s, a); break;
                case 3: hipLaunchKernelGGL((halo_flat_kernel<3, uint16_t>), grid, dim3(kBlock), 0, s, a); break;
                case 4: hipLaunchKernelGGL((halo_flat_kernel<4, uint16_t>), grid, dim3(kBlock), 0, s, a); break;
                case 5: hipLaunchKernelGGL((halo_flat_kernel<5, uint16_t>), grid, dim3(kBlock), 0, s, a); break;
                default: hipLaunchKernelGGL((halo_flat_kernel<6, uint16_t>), grid, dim3(kBlock), 0, s, a); break;
            }
        }
        return check_launch("halo_flat_kernel");
    }
    switch (es) {
        case 1: return launch_halo<uint8_t>(a, lpr, s);
        case 2: return launch_halo<uint16_t>(a, lpr, s);
        case 4: return launch_halo<uint32_t>(a, lpr, s);
        default: return launch_halo<uint64_t>(a, lpr, s);
    }
}
