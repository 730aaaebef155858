// DistributedLinear shard GEMM in fp32, tiled like the 16-bit kernel:
// y[M,N] = a[M,K] . b[N,K]^T + bias[N] on v_mfma_f32_32x32x2_f32 (reference:
// nn/linear.py:103, nn/linear_ag.py:486 -- torch.nn.functional.linear in the
// default dtype of the reference's layers), and the two products of its adjoint,
// whose operands are contiguous along their rows instead of along k.
//
//   workgroup  512 threads = 8 wavefronts, tile 256(m) x 256(n) (2 x 4 wavefronts
//              of 128 x 64 = 4 x 2 MFMA tiles of 32 x 32, 128 accumulators per
//              lane) or 256 x 192 (4 x 2 wavefronts of 64 x 96); the host splits
//              the columns between the two kinds so that both fill whole rounds
//              of one workgroup per CU, and workgroup b computes wide tile b,
//              then narrow tile b
//   LDS        the ring of five 32 KiB operand tiles of the 16-bit kernel; a
//              k-tile is 32 floats (128 B per row).  Operand contiguous along
//              k: rows of 128 B, 16-byte chunk index XOR-ed with (row >> 1) & 7;
//              lane (r = lane % 32, h = lane / 32) reads chunk 2 g + h of row r
//              with one ds_read_b128 and feeds its four floats to the four MFMAs
//              of k-group g (any assignment of k to lanes and steps is valid as
//              long as both operands use the same one: here k = 8 g + 4 h + e in
//              step e).  Operand contiguous along its rows: kept as it lies in
//              memory, panels of 32 rows x 32 k-lines of 128 B; lane (r, h)
//              reads element r of k-line 8 g + 4 h + e with a ds_read_b32.  Lines
//              k and k + 4 would start on the same bank, so the lines 4..7 of
//              every eight are stored with neighbours swapped (line position
//              k ^ ((k >> 2) & 1)): the two halves of the wavefront then read
//              banks 0..31 and 32..63
//   global     tiles go from global memory straight into LDS, one whole
//              128-byte line per eight lanes (see gemm_tiles.h)
//   schedule   per k-tile four k-groups of 8 x 4 MFMAs (wide tile); the fragments
//              of the next k-group are read behind the first odd MFMAs of the
//              current one.  W(t+2) is requested in k-group 0, X(t+2) in k-group
//              3; between k-groups 2 and 3 each wavefront waits for its own
//              requests of tile t+1 and for its LDS reads, then one barrier:
//              tile t+1 is readable, tile t's slots are free.  A k-tile is 8192
//              MFMA cycles per wavefront, so operand requests have microseconds
//              of lead and the barrier is a fraction of a percent
//   epilogue   bias add in registers, 16-byte stores (a lane holds four
//              consecutive n of one output row per 8 x 32 piece of a tile)
#include "gemm_tiles.h"
#include <type_traits>

namespace ddl {
namespace {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int BK = kRowBytes / 4;   // floats of a k-tile
constexpr int kGroups = 4;          // k-groups of 8 floats per k-tile

typedef PartOf<float> Part;
typedef PartsOf<float> Parts;

// acc += a . b (32 x 32 x 2, fp32).  Assembly so that the accumulators live in
// the accumulation registers; the kernel pads the distance between the last
// MFMA and the first other read of acc itself.
__device__ inline void mfma_32x32x2(floatx16& acc, float a, float b) {
    asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// NWM x NWN wavefronts, each owning TM x TN sub-tiles of 32 x 32.
template <bool XT, bool WT, int NWM, int NWN, int TM, int TN>
__device__ __forceinline__ void gemm32_tile(const Part& part, int tile_id, char* lds) {
    static_assert(NWM * NWN == 8, "eight wavefronts per workgroup");
    const float* __restrict__ x = part.x;
    const float* __restrict__ w = part.w;
    const float* __restrict__ bias = part.bias;
    float* __restrict__ y = part.y;
    const int64_t M = part.M, N = part.N, K = part.K, ldx = part.ldx, ldw = part.ldw, ldy = part.ldy;

    int tm, tn;
    tile_of_workgroup(tile_id, part.tiles_m, part.tiles_n, tm, tn);

    constexpr int BM = 32 * NWM * TM, BN = 32 * NWN * TN;
    static_assert(BM <= kMaxTileRows && BN <= kMaxTileRows, "operand tile larger than a ring slot");
    const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int NW = NWM * NWN;
    constexpr int JW_W = BN / 8 / NW, JW_X = BM / 8 / NW;   // request instructions (1 KiB each) per wavefront and operand tile
    static_assert(JW_W * 8 * NW == BN && JW_X * 8 * NW == BM, "tile rows do not divide among the wavefronts");
    const int wm = (wave % NWM) * (TM * 32), wn = (wave / NWM) * (TN * 32);   // wavefront origin inside the tile
    const int l32 = lane & 31, kh = lane >> 5;

    floatx16 acc[TN][TM];   // [n sub-tile][m sub-tile]
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

    // Global -> LDS requests of this lane: a 32-bit byte offset from the tile's
    // first row (or first column, for an operand contiguous along its rows).
    // Request instruction q = J wave + j of a tile fills LDS bytes q KiB .. + 1023.
    //   along k:     rows 8 q .. + 7, lane l on row l / 8, physical chunk l % 8
    //   along rows:  panel q / 4, k-lines 8 (q % 4) .. + 7; lane l sits on line
    //                position l / 8 and fetches k-line p ^ ((p >> 2) & 1), rows
    //                4 (l % 8) .. + 3 of the panel
    const char* const base_w = reinterpret_cast<const char*>(WT ? w + n0 : w + n0 * ldw);
    const char* const base_x = reinterpret_cast<const char*>(XT ? x + m0 : x + m0 * ldx);
    const u32x4 buf_w = raw_buffer(base_w), buf_x = raw_buffer(base_x);
    const int step_w = WT ? static_cast<int>(ldw) * (BK * 4) : BK * 4;   // bytes from one k-tile to the next
    const int step_x = XT ? static_cast<int>(ldx) * (BK * 4) : BK * 4;
    int off_gw[JW_W], off_gx[JW_X];
    auto line_of = [&](int q) {   // k-line of this lane in request q of an operand read along its rows
        const int p = lane >> 3;
        return 8 * (q & 3) + (p ^ ((p >> 2) & 1));
    };
    {
        auto lane_offset = [&](bool transposed, int q, int64_t origin, int64_t rows, int64_t ld) -> int {
            if (!transposed) {
                const int row = q * 8 + (lane >> 3);
                const int ck = ((lane & 7) ^ ((row >> 1) & 7)) * 4;   // first k of this lane's chunk inside a k-tile
                const int64_t rr = origin + row < rows ? row : rows - 1 - origin;
                return static_cast<int>((rr * ld + ck) * 4);
            }
            int col = (q >> 2) * 32 + (lane & 7) * 4;   // first tile row of this lane's chunk
            if (origin + col >= rows) col = 0;
            return static_cast<int>((line_of(q) * ld + col) * 4);
        };
#pragma unroll
        for (int j = 0; j < JW_W; ++j) off_gw[j] = lane_offset(WT, JW_W * wave + j, n0, N, ldw);
#pragma unroll
        for (int j = 0; j < JW_X; ++j) off_gx[j] = lane_offset(XT, JW_X * wave + j, m0, M, ldx);
    }

    const int ktiles = static_cast<int>((K + BK - 1) / BK);
    const int full_tiles = static_cast<int>(K / BK);   // tiles [full_tiles, ktiles) straddle K

    auto request_part = [&](u32x4 buf, const auto& off, int step, int t, int unit_off, int j) {
        constexpr int J = sizeof(off) / sizeof(int);
        dma16(buf, off[j], t * step, lds + unit_off + (J * wave + j) * 1024);
    };
    // A whole operand tile.  One that straddles K goes through registers so
    // that the elements past K can be written as zeros.
    auto request_unit = [&](auto transposed, u32x4 buf, const char* base, const auto& off, int step, int t, int unit_off) {
        constexpr int J = sizeof(off) / sizeof(int);
        constexpr bool T = decltype(transposed)::value;
        if (t < full_tiles) {
#pragma unroll
            for (int j = 0; j < J; ++j) request_part(buf, off, step, t, unit_off, j);
        } else {
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const int q = J * wave + j;
                bool inside;
                if (T) {
                    inside = static_cast<int64_t>(t) * BK + line_of(q) < K;
                } else {
                    const int row = q * 8 + (lane >> 3);
                    const int ck = ((lane & 7) ^ ((row >> 1) & 7)) * 4;
                    inside = static_cast<int64_t>(t) * BK + ck < K;
                }
                uint4 v = make_uint4(0, 0, 0, 0);
                if (inside) v = *reinterpret_cast<const uint4*>(base + off[j] + static_cast<int64_t>(t) * step);
                *reinterpret_cast<uint4*>(lds + unit_off + q * 1024 + lane * 16) = v;
            }
        }
    };
    const std::integral_constant<bool, WT> w_kind{};
    const std::integral_constant<bool, XT> x_kind{};

    // Fragment addresses.  Along k: row (sub-tile origin + l32), logical chunk
    // 2 g + kh; sub-tile origins are multiples of 32, so the swizzle term is
    // (l32 >> 1) & 7.  Along rows: panel of the sub-tile, element l32 of the line
    // at position p(k), k = 8 g + 4 kh + e; p(k) = k ^ 1 for kh = 1, k for kh = 0.
    int sw_off[kGroups];
#pragma unroll
    for (int g = 0; g < kGroups; ++g) sw_off[g] = ((2 * g + kh) ^ ((l32 >> 1) & 7)) << 4;
    const int row_off = l32 * kRowBytes;
    const int tr_off = l32 * 4 + kh * (4 * kRowBytes);
    auto read_piece = [&](auto transposed, const char* tile, int sub, int g) -> floatx4 {   // 32-row block `sub` of the tile, k-group g
        floatx4 out;
        if (decltype(transposed)::value) {
            const char* p = tile + sub * 4096 + g * (8 * kRowBytes) + tr_off;
#pragma unroll
            for (int e = 0; e < 4; ++e) out[e] = *reinterpret_cast<const float*>(p + (e ^ kh) * kRowBytes);
        } else {
            out = *reinterpret_cast<const floatx4*>(tile + sub * (32 * kRowBytes) + row_off + sw_off[g]);
        }
        return out;
    };
    const int sub_w = (wave / NWM) * TN, sub_x = (wave % NWM) * TM;

    constexpr int NMFMA = 4 * TN * TM, NREAD = TN + TM;
    static_assert(2 * NREAD - 1 < NMFMA, "a k-group has too few MFMAs to hide its fragment reads");
    static_assert(2 * JW_W <= NMFMA && 2 * JW_X <= NMFMA, "request slots must fall on even MFMAs");
    floatx4 fa[2][TN], fb[2][TM];
    auto read_frag = [&](const char* wt, const char* xt, int g, floatx4 (&na)[TN], floatx4 (&nb)[TM], int r) {
        if (r < TN)
            na[r] = read_piece(w_kind, wt, sub_w + r, g);
        else
            nb[r - TN] = read_piece(x_kind, xt, sub_x + r - TN, g);
    };

    // One k-group: NMFMA MFMAs on fa[cur] / fb[cur]; the pieces of k-group
    // `g_next` of (wt, xt) are read into the other set; `request(j)` issues request
    // instruction j of `nreq` behind MFMA 2 j.
    auto k_group = [&](int cur, const char* wt, const char* xt, int g_next, int nreq, auto request) {
#pragma unroll
        for (int q = 0; q < NMFMA; ++q) {
            const int e = q / (TN * TM), a = (q / TM) % TN, b = q % TM;
            mfma_32x32x2(acc[a][b], fa[cur][a][e], fb[cur][b][e]);
            if ((q & 1) && (q >> 1) < NREAD) read_frag(wt, xt, g_next, fa[cur ^ 1], fb[cur ^ 1], q >> 1);
            if (!(q & 1) && (q >> 1) < nreq) request(q >> 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    auto unit_off = [](int slot) { return (slot >= kUnits ? slot - kUnits : slot) * kUnitBytes; };
    int s0 = 0;   // ring slot of W(t); X(t), W(t+1), X(t+1), W(t+2) follow
    // One k-tile.  On entry the fragments of (t, k-group 0) are in set 0 or on
    // their way, W(t+1) and X(t+1) have been requested.  STEADY: tile t+2 exists
    // and is a full tile.  `slot`: the running s0 or a compile-time constant (the
    // steady loop is unrolled over the five positions of the ring, so that LDS
    // addresses are immediates).
    auto k_tile = [&](int t, auto steady, auto slot) {
        constexpr bool STEADY = decltype(steady)::value;
        const int s = slot;
        const char* wt = lds + unit_off(s);
        const char* xt = lds + unit_off(s + 1);
        const char* wn1 = lds + unit_off(s + 2);
        const char* xn1 = lds + unit_off(s + 3);
        const int w2_off = unit_off(s + 4);   // slot of X(t-1), free since the barrier of tile t-1
        const int x2_off = unit_off(s);       // slot of W(t), free after this tile's barrier
        if (!STEADY && t + 2 < ktiles) request_unit(w_kind, buf_w, base_w, off_gw, step_w, t + 2, w2_off);
        k_group(0, wt, xt, 1, STEADY ? JW_W : 0, [&](int j) { request_part(buf_w, off_gw, step_w, t + 2, w2_off, j); });
        k_group(1, wt, xt, 2, 0, [](int) {});
        k_group(0, wt, xt, 3, 0, [](int) {});
        // Own requests of W(t+1), X(t+1) have landed (W(t+2)'s may still be in
        // flight) and every LDS read of tile t has returned; the barrier extends
        // both to the workgroup.
        __builtin_amdgcn_s_waitcnt(STEADY ? wait_vm_lgkm0(JW_W) : wait_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (!STEADY && t + 2 < ktiles) request_unit(x_kind, buf_x, base_x, off_gx, step_x, t + 2, x2_off);
        // Past the last tile these reads fetch stale LDS contents that are never used.
        k_group(1, wn1, xn1, 0, STEADY ? JW_X : 0, [&](int j) { request_part(buf_x, off_gx, step_x, t + 2, x2_off, j); });
    };
    auto advance = [&]() { s0 = s0 + 2 >= kUnits ? s0 + 2 - kUnits : s0 + 2; };

    request_unit(w_kind, buf_w, base_w, off_gw, step_w, 0, 0);
    request_unit(x_kind, buf_x, base_x, off_gx, step_x, 0, kUnitBytes);
    if (ktiles > 1) {
        request_unit(w_kind, buf_w, base_w, off_gw, step_w, 1, 2 * kUnitBytes);
        request_unit(x_kind, buf_x, base_x, off_gx, step_x, 1, 3 * kUnitBytes);
    }
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < NREAD; ++r) read_frag(lds, lds + kUnitBytes, 0, fa[0], fb[0], r);

    const int steady_end = full_tiles - 2 > 0 ? full_tiles - 2 : 0;
    int t = 0;
#pragma unroll 1
    for (; t + kUnits <= steady_end; t += kUnits) {
        k_tile(t, std::true_type{}, std::integral_constant<int, 0>{});
        k_tile(t + 1, std::true_type{}, std::integral_constant<int, 2>{});
        k_tile(t + 2, std::true_type{}, std::integral_constant<int, 4>{});
        k_tile(t + 3, std::true_type{}, std::integral_constant<int, 1>{});
        k_tile(t + 4, std::true_type{}, std::integral_constant<int, 3>{});
    }
#pragma unroll 1
    for (; t < steady_end; ++t, advance()) k_tile(t, std::true_type{}, s0);
#pragma unroll 1
    for (; t < ktiles; ++t, advance()) k_tile(t, std::false_type{}, s0);

    // The last MFMAs must have left the pipeline before acc is read by anything else.
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    // Lane holds, per 32 x 32 tile, output row m = l32 and the columns
    // n = 8 g + 4 kh + {0..3} in acc[..][4 g + {0..3}].
    const bool vec = part.vec_store != 0;
#pragma unroll
    for (int a = 0; a < TN; ++a) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int64_t n = n0 + wn + 32 * a + 8 * g + 4 * kh;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) bv[e] = bias[n + e];
            }
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                const int64_t m = m0 + wm + 32 * b + l32;
                if (m >= M) continue;
                float* dst = y + m * ldy + n;
                if (vec && n + 3 < N) {
                    floatx4 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = acc[a][b][4 * g + e] + bv[e];
                    __builtin_nontemporal_store(o, reinterpret_cast<floatx4*>(dst));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) dst[e] = acc[a][b][4 * g + e] + bv[e];
                }
            }
        }
    }
}

constexpr int kThreads = 512;

// Workgroup b computes wide tile b and then narrow tile b (where they exist).
template <bool XT, bool WT>
__global__ __launch_bounds__(kThreads) void gemm32_tiles(const Parts parts) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int b = static_cast<int>(blockIdx.x);
    const bool has_wide = b < parts.wide.tiles_m * parts.wide.tiles_n;
    if (has_wide) gemm32_tile<XT, WT, 2, 4, 4, 2>(parts.wide, b, lds);
    if (b < parts.narrow.tiles_m * parts.narrow.tiles_n) {
        if (has_wide) __syncthreads();   // every wavefront is done with the first tile's operands in LDS
        gemm32_tile<XT, WT, 4, 2, 2, 3>(parts.narrow, b, lds);
    }
}

typedef void (*Kernel)(const Parts);
const Kernel kKernels[4] = {gemm32_tiles<false, false>, gemm32_tiles<false, true>, gemm32_tiles<true, false>, gemm32_tiles<true, true>};   // 2 (x along rows) + (w along rows)
std::atomic<bool> lds_reserved[kMaxDevices][4];   // the dynamic LDS size of kKernels[i] has been raised on that device

struct Operand {
    const float* p;
    int64_t row_stride, k_stride;
    bool transposed() const { return row_stride == 1 && k_stride != 1; }
    int64_t ld() const { return transposed() ? k_stride : row_stride; }
};

// Can the tiled kernel read this operand (`rows` rows) where it lies?
bool operand_ok(const Operand& o, int64_t rows, int64_t K) {
    if (o.row_stride != 1 && o.k_stride != 1) return false;
    const int64_t ld = o.ld();
    if (!aligned_to(o.p, 16) || ld % 4 != 0 || ld > 0x1FFFFF) return false;   // 32-bit byte offsets inside a tile
    if (o.transposed()) return ld >= rows && rows % 4 == 0 && (K + BK) * ld <= 0x1FFFFFFF;
    return ld >= K && K % 4 == 0 && K <= 0x1FFFFFFF;
}

}  // namespace

// y = a . b^T + bias through the tiled kernel; false if the operands do not
// qualify (the caller then takes the strided kernel), otherwise *rc is the result.
bool gemm_f32_tiled(const float* a, int64_t a_rs, int64_t a_ks, const float* b, int64_t b_rs, int64_t b_ks, const float* bias, float* y,
                    int64_t ldy, int64_t M, int64_t N, int64_t K, void* stream, int* rc) {
    const Operand oa{a, a_rs, a_ks}, ob{b, b_rs, b_ks};
    if (!operand_ok(oa, M, K) || !operand_ok(ob, N, K)) return false;
    const int64_t tiles_m = (M + 255) / 256, cols = (N + 255) / 256;
    if (tiles_m > 0x7FFFFFll || cols > 0x7FFFFFll || tiles_m * (cols + 1) > 0x7FFFFFFFll) return false;
    int dev = 0;
    const int cus = compute_units(dev);
    const int64_t wide_cols = wide_tile_columns(tiles_m, N, cus);
    const int vec_store = (ldy % 4 == 0 && aligned_to(y, 16)) ? 1 : 0;
    auto part = [&](int bn, int64_t n_begin, int64_t n_count) {
        Part p{};
        p.x = oa.p, p.w = ob.p + n_begin * ob.row_stride, p.bias = bias ? bias + n_begin : nullptr, p.y = y + n_begin;
        p.M = M, p.N = n_count, p.K = K, p.ldx = oa.ld(), p.ldw = ob.ld(), p.ldy = ldy;
        p.tiles_m = static_cast<int>(tiles_m), p.tiles_n = static_cast<int>((n_count + bn - 1) / bn), p.vec_store = vec_store;
        return p;
    };
    Parts parts{};
    if (wide_cols > 0) parts.wide = part(256, 0, wide_cols);
    if (wide_cols < N) parts.narrow = part(192, wide_cols, N - wide_cols);
    const int n_wide = parts.wide.tiles_m * parts.wide.tiles_n, n_narrow = parts.narrow.tiles_m * parts.narrow.tiles_n;
    const int k = (oa.transposed() ? 2 : 0) + (ob.transposed() ? 1 : 0);
    if (!lds_reserved[dev][k].load(std::memory_order_acquire)) {   // the attribute sticks to the function on this device
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kKernels[k]), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        if (e != hipSuccess) {
            *rc = fail(static_cast<int>(e), "gemm f32: cannot reserve %d bytes of LDS: %s", kLdsBytes, hipGetErrorString(e));
            return true;
        }
        lds_reserved[dev][k].store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(kKernels[k], dim3(static_cast<uint32_t>(n_wide > n_narrow ? n_wide : n_narrow)), dim3(kThreads), kLdsBytes,
                       static_cast<hipStream_t>(stream), parts);
    *rc = check_launch("gemm32_tiles");
    return true;
}

}  // namespace ddl
