// DistributedLinear shard GEMM: y[M,N] = x[M,K] . w[N,K]^T + bias[N], bf16
// operands, fp32 accumulation on the matrix cores, bf16 result (reference:
// nn/linear.py:103, nn/linear_ag.py:486 -- torch.nn.functional.linear).
//
// Both operands are K-contiguous, so a 16-byte load anywhere gives eight
// consecutive k of one row: exactly one lane's share of an MFMA operand.  The
// product is formed transposed (w rows feed the A port, x rows the B port) so
// that each lane ends up with four consecutive n of one output row and can
// store them as one 8-byte word.
//
//   workgroup  512 threads = 8 wavefronts (2 along m x 4 along n), tile
//              256(m) x 256(n); two wavefronts share a SIMD so that one can
//              issue MFMAs while the other waits
//   wavefront  128(m) x 64(n) = 4 x 2 tiles of v_mfma_f32_32x32x16_bf16, 128 fp32
//              accumulators per lane
//   LDS        ring of five operand tiles (W0 X0 W1 X1 W2 | X2 W3 ...), each
//              256 rows x 64 k = 32 KiB, 160 KiB in all.  Rows are 128 B; the
//              16-byte chunk index is XOR-ed with ((row >> 1) & 7): the 16
//              lanes served per LDS cycle read 16 consecutive rows, and
//              (row & 1, (row >> 1) & 7) is distinct for each, so they cover all
//              64 banks
//   global     tiles go from global memory straight into LDS
//              (buffer_load_dwordx4 ... lds: each wavefront instruction fills
//              1 KiB = 8 rows, the eight lanes of a row fetching one whole
//              128-byte line; half-line requests run at little more than half
//              the rate).  No staging registers, no LDS stores, one 32-bit
//              offset per lane and the k offset in a scalar
//   schedule   per k-tile of 64: four k-steps of 8 MFMAs, one LDS fragment
//              read issued behind each MFMA (the fragments of the next k-step,
//              crossing into tile t+1 at the end).  W(t+2) is requested during
//              k-step 0 into the slot X(t-1) left, X(t+2) during k-step 3 into
//              the slot of W(t); before k-step 3 each wavefront waits for its
//              own requests of tile t+1 and all its LDS reads, then one
//              barrier: tile t+1 is readable, tile t's slots are free
//   epilogue   bias add and bf16 rounding in registers, then each wavefront
//              transposes its block through LDS so that rows of y are written
//              in 16-byte pieces, whole 128-byte lines per instruction
//   launch     workgroup ids are regrouped so that the 32 workgroups resident
//              on one XCD cover a compact patch of the tile grid and share
//              their operand panels in that XCD's L2
#include "ddl_common.h"
#include <type_traits>

namespace ddl {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

constexpr int BK = 64;
constexpr int kMaxTileRows = 256;                    // rows of an operand tile: 256 of x; 256 or 192 of w
constexpr int kUnitBytes = kMaxTileRows * BK * 2;    // ring slot for one operand tile (rows x 128 B), 32 KiB
constexpr int kUnits = 5;                            // ring of operand tiles: W0 X0 W1 X1 W2 | X2 W3 ...
constexpr int kLdsBytes = kUnits * kUnitBytes;       // 160 KiB: all of a CU's LDS
constexpr int kXcds = 8;

__device__ inline uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if (f != f) return 0x7FC0;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__device__ inline float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }

typedef __attribute__((address_space(3))) void* lds_ptr;

// One wavefront instruction: lane l copies the 16 bytes at byte (voffset +
// soffset) of the buffer to LDS byte (dst + 16 l); dst and soffset are the same
// for all lanes.
__device__ inline void dma16(__amdgpu_buffer_rsrc_t buffer, int voffset, int soffset, char* dst) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(buffer, (lds_ptr)dst, 16, voffset, soffset, 0, 0);
}

// acc += a . b (32 x 32 x 16, bf16 in, fp32 accumulate).  Written as assembly
// so that the accumulators live in the accumulation registers ("a" operands):
// left to itself the compiler keeps them in the vector registers next to the
// fragments, which measures 2 % slower.  The compiler still tracks the
// operands (it waits for the LDS reads that produce a and b); what it does not
// do for assembly is pad the distance between an MFMA and a later non-MFMA
// read of acc -- the kernel does that once, in front of the epilogue.
__device__ inline void mfma_32x32x16(floatx16& acc, const bf16x8& a, const bf16x8& b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// s_waitcnt immediate (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4,
// lgkmcnt 11:8): wait until at most n vector-memory requests are outstanding
// and all LDS reads have returned.
constexpr int wait_vm_lgkm0(int n) { return 0x0070 | (n & 15) | ((n >> 4) << 14); }

// NWM x NWN wavefronts, each owning TM x TN sub-tiles of 32 x 32: the workgroup
// tile is (32 NWM TM) x (32 NWN TN).
template <int NWM, int NWN, int TM, int TN>
__global__ __launch_bounds__(64 * NWM * NWN) void linear_bf16_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                               const uint16_t* __restrict__ bias, uint16_t* __restrict__ y,
                                                               int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw,
                                                               int64_t ldy, int tiles_m, int tiles_n, int vec_store) {
    extern __shared__ __attribute__((aligned(16))) char lds[];

    // XCD-aware tile assignment: hardware deals workgroup ids round-robin over
    // the XCDs, so id % 8 names the XCD.  Give each XCD a contiguous range of
    // the tile sequence, and walk that sequence in bands of 8 m-tiles.
    const int ntiles = tiles_m * tiles_n;
    int id = blockIdx.x;
    {
        const int per = ntiles / kXcds, main = per * kXcds;
        if (id < main) id = (id % kXcds) * per + id / kXcds;
    }
    constexpr int kBand = 8;
    const int band = id / (kBand * tiles_n);
    const int band_m0 = band * kBand;
    const int band_h = (tiles_m - band_m0) < kBand ? (tiles_m - band_m0) : kBand;
    const int in_band = id - band * kBand * tiles_n;
    const int tm = band_m0 + in_band % band_h;
    const int tn = in_band / band_h;

    constexpr int BM = 32 * NWM * TM, BN = 32 * NWN * TN;
    static_assert(BM <= kMaxTileRows && BN <= kMaxTileRows, "operand tile larger than a ring slot");
    const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int NW = NWM * NWN;
    // request instructions (8 rows each) per wavefront for a w tile and an x tile
    constexpr int JW_W = BN / 8 / NW, JW_X = BM / 8 / NW;
    static_assert(JW_W * 8 * NW == BN && JW_X * 8 * NW == BM, "tile rows do not divide among the wavefronts");
    const int wm = (wave % NWM) * (TM * 32), wn = (wave / NWM) * (TN * 32);   // wavefront origin inside the tile
    const int l32 = lane & 31, kg = lane >> 5;

    floatx16 acc[TN][TM];           // [n sub-tile][m sub-tile]
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

    // Global -> LDS requests of this lane.  Instruction j of this wavefront
    // fills rows (J wave + j) 8 .. +7 of an operand tile (J instructions per
    // wavefront); lane l lands on row
    // l / 8, physical chunk l % 8 of that row, i.e. logical chunk
    // (l % 8) ^ ((row >> 1) & 7): the eight lanes of a row fetch one whole
    // 128-byte line.  Rows past the end of the matrix repeat its last row
    // (their products are never stored).
    // The operands are addressed as raw buffers that start at the tile's first
    // row: a 32-bit byte offset per lane, the k-tile offset in a scalar.
    const char* const base_w = reinterpret_cast<const char*>(w + n0 * ldw);
    const char* const base_x = reinterpret_cast<const char*>(x + m0 * ldx);
    const __amdgpu_buffer_rsrc_t buf_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base_w), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t buf_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base_x), 0, -1, 0x00020000);
    int off_gw[JW_W], off_gx[JW_X];
    {
        const int r = lane >> 3;
#pragma unroll
        for (int j = 0; j < JW_W; ++j) {
            const int row = (JW_W * wave + j) * 8 + r;
            const int ck = ((lane & 7) ^ ((row >> 1) & 7)) * 8;   // first k of this lane's chunk inside a k-tile
            const int64_t rn = n0 + row < N ? row : N - 1 - n0;
            off_gw[j] = static_cast<int>((rn * ldw + ck) * 2);
        }
#pragma unroll
        for (int j = 0; j < JW_X; ++j) {
            const int row = (JW_X * wave + j) * 8 + r;
            const int ck = ((lane & 7) ^ ((row >> 1) & 7)) * 8;
            const int64_t rm = m0 + row < M ? row : M - 1 - m0;
            off_gx[j] = static_cast<int>((rm * ldx + ck) * 2);
        }
    }

    const int ktiles = static_cast<int>((K + BK - 1) / BK);
    const int full_tiles = static_cast<int>(K / BK);   // tiles [full_tiles, ktiles) straddle K

    // One request instruction (j = 0 .. J-1) of operand tile t, a full tile.
    auto request_part = [&](__amdgpu_buffer_rsrc_t buf, const auto& off, int t, int unit_off, int j) {
        constexpr int J = sizeof(off) / sizeof(int);
        dma16(buf, off[j], t * (BK * 2), lds + unit_off + (J * wave + j) * 1024);
    };
    // A whole operand tile.  One that straddles K goes through registers so
    // that the chunks past K can be written as zeros.
    auto request_unit = [&](__amdgpu_buffer_rsrc_t buf, const char* base, const auto& off, int t, int unit_off) {
        constexpr int J = sizeof(off) / sizeof(int);
        if (t < full_tiles) {
#pragma unroll
            for (int j = 0; j < J; ++j) request_part(buf, off, t, unit_off, j);
        } else {
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const int row = (J * wave + j) * 8 + (lane >> 3);
                const int ck = ((lane & 7) ^ ((row >> 1) & 7)) * 8;
                uint4 v = make_uint4(0, 0, 0, 0);
                if (static_cast<int64_t>(t) * BK + ck < K)
                    v = *reinterpret_cast<const uint4*>(base + off[j] + static_cast<int64_t>(t) * (BK * 2));
                *reinterpret_cast<uint4*>(lds + unit_off + (J * wave + j) * 1024 + lane * 16) = v;
            }
        }
    };

    // Fragment addresses: row (sub-tile origin + l32), logical chunk 2 ks + kg.
    // Sub-tile origins are multiples of 32, so the swizzle term is (l32 >> 1) & 7.
    const int frag_row = l32 * (BK * 2);
    int sw_off[4];   // byte offset of this lane's chunk in its row, per k-step
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) sw_off[ks] = ((2 * ks + kg) ^ ((l32 >> 1) & 7)) << 4;
    const int off_w = wn * (BK * 2) + frag_row;
    const int off_x = wm * (BK * 2) + frag_row;

    auto read_frag = [&](const char* wt, const char* xt, int ks, bf16x8 (&fa)[TN], bf16x8 (&fb)[TM], int i) {
        const int sw = sw_off[ks];
        if (i < TN)
            fa[i] = *reinterpret_cast<const bf16x8*>(wt + off_w + i * (32 * BK * 2) + sw);
        else
            fb[i - TN] = *reinterpret_cast<const bf16x8*>(xt + off_x + (i - TN) * (32 * BK * 2) + sw);
    };

    constexpr int kGapW = (TN * TM) / JW_W, kGapX = (TN * TM) / JW_X;   // MFMAs from one request instruction to the next
    auto unit_off = [](int slot) { return (slot >= kUnits ? slot - kUnits : slot) * kUnitBytes; };
    int s0 = 0;   // ring slot of W(t); X(t), W(t+1), X(t+1), W(t+2) follow
    bf16x8 fa[2][TN], fb[2][TM];

    // One k-tile = four k-steps of 16.  On entry the fragments of (t, k-step 0)
    // are in fa[0] / fb[0] or on their way, W(t+1) and X(t+1) have been
    // requested.  STEADY: tile t+2 exists and is a full tile; its request
    // instructions are spread between the MFMAs.
    auto k_tile = [&](int t, auto steady) {
        constexpr bool STEADY = decltype(steady)::value;
        const char* wt = lds + unit_off(s0);
        const char* xt = lds + unit_off(s0 + 1);
        const char* wn1 = lds + unit_off(s0 + 2);
        const char* xn1 = lds + unit_off(s0 + 3);
        const int w2_off = unit_off(s0 + 4);   // slot of X(t-1), free since the barrier of tile t-1
        const int x2_off = unit_off(s0);       // slot of W(t), free after this tile's barrier
        if (!STEADY && t + 2 < ktiles) request_unit(buf_w, base_w, off_gw, t + 2, w2_off);
#pragma unroll
        for (int ks = 0; ks < 3; ++ks) {
#pragma unroll
            for (int i = 0; i < TN * TM; ++i) {
                const int a = i / TM, b = i % TM;
                mfma_32x32x16(acc[a][b], fa[ks & 1][a], fb[ks & 1][b]);
                if (i < TN + TM) read_frag(wt, xt, ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1], i);
                if (STEADY && ks == 0 && i % kGapW == kGapW - 1 && i / kGapW < JW_W) request_part(buf_w, off_gw, t + 2, w2_off, i / kGapW);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // Own requests of W(t+1), X(t+1) have landed (W(t+2)'s may still be in
        // flight) and every LDS read issued so far -- all of tile t's -- has
        // returned; the barrier extends both to the workgroup, so tile t+1 may
        // be read and tile t's slots may be overwritten.
        __builtin_amdgcn_s_waitcnt(STEADY ? wait_vm_lgkm0(JW_W) : wait_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (!STEADY && t + 2 < ktiles) request_unit(buf_x, base_x, off_gx, t + 2, x2_off);
#pragma unroll
        for (int i = 0; i < TN * TM; ++i) {
            const int a = i / TM, b = i % TM;
            mfma_32x32x16(acc[a][b], fa[1][a], fb[1][b]);
            // Past the last tile these reads fetch stale LDS contents that are never used.
            if (i < TN + TM) read_frag(wn1, xn1, 0, fa[0], fb[0], i);
            if (STEADY && i % kGapX == kGapX - 1 && i / kGapX < JW_X) request_part(buf_x, off_gx, t + 2, x2_off, i / kGapX);
            __builtin_amdgcn_sched_barrier(0);
        }
        s0 = s0 + 2 >= kUnits ? s0 + 2 - kUnits : s0 + 2;
    };

    static_assert(TN * TM >= JW_W && TN * TM >= JW_X, "not enough MFMAs in a k-step to spread the requests");
    request_unit(buf_w, base_w, off_gw, 0, 0);
    request_unit(buf_x, base_x, off_gx, 0, kUnitBytes);
    if (ktiles > 1) {
        request_unit(buf_w, base_w, off_gw, 1, 2 * kUnitBytes);
        request_unit(buf_x, base_x, off_gx, 1, 3 * kUnitBytes);
    }
    // Tile 0 complete and visible, then its first fragments.
    __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < TN + TM; ++i) read_frag(lds, lds + kUnitBytes, 0, fa[0], fb[0], i);

    const int steady_end = full_tiles - 2 > 0 ? full_tiles - 2 : 0;
    int t = 0;
#pragma unroll 1
    for (; t < steady_end; ++t) k_tile(t, std::true_type{});
#pragma unroll 1
    for (; t < ktiles; ++t) k_tile(t, std::false_type{});

    // The last MFMAs must have left the pipeline before acc is read by anything
    // else (18 wait states cover every case; these are 32).
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    // Epilogue.  Lane holds, per 32x32 tile, output row m = l32 and the columns
    // n = 8*g + 4*kg + {0,1,2,3} for g = 0..3 in acc[...][4*g + {0..3}].
    if (vec_store == 2) {
        // Through LDS, so that global stores are 16 bytes per lane and whole
        // 128-byte (or longer) row segments per instruction.  Each wavefront
        // transposes its own (32 TM) x (32 TN) block in a private LDS region:
        // row pitch 64 TN bytes, the 16-byte chunk index XOR-ed with a function
        // of the row so that neither the 8-byte writes (32 rows, one column
        // group) nor the 16-byte reads (whole rows) pile up on banks.
        constexpr int kChunks = TN * 4;              // 16-byte chunks per row of the block
        constexpr bool kPow2 = (kChunks & (kChunks - 1)) == 0;
        // A power-of-two row is swizzled; any other row length is padded by one
        // chunk instead, which staggers consecutive rows over the banks.
        constexpr int kPitch = kPow2 ? TN * 64 : TN * 64 + 16;
        auto swz = [](int row) { return !kPow2 ? 0 : kChunks == 8 ? ((row >> 1) & 7) : (row & (kChunks - 1)); };
        __syncthreads();   // every wavefront is done with the operand stages (and every request has landed)
        char* region = lds + wave * (TM * 32 * kPitch);
#pragma unroll
        for (int a = 0; a < TN; ++a) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int64_t n = n0 + wn + a * 32 + 8 * g + 4 * kg;
                float bv[4] = {0.f, 0.f, 0.f, 0.f};
                if (bias) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) bv[e] = bf16_bits_to_f32(bias[n + e]);
                }
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    const int row = b * 32 + l32;
                    uint16_t o[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = f32_to_bf16_bits(acc[a][b][4 * g + e] + bv[e]);
                    uint2 pk;
                    pk.x = static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16);
                    pk.y = static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16);
                    *reinterpret_cast<uint2*>(region + row * kPitch + (((a * 4 + g) ^ swz(row)) << 4) + kg * 8) = pk;
                }
            }
        }
        // LDS operations of one wavefront complete in order, so its reads below
        // see its writes above; no other wavefront touches this region.
        asm volatile("" ::: "memory");
        static_assert((TM * 32 * kChunks) % 64 == 0, "block does not split into whole wavefront passes");
#pragma unroll 4
        for (int p = 0; p < TM * 32 * kChunks / 64; ++p) {
            const int idx = p * 64 + lane;
            const int row = idx / kChunks, chunk = idx % kChunks;
            const int64_t m = m0 + wm + row;
            const int64_t n = n0 + wn + chunk * 8;
            const uint4 v = *reinterpret_cast<const uint4*>(region + row * kPitch + ((chunk ^ swz(row)) << 4));
            if (m >= M || n >= N) continue;
            uint16_t* dst = y + m * ldy + n;
            if (n + 8 <= N) {
                typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // y is not read again here: streaming store
                u32x4 nv;
                nv[0] = v.x, nv[1] = v.y, nv[2] = v.z, nv[3] = v.w;
                __builtin_nontemporal_store(nv, reinterpret_cast<u32x4*>(dst));
            } else {
                const uint32_t words[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (n + e < N) dst[e] = static_cast<uint16_t>(words[e >> 1] >> (16 * (e & 1)));
            }
        }
    } else {
    #pragma unroll
        for (int a = 0; a < TN; ++a) {
    #pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int64_t n = n0 + wn + a * 32 + 8 * g + 4 * kg;
                float bv[4] = {0.f, 0.f, 0.f, 0.f};
                if (bias) {
    #pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) bv[e] = bf16_bits_to_f32(bias[n + e]);
                }
    #pragma unroll
                for (int b = 0; b < TM; ++b) {
                    const int64_t m = m0 + wm + b * 32 + l32;
                    if (m >= M) continue;
                    uint16_t o[4];
    #pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = f32_to_bf16_bits(acc[a][b][4 * g + e] + bv[e]);
                    uint16_t* dst = y + m * ldy + n;
                    if (vec_store && n + 3 < N) {
                        uint2 pk;
                        pk.x = static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16);
                        pk.y = static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16);
                        *reinterpret_cast<uint2*>(dst) = pk;
                    } else {
    #pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < N) dst[e] = o[e];
                    }
                }
            }
        }
    }
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_linear_bf16(const void* x, const void* w, const void* bias, void* y, int64_t M, int64_t N, int64_t K,
                               int64_t ldx, int64_t ldw, int64_t ldy, void* stream) {
    using namespace ddl;
    if (M < 0 || N < 0 || K < 0 || ldx < K || ldw < K || ldy < N)
        return fail(DDL_E_ARG, "linear: M=%lld N=%lld K=%lld ldx=%lld ldw=%lld ldy=%lld", (long long)M, (long long)N,
                    (long long)K, (long long)ldx, (long long)ldw, (long long)ldy);
    if (M == 0 || N == 0) return 0;
    if (!x || !w || !y) return fail(DDL_E_ARG, "linear: null pointer");
    if (K == 0) return fail(DDL_E_UNSUPP, "linear: K = 0");
    if (K % 8 != 0 || ldx % 8 != 0 || ldw % 8 != 0 || !aligned_to(x, 16) || !aligned_to(w, 16))
        return fail(DDL_E_ALIGN, "linear: K, ldx, ldw must be multiples of 8 and x, w 16-byte aligned");
    if (!aligned_to(y, 2) || (bias && !aligned_to(bias, 2))) return fail(DDL_E_ALIGN, "linear: y / bias misaligned");
    if (ldx > 0x3FFFFF || ldw > 0x3FFFFF || K > 0x3FFFFFFF)
        return fail(DDL_E_UNSUPP, "linear: row pitch above 2^22 elements or K above 2^30");   // 32-bit byte offsets inside a tile
    // 2: rows of y can be stored 16 bytes at a time, 1: 8 bytes, 0: element by element
    const int vec_store = (ldy % 8 == 0 && aligned_to(y, 16)) ? 2 : (ldy % 4 == 0 && aligned_to(y, 8)) ? 1 : 0;
    const uint16_t* const xp = static_cast<const uint16_t*>(x);
    const uint16_t* const wp = static_cast<const uint16_t*>(w);
    const uint16_t* const bp = static_cast<const uint16_t*>(bias);
    uint16_t* const yp = static_cast<uint16_t*>(y);

    // Columns [n_begin, n_begin + n_count) of the output with tiles of 256 x bn.
    auto launch = [&](auto kernel, bool& attr_done, int threads, int bn, int64_t n_begin, int64_t n_count) -> int {
        const int64_t tiles_m = (M + 255) / 256, tiles_n = (n_count + bn - 1) / bn;
        if (tiles_m * tiles_n > 0x7FFFFFFFll || tiles_m > 0x7FFFFFll || tiles_n > 0x7FFFFFll)
            return fail(DDL_E_UNSUPP, "linear: too many output tiles");
        if (!attr_done) {   // the attribute sticks to the function; set it on first use
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
            if (e != hipSuccess) return fail(static_cast<int>(e), "linear: cannot reserve %d bytes of LDS: %s", kLdsBytes, hipGetErrorString(e));
            attr_done = true;
        }
        hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(tiles_m * tiles_n)), dim3(threads), kLdsBytes,
                           static_cast<hipStream_t>(stream), xp, wp + n_begin * ldw, bp ? bp + n_begin : nullptr, yp + n_begin, M,
                           n_count, K, ldx, ldw, ldy, static_cast<int>(tiles_m), static_cast<int>(tiles_n), vec_store);
        return check_launch("linear_bf16_kernel");
    };
    static bool wide_ready = false, narrow_ready = false;
    auto wide = [&](int64_t n_begin, int64_t n_count) { return launch(linear_bf16_kernel<2, 4, 4, 2>, wide_ready, 512, 256, n_begin, n_count); };
    auto narrow = [&](int64_t n_begin, int64_t n_count) { return launch(linear_bf16_kernel<4, 2, 2, 3>, narrow_ready, 512, 192, n_begin, n_count); };

    // One workgroup per CU is resident, so the tiles run in rounds of one per
    // CU and a last round that is only partly filled costs as much as a full
    // one.  When it pays, the columns are split: whole rounds of 256-wide
    // tiles first, the rest with 192-wide tiles, whose rounds are shorter.
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1)
            n = 256;
        cus = n;
    }
    const int64_t tiles_m = (M + 255) / 256, cols = (N + 255) / 256;
    auto rounds = [&](int64_t tiles) { return (tiles + cus - 1) / cus; };
    const int64_t cost_wide = rounds(tiles_m * cols) * 256;
    int64_t best_cost = cost_wide, best_split = cols;   // columns of 256 given to the wide kernel
    for (int64_t c = cols - 1; c >= 0 && c >= cols - 16; --c) {
        const int64_t rest = N - c * 256;
        const int64_t cost = rounds(tiles_m * c) * 256 + rounds(tiles_m * ((rest + 191) / 192)) * 192;
        if (cost < best_cost) {
            best_cost = cost;
            best_split = c;
        }
    }
    if (best_split == cols) return wide(0, N);
    if (best_split > 0) {
        const int rc = wide(0, best_split * 256);
        if (rc) return rc;
    }
    return narrow(best_split * 256, N - best_split * 256);
}
