// DistributedLinear shard GEMM: y[M,N] = x[M,K] . w[N,K]^T + bias[N], bf16 (or
// fp16) operands, fp32 accumulation on the matrix cores, result in the operands'
// type (reference: nn/linear.py:103, nn/linear_ag.py:486 --
// torch.nn.functional.linear).
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
//   wavefront  128(m) x 64(n) = 8 x 4 tiles of v_mfma_f32_16x16x32_bf16, 128 fp32
//              accumulators per lane.  On random operands the chip is limited
//              by power, and this instruction delivers about 14 % more flop/s
//              under that limit than the 32x32x16 one (it moves half as many
//              accumulator bytes per flop)
//   LDS        ring of five operand tiles (W0 X0 W1 X1 W2 | X2 W3 ...), each
//              256 rows x 64 k = 32 KiB, 160 KiB in all.  Rows are 128 B; the
//              16-byte chunk index is XOR-ed with ((row >> 1) & 7): the 16
//              lanes served per LDS cycle read 16 consecutive rows, and
//              (row & 1, (row >> 1) & 7) is distinct for each, so they cover all
//              64 banks (an MFMA operand piece is 16 rows x 32 k: lane l reads
//              row l % 16, chunk l / 16 of the k-step)
//   global     tiles go from global memory straight into LDS
//              (buffer_load_dwordx4 ... lds: each wavefront instruction fills
//              1 KiB = 8 rows, the eight lanes of a row fetching one whole
//              128-byte line; half-line requests run at little more than half
//              the rate).  No staging registers, no LDS stores, one 32-bit
//              offset per lane and the k offset in a scalar
//   schedule   per k-tile of 64: two k-steps of 32 MFMAs, one LDS fragment
//              read issued behind every second MFMA (the fragments of the next
//              k-step, crossing into tile t+1 in the second k-step).  W(t+2) is
//              requested during k-step 0 into the slot X(t-1) left, X(t+2)
//              during k-step 1 into the slot of W(t); between the two k-steps
//              each wavefront waits for its own requests of tile t+1 and all
//              its LDS reads, then one barrier: tile t+1 is readable, tile t's
//              slots are free
//   epilogue   bias add and bf16 rounding in registers, then each wavefront
//              transposes its block through LDS so that rows of y are written
//              in 16-byte pieces, whole 128-byte lines per instruction
//   launch     one workgroup per CU is resident, so the tiles run in rounds of
//              one per CU and a last round that is only partly filled costs as
//              much as a full one; when it pays, the columns are split between
//              256-wide tiles (whole rounds) and 192-wide tiles (4 x 2
//              wavefronts of 64 x 96), whose rounds are shorter.  One launch:
//              workgroup b computes wide tile b and then narrow tile b, so the
//              stores of its first tile drain while it computes the second and
//              the workgroups of an XCD stay in step.  (Both kinds as separate
//              workgroups of one grid, so that a CU starts on a narrow tile the
//              moment its wide one is stored, measured 2 % slower: the
//              workgroups of an XCD then drift apart in k and share fewer
//              operand lines in its L2; two launches measured 1 % slower.)
//              Workgroup ids are regrouped so that the 32 workgroups resident on
//              one XCD cover a compact patch of the tile grid and share their
//              operand panels in that XCD's L2
#include "gemm_tiles.h"
#include <hip/hip_fp16.h>
#include <type_traits>

namespace ddl {
namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int BK = kRowBytes / 2;   // 16-bit elements of a k-tile

__device__ inline uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if (f != f) return 0x7FC0;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__device__ inline float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(static_cast<uint32_t>(b) << 16); }

// acc += a . b (16 x 16 x 32, bf16 in, fp32 accumulate).  Written as assembly
// so that the accumulators live in the accumulation registers ("a" operands):
// left to itself the compiler keeps them in the vector registers next to the
// fragments, which measures 2 % slower.  The compiler still tracks the
// operands (it waits for the LDS reads that produce a and b); what it does not
// do for assembly is pad the distance between an MFMA and a later non-MFMA
// read of acc -- the kernel does that once, in front of the epilogue.
template <bool F16>
__device__ inline void mfma_16x16x32(floatx4& acc, const bf16x8& a, const bf16x8& b) {
    if (F16)   // the same eight 16-bit elements per lane, read as fp16
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
    else
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// 16-bit element <-> fp32, round to nearest even on the way back.
template <bool F16>
__device__ inline float elem_to_f32(uint16_t b) {
    if (F16) {
        __half h;
        __builtin_memcpy(&h, &b, 2);
        return __half2float(h);
    }
    return bf16_bits_to_f32(b);
}
template <bool F16>
__device__ inline uint16_t f32_to_elem(float f) {
    if (F16) {
        const __half h = __float2half_rn(f);
        uint16_t b;
        __builtin_memcpy(&b, &h, 2);
        return b;
    }
    return f32_to_bf16_bits(f);
}

// NWM x NWN wavefronts, each owning TM x TN sub-tiles of 16 x 16: the workgroup
// tile is (16 NWM TM) x (16 NWN TN).
typedef PartOf<uint16_t> Part;

template <bool F16, bool XT, bool WT, int NWM, int NWN, int TM, int TN>
__device__ __forceinline__ void gemm_tile(const Part& part, int tile_id, char* lds) {
    static_assert(NWM * NWN == 8, "eight wavefronts per workgroup");
    const uint16_t* __restrict__ x = part.x;
    const uint16_t* __restrict__ w = part.w;
    const uint16_t* __restrict__ bias = part.bias;
    uint16_t* __restrict__ y = part.y;
    const int64_t M = part.M, N = part.N, K = part.K, ldx = part.ldx, ldw = part.ldw, ldy = part.ldy;
    const int tiles_m = part.tiles_m, tiles_n = part.tiles_n, vec_store = part.vec_store;

    int tm, tn;
    tile_of_workgroup(tile_id, tiles_m, tiles_n, tm, tn);

    constexpr int BM = 16 * NWM * TM, BN = 16 * NWN * TN;
    static_assert(BM <= kMaxTileRows && BN <= kMaxTileRows, "operand tile larger than a ring slot");
    const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // the same in all lanes: keep it scalar
    constexpr int NW = NWM * NWN;
    // request instructions (8 rows each) per wavefront for a w tile and an x tile
    constexpr int JW_W = BN / 8 / NW, JW_X = BM / 8 / NW;
    static_assert(JW_W * 8 * NW == BN && JW_X * 8 * NW == BM, "tile rows do not divide among the wavefronts");
    const int wm = (wave % NWM) * (TM * 16), wn = (wave / NWM) * (TN * 16);   // wavefront origin inside the tile
    const int l16 = lane & 15, kg = lane >> 4;

    floatx4 acc[TN][TM];           // [n sub-tile][m sub-tile]
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[a][b][e] = 0.f;

    // Global -> LDS requests of this lane.  The operands are addressed as raw
    // buffers that start at the tile's first row: a 32-bit byte offset per lane,
    // the k-tile offset in a scalar.
    //
    // Operand contiguous along k: instruction j of this wavefront fills rows
    // (J wave + j) 8 .. +7 of an operand tile (J instructions per wavefront);
    // lane l lands on row l / 8, physical chunk l % 8 of that row, i.e. logical
    // chunk (l % 8) ^ ((row >> 1) & 7): the eight lanes of a row fetch one whole
    // 128-byte line.  Rows past the end of the matrix repeat its last row (their
    // products are never stored).
    //
    // Operand contiguous along its rows ("transposed": element (row, k) lies at
    // k ld + row): the tile is kept in LDS as panels of 64 rows, each panel 64
    // k-lines of 128 bytes.  Instruction j of wavefront v fills k-lines 8 v .. +7
    // of panel j; lane l lands on k-line l / 8, physical chunk l % 8, and fetches
    // the logical chunk (l % 8) ^ 2 h(k), h(k) = bit 1 of k + 2 (bit 3 of k): again
    // one whole 128-byte line per eight lanes.  Chunks past the last row of the
    // matrix repeat the first chunk of the tile.
    const char* const base_w = reinterpret_cast<const char*>(WT ? w + n0 : w + n0 * ldw);
    const char* const base_x = reinterpret_cast<const char*>(XT ? x + m0 : x + m0 * ldx);
    const u32x4 buf_w = raw_buffer(base_w), buf_x = raw_buffer(base_x);
    // bytes from one k-tile of an operand to the next
    const int step_w = WT ? static_cast<int>(ldw) * (BK * 2) : BK * 2;
    const int step_x = XT ? static_cast<int>(ldx) * (BK * 2) : BK * 2;
    int off_gw[JW_W], off_gx[JW_X];
    {
        auto lane_offset = [&](bool transposed, int J, int j, int64_t origin, int64_t rows, int64_t ld) -> int {
            if (!transposed) {
                const int row = (J * wave + j) * 8 + (lane >> 3);
                const int ck = ((lane & 7) ^ ((row >> 1) & 7)) * 8;   // first k of this lane's chunk inside a k-tile
                const int64_t rr = origin + row < rows ? row : rows - 1 - origin;
                return static_cast<int>((rr * ld + ck) * 2);
            }
            const int k = 8 * wave + (lane >> 3);
            const int h = ((k >> 1) & 1) | (((k >> 3) & 1) << 1);
            int col = j * 64 + ((lane & 7) ^ (h << 1)) * 8;              // first tile row of this lane's chunk
            if (origin + col >= rows) col = 0;
            return static_cast<int>((k * ld + col) * 2);
        };
#pragma unroll
        for (int j = 0; j < JW_W; ++j) off_gw[j] = lane_offset(WT, JW_W, j, n0, N, ldw);
#pragma unroll
        for (int j = 0; j < JW_X; ++j) off_gx[j] = lane_offset(XT, JW_X, j, m0, M, ldx);
    }

    const int ktiles = static_cast<int>((K + BK - 1) / BK);
    const int full_tiles = static_cast<int>(K / BK);   // tiles [full_tiles, ktiles) straddle K

    // LDS byte, inside an operand tile, where request instruction j of this wavefront starts.
    auto lds_dst = [&](bool transposed, int J, int j) { return transposed ? j * 8192 + wave * 1024 : (J * wave + j) * 1024; };
    // One request instruction (j = 0 .. J-1) of operand tile t, a full tile.
    auto request_part = [&](auto transposed, u32x4 buf, const auto& off, int step, int t, int unit_off, int j) {
        constexpr int J = sizeof(off) / sizeof(int);
        dma16(buf, off[j], t * step, lds + unit_off + lds_dst(decltype(transposed)::value, J, j));
    };
    // A whole operand tile.  One that straddles K goes through registers so
    // that the elements past K can be written as zeros.
    auto request_unit = [&](auto transposed, u32x4 buf, const char* base, const auto& off, int step, int t, int unit_off) {
        constexpr int J = sizeof(off) / sizeof(int);
        constexpr bool T = decltype(transposed)::value;
        if (t < full_tiles) {
#pragma unroll
            for (int j = 0; j < J; ++j) request_part(transposed, buf, off, step, t, unit_off, j);
        } else {
#pragma unroll
            for (int j = 0; j < J; ++j) {
                bool inside;
                if (T) {
                    inside = static_cast<int64_t>(t) * BK + 8 * wave + (lane >> 3) < K;
                } else {
                    const int row = (J * wave + j) * 8 + (lane >> 3);
                    const int ck = ((lane & 7) ^ ((row >> 1) & 7)) * 8;
                    inside = static_cast<int64_t>(t) * BK + ck < K;
                }
                uint4 v = make_uint4(0, 0, 0, 0);
                if (inside) v = *reinterpret_cast<const uint4*>(base + off[j] + static_cast<int64_t>(t) * step);
                *reinterpret_cast<uint4*>(lds + unit_off + lds_dst(T, J, j) + lane * 16) = v;
            }
        }
    };
    const std::integral_constant<bool, WT> w_kind{};
    const std::integral_constant<bool, XT> x_kind{};

    // Fragment addresses.  Operand contiguous along k: row (sub-tile origin +
    // l16), logical chunk 4 ks + kg; sub-tile origins are multiples of 16, so the
    // swizzle term is (l16 >> 1) & 7.
    const int frag_row = l16 * (BK * 2);
    int sw_off[2];   // byte offset of this lane's chunk in its row, per k-step
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) sw_off[ks] = ((4 * ks + kg) ^ ((l16 >> 1) & 7)) << 4;
    const int off_w = wn * (BK * 2) + frag_row;
    const int off_x = wm * (BK * 2) + frag_row;
    // Transposed operand: the 16 rows of a sub-tile are 32 bytes of a k-line.  A
    // transposing read (ds_read_b64_tr_b16) works per group of 16 lanes: lane i
    // of the group points at 8 bytes = 4 rows, (k-line i / 4, rows 4 (i % 4) ..
    // +3), and receives row i of k-lines 0 .. 3 -- half of the eight k this lane
    // feeds to the MFMA; the k-lines four further down give the other half.
    // Group kg of the wavefront covers k-lines 8 kg .. + 7 of the k-step.  The
    // 32-byte unit index is XOR-ed with h(k) (see the requests): the 32 lanes
    // served per LDS cycle read 8 different k-lines, and (k & 1, unit ^ h(k)) is
    // distinct for each, so they cover all 64 banks.
    const int tr_lane = (8 * kg + (l16 >> 2)) * 128 + (l16 & 3) * 8;
    const int tr_h = (((l16 >> 3) & 1) | ((kg & 1) << 1)) << 5;
    typedef short short4v __attribute__((ext_vector_type(4)));
    typedef short short8v __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) short4v* lds_short4;
    // Piece of a transposed operand tile: 16-row block `sub` of the tile, k-step ks.
    auto read_transposed = [&](const char* tile, int sub, int ks) -> bf16x8 {
        const char* p = tile + (sub >> 2) * 8192 + ks * (32 * 128) + (tr_lane + (((sub & 3) << 5) ^ tr_h));
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4)(p));
        const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4)(p + 4 * 128));
        const short8v both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        bf16x8 out;
        __builtin_memcpy(&out, &both, 16);
        return out;
    };
    const int sub_w = (wave / NWM) * TN, sub_x = (wave % NWM) * TM;   // first 16-row block of this wavefront in the w and x tiles

    // The operand with more pieces per wavefront runs in the outer loop of a
    // k-step: a piece of it is used by a few consecutive MFMAs and is dead
    // afterwards, so that its successor can take its registers; the pieces of the
    // other operand stay live for the whole k-step.
    constexpr bool kOuterX = TM >= TN;
    constexpr int NI = kOuterX ? TN : TM;    // pieces of the inner operand
    constexpr int NMFMA = TN * TM, NREAD = TN + TM;
    static_assert(2 * NREAD - 1 < NMFMA, "a k-step has too few MFMAs to hide its fragment reads");

    // Read number r of a k-step (issued behind MFMA 2 r + 1), in the order the
    // next k-step needs the pieces: outer 0, all inner ones, outer 1, 2, ...
    auto read_frag = [&](const char* wt, const char* xt, int ks, bf16x8 (&fa)[TN], bf16x8 (&fb)[TM], int r) {
        const int sw = sw_off[ks];
        const bool outer = r == 0 || r > NI;
        const int idx = r == 0 ? 0 : (r <= NI ? r - 1 : r - NI);
        const bool is_x = outer == kOuterX;
        if (is_x)
            fb[idx] = XT ? read_transposed(xt, sub_x + idx, ks) : *reinterpret_cast<const bf16x8*>(xt + off_x + idx * (16 * BK * 2) + sw);
        else
            fa[idx] = WT ? read_transposed(wt, sub_w + idx, ks) : *reinterpret_cast<const bf16x8*>(wt + off_w + idx * (16 * BK * 2) + sw);
    };

    // Request instructions go behind even MFMAs (the fragment reads take the odd
    // ones).  Those of W(t+2) have a tile and a half to land and are spread over
    // their k-step; those of X(t+2) have one tile, so they go out in the first
    // slots after the barrier that frees their ring slot.
    constexpr int kGapW = NMFMA / JW_W;   // MFMAs from one request instruction of W to the next
    static_assert(kGapW % 2 == 0 && kGapW >= 2 && 2 * JW_X <= NMFMA, "request slots must fall on even MFMAs");
    auto unit_off = [](int slot) { return (slot >= kUnits ? slot - kUnits : slot) * kUnitBytes; };
    int s0 = 0;   // ring slot of W(t); X(t), W(t+1), X(t+1), W(t+2) follow
    bf16x8 fa[2][TN], fb[2][TM];

    // One k-step: NMFMA MFMAs on the pieces in fa[cur] / fb[cur]; the pieces
    // of the next k-step are read from (wt, xt) at k-step `ks_next` into
    // fa[cur ^ 1] / fb[cur ^ 1]; `request(j)` issues request instruction j of
    // `nreq`, behind MFMA `first + j * gap`.
    auto k_step = [&](int cur, const char* wt, const char* xt, int ks_next, int first, int gap, int nreq, auto request) {
#pragma unroll
        for (int q = 0; q < NMFMA; ++q) {
            const int o = q / NI, i = (o & 1) ? NI - 1 - q % NI : q % NI;   // back and forth: the inner piece stays across a change of the outer one
            const int a = kOuterX ? i : o, b = kOuterX ? o : i;
            mfma_16x16x32<F16>(acc[a][b], fa[cur][a], fb[cur][b]);
            if ((q & 1) && (q >> 1) < NREAD) read_frag(wt, xt, ks_next, fa[cur ^ 1], fb[cur ^ 1], q >> 1);
            if (q >= first && (q - first) % gap == 0 && (q - first) / gap < nreq) request((q - first) / gap);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // One k-tile = two k-steps of 32.  On entry the fragments of (t, k-step 0)
    // are in fa[0] / fb[0] or on their way, W(t+1) and X(t+1) have been
    // requested.  STEADY: tile t+2 exists and is a full tile; its request
    // instructions are spread between the MFMAs.
    // `slot` is the ring slot of W(t): the running s0, or a compile-time constant
    // (the steady loop is unrolled over the five positions of the ring, so
    // that LDS addresses are immediates instead of scalar arithmetic that all
    // wavefronts of a SIMD would run at the same moment, right after a barrier,
    // with the matrix cores idle).
    auto k_tile = [&](int t, auto steady, auto slot) {
        constexpr bool STEADY = decltype(steady)::value;
        const int s0 = slot;
        const char* wt = lds + unit_off(s0);
        const char* xt = lds + unit_off(s0 + 1);
        const char* wn1 = lds + unit_off(s0 + 2);
        const char* xn1 = lds + unit_off(s0 + 3);
        const int w2_off = unit_off(s0 + 4);   // slot of X(t-1), free since the barrier of tile t-1
        const int x2_off = unit_off(s0);       // slot of W(t), free after this tile's barrier
        if (!STEADY && t + 2 < ktiles) request_unit(w_kind, buf_w, base_w, off_gw, step_w, t + 2, w2_off);
        k_step(0, wt, xt, 1, kGapW - 2, kGapW, STEADY ? JW_W : 0, [&](int j) { request_part(w_kind, buf_w, off_gw, step_w, t + 2, w2_off, j); });
        // Own requests of W(t+1), X(t+1) have landed (W(t+2)'s may still be in
        // flight) and every LDS read issued so far -- all of tile t's -- has
        // returned; the barrier extends both to the workgroup, so tile t+1 may
        // be read and tile t's slots may be overwritten.
        __builtin_amdgcn_s_waitcnt(STEADY ? wait_vm_lgkm0(JW_W) : wait_vm_lgkm0(0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (!STEADY && t + 2 < ktiles) request_unit(x_kind, buf_x, base_x, off_gx, step_x, t + 2, x2_off);
        // Past the last tile the reads of this k-step fetch stale LDS contents that are never used.
        k_step(1, wn1, xn1, 0, 0, 2, STEADY ? JW_X : 0, [&](int j) { request_part(x_kind, buf_x, off_gx, step_x, t + 2, x2_off, j); });
    };
    auto advance = [&]() { s0 = s0 + 2 >= kUnits ? s0 + 2 - kUnits : s0 + 2; };

    request_unit(w_kind, buf_w, base_w, off_gw, step_w, 0, 0);
    request_unit(x_kind, buf_x, base_x, off_gx, step_x, 0, kUnitBytes);
    if (ktiles > 1) {
        request_unit(w_kind, buf_w, base_w, off_gw, step_w, 1, 2 * kUnitBytes);
        request_unit(x_kind, buf_x, base_x, off_gx, step_x, 1, 3 * kUnitBytes);
    }
    // Tile 0 complete and visible, then its first fragments.  The requests of
    // tile 1 (the last JW_W + JW_X of this wavefront, when they went out as
    // requests) may stay in flight: the wait in the middle of k-tile 0 covers them.
    if (full_tiles > 1)
        __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(JW_W + JW_X));
    else
        __builtin_amdgcn_s_waitcnt(wait_vm_lgkm0(0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < NREAD; ++r) read_frag(lds, lds + kUnitBytes, 0, fa[0], fb[0], r);

    const int steady_end = full_tiles - 2 > 0 ? full_tiles - 2 : 0;
    int t = 0;
#pragma unroll 1
    for (; t + kUnits <= steady_end; t += kUnits) {   // s0 == 0 here: five tiles bring the ring back to where it was
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

    // The last MFMAs must have left the pipeline before acc is read by anything
    // else (18 wait states cover every case; these are 32).
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    // Epilogue.  Lane holds, per 16x16 tile, output row m = l16 and the columns
    // n = 4 kg + {0,1,2,3} in acc[...][0..3].
    if (vec_store == 2) {
        // Through LDS, so that global stores are 16 bytes per lane and whole
        // 128-byte (or longer) row segments per instruction.  Each wavefront
        // transposes its own (16 TM) x (16 TN) block in a private LDS region:
        // row pitch 32 TN bytes, the 16-byte chunk index XOR-ed with a function
        // of the row so that neither the 8-byte writes (16 rows, four column
        // groups) nor the 16-byte reads (whole rows) pile up on banks.
        constexpr int kChunks = TN * 2;              // 16-byte chunks per row of the block
        constexpr bool kPow2 = (kChunks & (kChunks - 1)) == 0;
        // A power-of-two row is swizzled; any other row length is padded by one
        // chunk instead, which staggers consecutive rows over the banks.
        constexpr int kPitch = kPow2 ? TN * 32 : TN * 32 + 16;
        auto swz = [](int row) { return !kPow2 ? 0 : kChunks == 8 ? ((row >> 1) & 7) : (row & (kChunks - 1)); };
        __syncthreads();   // every wavefront is done with the operand stages (and every request has landed)
        char* region = lds + wave * (TM * 16 * kPitch);
#pragma unroll
        for (int a = 0; a < TN; ++a) {
            const int64_t n = n0 + wn + a * 16 + 4 * kg;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) bv[e] = elem_to_f32<F16>(bias[n + e]);
            }
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                const int row = b * 16 + l16;
                uint16_t o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = f32_to_elem<F16>(acc[a][b][e] + bv[e]);
                uint2 pk;
                pk.x = static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16);
                pk.y = static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16);
                // columns a 16 + 4 kg .. + 3 of the block: chunk 2 a + kg / 2, half kg % 2
                *reinterpret_cast<uint2*>(region + row * kPitch + (((a * 2 + (kg >> 1)) ^ swz(row)) << 4) + (kg & 1) * 8) = pk;
            }
        }
        // LDS operations of one wavefront complete in order, so its reads below
        // see its writes above; no other wavefront touches this region.
        asm volatile("" ::: "memory");
        static_assert((TM * 16 * kChunks) % 64 == 0, "block does not split into whole wavefront passes");
#pragma unroll 4
        for (int p = 0; p < TM * 16 * kChunks / 64; ++p) {
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
            const int64_t n = n0 + wn + a * 16 + 4 * kg;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (n + e < N) bv[e] = elem_to_f32<F16>(bias[n + e]);
            }
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                const int64_t m = m0 + wm + b * 16 + l16;
                if (m >= M) continue;
                uint16_t o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = f32_to_elem<F16>(acc[a][b][e] + bv[e]);
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

constexpr int kThreads = 512;

typedef PartsOf<uint16_t> Parts;

// Workgroup b computes wide tile b and then narrow tile b (where they exist):
// the stores of the first tile drain while the second is computed, and there
// is no kernel boundary between the two rounds.
template <bool F16, bool XT, bool WT>
__global__ __launch_bounds__(kThreads) void gemm16_tiles(const Parts parts) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int b = static_cast<int>(blockIdx.x);
    const bool has_wide = b < parts.wide.tiles_m * parts.wide.tiles_n;
    if (has_wide) gemm_tile<F16, XT, WT, 2, 4, 8, 4>(parts.wide, b, lds);
    if (b < parts.narrow.tiles_m * parts.narrow.tiles_n) {
        if (has_wide) __syncthreads();   // every wavefront has read its part of the first tile out of LDS
        gemm_tile<F16, XT, WT, 4, 2, 4, 6>(parts.narrow, b, lds);
    }
}

// Tiles of 128 x 256 (2 x 4 wavefronts of 64 x 64), for products too small to
// give every CU a 256 x 256 tile: twice as many workgroups, each half the work.
template <bool F16, bool XT, bool WT>
__global__ __launch_bounds__(kThreads) void gemm16_low_tiles(const Part part) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    gemm_tile<F16, XT, WT, 2, 4, 4, 4>(part, blockIdx.x, lds);
}

typedef void (*LowKernel)(const Part);
const LowKernel kLowKernels[8] = {
    gemm16_low_tiles<false, false, false>, gemm16_low_tiles<false, false, true>, gemm16_low_tiles<false, true, false>, gemm16_low_tiles<false, true, true>,
    gemm16_low_tiles<true, false, false>,  gemm16_low_tiles<true, false, true>,  gemm16_low_tiles<true, true, false>,  gemm16_low_tiles<true, true, true>,
};

typedef void (*Kernel)(const Parts);
// index: 4 fp16 + 2 (x transposed) + (w transposed)
const Kernel kKernels[8] = {
    gemm16_tiles<false, false, false>, gemm16_tiles<false, false, true>, gemm16_tiles<false, true, false>, gemm16_tiles<false, true, true>,
    gemm16_tiles<true, false, false>,  gemm16_tiles<true, false, true>,  gemm16_tiles<true, true, false>,  gemm16_tiles<true, true, true>,
};

std::atomic<bool> lds_reserved[kMaxDevices][16];   // the dynamic LDS size of kKernels[i] (8 + i: kLowKernels[i]) has been raised on that device (first use, any thread)

// One operand of the product: element (row, k) at p[row * row_stride + k * k_stride],
// one of the strides being 1.
struct Operand {
    const uint16_t* p;
    int64_t row_stride, k_stride;
    bool transposed() const { return row_stride == 1 && k_stride != 1; }
    int64_t ld() const { return transposed() ? k_stride : row_stride; }
};

// What the kernel asks of an operand with `rows` rows; 0 or an error code.
int check_operand(const char* who, const char* name, const Operand& o, int64_t rows, int64_t K) {
    if (o.row_stride != 1 && o.k_stride != 1)
        return fail(DDL_E_UNSUPP, "%s: operand %s has no unit stride (row stride %lld, k stride %lld)", who, name, (long long)o.row_stride,
                    (long long)o.k_stride);
    const int64_t ld = o.ld();
    if (!aligned_to(o.p, 16) || ld % 8 != 0) return fail(DDL_E_ALIGN, "%s: operand %s must be 16-byte aligned with a pitch that is a multiple of 8", who, name);
    if (ld > 0x3FFFFF) return fail(DDL_E_UNSUPP, "%s: pitch of %s above 2^22 elements", who, name);   // 32-bit byte offsets inside a tile
    if (o.transposed()) {
        if (ld < rows) return fail(DDL_E_ARG, "%s: pitch %lld of %s below its %lld rows", who, (long long)ld, name, (long long)rows);
        if (rows % 8 != 0) return fail(DDL_E_ALIGN, "%s: %s is read along its rows, whose number must be a multiple of 8", who, name);
        if ((K + BK) * ld > 0x3FFFFFFF) return fail(DDL_E_UNSUPP, "%s: %s spans more than 2^31 bytes along k", who, name);
    } else {
        if (ld < K) return fail(DDL_E_ARG, "%s: pitch %lld of %s below K=%lld", who, (long long)ld, name, (long long)K);
        if (K % 8 != 0) return fail(DDL_E_ALIGN, "%s: %s is read along k, so K must be a multiple of 8", who, name);
        if (K > 0x3FFFFFFF) return fail(DDL_E_UNSUPP, "%s: K above 2^30", who);
    }
    return 0;
}

// y[M, N] = a[M, K] . b[N, K]^T + bias in 16-bit elements.
int gemm16(const char* who, bool f16, Operand a, Operand b, const uint16_t* bias, uint16_t* y, int64_t ldy, int64_t M, int64_t N, int64_t K,
           void* stream) {
    if (M < 0 || N < 0 || K < 0 || ldy < N)
        return fail(DDL_E_ARG, "%s: M=%lld N=%lld K=%lld ldy=%lld", who, (long long)M, (long long)N, (long long)K, (long long)ldy);
    if (M == 0 || N == 0) return 0;
    if (!a.p || !b.p || !y) return fail(DDL_E_ARG, "%s: null pointer", who);
    if (K == 0) return fail(DDL_E_UNSUPP, "%s: K = 0", who);
    if (int rc = check_operand(who, "a", a, M, K)) return rc;
    if (int rc = check_operand(who, "b", b, N, K)) return rc;
    if (!aligned_to(y, 2) || (bias && !aligned_to(bias, 2))) return fail(DDL_E_ALIGN, "%s: y / bias misaligned", who);
    // 2: rows of y can be stored 16 bytes at a time, 1: 8 bytes, 0: element by element
    const int vec_store = (ldy % 8 == 0 && aligned_to(y, 16)) ? 2 : (ldy % 4 == 0 && aligned_to(y, 8)) ? 1 : 0;
    const bool at = a.transposed(), bt = b.transposed();

    int dev = 0;
    const int cus = compute_units(dev);
    const int64_t tiles_m = (M + 255) / 256, cols = (N + 255) / 256;
    if (tiles_m > 0x7FFFFFll || cols > 0x7FFFFFll || tiles_m * (cols + 1) > 0x7FFFFFFFll)
        return fail(DDL_E_UNSUPP, "%s: too many output tiles", who);
    int64_t cost = 0;
    const int64_t wide_cols = wide_tile_columns(tiles_m, N, cus, &cost);
    // Columns [n_begin, n_begin + n_count) of the output with tiles of bm x bn.
    auto part = [&](int bm, int bn, int64_t n_begin, int64_t n_count) {
        Part p{};
        p.x = a.p, p.w = b.p + n_begin * b.row_stride, p.bias = bias ? bias + n_begin : nullptr, p.y = y + n_begin;
        p.M = M, p.N = n_count, p.K = K, p.ldx = a.ld(), p.ldw = b.ld(), p.ldy = ldy;
        p.tiles_m = static_cast<int>((M + bm - 1) / bm), p.tiles_n = static_cast<int>((n_count + bn - 1) / bn), p.vec_store = vec_store;
        return p;
    };
    const int k = (f16 ? 4 : 0) + (at ? 2 : 0) + (bt ? 1 : 0);
    auto reserve_lds = [&](int slot, const void* kernel) -> int {
        if (!lds_reserved[dev][slot].load(std::memory_order_acquire)) {   // the attribute sticks to the function on this device
            const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
            if (e != hipSuccess) return fail(static_cast<int>(e), "%s: cannot reserve %d bytes of LDS: %s", who, kLdsBytes, hipGetErrorString(e));
            lds_reserved[dev][slot].store(true, std::memory_order_release);
        }
        return 0;
    };
    // Tiles of half the height: twice the workgroups.  Taken when that shortens
    // the schedule by more than the 10 % a smaller tile loses in efficiency.
    const int64_t low_tiles = ((M + 127) / 128) * cols;
    const int64_t low_cost = (low_tiles + cus - 1) / cus * 128;
    if (low_cost * 11 < cost * 10) {
        if (int rc = reserve_lds(8 + k, reinterpret_cast<const void*>(kLowKernels[k]))) return rc;
        hipLaunchKernelGGL(kLowKernels[k], dim3(static_cast<uint32_t>(low_tiles)), dim3(kThreads), kLdsBytes, static_cast<hipStream_t>(stream),
                           part(128, 256, 0, N));
        return check_launch("gemm16_low_tiles");
    }
    Parts parts{};
    if (wide_cols > 0) parts.wide = part(256, 256, 0, wide_cols);
    if (wide_cols < N) parts.narrow = part(256, 192, wide_cols, N - wide_cols);
    const int n_wide = parts.wide.tiles_m * parts.wide.tiles_n, n_narrow = parts.narrow.tiles_m * parts.narrow.tiles_n;
    if (int rc = reserve_lds(k, reinterpret_cast<const void*>(kKernels[k]))) return rc;
    hipLaunchKernelGGL(kKernels[k], dim3(static_cast<uint32_t>(n_wide > n_narrow ? n_wide : n_narrow)), dim3(kThreads), kLdsBytes,
                       static_cast<hipStream_t>(stream), parts);
    return check_launch("gemm16_tiles");
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_gemm_f32(const float* a, int64_t a_row_stride, int64_t a_k_stride, const float* b, int64_t b_row_stride,
                            int64_t b_k_stride, const float* bias, float* y, int64_t ldy, int64_t M, int64_t N, int64_t K,
                            void* stream);

extern "C" int ddl_linear_bf16(const void* x, const void* w, const void* bias, void* y, int64_t M, int64_t N, int64_t K,
                               int64_t ldx, int64_t ldw, int64_t ldy, void* stream) {
    return ddl_linear(x, w, bias, y, DDL_DT_BF16, M, N, K, ldx, ldw, ldy, stream);
}

extern "C" int ddl_linear(const void* x, const void* w, const void* bias, void* y, int dtype, int64_t M, int64_t N, int64_t K,
                          int64_t ldx, int64_t ldw, int64_t ldy, void* stream) {
    using namespace ddl;
    if (dtype != DDL_DT_BF16 && dtype != DDL_DT_F16 && dtype != DDL_DT_F32)
        return fail(DDL_E_UNSUPP, "linear: dtype %d (bf16, f16 and f32 only)", dtype);
    if (ldx < K || ldw < K) return fail(DDL_E_ARG, "linear: ldx=%lld ldw=%lld below K=%lld", (long long)ldx, (long long)ldw, (long long)K);
    // A pitch of 1 would read as "contiguous along the rows" below; it can only belong to a K = 1 operand, which the 16-bit kernel refuses anyway.
    return ddl_gemm(x, ldx, 1, w, ldw, 1, bias, y, dtype, ldy, M, N, K, stream);
}

extern "C" int ddl_gemm(const void* a, int64_t a_row_stride, int64_t a_k_stride, const void* b, int64_t b_row_stride, int64_t b_k_stride,
                        const void* bias, void* y, int dtype, int64_t ldy, int64_t M, int64_t N, int64_t K, void* stream) {
    using namespace ddl;
    if (dtype == DDL_DT_F32)
        return ddl_gemm_f32(static_cast<const float*>(a), a_row_stride, a_k_stride, static_cast<const float*>(b), b_row_stride, b_k_stride,
                            static_cast<const float*>(bias), static_cast<float*>(y), ldy, M, N, K, stream);
    if (dtype != DDL_DT_BF16 && dtype != DDL_DT_F16) return fail(DDL_E_UNSUPP, "gemm: dtype %d (bf16, f16 and f32 only)", dtype);
    const Operand oa{static_cast<const uint16_t*>(a), a_row_stride, a_k_stride};
    const Operand ob{static_cast<const uint16_t*>(b), b_row_stride, b_k_stride};
    return gemm16("gemm", dtype == DDL_DT_F16, oa, ob, static_cast<const uint16_t*>(bias), static_cast<uint16_t*>(y), ldy, M, N, K, stream);
}
