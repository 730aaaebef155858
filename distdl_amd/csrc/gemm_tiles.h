// Pieces shared by the tiled MFMA GEMM kernels (16-bit and fp32 elements): the
// LDS ring of operand tiles, global -> LDS requests, the assignment of output
// tiles to workgroups, and the host's split of the output columns into wide and
// narrow tiles.
#ifndef DDL_GEMM_TILES_H
#define DDL_GEMM_TILES_H
#include "ddl_common.h"
#include <atomic>

namespace ddl {

constexpr int kRowBytes = 128;                           // one row of an operand tile in LDS: a k-tile is 128 bytes deep
constexpr int kMaxTileRows = 256;                        // rows of an operand tile: 256 of x; 256 or 192 of w
constexpr int kUnitBytes = kMaxTileRows * kRowBytes;     // ring slot for one operand tile, 32 KiB
constexpr int kUnits = 5;                                // ring of operand tiles: W0 X0 W1 X1 W2 | X2 W3 ...
constexpr int kLdsBytes = kUnits * kUnitBytes;           // 160 KiB: all of a CU's LDS
constexpr int kXcds = 8;
constexpr int kMaxDevices = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Raw buffer descriptor over all of memory from `base` on (no stride, no bounds).
__device__ inline u32x4 raw_buffer(const void* base) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    u32x4 r;
    r[0] = static_cast<uint32_t>(a), r[1] = static_cast<uint32_t>(a >> 32) & 0xFFFFu, r[2] = 0xFFFFFFFFu, r[3] = 0x00020000u;
    return r;
}

// One wavefront instruction: lane l copies the 16 bytes at byte (voffset +
// soffset) of the buffer to LDS byte (dst + 16 l); dst and soffset are the same
// for all lanes.  Written as assembly: the compiler makes every later LDS read
// through a transposing read wait for all such copies in flight (it cannot
// tell that they go to another ring slot), which would serialise the pipeline.
// The kernel waits for these copies itself (s_waitcnt vmcnt in front of the
// barriers); the compiler does not count them, which only makes its own waits
// for ordinary loads longer, never shorter (requests complete in order).
__device__ inline void dma16(u32x4 buffer, int voffset, int soffset, const char* dst) {
    const uint32_t lds_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(dst));   // low half of a generic LDS address: the LDS offset
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voffset), "s"(buffer), "s"(soffset)
                 : "memory", "m0");
}

// s_waitcnt immediate (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4,
// lgkmcnt 11:8): wait until at most n vector-memory requests are outstanding
// and all LDS reads have returned.
constexpr int wait_vm_lgkm0(int n) { return 0x0070 | (n & 15) | ((n >> 4) << 14); }

// The columns of the output that one kind of tile covers: operands and result
// already offset to the first of those columns.
template <typename E>
struct PartOf {
    const E* x;
    const E* w;
    const E* bias;
    E* y;
    int64_t M, N, K, ldx, ldw, ldy;
    int tiles_m, tiles_n, vec_store;
};

// The two kinds of tiles of one product.
template <typename E>
struct PartsOf {
    PartOf<E> wide;     // 256 x 256 tiles
    PartOf<E> narrow;   // 256 x 192 tiles
};

// XCD-aware tile assignment: hardware deals workgroup ids round-robin over the
// XCDs, so id % 8 names the XCD.  Each XCD gets a contiguous range of the tile
// sequence, which is walked in bands of 8 m-tiles, so that the workgroups
// resident on an XCD cover a compact patch of the tile grid.
__device__ inline void tile_of_workgroup(int id, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int ntiles = tiles_m * tiles_n;
    const int per = ntiles / kXcds, main = per * kXcds;
    if (id < main) id = (id % kXcds) * per + id / kXcds;
    constexpr int kBand = 8;
    const int band = id / (kBand * tiles_n);
    const int band_m0 = band * kBand;
    const int band_h = (tiles_m - band_m0) < kBand ? (tiles_m - band_m0) : kBand;
    const int in_band = id - band * kBand * tiles_n;
    tm = band_m0 + in_band % band_h;
    tn = in_band / band_h;
}

// Compute units of the current device (asked once per device; any thread may
// get there first, the value is the same for all).  `dev` receives the device.
inline int compute_units(int& dev) {
    static std::atomic<int> cu_count[kMaxDevices];   // 0: not asked yet
    dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
    int cus = cu_count[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        cus = n;
        cu_count[dev].store(n, std::memory_order_relaxed);
    }
    return cus;
}

// One workgroup per CU is resident, so the tiles run in rounds of one per CU
// and a last round that is only partly filled costs as much as a full one.
// How many of the N output columns go to 256-wide tiles (whole rounds of them;
// a multiple of 256, or N), the rest to 192-wide tiles, if that shortens the
// last round.  *cost receives the length of the schedule in tile columns
// (rounds of wide tiles x 256 + rounds of narrow tiles x 192).
inline int64_t wide_tile_columns(int64_t tiles_m, int64_t N, int cus, int64_t* cost = nullptr) {
    const int64_t cols = (N + 255) / 256;
    auto rounds = [&](int64_t tiles) { return (tiles + cus - 1) / cus; };
    int64_t best_cost = rounds(tiles_m * cols) * 256, best_split = cols;   // strips of 256 columns given to the wide tiles
    for (int64_t c = cols - 1; c >= 0 && c >= cols - 16; --c) {
        const int64_t rest = N - c * 256;
        const int64_t c_cost = rounds(tiles_m * c) * 256 + rounds(tiles_m * ((rest + 191) / 192)) * 192;
        if (c_cost < best_cost) {
            best_cost = c_cost;
            best_split = c;
        }
    }
    if (cost) *cost = best_cost;
    return best_split == cols ? N : best_split * 256;
}

}  // namespace ddl
#endif  // DDL_GEMM_TILES_H
