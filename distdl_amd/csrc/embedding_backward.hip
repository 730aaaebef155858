// Backward of the DistributedEmbedding shard gather: the adjoint of
// torch.nn.functional.embedding on the local table (reference:
// nn/embedding.py:244-246),
//
//   dweight[r, :] = sum over the tokens t with ids[t] - lo == r of dy[t, :]
//
// for the rows r of the shard window [lo, hi); tokens outside the window and
// tokens equal to padding_idx contribute nothing.  No atomics on the gradient:
// the tokens are first bucketed by table row (a counting sort on 32-bit
// counters), then one wavefront per (row, column chunk) adds the dy rows of its
// bucket in fp32, in ascending token order, and writes every element of
// dweight exactly once -- rows nobody looked up get their zeros from the same
// pass, so dweight needs no clearing.
//
//   emb_bwd_clear    count = cursor = 0
//   emb_bwd_count    count[row]++ per token in the window
//   emb_bwd_fill     begin = exclusive prefix sum of count, formed by every workgroup for itself in LDS
//                    (no launch of its own, no kernel boundary to wait behind); bucket[begin[row] + cursor[row]++] = t
//   emb_bwd_reduce   a workgroup per row (or per few rows of a narrow table): buckets longer than a wavefront are put
//                    in ascending token order first (bitonic network over the workgroup), short ones in registers;
//                    then sum, scale, convert, store
//
// The order in which the fill kernel's atomics hand out bucket slots varies
// from run to run; both sorts exist so that the fp32 sums do not.  Tables of
// more rows than a workgroup's LDS holds counters for get their prefix sum from
// a kernel of its own (emb_bwd_scan) in front of the fill kernel.
#include "ddl_common.h"

#include <mutex>

// Workspace of ddl_embedding_backward_static: the counters, bucket cursors, bucket starts and
// token buckets of one call, for callers that cannot hand over (or allocate)
// device memory.  Every GPU the library runs on holds its own 4 MiB copy until
// the process ends; its device address is looked up once per device.
static __device__ __align__(256) int32_t scratch[DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS];

namespace ddl {
namespace {

constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kScanBlock = 1024;
constexpr int kChunk = 512;    // columns per wavefront of the reduce kernel: 8 per lane

__global__ __launch_bounds__(kBlock) void emb_bwd_clear(int32_t* __restrict__ p, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < n) p[i] = 0;
}

template <typename IdT>
__device__ inline int64_t token_row(const IdT* __restrict__ ids, int64_t t, int64_t lo, int64_t hi, int64_t padding_idx) {
    const int64_t id = static_cast<int64_t>(ids[t]);
    return (id >= lo && id < hi && id != padding_idx) ? id - lo : -1;
}

template <typename IdT>
__global__ __launch_bounds__(kBlock) void emb_bwd_count(const IdT* __restrict__ ids, int64_t n_ids, int64_t lo, int64_t hi,
                                                        int64_t padding_idx, int32_t* __restrict__ count) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (t >= n_ids) return;
    const int64_t r = token_row(ids, t, lo, hi, padding_idx);
    if (r >= 0) atomicAdd(&count[r], 1);
}

// Exclusive prefix sum of count[0..n) into start[0..n), one workgroup, 16384
// counters per round.  The counters come in and the sums go out with
// consecutive lanes on consecutive addresses; in between they sit in LDS, where
// a thread owns 16 consecutive ones (pitch 17 keeps the lanes on different
// banks).  Thread totals are scanned across the wavefront with shuffles, the 16
// wavefront totals through LDS.
constexpr int kScanItems = 16;
constexpr int kScanWaves = kScanBlock / kWave;
constexpr int kScanRound = kScanBlock * kScanItems;
__device__ inline int scan_slot(int i) { return i + (i >> 4); }
__global__ __launch_bounds__(kScanBlock) void emb_bwd_scan(const int32_t* __restrict__ count, int64_t n, int32_t* __restrict__ start) {
    __shared__ int32_t stage[kScanRound + kScanRound / 16];
    __shared__ int32_t wave_total[kScanWaves];
    const int t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
    int32_t carry = 0;                                         // sum of all earlier rounds, the same in every thread
    for (int64_t base = 0; base < n; base += kScanRound) {
#pragma unroll
        for (int j = 0; j < kScanItems; ++j) {
            const int i = j * kScanBlock + t;
            stage[scan_slot(i)] = base + i < n ? count[base + i] : 0;
        }
        __syncthreads();
        int32_t v[kScanItems];
        int32_t total = 0;
#pragma unroll
        for (int k = 0; k < kScanItems; ++k) {
            v[k] = stage[scan_slot(t * kScanItems + k)];
            total += v[k];
        }
        int32_t incl = total;                                  // inclusive scan over the wavefront
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const int32_t up = __shfl_up(incl, off, kWave);
            if (lane >= off) incl += up;
        }
        if (lane == kWave - 1) wave_total[wave] = incl;
        __syncthreads();
        int32_t before = 0, all = 0;
#pragma unroll
        for (int k = 0; k < kScanWaves; ++k) {
            const int32_t wt = wave_total[k];
            before += k < wave ? wt : 0;
            all += wt;
        }
        int32_t run = carry + before + incl - total;
#pragma unroll
        for (int k = 0; k < kScanItems; ++k) {
            stage[scan_slot(t * kScanItems + k)] = run;
            run += v[k];
        }
        carry += all;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kScanItems; ++j) {
            const int i = j * kScanBlock + t;
            if (base + i < n) start[base + i] = stage[scan_slot(i)];
        }
        __syncthreads();                                       // stage and wave_total are rewritten by the next round
    }
}

// Bucket fill.  SCAN: every workgroup forms the exclusive prefix sum of the
// counters for itself, in LDS (a thread owns ceil(rows / 1024) consecutive
// counters; thread totals are scanned across the wavefront with shuffles, the
// 16 wavefront totals through LDS), workgroup 0 also writes it to `begin` for the
// reduce kernel; otherwise `begin` has been filled by emb_bwd_scan.  A token's
// slot is begin[row] plus the number of tokens of that row that came before it
// in this run (an atomic counter per row, zero on entry).
constexpr int kFillBlock = 1024;
constexpr int kFillWaves = kFillBlock / kWave;
constexpr int64_t kFillScanRows = 32768;  // counters a workgroup scans in LDS (128 KiB)

template <typename IdT, bool SCAN>
__global__ __launch_bounds__(kFillBlock) void emb_bwd_fill(const IdT* __restrict__ ids, int64_t n_ids, int64_t lo, int64_t hi,
                                                           int64_t padding_idx, const int32_t* __restrict__ count,
                                                           int32_t* __restrict__ begin, int32_t* __restrict__ cursor,
                                                           int32_t* __restrict__ bucket) {
    // Counter i sits in slot i + i / per, per = counters per thread (a power of two): a thread walks consecutive slots,
    // the lanes of a wavefront are per + 1 slots apart and so on different banks.
    __shared__ int32_t base[SCAN ? kFillScanRows + kFillBlock : 1];
    __shared__ int32_t wave_total[kFillWaves];
    const int t = threadIdx.x, lane = t & (kWave - 1), wave = t / kWave;
    // The token's row and its place among the tokens of that row first: neither waits for the prefix sum.
    const int64_t tok = static_cast<int64_t>(blockIdx.x) * kFillBlock + t;
    const int64_t r = tok < n_ids ? token_row(ids, tok, lo, hi, padding_idx) : -1;
    const int32_t place = r >= 0 ? atomicAdd(&cursor[r], 1) : 0;
    int per_log = 0;
    if (SCAN) {
        const int32_t rows = static_cast<int32_t>(hi - lo);
        while ((kFillBlock << per_log) < rows) ++per_log;
        const int32_t per = 1 << per_log;
        for (int32_t i = t; i < rows; i += kFillBlock) base[i + (i >> per_log)] = count[i];
        __syncthreads();
        const int32_t i0 = t << per_log, i1 = i0 + per < rows ? i0 + per : rows;
        int32_t* const mine = base + i0 + t;                   // slot of counter i0
        int32_t total = 0;
        for (int32_t i = i0; i < i1; ++i) total += mine[i - i0];
        int32_t incl = total;                                  // inclusive scan over the wavefront
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const int32_t up = __shfl_up(incl, off, kWave);
            if (lane >= off) incl += up;
        }
        if (lane == kWave - 1) wave_total[wave] = incl;
        __syncthreads();
        int32_t before = 0, all = 0;
#pragma unroll
        for (int k = 0; k < kFillWaves; ++k) {
            const int32_t wt = wave_total[k];
            before += k < wave ? wt : 0;
            all += wt;
        }
        int32_t run = before + incl - total;
        for (int32_t i = i0; i < i1; ++i) {
            const int32_t c = mine[i - i0];
            mine[i - i0] = run;
            run += c;
        }
        __syncthreads();
        if (blockIdx.x == 0) {
            for (int32_t i = t; i < rows; i += kFillBlock) begin[i] = base[i + (i >> per_log)];
            if (t == 0) begin[rows] = all;
        }
    }
    if (r >= 0) bucket[(SCAN ? base[r + (r >> per_log)] : begin[r]) + place] = static_cast<int32_t>(tok);
}

// Ascending order of a bucket of more than 64 tokens, by the whole workgroup.
// The network is the bitonic sort in the form whose exchanges all put the
// smaller key first: partner of i is its mirror image inside blocks of k in the
// first pass of a merge, i + j in the others.  Keys beyond the end of the bucket
// count as +infinity and never move, so any length works.  Buckets of up to
// kSortLds tokens are sorted in LDS and written back, longer ones where they
// lie (a workgroup's stores are visible to its own later loads once the barrier
// between the passes has been passed; the loads are volatile so that none is
// served from a stale cache line).
constexpr int kSortLds = 4096;

template <typename P>
__device__ inline void bitonic_passes(P a, int32_t n) {
    int32_t pow2 = 1;
    while (pow2 < n) pow2 <<= 1;
    for (int32_t k = 2; k <= pow2; k <<= 1) {
        for (int32_t j = k >> 1; j > 0; j >>= 1) {
            const bool mirror = j == (k >> 1);
            for (int32_t t = threadIdx.x; t < (pow2 >> 1); t += kBlock) {
                int32_t i, l;
                if (mirror) {
                    const int32_t blk = t / j, off = t - blk * j;
                    i = blk * k + off;
                    l = blk * k + k - 1 - off;
                } else {
                    const int32_t blk = t / j, off = t - blk * j;
                    i = blk * 2 * j + off;
                    l = i + j;
                }
                if (l < n) {
                    const int32_t lo = a[i], hi = a[l];
                    if (lo > hi) {
                        a[i] = hi;
                        a[l] = lo;
                    }
                }
            }
            __syncthreads();
        }
    }
}

// Called by every thread of the workgroup with the same arguments.
__device__ inline void sort_bucket_long(int32_t* stage, int32_t* bucket, int32_t n) {
    if (n <= kSortLds) {
        for (int32_t i = threadIdx.x; i < n; i += kBlock) stage[i] = bucket[i];
        __syncthreads();
        bitonic_passes(stage, n);
        for (int32_t i = threadIdx.x; i < n; i += kBlock) bucket[i] = stage[i];
    } else {
        bitonic_passes(static_cast<volatile int32_t*>(bucket), n);
    }
    __syncthreads();   // the bucket is in order for every wavefront of the workgroup; stage may be refilled
}

// Elements: uint16_t holds bf16 bits, f16_bits fp16 bits; both are summed in fp32 and rounded once on the way out.
struct f16_bits {
    uint16_t u;
};
__device__ inline float f16_to_f32(uint16_t u) {
    _Float16 h;
    __builtin_memcpy(&h, &u, 2);
    return static_cast<float>(h);
}
__device__ inline uint16_t f32_to_f16(float f) {
    const _Float16 h = static_cast<_Float16>(f);
    uint16_t u;
    __builtin_memcpy(&u, &h, 2);
    return u;
}
__device__ inline float load_as_f32(const uint16_t* p) { return __uint_as_float(static_cast<uint32_t>(*p) << 16); }
__device__ inline float load_as_f32(const f16_bits* p) { return f16_to_f32(p->u); }
__device__ inline float load_as_f32(const float* p) { return *p; }

__device__ inline void store_from_f32(uint16_t* p, float f) {
    uint32_t u = __float_as_uint(f);
    uint16_t b = 0x7FC0;
    if (f == f) {
        u += 0x7FFFu + ((u >> 16) & 1u);
        b = static_cast<uint16_t>(u >> 16);
    }
    *p = b;
}
__device__ inline void store_from_f32(f16_bits* p, float f) { p->u = f32_to_f16(f); }
__device__ inline void store_from_f32(float* p, float f) { *p = f; }

// Order of the tokens of a bucket of at most 64: lane i holds one token and
// counts the smaller ones (its rank), then every lane picks the token whose
// rank is its own lane number.  Ascending token order makes the sums
// independent of how the fill kernel's atomics interleaved; longer buckets are
// put in order by sort_bucket_long.
__device__ inline int32_t sort_bucket(int32_t mine, int32_t m, int lane) {
    int32_t rank = 0;
    for (int k = 0; k < m; ++k) rank += __shfl(mine, k, kWave) < mine ? 1 : 0;
    int32_t sorted = 0x7FFFFFFF;
    for (int k = 0; k < m; ++k) {
        const int32_t tk = __shfl(mine, k, kWave), rk = __shfl(rank, k, kWave);
        if (rk == lane) sorted = tk;
    }
    return sorted;
}

// Both reduce kernels: a workgroup owns rows_per_block consecutive rows
// (one when a row has work for all four wavefronts, more for narrow tables).
// First its long buckets are sorted, one after the other, by all its threads;
// then wavefront w takes the items (row, group of columns) w, w + 4, ...
struct RowsOfBlock {
    int64_t row0;
    int n_rows;        // rows of this workgroup that exist
    int32_t n0, b0;    // tokens and first slot of row0 (fetched once: most workgroups own one row)
};
__device__ inline RowsOfBlock sort_long_buckets_of_block(const int32_t* __restrict__ count, const int32_t* __restrict__ begin,
                                                        int32_t* bucket, int64_t rows, int rows_per_block, int32_t* stage) {
    RowsOfBlock rb;
    rb.row0 = static_cast<int64_t>(blockIdx.x) * rows_per_block;
    const int64_t left = rows - rb.row0;
    rb.n_rows = left < rows_per_block ? static_cast<int>(left) : rows_per_block;
    rb.n0 = count[rb.row0];                                   // the grid has no workgroup without a row
    rb.b0 = begin[rb.row0];
    if (rb.n0 > kWave) sort_bucket_long(stage, bucket + rb.b0, rb.n0);
    for (int q = 1; q < rb.n_rows; ++q) {                     // the same trip count and branches in every thread
        const int32_t n = count[rb.row0 + q];
        if (n > kWave) sort_bucket_long(stage, bucket + begin[rb.row0 + q], n);
    }
    return rb;
}

// Tokens base .. base + 63 of a bucket, one per lane.  A bucket that this
// workgroup has just sorted is read around the vector cache.
__device__ inline int32_t bucket_tokens(const int32_t* bucket, int32_t b0, int32_t base, int32_t m, int32_t n, int lane) {
    if (lane >= m) return 0x7FFFFFFF;
    if (n > kWave) return *static_cast<const volatile int32_t*>(bucket + b0 + base + lane);
    return bucket[b0 + base + lane];
}

// Wavefront item (row, chunk): columns chunk * kChunk + lane + 64 j, j = 0..7.
template <typename T>
__global__ __launch_bounds__(kBlock) void emb_bwd_reduce(const T* __restrict__ dy, int64_t dim, int64_t ld_dy,
                                                         const int32_t* __restrict__ count, const int32_t* __restrict__ begin,
                                                         int32_t* bucket, int64_t rows, int chunks, int rows_per_block,
                                                         T* __restrict__ dw, int64_t ld_dw, int scale_by_freq) {
    __shared__ int32_t stage[kSortLds];
    const RowsOfBlock rb = sort_long_buckets_of_block(count, begin, bucket, rows, rows_per_block, stage);
    const int lane = threadIdx.x & (kWave - 1);
    for (int item = threadIdx.x / kWave; item < rb.n_rows * chunks; item += kWavesPerBlock) {
        const int q = item / chunks, chunk = item - q * chunks;
        const int64_t row = rb.row0 + q;
        const int32_t b0 = q ? begin[row] : rb.b0, n = q ? count[row] : rb.n0;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const int64_t c0 = static_cast<int64_t>(chunk) * kChunk + lane;
        for (int32_t base = 0; base < n; base += kWave) {
            const int32_t m = n - base < kWave ? n - base : kWave;
            int32_t mine = bucket_tokens(bucket, b0, base, m, n, lane);
            if (n <= kWave) mine = sort_bucket(mine, m, lane);
            for (int k = 0; k < m; ++k) {
                const int64_t t = __shfl(mine, k, kWave);
                const T* src = dy + t * ld_dy;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int64_t c = c0 + 64 * j;
                    if (c < dim) acc[j] += load_as_f32(src + c);
                }
            }
        }
        T* dst = dw + row * ld_dw;
        const float scale = (scale_by_freq && n > 1) ? 1.0f / static_cast<float>(n) : 1.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t c = c0 + 64 * j;
            if (c < dim) store_from_f32(dst + c, acc[j] * scale);
        }
    }
}

// The same for bf16 or fp16 (HALF) rows that can be moved 16 bytes at a time: a lane owns the
// eight consecutive columns chunk * kChunk + 8 lane .. + 7, so one load
// instruction of the wavefront covers a chunk, and an item is a group of CPW
// chunks of its row so that the loads of a token overlap and the walk through
// the bucket is paid once for all of them.
template <int CPW, bool HALF>
__global__ __launch_bounds__(kBlock) void emb_bwd_reduce_bf16x8(const uint16_t* __restrict__ dy, int64_t dim, int64_t ld_dy,
                                                                const int32_t* __restrict__ count, const int32_t* __restrict__ begin,
                                                                int32_t* bucket, int64_t rows, int groups, int rows_per_block,
                                                                uint16_t* __restrict__ dw, int64_t ld_dw, int scale_by_freq) {
    __shared__ int32_t stage[kSortLds];
    const RowsOfBlock rb = sort_long_buckets_of_block(count, begin, bucket, rows, rows_per_block, stage);
    const int lane = threadIdx.x & (kWave - 1);
    for (int item = threadIdx.x / kWave; item < rb.n_rows * groups; item += kWavesPerBlock) {
        const int q = item / groups, group = item - q * groups;
        const int64_t row = rb.row0 + q;
        const int32_t b0 = q ? begin[row] : rb.b0, n = q ? count[row] : rb.n0;
        float acc[CPW][8];
#pragma unroll
        for (int j = 0; j < CPW; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[j][e] = 0.f;
        const int64_t c0 = static_cast<int64_t>(group) * CPW * kChunk + lane * 8;   // dim is a multiple of 8 on this path
        for (int32_t base = 0; base < n; base += kWave) {
            const int32_t m = n - base < kWave ? n - base : kWave;
            int32_t mine = bucket_tokens(bucket, b0, base, m, n, lane);
            if (n <= kWave) mine = sort_bucket(mine, m, lane);
            for (int k = 0; k < m; ++k) {
                const int64_t t = __shfl(mine, k, kWave);
                const uint16_t* src = dy + t * ld_dy + c0;
                uint4 q[CPW];
#pragma unroll
                for (int j = 0; j < CPW; ++j) q[j] = c0 + j * kChunk < dim ? *reinterpret_cast<const uint4*>(src + j * kChunk) : make_uint4(0, 0, 0, 0);
#pragma unroll
                for (int j = 0; j < CPW; ++j) {
                    const uint32_t w4[4] = {q[j].x, q[j].y, q[j].z, q[j].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        acc[j][2 * e] += HALF ? f16_to_f32(static_cast<uint16_t>(w4[e])) : __uint_as_float(w4[e] << 16);
                        acc[j][2 * e + 1] += HALF ? f16_to_f32(static_cast<uint16_t>(w4[e] >> 16)) : __uint_as_float(w4[e] & 0xFFFF0000u);
                    }
                }
            }
        }
        uint16_t* dst = dw + row * ld_dw + c0;
        const float scale = (scale_by_freq && n > 1) ? 1.0f / static_cast<float>(n) : 1.0f;
#pragma unroll
        for (int j = 0; j < CPW; ++j) {
            if (c0 + j * kChunk >= dim) continue;
            uint16_t o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                if (HALF)
                    o[e] = f32_to_f16(acc[j][e] * scale);
                else
                    store_from_f32(&o[e], acc[j][e] * scale);
            }
            uint4 q;
            q.x = o[0] | (static_cast<uint32_t>(o[1]) << 16);
            q.y = o[2] | (static_cast<uint32_t>(o[3]) << 16);
            q.z = o[4] | (static_cast<uint32_t>(o[5]) << 16);
            q.w = o[6] | (static_cast<uint32_t>(o[7]) << 16);
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // streaming store: the gradient is not read again here
            u32x4 nv;
            nv[0] = q.x, nv[1] = q.y, nv[2] = q.z, nv[3] = q.w;
            __builtin_nontemporal_store(nv, reinterpret_cast<u32x4*>(dst + j * kChunk));
        }
    }
}

// Rows a workgroup of the reduce kernels takes: one when a row has items for
// all four wavefronts (or three), else as many as fill them.
inline int rows_per_block_for(int items_per_row) { return items_per_row >= 3 ? 1 : kWavesPerBlock / items_per_row; }

template <int CPW>
void launch_reduce_x8(const void* dy, int64_t dim, int64_t ld_dy, const int32_t* count, const int32_t* begin, int32_t* bucket,
                      int64_t rows, int chunks, void* dw, int64_t ld_dw, int scale_by_freq, bool half, hipStream_t s) {
    const int groups = (chunks + CPW - 1) / CPW;
    const int rpb = rows_per_block_for(groups);
    const dim3 grid(static_cast<uint32_t>((rows + rpb - 1) / rpb));
    if (half)
        hipLaunchKernelGGL((emb_bwd_reduce_bf16x8<CPW, true>), grid, dim3(kBlock), 0, s, static_cast<const uint16_t*>(dy), dim, ld_dy, count,
                           begin, bucket, rows, groups, rpb, static_cast<uint16_t*>(dw), ld_dw, scale_by_freq);
    else
        hipLaunchKernelGGL((emb_bwd_reduce_bf16x8<CPW, false>), grid, dim3(kBlock), 0, s, static_cast<const uint16_t*>(dy), dim, ld_dy, count,
                           begin, bucket, rows, groups, rpb, static_cast<uint16_t*>(dw), ld_dw, scale_by_freq);
}

template <typename IdT>
int run(const void* dy, int dtype, int64_t dim, int64_t ld_dy, const IdT* ids, int64_t n_ids, int64_t lo, int64_t hi,
        int64_t padding_idx, int scale_by_freq, void* dw, int64_t ld_dw, int32_t* ws, hipStream_t s) {
    const int64_t rows = hi - lo;
    int32_t* count = ws;                 // [rows]      tokens of each row
    int32_t* cursor = ws + rows;         // [rows]      slots of each bucket handed out so far
    int32_t* begin = cursor + rows;      // [rows + 1]  first slot of each bucket
    int32_t* bucket = begin + rows + 1;  // [n_ids]
    auto grid = [](int64_t n) { return dim3(static_cast<uint32_t>((n + kBlock - 1) / kBlock)); };
    hipLaunchKernelGGL(emb_bwd_clear, grid(2 * rows), dim3(kBlock), 0, s, count, 2 * rows);
    if (n_ids > 0) hipLaunchKernelGGL((emb_bwd_count<IdT>), grid(n_ids), dim3(kBlock), 0, s, ids, n_ids, lo, hi, padding_idx, count);
    const dim3 fgrid(static_cast<uint32_t>((n_ids + kFillBlock - 1) / kFillBlock));
    if (rows <= kFillScanRows) {
        // Without tokens one workgroup still runs: it writes `begin` (all zeros).
        hipLaunchKernelGGL((emb_bwd_fill<IdT, true>), n_ids > 0 ? fgrid : dim3(1), dim3(kFillBlock), 0, s, ids, n_ids, lo, hi, padding_idx,
                           count, begin, cursor, bucket);
    } else {
        hipLaunchKernelGGL(emb_bwd_scan, dim3(1), dim3(kScanBlock), 0, s, count, rows, begin);
        if (n_ids > 0)
            hipLaunchKernelGGL((emb_bwd_fill<IdT, false>), fgrid, dim3(kFillBlock), 0, s, ids, n_ids, lo, hi, padding_idx, count, begin,
                               cursor, bucket);
    }
    const int chunks = static_cast<int>((dim + kChunk - 1) / kChunk);
    const bool half = dtype == DDL_DT_F16;
    const bool vec = (dtype == DDL_DT_BF16 || half) && dim % 8 == 0 && ld_dy % 8 == 0 && ld_dw % 8 == 0 && aligned_to(dy, 16) && aligned_to(dw, 16);
    if (vec) {
        if (chunks >= 2) launch_reduce_x8<2>(dy, dim, ld_dy, count, begin, bucket, rows, chunks, dw, ld_dw, scale_by_freq, half, s);
        else launch_reduce_x8<1>(dy, dim, ld_dy, count, begin, bucket, rows, chunks, dw, ld_dw, scale_by_freq, half, s);
    } else {
        const int rpb = rows_per_block_for(chunks);
        const dim3 rgrid(static_cast<uint32_t>((rows + rpb - 1) / rpb));
        if (half)
            hipLaunchKernelGGL((emb_bwd_reduce<f16_bits>), rgrid, dim3(kBlock), 0, s, static_cast<const f16_bits*>(dy), dim, ld_dy, count,
                               begin, bucket, rows, chunks, rpb, static_cast<f16_bits*>(dw), ld_dw, scale_by_freq);
        else if (dtype == DDL_DT_BF16)
            hipLaunchKernelGGL((emb_bwd_reduce<uint16_t>), rgrid, dim3(kBlock), 0, s, static_cast<const uint16_t*>(dy), dim, ld_dy, count,
                               begin, bucket, rows, chunks, rpb, static_cast<uint16_t*>(dw), ld_dw, scale_by_freq);
        else
            hipLaunchKernelGGL((emb_bwd_reduce<float>), rgrid, dim3(kBlock), 0, s, static_cast<const float*>(dy), dim, ld_dy, count, begin,
                               bucket, rows, chunks, rpb, static_cast<float*>(dw), ld_dw, scale_by_freq);
    }
    return check_launch("embedding backward");
}

constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
int32_t* scratch_address[kMaxDevices] = {};   // device address of `scratch` on each GPU, filled on first use

// The device address of `scratch` on the current GPU.  In host code the name
// `scratch` is only a handle for the runtime, never a pointer a kernel may use.
int scratch_on_current_device(int32_t** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(static_cast<int>(e), "embedding backward (static): hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(DDL_E_UNSUPP, "embedding backward (static): device index %d (at most %d devices)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_address[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(e != hipSuccess ? static_cast<int>(e) : DDL_E_ARG, "embedding backward (static): hipGetSymbolAddress: %s", hipGetErrorString(e));
        scratch_address[dev] = static_cast<int32_t*>(p);
    }
    *out = scratch_address[dev];
    return 0;
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_embedding_backward_static(const void* dy, int dtype, int64_t dim, int64_t ld_dy, const void* ids, int ids_is_i64,
                                             int64_t n_ids, int64_t lo, int64_t hi, int64_t padding_idx, int scale_grad_by_freq,
                                             void* dweight, int64_t ld_dw, void* stream) {
    using namespace ddl;
    if (n_ids < 0 || hi < lo) return fail(DDL_E_ARG, "embedding backward (static): n_ids=%lld window=[%lld,%lld)", (long long)n_ids, (long long)lo, (long long)hi);
    const int64_t rows = hi - lo;
    // compared without forming 2 rows + 1 + n_ids, which could overflow
    if (rows > DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS || n_ids > DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS ||
        3 * rows + 1 + n_ids > DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS)
        return fail(DDL_E_UNSUPP,
                    "embedding backward (static): 3 * %lld rows + 1 + %lld tokens exceeds the built-in workspace of %lld int32; "
                    "use ddl_embedding_backward with a workspace of your own", (long long)rows, (long long)n_ids,
                    (long long)DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS);
    int32_t* ws = nullptr;
    const int rc = scratch_on_current_device(&ws);
    if (rc) return rc;
    return ddl_embedding_backward(dy, dtype, dim, ld_dy, ids, ids_is_i64, n_ids, lo, hi, padding_idx, scale_grad_by_freq, dweight,
                                  ld_dw, ws, DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS, stream);
}

extern "C" int ddl_embedding_backward(const void* dy, int dtype, int64_t dim, int64_t ld_dy, const void* ids, int ids_is_i64,
                                      int64_t n_ids, int64_t lo, int64_t hi, int64_t padding_idx, int scale_grad_by_freq,
                                      void* dweight, int64_t ld_dw, int32_t* workspace, int64_t workspace_elems, void* stream) {
    using namespace ddl;
    if (dim < 0 || ld_dy < dim || ld_dw < dim || n_ids < 0 || hi < lo)
        return fail(DDL_E_ARG, "embedding backward: dim=%lld ld_dy=%lld ld_dw=%lld n_ids=%lld window=[%lld,%lld)", (long long)dim,
                    (long long)ld_dy, (long long)ld_dw, (long long)n_ids, (long long)lo, (long long)hi);
    if (dtype != DDL_DT_BF16 && dtype != DDL_DT_F16 && dtype != DDL_DT_F32)
        return fail(DDL_E_UNSUPP, "embedding backward: dtype %d (bf16, f16 and f32 only)", dtype);
    const int64_t rows = hi - lo;
    if (rows == 0 || dim == 0) return 0;
    if (n_ids > 0x7FFFFFFFll || rows > 0x3FFFFFFFll) return fail(DDL_E_UNSUPP, "embedding backward: more than 2^31 tokens or 2^30 rows");
    if (!dweight || !workspace || (n_ids > 0 && (!dy || !ids))) return fail(DDL_E_ARG, "embedding backward: null pointer");
    const int es = dtype == DDL_DT_F32 ? 4 : 2;
    if (!aligned_to(dy, es) || !aligned_to(dweight, es) || !aligned_to(workspace, 4) || !aligned_to(ids, ids_is_i64 ? 8 : 4))
        return fail(DDL_E_ALIGN, "embedding backward: pointer misaligned");
    const int64_t need = 3 * rows + 1 + n_ids;
    if (workspace_elems < need)
        return fail(DDL_E_ARG, "embedding backward: workspace of %lld int32 is smaller than the %lld needed (3 rows + 1 + tokens)",
                    (long long)workspace_elems, (long long)need);
    const int64_t chunks = (dim + kChunk - 1) / kChunk;
    if (rows >= 0x7FFFFFFFll || chunks > 0xFFFFFF) return fail(DDL_E_UNSUPP, "embedding backward: too many workgroups or columns");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (ids_is_i64)
        return run(dy, dtype, dim, ld_dy, static_cast<const int64_t*>(ids), n_ids, lo, hi, padding_idx, scale_grad_by_freq != 0, dweight,
                   ld_dw, workspace, s);
    return run(dy, dtype, dim, ld_dy, static_cast<const int32_t*>(ids), n_ids, lo, hi, padding_idx, scale_grad_by_freq != 0, dweight, ld_dw,
               workspace, s);
}
