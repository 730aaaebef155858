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
//   emb_bwd_clear    counters = 0
//   emb_bwd_count    count[row]++ per token in the window
//   emb_bwd_scan     start[row] = exclusive prefix sum of count (one workgroup)
//   emb_bwd_fill     bucket[start[row]++] = t, which leaves start[row] at the bucket's end
//   emb_bwd_sort     buckets longer than a wavefront: ascending token order (bitonic network)
//   emb_bwd_reduce   order the short buckets in registers, sum, scale, convert, store
//
// The order in which the fill kernel's atomics hand out bucket slots varies
// from run to run; both sorts exist so that the fp32 sums do not.
#include "ddl_common.h"

#include <mutex>

// Workspace of ddl_embedding_backward_static: the counters, bucket starts and
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

template <typename IdT>
__global__ __launch_bounds__(kBlock) void emb_bwd_fill(const IdT* __restrict__ ids, int64_t n_ids, int64_t lo, int64_t hi,
                                                       int64_t padding_idx, int32_t* __restrict__ start,
                                                       int32_t* __restrict__ bucket) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (t >= n_ids) return;
    const int64_t r = token_row(ids, t, lo, hi, padding_idx);
    if (r >= 0) bucket[atomicAdd(&start[r], 1)] = static_cast<int32_t>(t);   // start[r] ends as the end of bucket r
}

// Buckets of more than 64 tokens, sorted ascending in place.  Thread t of a
// workgroup looks at row blockIdx.x * kBlock + t; the rows of the workgroup
// that need sorting (few: tokens looked up that often are rare) are then taken
// one after the other by the whole workgroup.  The network is the bitonic sort
// in the form whose exchanges all put the smaller key first: partner of i is
// its mirror image inside blocks of k in the first pass of a merge, i + j in
// the others.  Keys beyond the end of the bucket count as +infinity and never
// move, so any length works.  Buckets of up to kSortLds tokens are sorted in
// LDS, longer ones where they lie (a workgroup's stores are visible to its own
// later loads once the barrier between the passes has been passed; the loads
// are volatile so that none is served from a stale cache line).
constexpr int kSortLds = 8192;

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

__global__ __launch_bounds__(kBlock) void emb_bwd_sort_long(const int32_t* __restrict__ start, int32_t* bucket, int64_t rows) {
    __shared__ int32_t stage[kSortLds];
    __shared__ int32_t todo[kBlock];
    __shared__ int32_t n_todo;
    if (threadIdx.x == 0) n_todo = 0;
    __syncthreads();
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (r < rows) {
        const int32_t b0 = r ? start[r - 1] : 0;
        if (start[r] - b0 > kWave) todo[atomicAdd(&n_todo, 1)] = static_cast<int32_t>(threadIdx.x);
    }
    __syncthreads();
    const int32_t cnt = n_todo;
    for (int32_t q = 0; q < cnt; ++q) {
        const int64_t row = static_cast<int64_t>(blockIdx.x) * kBlock + todo[q];
        const int32_t b0 = row ? start[row - 1] : 0, n = start[row] - b0;
        if (n <= kSortLds) {
            for (int32_t i = threadIdx.x; i < n; i += kBlock) stage[i] = bucket[b0 + i];
            __syncthreads();
            bitonic_passes(stage, n);
            for (int32_t i = threadIdx.x; i < n; i += kBlock) bucket[b0 + i] = stage[i];
            __syncthreads();   // stage is refilled for the next row
        } else {
            __syncthreads();
            bitonic_passes(static_cast<volatile int32_t*>(bucket + b0), n);
        }
    }
}

__device__ inline float load_as_f32(const uint16_t* p) { return __uint_as_float(static_cast<uint32_t>(*p) << 16); }
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
__device__ inline void store_from_f32(float* p, float f) { *p = f; }

// Order of the tokens of a bucket of at most 64: lane i holds one token and
// counts the smaller ones (its rank), then every lane picks the token whose
// rank is its own lane number.  Ascending token order makes the sums
// independent of how the fill kernel's atomics interleaved; longer buckets have
// been put in order by emb_bwd_sort_long.
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

// Wavefront (row, chunk): columns chunk * kChunk + lane + 64 j, j = 0..7.
template <typename T>
__global__ __launch_bounds__(kBlock) void emb_bwd_reduce(const T* __restrict__ dy, int64_t dim, int64_t ld_dy,
                                                         const int32_t* __restrict__ start, const int32_t* __restrict__ bucket,
                                                         int64_t rows, int chunks, T* __restrict__ dw, int64_t ld_dw,
                                                         int scale_by_freq) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t w = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t row = w / chunks;
    const int chunk = static_cast<int>(w - row * chunks);
    if (row >= rows) return;
    const int32_t b0 = row ? start[row - 1] : 0, n = start[row] - b0;   // the fill pass moved start[r] to the end of bucket r
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const int64_t c0 = static_cast<int64_t>(chunk) * kChunk + lane;
    for (int32_t base = 0; base < n; base += kWave) {
        const int32_t m = n - base < kWave ? n - base : kWave;
        int32_t mine = lane < m ? bucket[b0 + base + lane] : 0x7FFFFFFF;
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

// The same for bf16 rows that can be moved 16 bytes at a time: a lane owns the
// eight consecutive columns chunk * kChunk + 8 lane .. + 7, so one load
// instruction of the wavefront covers a chunk, and a wavefront takes CPW
// chunks of its row so that the loads of a token overlap and the walk through
// start and bucket is paid once for all of them.
template <int CPW>
__global__ __launch_bounds__(kBlock) void emb_bwd_reduce_bf16x8(const uint16_t* __restrict__ dy, int64_t dim, int64_t ld_dy,
                                                                const int32_t* __restrict__ start, const int32_t* __restrict__ bucket,
                                                                int64_t rows, int groups, uint16_t* __restrict__ dw, int64_t ld_dw,
                                                                int scale_by_freq) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t w = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t row = w / groups;
    const int group = static_cast<int>(w - row * groups);
    if (row >= rows) return;
    const int32_t b0 = row ? start[row - 1] : 0, n = start[row] - b0;   // the fill pass moved start[r] to the end of bucket r
    float acc[CPW][8];
#pragma unroll
    for (int j = 0; j < CPW; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[j][e] = 0.f;
    const int64_t c0 = static_cast<int64_t>(group) * CPW * kChunk + lane * 8;   // dim is a multiple of 8 on this path
    for (int32_t base = 0; base < n; base += kWave) {
        const int32_t m = n - base < kWave ? n - base : kWave;
        int32_t mine = lane < m ? bucket[b0 + base + lane] : 0x7FFFFFFF;
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
                    acc[j][2 * e] += __uint_as_float(w4[e] << 16);
                    acc[j][2 * e + 1] += __uint_as_float(w4[e] & 0xFFFF0000u);
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
        for (int e = 0; e < 8; ++e) store_from_f32(&o[e], acc[j][e] * scale);
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

template <int CPW>
void launch_reduce_x8(const void* dy, int64_t dim, int64_t ld_dy, const int32_t* start, const int32_t* bucket, int64_t rows, int chunks,
                      void* dw, int64_t ld_dw, int scale_by_freq, hipStream_t s) {
    const int groups = (chunks + CPW - 1) / CPW;
    const int64_t waves = rows * groups;
    hipLaunchKernelGGL((emb_bwd_reduce_bf16x8<CPW>), dim3(static_cast<uint32_t>((waves + kWavesPerBlock - 1) / kWavesPerBlock)),
                       dim3(kBlock), 0, s, static_cast<const uint16_t*>(dy), dim, ld_dy, start, bucket, rows, groups,
                       static_cast<uint16_t*>(dw), ld_dw, scale_by_freq);
}

template <typename IdT>
int run(const void* dy, int dtype, int64_t dim, int64_t ld_dy, const IdT* ids, int64_t n_ids, int64_t lo, int64_t hi,
        int64_t padding_idx, int scale_by_freq, void* dw, int64_t ld_dw, int32_t* ws, hipStream_t s) {
    const int64_t rows = hi - lo;
    int32_t* count = ws;                 // [rows]
    int32_t* start = ws + rows;          // [rows + 1]: begin of each bucket, advanced to its end by the fill pass
    int32_t* bucket = start + rows + 1;  // [n_ids]
    auto grid = [](int64_t n) { return dim3(static_cast<uint32_t>((n + kBlock - 1) / kBlock)); };
    hipLaunchKernelGGL(emb_bwd_clear, grid(rows), dim3(kBlock), 0, s, count, rows);
    if (n_ids > 0) hipLaunchKernelGGL((emb_bwd_count<IdT>), grid(n_ids), dim3(kBlock), 0, s, ids, n_ids, lo, hi, padding_idx, count);
    hipLaunchKernelGGL(emb_bwd_scan, dim3(1), dim3(kScanBlock), 0, s, count, rows, start);
    if (n_ids > 0)
        hipLaunchKernelGGL((emb_bwd_fill<IdT>), grid(n_ids), dim3(kBlock), 0, s, ids, n_ids, lo, hi, padding_idx, start, bucket);
    if (n_ids > kWave) hipLaunchKernelGGL(emb_bwd_sort_long, grid(rows), dim3(kBlock), 0, s, start, bucket, rows);
    const int chunks = static_cast<int>((dim + kChunk - 1) / kChunk);
    const int64_t waves = rows * chunks;
    const dim3 rgrid(static_cast<uint32_t>((waves + kWavesPerBlock - 1) / kWavesPerBlock));
    const bool vec = dtype == DDL_DT_BF16 && dim % 8 == 0 && ld_dy % 8 == 0 && ld_dw % 8 == 0 && aligned_to(dy, 16) && aligned_to(dw, 16);
    if (vec) {
        if (chunks >= 2) launch_reduce_x8<2>(dy, dim, ld_dy, start, bucket, rows, chunks, dw, ld_dw, scale_by_freq, s);
        else launch_reduce_x8<1>(dy, dim, ld_dy, start, bucket, rows, chunks, dw, ld_dw, scale_by_freq, s);
    } else if (dtype == DDL_DT_BF16)
        hipLaunchKernelGGL((emb_bwd_reduce<uint16_t>), rgrid, dim3(kBlock), 0, s, static_cast<const uint16_t*>(dy), dim, ld_dy,
                           start, bucket, rows, chunks, static_cast<uint16_t*>(dw), ld_dw, scale_by_freq);
    else
        hipLaunchKernelGGL((emb_bwd_reduce<float>), rgrid, dim3(kBlock), 0, s, static_cast<const float*>(dy), dim, ld_dy, start,
                           bucket, rows, chunks, static_cast<float*>(dw), ld_dw, scale_by_freq);
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
        2 * rows + 1 + n_ids > DDL_EMBEDDING_BACKWARD_STATIC_MAX_ELEMS)
        return fail(DDL_E_UNSUPP,
                    "embedding backward (static): 2 * %lld rows + 1 + %lld tokens exceeds the built-in workspace of %lld int32; "
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
    if (dtype != DDL_DT_BF16 && dtype != DDL_DT_F32) return fail(DDL_E_UNSUPP, "embedding backward: dtype %d (bf16 and f32 only)", dtype);
    const int64_t rows = hi - lo;
    if (rows == 0 || dim == 0) return 0;
    if (n_ids > 0x7FFFFFFFll || rows > 0x3FFFFFFFll) return fail(DDL_E_UNSUPP, "embedding backward: more than 2^31 tokens or 2^30 rows");
    if (!dweight || !workspace || (n_ids > 0 && (!dy || !ids))) return fail(DDL_E_ARG, "embedding backward: null pointer");
    const int es = dtype == DDL_DT_BF16 ? 2 : 4;
    if (!aligned_to(dy, es) || !aligned_to(dweight, es) || !aligned_to(workspace, 4) || !aligned_to(ids, ids_is_i64 ? 8 : 4))
        return fail(DDL_E_ALIGN, "embedding backward: pointer misaligned");
    const int64_t need = 2 * rows + 1 + n_ids;
    if (workspace_elems < need)
        return fail(DDL_E_ARG, "embedding backward: workspace of %lld int32 is smaller than the %lld needed (2 rows + 1 + tokens)",
                    (long long)workspace_elems, (long long)need);
    const int64_t chunks = (dim + kChunk - 1) / kChunk;
    if (rows * chunks / kWavesPerBlock >= 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "embedding backward: too many workgroups");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (ids_is_i64)
        return run(dy, dtype, dim, ld_dy, static_cast<const int64_t*>(ids), n_ids, lo, hi, padding_idx, scale_grad_by_freq != 0, dweight,
                   ld_dw, workspace, s);
    return run(dy, dtype, dim, ld_dy, static_cast<const int32_t*>(ids), n_ids, lo, hi, padding_idx, scale_grad_by_freq != 0, dweight, ld_dw,
               workspace, s);
}
