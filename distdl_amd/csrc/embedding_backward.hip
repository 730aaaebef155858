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
//   emb_bwd_fill     bucket[start[row] + cursor[row]++] = t
//   emb_bwd_reduce   sort each bucket (it is short), sum, convert, store
#include "ddl_common.h"

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

// Exclusive prefix sum of count[0..n) into start[0..n], start[n] = total.
__global__ __launch_bounds__(kScanBlock) void emb_bwd_scan(const int32_t* __restrict__ count, int64_t n, int32_t* __restrict__ start) {
    __shared__ int32_t part[kScanBlock];
    __shared__ int32_t carry_s;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    for (int64_t base = 0; base < n; base += kScanBlock) {
        const int64_t i = base + threadIdx.x;
        const int32_t v = i < n ? count[i] : 0;
        part[threadIdx.x] = v;
        __syncthreads();
        for (int off = 1; off < kScanBlock; off <<= 1) {     // Hillis-Steele inclusive scan
            const int32_t add = threadIdx.x >= static_cast<unsigned>(off) ? part[threadIdx.x - off] : 0;
            __syncthreads();
            part[threadIdx.x] += add;
            __syncthreads();
        }
        const int32_t carry = carry_s;
        if (i < n) start[i] = carry + part[threadIdx.x] - v;
        __syncthreads();
        if (threadIdx.x == kScanBlock - 1) carry_s = carry + part[kScanBlock - 1];
        __syncthreads();
    }
    if (threadIdx.x == 0) start[n] = carry_s;
}

template <typename IdT>
__global__ __launch_bounds__(kBlock) void emb_bwd_fill(const IdT* __restrict__ ids, int64_t n_ids, int64_t lo, int64_t hi,
                                                       int64_t padding_idx, const int32_t* __restrict__ start,
                                                       int32_t* __restrict__ cursor, int32_t* __restrict__ bucket) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (t >= n_ids) return;
    const int64_t r = token_row(ids, t, lo, hi, padding_idx);
    if (r >= 0) bucket[start[r] + atomicAdd(&cursor[r], 1)] = static_cast<int32_t>(t);
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

// Wavefront (row, chunk): columns chunk * kChunk + lane + 64 j, j = 0..7.
template <typename T>
__global__ __launch_bounds__(kBlock) void emb_bwd_reduce(const T* __restrict__ dy, int64_t dim, int64_t ld_dy,
                                                         const int32_t* __restrict__ start, int32_t* __restrict__ bucket,
                                                         int64_t rows, int chunks, T* __restrict__ dw, int64_t ld_dw) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t w = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t row = w / chunks;
    const int chunk = static_cast<int>(w - row * chunks);
    if (row >= rows) return;
    const int32_t b0 = start[row], n = start[row + 1] - b0;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const int64_t c0 = static_cast<int64_t>(chunk) * kChunk + lane;
    // Ascending token order makes the sum independent of how the fill kernel's
    // atomics interleaved.  Buckets of up to 64 tokens are ordered by rank (lane
    // i holds one token and counts the smaller ones); longer ones are taken as
    // they are.
    for (int32_t base = 0; base < n; base += kWave) {
        const int32_t m = n - base < kWave ? n - base : kWave;
        int32_t mine = lane < m ? bucket[b0 + base + lane] : 0x7FFFFFFF;
        if (n <= kWave) {
            int32_t rank = 0;
            for (int k = 0; k < m; ++k) rank += __shfl(mine, k, kWave) < mine ? 1 : 0;
            // scatter by rank: lane r reads the token whose rank is r
            int32_t sorted = 0x7FFFFFFF;
            for (int k = 0; k < m; ++k) {
                const int32_t tk = __shfl(mine, k, kWave), rk = __shfl(rank, k, kWave);
                if (rk == lane) sorted = tk;
            }
            mine = sorted;
        }
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
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int64_t c = c0 + 64 * j;
        if (c < dim) store_from_f32(dst + c, acc[j]);
    }
}

template <typename IdT>
int run(const void* dy, int dtype, int64_t dim, int64_t ld_dy, const IdT* ids, int64_t n_ids, int64_t lo, int64_t hi,
        int64_t padding_idx, void* dw, int64_t ld_dw, int32_t* ws, hipStream_t s) {
    const int64_t rows = hi - lo;
    int32_t* count = ws;                 // [rows]   -> reused as cursor after the scan
    int32_t* start = ws + rows;          // [rows + 1]
    int32_t* bucket = start + rows + 1;  // [n_ids]
    auto grid = [](int64_t n) { return dim3(static_cast<uint32_t>((n + kBlock - 1) / kBlock)); };
    hipLaunchKernelGGL(emb_bwd_clear, grid(rows), dim3(kBlock), 0, s, count, rows);
    if (n_ids > 0) hipLaunchKernelGGL((emb_bwd_count<IdT>), grid(n_ids), dim3(kBlock), 0, s, ids, n_ids, lo, hi, padding_idx, count);
    hipLaunchKernelGGL(emb_bwd_scan, dim3(1), dim3(kScanBlock), 0, s, count, rows, start);
    hipLaunchKernelGGL(emb_bwd_clear, grid(rows), dim3(kBlock), 0, s, count, rows);
    if (n_ids > 0)
        hipLaunchKernelGGL((emb_bwd_fill<IdT>), grid(n_ids), dim3(kBlock), 0, s, ids, n_ids, lo, hi, padding_idx, start, count, bucket);
    const int chunks = static_cast<int>((dim + kChunk - 1) / kChunk);
    const int64_t waves = rows * chunks;
    const dim3 rgrid(static_cast<uint32_t>((waves + kWavesPerBlock - 1) / kWavesPerBlock));
    if (dtype == DDL_DT_BF16)
        hipLaunchKernelGGL((emb_bwd_reduce<uint16_t>), rgrid, dim3(kBlock), 0, s, static_cast<const uint16_t*>(dy), dim, ld_dy,
                           start, bucket, rows, chunks, static_cast<uint16_t*>(dw), ld_dw);
    else
        hipLaunchKernelGGL((emb_bwd_reduce<float>), rgrid, dim3(kBlock), 0, s, static_cast<const float*>(dy), dim, ld_dy, start,
                           bucket, rows, chunks, static_cast<float*>(dw), ld_dw);
    return check_launch("embedding backward");
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_embedding_backward(const void* dy, int dtype, int64_t dim, int64_t ld_dy, const void* ids, int ids_is_i64,
                                      int64_t n_ids, int64_t lo, int64_t hi, int64_t padding_idx, void* dweight,
                                      int64_t ld_dw, int32_t* workspace, int64_t workspace_elems, void* stream) {
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
        return run(dy, dtype, dim, ld_dy, static_cast<const int64_t*>(ids), n_ids, lo, hi, padding_idx, dweight, ld_dw, workspace, s);
    return run(dy, dtype, dim, ld_dy, static_cast<const int32_t*>(ids), n_ids, lo, hi, padding_idx, dweight, ld_dw, workspace, s);
}
