// DistributedLayerNorm, local shard (reference: nn/layernorm.py:218-247,
// 295-321).  Elements are fp32, bf16 or fp16; every sum is fp32.
//
//   ln_stats     x[rows, cols] -> {mean_r, M2_r} per row     (one read of x)
//   ln_normalize gathered {mean_p, M2_p} of the P workers sharing a row
//                -> combined mean / var -> y = (x-mean)*rstd*gamma+beta
//   ln_fused     both in one launch, for rows that one worker holds whole
//                (the reference's torch.nn.functional.layer_norm branch, :310-319)
//   ln_joined    both in one launch for rows shared with other workers whose
//                {mean, M2} are in memory before the launch: the row stays in
//                registers between the two halves, so x is read once
//
// Three ways of holding a row, chosen by its length:
//   wavefront rows  up to 2048 columns: one wavefront owns a row, each lane
//                   holds pieces of four elements, sums go through shuffle
//                   butterflies; a long input keeps two rows per wavefront in
//                   flight
//   workgroup rows  up to 16384 columns: a 256-thread workgroup owns a row, still
//                   in registers (up to 16 pieces of four per thread), sums go
//                   through the wavefronts and four words of LDS
//   streamed rows   anything longer, or rows whose length, pitch or address
//                   rule out four-element accesses: a workgroup walks the row
//                   once per reduction
#include "ddl_common.h"

#include "ln_elements.h"

namespace ddl {
namespace {

constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kMaxParts = 256;
constexpr int kWaveRowCols = 2048;     // longest row a wavefront keeps in registers
constexpr int kBlockRowCols = 16384;   // longest row a workgroup keeps in registers

struct PartCounts {
    float inv_n[kMaxParts];  // 1 / columns held by worker p
};

__device__ inline float sum4(float4 v) { return (v.x + v.y) + (v.z + v.w); }
__device__ inline float sq4(float4 v, float m) {
    const float a = v.x - m, b = v.y - m, c = v.z - m, d = v.w - m;
    return (a * a + b * b) + (c * c + d * d);
}
__device__ inline float4 norm4(float4 v, float mean, float rstd) {
    return make_float4((v.x - mean) * rstd, (v.y - mean) * rstd, (v.z - mean) * rstd, (v.w - mean) * rstd);
}
__device__ inline float4 affine4(float4 g, float4 o, float4 b) {
    return make_float4(g.x * o.x + b.x, g.y * o.y + b.y, g.z * o.z + b.z, g.w * o.w + b.w);
}

// Sum over the workgroup, the same value in every thread.  `scratch` holds one
// float per wavefront; the leading barrier lets it be reused call after call.
__device__ inline float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) t += scratch[w];
    return t;
}

// Mean-of-local-means / mean-of-local-variances of nn/layernorm.py:230-247,
// written on the gathered {mean_p, M2_p}:
//   mean((x-mean)^2 over worker p) = (M2_p + n_p (mean_p-mean)^2) / n_p.
// A whole wavefront works on one row: lane p holds worker p's pair (`first`,
// loaded by the caller so that it travels together with the row itself; zeros
// for lanes >= nparts) and 1/n_p; workers beyond the 64th are fetched here.
__device__ inline float2 load_part(const float* __restrict__ part_stats, int64_t rows, int64_t r, int p) {
    return reinterpret_cast<const float2*>(part_stats)[static_cast<int64_t>(p) * rows + r];
}

__device__ inline void combine_parts(const float* __restrict__ part_stats, int64_t rows, int64_t r, int nparts,
                                     const PartCounts& pc, float eps, int lane, float2 first, float first_inv_n,
                                     float* mean_out, float* rstd_out) {
    float msum = lane < nparts ? first.x : 0.f;
    for (int p = lane + kWave; p < nparts; p += kWave) msum += load_part(part_stats, rows, r, p).x;
    const float mean = wave_sum(msum) / static_cast<float>(nparts);
    float vsum = 0.f;
    if (lane < nparts) {
        const float d = first.x - mean;
        vsum = first.y * first_inv_n + d * d;
    }
    for (int p = lane + kWave; p < nparts; p += kWave) {
        const float2 s = load_part(part_stats, rows, r, p);
        const float d = s.x - mean;
        vsum += s.y * pc.inv_n[p] + d * d;
    }
    const float var = wave_sum(vsum) / static_cast<float>(nparts);
    *mean_out = mean;
    *rstd_out = 1.0f / sqrtf(var + eps);
}

// What the three kernels of a family do with a row once its statistics exist.
enum Mode {
    kStats = 0,   // emit {mean, M2} of the local columns
    kNorm = 1,    // statistics come from the gathered pairs
    kFused = 2,   // statistics of the local columns are the row's statistics
    kJoined = 3,  // emit {mean, M2} of the local columns, take the other workers' pairs from memory, normalise
};

struct LnArgs {
    const void* x;
    void* y;
    const void* gamma;
    const void* beta;
    const float* part_stats;
    float* stats;
    float* mean_out;
    float* rstd_out;
    int64_t rows, ld, ldy;
    int cols;
    int nparts;
    int my_part;   // kJoined: this worker's place among the nparts
    float eps;
};

// --------------------------------------------------------- wavefront rows --

// One wavefront per row, NV pieces of four per lane (cols <= 256 NV, cols % 4
// == 0), RPW rows of a wavefront in flight at once.
template <typename T, int NV, int RPW, int MODE, bool AFFINE>
__global__ __launch_bounds__(kBlock) void ln_wave_rows(const void* x_first, int64_t rows_first, int64_t ld_first, int cols_first,
                                                       const LnArgs a_rest, const PartCounts pc) {
    // The leading arguments repeat four fields of the block that follows: plain
    // leading arguments arrive in scalar registers with the wavefront (kernel
    // argument preload), so the loads of the row can be issued without waiting
    // for a first fetch from the argument block -- 0.35 us of a 4 us kernel.
    LnArgs a = a_rest;
    a.x = x_first, a.rows = rows_first, a.ld = ld_first, a.cols = cols_first;
    const T* __restrict__ x = static_cast<const T*>(a.x);
    T* __restrict__ y = static_cast<T*>(a.y);
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t r0 = wave * RPW;
    const int64_t rows = a.rows;
    const int nv = a.cols >> 2;
    float4 g[NV], b[NV];
    if (MODE != kStats && AFFINE) {
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = lane + k * kWave;
            if (c < nv) {
                g[k] = load4(static_cast<const T*>(a.gamma) + 4 * c);
                b[k] = load4(static_cast<const T*>(a.beta) + 4 * c);
            }
        }
    }
    // Everything this wavefront reads is requested before anything is used:
    // the gathered statistics of its rows (lane p fetches worker p's pair) and
    // the rows themselves.
    float2 ps[RPW];
    float inv_n = 0.f;
    if (MODE == kNorm || MODE == kJoined) {
        inv_n = lane < a.nparts ? pc.inv_n[lane] : 0.f;
#pragma unroll
        for (int i = 0; i < RPW; ++i) {
            const int64_t r = r0 + i;
            ps[i] = (r < rows && lane < a.nparts) ? load_part(a.part_stats, rows, r, lane) : make_float2(0.f, 0.f);
        }
    }
    float4 v[RPW][NV];
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        const int64_t r = r0 + i;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = lane + k * kWave;
            v[i][k] = (r < rows && c < nv) ? load4(x + r * a.ld + 4 * c) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    const float inv = 1.0f / static_cast<float>(a.cols);
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        const int64_t r = r0 + i;
        if (r >= rows) continue;   // the whole wavefront takes the same branch
        float mean, rstd;
        if (MODE == kNorm) {
            combine_parts(a.part_stats, rows, r, a.nparts, pc, a.eps, lane, ps[i], inv_n, &mean, &rstd);
        } else {
            float s = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k) s += sum4(v[i][k]);
            mean = wave_sum(s) * inv;
            float q = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k)
                if (lane + k * kWave < nv) q += sq4(v[i][k], mean);
            q = wave_sum(q);
            if (MODE == kStats || MODE == kJoined) {
                if (lane == 0) reinterpret_cast<float2*>(a.stats)[r] = make_float2(mean, q);
                if (MODE == kStats) continue;
            }
            if (MODE == kJoined)   // this worker's pair comes from the registers, the others' from memory (nparts <= 64)
                combine_parts(a.part_stats, rows, r, a.nparts, pc, a.eps, lane, lane == a.my_part ? make_float2(mean, q) : ps[i],
                              inv_n, &mean, &rstd);
            else
                rstd = 1.0f / sqrtf(q * inv + a.eps);
        }
        if (lane == 0) {
            if (a.mean_out) a.mean_out[r] = mean;
            if (a.rstd_out) a.rstd_out[r] = rstd;
        }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = lane + k * kWave;
            if (c < nv) {
                float4 o = norm4(v[i][k], mean, rstd);
                if (AFFINE) o = affine4(g[k], o, b[k]);
                store4(y + r * a.ldy + 4 * c, o);
            }
        }
    }
}

// --------------------------------------------------------- workgroup rows --

// One workgroup per row, NV pieces of four per thread (cols <= 1024 NV, cols
// % 4 == 0); the grid walks the rows.
template <typename T, int NV, int MODE, bool AFFINE>
__global__ __launch_bounds__(kBlock) void ln_block_rows(const LnArgs a, const PartCounts pc) {
    __shared__ float scratch[kWavesPerBlock];
    const T* __restrict__ x = static_cast<const T*>(a.x);
    T* __restrict__ y = static_cast<T*>(a.y);
    const int t = threadIdx.x, lane = t & (kWave - 1);
    const int nv = a.cols >> 2;
    const float inv = 1.0f / static_cast<float>(a.cols);
    for (int64_t r = blockIdx.x; r < a.rows; r += gridDim.x) {
        float2 first = make_float2(0.f, 0.f);
        if ((MODE == kNorm || MODE == kJoined) && lane < a.nparts) first = load_part(a.part_stats, a.rows, r, lane);
        float4 v[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = t + k * kBlock;
            v[k] = c < nv ? load4(x + r * a.ld + 4 * c) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float mean, rstd;
        if (MODE == kNorm) {
            // every wavefront combines the pairs for itself: no exchange needed
            combine_parts(a.part_stats, a.rows, r, a.nparts, pc, a.eps, lane, first, lane < a.nparts ? pc.inv_n[lane] : 0.f,
                          &mean, &rstd);
        } else {
            float s = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k) s += sum4(v[k]);
            mean = block_sum(s, scratch) * inv;
            float q = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k)
                if (t + k * kBlock < nv) q += sq4(v[k], mean);
            q = block_sum(q, scratch);
            if (MODE == kStats || MODE == kJoined) {
                if (t == 0) reinterpret_cast<float2*>(a.stats)[r] = make_float2(mean, q);
                if (MODE == kStats) continue;
            }
            if (MODE == kJoined)
                combine_parts(a.part_stats, a.rows, r, a.nparts, pc, a.eps, lane, lane == a.my_part ? make_float2(mean, q) : first,
                              lane < a.nparts ? pc.inv_n[lane] : 0.f, &mean, &rstd);
            else
                rstd = 1.0f / sqrtf(q * inv + a.eps);
        }
        if (t == 0) {
            if (a.mean_out) a.mean_out[r] = mean;
            if (a.rstd_out) a.rstd_out[r] = rstd;
        }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = t + k * kBlock;
            if (c < nv) {
                float4 o = norm4(v[k], mean, rstd);
                if (AFFINE) o = affine4(load4(static_cast<const T*>(a.gamma) + 4 * c), o, load4(static_cast<const T*>(a.beta) + 4 * c));
                store4(y + r * a.ldy + 4 * c, o);
            }
        }
    }
}

// ---------------------------------------------------------- streamed rows --

// One workgroup per row, the row read once per reduction.  VEC: pieces of four
// (cols % 4 == 0, pitches and addresses allow it), else element by element.
template <typename T, int MODE, bool VEC>
__global__ __launch_bounds__(kBlock) void ln_stream_rows(const LnArgs a, const PartCounts pc) {
    __shared__ float scratch[kWavesPerBlock];
    const T* __restrict__ x = static_cast<const T*>(a.x);
    T* __restrict__ y = static_cast<T*>(a.y);
    const T* __restrict__ gamma = static_cast<const T*>(a.gamma);
    const T* __restrict__ beta = static_cast<const T*>(a.beta);
    const int t = threadIdx.x, lane = t & (kWave - 1);
    const int64_t cols = a.cols;
    const float inv = 1.0f / static_cast<float>(a.cols);
    for (int64_t r = blockIdx.x; r < a.rows; r += gridDim.x) {
        const T* xr = x + r * a.ld;
        float mean, rstd;
        if (MODE == kNorm) {
            combine_parts(a.part_stats, a.rows, r, a.nparts, pc, a.eps, lane,
                          lane < a.nparts ? load_part(a.part_stats, a.rows, r, lane) : make_float2(0.f, 0.f),
                          lane < a.nparts ? pc.inv_n[lane] : 0.f, &mean, &rstd);
        } else {
            float s = 0.f;
            if (VEC) {
                for (int64_t c = 4 * t; c < cols; c += 4 * kBlock) s += sum4(load4(xr + c));
            } else {
                for (int64_t c = t; c < cols; c += kBlock) s += load1(xr + c);
            }
            mean = block_sum(s, scratch) * inv;
            float q = 0.f;
            if (VEC) {
                for (int64_t c = 4 * t; c < cols; c += 4 * kBlock) q += sq4(load4(xr + c), mean);
            } else {
                for (int64_t c = t; c < cols; c += kBlock) {
                    const float d = load1(xr + c) - mean;
                    q += d * d;
                }
            }
            q = block_sum(q, scratch);
            if (MODE == kStats) {
                if (t == 0) reinterpret_cast<float2*>(a.stats)[r] = make_float2(mean, q);
                continue;
            }
            rstd = 1.0f / sqrtf(q * inv + a.eps);
        }
        if (t == 0) {
            if (a.mean_out) a.mean_out[r] = mean;
            if (a.rstd_out) a.rstd_out[r] = rstd;
        }
        T* yr = y + r * a.ldy;
        if (VEC) {
            for (int64_t c = 4 * t; c < cols; c += 4 * kBlock) {
                float4 o = norm4(load4(xr + c), mean, rstd);
                if (gamma) o = affine4(load4(gamma + c), o, load4(beta + c));
                store4(yr + c, o);
            }
        } else {
            for (int64_t c = t; c < cols; c += kBlock) {
                float o = (load1(xr + c) - mean) * rstd;
                if (gamma) o = load1(gamma + c) * o + load1(beta + c);
                store1(yr + c, o);
            }
        }
    }
}

// ------------------------------------------------------------------ host ---

// Rows a wavefront keeps in flight.  Few rows per wavefront mean more
// wavefronts, which is what a small input needs to occupy the whole chip; two
// rows per wavefront stream a long input a little faster.
constexpr int64_t kSmallRows = 65536;

template <typename T, int MODE, bool AFFINE, int NV, int RPW>
void launch_wave_rpw(const LnArgs& a, const PartCounts& pc, hipStream_t s) {
    const int64_t waves = (a.rows + RPW - 1) / RPW;
    const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    hipLaunchKernelGGL((ln_wave_rows<T, NV, RPW, MODE, AFFINE>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, s, a.x, a.rows, a.ld,
                       a.cols, a, pc);
}

template <typename T, int MODE, bool AFFINE, int NV>
void launch_wave(const LnArgs& a, const PartCounts& pc, hipStream_t s) {
    if (NV <= 2 && a.rows > kSmallRows)
        launch_wave_rpw<T, MODE, AFFINE, NV, 2>(a, pc, s);
    else
        launch_wave_rpw<T, MODE, AFFINE, NV, 1>(a, pc, s);
}

template <typename T, int MODE, bool AFFINE, int NV>
void launch_block(const LnArgs& a, const PartCounts& pc, hipStream_t s) {
    const uint32_t blocks = static_cast<uint32_t>(a.rows < (1 << 20) ? a.rows : (1 << 20));
    hipLaunchKernelGGL((ln_block_rows<T, NV, MODE, AFFINE>), dim3(blocks), dim3(kBlock), 0, s, a, pc);
}

template <typename T, int MODE, bool AFFINE>
int launch_typed(const LnArgs& a, const PartCounts& pc, bool vec, hipStream_t s) {
    const int cols = a.cols;
    if (vec && cols <= kWaveRowCols) {
        if (cols <= 256) launch_wave<T, MODE, AFFINE, 1>(a, pc, s);
        else if (cols <= 512) launch_wave<T, MODE, AFFINE, 2>(a, pc, s);
        else if (cols <= 1024) launch_wave<T, MODE, AFFINE, 4>(a, pc, s);
        else launch_wave<T, MODE, AFFINE, 8>(a, pc, s);
        return check_launch("ln_wave_rows");
    }
    if (vec && cols <= kBlockRowCols) {
        if (cols <= 4096) launch_block<T, MODE, AFFINE, 4>(a, pc, s);
        else if (cols <= 8192) launch_block<T, MODE, AFFINE, 8>(a, pc, s);
        else launch_block<T, MODE, AFFINE, 16>(a, pc, s);
        return check_launch("ln_block_rows");
    }
    if constexpr (MODE == kJoined) {
        return fail(DDL_E_UNSUPP, "ln stats+normalize: rows of more than %d columns take the two-launch form", kBlockRowCols);
    } else {
        const uint32_t blocks = static_cast<uint32_t>(a.rows < 65536 ? a.rows : 65536);
        if (vec)
            hipLaunchKernelGGL((ln_stream_rows<T, MODE, true>), dim3(blocks), dim3(kBlock), 0, s, a, pc);
        else
            hipLaunchKernelGGL((ln_stream_rows<T, MODE, false>), dim3(blocks), dim3(kBlock), 0, s, a, pc);
        return check_launch("ln_stream_rows");
    }
}

template <int MODE>
int launch_mode(int dtype, const LnArgs& a, const PartCounts& pc, bool vec, hipStream_t s) {
    const bool affine = MODE != kStats && a.gamma != nullptr;
    switch (dtype) {
        case DDL_DT_F32:
            return affine ? launch_typed<float, MODE, true>(a, pc, vec, s) : launch_typed<float, MODE, false>(a, pc, vec, s);
        case DDL_DT_BF16:
            return affine ? launch_typed<bf16_t, MODE, true>(a, pc, vec, s) : launch_typed<bf16_t, MODE, false>(a, pc, vec, s);
        default:
            return affine ? launch_typed<__half, MODE, true>(a, pc, vec, s) : launch_typed<__half, MODE, false>(a, pc, vec, s);
    }
}

int elem_size_of(int dtype) { return dtype == DDL_DT_F32 ? 4 : (dtype == DDL_DT_BF16 || dtype == DDL_DT_F16) ? 2 : 0; }

// Four-element accesses need rows of a multiple of four columns whose first
// elements are all aligned to four elements.
bool quad_access(const void* p, int es, int64_t cols, int64_t ld) { return cols % 4 == 0 && ld % 4 == 0 && aligned_to(p, 4 * es); }

int check_common(const char* what, int dtype, int64_t rows, int64_t cols, int64_t ld) {
    if (elem_size_of(dtype) == 0) return fail(DDL_E_UNSUPP, "%s: dtype %d (f32, bf16 and f16 only)", what, dtype);
    if (rows < 0 || cols < 1 || ld < cols) return fail(DDL_E_ARG, "%s: rows=%lld cols=%lld ld=%lld", what, (long long)rows, (long long)cols, (long long)ld);
    if (rows > 0x7FFFFFFFll || cols > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "%s: more than 2^31 rows or columns", what);
    return 0;
}

}  // namespace
}  // namespace ddl

extern "C" {

int ddl_ln_partial_stats(const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld, float* stats, void* stream) {
    using namespace ddl;
    if (const int rc = check_common("ln stats", dtype, rows, cols, ld)) return rc;
    if (rows == 0) return 0;
    if (!x || !stats) return fail(DDL_E_ARG, "ln stats: null pointer");
    const int es = elem_size_of(dtype);
    if (!aligned_to(x, es) || !aligned_to(stats, 8)) return fail(DDL_E_ALIGN, "ln stats: x must be element-aligned and stats 8-byte aligned");
    LnArgs a{};
    a.x = x;
    a.stats = stats;
    a.rows = rows, a.ld = ld, a.cols = static_cast<int>(cols);
    const PartCounts pc{};
    return launch_mode<kStats>(dtype, a, pc, quad_access(x, es, cols, ld), static_cast<hipStream_t>(stream));
}

int ddl_ln_normalize_affine(const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld, const float* part_stats,
                            int nparts, const int64_t* part_cols, const void* gamma, const void* beta, float eps, void* y,
                            int64_t ldy, float* mean_out, float* rstd_out, void* stream) {
    using namespace ddl;
    if (const int rc = check_common("ln normalize", dtype, rows, cols, ld)) return rc;
    if (ldy < cols) return fail(DDL_E_ARG, "ln normalize: ldy=%lld below cols=%lld", (long long)ldy, (long long)cols);
    if (nparts < 1 || nparts > kMaxParts) return fail(DDL_E_UNSUPP, "ln normalize: nparts=%d outside [1,%d]", nparts, kMaxParts);
    if ((gamma == nullptr) != (beta == nullptr)) return fail(DDL_E_ARG, "ln normalize: gamma and beta must both be given or both be NULL");
    if (rows == 0) return 0;
    if (!x || !y || !part_stats || !part_cols) return fail(DDL_E_ARG, "ln normalize: null pointer");
    const int es = elem_size_of(dtype);
    if (!aligned_to(x, es) || !aligned_to(y, es) || !aligned_to(gamma, es) || !aligned_to(beta, es) || !aligned_to(part_stats, 8))
        return fail(DDL_E_ALIGN, "ln normalize: x, y, gamma, beta must be element-aligned and the statistics 8-byte aligned");
    PartCounts pc{};
    for (int p = 0; p < nparts; ++p) {
        if (part_cols[p] < 1) return fail(DDL_E_ARG, "ln normalize: worker %d holds %lld columns", p, (long long)part_cols[p]);
        pc.inv_n[p] = 1.0f / static_cast<float>(part_cols[p]);
    }
    LnArgs a{};
    a.x = x, a.y = y, a.gamma = gamma, a.beta = beta, a.part_stats = part_stats;
    a.mean_out = mean_out, a.rstd_out = rstd_out;
    a.rows = rows, a.ld = ld, a.ldy = ldy, a.cols = static_cast<int>(cols), a.nparts = nparts, a.eps = eps;
    const bool vec = quad_access(x, es, cols, ld) && quad_access(y, es, cols, ldy) &&
                     (!gamma || (aligned_to(gamma, 4 * es) && aligned_to(beta, 4 * es)));
    return launch_mode<kNorm>(dtype, a, pc, vec, static_cast<hipStream_t>(stream));
}

int ddl_layer_norm(const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld, const void* gamma, const void* beta,
                   float eps, void* y, int64_t ldy, float* mean_out, float* rstd_out, void* stream) {
    using namespace ddl;
    if (const int rc = check_common("layer norm", dtype, rows, cols, ld)) return rc;
    if (ldy < cols) return fail(DDL_E_ARG, "layer norm: ldy=%lld below cols=%lld", (long long)ldy, (long long)cols);
    if ((gamma == nullptr) != (beta == nullptr)) return fail(DDL_E_ARG, "layer norm: gamma and beta must both be given or both be NULL");
    if (rows == 0) return 0;
    if (!x || !y) return fail(DDL_E_ARG, "layer norm: null pointer");
    const int es = elem_size_of(dtype);
    if (!aligned_to(x, es) || !aligned_to(y, es) || !aligned_to(gamma, es) || !aligned_to(beta, es))
        return fail(DDL_E_ALIGN, "layer norm: x, y, gamma, beta must be element-aligned");
    LnArgs a{};
    a.x = x, a.y = y, a.gamma = gamma, a.beta = beta;
    a.mean_out = mean_out, a.rstd_out = rstd_out;
    a.rows = rows, a.ld = ld, a.ldy = ldy, a.cols = static_cast<int>(cols), a.nparts = 1, a.eps = eps;
    const PartCounts pc{};
    const bool vec = quad_access(x, es, cols, ld) && quad_access(y, es, cols, ldy) &&
                     (!gamma || (aligned_to(gamma, 4 * es) && aligned_to(beta, 4 * es)));
    return launch_mode<kFused>(dtype, a, pc, vec, static_cast<hipStream_t>(stream));
}

int ddl_ln_stats_normalize(const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld, float* part_stats, int nparts,
                           int my_part, const int64_t* part_cols, const void* gamma, const void* beta, float eps, void* y,
                           int64_t ldy, float* mean_out, float* rstd_out, void* stream) {
    using namespace ddl;
    if (const int rc = check_common("ln stats+normalize", dtype, rows, cols, ld)) return rc;
    if (ldy < cols) return fail(DDL_E_ARG, "ln stats+normalize: ldy=%lld below cols=%lld", (long long)ldy, (long long)cols);
    if (nparts < 1 || nparts > kWave) return fail(DDL_E_UNSUPP, "ln stats+normalize: nparts=%d outside [1,%d]", nparts, kWave);
    if (my_part < 0 || my_part >= nparts) return fail(DDL_E_ARG, "ln stats+normalize: my_part=%d outside [0,%d)", my_part, nparts);
    if ((gamma == nullptr) != (beta == nullptr)) return fail(DDL_E_ARG, "ln stats+normalize: gamma and beta must both be given or both be NULL");
    if (rows == 0) return 0;
    if (!x || !y || !part_stats || !part_cols) return fail(DDL_E_ARG, "ln stats+normalize: null pointer");
    const int es = elem_size_of(dtype);
    if (!aligned_to(x, es) || !aligned_to(y, es) || !aligned_to(gamma, es) || !aligned_to(beta, es) || !aligned_to(part_stats, 8))
        return fail(DDL_E_ALIGN, "ln stats+normalize: x, y, gamma, beta must be element-aligned and the statistics 8-byte aligned");
    PartCounts pc{};
    for (int p = 0; p < nparts; ++p) {
        if (part_cols[p] < 1) return fail(DDL_E_ARG, "ln stats+normalize: worker %d holds %lld columns", p, (long long)part_cols[p]);
        pc.inv_n[p] = 1.0f / static_cast<float>(part_cols[p]);
    }
    if (part_cols[my_part] != cols) return fail(DDL_E_ARG, "ln stats+normalize: worker %d holds %lld columns, x has %lld", my_part, (long long)part_cols[my_part], (long long)cols);
    LnArgs a{};
    a.x = x, a.y = y, a.gamma = gamma, a.beta = beta, a.part_stats = part_stats;
    a.stats = part_stats + static_cast<int64_t>(my_part) * rows * 2;
    a.mean_out = mean_out, a.rstd_out = rstd_out;
    a.rows = rows, a.ld = ld, a.ldy = ldy, a.cols = static_cast<int>(cols), a.nparts = nparts, a.my_part = my_part, a.eps = eps;
    const bool vec = quad_access(x, es, cols, ld) && quad_access(y, es, cols, ldy) &&
                     (!gamma || (aligned_to(gamma, 4 * es) && aligned_to(beta, 4 * es)));
    if (!vec) return fail(DDL_E_UNSUPP, "ln stats+normalize: rows must allow four-element accesses (columns and pitches multiples of 4, aligned)");
    return launch_mode<kJoined>(dtype, a, pc, vec, static_cast<hipStream_t>(stream));
}

int ddl_ln_partial_stats_f32(const float* x, int64_t rows, int64_t cols, int64_t ld, float* stats, void* stream) {
    return ddl_ln_partial_stats(x, DDL_DT_F32, rows, cols, ld, stats, stream);
}

int ddl_ln_normalize_affine_f32(const float* x, int64_t rows, int64_t cols, int64_t ld, const float* part_stats,
                                int nparts, const int64_t* part_cols, const float* gamma, const float* beta, float eps,
                                float* y, int64_t ldy, float* mean_out, float* rstd_out, void* stream) {
    return ddl_ln_normalize_affine(x, DDL_DT_F32, rows, cols, ld, part_stats, nparts, part_cols, gamma, beta, eps, y, ldy,
                                   mean_out, rstd_out, stream);
}

}  // extern "C"
