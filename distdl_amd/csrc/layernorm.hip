// DistributedLayerNorm, local shard, fp32 (reference: nn/layernorm.py:218-247,
// 295-309).  Two kernels with the cross-worker exchange between them:
//
//   ln_stats     x[rows, cols] -> {mean_r, M2_r} per row     (one read of x)
//   ln_normalize gathered {mean_p, M2_p} of the P workers sharing a row
//                -> combined mean / var -> y = (x-mean)*rstd*gamma+beta
//
// Rows of up to 2048 columns live in registers: one wavefront owns a row, each
// lane holds float4 pieces, sums go through DPP/shuffle butterflies; a long
// input keeps two rows per wavefront in flight.  Longer (or unaligned)
// rows are staged once in LDS by a 256-thread workgroup and reduced from there.
#include "ddl_common.h"

namespace ddl {
namespace {

constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kMaxParts = 256;
constexpr int kLdsFloats = 16384;  // 64 KiB of staged row

struct PartCounts {
    float inv_n[kMaxParts];  // 1 / columns held by worker p
};

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

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

// ------------------------------------------------------ register-row path --

// One wavefront per row, NV float4 per lane (cols <= 256*NV, cols % 4 == 0),
// RPW rows of a wavefront in flight at once.
template <int NV, int RPW>
__global__ __launch_bounds__(kBlock) void ln_stats_rows(const float* __restrict__ x, int64_t rows, int cols, int64_t ld,
                                                        float* __restrict__ stats) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t r0 = wave * RPW;
    const int nv = cols >> 2;
    float4 v[RPW][NV];
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        const int64_t r = r0 + i;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = lane + k * kWave;
            v[i][k] = (r < rows && c < nv) ? reinterpret_cast<const float4*>(x + r * ld)[c] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    const float inv = 1.0f / static_cast<float>(cols);
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        const int64_t r = r0 + i;
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < NV; ++k) s += (v[i][k].x + v[i][k].y) + (v[i][k].z + v[i][k].w);
        const float mean = wave_sum(s) * inv;
        float q = 0.f;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (lane + k * kWave < nv) {
                const float a = v[i][k].x - mean, b = v[i][k].y - mean, c = v[i][k].z - mean, d = v[i][k].w - mean;
                q += (a * a + b * b) + (c * c + d * d);
            }
        }
        q = wave_sum(q);
        if (lane == 0 && r < rows) reinterpret_cast<float2*>(stats)[r] = make_float2(mean, q);
    }
}

template <int NV, int RPW, bool AFFINE>
__global__ __launch_bounds__(kBlock) void ln_norm_rows(const float* __restrict__ x, int64_t rows, int cols, int64_t ld,
                                                       const float* __restrict__ part_stats, int nparts,
                                                       const PartCounts pc, const float* __restrict__ gamma,
                                                       const float* __restrict__ beta, float eps, float* __restrict__ y,
                                                       int64_t ldy, float* __restrict__ mean_out,
                                                       float* __restrict__ rstd_out) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t r0 = wave * RPW;
    const int nv = cols >> 2;
    float4 g[NV], b[NV];
    if (AFFINE) {
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = lane + k * kWave;
            if (c < nv) {
                g[k] = reinterpret_cast<const float4*>(gamma)[c];
                b[k] = reinterpret_cast<const float4*>(beta)[c];
            }
        }
    }
    // Everything this wavefront reads is requested before anything is used:
    // the gathered statistics of its rows (lane p fetches worker p's pair) and
    // the rows themselves.
    float2 ps[RPW];
    const float inv_n = lane < nparts ? pc.inv_n[lane] : 0.f;
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        const int64_t r = r0 + i;
        ps[i] = (r < rows && lane < nparts) ? load_part(part_stats, rows, r, lane) : make_float2(0.f, 0.f);
    }
    float4 v[RPW][NV];
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        const int64_t r = r0 + i;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = lane + k * kWave;
            if (r < rows && c < nv) v[i][k] = reinterpret_cast<const float4*>(x + r * ld)[c];
        }
    }
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
        const int64_t r = r0 + i;
        if (r >= rows) continue;
        float mean, rstd;
        combine_parts(part_stats, rows, r, nparts, pc, eps, lane, ps[i], inv_n, &mean, &rstd);
        if (lane == 0) {
            if (mean_out) mean_out[r] = mean;
            if (rstd_out) rstd_out[r] = rstd;
        }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int c = lane + k * kWave;
            if (c < nv) {
                float4 o;
                o.x = (v[i][k].x - mean) * rstd;
                o.y = (v[i][k].y - mean) * rstd;
                o.z = (v[i][k].z - mean) * rstd;
                o.w = (v[i][k].w - mean) * rstd;
                if (AFFINE) {
                    o.x = g[k].x * o.x + b[k].x;
                    o.y = g[k].y * o.y + b[k].y;
                    o.z = g[k].z * o.z + b[k].z;
                    o.w = g[k].w * o.w + b[k].w;
                }
                // y is not read again by this kernel: streaming store
                typedef float f32x4 __attribute__((ext_vector_type(4)));
                f32x4 ov;
                ov[0] = o.x, ov[1] = o.y, ov[2] = o.z, ov[3] = o.w;
                __builtin_nontemporal_store(ov, reinterpret_cast<f32x4*>(y + r * ldy) + c);
            }
        }
    }
}

// ------------------------------------------------------ LDS-staged path ----

// One workgroup per row; the row is read from HBM once into LDS (when it fits)
// and both reductions run from the staged copy.
__global__ __launch_bounds__(kBlock) void ln_stats_lds(const float* __restrict__ x, int64_t rows, int64_t cols, int64_t ld,
                                                       float* __restrict__ stats, int staged) {
    __shared__ float row[kLdsFloats];
    __shared__ float scratch[kWavesPerBlock];
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        const float* xr = x + r * ld;
        float s = 0.f;
        for (int64_t c = threadIdx.x; c < cols; c += kBlock) {
            const float t = xr[c];
            if (staged) row[c] = t;
            s += t;
        }
        const float mean = block_sum(s, scratch) / static_cast<float>(cols);
        float q = 0.f;
        for (int64_t c = threadIdx.x; c < cols; c += kBlock) {
            const float d = (staged ? row[c] : xr[c]) - mean;
            q += d * d;
        }
        q = block_sum(q, scratch);
        if (threadIdx.x == 0) reinterpret_cast<float2*>(stats)[r] = make_float2(mean, q);
        __syncthreads();
    }
}

__global__ __launch_bounds__(kBlock) void ln_norm_stream(const float* __restrict__ x, int64_t rows, int64_t cols, int64_t ld,
                                                         const float* __restrict__ part_stats, int nparts,
                                                         const PartCounts pc, const float* __restrict__ gamma,
                                                         const float* __restrict__ beta, float eps, float* __restrict__ y,
                                                         int64_t ldy, float* __restrict__ mean_out,
                                                         float* __restrict__ rstd_out) {
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        float mean, rstd;
        const int lane = threadIdx.x & (kWave - 1);
        combine_parts(part_stats, rows, r, nparts, pc, eps, lane,
                      lane < nparts ? load_part(part_stats, rows, r, lane) : make_float2(0.f, 0.f),
                      lane < nparts ? pc.inv_n[lane] : 0.f, &mean, &rstd);
        if (threadIdx.x == 0) {
            if (mean_out) mean_out[r] = mean;
            if (rstd_out) rstd_out[r] = rstd;
        }
        const float* xr = x + r * ld;
        float* yr = y + r * ldy;
        for (int64_t c = threadIdx.x; c < cols; c += kBlock) {
            float o = (xr[c] - mean) * rstd;
            if (gamma) o = gamma[c] * o + beta[c];
            yr[c] = o;
        }
    }
}

bool rows_vectorizable(const void* p, int64_t cols, int64_t ld) {
    return cols % 4 == 0 && ld % 4 == 0 && cols <= 2048 && aligned_to(p, 16);
}

// Rows a wavefront keeps in flight.  Few rows per wavefront mean more
// wavefronts, which is what a small input needs to occupy the whole chip; two
// rows per wavefront stream a long input a little faster.
constexpr int64_t kSmallRows = 65536;

template <int NV, int RPW>
int launch_stats_rpw(const float* x, int64_t rows, int cols, int64_t ld, float* stats, hipStream_t s) {
    const int64_t waves = (rows + RPW - 1) / RPW;
    const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    hipLaunchKernelGGL((ln_stats_rows<NV, RPW>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, s, x, rows, cols, ld, stats);
    return check_launch("ln_stats_rows");
}

template <int NV>
int launch_stats(const float* x, int64_t rows, int cols, int64_t ld, float* stats, hipStream_t s) {
    if (NV <= 2 && rows > kSmallRows) return launch_stats_rpw<NV, 2>(x, rows, cols, ld, stats, s);
    return launch_stats_rpw<NV, 1>(x, rows, cols, ld, stats, s);
}

template <int NV, int RPW>
int launch_norm_rpw(const float* x, int64_t rows, int cols, int64_t ld, const float* ps, int nparts, const PartCounts& pc,
                    const float* gamma, const float* beta, float eps, float* y, int64_t ldy, float* mo, float* ro,
                    hipStream_t s) {
    const int64_t waves = (rows + RPW - 1) / RPW;
    const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    if (gamma)
        hipLaunchKernelGGL((ln_norm_rows<NV, RPW, true>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, s, x, rows, cols,
                           ld, ps, nparts, pc, gamma, beta, eps, y, ldy, mo, ro);
    else
        hipLaunchKernelGGL((ln_norm_rows<NV, RPW, false>), dim3(static_cast<uint32_t>(blocks)), dim3(kBlock), 0, s, x, rows,
                           cols, ld, ps, nparts, pc, gamma, beta, eps, y, ldy, mo, ro);
    return check_launch("ln_norm_rows");
}

template <int NV>
int launch_norm(const float* x, int64_t rows, int cols, int64_t ld, const float* ps, int nparts, const PartCounts& pc,
                const float* gamma, const float* beta, float eps, float* y, int64_t ldy, float* mo, float* ro,
                hipStream_t s) {
    if (NV <= 2 && rows > kSmallRows) return launch_norm_rpw<NV, 2>(x, rows, cols, ld, ps, nparts, pc, gamma, beta, eps, y, ldy, mo, ro, s);
    return launch_norm_rpw<NV, 1>(x, rows, cols, ld, ps, nparts, pc, gamma, beta, eps, y, ldy, mo, ro, s);
}

}  // namespace
}  // namespace ddl

extern "C" {

int ddl_ln_partial_stats_f32(const float* x, int64_t rows, int64_t cols, int64_t ld, float* stats, void* stream) {
    using namespace ddl;
    if (rows < 0 || cols < 1 || ld < cols) return fail(DDL_E_ARG, "ln stats: rows=%lld cols=%lld ld=%lld", (long long)rows, (long long)cols, (long long)ld);
    if (rows == 0) return 0;
    if (!x || !stats) return fail(DDL_E_ARG, "ln stats: null pointer");
    if (!aligned_to(x, 4) || !aligned_to(stats, 8)) return fail(DDL_E_ALIGN, "ln stats: x must be 4-byte and stats 8-byte aligned");
    if (rows > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "ln stats: more than 2^31 rows");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (rows_vectorizable(x, cols, ld)) {
        const int c = static_cast<int>(cols);
        if (cols <= 256) return launch_stats<1>(x, rows, c, ld, stats, s);
        if (cols <= 512) return launch_stats<2>(x, rows, c, ld, stats, s);
        if (cols <= 1024) return launch_stats<4>(x, rows, c, ld, stats, s);
        return launch_stats<8>(x, rows, c, ld, stats, s);
    }
    const uint32_t blocks = static_cast<uint32_t>(rows < 65536 ? rows : 65536);
    hipLaunchKernelGGL(ln_stats_lds, dim3(blocks), dim3(kBlock), 0, s, x, rows, cols, ld, stats, cols <= kLdsFloats ? 1 : 0);
    return check_launch("ln_stats_lds");
}

int ddl_ln_normalize_affine_f32(const float* x, int64_t rows, int64_t cols, int64_t ld, const float* part_stats,
                                int nparts, const int64_t* part_cols, const float* gamma, const float* beta, float eps,
                                float* y, int64_t ldy, float* mean_out, float* rstd_out, void* stream) {
    using namespace ddl;
    if (rows < 0 || cols < 1 || ld < cols || ldy < cols) return fail(DDL_E_ARG, "ln normalize: rows=%lld cols=%lld ld=%lld ldy=%lld", (long long)rows, (long long)cols, (long long)ld, (long long)ldy);
    if (nparts < 1 || nparts > kMaxParts) return fail(DDL_E_UNSUPP, "ln normalize: nparts=%d outside [1,%d]", nparts, kMaxParts);
    if ((gamma == nullptr) != (beta == nullptr)) return fail(DDL_E_ARG, "ln normalize: gamma and beta must both be given or both be NULL");
    if (rows == 0) return 0;
    if (!x || !y || !part_stats || !part_cols) return fail(DDL_E_ARG, "ln normalize: null pointer");
    if (rows > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "ln normalize: more than 2^31 rows");
    if (!aligned_to(x, 4) || !aligned_to(y, 4) || !aligned_to(part_stats, 8))
        return fail(DDL_E_ALIGN, "ln normalize: x, y must be 4-byte and the statistics 8-byte aligned");
    PartCounts pc{};
    for (int p = 0; p < nparts; ++p) {
        if (part_cols[p] < 1) return fail(DDL_E_ARG, "ln normalize: worker %d holds %lld columns", p, (long long)part_cols[p]);
        pc.inv_n[p] = 1.0f / static_cast<float>(part_cols[p]);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool vec = rows_vectorizable(x, cols, ld) && ldy % 4 == 0 && aligned_to(y, 16) &&
                     (!gamma || (aligned_to(gamma, 16) && aligned_to(beta, 16)));
    if (vec) {
        const int c = static_cast<int>(cols);
        if (cols <= 256) return launch_norm<1>(x, rows, c, ld, part_stats, nparts, pc, gamma, beta, eps, y, ldy, mean_out, rstd_out, s);
        if (cols <= 512) return launch_norm<2>(x, rows, c, ld, part_stats, nparts, pc, gamma, beta, eps, y, ldy, mean_out, rstd_out, s);
        if (cols <= 1024) return launch_norm<4>(x, rows, c, ld, part_stats, nparts, pc, gamma, beta, eps, y, ldy, mean_out, rstd_out, s);
        return launch_norm<8>(x, rows, c, ld, part_stats, nparts, pc, gamma, beta, eps, y, ldy, mean_out, rstd_out, s);
    }
    const uint32_t blocks = static_cast<uint32_t>(rows < 65536 ? rows : 65536);
    hipLaunchKernelGGL(ln_norm_stream, dim3(blocks), dim3(kBlock), 0, s, x, rows, cols, ld, part_stats, nparts, pc, gamma,
                       beta, eps, y, ldy, mean_out, rstd_out);
    return check_launch("ln_norm_stream");
}

}  // extern "C"
