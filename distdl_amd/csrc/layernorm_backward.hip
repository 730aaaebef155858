// Backward of the DistributedLayerNorm shard: what autograd derives from
// the reference's forward (nn/layernorm.py:230-247, 295-309)
//
//   mean = allreduce(local mean) / P        var = allreduce(local mean((x-mean)^2)) / P
//   xhat = (x - mean) rstd                  y = gamma xhat + beta
//
// Every element of worker p enters mean and var with weight a_p = 1 / (P n_p)
// (n_p = columns held by p; the weights of a row add up to 1), which gives
//
//   g    = dy gamma
//   S1   = sum over the whole row of g           S2 = sum over the whole row of g xhat
//   dx   = rstd (g - a_p (S1 + xhat S2))
//   dgamma[c] = sum over rows of dy xhat         dbeta[c] = sum over rows of dy
//
// S1 and S2 span all workers of the row, so the work is split like the forward:
//   ln_bwd_partial   local {sum g, sum g xhat} per row      (one read of dy, x)
//   -- the caller gathers the pairs of the P workers --
//   ln_bwd_input     sums the gathered pairs, writes dx      (one read of dy, x)
//   ln_bwd_params    column sums over the local rows, in row splits through a
//                    workspace, for dgamma and dbeta
// One wavefront owns a row and strides over its columns (four elements at a time
// when the row is aligned); nothing is kept between passes, so rows of any length
// work.  dy, x, gamma, dx, dgamma and dbeta are float, bf16 or fp16 (one type per
// call); the arithmetic, the saved mean and rstd, the row sums and the workspace
// are fp32.
#include "ln_elements.h"

namespace ddl {
namespace {

constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kStrip = 64;     // columns per workgroup of the parameter kernel

template <typename T, bool VEC>
__global__ __launch_bounds__(kBlock) void ln_bwd_partial(const T* __restrict__ dy, const T* __restrict__ x, int64_t rows,
                                                         int64_t cols, int64_t ld_dy, int64_t ld_x,
                                                         const float* __restrict__ mean, const float* __restrict__ rstd,
                                                         const T* __restrict__ gamma, float* __restrict__ sums) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + threadIdx.x / kWave;
    if (r >= rows) return;
    const float m = mean[r], rs = rstd[r];
    const T* dyr = dy + r * ld_dy;
    const T* xr = x + r * ld_x;
    float s1 = 0.f, s2 = 0.f;
    if (VEC) {
        for (int64_t c = lane * 4; c < cols; c += kWave * 4) {
            const float4 d = load4(dyr + c);
            const float4 v = load4(xr + c);
            float4 g = make_float4(1.f, 1.f, 1.f, 1.f);
            if (gamma) g = load4(gamma + c);
            const float g0 = d.x * g.x, g1 = d.y * g.y, g2 = d.z * g.z, g3 = d.w * g.w;
            s1 += (g0 + g1) + (g2 + g3);
            s2 += (g0 * ((v.x - m) * rs) + g1 * ((v.y - m) * rs)) + (g2 * ((v.z - m) * rs) + g3 * ((v.w - m) * rs));
        }
    } else {
        for (int64_t c = lane; c < cols; c += kWave) {
            const float g = load1(dyr + c) * (gamma ? load1(gamma + c) : 1.f);
            s1 += g;
            s2 += g * ((load1(xr + c) - m) * rs);
        }
    }
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    if (lane == 0) reinterpret_cast<float2*>(sums)[r] = make_float2(s1, s2);
}

// One element of dx = rstd (g - (S1 + xhat S2)), S already times a_p.  Every
// kernel that writes dx goes through this one sequence of roundings (no
// contraction left to the compiler), so they agree bit for bit.
__device__ inline float dx_value(float dyv, float gv, float xv, float m, float rs, float S1, float S2) {
#pragma clang fp contract(off)
    const float h = (xv - m) * rs;
    const float t = __builtin_fmaf(h, S2, S1);
    const float q = dyv * gv - t;
    return rs * q;
}

template <typename T, bool VEC>
__device__ inline void ln_bwd_input_body(uint32_t block, const T* __restrict__ dy, const T* __restrict__ x, int64_t rows,
                                         int64_t cols, int64_t ld_dy, int64_t ld_x, const float* __restrict__ mean,
                                         const float* __restrict__ rstd, const T* __restrict__ gamma,
                                         const float* __restrict__ part_sums, int nparts, float weight, T* __restrict__ dx,
                                         int64_t ld_dx) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t r = static_cast<int64_t>(block) * kWavesPerBlock + threadIdx.x / kWave;
    if (r >= rows) return;
    // the pairs of all workers of this row, one worker per lane (and round)
    float p1 = 0.f, p2 = 0.f;
    for (int p = lane; p < nparts; p += kWave) {
        const float2 s = reinterpret_cast<const float2*>(part_sums)[static_cast<int64_t>(p) * rows + r];
        p1 += s.x;
        p2 += s.y;
    }
    const float m = mean[r], rs = rstd[r];
    const T* dyr = dy + r * ld_dy;
    const T* xr = x + r * ld_x;
    T* dxr = dx + r * ld_dx;
    // The first kAhead pieces of the row are requested before the sums are
    // reduced: the reduction waits for the gathered pairs, and the row should
    // not wait behind it (one memory round trip instead of two for rows of up
    // to 1024 columns).
    constexpr int kAhead = 4;
    float4 d0[kAhead], v0[kAhead], g0[kAhead];
    if (VEC) {
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            const int64_t c = lane * 4 + static_cast<int64_t>(k) * (kWave * 4);
            g0[k] = make_float4(1.f, 1.f, 1.f, 1.f);
            if (c < cols) {
                d0[k] = load4(dyr + c);
                v0[k] = load4(xr + c);
                if (gamma) g0[k] = load4(gamma + c);
            }
        }
    }
    const float S1 = wave_sum(p1) * weight, S2 = wave_sum(p2) * weight;   // already times a_p
    if (VEC) {
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            const int64_t c = lane * 4 + static_cast<int64_t>(k) * (kWave * 4);
            if (c < cols) {
                float4 o;
                o.x = dx_value(d0[k].x, g0[k].x, v0[k].x, m, rs, S1, S2);
                o.y = dx_value(d0[k].y, g0[k].y, v0[k].y, m, rs, S1, S2);
                o.z = dx_value(d0[k].z, g0[k].z, v0[k].z, m, rs, S1, S2);
                o.w = dx_value(d0[k].w, g0[k].w, v0[k].w, m, rs, S1, S2);
                store4(dxr + c, o);
            }
        }
        for (int64_t c = lane * 4 + static_cast<int64_t>(kAhead) * (kWave * 4); c < cols; c += kWave * 4) {
            const float4 d = load4(dyr + c);
            const float4 v = load4(xr + c);
            float4 g = make_float4(1.f, 1.f, 1.f, 1.f);
            if (gamma) g = load4(gamma + c);
            float4 o;
            o.x = dx_value(d.x, g.x, v.x, m, rs, S1, S2);
            o.y = dx_value(d.y, g.y, v.y, m, rs, S1, S2);
            o.z = dx_value(d.z, g.z, v.z, m, rs, S1, S2);
            o.w = dx_value(d.w, g.w, v.w, m, rs, S1, S2);
            store4(dxr + c, o);   // dx is not read again here: streaming store
        }
    } else {
        for (int64_t c = lane; c < cols; c += kWave) {
            store1(dxr + c, dx_value(load1(dyr + c), gamma ? load1(gamma + c) : 1.f, load1(xr + c), m, rs, S1, S2));
        }
    }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kBlock) void ln_bwd_input(const T* __restrict__ dy, const T* __restrict__ x, int64_t rows,
                                                       int64_t cols, int64_t ld_dy, int64_t ld_x,
                                                       const float* __restrict__ mean, const float* __restrict__ rstd,
                                                       const T* __restrict__ gamma, const float* __restrict__ part_sums,
                                                       int nparts, float weight, T* __restrict__ dx, int64_t ld_dx) {
    ln_bwd_input_body<T, VEC>(blockIdx.x, dy, x, rows, cols, ld_dy, ld_x, mean, rstd, gamma, part_sums, nparts, weight, dx, ld_dx);
}

// Workgroup (strip, split): rows [split * rows_per_split, ...) of a 64-column
// strip; lane group t / 64 takes every fourth row, thread t % 64 one column.
// partial[split, 0, c] = sum dy xhat, partial[split, 1, c] = sum dy.
template <typename T>
__global__ __launch_bounds__(kBlock) void ln_bwd_params_partial(const T* __restrict__ dy, const T* __restrict__ x,
                                                                int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x,
                                                                const float* __restrict__ mean, const float* __restrict__ rstd,
                                                                int64_t rows_per_split, float* __restrict__ partial, int strips) {
    __shared__ float fold[2][kWavesPerBlock][kStrip];
    const int split = blockIdx.x / strips, strip = blockIdx.x - split * strips;
    const int g = threadIdx.x / kStrip, t = threadIdx.x % kStrip;
    const int64_t c = static_cast<int64_t>(strip) * kStrip + t;
    const int64_t r_begin = split * rows_per_split;
    const int64_t r_end = r_begin + rows_per_split < rows ? r_begin + rows_per_split : rows;
    float a = 0.f, b = 0.f;
    if (c < cols) {
        for (int64_t r = r_begin + g; r < r_end; r += kWavesPerBlock) {
            const float d = load1(dy + r * ld_dy + c);
            a += d * ((load1(x + r * ld_x + c) - mean[r]) * rstd[r]);
            b += d;
        }
    }
    fold[0][g][t] = a;
    fold[1][g][t] = b;
    __syncthreads();
    if (threadIdx.x < 2 * kStrip) {
        const int which = threadIdx.x / kStrip;
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < kWavesPerBlock; ++k) s += fold[which][k][t];
        if (c < cols) partial[(static_cast<int64_t>(split) * 2 + which) * cols + c] = s;
    }
}

// Workgroup per 64-column strip: lane group g = t / 64 adds the splits g, g+4,
// ... of column t % 64 (independent loads, kInFlight of them requested together:
// many when this is all a kernel does, few when it shares its registers with
// the dx pass), LDS folds the four
// groups.
template <typename T, int kInFlight>
__device__ inline void ln_bwd_params_final_body(uint32_t block, const float* __restrict__ partial, int64_t cols, int splits,
                                                T* __restrict__ dgamma, T* __restrict__ dbeta) {
    __shared__ float fold[2][kWavesPerBlock][kStrip];
    const int g = threadIdx.x / kStrip, t = threadIdx.x % kStrip;
    const int64_t c = static_cast<int64_t>(block) * kStrip + t;
    float a = 0.f, b = 0.f;
    if (c < cols) {
        int k = g;
        for (; k + (kInFlight - 1) * kWavesPerBlock < splits; k += kInFlight * kWavesPerBlock) {
            float va[kInFlight], vb[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                va[u] = partial[(static_cast<int64_t>(k + u * kWavesPerBlock) * 2) * cols + c];
                vb[u] = partial[(static_cast<int64_t>(k + u * kWavesPerBlock) * 2 + 1) * cols + c];
            }
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                a += va[u];
                b += vb[u];
            }
        }
        for (; k < splits; k += kWavesPerBlock) {
            a += partial[(static_cast<int64_t>(k) * 2) * cols + c];
            b += partial[(static_cast<int64_t>(k) * 2 + 1) * cols + c];
        }
    }
    fold[0][g][t] = a;
    fold[1][g][t] = b;
    __syncthreads();
    if (threadIdx.x < 2 * kStrip && c < cols) {
        const int which = threadIdx.x / kStrip;
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < kWavesPerBlock; ++k) s += fold[which][k][t];
        T* out = which == 0 ? dgamma : dbeta;
        if (out) store1(out + c, s);
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void ln_bwd_params_final(const float* __restrict__ partial, int64_t cols, int splits,
                                                              T* __restrict__ dgamma, T* __restrict__ dbeta) {
    ln_bwd_params_final_body<T, 32>(blockIdx.x, partial, cols, splits, dgamma, dbeta);
}

// dx and the final parameter sums in one launch: the first final_blocks
// workgroups (one per 64-column strip) add up the partial column sums -- a chain
// of dependent loads, so they start first -- and the rest write dx.  The two
// parts are independent.
template <typename T, bool VEC>
__global__ __launch_bounds__(kBlock) void ln_bwd_input_final(const T* __restrict__ dy, const T* __restrict__ x, int64_t rows,
                                                             int64_t cols, int64_t ld_dy, int64_t ld_x,
                                                             const float* __restrict__ mean, const float* __restrict__ rstd,
                                                             const T* __restrict__ gamma, const float* __restrict__ part_sums,
                                                             int nparts, float weight, T* __restrict__ dx, int64_t ld_dx,
                                                             uint32_t final_blocks, const float* __restrict__ partial, int splits,
                                                             T* __restrict__ dgamma, T* __restrict__ dbeta) {
    if (blockIdx.x < final_blocks)
        ln_bwd_params_final_body<T, 8>(blockIdx.x, partial, cols, splits, dgamma, dbeta);
    else
        ln_bwd_input_body<T, VEC>(blockIdx.x - final_blocks, dy, x, rows, cols, ld_dy, ld_x, mean, rstd, gamma, part_sums, nparts,
                               weight, dx, ld_dx);
}

constexpr int kFusedBlock = 512;   // eight wavefronts: a split of 32 rows is one round of four rows per wavefront
constexpr int kFusedWaves = kFusedBlock / kWave;

// What ln_bwd_partial_cols<.., true> needs beyond the sums: the other workers'
// row sums (already in memory), this worker's place among them, and where dx goes.
struct DxArgs {
    const float* part_sums;   // [nparts][rows][2]; slot my_part is not read
    int nparts, my_part;
    float weight;
    void* dx;
    int64_t ld_dx;
};

// Row sums {sum g, sum g xhat} and the partial column sums of a row split in one
// pass over dy and x: workgroup = split, its wavefronts take every eighth row
// and each lane keeps the columns (lane + 64 k) * 4 .. + 3, k < NV, in registers.
// partial has the layout of ln_bwd_params_partial.  WITH_DX: the sums of the
// whole row are complete once this worker's are (it holds the row whole, or the
// other workers' pairs are in memory), so dx is written in the same pass, from
// the registers that hold the row.
template <typename T, int NV, bool WITH_DX>
__global__ __launch_bounds__(kFusedBlock) void ln_bwd_partial_cols(const T* __restrict__ dy, const T* __restrict__ x, int64_t rows,
                                                              int64_t cols, int64_t ld_dy, int64_t ld_x,
                                                              const float* __restrict__ mean, const float* __restrict__ rstd,
                                                              const T* __restrict__ gamma, float* __restrict__ sums,
                                                              int64_t rows_per_split, float* __restrict__ partial, const DxArgs dxa) {
#pragma clang fp contract(off)   // both instantiations round alike: sums, column sums and dx do not depend on WITH_DX
    __shared__ float fold[2][kFusedWaves][NV * kWave * 4];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int nv = static_cast<int>(cols >> 2);
    const int64_t r_begin = static_cast<int64_t>(blockIdx.x) * rows_per_split;
    const int64_t r_end = r_begin + rows_per_split < rows ? r_begin + rows_per_split : rows;
    float4 g[NV], ca[NV], cb[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int c = lane + k * kWave;
        g[k] = make_float4(1.f, 1.f, 1.f, 1.f);
        if (gamma && c < nv) g[k] = load4(gamma + 4 * c);
        ca[k] = cb[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    constexpr int RU = NV <= 2 ? 4 : 2;   // rows whose loads are in flight together
    for (int64_t r0 = r_begin + wave; r0 < r_end; r0 += kFusedWaves * RU) {
        float m[RU], rs[RU];
        float4 d[RU][NV], v[RU][NV];
        float2 peer[RU];   // WITH_DX: the pair of worker `lane` for this row, requested together with the row
#pragma unroll
        for (int u = 0; u < RU; ++u) {
            const int64_t r = r0 + u * kFusedWaves;
            const bool on = r < r_end;
            m[u] = on ? mean[r] : 0.f;
            rs[u] = on ? rstd[r] : 0.f;
            peer[u] = make_float2(0.f, 0.f);
            if (WITH_DX && on && lane < dxa.nparts && lane != dxa.my_part)
                peer[u] = reinterpret_cast<const float2*>(dxa.part_sums)[static_cast<int64_t>(lane) * rows + r];
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const int c = lane + k * kWave;
                d[u][k] = v[u][k] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (on && c < nv) {
                    d[u][k] = load4(dy + r * ld_dy + 4 * c);
                    v[u][k] = load4(x + r * ld_x + 4 * c);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < RU; ++u) {
            const int64_t r = r0 + u * kFusedWaves;
            if (r >= r_end) break;                              // wave-uniform
            float s1 = 0.f, s2 = 0.f;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                // columns past the row hold zeros in d, so they add nothing
                const float4 dd = d[u][k], vv = v[u][k];
                const float h0 = (vv.x - m[u]) * rs[u], h1 = (vv.y - m[u]) * rs[u], h2 = (vv.z - m[u]) * rs[u], h3 = (vv.w - m[u]) * rs[u];
                const float g0 = dd.x * g[k].x, g1 = dd.y * g[k].y, g2 = dd.z * g[k].z, g3 = dd.w * g[k].w;
                s1 += (g0 + g1) + (g2 + g3);
                s2 += (g0 * h0 + g1 * h1) + (g2 * h2 + g3 * h3);
                ca[k].x += dd.x * h0, ca[k].y += dd.y * h1, ca[k].z += dd.z * h2, ca[k].w += dd.w * h3;
                cb[k].x += dd.x, cb[k].y += dd.y, cb[k].z += dd.z, cb[k].w += dd.w;
            }
            s1 = wave_sum(s1);
            s2 = wave_sum(s2);
            if (lane == 0 && sums) reinterpret_cast<float2*>(sums)[r] = make_float2(s1, s2);
            if (WITH_DX) {
                // the pairs of all workers of this row, one worker per lane (at most 64 workers)
                float p1 = peer[u].x, p2 = peer[u].y;
                if (lane == dxa.my_part) p1 = s1, p2 = s2;
                const float S1 = wave_sum(p1) * dxa.weight, S2 = wave_sum(p2) * dxa.weight;
                T* dxr = static_cast<T*>(dxa.dx) + r * dxa.ld_dx;
#pragma unroll
                for (int k = 0; k < NV; ++k) {
                    const int c = lane + k * kWave;
                    if (c >= nv) continue;
                    const float4 dd = d[u][k], vv = v[u][k];
                    float4 o;
                    o.x = dx_value(dd.x, g[k].x, vv.x, m[u], rs[u], S1, S2);
                    o.y = dx_value(dd.y, g[k].y, vv.y, m[u], rs[u], S1, S2);
                    o.z = dx_value(dd.z, g[k].z, vv.z, m[u], rs[u], S1, S2);
                    o.w = dx_value(dd.w, g[k].w, vv.w, m[u], rs[u], S1, S2);
                    store4(dxr + 4 * c, o);
                }
            }
        }
    }
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int c4 = (lane + k * kWave) * 4;
        *reinterpret_cast<float4*>(&fold[0][wave][c4]) = ca[k];
        *reinterpret_cast<float4*>(&fold[1][wave][c4]) = cb[k];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * static_cast<int>(cols); i += kFusedBlock) {
        const int which = i >= static_cast<int>(cols) ? 1 : 0, c = i - which * static_cast<int>(cols);
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < kFusedWaves; ++w) t += fold[which][w][c];
        partial[(static_cast<int64_t>(blockIdx.x) * 2 + which) * cols + c] = t;
    }
}

// Can rows be read four elements at a time?  elem = bytes per element.
bool vectorizable(int elem, int64_t cols, std::initializer_list<int64_t> lds, std::initializer_list<const void*> ptrs) {
    if (cols % 4 != 0) return false;
    for (int64_t ld : lds)
        if (ld % 4 != 0) return false;
    for (const void* p : ptrs)
        if (p && !aligned_to(p, 4 * elem)) return false;
    return true;
}

int check_rows(const char* what, int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x) {
    if (rows < 0 || cols < 1 || ld_dy < cols || ld_x < cols)
        return fail(DDL_E_ARG, "%s: rows=%lld cols=%lld ld_dy=%lld ld_x=%lld", what, (long long)rows, (long long)cols,
                    (long long)ld_dy, (long long)ld_x);
    if (rows > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "%s: more than 2^31 rows", what);
    return 0;
}

int elem_bytes(int dtype) { return dtype == DDL_DT_F32 ? 4 : (dtype == DDL_DT_BF16 || dtype == DDL_DT_F16) ? 2 : 0; }

// Elements aligned to their own size, fp32 side arrays to 4 bytes, pairs to 8.
bool elems_aligned(int elem, std::initializer_list<const void*> ptrs) {
    for (const void* p : ptrs)
        if (p && !aligned_to(p, elem)) return false;
    return true;
}

// Row splits of the parameter gradients: as many as the workspace holds, at most
// 256 and at least 32 rows each.  0 when the workspace cannot hold one split.
int64_t param_splits(int64_t rows, int64_t cols, int64_t workspace_elems) {
    int64_t splits = workspace_elems / (2 * cols);
    if (splits < 1) return 0;
    if (splits > 256) splits = 256;
    const int64_t by_rows = (rows + 31) / 32;
    if (splits > by_rows) splits = by_rows > 0 ? by_rows : 1;
    return splits;
}

template <typename T>
const T* as(const void* p) { return static_cast<const T*>(p); }
template <typename T>
T* as(void* p) { return static_cast<T*>(p); }

}  // namespace
}  // namespace ddl

extern "C" int ddl_ln_bwd_partial(const void* dy, const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x,
                                  const float* mean, const float* rstd, const void* gamma, float* sums, void* stream) {
    using namespace ddl;
    const int elem = elem_bytes(dtype);
    if (!elem) return fail(DDL_E_UNSUPP, "ln backward sums: dtype %d (f32, bf16, f16 only)", dtype);
    if (int rc = check_rows("ln backward sums", rows, cols, ld_dy, ld_x)) return rc;
    if (rows == 0) return 0;
    if (!dy || !x || !mean || !rstd || !sums) return fail(DDL_E_ARG, "ln backward sums: null pointer");
    if (!elems_aligned(elem, {dy, x, gamma}) || !aligned_to(mean, 4) || !aligned_to(rstd, 4) || !aligned_to(sums, 8))
        return fail(DDL_E_ALIGN, "ln backward sums: elements must be aligned to their size, mean and rstd to 4 bytes, the sums to 8");
    const uint32_t blocks = static_cast<uint32_t>((rows + kWavesPerBlock - 1) / kWavesPerBlock);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool vec = vectorizable(elem, cols, {ld_dy, ld_x}, {dy, x, gamma});
    with_ln_element(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (vec)
            hipLaunchKernelGGL((ln_bwd_partial<T, true>), dim3(blocks), dim3(kBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd, as<T>(gamma), sums);
        else
            hipLaunchKernelGGL((ln_bwd_partial<T, false>), dim3(blocks), dim3(kBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd, as<T>(gamma), sums);
    });
    return check_launch("ln_bwd_partial");
}

extern "C" int ddl_ln_bwd_input(const void* dy, const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x,
                                const float* mean, const float* rstd, const void* gamma, const float* part_sums, int nparts,
                                float weight, void* dx, int64_t ld_dx, void* stream) {
    using namespace ddl;
    const int elem = elem_bytes(dtype);
    if (!elem) return fail(DDL_E_UNSUPP, "ln backward input: dtype %d (f32, bf16, f16 only)", dtype);
    if (int rc = check_rows("ln backward input", rows, cols, ld_dy, ld_x)) return rc;
    if (ld_dx < cols || nparts < 1) return fail(DDL_E_ARG, "ln backward input: ld_dx=%lld nparts=%d", (long long)ld_dx, nparts);
    if (rows == 0) return 0;
    if (!dy || !x || !mean || !rstd || !part_sums || !dx) return fail(DDL_E_ARG, "ln backward input: null pointer");
    if (!elems_aligned(elem, {dy, x, gamma, dx}) || !aligned_to(mean, 4) || !aligned_to(rstd, 4) || !aligned_to(part_sums, 8))
        return fail(DDL_E_ALIGN, "ln backward input: elements must be aligned to their size, mean and rstd to 4 bytes, the sums to 8");
    const uint32_t blocks = static_cast<uint32_t>((rows + kWavesPerBlock - 1) / kWavesPerBlock);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool vec = vectorizable(elem, cols, {ld_dy, ld_x, ld_dx}, {dy, x, gamma, dx});
    with_ln_element(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (vec)
            hipLaunchKernelGGL((ln_bwd_input<T, true>), dim3(blocks), dim3(kBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd,
                               as<T>(gamma), part_sums, nparts, weight, as<T>(dx), ld_dx);
        else
            hipLaunchKernelGGL((ln_bwd_input<T, false>), dim3(blocks), dim3(kBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd,
                               as<T>(gamma), part_sums, nparts, weight, as<T>(dx), ld_dx);
    });
    return check_launch("ln_bwd_input");
}

extern "C" int ddl_ln_bwd_params(const void* dy, const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x,
                                 const float* mean, const float* rstd, void* dgamma, void* dbeta, float* workspace,
                                 int64_t workspace_elems, void* stream) {
    using namespace ddl;
    const int elem = elem_bytes(dtype);
    if (!elem) return fail(DDL_E_UNSUPP, "ln backward parameters: dtype %d (f32, bf16, f16 only)", dtype);
    if (int rc = check_rows("ln backward parameters", rows, cols, ld_dy, ld_x)) return rc;
    if (!dgamma && !dbeta) return 0;
    if (!workspace || (rows > 0 && (!dy || !x || !mean || !rstd))) return fail(DDL_E_ARG, "ln backward parameters: null pointer");
    if (!elems_aligned(elem, {dy, x, dgamma, dbeta}) || !aligned_to(mean, 4) || !aligned_to(rstd, 4) || !aligned_to(workspace, 4))
        return fail(DDL_E_ALIGN, "ln backward parameters: elements must be aligned to their size, fp32 arrays to 4 bytes");
    const int64_t splits = param_splits(rows, cols, workspace_elems);
    if (splits < 1) return fail(DDL_E_ARG, "ln backward parameters: workspace of %lld floats is smaller than 2 x %lld", (long long)workspace_elems, (long long)cols);
    const int64_t rows_per_split = rows > 0 ? (rows + splits - 1) / splits : 1;
    const int64_t strips = (cols + kStrip - 1) / kStrip;
    if (strips * splits > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "ln backward parameters: too many workgroups");
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc = 0;
    with_ln_element(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        hipLaunchKernelGGL(ln_bwd_params_partial<T>, dim3(static_cast<uint32_t>(strips * splits)), dim3(kBlock), 0, s, as<T>(dy), as<T>(x), rows,
                           cols, ld_dy, ld_x, mean, rstd, rows_per_split, workspace, static_cast<int>(strips));
        rc = check_launch("ln_bwd_params_partial");
        if (rc) return;
        hipLaunchKernelGGL(ln_bwd_params_final<T>, dim3(static_cast<uint32_t>(strips)), dim3(kBlock), 0, s, workspace, cols,
                           static_cast<int>(splits), as<T>(dgamma), as<T>(dbeta));
        rc = check_launch("ln_bwd_params_final");
    });
    return rc;
}

extern "C" int ddl_ln_bwd_partial_params(const void* dy, const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld_dy,
                                         int64_t ld_x, const float* mean, const float* rstd, const void* gamma, float* sums,
                                         float* workspace, int64_t workspace_elems, void* stream) {
    using namespace ddl;
    const int elem = elem_bytes(dtype);
    if (!elem) return fail(DDL_E_UNSUPP, "ln backward sums: dtype %d (f32, bf16, f16 only)", dtype);
    if (int rc = check_rows("ln backward sums", rows, cols, ld_dy, ld_x)) return rc;
    if (!workspace) return fail(DDL_E_ARG, "ln backward sums: null workspace");
    const int64_t splits = param_splits(rows, cols, workspace_elems);
    if (splits < 1) return fail(DDL_E_ARG, "ln backward sums: workspace of %lld floats is smaller than 2 x %lld", (long long)workspace_elems, (long long)cols);
    if (rows > 0 && (!dy || !x || !mean || !rstd || !sums)) return fail(DDL_E_ARG, "ln backward sums: null pointer");
    if (!elems_aligned(elem, {dy, x, gamma}) || !aligned_to(mean, 4) || !aligned_to(rstd, 4) || !aligned_to(sums, 8) || !aligned_to(workspace, 4))
        return fail(DDL_E_ALIGN, "ln backward sums: elements must be aligned to their size, fp32 arrays to 4 bytes, the sums to 8");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t rows_per_split = rows > 0 ? (rows + splits - 1) / splits : 1;
    if (rows > 0 && cols <= 4 * kWave * 4 && vectorizable(elem, cols, {ld_dy, ld_x}, {dy, x, gamma})) {
        const dim3 grid(static_cast<uint32_t>(splits));
        with_ln_element(dtype, [&](auto* tag) {
            using T = std::remove_pointer_t<decltype(tag)>;
            if (cols <= kWave * 4)
                hipLaunchKernelGGL((ln_bwd_partial_cols<T, 1, false>), grid, dim3(kFusedBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd, as<T>(gamma), sums, rows_per_split, workspace, DxArgs{});
            else if (cols <= 2 * kWave * 4)
                hipLaunchKernelGGL((ln_bwd_partial_cols<T, 2, false>), grid, dim3(kFusedBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd, as<T>(gamma), sums, rows_per_split, workspace, DxArgs{});
            else
                hipLaunchKernelGGL((ln_bwd_partial_cols<T, 4, false>), grid, dim3(kFusedBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd, as<T>(gamma), sums, rows_per_split, workspace, DxArgs{});
        });
        return check_launch("ln_bwd_partial_cols");
    }
    // long or unaligned rows: the two passes separately, same results in the same places
    if (rows > 0) {
        if (int rc = ddl_ln_bwd_partial(dy, x, dtype, rows, cols, ld_dy, ld_x, mean, rstd, gamma, sums, stream)) return rc;
    }
    const int64_t strips = (cols + kStrip - 1) / kStrip;
    if (strips * splits > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "ln backward sums: too many workgroups");
    with_ln_element(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        hipLaunchKernelGGL(ln_bwd_params_partial<T>, dim3(static_cast<uint32_t>(strips * splits)), dim3(kBlock), 0, s, as<T>(dy), as<T>(x), rows,
                           cols, ld_dy, ld_x, mean, rstd, rows_per_split, workspace, static_cast<int>(strips));
    });
    return check_launch("ln_bwd_params_partial");
}

extern "C" int ddl_ln_bwd_input_params(const void* dy, const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld_dy,
                                       int64_t ld_x, const float* mean, const float* rstd, const void* gamma, const float* part_sums,
                                       int nparts, float weight, void* dx, int64_t ld_dx, const float* workspace,
                                       int64_t workspace_elems, void* dgamma, void* dbeta, void* stream) {
    using namespace ddl;
    const int elem = elem_bytes(dtype);
    if (!elem) return fail(DDL_E_UNSUPP, "ln backward input: dtype %d (f32, bf16, f16 only)", dtype);
    if (int rc = check_rows("ln backward input", rows, cols, ld_dy, ld_x)) return rc;
    if (ld_dx < cols || nparts < 1) return fail(DDL_E_ARG, "ln backward input: ld_dx=%lld nparts=%d", (long long)ld_dx, nparts);
    if (!workspace) return fail(DDL_E_ARG, "ln backward input: null workspace");
    const int64_t splits = param_splits(rows, cols, workspace_elems);
    if (splits < 1) return fail(DDL_E_ARG, "ln backward input: workspace of %lld floats is smaller than 2 x %lld", (long long)workspace_elems, (long long)cols);
    if (rows > 0 && (!dy || !x || !mean || !rstd || !part_sums || !dx)) return fail(DDL_E_ARG, "ln backward input: null pointer");
    if (!elems_aligned(elem, {dy, x, gamma, dx, dgamma, dbeta}) || !aligned_to(mean, 4) || !aligned_to(rstd, 4) || !aligned_to(part_sums, 8) ||
        !aligned_to(workspace, 4))
        return fail(DDL_E_ALIGN, "ln backward input: elements must be aligned to their size, fp32 arrays to 4 bytes, the sums to 8");
    const int64_t input_blocks = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
    const int64_t strips = (dgamma || dbeta) ? (cols + kStrip - 1) / kStrip : 0;
    if (input_blocks + strips == 0) return 0;
    if (input_blocks + strips > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "ln backward input: too many workgroups");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<uint32_t>(input_blocks + strips));
    const bool vec = vectorizable(elem, cols, {ld_dy, ld_x, ld_dx}, {dy, x, gamma, dx});
    with_ln_element(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (vec)
            hipLaunchKernelGGL((ln_bwd_input_final<T, true>), grid, dim3(kBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd,
                               as<T>(gamma), part_sums, nparts, weight, as<T>(dx), ld_dx, static_cast<uint32_t>(strips), workspace,
                               static_cast<int>(splits), as<T>(dgamma), as<T>(dbeta));
        else
            hipLaunchKernelGGL((ln_bwd_input_final<T, false>), grid, dim3(kBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd,
                               as<T>(gamma), part_sums, nparts, weight, as<T>(dx), ld_dx, static_cast<uint32_t>(strips), workspace,
                               static_cast<int>(splits), as<T>(dgamma), as<T>(dbeta));
    });
    return check_launch("ln_bwd_input_final");
}

extern "C" int ddl_ln_bwd_one_pass(const void* dy, const void* x, int dtype, int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x,
                                   const float* mean, const float* rstd, const void* gamma, float* part_sums, int nparts, int my_part,
                                   float weight, void* dx, int64_t ld_dx, float* workspace, int64_t workspace_elems, void* dgamma,
                                   void* dbeta, void* stream) {
    using namespace ddl;
    const int elem = elem_bytes(dtype);
    if (!elem) return fail(DDL_E_UNSUPP, "ln backward (one pass): dtype %d (f32, bf16, f16 only)", dtype);
    if (int rc = check_rows("ln backward (one pass)", rows, cols, ld_dy, ld_x)) return rc;
    if (ld_dx < cols) return fail(DDL_E_ARG, "ln backward (one pass): ld_dx=%lld below cols=%lld", (long long)ld_dx, (long long)cols);
    if (nparts < 1 || nparts > kWave) return fail(DDL_E_UNSUPP, "ln backward (one pass): nparts=%d outside [1,%d]", nparts, kWave);
    if (my_part < 0 || my_part >= nparts) return fail(DDL_E_ARG, "ln backward (one pass): my_part=%d outside [0,%d)", my_part, nparts);
    if (nparts > 1 && !part_sums) return fail(DDL_E_ARG, "ln backward (one pass): the other workers' sums are missing");
    if (!workspace) return fail(DDL_E_ARG, "ln backward (one pass): null workspace");
    const int64_t splits = param_splits(rows, cols, workspace_elems);
    if (splits < 1) return fail(DDL_E_ARG, "ln backward (one pass): workspace of %lld floats is smaller than 2 x %lld", (long long)workspace_elems, (long long)cols);
    if (rows > 0 && (!dy || !x || !mean || !rstd || !dx)) return fail(DDL_E_ARG, "ln backward (one pass): null pointer");
    if (!elems_aligned(elem, {dy, x, gamma, dx, dgamma, dbeta}) || !aligned_to(mean, 4) || !aligned_to(rstd, 4) || !aligned_to(part_sums, 8) ||
        !aligned_to(workspace, 4))
        return fail(DDL_E_ALIGN, "ln backward (one pass): elements must be aligned to their size, fp32 arrays to 4 bytes, the sums to 8");
    if (cols > 4 * kWave * 4 || !vectorizable(elem, cols, {ld_dy, ld_x, ld_dx}, {dy, x, gamma, dx}))
        return fail(DDL_E_UNSUPP, "ln backward (one pass): rows of at most %d columns, columns and pitches multiples of 4, pointers aligned to 4 elements", 4 * kWave * 4);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t strips = (dgamma || dbeta) ? (cols + kStrip - 1) / kStrip : 0;
    if (rows > 0) {
        const int64_t rows_per_split = (rows + splits - 1) / splits;
        float* sums = part_sums ? part_sums + static_cast<int64_t>(my_part) * rows * 2 : nullptr;
        const DxArgs dxa{part_sums, nparts, my_part, weight, dx, ld_dx};
        const dim3 grid(static_cast<uint32_t>(splits));
        with_ln_element(dtype, [&](auto* tag) {
            using T = std::remove_pointer_t<decltype(tag)>;
            if (cols <= kWave * 4)
                hipLaunchKernelGGL((ln_bwd_partial_cols<T, 1, true>), grid, dim3(kFusedBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd, as<T>(gamma), sums, rows_per_split, workspace, dxa);
            else if (cols <= 2 * kWave * 4)
                hipLaunchKernelGGL((ln_bwd_partial_cols<T, 2, true>), grid, dim3(kFusedBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd, as<T>(gamma), sums, rows_per_split, workspace, dxa);
            else
                hipLaunchKernelGGL((ln_bwd_partial_cols<T, 4, true>), grid, dim3(kFusedBlock), 0, s, as<T>(dy), as<T>(x), rows, cols, ld_dy, ld_x, mean, rstd, as<T>(gamma), sums, rows_per_split, workspace, dxa);
        });
        if (int rc = check_launch("ln_bwd_partial_cols")) return rc;
    }
    if (strips == 0) return 0;
    with_ln_element(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        hipLaunchKernelGGL(ln_bwd_params_final<T>, dim3(static_cast<uint32_t>(strips)), dim3(kBlock), 0, s, workspace, cols,
                           static_cast<int>(rows > 0 ? splits : 0), as<T>(dgamma), as<T>(dbeta));
    });
    return check_launch("ln_bwd_params_final");
}

// The float32 forms.
extern "C" int ddl_ln_bwd_partial_f32(const float* dy, const float* x, int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x,
                                      const float* mean, const float* rstd, const float* gamma, float* sums, void* stream) {
    return ddl_ln_bwd_partial(dy, x, DDL_DT_F32, rows, cols, ld_dy, ld_x, mean, rstd, gamma, sums, stream);
}
extern "C" int ddl_ln_bwd_input_f32(const float* dy, const float* x, int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x,
                                    const float* mean, const float* rstd, const float* gamma, const float* part_sums,
                                    int nparts, float weight, float* dx, int64_t ld_dx, void* stream) {
    return ddl_ln_bwd_input(dy, x, DDL_DT_F32, rows, cols, ld_dy, ld_x, mean, rstd, gamma, part_sums, nparts, weight, dx, ld_dx, stream);
}
extern "C" int ddl_ln_bwd_params_f32(const float* dy, const float* x, int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x,
                                     const float* mean, const float* rstd, float* dgamma, float* dbeta, float* workspace,
                                     int64_t workspace_elems, void* stream) {
    return ddl_ln_bwd_params(dy, x, DDL_DT_F32, rows, cols, ld_dy, ld_x, mean, rstd, dgamma, dbeta, workspace, workspace_elems, stream);
}
extern "C" int ddl_ln_bwd_partial_params_f32(const float* dy, const float* x, int64_t rows, int64_t cols, int64_t ld_dy,
                                             int64_t ld_x, const float* mean, const float* rstd, const float* gamma, float* sums,
                                             float* workspace, int64_t workspace_elems, void* stream) {
    return ddl_ln_bwd_partial_params(dy, x, DDL_DT_F32, rows, cols, ld_dy, ld_x, mean, rstd, gamma, sums, workspace, workspace_elems, stream);
}
extern "C" int ddl_ln_bwd_input_params_f32(const float* dy, const float* x, int64_t rows, int64_t cols, int64_t ld_dy, int64_t ld_x,
                                           const float* mean, const float* rstd, const float* gamma, const float* part_sums,
                                           int nparts, float weight, float* dx, int64_t ld_dx, const float* workspace,
                                           int64_t workspace_elems, float* dgamma, float* dbeta, void* stream) {
    return ddl_ln_bwd_input_params(dy, x, DDL_DT_F32, rows, cols, ld_dy, ld_x, mean, rstd, gamma, part_sums, nparts, weight, dx, ld_dx,
                                   workspace, workspace_elems, dgamma, dbeta, stream);
}
