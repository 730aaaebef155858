// DistributedEmbedding shard gather (reference: nn/embedding.py:244-246,
// torch.nn.functional.embedding on the local table).  out[t] is row ids[t]-lo of
// the table when lo <= ids[t] < hi and a row of zero bits otherwise.  Rows are
// opaque bytes: one wavefront moves one token's row as 16-byte vectors, eight
// vectors per lane in flight; misses issue no loads at all.
//
// max_norm (the renormalisation F.embedding performs before the lookup): the
// rows that are looked up are flagged, then one wavefront per flagged row forms
// the p-norm in fp32 and, where it exceeds max_norm, scales the row in place by
// max_norm / (norm + 1e-7) -- once per row however often it is looked up.
#include "ddl_common.h"
#include "ln_elements.h"

namespace ddl {
namespace {

constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kInFlight = 8;
// The gather runs two tokens per workgroup.  Workgroups go to the eight XCDs in
// turn, so a workgroup's bytes decide which address bits an XCD's stores agree
// in: with rows of 8 KiB, four tokens per workgroup (bits 15-17) take 200.0 us on
// configuration 3, two (14-16) 199.0, one 198.0 -- and eight (16-18) 210.
constexpr int kGatherBlock = 128;
constexpr int kGatherWaves = kGatherBlock / kWave;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

template <typename V, typename IdT>
__global__ __launch_bounds__(kGatherBlock) void gather_rows(const char* __restrict__ weight, int64_t ldw_bytes, int64_t nvec,
                                                      const IdT* __restrict__ ids, int64_t n_ids, int64_t lo, int64_t hi,
                                                      char* __restrict__ out) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kGatherWaves + threadIdx.x / kWave;
    if (t >= n_ids) return;
    const int64_t id = static_cast<int64_t>(ids[t]);
    const bool hit = id >= lo && id < hi;
    V* dst = reinterpret_cast<V*>(out + t * nvec * static_cast<int64_t>(sizeof(V)));
    if (!hit) {
        V z;
        __builtin_memset(&z, 0, sizeof(V));
        for (int64_t c = lane; c < nvec; c += kWave) __builtin_nontemporal_store(z, dst + c);
        return;
    }
    const V* src = reinterpret_cast<const V*>(weight + (id - lo) * ldw_bytes);
    for (int64_t c0 = 0; c0 < nvec; c0 += kWave * kInFlight) {
        V v[kInFlight];
#pragma unroll
        for (int k = 0; k < kInFlight; ++k) {
            const int64_t c = c0 + lane + k * kWave;
            if (c < nvec) v[k] = src[c];
        }
#pragma unroll
        for (int k = 0; k < kInFlight; ++k) {
            const int64_t c = c0 + lane + k * kWave;
            if (c < nvec) __builtin_nontemporal_store(v[k], dst + c);
        }
    }
}

template <typename V>
int launch_gather(const void* w, int64_t ldw_bytes, int64_t row_bytes, const void* ids, int i64, int64_t n, int64_t lo,
                  int64_t hi, void* out, hipStream_t s) {
    const int64_t nvec = row_bytes / static_cast<int64_t>(sizeof(V));
    const int64_t blocks = (n + kGatherWaves - 1) / kGatherWaves;
    if (blocks > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "embedding gather: more than 2^32 ids in one call");
    if (i64)
        hipLaunchKernelGGL((gather_rows<V, int64_t>), dim3(static_cast<uint32_t>(blocks)), dim3(kGatherBlock), 0, s,
                           static_cast<const char*>(w), ldw_bytes, nvec, static_cast<const int64_t*>(ids), n, lo, hi,
                           static_cast<char*>(out));
    else
        hipLaunchKernelGGL((gather_rows<V, int32_t>), dim3(static_cast<uint32_t>(blocks)), dim3(kGatherBlock), 0, s,
                           static_cast<const char*>(w), ldw_bytes, nvec, static_cast<const int32_t*>(ids), n, lo, hi,
                           static_cast<char*>(out));
    return check_launch("gather_rows");
}

__global__ __launch_bounds__(kBlock) void renorm_clear(int32_t* __restrict__ flags, int64_t rows) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < rows) flags[i] = 0;
}

template <typename IdT>
__global__ __launch_bounds__(kBlock) void renorm_mark(const IdT* __restrict__ ids, int64_t n_ids, int64_t lo, int64_t hi,
                                                      int32_t* __restrict__ flags) {
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (t >= n_ids) return;
    const int64_t id = static_cast<int64_t>(ids[t]);
    if (id >= lo && id < hi) flags[id - lo] = 1;   // every writer stores the same value
}

__device__ inline float wave_max(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// kind: 1 = sum of magnitudes, 2 = Euclidean, 3 = maximum, 0 = general p.
template <typename T>
__global__ __launch_bounds__(kBlock) void renorm_rows(T* __restrict__ weight, int64_t rows, int64_t dim, int64_t ldw,
                                                      const int32_t* __restrict__ flags, float max_norm, float p, int kind) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + threadIdx.x / kWave;
    if (row >= rows || flags[row] == 0) return;   // the same for all lanes of the wavefront
    T* w = weight + row * ldw;
    float acc = 0.f;
    for (int64_t c = lane; c < dim; c += kWave) {
        const float a = fabsf(load1(w + c));
        if (kind == 1)
            acc += a;
        else if (kind == 2)
            acc += a * a;
        else if (kind == 3)
            acc = fmaxf(acc, a);
        else
            acc += powf(a, p);
    }
    float norm;
    if (kind == 3) {
        norm = wave_max(acc);
    } else {
        const float total = wave_sum(acc);
        norm = kind == 1 ? total : kind == 2 ? sqrtf(total) : powf(total, 1.f / p);
    }
    if (!(norm > max_norm)) return;
    const float scale = max_norm / (norm + 1e-7f);
    for (int64_t c = lane; c < dim; c += kWave) store1(w + c, load1(w + c) * scale);
}

}  // namespace
}  // namespace ddl

extern "C" int ddl_embedding_renorm(void* weight, int dtype, int64_t dim, int64_t ldw, const void* ids, int ids_is_i64,
                                    int64_t n_ids, int64_t lo, int64_t hi, float max_norm, float norm_type, int32_t* flags,
                                    void* stream) {
    using namespace ddl;
    if (dim < 1 || ldw < dim || n_ids < 0 || hi < lo)
        return fail(DDL_E_ARG, "embedding renorm: dim=%lld ldw=%lld n_ids=%lld window=[%lld,%lld)", (long long)dim,
                    (long long)ldw, (long long)n_ids, (long long)lo, (long long)hi);
    if (!(max_norm >= 0.f) || !(norm_type > 0.f))
        return fail(DDL_E_ARG, "embedding renorm: max_norm=%g norm_type=%g", (double)max_norm, (double)norm_type);
    const int64_t rows = hi - lo;
    if (n_ids == 0 || rows == 0) return 0;
    if (!weight || !ids || !flags) return fail(DDL_E_ARG, "embedding renorm: null pointer");
    if (!aligned_to(ids, ids_is_i64 ? 8 : 4) || !aligned_to(flags, 4)) return fail(DDL_E_ALIGN, "embedding renorm: ids or flags misaligned");
    const int64_t row_blocks = (rows + kWavesPerBlock - 1) / kWavesPerBlock, id_blocks = (n_ids + kBlock - 1) / kBlock;
    if (row_blocks > 0x7FFFFFFFll || id_blocks > 0x7FFFFFFFll) return fail(DDL_E_UNSUPP, "embedding renorm: too many rows or ids for one call");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int kind = norm_type == 1.f ? 1 : norm_type == 2.f ? 2 : std::isinf(norm_type) ? 3 : 0;
    int rc = 0;
    const bool known = with_ln_element(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (!aligned_to(weight, sizeof(T))) {
            rc = fail(DDL_E_ALIGN, "embedding renorm: table not aligned to its element size");
            return;
        }
        hipLaunchKernelGGL(renorm_clear, dim3(static_cast<uint32_t>((rows + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, flags, rows);
        if (ids_is_i64)
            hipLaunchKernelGGL(renorm_mark<int64_t>, dim3(static_cast<uint32_t>(id_blocks)), dim3(kBlock), 0, s,
                               static_cast<const int64_t*>(ids), n_ids, lo, hi, flags);
        else
            hipLaunchKernelGGL(renorm_mark<int32_t>, dim3(static_cast<uint32_t>(id_blocks)), dim3(kBlock), 0, s,
                               static_cast<const int32_t*>(ids), n_ids, lo, hi, flags);
        hipLaunchKernelGGL(renorm_rows<T>, dim3(static_cast<uint32_t>(row_blocks)), dim3(kBlock), 0, s, static_cast<T*>(weight), rows,
                           dim, ldw, flags, max_norm, norm_type, kind);
        rc = check_launch("renorm_rows");
    });
    if (!known) return fail(DDL_E_UNSUPP, "embedding renorm: dtype %d (f32, bf16 and f16 only)", dtype);
    return rc;
}

extern "C" int ddl_embedding_gather(const void* weight, int64_t dim, int64_t ldw, int elem_size, const void* ids,
                                    int ids_is_i64, int64_t n_ids, int64_t lo, int64_t hi, void* out, void* stream) {
    using namespace ddl;
    if (dim < 1 || ldw < dim || n_ids < 0 || hi < lo)
        return fail(DDL_E_ARG, "embedding gather: dim=%lld ldw=%lld n_ids=%lld window=[%lld,%lld)", (long long)dim,
                    (long long)ldw, (long long)n_ids, (long long)lo, (long long)hi);
    if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8)
        return fail(DDL_E_ARG, "embedding gather: element size %d not in {1,2,4,8}", elem_size);
    if (n_ids == 0) return 0;
    if (!ids || !out || (!weight && hi > lo)) return fail(DDL_E_ARG, "embedding gather: null pointer");
    if (!aligned_to(ids, ids_is_i64 ? 8 : 4)) return fail(DDL_E_ALIGN, "embedding gather: ids misaligned");
    if (!aligned_to(out, elem_size) || !aligned_to(weight, elem_size))
        return fail(DDL_E_ALIGN, "embedding gather: table or output not aligned to the element size");
    const int64_t row_bytes = dim * elem_size, ldw_bytes = ldw * elem_size;
    const uint64_t bits = static_cast<uint64_t>(row_bytes) | static_cast<uint64_t>(ldw_bytes) |
                          reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if ((bits & 15) == 0) return launch_gather<u32x4>(weight, ldw_bytes, row_bytes, ids, ids_is_i64, n_ids, lo, hi, out, s);
    if ((bits & 7) == 0) return launch_gather<u32x2>(weight, ldw_bytes, row_bytes, ids, ids_is_i64, n_ids, lo, hi, out, s);
    if ((bits & 3) == 0) return launch_gather<uint32_t>(weight, ldw_bytes, row_bytes, ids, ids_is_i64, n_ids, lo, hi, out, s);
    if ((bits & 1) == 0) return launch_gather<uint16_t>(weight, ldw_bytes, row_bytes, ids, ids_is_i64, n_ids, lo, hi, out, s);
    return launch_gather<uint8_t>(weight, ldw_bytes, row_bytes, ids, ids_is_i64, n_ids, lo, hi, out, s);
}
