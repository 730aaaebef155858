// Element types of the LayerNorm kernels (float, bf16, fp16) and their loads and
// stores as fp32 values, one element or four consecutive ones at a time.
#ifndef DDL_LN_ELEMENTS_H
#define DDL_LN_ELEMENTS_H
#include "ddl_common.h"
#include <hip/hip_fp16.h>

namespace ddl {

struct bf16_t {
    uint16_t bits;
};

__device__ inline float bf16_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ inline uint32_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if (f != f) return 0x7FC0u;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return u >> 16;
}

// Sum over the 64 lanes of a wavefront, the same value in every lane.  Data
// moves between lanes inside the vector ALU (DPP: pairs, quads, half rows and
// rows of 16 lanes by mirroring, then lane 15 / 31 of the rows below broadcast
// into the rows above), six dependent additions of a few cycles each; the
// total ends in lane 63 and is read from there.  (A butterfly of __shfl_xor goes
// through the LDS crossbar six times, about a hundred cycles each, which at
// 8 MiB inputs was a tenth of a kernel's duration per reduction.)
template <int CTRL, int ROW_MASK>
__device__ inline float dpp_moved(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, false));
}
__device__ inline float wave_sum(float v) {
    v += dpp_moved<0xB1, 0xF>(v);    // quad_perm [1,0,3,2]
    v += dpp_moved<0x4E, 0xF>(v);    // quad_perm [2,3,0,1]
    v += dpp_moved<0x141, 0xF>(v);   // row_half_mirror
    v += dpp_moved<0x140, 0xF>(v);   // row_mirror: every lane holds the sum of its row of 16
    v += dpp_moved<0x142, 0xA>(v);   // row_bcast15 into rows 1 and 3
    v += dpp_moved<0x143, 0xC>(v);   // row_bcast31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Four consecutive elements as floats; what these kernels store is never read
// again by them, so it leaves with streaming stores.
__device__ inline float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ inline float4 load4(const bf16_t* p) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    return make_float4(bf16_to_f32(w.x & 0xFFFFu), bf16_to_f32(w.x >> 16), bf16_to_f32(w.y & 0xFFFFu), bf16_to_f32(w.y >> 16));
}
__device__ inline float4 load4(const __half* p) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    const __half2 a = *reinterpret_cast<const __half2*>(&w.x), b = *reinterpret_cast<const __half2*>(&w.y);
    const float2 fa = __half22float2(a), fb = __half22float2(b);
    return make_float4(fa.x, fa.y, fb.x, fb.y);
}
__device__ inline void store4(float* p, float4 v) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    f32x4 o;
    o[0] = v.x, o[1] = v.y, o[2] = v.z, o[3] = v.w;
    __builtin_nontemporal_store(o, reinterpret_cast<f32x4*>(p));
}
__device__ inline void store4(bf16_t* p, float4 v) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    u32x2 o;
    o[0] = f32_to_bf16(v.x) | (f32_to_bf16(v.y) << 16);
    o[1] = f32_to_bf16(v.z) | (f32_to_bf16(v.w) << 16);
    __builtin_nontemporal_store(o, reinterpret_cast<u32x2*>(p));
}
__device__ inline void store4(__half* p, float4 v) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const __half2 a = __floats2half2_rn(v.x, v.y), b = __floats2half2_rn(v.z, v.w);
    u32x2 o;
    o[0] = *reinterpret_cast<const uint32_t*>(&a);
    o[1] = *reinterpret_cast<const uint32_t*>(&b);
    __builtin_nontemporal_store(o, reinterpret_cast<u32x2*>(p));
}
__device__ inline float load1(const float* p) { return *p; }
__device__ inline float load1(const bf16_t* p) { return bf16_to_f32(p->bits); }
__device__ inline float load1(const __half* p) { return __half2float(*p); }
__device__ inline void store1(float* p, float v) { *p = v; }
__device__ inline void store1(bf16_t* p, float v) { p->bits = static_cast<uint16_t>(f32_to_bf16(v)); }
__device__ inline void store1(__half* p, float v) { *p = __float2half_rn(v); }

// Calls fn(T{}) with the element type that `dtype` names; false for any other dtype.
template <typename Fn>
inline bool with_ln_element(int dtype, Fn&& fn) {
    switch (dtype) {
        case DDL_DT_F32: fn(static_cast<float*>(nullptr)); return true;
        case DDL_DT_BF16: fn(static_cast<bf16_t*>(nullptr)); return true;
        case DDL_DT_F16: fn(static_cast<__half*>(nullptr)); return true;
        default: return false;
    }
}

}  // namespace ddl
#endif  // DDL_LN_ELEMENTS_H
