// Device-side helpers shared by the gfx950 kernels: 16-byte vector access,
// fp16/bf16 dot products with fp32 accumulation, and 16-lane DPP reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlora {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf162_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf168_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int DT_F16 = 0;
constexpr int DT_BF16 = 1;

__device__ __forceinline__ uint4 ldg16(const void *p) { return *reinterpret_cast<const uint4 *>(p); }
__device__ __forceinline__ void stg16(void *p, uint4 v) { *reinterpret_cast<uint4 *>(p) = v; }
__device__ __forceinline__ uint4 zero16() { return make_uint4(0u, 0u, 0u, 0u); }

// The same address seen as constant memory (address space 4): data that no launch of the running kernel writes
// (work records, tile records and sums written by an earlier launch).  A load through such a pointer whose address
// is uniform over the wavefront is a scalar load into SGPRs; through an ordinary global pointer the compiler only
// does that while it can prove that no store of the kernel comes before the load, which a loop over work items
// with a store at its end rules out.
template <class T>
__device__ __forceinline__ const __attribute__((address_space(4))) T *as_const(const T *p)
{
    return (const __attribute__((address_space(4))) T *)(__UINTPTR_TYPE__)p;
}
typedef const __attribute__((address_space(4))) int32_t *const_i32_ptr;

// Streaming forms for data that is read or written once per launch (adapter rows, activations,
// outputs): the nontemporal hint keeps these lines from displacing the small data every workgroup
// re-reads (work records, partial sums) and measurably shortens the launches.
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ldg16_stream(const void *p)
{
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stg16_stream(void *p, uint4 v)
{
    const u32x4_t w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t *>(p));
}

// acc + sum_{e<2} a[e]*b[e], both 16-bit pairs packed in one dword, fp32 accumulate.
template <int DT>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc)
{
    if constexpr (DT == DT_F16) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), acc, false);
    } else {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf162_t, a), __builtin_bit_cast(bf162_t, b), acc, false);
    }
}

template <int DT>
__device__ __forceinline__ float dot8(const uint4 &a, const uint4 &b, float acc)
{
    acc = dot2<DT>(a.x, b.x, acc);
    acc = dot2<DT>(a.y, b.y, acc);
    acc = dot2<DT>(a.z, b.z, acc);
    acc = dot2<DT>(a.w, b.w, acc);
    return acc;
}

// low / high 16-bit lane of a dword as fp32
template <int DT>
__device__ __forceinline__ float lo_f32(uint32_t u)
{
    if constexpr (DT == DT_F16) return (float)__builtin_bit_cast(half2_t, u)[0];
    else return __builtin_bit_cast(float, u << 16);
}
template <int DT>
__device__ __forceinline__ float hi_f32(uint32_t u)
{
    if constexpr (DT == DT_F16) return (float)__builtin_bit_cast(half2_t, u)[1];
    else return __builtin_bit_cast(float, u & 0xffff0000u);
}

template <int DT>
__device__ __forceinline__ void unpack8(const uint4 &v, float (&f)[8])
{
    f[0] = lo_f32<DT>(v.x); f[1] = hi_f32<DT>(v.x);
    f[2] = lo_f32<DT>(v.y); f[3] = hi_f32<DT>(v.y);
    f[4] = lo_f32<DT>(v.z); f[5] = hi_f32<DT>(v.z);
    f[6] = lo_f32<DT>(v.w); f[7] = hi_f32<DT>(v.w);
}

// fp32 -> 16-bit pattern, round to nearest even.
template <int DT>
__device__ __forceinline__ uint32_t cvt16(float f)
{
    if constexpr (DT == DT_F16) {
        return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
    } else {
        uint32_t u = __builtin_bit_cast(uint32_t, f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x0040u;
        u += 0x7fffu + ((u >> 16) & 1u);
        return u >> 16;
    }
}

template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
    if constexpr (DT == DT_F16) {
        // Converted as a pair (v_cvt_pk_f16_f32).  A scalar conversion can be folded by the compiler
        // into the last multiply-add of a chain (v_fma_mixlo_f16), which rounds the exact sum to 16
        // bits in one step; it does so for some outputs and not for others, so results would depend
        // on register allocation.  Every output is rounded fp32 -> fp16 here.
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    } else {
        // v_cvt_pk_bf16_f32: round to nearest even in one instruction (cvt16's integer sequence costs six);
        // the same bits for every finite input and infinity, NaN payloads may differ
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
}

template <int DT>
__device__ __forceinline__ uint4 pack8(const float (&f)[8])
{
    return make_uint4(pack2<DT>(f[0], f[1]), pack2<DT>(f[2], f[3]), pack2<DT>(f[4], f[5]), pack2<DT>(f[6], f[7]));
}

// Sum over each aligned group of 16 lanes (a DPP "row"); every lane of the row gets the sum.
__device__ __forceinline__ float row16_sum(float v)
{
    // quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false));
    return v;
}

// Sum over the 64 lanes of a wavefront; every lane gets the sum.
__device__ __forceinline__ float wave_sum(float v)
{
    v = row16_sum(v);
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

}  // namespace mlora
