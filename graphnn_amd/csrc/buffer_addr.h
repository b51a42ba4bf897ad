// Buffer addressing for gfx950 kernels: a 128-bit resource descriptor (base, byte count) in
// scalar registers plus a 32-bit byte offset per lane.  The hardware compares the offset with
// the byte count: a load past the end returns zeros without touching memory and a store past
// the end is dropped, which replaces predicates and branches around memory instructions.
// A buffer covers less than 4 GiB.
#ifndef GNNHIP_BUFFER_ADDR_H
#define GNNHIP_BUFFER_ADDR_H

#include <hip/hip_runtime.h>

namespace gnnhip {

using rsrc_t = __amdgpu_buffer_rsrc_t;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
constexpr int kRsrcWord3 = 0x00020000;       // raw buffer of 32-bit data on gfx9-family hardware
constexpr int kBufPastEnd = -1;              // byte offset 0xFFFFFFFF: out of range for every buffer

__device__ __forceinline__ rsrc_t make_rsrc(const void* base, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, kRsrcWord3);
}
__device__ __forceinline__ float4 buf_load4(rsrc_t r, int voff, int soff)
{
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}
__device__ __forceinline__ float2 buf_load2(rsrc_t r, int voff, int soff)
{
    const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
    return make_float2(__uint_as_float(v.x), __uint_as_float(v.y));
}
__device__ __forceinline__ int buf_load_i(rsrc_t r, int voff, int soff)
{
    return (int)__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0);
}
__device__ __forceinline__ float buf_load_f(rsrc_t r, int voff, int soff)
{
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ void buf_store4(rsrc_t r, int voff, int soff, const float4& x)
{
    const u32x4 v = {__float_as_uint(x.x), __float_as_uint(x.y), __float_as_uint(x.z), __float_as_uint(x.w)};
    __builtin_amdgcn_raw_buffer_store_b128(v, r, voff, soff, 0);
}

__device__ __forceinline__ void buf_store2(rsrc_t r, int voff, int soff, const float2& x)
{
    const u32x2 v = {__float_as_uint(x.x), __float_as_uint(x.y)};
    __builtin_amdgcn_raw_buffer_store_b64(v, r, voff, soff, 0);
}

}  // namespace gnnhip

#endif
