// 16-byte streaming loads / stores and the f32 / bf16 storage traits shared by the elementwise kernels.
#ifndef MIQ_IO_H
#define MIQ_IO_H

#include "miq_common.h"

namespace miq
{
// ------------------------------------------------------------------------------------------------ IO vector types
// Streaming accesses are marked non-temporal: every byte is touched exactly once, and on this part that alone is
// worth about 10 % of bandwidth for both the read-once inputs and the write-once outputs.
typedef float nt_f4 __attribute__((ext_vector_type(4)));
typedef unsigned int nt_u4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float4 stream_load(const float4* p)
{
    const nt_f4 v = __builtin_nontemporal_load(reinterpret_cast<const nt_f4*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint4 stream_load(const uint4* p)
{
    const nt_u4 v = __builtin_nontemporal_load(reinterpret_cast<const nt_u4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stream_store(float4* p, const float4& v)
{
    const nt_f4 w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, reinterpret_cast<nt_f4*>(p));
}
__device__ __forceinline__ void stream_store(uint4* p, const uint4& v)
{
    const nt_u4 w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, reinterpret_cast<nt_u4*>(p));
}

template <typename IO>
struct IOTraits;

template <>
struct IOTraits<float>
{
    using Vec                = float4;
    static constexpr int VEC = 4;
    __device__ static void unpack(const Vec& v, float* f)
    {
        f[0] = v.x;
        f[1] = v.y;
        f[2] = v.z;
        f[3] = v.w;
    }
    __device__ static Vec pack(const float* f)
    {
        return make_float4(f[0], f[1], f[2], f[3]);
    }
    __device__ static Vec pack_no_nan(const float* f)
    {
        return pack(f);
    }
    __device__ static float load1(const float* p)
    {
        return *p;
    }
    __device__ static void store1(float* p, float v)
    {
        *p = v;
    }
};

template <>
struct IOTraits<uint16_t>
{
    using Vec                = uint4;
    static constexpr int VEC = 8;
    __device__ static void unpack(const Vec& v, float* f)
    {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            f[2 * i]     = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ static Vec pack(const float* f)
    {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = f32x2_to_bf16x2(f[2 * i], f[2 * i + 1]);
        return make_uint4(w[0], w[1], w[2], w[3]);
    }
    // for results that cannot be NaN: the canonicalisation of pack() costs three to four operations per element, which
    // the bf16 forward kernel -- bound by instruction issue, not by HBM -- feels
    __device__ static Vec pack_no_nan(const float* f)
    {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = f32x2_to_bf16x2_no_nan(f[2 * i], f[2 * i + 1]);
        return make_uint4(w[0], w[1], w[2], w[3]);
    }
    __device__ static float load1(const uint16_t* p)
    {
        return bf16_to_f32(*p);
    }
    __device__ static void store1(uint16_t* p, float v)
    {
        *p = (uint16_t) f32_to_bf16(v);
    }
};

}   // namespace miq

#endif
