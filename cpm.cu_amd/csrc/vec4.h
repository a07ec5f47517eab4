// Four columns a thread with 16-byte accesses: what the row kernels of steps with few rows share (a row's work
// spread over up to 1024 threads, a branch's partial sums asked for together).
#pragma once
#include "common.h"

__device__ inline void store4(float* p, float a, float b, float c, float d) { *(float4*)p = make_float4(a, b, c, d); }
__device__ inline void store4(bf16_t* p, float a, float b, float c, float d) {
    const bf16_t o0 = f32_to_bf16(a), o1 = f32_to_bf16(b), o2 = f32_to_bf16(c), o3 = f32_to_bf16(d);
    *(uint2*)p = make_uint2((uint32_t)o0.v | ((uint32_t)o1.v << 16), (uint32_t)o2.v | ((uint32_t)o3.v << 16));
}
__device__ inline float4 load4(const float* p) { return *(const float4*)p; }
__device__ inline float4 load4(const bf16_t* p) {
    const uint2 u = *(const uint2*)p;
    float4 r;
    r.x = __uint_as_float(u.x << 16);
    r.y = __uint_as_float(u.x & 0xffff0000u);
    r.z = __uint_as_float(u.y << 16);
    r.w = __uint_as_float(u.y & 0xffff0000u);
    return r;
}
// acc + the partial results first .. first + W - 1 (of nparts, `stride` elements apart), added in the order of
// the parts.  The W loads are asked for together: a loop of single loads whose trip count the compiler does not
// know waits for each load before it asks for the next, a trip to memory a part.  A part beyond the last repeats
// the last one and is not added.
template <int W, typename BT>
__device__ inline float4 add_parts4(float4 acc, const BT* p, int first, int nparts, long stride) {
    float4 t[W];
#pragma unroll
    for (int j = 0; j < W; ++j) t[j] = load4(p + (long)min(first + j, nparts - 1) * stride);
#pragma unroll
    for (int j = 0; j < W; ++j)
        if (first + j < nparts) {
            acc.x += t[j].x; acc.y += t[j].y; acc.z += t[j].z; acc.w += t[j].w;
        }
    return acc;
}
template <typename BT>
__device__ inline float4 sum_parts4(const BT* p, int nparts, long stride) {
    float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
    if (nparts <= 4) return add_parts4<4>(b, p, 0, nparts, stride);
    for (int f = 0; f < nparts; f += 8) b = add_parts4<8>(b, p, f, nparts, stride);
    return b;
}

