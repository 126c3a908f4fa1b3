// ifa_f32_common.h -- device helpers of the kernels that keep activations, the residual stream and every recurrent
// state in 32-bit floats and read their weights as bfloat16 (the layer-list worker, ifa_engine_layered.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ifa32 {

typedef uint16_t bf16_t;      // bit pattern of a bfloat16

__host__ __device__ __forceinline__ float bf2f(bf16_t b)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __uint_as_float((uint32_t)b << 16);
#else
    uint32_t u = (uint32_t)b << 16; float f; __builtin_memcpy(&f, &u, 4); return f;
#endif
}

// round to nearest even (inputs are finite here)
__device__ __forceinline__ bf16_t f2bf(float f)
{
    uint32_t u = __float_as_uint(f);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// sum over the four lanes 4 q .. 4 q + 3 (two DPP quad permutes); every one of them gets the result
__device__ __forceinline__ float quad_sum(float v)
{
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));      // lanes ^ 1
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));      // lanes ^ 2
    return v;
}

// sum over the eight lanes 8 q .. 8 q + 7: the quad sums, then the other quad's through a half-row mirror (lane i <-> 7 - i)
__device__ __forceinline__ float oct_sum(float v)
{
    v = quad_sum(v);
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));
    return v;
}

// sum over the sixteen lanes 16 q .. 16 q + 15 (a DPP row): the oct sums, then the other half's through a rotation of the row by 8
__device__ __forceinline__ float hex_sum(float v)
{
    v = oct_sum(v);
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x128, 0xF, 0xF, true));
    return v;
}

// sum over a workgroup of up to 1024 threads; red: 17 floats of LDS; every thread gets the result
__device__ __forceinline__ float block_sum(float v, float *red)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nw; w++) t += red[w];
    return t;
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + __expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu_exact(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float gelu_tanh_f(float z)
{
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// One sequence of a step: rows [row0, row0 + n) of the step's activation tensors are the tokens at positions
// [pos0, pos0 + n) of the sequence whose cache / state lives in slot `slot`.
struct SeqDesc { int row0, n, pos0, slot; };

} // namespace ifa32
