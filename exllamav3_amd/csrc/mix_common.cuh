// Device helpers of the sequence-mixer library (libexl3_mix.so): element types, conversions, reductions.  gfx950 only (wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include "../../include/exl3_mix.h"

struct bf16_t { uint16_t u; };

__device__ __forceinline__ float to_f(bf16_t v) { return __uint_as_float(((uint32_t) v.u) << 16); }
__device__ __forceinline__ float to_f(float v) { return v; }

template <typename T> __device__ __forceinline__ T from_f(float f);
template <> __device__ __forceinline__ bf16_t from_f<bf16_t>(float f)
{
    const __bf16 h = (__bf16) f;                     // the hardware's conversion: round to nearest, ties to even
    bf16_t r;
    __builtin_memcpy(&r.u, &h, sizeof(r.u));
    return r;
}
template <> __device__ __forceinline__ float from_f<float>(float f) { return f; }

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

// sum over each row of 16 consecutive lanes, every lane of the row gets it: two quad permutes, then the mirror within 8 and within 16 lanes (data-parallel
// primitives of the vector unit: no trip through the LDS crossbar)
__device__ __forceinline__ float row16_sum(float v)
{
    #define MIX_DPP(x, ctrl) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), ctrl, 0xf, 0xf, true))
    v += MIX_DPP(v, 0xB1);
    v += MIX_DPP(v, 0x4E);
    v += MIX_DPP(v, 0x141);
    v += MIX_DPP(v, 0x140);
    #undef MIX_DPP
    return v;
}

// sum over a workgroup of NW waves; every thread gets the result.  `red` holds NW floats; two barriers.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red)
{
    v = wave_sum(v);
    const int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float s = 0.f;
    #pragma unroll
    for (int i = 0; i < NW; ++i) s += red[i];
    return s;
}

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
// gated activations of two projections (g: gate, u: up).  EXL3_MIX_GLU_SILU: silu(g) u.  EXL3_MIX_GLU_CLAMPED_SWISH: g' = min(g, limit),
// u' = clamp(u, -limit, limit), g' sigmoid(1.702 g') (u' + 1).
__device__ __forceinline__ float glu_act_f(float g, float u, int kind, float limit)
{
    if (kind == EXL3_MIX_GLU_SILU) return silu_f(g) * u;
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoid_f(1.702f * g) * (u + 1.0f);
}
// plain activations (EXL3_MIX_ACT_*): relu(z)^2, gelu in its tanh form, silu
__device__ __forceinline__ float gelu_tanh_f(float z) { return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }
__device__ __forceinline__ float act_f(float v, int kind)
{
    if (kind == EXL3_MIX_ACT_RELU2) { const float t = fmaxf(v, 0.f); return t * t; }
    if (kind == EXL3_MIX_ACT_GELU_TANH) return gelu_tanh_f(v);
    return silu_f(v);
}
// log(sigmoid(z)) without cancellation on either side
__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
// log(1 + exp(z)) without overflow
__device__ __forceinline__ float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// error reporting shared by the translation units of this library (thread-local message, negative return codes)
void mix_set_error(const char* fmt, ...);
int  mix_check_launch(const char* what);
#define MIX_CHECK(cond, ...) do { if (!(cond)) { mix_set_error(__VA_ARGS__); return EXL3_MIX_ERR_ARG; } } while (0)

// dispatch on the activation element type: 0 = bfloat16, 1 = float32
#define MIX_DISPATCH_T(dtype, ...) \
    do { if ((dtype) == EXL3_MIX_BF16) { using T = bf16_t; __VA_ARGS__; } else { using T = float; __VA_ARGS__; } } while (0)
