// Shared device helpers and the host-side error channel of the kernel library (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

typedef uint16_t bf16_t;   // raw bfloat16 bits

enum { TP_F32 = 0, TP_BF16 = 1 };

// ---- host: errors -----------------------------------------------------------------------------
// Every entry point returns 0, or a non-zero code after storing a message that tp_last_error() gives back.
extern "C" const char* tp_last_error();
int tp_fail(const char* fmt, ...);
int tp_check_launch(const char* what);

#define TP_REQUIRE(cond, ...) do { if (!(cond)) return tp_fail(__VA_ARGS__); } while (0)

static inline int tp_cdiv(long a, long b) { return (int)((a + b - 1) / b); }

// ---- device: number formats ------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

__device__ __forceinline__ bf16_t f32_to_bf16(float f) {      // round to nearest even; NaN stays NaN
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

__device__ __forceinline__ float ld_f32(const float* p) { return *p; }
__device__ __forceinline__ float ld_f32(const bf16_t* p) { return bf16_to_f32(*p); }
__device__ __forceinline__ void st_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ void st_f32(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// ---- device: reductions over a wave of 64 and over a block -------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `red` holds 16 floats of LDS.
// The order of additions depends only on the block size, never on timing.
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = (blockDim.x + 63) >> 6;
    __syncthreads();                       // red may still be read from an earlier call
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; i++) t += red[i];
    return t;
}

// The same where `red` has not been used by the block before (a call's own 16 floats): one barrier less.
__device__ __forceinline__ float block_sum_once(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = (blockDim.x + 63) >> 6;
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; i++) t += red[i];
    return t;
}

// ---- device: functions of the model ---------------------------------------------------------------
__device__ __forceinline__ float gelu_tanh_f(float g) {
    return 0.5f * g * (1.0f + tanhf(0.7978845608f * (g + 0.044715f * g * g * g)));
}
__device__ __forceinline__ float softcap_f(float s, float cap) { return cap * tanhf(s / cap); }
// The same function for the bf16 products' epilogues, where it is evaluated once per output element of the largest
// product: 0.5 g (1 + tanh u) = g / (1 + e^(-2u)), one exponential and one reciprocal instruction instead of the
// library's tanh (relative error of a few 1e-7; the result is rounded to bf16).
__device__ __forceinline__ float gelu_tanh_fast(float g) {
    constexpr float C1 = -2.f * 0.7978845608f * 1.4426950408889634f, C3 = C1 * 0.044715f;
    return g * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * __builtin_fmaf(C3, g * g, C1)));
}

// ---- gate activations of a gated product -----------------------------------------------------------------------
// The activations offered are of one form, act(g) = g / (1 + 2^(g (c1 + c3 g^2))): gelu-tanh (above) with
// c1 = -2 * 0.7978845608 * log2(e), c3 = c1 * 0.044715, and SiLU, g / (1 + e^-g), with c1 = -log2(e), c3 = 0.  The
// bf16 products' epilogues take the two constants (`epi.x`, `epi.y`) and have no branch on the activation's kind.
enum { TP_ACT_GELU_TANH = 0, TP_ACT_SILU = 1 };
// which elements of a head a rotation pairs: (f, f + rotary_dim / 2) as the reference does
// (runtime/cuda/codebook_gemv.cu:219-230), or neighbours (2f, 2f + 1)
enum { TP_ROPE_HALVES = 0, TP_ROPE_NEIGHBOURS = 1 };
static inline bool tp_gate_constants(int act, float* c1, float* c3) {
    constexpr float LOG2E = 1.4426950408889634f;
    if (act == TP_ACT_GELU_TANH) { *c1 = -2.f * 0.7978845608f * LOG2E; *c3 = *c1 * 0.044715f; return true; }
    if (act == TP_ACT_SILU) { *c1 = -LOG2E; *c3 = 0.f; return true; }
    return false;
}
__device__ __forceinline__ float gate_act_fast(float g, float2 epi) {
    return g * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(g * __builtin_fmaf(epi.y, g * g, epi.x)));
}
// the same in full float32 arithmetic, for the float32 path
__device__ __forceinline__ float gate_act_exact(float g, int act) {
    return act == TP_ACT_SILU ? g / (1.f + expf(-g)) : gelu_tanh_f(g);
}
