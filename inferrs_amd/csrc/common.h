// Shared device helpers for the gfx950 kernels: storage types, wave and block
// reductions, and the error channel of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define IA_WAVE 64

// ---- storage types --------------------------------------------------------------------------
// bfloat16 is handled as raw bits: widening is a shift, narrowing rounds to nearest even.
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Two 32-bit values to two bfloat16 in one word (low half first), rounded to nearest even by
// the hardware conversion.
typedef __bf16 ia_bf16x2 __attribute__((ext_vector_type(2)));
typedef float ia_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const ia_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, ia_bf16x2));
}

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const bf16_t* p) { return bf16_bits_to_f32(p->bits); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16_t* p, float v) { p->bits = f32_to_bf16_bits(v); }

// The value a store of `v` would leave behind, widened again.
__device__ __forceinline__ float round_to(const float*, float v) { return v; }
__device__ __forceinline__ float round_to(const bf16_t*, float v) {
    return bf16_bits_to_f32(f32_to_bf16_bits(v));
}

// ---- the activation of a gated feed-forward ---------------------------------------------------
// act(gate) * up, in 32-bit.  The entry points' `dual` / `act` argument names the activation: 1 SiLU,
// gate / (1 + exp(-gate)); 2 GELU in its tanh form, gate / 2 * (1 + tanh(sqrt(2 / pi) * (gate + 0.044715 gate^3))).
// The choice is the same for all lanes of a launch.
enum { IA_ACT_NONE = 0, IA_ACT_SILU = 1, IA_ACT_GELU_TANH = 2, IA_ACT_LAST = IA_ACT_GELU_TANH };

__device__ __forceinline__ float gate_act(float g, int act) {
    if (act == IA_ACT_GELU_TANH) return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    return g / (1.0f + expf(-g));
}

// ---- reductions -----------------------------------------------------------------------------
// Butterfly over the 64 lanes: every lane ends with the same value, and the order of the
// additions is fixed by the lane numbers alone.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = IA_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, IA_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = IA_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, IA_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds 16 floats of shared memory.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & (IA_WAVE - 1);
    const int wave = threadIdx.x / IA_WAVE;
    const int nwaves = (blockDim.x + IA_WAVE - 1) / IA_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < nwaves; ++w) total += scratch[w];
    return total;
}

// ---- error channel --------------------------------------------------------------------------
// Entry points return 0 on success.  On failure they return a non-zero code and leave a
// message that ia_last_error() hands out.
void ia_set_error(const char* fmt, ...);

#define IA_CHECK(cond, ...)            \
    do {                               \
        if (!(cond)) {                 \
            ia_set_error(__VA_ARGS__); \
            return 1;                  \
        }                              \
    } while (0)

#define IA_LAUNCH_CHECK(name)                                                   \
    do {                                                                        \
        hipError_t e_ = hipGetLastError();                                      \
        if (e_ != hipSuccess) {                                                 \
            ia_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return 2;                                                           \
        }                                                                       \
    } while (0)

enum { IA_F32 = 0, IA_BF16 = 1 };
