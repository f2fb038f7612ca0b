// Device helpers shared by the translation units of the layer-list host layer (hybrid_kernels.hip, hybrid_blocks.hip): typed loads and
// stores of f32 / bf16 operands, the scalar activations, and the sum over neighbouring lanes that share a state column.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>

#include "common.h"

namespace {

template <typename T> __device__ __forceinline__ float ld(const T* p, size_t i);
template <> __device__ __forceinline__ float ld<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float ld<uint16_t>(const uint16_t* p, size_t i) { return bf16_to_f32(p[i]); }
template <typename T> __device__ __forceinline__ void st(T* p, size_t i, float v);
template <> __device__ __forceinline__ void st<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void st<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// sum over the LPC neighbouring lanes that share a state column
// (data-parallel-primitive moves inside a row of 16 lanes: swap inside pairs, swap pairs inside quads, mirror inside half rows,
// mirror inside the row -- after each add every lane holds the sum of twice as many lanes; no LDS traffic, a few cycles each)
template <int CTRL> __device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
template <int LPC> __device__ __forceinline__ float column_sum(float x) {
    static_assert(LPC == 4 || LPC == 16, "a column is shared by a quad or by a row of 16 lanes");
    x += dpp_move<0xB1>(x);                      // quad_perm [1, 0, 3, 2]
    x += dpp_move<0x4E>(x);                      // quad_perm [2, 3, 0, 1]
    if (LPC == 16) {
        x += dpp_move<0x141>(x);                 // row_half_mirror
        x += dpp_move<0x140>(x);                 // row_mirror
    }
    return x;
}

inline bool is_dt(int dt) { return dt == 0 || dt == 2; }               // MI355_DTYPE_F32, MI355_DTYPE_BF16
#define LAUNCH_OK() do { const hipError_t e_ = hipGetLastError(); if (e_ != hipSuccess) return (int)e_; } while (0)

}  // namespace
