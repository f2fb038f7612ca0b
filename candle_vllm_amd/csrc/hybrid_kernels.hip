// Kernels of the layer-list ("hybrid") host layer (include/mi355_hybrid.h): sliding-window attention with a softmax sink over the
// block engine's pages, the gated delta rule and the minGRU over the block engine's state slots, the short causal convolution in
// front of the delta rule, and the f32-residual glue around them.  Numerics: residual stream, norms, scores, probabilities,
// decays, gates of a recurrence and all recurrent state are f32; MI355_DTYPE_BF16 keeps matrices, K/V pages and the operands of
// a matrix product in bf16 (matrix cores, f32 accumulation), MI355_DTYPE_F32 multiplies with f32 FMAs.
// One step function serves prompts, portions of prompts and decoded tokens: a sequence brings cu_q[s+1] - cu_q[s] new tokens behind
// ctx[s] - that many cached ones; a portion that starts at position 0 starts from zero state whatever its slot holds.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>

#include "common.h"
#include "hybrid_device.h"
#include "../../include/mi355_hybrid.h"

namespace {

// ------------------------------------------------------------------------------------------------------------ matrix products
// 8 consecutive operands of a row as one MFMA fragment (bf16), zero beyond `kend`
template <typename TA> __device__ __forceinline__ uint4 frag8(const TA* row, int k, int kend, bool vec_ok);
template <> __device__ __forceinline__ uint4 frag8<uint16_t>(const uint16_t* row, int k, int kend, bool vec_ok) {
    if (vec_ok && k + 8 <= kend) return *reinterpret_cast<const uint4*>(row + k);
    uint16_t h[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) h[j] = (k + j < kend) ? row[k + j] : (uint16_t)0;
    return uint4{(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16),
                 (uint32_t)h[4] | ((uint32_t)h[5] << 16), (uint32_t)h[6] | ((uint32_t)h[7] << 16)};
}
template <> __device__ __forceinline__ uint4 frag8<float>(const float* row, int k, int kend, bool vec_ok) {
    float f[8];
    if (vec_ok && k + 8 <= kend) {
        const float4 a = *reinterpret_cast<const float4*>(row + k), b = *reinterpret_cast<const float4*>(row + k + 4);
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = (k + j < kend) ? row[k + j] : 0.f;
    }
    return uint4{cvt_pk_bf16(f[0], f[1]), cvt_pk_bf16(f[2], f[3]), cvt_pk_bf16(f[4], f[5]), cvt_pk_bf16(f[6], f[7])};
}
__device__ __forceinline__ f32x4_t mfma_bf16(const uint4& a, const uint4& b, const f32x4_t& c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

struct LinArgs {
    float* out; int ldo;
    const void* a; int lda;
    const void* w; const float* bias;
    int T, N, K;
    int a_vec, w_vec;       // rows may be read 16 bytes at a time
    int64_t a_bs, w_bs, o_bs;   // blockIdx.z = one of several independent products of this shape: element strides of its operands
    // grouped product (blk != NULL): the rows come in blocks of blk_rows = the kernel's tile height; block b = blockIdx.y multiplies its
    // rows [b blk_rows, blk[2b + 1]) with matrix blk[2b] (w + blk[2b] w_bs); row r of `a` is read at row_src[r] when row_src != NULL
    const int32_t* blk; const int32_t* row_src; int blk_rows;
};
// the block's matrix and the end of its rows (one past the last); false = nothing to do
__device__ __forceinline__ bool lin_group(LinArgs& p, int t0, int64_t& w_off) {
    w_off = (int64_t)blockIdx.z * p.w_bs;
    if (!p.blk) return true;
    const int b = t0 / p.blk_rows;
    const int e = p.blk[2 * b], end = p.blk[2 * b + 1];
    if (t0 >= end) return false;
    p.T = end;
    w_off = (int64_t)e * p.w_bs;
    return true;
}
__device__ __forceinline__ int lin_row(const LinArgs& p, int t) { return p.row_src ? p.row_src[t] : t; }
template <typename TA> __device__ __forceinline__ void lin_batch(LinArgs& p) {
    const int64_t z = blockIdx.z;
    p.a = static_cast<const TA*>(p.a) + z * p.a_bs;
    p.out += z * p.o_bs;
}

// Prompt-sized products, bf16 weights.  A workgroup of four waves owns 64 output columns (16 weight rows per wave) and 16 MT tokens;
// fragments go from global memory / L2 straight into registers: lane (m16, kg) holds operands 8 kg .. 8 kg + 7 of row m16 of a
// 32-wide K step on both sides, the accumulator holds tokens 4 kg + v of column m16.
template <typename TA, int MT> __global__ __launch_bounds__(256) void linear_bf16_tile_kernel(LinArgs p) {
    lin_batch<TA>(p);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, m16 = lane & 15, kg = lane >> 4;
    const int n = blockIdx.x * 64 + wave * 16 + m16;
    const int t0 = blockIdx.y * (16 * MT);
    int64_t w_off;
    if (!lin_group(p, t0, w_off)) return;
    const uint16_t* wrow = static_cast<const uint16_t*>(p.w) + w_off + (size_t)(n < p.N ? n : 0) * p.K;
    const TA* arow[MT];
    bool aok[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int t = t0 + i * 16 + m16;
        aok[i] = t < p.T;
        arow[i] = static_cast<const TA*>(p.a) + (size_t)(aok[i] ? lin_row(p, t) : 0) * p.lda;
    }
    f32x4_t acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const bool nok = n < p.N;
    for (int k0 = 0; k0 < p.K; k0 += 32) {
        const int k = k0 + 8 * kg;
        const uint4 b = nok ? frag8<uint16_t>(wrow, k, p.K, p.w_vec) : uint4{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const uint4 a = aok[i] ? frag8<TA>(arow[i], k, p.K, p.a_vec) : uint4{0, 0, 0, 0};
            acc[i] = mfma_bf16(a, b, acc[i]);
        }
    }
    if (!nok) return;
    const float bias = p.bias ? p.bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int t = t0 + i * 16 + 4 * kg + v;
            if (t < p.T) p.out[(size_t)t * p.ldo + n] = acc[i][v] + bias;
        }
}

// Prompt-sized products whose operands are both bf16 with 16-byte aligned rows and K a multiple of 32: a workgroup of four waves
// owns a 128-token x 128-column tile, each wave a 64 x 64 quarter (4 x 4 MFMA tiles).  The 128 x 32 slices of both operands go
// through LDS (rows padded to 80 bytes so that the 16 rows a fragment read touches fall into different 16-byte banks), the slice
// of the next K step is fetched into registers while the current one is multiplied: one barrier per K step.
__global__ __launch_bounds__(256) void linear_bf16_lds_kernel(LinArgs p) {
    constexpr int ROWB = 80;                                        // bytes per staged row: 64 of data + 16 of padding
    __shared__ __align__(16) uint8_t sa[2][128 * ROWB], sw[2][128 * ROWB];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, m16 = lane & 15, kg = lane >> 4;
    const int wr = wave >> 1, wc = wave & 1;
    const int n0 = blockIdx.x * 128, t0 = blockIdx.y * 128;
    lin_batch<uint16_t>(p);
    int64_t w_off;
    if (!lin_group(p, t0, w_off)) return;
    const uint16_t* A = static_cast<const uint16_t*>(p.a);
    const uint16_t* W = static_cast<const uint16_t*>(p.w) + w_off;
    // staging: thread -> rows r0 and r0 + 64 of both slices, 16-byte chunk ch of the 64-byte row
    const int r0 = tid >> 2, ch = tid & 3;
    const uint16_t* asrc[2]; const uint16_t* wsrc[2]; bool aok[2], wok[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int t = t0 + r0 + 64 * j, n = n0 + r0 + 64 * j;
        aok[j] = t < p.T; wok[j] = n < p.N;
        asrc[j] = A + (size_t)(aok[j] ? lin_row(p, t) : 0) * p.lda + ch * 8;
        wsrc[j] = W + (size_t)(wok[j] ? n : 0) * p.K + ch * 8;
    }
    uint4 ra[2], rw[2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ra[j] = aok[j] ? *reinterpret_cast<const uint4*>(asrc[j] + k0) : uint4{0, 0, 0, 0};
            rw[j] = wok[j] ? *reinterpret_cast<const uint4*>(wsrc[j] + k0) : uint4{0, 0, 0, 0};
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            *reinterpret_cast<uint4*>(&sa[buf][(r0 + 64 * j) * ROWB + ch * 16]) = ra[j];
            *reinterpret_cast<uint4*>(&sw[buf][(r0 + 64 * j) * ROWB + ch * 16]) = rw[j];
        }
    };
    f32x4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    fetch(0);
    stage(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < p.K; k0 += 32, buf ^= 1) {
        const bool more = k0 + 32 < p.K;
        if (more) fetch(k0 + 32);
        uint4 af[4], bf[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const uint4*>(&sa[buf][(wr * 64 + i * 16 + m16) * ROWB + kg * 16]);
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[j] = *reinterpret_cast<const uint4*>(&sw[buf][(wc * 64 + j * 16 + m16) * ROWB + kg * 16]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = mfma_bf16(af[i], bf[j], acc[i][j]);
        if (more) stage(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = n0 + wc * 64 + j * 16 + m16;
        if (n >= p.N) continue;
        const float bias = p.bias ? p.bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int t = t0 + wr * 64 + i * 16 + 4 * kg + v;
                if (t < p.T) p.out[(size_t)t * p.ldo + n] = acc[i][j][v] + bias;
            }
    }
}

// Up to 16 tokens, bf16 weights: the product is a stream over the weights.  A workgroup owns 16 weight rows; its NW waves take the
// 32-wide K steps in turn (UNR steps in flight per wave) and add their partial tiles through LDS.
template <typename TA, int NW, int UNR> __global__ __launch_bounds__(64 * NW) void linear_bf16_stream_kernel(LinArgs p) {
    __shared__ float part[NW][4][64];
    lin_batch<TA>(p);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, m16 = lane & 15, kg = lane >> 4;
    const int n = blockIdx.x * 16 + m16;
    const int t0 = blockIdx.y * 16;                                  // a grouped product: block blockIdx.y of 16 rows; else 0
    int64_t w_off;
    if (!lin_group(p, t0, w_off)) return;
    const bool nok = n < p.N, aok = t0 + m16 < p.T;
    const uint16_t* wrow = static_cast<const uint16_t*>(p.w) + w_off + (size_t)(nok ? n : 0) * p.K;
    const TA* arow = static_cast<const TA*>(p.a) + (size_t)(aok ? lin_row(p, t0 + m16) : 0) * p.lda;
    f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int k0 = wave * 32 * UNR; k0 < p.K; k0 += NW * 32 * UNR) {
        uint4 a[UNR], b[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int k = k0 + u * 32 + 8 * kg;
            b[u] = (nok && k < p.K) ? frag8<uint16_t>(wrow, k, p.K, p.w_vec) : uint4{0, 0, 0, 0};
            a[u] = (aok && k < p.K) ? frag8<TA>(arow, k, p.K, p.a_vec) : uint4{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) acc = mfma_bf16(a[u], b[u], acc);
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) part[wave][v][lane] = acc[v];
    __syncthreads();
    if (wave == 0) {
        const float bias = (p.bias && nok) ? p.bias[n] : 0.f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += part[w][v][lane];
            const int t = t0 + 4 * kg + v;
            if (nok && t < p.T) p.out[(size_t)t * p.ldo + n] = s + bias;
        }
    }
}

// f32 weights and operands: plain FMAs in f32 (no reduced-precision matrix mode).  64 x 64 tile, 16-wide K steps through LDS,
// every thread owns 4 tokens x 4 columns.
__global__ __launch_bounds__(256) void linear_f32_kernel(LinArgs p) {
    __shared__ float As[16][68], Ws[16][68];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int n0 = blockIdx.x * 64, t0 = blockIdx.y * 64;
    lin_batch<float>(p);
    int64_t w_off;
    if (!lin_group(p, t0, w_off)) return;
    const float* A = static_cast<const float*>(p.a);
    const float* W = static_cast<const float*>(p.w) + w_off;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < p.K; k0 += 16) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int idx = threadIdx.x + r * 256;            // 1024 elements of each 64 x 16 tile
            const int row = idx >> 4, kk = idx & 15;
            const int k = k0 + kk;
            As[kk][row] = (t0 + row < p.T && k < p.K) ? A[(size_t)lin_row(p, t0 + row) * p.lda + k] : 0.f;
            Ws[kk][row] = (n0 + row < p.N && k < p.K) ? W[(size_t)(n0 + row) * p.K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty * 4 + i]; w[i] = Ws[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int t = t0 + ty * 4 + i;
        if (t >= p.T) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < p.N) p.out[(size_t)t * p.ldo + n] = acc[i][j] + (p.bias ? p.bias[n] : 0.f);
        }
    }
}

// ------------------------------------------------------------------------------------------------------------ residual glue
template <typename TW> __global__ void embed_kernel(float* x, uint16_t* xcopy, const TW* table, const uint32_t* ids, int width, int vocab) {
    const int t = blockIdx.x;
    const uint32_t id = ids[t] < (uint32_t)vocab ? ids[t] : 0u;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = ld<TW>(table, (size_t)id * width + i);
        x[(size_t)t * width + i] = v;
        if (xcopy) xcopy[(size_t)t * width + i] = f32_to_bf16(v);
    }
}

__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float s = 0.f;
    for (int w = 0; w < nw; ++w) s += red[w];
    return s;
}

// x += y / rms(y) * w  (the norm sits on the sublayer's OUTPUT), one workgroup per token
__global__ __launch_bounds__(256) void norm_add_kernel(float* x, uint16_t* xcopy, const float* y, int ldy, const float* w, int width, float eps) {
    __shared__ float red[4];
    const int t = blockIdx.x;
    const float* yr = y + (size_t)t * ldy;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) ss += yr[i] * yr[i];
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = x[(size_t)t * width + i] + yr[i] * inv * w[i];
        x[(size_t)t * width + i] = v;
        if (xcopy) xcopy[(size_t)t * width + i] = f32_to_bf16(v);
    }
}

// rows[r] of x -> RMS norm with weight -> out (dt) [n_rows, width]   (the model's last norm, on the wanted rows only)
template <typename TO> __global__ __launch_bounds__(256) void gather_norm_kernel(TO* out, const float* x, const int32_t* rows, const float* w, int width, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : r) * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) ss += xr[i] * xr[i];
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) st<TO>(out, (size_t)r * width + i, xr[i] * inv * w[i]);
}

// x <- N(alpha x + y) w with the norm BEHIND the sum: the vector is cut into `groups` equal consecutive parts and every part is
// divided by its own root mean square.  One workgroup per token; the sum stays in registers between the two passes (width <= 256 x 16).
__global__ __launch_bounds__(256) void resid_norm_kernel(float* x, uint16_t* xcopy, const float* y, int ldy, const float* w, int width,
                                                         int groups, float alpha, float eps) {
    __shared__ float red[4];
    __shared__ float inv_s[64];
    const int t = blockIdx.x, part = width / groups;
    float* xr = x + (size_t)t * width;
    const float* yr = y + (size_t)t * ldy;
    if (groups >= (int)(blockDim.x >> 6)) {                    // a wave per part, parts in turn: no workgroup-wide exchange at all
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
        for (int g = wave; g < groups; g += nw) {
            float ss = 0.f;
            for (int i = lane; i < part; i += 64) { const float v = fmaf(alpha, xr[g * part + i], yr[g * part + i]); ss = fmaf(v, v, ss); }
            ss = wave_sum(ss);
            const float inv = 1.f / sqrtf(ss / (float)part + eps);
            for (int i = lane; i < part; i += 64) {
                const int c = g * part + i;
                const float v = fmaf(alpha, xr[c], yr[c]) * inv * w[c];
                xr[c] = v;
                if (xcopy) xcopy[(size_t)t * width + c] = f32_to_bf16(v);
            }
        }
        return;
    }
    for (int g0 = 0; g0 < groups; g0 += 64) {
        const int gn = min(64, groups - g0);
        for (int g = 0; g < gn; ++g) {
            float ss = 0.f;
            for (int i = threadIdx.x; i < part; i += blockDim.x) {
                const int c = (g0 + g) * part + i;
                const float v = fmaf(alpha, xr[c], yr[c]);
                ss = fmaf(v, v, ss);
            }
            ss = block_sum(ss, red);
            if (threadIdx.x == 0) inv_s[g] = 1.f / sqrtf(ss / (float)part + eps);
        }
        __syncthreads();
        for (int i = threadIdx.x; i < gn * part; i += blockDim.x) {
            const int c = g0 * part + i;
            const float v = fmaf(alpha, xr[c], yr[c]) * inv_s[i / part] * w[c];
            xr[c] = v;
            if (xcopy) xcopy[(size_t)t * width + c] = f32_to_bf16(v);
        }
        __syncthreads();
    }
}

// rows[r] of x -> group RMS norm with weight -> out (dt) [n_rows, width]
template <typename TO> __global__ __launch_bounds__(256) void gather_group_norm_kernel(TO* out, const float* x, const int32_t* rows, const float* w,
                                                                                      int width, int groups, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x, part = width / groups;
    const float* xr = x + (size_t)rows[r] * width;
    for (int g = 0; g < groups; ++g) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < part; i += blockDim.x) { const float v = xr[g * part + i]; ss = fmaf(v, v, ss); }
        ss = block_sum(ss, red);
        const float inv = 1.f / sqrtf(ss / (float)part + eps);
        for (int i = threadIdx.x; i < part; i += blockDim.x) { const int c = g * part + i; st<TO>(out, (size_t)r * width + c, xr[c] * inv * w[c]); }
    }
}

__device__ __forceinline__ float gelu_tanhf_(float z) {
    return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
template <typename TO> __global__ void gelu_glu_kernel(TO* out, const float* gu, int64_t n, int ff) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t t = i / ff; const int j = (int)(i - t * ff);
    st<TO>(out, (size_t)i, gelu_tanhf_(gu[t * 2 * ff + j]) * gu[t * 2 * ff + ff + j]);
}

template <typename TO> __global__ void clamped_glu_kernel(TO* out, const float* gu, int64_t n, int ff, float limit, float alpha) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t t = i / ff; const int j = (int)(i - t * ff);
    const float g = fminf(gu[t * 2 * ff + j], limit);
    const float u = fminf(fmaxf(gu[t * 2 * ff + ff + j], -limit), limit);
    st<TO>(out, (size_t)i, g * sigmoidf_(alpha * g) * (u + 1.f));
}

// ------------------------------------------------------------------------------------------------------------ attention
struct PrepArgs {
    void* q_out; void* k_pages; void* v_pages;
    const float* proj; int ldp, q_off, k_off, v_off;
    const float* qw; const float* kw; const float* cos_t; const float* sin_t;
    const int64_t* positions; const int64_t* slots;
    int H, G, d, vd, rot; float eps;
    int interleaved;        // rotated pairs are (2i, 2i + 1) instead of (i, i + rot / 2)
    int norm_mode;          // 0 none, 1 RMS norm (weights qw / kw or none) before the rotation, 2 weightless RMS norm after it
    const float* q_scale;   // [H] or NULL: head h's query times q_scale[h]
};
// one wave per (token, vector): query heads 0 .. H-1, key heads H .. H+G-1, value heads H+G .. H+2G-1
template <typename TC> __global__ __launch_bounds__(64) void attn_prepare_kernel(PrepArgs p) {
    extern __shared__ float vec[];
    const int t = blockIdx.x, hv = blockIdx.y, lane = threadIdx.x;
    const float* row = p.proj + (size_t)t * p.ldp;
    const int64_t slot = p.slots[t];
    if (hv >= p.H + p.G) {                                          // value head: a copy into the page
        const int g = hv - p.H - p.G;
        if (slot < 0) return;
        TC* dst = static_cast<TC*>(p.v_pages) + ((size_t)slot * p.G + g) * p.vd;
        for (int i = lane; i < p.vd; i += 64) st<TC>(dst, i, row[p.v_off + g * p.vd + i]);
        return;
    }
    const bool is_q = hv < p.H;
    const int h = is_q ? hv : hv - p.H;
    const float* src = row + (is_q ? p.q_off : p.k_off) + h * p.d;
    const float* w = is_q ? p.qw : p.kw;
    float ss = 0.f;
    for (int i = lane; i < p.d; i += 64) { const float v = src[i]; vec[i] = v; ss += v * v; }
    if (p.norm_mode == 1 && w) {
        ss = wave_sum(ss);
        const float inv = 1.f / sqrtf(ss / (float)p.d + p.eps);
        __syncthreads();
        for (int i = lane; i < p.d; i += 64) vec[i] = vec[i] * inv * w[i];
    }
    __syncthreads();
    TC* dst;
    if (is_q) dst = static_cast<TC*>(p.q_out) + ((size_t)t * p.H + h) * p.d;
    else { if (slot < 0) return; dst = static_cast<TC*>(p.k_pages) + ((size_t)slot * p.G + h) * p.d; }
    const int half = p.rot / 2;
    const int64_t pos = p.positions[t];
    float* rotated = vec + p.d;
    float s2 = 0.f;
    for (int i = lane; i < p.d; i += 64) {
        float v = vec[i];
        if (i < p.rot) {
            if (p.interleaved) {
                const int pr = i >> 1;
                const float c = p.cos_t[pos * half + pr], s = p.sin_t[pos * half + pr];
                v = (i & 1) ? vec[i] * c + vec[i - 1] * s : vec[i] * c - vec[i + 1] * s;
            } else if (i < half) {
                const float c = p.cos_t[pos * half + i], s = p.sin_t[pos * half + i];
                v = vec[i] * c - vec[i + half] * s;
            } else {
                const float c = p.cos_t[pos * half + i - half], s = p.sin_t[pos * half + i - half];
                v = vec[i] * c + vec[i - half] * s;
            }
        }
        rotated[i] = v;
        s2 += v * v;
    }
    float mul = 1.f;
    if (p.norm_mode == 2) mul = 1.f / sqrtf(wave_sum(s2) / (float)p.d + p.eps);
    if (is_q && p.q_scale) mul *= p.q_scale[h];
    for (int i = lane; i < p.d; i += 64) st<TC>(dst, i, rotated[i] * mul);
}

struct AttnArgs {
    void* out; int ldo, out_off;
    const void* q; const void* k_pages; const void* v_pages;
    const uint32_t* bt; const uint32_t* ctx; const uint32_t* cu_q; const int32_t* tok_seq; const float* sink;
    int n_seqs, H, G, d, vd, bs, max_blocks, window; float scale, out_scale; int cp2, out_f32;
    int k_ld, v_ld;         // elements per page row (all key/value heads of a token; latent attention: one row serves as both)
    float softcap;          // > 0: score <- cap tanh(score / cap)
    int cross;              // blockIdx.z = the key/value head whose VALUES this block sums (scores still against the head's own keys)
    int cpk;                // lanes that share a key row when it is read 16 bytes a lane (power of two >= d / elements per 16 bytes)
    int keep;               // with a window: keys at positions < keep stay visible (the first tokens of the sequence)
    const float* dist;      // != NULL: [2, H] = r1, r2; score <- score - r1[h] ln(1 + r2[h] (query position - key position))
};
// (the hardware's log2: the argument is at least 1, so the absolute error stays near the f32 rounding of the score it is taken from)
__device__ __forceinline__ float dist_bias(float r1, float r2, int d) { return r1 * 0.6931471805599453f * __log2f(fmaf(r2, (float)d, 1.f)); }
__device__ __forceinline__ float cap_score(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }
// 16 bytes of a page row as floats (EPV = 8 bf16 or 4 f32)
template <typename TC> struct Vec16;
template <> struct Vec16<uint16_t> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void load(const uint16_t* p, float* x) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        x[0] = bf16lo_to_f32(v.x); x[1] = bf16hi_to_f32(v.x); x[2] = bf16lo_to_f32(v.y); x[3] = bf16hi_to_f32(v.y);
        x[4] = bf16lo_to_f32(v.z); x[5] = bf16hi_to_f32(v.z); x[6] = bf16lo_to_f32(v.w); x[7] = bf16hi_to_f32(v.w);
    }
};
template <> struct Vec16<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void load(const float* p, float* x) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    }
};

// One workgroup of NW waves per (new token, head).  Wave w takes the 64-key chunks w, w + NW, ... of the token's window: a lane
// scores one key (q from LDS, the key row from its page), the wave keeps a running maximum / denominator / value sum, and the waves'
// partial results are merged through LDS.  The sink enters the merge as a partial result with maximum sink, denominator 1 and no
// value.  VEC (head sizes that are multiples of 16 bytes): rows are read 16 bytes at a time; for the value sum the wave's lanes
// are (key, 16-byte chunk of the row) pairs -- 64 / cp2 keys per pass -- and the keys' partial sums are added by lane exchanges.
// (DQ: unused, 0.)
// NV > 1 (cross mode): the head's weights are applied to the values of NV key/value heads; the scores are computed once.
template <typename TC, int NW, bool VEC, int DQ, int NV> __global__ __launch_bounds__(64 * NW) void window_attention_kernel(AttnArgs p) {
    constexpr int EPV = Vec16<TC>::N;
    constexpr int NACC = VEC ? EPV : 8;
    extern __shared__ __align__(16) float smem[];
    float* qs = smem;                                   // [d rounded up to 4]
    float* pm = qs + ((p.d + 3) & ~3);                  // [NW] maxima, [NW] denominators, [NW][vd] sums
    float* pl = pm + NW;
    float* pacc = pl + NW;
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int s = p.tok_seq[t];
    const int n_new = (int)(p.cu_q[s + 1] - p.cu_q[s]);
    const int pos = (int)p.ctx[s] - n_new + (t - (int)p.cu_q[s]);
    const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
    // the visible keys in one run of indices: the kept first tokens below the window (nkeep of them), then the window [lo, pos]
    const int nkeep = min(p.keep, lo), n_vis = nkeep + pos - lo + 1;
    const int g = h / (p.H / p.G);
    const int gv0 = p.cross ? (int)blockIdx.z * NV : g, oh0 = p.cross ? h * p.G + gv0 : h;
    const TC* q = static_cast<const TC*>(p.q) + ((size_t)t * p.H + h) * p.d;
    for (int i = threadIdx.x; i < p.d; i += blockDim.x) qs[i] = ld<TC>(q, i);
    __syncthreads();
    const uint32_t* bt = p.bt + (size_t)s * p.max_blocks;
    const int cp2 = p.cp2, chunk = lane & (cp2 - 1), ksub = lane / cp2, kpp = 64 / cp2;     // VEC only
    const bool chunk_ok = chunk * EPV < p.vd;
    // VEC scores: lanes are (key, 16-byte chunk of its row) pairs too -- kq keys per pass, a pass reads kq whole rows (a lane per
    // 16 bytes, neighbouring lanes neighbouring bytes) instead of 16 bytes of 64 different rows; the chunk of the query that a lane
    // multiplies stays in its registers
    const int cpk = p.cpk, qchunk = lane & (cpk - 1), qsub = lane / cpk, kq = 64 / cpk;
    const bool qok = qchunk * EPV < p.d;
    float qv[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) qv[e] = (VEC && qok) ? qs[qchunk * EPV + e] : 0.f;
    const float r1 = p.dist ? p.dist[h] : 0.f, r2 = p.dist ? p.dist[p.H + h] : 0.f;
    float m = -INFINITY, l = 0.f, acc[NV][NACC];
#pragma unroll
    for (int n = 0; n < NV; ++n)
#pragma unroll
        for (int e = 0; e < NACC; ++e) acc[n][e] = 0.f;
    for (int i0 = wave * 64; i0 < n_vis; i0 += NW * 64) {
        const int cnt = min(64, n_vis - i0);
        const int j = lane < cnt ? (i0 + lane < nkeep ? i0 + lane : lo + (i0 + lane - nkeep)) : pos + 1;
        float sc = -INFINITY;
        unsigned page_row = 0;
        if (j <= pos) page_row = bt[j / p.bs] * (unsigned)p.bs + (unsigned)(j % p.bs);
        if (VEC) {
            constexpr int SU = 8;                                         // passes whose loads are in flight together
            float dot = 0.f;
            const int qcol = g * p.d + (qok ? qchunk * EPV : 0);
            for (int u0 = 0; u0 * kq < cnt; u0 += SU) {
                float part[SU];
#pragma unroll
                for (int u = 0; u < SU; ++u) {
                    const int jj = (u0 + u) * kq + qsub;
                    const bool on = jj < cnt && qok;
                    const size_t pr = (size_t)__shfl(page_row, jj & 63);
                    float x[EPV];
                    Vec16<TC>::load(static_cast<const TC*>(p.k_pages) + (on ? pr : (size_t)0) * p.k_ld + qcol, x);
                    float a = 0.f;
#pragma unroll
                    for (int e = 0; e < EPV; ++e) a = fmaf(qv[e], x[e], a);
                    part[u] = on ? a : 0.f;
                }
                for (int o = 1; o < cpk; o <<= 1)
#pragma unroll
                    for (int u = 0; u < SU; ++u) part[u] += __shfl_xor(part[u], o);
#pragma unroll
                for (int u = 0; u < SU; ++u) {                            // the lane that owns key (u0 + u) kq + i takes it from group i
                    const float v = __shfl(part[u], (lane % kq) * cpk);
                    if (lane / kq == u0 + u) dot = v;
                }
            }
            if (j <= pos) sc = cap_score(dot * p.scale, p.softcap) - (p.dist ? dist_bias(r1, r2, pos - j) : 0.f);
        } else if (j <= pos) {
            const TC* kr = static_cast<const TC*>(p.k_pages) + (size_t)page_row * p.k_ld + g * p.d;
            float dot = 0.f;
            for (int i = 0; i < p.d; ++i) dot = fmaf(qs[i], ld<TC>(kr, i), dot);
            sc = cap_score(dot * p.scale, p.softcap) - (p.dist ? dist_bias(r1, r2, pos - j) : 0.f);
        }
        const float mn = fmaxf(m, wave_max(sc));
        const float pj = (j <= pos) ? expf(sc - mn) : 0.f;
        const float corr = (m == -INFINITY) ? 0.f : expf(m - mn);
        l = l * corr + wave_sum(pj);
#pragma unroll
        for (int n = 0; n < NV; ++n)
#pragma unroll
            for (int e = 0; e < NACC; ++e) acc[n][e] *= corr;
        m = mn;
        if (VEC) {
            // PU passes of kpp keys at a time: the value rows of all of them are requested before the first is summed, so a chunk
            // costs 64 / (kpp PU) memory round trips instead of 64 / kpp.  A pass beyond the chunk's end (or a lane whose 16-byte
            // chunk lies beyond the row) reads a valid row with weight 0 and its values are replaced by zeros.
            constexpr int PU = NV >= 2 ? 2 : 8;
            const int vcol = chunk_ok ? chunk * EPV : 0;
            for (int k0 = 0; k0 < cnt; k0 += kpp * PU) {
                float pv[PU], x[PU][NV][EPV];
#pragma unroll
                for (int u = 0; u < PU; ++u) {
                    const int jj = k0 + u * kpp + ksub;
                    const bool on = jj < cnt && chunk_ok;
                    const float pjj = __shfl(pj, jj & 63);
                    pv[u] = on ? pjj : 0.f;
                    const size_t pr = (size_t)__shfl(page_row, jj & 63);
                    const TC* vr = static_cast<const TC*>(p.v_pages) + (on ? pr : (size_t)0) * p.v_ld + gv0 * p.vd + vcol;
#pragma unroll
                    for (int n = 0; n < NV; ++n) Vec16<TC>::load(vr + n * p.vd, x[u][n]);
                }
#pragma unroll
                for (int u = 0; u < PU; ++u)
#pragma unroll
                    for (int n = 0; n < NV; ++n)
#pragma unroll
                        for (int e = 0; e < EPV; ++e) acc[n][e] = fmaf(pv[u], pv[u] != 0.f ? x[u][n][e] : 0.f, acc[n][e]);
            }
        } else {
            for (int jj = 0; jj < cnt; ++jj) {
                const float pv = __shfl(pj, jj);
                const size_t pr = (size_t)__shfl(page_row, jj);
#pragma unroll
                for (int n = 0; n < NV; ++n) {
                    const TC* vr = static_cast<const TC*>(p.v_pages) + pr * p.v_ld + (gv0 + n) * p.vd;
#pragma unroll
                    for (int e = 0; e < NACC; ++e) { const int c = lane + 64 * e; if (c < p.vd) acc[n][e] = fmaf(pv, ld<TC>(vr, c), acc[n][e]); }
                }
            }
        }
    }
    if (lane == 0) { pm[wave] = m; pl[wave] = l; }
    if (VEC) {
        for (int off = cp2; off < 64; off <<= 1)
#pragma unroll
            for (int n = 0; n < NV; ++n)
#pragma unroll
                for (int e = 0; e < NACC; ++e) acc[n][e] += __shfl_xor(acc[n][e], off);
        if (ksub == 0 && chunk_ok)
#pragma unroll
            for (int n = 0; n < NV; ++n)
#pragma unroll
                for (int e = 0; e < EPV; ++e) pacc[(wave * NV + n) * p.vd + chunk * EPV + e] = acc[n][e];
    } else {
#pragma unroll
        for (int n = 0; n < NV; ++n)
#pragma unroll
            for (int e = 0; e < NACC; ++e) { const int c = lane + 64 * e; if (c < p.vd) pacc[(wave * NV + n) * p.vd + c] = acc[n][e]; }
    }
    __syncthreads();
    if (wave == 0) {
        float M = p.sink ? p.sink[h] : -INFINITY;
        for (int w = 0; w < NW; ++w) M = fmaxf(M, pm[w]);
        float L = p.sink ? expf(p.sink[h] - M) : 0.f;
        float cw[NW];
        for (int w = 0; w < NW; ++w) { cw[w] = pm[w] == -INFINITY ? 0.f : expf(pm[w] - M); L += pl[w] * cw[w]; }
        for (int n = 0; n < NV; ++n) {
            const size_t base = (size_t)t * p.ldo + p.out_off + (size_t)(oh0 + n) * p.vd;
            for (int col = lane; col < p.vd; col += 64) {
                float o = 0.f;
                for (int w = 0; w < NW; ++w) o += pacc[(w * NV + n) * p.vd + col] * cw[w];
                if (p.out_f32) st<float>(static_cast<float*>(p.out), base + col, o / L * p.out_scale);
                else st<uint16_t>(static_cast<uint16_t*>(p.out), base + col, o / L * p.out_scale);
            }
        }
    }
}

// Prompt-sized steps, bf16 pages: one wave per (tile of 16 consecutive new tokens of one sequence, head), 64 keys per iteration.
//   S = Q K^T on the matrix cores: the query tile's fragments stay in registers, a key's fragments come straight from its page row
//   (lane (m16, kg) = 16 bytes of key m16 of a 16-key tile); the accumulator holds queries 4 kg + v against key m16.
//   Mask, scale and the online softmax run on that layout in f32 (row maxima / sums: exchanges among the 16 lanes of a kg group).
//   P V: the probabilities go through LDS into A-fragment order as TWO bf16 planes (p = hi + lo, so the weights keep about 16 bits
//   of mantissa), the 64 value rows go through LDS to become B fragments (8 keys of one column per lane).
// The sink is applied at the end: denominator += exp(sink - max).
// NV > 1 (cross mode): the block applies its head's weights to the values of NV key/value heads one after the other -- Q K^T, the
// softmax and the probability planes are made once per chunk, the transposed value tile in LDS is refilled per value head.
template <int DK, int VT, int NV> __global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(NV == 2 ? 2 : 1)))
void window_attention_mfma_kernel(AttnArgs p) {
    constexpr int RS = 72;                                           // bf16 per LDS row: 64 keys + 8 of padding (144 bytes)
    // NV > 1: the value rows lie in LDS as rows (VRS bf16 each: 8 rows on are 16 banks on) and a B fragment gathers its 8 keys of one
    // column with 2-byte reads; NV == 1: they are transposed by the store ([column][key]) and a B fragment is one 16-byte read
    constexpr bool ROWS = NV > 1;
    constexpr int VRS = VT * 16 + 4;
    __shared__ __align__(16) uint16_t Ph[16 * RS], Pl[16 * RS], Vt[ROWS ? 64 * VRS : VT * 16 * RS];
    const int lane = threadIdx.x, m16 = lane & 15, kg = lane >> 4;
    int b = blockIdx.x, s = 0, n_new = 0;
    for (; s < p.n_seqs; ++s) {
        n_new = (int)(p.cu_q[s + 1] - p.cu_q[s]);
        const int tiles = (n_new + 15) >> 4;
        if (b < tiles) break;
        b -= tiles;
    }
    if (s >= p.n_seqs) return;
    const int t0 = (int)p.cu_q[s] + b * 16, nq = min(16, (int)p.cu_q[s + 1] - t0);
    const int pos0 = (int)p.ctx[s] - n_new + b * 16;
    const int h = blockIdx.y, g = h / (p.H / p.G), d = p.d, vd = p.vd;
    const int gv0 = p.cross ? (int)blockIdx.z * NV : g, oh0 = p.cross ? h * p.G + gv0 : h;
    const uint16_t* Q = static_cast<const uint16_t*>(p.q);
    const uint16_t* K = static_cast<const uint16_t*>(p.k_pages);
    const uint16_t* V = static_cast<const uint16_t*>(p.v_pages);
    const uint32_t* bt = p.bt + (size_t)s * p.max_blocks;
    uint4 qf[DK];
#pragma unroll
    for (int ks = 0; ks < DK; ++ks)
        qf[ks] = m16 < nq ? *reinterpret_cast<const uint4*>(Q + ((size_t)(t0 + m16) * p.H + h) * d + ks * 32 + 8 * kg) : uint4{0, 0, 0, 0};
    float mrow[4], lrow[4];
    f32x4_t acc[NV][VT];
#pragma unroll
    for (int v = 0; v < 4; ++v) { mrow[v] = -INFINITY; lrow[v] = 0.f; }
#pragma unroll
    for (int n = 0; n < NV; ++n)
#pragma unroll
        for (int c = 0; c < VT; ++c) acc[n][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int hi = pos0 + nq - 1;
    const float r1 = p.dist ? p.dist[h] : 0.f, r2 = p.dist ? p.dist[p.H + h] : 0.f;
    const int lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
    // the keys any query of the tile may see, in one run of indices: the kept first tokens below the lowest window, then [lo, hi]
    const int nkeep = min(p.keep, lo), n_vis = nkeep + hi - lo + 1;
    auto key_at = [&](int i) { return i < nkeep ? i : (i < n_vis ? lo + (i - nkeep) : hi + 1); };
    for (int j0 = 0; j0 < n_vis; j0 += 64) {
        // the 64 value rows of this chunk, transposed into LDS (zeros past the end: a stale NaN times a zero weight would poison the sum)
        // (a value head's rows are requested into registers one head ahead of their use: the next head's loads are in flight while the
        // current head multiplies)
        uint4 vreg[VT * 2];
        const int vkey = key_at(j0 + lane);
        const bool vkv = vkey <= hi;
        const uint16_t* vrow = V + (vkv ? (size_t)bt[vkey / p.bs] * p.bs + (vkey % p.bs) : 0) * p.v_ld + gv0 * vd;
        auto fetch_values = [&](int n) {
#pragma unroll
            for (int c8 = 0; c8 < VT * 2; ++c8) vreg[c8] = vkv ? *reinterpret_cast<const uint4*>(vrow + n * vd + c8 * 8) : uint4{0, 0, 0, 0};
        };
        // transposing store: a word holds two neighbouring columns of this lane's key; the lane pair (2a, 2a + 1) swaps words, the
        // even lane keeps the even column of both keys and the odd lane the odd column, so every lane writes ONE 4-byte word (two
        // keys of one column) instead of two 2-byte halves
        auto stage_values = [&]() {
            if (ROWS) {
#pragma unroll
                for (int c8 = 0; c8 < VT * 2; ++c8) {
                    *reinterpret_cast<uint2*>(&Vt[lane * VRS + c8 * 8]) = uint2{vreg[c8].x, vreg[c8].y};
                    *reinterpret_cast<uint2*>(&Vt[lane * VRS + c8 * 8 + 4]) = uint2{vreg[c8].z, vreg[c8].w};
                }
                return;
            }
            const int col_odd = lane & 1, key_even = lane & ~1;
#pragma unroll
            for (int c8 = 0; c8 < VT * 2; ++c8) {
                const uint32_t w[4] = {vreg[c8].x, vreg[c8].y, vreg[c8].z, vreg[c8].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w[e], 0xB1, 0xF, 0xF, true);   // quad_perm [1, 0, 3, 2]
                    const uint32_t pair = col_odd ? ((other >> 16) | (w[e] & 0xFFFF0000u)) : ((w[e] & 0xFFFFu) | (other << 16));
                    *reinterpret_cast<uint32_t*>(&Vt[(c8 * 8 + 2 * e + col_odd) * RS + key_even]) = pair;
                }
            }
        };
        auto value_fragment = [&](int k2, int c) {
            if (!ROWS) return *reinterpret_cast<const uint4*>(&Vt[(c * 16 + m16) * RS + k2 * 32 + 8 * kg]);
            const uint16_t* col = &Vt[(k2 * 32 + 8 * kg) * VRS + c * 16 + m16];
            uint4 f;
            f.x = (uint32_t)col[0] | ((uint32_t)col[VRS] << 16);
            f.y = (uint32_t)col[2 * VRS] | ((uint32_t)col[3 * VRS] << 16);
            f.z = (uint32_t)col[4 * VRS] | ((uint32_t)col[5 * VRS] << 16);
            f.w = (uint32_t)col[6 * VRS] | ((uint32_t)col[7 * VRS] << 16);
            return f;
        };
        fetch_values(0);
        f32x4_t sacc[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            sacc[kt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            const int key = key_at(j0 + kt * 16 + m16);
            const bool kv = key <= hi;
            const size_t pr = kv ? (size_t)bt[key / p.bs] * p.bs + (key % p.bs) : 0;
            const uint16_t* kr = K + pr * p.k_ld + g * d + 8 * kg;
#pragma unroll
            for (int ks = 0; ks < DK; ++ks) {
                const uint4 kf = kv ? *reinterpret_cast<const uint4*>(kr + ks * 32) : uint4{0, 0, 0, 0};
                sacc[kt] = mfma_bf16(qf[ks], kf, sacc[kt]);
            }
        }
        stage_values();
        if (NV > 1) fetch_values(1);
        // mask, scale, online softmax (rows 4 kg + v; this lane's keys: kt * 16 + m16)
        float mx[4], sc[4][4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int r = 4 * kg + v, qpos = pos0 + r;
            mx[v] = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                const int key = key_at(j0 + kt * 16 + m16);
                const bool ok_ = r < nq && key <= qpos && (p.window == 0 || qpos - key < p.window || key < p.keep);
                sc[v][kt] = ok_ ? cap_score(sacc[kt][v] * p.scale, p.softcap) - (p.dist ? dist_bias(r1, r2, qpos - key) : 0.f) : -INFINITY;
                mx[v] = fmaxf(mx[v], sc[v][kt]);
            }
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) mx[v] = fmaxf(mx[v], __shfl_xor(mx[v], o));
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float mn = fmaxf(mrow[v], mx[v]);
            const float corr = (mn == -INFINITY || mrow[v] == -INFINITY) ? (mn == -INFINITY ? 1.f : 0.f) : expf(mrow[v] - mn);
            float rs = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                const float pv = sc[v][kt] == -INFINITY ? 0.f : expf(sc[v][kt] - mn);
                rs += pv;
                const uint16_t ph = f32_to_bf16(pv);
                Ph[(4 * kg + v) * RS + kt * 16 + m16] = ph;
                Pl[(4 * kg + v) * RS + kt * 16 + m16] = f32_to_bf16(pv - bf16_to_f32(ph));
            }
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) rs += __shfl_xor(rs, o);
            lrow[v] = lrow[v] * corr + rs;
            mrow[v] = mn;
#pragma unroll
            for (int n = 0; n < NV; ++n)
#pragma unroll
                for (int c = 0; c < VT; ++c) acc[n][c][v] *= corr;
        }
        __syncthreads();
        uint4 ah[2], al[2];
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2) {
            ah[k2] = *reinterpret_cast<const uint4*>(&Ph[m16 * RS + k2 * 32 + 8 * kg]);
            al[k2] = *reinterpret_cast<const uint4*>(&Pl[m16 * RS + k2 * 32 + 8 * kg]);
        }
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            if (n > 0) {
                stage_values();
                __syncthreads();
                if (n + 1 < NV) fetch_values(n + 1);
            }
#pragma unroll
            for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
                for (int c = 0; c < VT; ++c) {
                    const uint4 vf = value_fragment(k2, c);
                    acc[n][c] = mfma_bf16(ah[k2], vf, acc[n][c]);
                    acc[n][c] = mfma_bf16(al[k2], vf, acc[n][c]);
                }
            __syncthreads();
        }
    }
    const float sink = p.sink ? p.sink[h] : -INFINITY;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int r = 4 * kg + v;
        if (r >= nq) continue;
        const float M = fmaxf(mrow[v], sink);
        const float cm = expf(mrow[v] - M);
        const float L = lrow[v] * cm + (p.sink ? expf(sink - M) : 0.f);
        const float f = cm / L * p.out_scale;
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            const size_t base = (size_t)(t0 + r) * p.ldo + p.out_off + (size_t)(oh0 + n) * vd;
#pragma unroll
            for (int c = 0; c < VT; ++c) {
                const float o = acc[n][c][v] * f;
                if (p.out_f32) static_cast<float*>(p.out)[base + c * 16 + m16] = o;
                else static_cast<uint16_t*>(p.out)[base + c * 16 + m16] = f32_to_bf16(o);
            }
        }
    }
}

// The same prompt-sized step for grouped-query attention: a workgroup of HPG waves takes HPG query heads that share ONE key/value head
// for the same tile of 16 tokens -- same keys, same mask -- so the 64 key rows and the transposed 64 value rows of a chunk are staged in
// LDS once per workgroup (cooperatively, the next chunk's rows already in flight in registers) instead of once per head from L2, and
// the key fragments of S = Q K^T are 16-byte LDS reads.  Softmax, the two probability planes and the products are as above, per wave.
template <int DK, int VT, int HPG> __global__ __launch_bounds__(64 * HPG) void window_attention_group_kernel(AttnArgs p) {
    constexpr int RS = 72;                                           // bf16 per row of P and V^T: 64 keys + 8 of padding
    constexpr int KRS = DK * 32 + 8;                                 // bf16 per staged key row (16 rows of a fragment read: 16 different bank groups)
    constexpr int NT = 64 * HPG;
    constexpr int KCH = DK * 4;                                      // 16-byte chunks of a key row
    constexpr int KPT = (64 * KCH + NT - 1) / NT;                    // key chunks per thread and stage
    constexpr int VPT = (VT * 2 + HPG - 1) / HPG;                    // value chunks (8 columns) per wave and stage
    __shared__ __align__(16) uint16_t Ks[64 * KRS], Vt[VT * 16 * RS], Ph[HPG][16 * RS], Pl[HPG][16 * RS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, m16 = lane & 15, kg = lane >> 4;
    int b = blockIdx.x, s = 0, n_new = 0;
    for (; s < p.n_seqs; ++s) {
        n_new = (int)(p.cu_q[s + 1] - p.cu_q[s]);
        const int tiles = (n_new + 15) >> 4;
        if (b < tiles) break;
        b -= tiles;
    }
    if (s >= p.n_seqs) return;
    const int t0 = (int)p.cu_q[s] + b * 16, nq = min(16, (int)p.cu_q[s + 1] - t0);
    const int pos0 = (int)p.ctx[s] - n_new + b * 16;
    const int h = blockIdx.y * HPG + wave, g = h / (p.H / p.G), d = p.d, vd = p.vd;
    const uint16_t* Q = static_cast<const uint16_t*>(p.q);
    const uint16_t* K = static_cast<const uint16_t*>(p.k_pages);
    const uint16_t* V = static_cast<const uint16_t*>(p.v_pages);
    const uint32_t* bt = p.bt + (size_t)s * p.max_blocks;
    uint4 qf[DK];
#pragma unroll
    for (int ks = 0; ks < DK; ++ks)
        qf[ks] = m16 < nq ? *reinterpret_cast<const uint4*>(Q + ((size_t)(t0 + m16) * p.H + h) * d + ks * 32 + 8 * kg) : uint4{0, 0, 0, 0};
    float mrow[4], lrow[4];
    f32x4_t acc[VT];
#pragma unroll
    for (int v = 0; v < 4; ++v) { mrow[v] = -INFINITY; lrow[v] = 0.f; }
#pragma unroll
    for (int c = 0; c < VT; ++c) acc[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int hi = pos0 + nq - 1;
    const float r1 = p.dist ? p.dist[h] : 0.f, r2 = p.dist ? p.dist[p.H + h] : 0.f;
    const int lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
    const int nkeep = min(p.keep, lo), n_vis = nkeep + hi - lo + 1;
    auto key_at = [&](int i) { return i < nkeep ? i : (i < n_vis ? lo + (i - nkeep) : hi + 1); };
    auto page_row = [&](int key) { return (size_t)bt[key / p.bs] * p.bs + (key % p.bs); };
    uint4 kreg[KPT], vreg[VPT];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int n = 0; n < KPT; ++n) {
            const int idx = tid + n * NT, ki = idx / KCH, c = idx - ki * KCH;
            const int key = ki < 64 ? key_at(j0 + ki) : hi + 1;
            kreg[n] = key <= hi ? *reinterpret_cast<const uint4*>(K + page_row(key) * p.k_ld + g * d + c * 8) : uint4{0, 0, 0, 0};
        }
        const int vkey = key_at(j0 + lane);
        const uint16_t* vrow = V + (vkey <= hi ? page_row(vkey) : 0) * p.v_ld + g * vd;
#pragma unroll
        for (int n = 0; n < VPT; ++n) {
            const int c8 = wave + n * HPG;
            vreg[n] = (vkey <= hi && c8 < VT * 2) ? *reinterpret_cast<const uint4*>(vrow + c8 * 8) : uint4{0, 0, 0, 0};
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int n = 0; n < KPT; ++n) {
            const int idx = tid + n * NT, ki = idx / KCH, c = idx - ki * KCH;
            if (ki < 64) *reinterpret_cast<uint4*>(&Ks[ki * KRS + c * 8]) = kreg[n];
        }
        // transposing store of the value rows (zeros past the end): the lane pair (2a, 2a + 1) swaps words, every lane writes one 4-byte
        // word = two keys of one column
        const int col_odd = lane & 1, key_even = lane & ~1;
#pragma unroll
        for (int n = 0; n < VPT; ++n) {
            const int c8 = wave + n * HPG;
            if (c8 >= VT * 2) break;
            const uint32_t w[4] = {vreg[n].x, vreg[n].y, vreg[n].z, vreg[n].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)w[e], 0xB1, 0xF, 0xF, true);   // quad_perm [1, 0, 3, 2]
                const uint32_t pair = col_odd ? ((other >> 16) | (w[e] & 0xFFFF0000u)) : ((w[e] & 0xFFFFu) | (other << 16));
                *reinterpret_cast<uint32_t*>(&Vt[(c8 * 8 + 2 * e + col_odd) * RS + key_even]) = pair;
            }
        }
    };
    uint16_t* ph = Ph[wave];
    uint16_t* pl = Pl[wave];
    fetch(0);
    for (int j0 = 0; j0 < n_vis; j0 += 64) {
        __syncthreads();                                             // the chunk before is multiplied: its rows may go
        stage();
        __syncthreads();
        if (j0 + 64 < n_vis) fetch(j0 + 64);
        f32x4_t sacc[4];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            sacc[kt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < DK; ++ks) {
                const uint4 kf = *reinterpret_cast<const uint4*>(&Ks[(kt * 16 + m16) * KRS + ks * 32 + 8 * kg]);
                sacc[kt] = mfma_bf16(qf[ks], kf, sacc[kt]);
            }
        }
        float mx[4], sc[4][4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int r = 4 * kg + v, qpos = pos0 + r;
            mx[v] = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                const int key = key_at(j0 + kt * 16 + m16);
                const bool ok_ = r < nq && key <= qpos && (p.window == 0 || qpos - key < p.window || key < p.keep);
                sc[v][kt] = ok_ ? cap_score(sacc[kt][v] * p.scale, p.softcap) - (p.dist ? dist_bias(r1, r2, qpos - key) : 0.f) : -INFINITY;
                mx[v] = fmaxf(mx[v], sc[v][kt]);
            }
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) mx[v] = fmaxf(mx[v], __shfl_xor(mx[v], o));
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float mn = fmaxf(mrow[v], mx[v]);
            const float corr = (mn == -INFINITY || mrow[v] == -INFINITY) ? (mn == -INFINITY ? 1.f : 0.f) : expf(mrow[v] - mn);
            float rs = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                const float pv = sc[v][kt] == -INFINITY ? 0.f : expf(sc[v][kt] - mn);
                rs += pv;
                const uint16_t hb = f32_to_bf16(pv);
                ph[(4 * kg + v) * RS + kt * 16 + m16] = hb;
                pl[(4 * kg + v) * RS + kt * 16 + m16] = f32_to_bf16(pv - bf16_to_f32(hb));
            }
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) rs += __shfl_xor(rs, o);
            lrow[v] = lrow[v] * corr + rs;
            mrow[v] = mn;
#pragma unroll
            for (int c = 0; c < VT; ++c) acc[c][v] *= corr;
        }
        __syncthreads();                                             // this wave's probability planes are written
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2) {
            const uint4 ah = *reinterpret_cast<const uint4*>(&ph[m16 * RS + k2 * 32 + 8 * kg]);
            const uint4 al = *reinterpret_cast<const uint4*>(&pl[m16 * RS + k2 * 32 + 8 * kg]);
#pragma unroll
            for (int c = 0; c < VT; ++c) {
                const uint4 vf = *reinterpret_cast<const uint4*>(&Vt[(c * 16 + m16) * RS + k2 * 32 + 8 * kg]);
                acc[c] = mfma_bf16(ah, vf, acc[c]);
                acc[c] = mfma_bf16(al, vf, acc[c]);
            }
        }
    }
    const float sink = p.sink ? p.sink[h] : -INFINITY;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int r = 4 * kg + v;
        if (r >= nq) continue;
        const float M = fmaxf(mrow[v], sink);
        const float cm = expf(mrow[v] - M);
        const float L = lrow[v] * cm + (p.sink ? expf(sink - M) : 0.f);
        const float f = cm / L * p.out_scale;
        const size_t base = (size_t)(t0 + r) * p.ldo + p.out_off + (size_t)h * vd;
#pragma unroll
        for (int c = 0; c < VT; ++c) {
            const float o = acc[c][v] * f;
            if (p.out_f32) static_cast<float*>(p.out)[base + c * 16 + m16] = o;
            else static_cast<uint16_t*>(p.out)[base + c * 16 + m16] = f32_to_bf16(o);
        }
    }
}

// ------------------------------------------------------------------------------------------------------------ short convolution
struct ConvArgs {
    float* out; const float* proj; int ldp, off; const float* w; float* state; int64_t state_stride;
    const uint32_t* ctx; const uint32_t* cu_q; const int32_t* slots; const int32_t* tok_seq; int C, taps, T;
    int act;                // 0 = none, 1 = silu
    int add_input;          // the convolution is added to its own input (h + conv(h))
    uint16_t* out_bf16;     // != NULL: the result goes here as bf16 instead of `out`
    const float* bias;      // != NULL: added per channel in front of the activation
};
__global__ void conv_silu_kernel(ConvArgs p) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)p.T * p.C) return;
    const int t = (int)(idx / p.C), c = (int)(idx - (int64_t)t * p.C);
    const int s = p.tok_seq[t];
    const int cs = (int)p.cu_q[s];
    const int start_pos = (int)p.ctx[s] - (int)(p.cu_q[s + 1] - p.cu_q[s]);
    const float* stt = p.state + (size_t)p.slots[s] * p.state_stride + (size_t)c * (p.taps - 1);
    float acc = 0.f;
    for (int i = 0; i < p.taps; ++i) {
        const int o = t - (p.taps - 1 - i);
        float v;
        if (o >= cs) v = p.proj[(size_t)o * p.ldp + p.off + c];
        else {
            const int back = cs - o;                                // 1 = the input just before the portion
            v = (start_pos > 0 && start_pos - back >= 0) ? stt[p.taps - 1 - back] : 0.f;
        }
        acc = fmaf(p.w[(size_t)c * p.taps + i], v, acc);
    }
    if (p.add_input) acc += p.proj[(size_t)t * p.ldp + p.off + c];
    if (p.bias) acc += p.bias[c];
    acc = p.act ? siluf_(acc) : acc;
    if (p.out_bf16) p.out_bf16[idx] = f32_to_bf16(acc); else p.out[idx] = acc;
}
// state[j], j = 0 .. taps-2 (oldest first) <- the taps - 1 inputs that end with the portion's last token
__global__ void conv_state_update_kernel(ConvArgs p, int n_seqs) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_seqs * p.C) return;
    const int s = idx / p.C, c = idx - s * p.C;
    const int cs = (int)p.cu_q[s], ce = (int)p.cu_q[s + 1], n = ce - cs;
    if (n <= 0) return;
    const int start_pos = (int)p.ctx[s] - n;
    float* stt = p.state + (size_t)p.slots[s] * p.state_stride + (size_t)c * (p.taps - 1);
    const int keep = p.taps - 1;
    float nv[15];
    for (int j = 0; j < keep; ++j) {
        const int back = keep - j;                                   // 1 = the portion's last token
        float v;
        if (back <= n) v = p.proj[(size_t)(ce - back) * p.ldp + p.off + c];
        else { const int b2 = back - n; v = (start_pos > 0 && start_pos - b2 >= 0) ? stt[keep - b2] : 0.f; }
        nv[j] = v;
    }
    for (int j = 0; j < keep; ++j) stt[j] = nv[j];
}

// The norm in front of a mixer and the convolution added to the mixer's input in one launch: h = x / rms(x) w (nw NULL: h = x),
// out = h + conv(h).  A workgroup per token recomputes the norms of the TAPS - 1 rows before it that lie in the same portion (the rows
// before the portion come from the state slot, zeros before position 0).  hn != NULL receives h (what conv_state_update_kernel then
// reads); update: every sequence of the step brings ONE token, and the token's workgroup moves the slot's rows itself (a thread reads
// and writes its own channels only).
struct NormConvArgs {
    float* out; uint16_t* out_bf16; float* hn; const float* x; const float* nw; const float* cw; float* state; int64_t state_stride;
    const uint32_t* ctx; const uint32_t* cu_q; const int32_t* slots; const int32_t* tok_seq; int W, update; float eps;
};
template <int TAPS, int NW> __global__ __launch_bounds__(64 * NW) void norm_conv_kernel(NormConvArgs p) {
    __shared__ float red[TAPS][NW];
    __shared__ float inv_s[TAPS];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int s = p.tok_seq[t], cs = (int)p.cu_q[s];
    const int start_pos = (int)p.ctx[s] - (int)(p.cu_q[s + 1] - p.cu_q[s]);
    if (p.nw) {
        float ss[TAPS];
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
            ss[j] = 0.f;
            const int o = t - (TAPS - 1 - j);
            if (o >= cs)
                for (int i = threadIdx.x; i < p.W; i += 64 * NW) { const float v = p.x[(size_t)o * p.W + i]; ss[j] = fmaf(v, v, ss[j]); }
        }
#pragma unroll
        for (int j = 0; j < TAPS; ++j) { ss[j] = wave_sum(ss[j]); if (lane == 0) red[j][wave] = ss[j]; }
        __syncthreads();
        if (threadIdx.x < TAPS) {
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) sum += red[threadIdx.x][w];
            inv_s[threadIdx.x] = 1.f / sqrtf(sum / (float)p.W + p.eps);
        }
        __syncthreads();
    }
    float* stt = p.state + (size_t)p.slots[s] * p.state_stride;
    for (int i = threadIdx.x; i < p.W; i += 64 * NW) {
        float h[TAPS], acc = 0.f;
#pragma unroll
        for (int j = 0; j < TAPS; ++j) {
            const int o = t - (TAPS - 1 - j);
            if (o >= cs) h[j] = p.nw ? p.x[(size_t)o * p.W + i] * inv_s[j] * p.nw[i] : p.x[(size_t)o * p.W + i];
            else { const int back = cs - o; h[j] = (start_pos > 0 && start_pos - back >= 0) ? stt[(size_t)i * (TAPS - 1) + (TAPS - 1 - back)] : 0.f; }
            acc = fmaf(p.cw[(size_t)i * TAPS + j], h[j], acc);
        }
        acc += h[TAPS - 1];
        if (p.out_bf16) p.out_bf16[(size_t)t * p.W + i] = f32_to_bf16(acc); else p.out[(size_t)t * p.W + i] = acc;
        if (p.hn) p.hn[(size_t)t * p.W + i] = h[TAPS - 1];
        if (p.update)
#pragma unroll
            for (int j = 0; j + 1 < TAPS; ++j) stt[(size_t)i * (TAPS - 1) + j] = h[j + 1];
    }
}

// ------------------------------------------------------------------------------------------------------------ gated delta rule
struct DeltaArgs {
    float* o; float* state; int64_t state_stride;
    const float* qkv; int ldq;
    const float* proj; int ldp, b_off;
    const float* decay_in; int ldd, decay_channels;
    const float* a_log; const float* dt_bias;
    const uint32_t* ctx; const uint32_t* cu_q; const int32_t* slots;
    int H, G, d, vd; float unit_eps;
};
// Everything of the rule that does not depend on the state is computed for all new tokens at once, one wave per (token, head):
// prep [T, P] = unit q times d^-1/2 and unit k per q/k head, the decays per head (or per head and key channel), beta per head.
__global__ __launch_bounds__(64) void delta_prep_kernel(DeltaArgs p, float* prep, int P, int T) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int d = p.d, hpg = p.H / p.G, g = h / hpg;
    float* out = prep + (size_t)t * P;
    const int q_off = 0, k_off = p.G * d, g_off = 2 * p.G * d, dd = p.decay_channels ? d : 1, b_off = g_off + p.H * dd;
    if (h % hpg == 0) {
        const float* row = p.qkv + (size_t)t * p.ldq;
        float qq = 0.f, kk = 0.f;
        for (int i = lane; i < d; i += 64) { const float a = row[g * d + i], b = row[p.G * d + g * d + i]; qq += a * a; kk += b * b; }
        qq = wave_sum(qq); kk = wave_sum(kk);
        const float qi = (1.f / sqrtf((float)d)) / sqrtf(qq + p.unit_eps), ki = 1.f / sqrtf(kk + p.unit_eps);
        for (int i = lane; i < d; i += 64) {
            out[q_off + g * d + i] = row[g * d + i] * qi;
            out[k_off + g * d + i] = row[p.G * d + g * d + i] * ki;
        }
    }
    const float a_rate = expf(p.a_log[h]);
    if (p.decay_channels) {
        for (int i = lane; i < d; i += 64) {
            const int ch = h * d + i;
            out[g_off + ch] = expf(-a_rate * softplusf_(p.decay_in[(size_t)t * p.ldd + ch] + p.dt_bias[ch]));
        }
    } else if (lane == 0) {
        out[g_off + h] = expf(-a_rate * softplusf_(p.decay_in[(size_t)t * p.ldd + h] + p.dt_bias[h]));
    }
    if (lane == 0) out[b_off + h] = sigmoidf_(p.proj[(size_t)t * p.ldp + p.b_off + h]);
}

// The scan.  A workgroup of 256 threads owns 256 / LPC columns of one (sequence, head)'s state S [d, vd]; LPC neighbouring lanes share
// a column, each holding DP = ceil(d / LPC) of its rows in registers, and walk the new tokens in order:
//   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// (the two sums over d are finished by lane exchanges among the LPC lanes).  The walk is a chain of dependent steps, so its time per
// token is the latency of one step: the more lanes share a column the shorter the step (LPC = 16 at d >= 64).  q, k, g of CH tokens
// at a time sit in LDS, rows padded so that the parts fall into different banks; the next CH tokens are fetched into registers
// while the current ones are used.
template <int DP, int LPC, int CH> __global__ __launch_bounds__(256) void delta_scan_kernel(DeltaArgs p, const float* __restrict__ prep, int P) {
    constexpr int RS = DP + 4, ROW = LPC * DP, TOT = CH * ROW, NPT = (TOT + 255) / 256, CPB = 256 / LPC;
    __shared__ __align__(16) float sq[2][CH][LPC][RS], sk[2][CH][LPC][RS], sg[2][CH][LPC][RS];
    __shared__ float sb[2][CH], sgh[2][CH];
    const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int col = blockIdx.z * CPB + tid / LPC, part = tid % LPC;
    const int d = p.d, vd = p.vd, g = h / (p.H / p.G);
    const int tb = (int)p.cu_q[s], te = (int)p.cu_q[s + 1];
    if (te <= tb) return;
    const int start_pos = (int)p.ctx[s] - (te - tb);
    const bool own = col < vd, chan = p.decay_channels != 0;
    float* stt = p.state + (size_t)p.slots[s] * p.state_stride + (size_t)h * d * vd;
    float S[DP];
#pragma unroll
    for (int r = 0; r < DP; ++r) { const int i = part * DP + r; S[r] = (own && i < d && start_pos > 0) ? stt[(size_t)i * vd + col] : 0.f; }
    const int q_off = g * d, k_off = p.G * d + g * d, g_off = 2 * p.G * d + (chan ? h * d : h), b_off = 2 * p.G * d + p.H * (chan ? d : 1) + h;
    const int v_col = 2 * p.G * d + h * vd + col;
    float rq[NPT], rk[NPT], rg[NPT], rv[CH], rbeta = 0.f, rgh = 1.f;
    auto fetch = [&](int t0) {
#pragma unroll
        for (int n = 0; n < NPT; ++n) {
            const int idx = tid + n * 256, c = idx / ROW, ii = idx - c * ROW, t = t0 + c;
            const bool ok_ = idx < TOT && t < te && ii < d;
            const float* row = prep + (size_t)(ok_ ? t : tb) * P;
            rq[n] = ok_ ? row[q_off + ii] : 0.f;
            rk[n] = ok_ ? row[k_off + ii] : 0.f;
            rg[n] = (ok_ && chan) ? row[g_off + ii] : 1.f;
        }
#pragma unroll
        for (int c = 0; c < CH; ++c) rv[c] = (own && t0 + c < te) ? p.qkv[(size_t)(t0 + c) * p.ldq + v_col] : 0.f;
        if (tid < CH && t0 + tid < te) {
            rbeta = prep[(size_t)(t0 + tid) * P + b_off];
            rgh = chan ? 1.f : prep[(size_t)(t0 + tid) * P + g_off];
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int n = 0; n < NPT; ++n) {
            const int idx = tid + n * 256;
            if (idx < TOT) {
                const int c = idx / ROW, ii = idx - c * ROW, pp = ii / DP, r = ii - pp * DP;
                sq[buf][c][pp][r] = rq[n]; sk[buf][c][pp][r] = rk[n]; sg[buf][c][pp][r] = rg[n];
            }
        }
        if (tid < CH) { sb[buf][tid] = rbeta; sgh[buf][tid] = rgh; }
    };
    fetch(tb);
    stage(0);
    __syncthreads();
    int buf = 0;
    for (int t0 = tb; t0 < te; t0 += CH, buf ^= 1) {
        float vc[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) vc[c] = rv[c];
        const bool more = t0 + CH < te;
        if (more) fetch(t0 + CH);
        const int cn = min(CH, te - t0);
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            if (c < cn) {
                float kv = 0.f;
                if (chan) {
#pragma unroll
                    for (int r = 0; r < DP; ++r) { S[r] *= sg[buf][c][part][r]; kv = fmaf(S[r], sk[buf][c][part][r], kv); }
                } else {
                    const float gh = sgh[buf][c];
#pragma unroll
                    for (int r = 0; r < DP; ++r) { S[r] *= gh; kv = fmaf(S[r], sk[buf][c][part][r], kv); }
                }
                kv = column_sum<LPC>(kv);
                const float u = sb[buf][c] * (vc[c] - kv);
                float o = 0.f;
#pragma unroll
                for (int r = 0; r < DP; ++r) { S[r] = fmaf(sk[buf][c][part][r], u, S[r]); o = fmaf(S[r], sq[buf][c][part][r], o); }
                o = column_sum<LPC>(o);
                if (own && part == 0) p.o[((size_t)(t0 + c) * p.H + h) * vd + col] = o;
            }
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
    }
    if (own)
#pragma unroll
        for (int r = 0; r < DP; ++r) { const int i = part * DP + r; if (i < d) stt[(size_t)i * vd + col] = S[r]; }
}

// out = o / rms(o) * w * gate * out_scale, one wave per (token, head)
template <typename TO> __global__ __launch_bounds__(64) void gated_norm_kernel(TO* out, int ldo, int out_off, const float* o, const float* w,
                                                                              const float* gate_in, int ldg, int gate, int H, int vd,
                                                                              float eps, float out_scale) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* orow = o + ((size_t)t * H + h) * vd;
    float ss = 0.f;
    for (int i = lane; i < vd; i += 64) ss += orow[i] * orow[i];
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)vd + eps);
    for (int i = lane; i < vd; i += 64) {
        const float gi = gate_in[(size_t)t * ldg + h * vd + i];
        const float gt = gate == MI355_HYB_GATE_SILU ? siluf_(gi) : sigmoidf_(gi);
        st<TO>(out, (size_t)t * ldo + out_off + h * vd + i, orow[i] * inv * w[i] * gt * out_scale);
    }
}

// ------------------------------------------------------------------------------------------------------------ minGRU
struct GruArgs {
    void* out; float* state; int64_t state_stride; const float* proj; int ldp, z_off, x_off, g_off;
    const uint32_t* ctx; const uint32_t* cu_q; const int32_t* slots; int width;
};
// thread = (sequence, channel); the gates read only the current token, so their loads run UNR tokens ahead of the recurrence
template <typename TO, int UNR> __global__ __launch_bounds__(64) void mingru_kernel(GruArgs p) {
    const int s = blockIdx.y, c = blockIdx.x * 64 + threadIdx.x;
    if (c >= p.width) return;
    const int tb = (int)p.cu_q[s], te = (int)p.cu_q[s + 1];
    if (te <= tb) return;
    const int start_pos = (int)p.ctx[s] - (te - tb);
    float* stt = p.state + (size_t)p.slots[s] * p.state_stride;
    float S = start_pos > 0 ? stt[c] : 0.f;
    for (int t0 = tb; t0 < te; t0 += UNR) {
        float z[UNR], u[UNR], gg[UNR];
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            const int t = min(t0 + k, te - 1);
            const float* row = p.proj + (size_t)t * p.ldp;
            z[k] = row[p.z_off + c]; u[k] = row[p.x_off + c]; gg[k] = row[p.g_off + c];
        }
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            if (t0 + k >= te) break;
            const float zz = sigmoidf_(z[k]);
            const float cand = u[k] >= 0.f ? u[k] + 0.5f : sigmoidf_(u[k]);
            S = (1.f - zz) * S + zz * cand;
            st<TO>(static_cast<TO*>(p.out), (size_t)(t0 + k) * p.width + c, S * siluf_(gg[k]));
        }
    }
    stt[c] = S;
}

// Long portions: S_t = (1 - z_t) S_(t-1) + z_t c_t is a composition of affine maps, so the portion is cut into NSEG segments, one wave
// each: pass 1 reduces a segment to (A, B) with S_end = A S_start + B, the waves exchange (A, B) through LDS, every wave folds the
// segments before its own into its starting state and walks its segment again writing the outputs.
template <typename TO, int NSEG, int UNR> __global__ __launch_bounds__(64 * NSEG) void mingru_seg_kernel(GruArgs p) {
    __shared__ float sA[NSEG][64], sB[NSEG][64];
    const int s = blockIdx.y, lane = threadIdx.x & 63, w = threadIdx.x >> 6, c = blockIdx.x * 64 + lane;
    const int tb = (int)p.cu_q[s], te = (int)p.cu_q[s + 1];
    if (te <= tb) return;
    const bool ok_ = c < p.width;
    const int cc = ok_ ? c : 0;
    const int seg = (te - tb + NSEG - 1) / NSEG;
    const int lo = min(te, tb + w * seg), hi = min(te, lo + seg);
    float A = 1.f, B = 0.f;
    for (int t0 = lo; t0 < hi; t0 += UNR) {
        float z[UNR], u[UNR];
#pragma unroll
        for (int k = 0; k < UNR; ++k) { const float* row = p.proj + (size_t)min(t0 + k, hi - 1) * p.ldp; z[k] = row[p.z_off + cc]; u[k] = row[p.x_off + cc]; }
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            if (t0 + k >= hi) break;
            const float zz = sigmoidf_(z[k]), cand = u[k] >= 0.f ? u[k] + 0.5f : sigmoidf_(u[k]);
            A *= (1.f - zz);
            B = (1.f - zz) * B + zz * cand;
        }
    }
    sA[w][lane] = A; sB[w][lane] = B;
    __syncthreads();
    const int start_pos = (int)p.ctx[s] - (te - tb);
    float* stt = p.state + (size_t)p.slots[s] * p.state_stride;
    float S = (start_pos > 0 && ok_) ? stt[cc] : 0.f;
    for (int v = 0; v < w; ++v) S = sA[v][lane] * S + sB[v][lane];
    for (int t0 = lo; t0 < hi; t0 += UNR) {
        float z[UNR], u[UNR], gg[UNR];
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            const float* row = p.proj + (size_t)min(t0 + k, hi - 1) * p.ldp;
            z[k] = row[p.z_off + cc]; u[k] = row[p.x_off + cc]; gg[k] = row[p.g_off + cc];
        }
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            if (t0 + k >= hi) break;
            const float zz = sigmoidf_(z[k]), cand = u[k] >= 0.f ? u[k] + 0.5f : sigmoidf_(u[k]);
            S = (1.f - zz) * S + zz * cand;
            if (ok_) st<TO>(static_cast<TO*>(p.out), (size_t)(t0 + k) * p.width + c, S * siluf_(gg[k]));
        }
    }
    if (w == NSEG - 1 && ok_) stt[c] = S;
}

__global__ void token_seq_kernel(int32_t* tok_seq, const uint32_t* cu_q, int n_seqs) {
    const int s = blockIdx.x;
    for (int t = (int)cu_q[s] + threadIdx.x; t < (int)cu_q[s + 1]; t += blockDim.x) tok_seq[t] = s;
}
__global__ void bf16_to_f32_kernel(float* out, const uint16_t* in, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = bf16_to_f32(in[i]);
}
__global__ void copy_f32_kernel(float* out, const float* in, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = in[i];
}
__global__ void fill_f32_kernel(float* out, float v, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = v;
}

// ------------------------------------------------------------------------------------------------------------ more attention glue
struct WholePrepArgs {
    void* q_out; void* k_pages; void* v_pages;
    const float* src; int ld, q_off, k_off, v_off;
    const float* qw; const float* kw; const int64_t* slots;
    int H, G, d, vd, v_unit; float eps;
};
// One workgroup per token.  q and k: ONE RMS norm over the whole row part (all heads at once), weights of that size; v: every head
// divided by its own root mean square (no weight).  q -> q_out, k and v -> the token's page row.  No rotation.
template <typename TC> __global__ __launch_bounds__(256) void attn_prepare_whole_kernel(WholePrepArgs p) {
    __shared__ float red[4];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* row = p.src + (size_t)t * p.ld;
    const int nq = p.H * p.d, nk = p.G * p.d;
    const int64_t slot = p.slots[t];
    float sq = 0.f, sk = 0.f;
    if (p.qw) for (int i = threadIdx.x; i < nq; i += blockDim.x) { const float v = row[p.q_off + i]; sq = fmaf(v, v, sq); }
    if (p.kw) for (int i = threadIdx.x; i < nk; i += blockDim.x) { const float v = row[p.k_off + i]; sk = fmaf(v, v, sk); }
    sq = block_sum(sq, red);
    sk = block_sum(sk, red);
    const float iq = p.qw ? 1.f / sqrtf(sq / (float)nq + p.eps) : 1.f, ik = p.kw ? 1.f / sqrtf(sk / (float)nk + p.eps) : 1.f;
    TC* qd = static_cast<TC*>(p.q_out) + (size_t)t * nq;
    for (int i = threadIdx.x; i < nq; i += blockDim.x) st<TC>(qd, i, row[p.q_off + i] * iq * (p.qw ? p.qw[i] : 1.f));
    if (slot < 0) return;
    TC* kd = static_cast<TC*>(p.k_pages) + (size_t)slot * nk;
    for (int i = threadIdx.x; i < nk; i += blockDim.x) st<TC>(kd, i, row[p.k_off + i] * ik * (p.kw ? p.kw[i] : 1.f));
    TC* vdst = static_cast<TC*>(p.v_pages) + (size_t)slot * p.G * p.vd;
    for (int g = wave; g < p.G; g += (int)(blockDim.x >> 6)) {          // a wave per value head
        const float* vr = row + p.v_off + g * p.vd;
        float ss = 0.f;
        if (p.v_unit) { for (int i = lane; i < p.vd; i += 64) ss = fmaf(vr[i], vr[i], ss); ss = wave_sum(ss); }
        const float iv = p.v_unit ? 1.f / sqrtf(ss / (float)p.vd + p.eps) : 1.f;
        for (int i = lane; i < p.vd; i += 64) st<TC>(vdst, (size_t)g * p.vd + i, vr[i] * iv);
    }
}

struct LatentPrepArgs {
    void* q_out; void* pages;
    const float* qsrc; int ldq, q_off; const float* csrc; int ldc, c_off;   // pages NULL: nothing is cached and csrc is not read
    const float* q_abs; const float* cw; const float* cos_t; const float* sin_t;
    const int64_t* positions; const int64_t* slots;
    int H, d, r, rank, rot, interleaved; float eps;
};
// element i of a rot_dim-wide vector v after the rotation of its first `rot` dimensions by the angles of position `pos`
__device__ __forceinline__ float rotated_elem(const float* v, int i, int rot, int interleaved, const float* cs, const float* sn) {
    if (i >= rot) return v[i];
    const int half = rot / 2;
    if (interleaved) {
        const int pr = i >> 1;
        return (i & 1) ? v[i] * cs[pr] + v[i - 1] * sn[pr] : v[i] * cs[pr] - v[i + 1] * sn[pr];
    }
    return i < half ? v[i] * cs[i] - v[i + half] * sn[i] : v[i] * cs[i - half] + v[i - half] * sn[i - half];
}
// One workgroup per token: the latent's RMS norm and the rotation of the shared key part -> the token's page row [latent | key part];
// per head [absorbed query (already multiplied by the key up-projection) | rotated query part] -> q_out.
template <typename TC> __global__ __launch_bounds__(256) void latent_prepare_kernel(LatentPrepArgs p) {
    __shared__ float red[4];
    const int t = blockIdx.x, dq = p.rank + p.r;
    const float* row = p.qsrc + (size_t)t * p.ldq;
    const int64_t pos = p.positions[t], slot = p.slots[t];
    const float* cs = p.cos_t + pos * (p.rot / 2);
    const float* sn = p.sin_t + pos * (p.rot / 2);
    if (p.pages) {
        const float* crow = p.csrc + (size_t)t * p.ldc + p.c_off;
        float ss = 0.f;
        for (int i = threadIdx.x; i < p.rank; i += blockDim.x) { const float v = crow[i]; ss = fmaf(v, v, ss); }
        ss = block_sum(ss, red);
        const float inv = 1.f / sqrtf(ss / (float)p.rank + p.eps);
        if (slot >= 0) {
            TC* dst = static_cast<TC*>(p.pages) + (size_t)slot * dq;
            for (int i = threadIdx.x; i < p.rank; i += blockDim.x) st<TC>(dst, i, crow[i] * inv * p.cw[i]);
            const float* kr = crow + p.rank;
            for (int i = threadIdx.x; i < p.r; i += blockDim.x) st<TC>(dst, p.rank + i, rotated_elem(kr, i, p.rot, p.interleaved, cs, sn));
        }
    }
    TC* qd = static_cast<TC*>(p.q_out) + (size_t)t * p.H * dq;
    for (int i = threadIdx.x; i < p.H * dq; i += blockDim.x) {
        const int h = i / dq, c = i - h * dq;
        const float v = c < p.rank ? p.q_abs[((size_t)t * p.H + h) * p.rank + c]
                                   : rotated_elem(row + p.q_off + h * (p.d + p.r) + p.d, c - p.rank, p.rot, p.interleaved, cs, sn);
        st<TC>(qd, i, v);
    }
}

// out[t, h, :] = sum_g talk[h, g] a[t, g, kv head of h, :]
template <typename TO> __global__ void head_mix_kernel(TO* out, const float* a, const float* talk, int64_t n, int H, int G, int vd) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t t = i / ((int64_t)H * vd);
    const int rem = (int)(i - t * H * vd), h = rem / vd, c = rem - h * vd, kv = h / (H / G);
    const float* at = a + (size_t)t * H * G * vd + (size_t)kv * vd + c;
    float acc = 0.f;
    for (int g = 0; g < H; ++g) acc = fmaf(talk[h * H + g], at[(size_t)g * G * vd], acc);
    st<TO>(out, (size_t)i, acc);
}

template <typename TO> __global__ void head_gate_kernel(TO* out, const float* in, const float* gate_in, int ldg, int64_t n, int H, int vd) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t t = i / ((int64_t)H * vd);
    const int h = (int)(i - t * H * vd) / vd;
    st<TO>(out, (size_t)i, gate_in ? in[i] * sigmoidf_(gate_in[(size_t)t * ldg + h]) : in[i]);
}


// ------------------------------------------------------------------------------------------------------------ mixture of experts
// Routing, one workgroup per token: the normalised row h is built once in LDS (and written out for the experts' products), a wave
// takes the experts e = wave, wave + 4, ... (f32 router rows . h), then wave 0 makes the softmax, the choice by s + correction
// (largest first, ties to the lower expert) and the weights s[chosen] * scale.  The shared expert's gate is one more row.
template <typename TO, int NW> __global__ __launch_bounds__(64 * NW) void moe_route_kernel(int32_t* ids, float* wts, float* sgate, TO* xn, const float* x,
                                                                               const float* norm_w, const float* router, const float* corr,
                                                                               const float* gate_row, int width, int E, int K, float scale,
                                                                               float eps, int append, int sig, int groups, int keep, int normalise) {
    extern __shared__ __align__(16) float rsm[];
    float* hs = rsm;                       // [width]
    float* logit = hs + width;             // [E + 1]
    float* sc = logit + E + 1;             // [E] scores
    float* cv = sc + E;                    // [E] choice scores
    float* gs = cv + E;                    // [E] group scores
    __shared__ float red[NW];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* xr = x + (size_t)t * width;
    float inv = 1.f;
    if (norm_w) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < width; i += blockDim.x) ss += xr[i] * xr[i];
        inv = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
    }
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = norm_w ? xr[i] * inv * norm_w[i] : xr[i];
        hs[i] = v;
        if (xn) st<TO>(xn, (size_t)t * width + i, v);
    }
    __syncthreads();
    const int rows = E + (gate_row ? 1 : 0);
    for (int e = wave; e < rows; e += NW) {
        const float* g = e < E ? router + (size_t)e * width : gate_row;
        float acc = 0.f;
        if ((width & 3) == 0) {
            // eight 16-byte pieces of the row per lane are requested before the first is used
            for (int i0 = 4 * lane; i0 < width; i0 += 8 * 256) {
                float4 gv[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) gv[u] = i0 + 256 * u < width ? *reinterpret_cast<const float4*>(g + i0 + 256 * u) : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (i0 + 256 * u >= width) break;
                    const float4 hv = *reinterpret_cast<const float4*>(hs + i0 + 256 * u);
                    acc = fmaf(hv.x, gv[u].x, fmaf(hv.y, gv[u].y, fmaf(hv.z, gv[u].z, fmaf(hv.w, gv[u].w, acc))));
                }
            }
        } else {
            for (int i = lane; i < width; i += 64) acc = fmaf(hs[i], g[i], acc);
        }
        acc = wave_sum(acc);
        if (lane == 0) logit[e] = acc;
    }
    __syncthreads();
    if (wave != 0) return;
    const int KS = K + (append ? 1 : 0);                                // pairs per token: the shared expert as one more pair of every token
    if (gate_row && lane == 0) {
        const float sg = sigmoidf_(logit[E]);
        if (sgate) sgate[t] = sg;
        if (append) { ids[(size_t)t * KS + K] = E; wts[(size_t)t * KS + K] = sg; }
    }
    // scores s (softmax or sigmoid of the logits) and choice scores s + correction, in LDS
    if (sig) {
        for (int e = lane; e < E; e += 64) { const float v = sigmoidf_(logit[e]); sc[e] = v; cv[e] = v + (corr ? corr[e] : 0.f); }
    } else {
        float m = -INFINITY;
        for (int e = lane; e < E; e += 64) m = fmaxf(m, logit[e]);
        m = wave_max(m);
        float den = 0.f;
        for (int e = lane; e < E; e += 64) den += expf(logit[e] - m);
        den = wave_sum(den);
        for (int e = lane; e < E; e += 64) { const float v = expf(logit[e] - m) / den; sc[e] = v; cv[e] = v + (corr ? corr[e] : 0.f); }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();
    if (groups > 0) {
        // a group's score: the sum of its two largest choice scores (its only one when a group is one expert); the experts of every
        // group but the keep best (ties to the lower group) leave the choice
        const int per = E / groups;
        for (int g = lane; g < groups; g += 64) {
            float b1 = -INFINITY, b2 = -INFINITY;
            for (int i = 0; i < per; ++i) { const float v = cv[g * per + i]; if (v > b1) { b2 = b1; b1 = v; } else if (v > b2) b2 = v; }
            gs[g] = per > 1 ? b1 + b2 : b1;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();
        for (int g = lane; g < groups; g += 64) {
            const float mine = gs[g];
            int rank = 0;
            for (int o = 0; o < groups; ++o) rank += (gs[o] > mine || (gs[o] == mine && o < g)) ? 1 : 0;
            if (rank >= keep) for (int i = 0; i < per; ++i) cv[g * per + i] = -INFINITY;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier();
    }
    // lane owns experts lane, lane + 64, ...: K rounds of (my best untaken choice score) -> wave maximum -> the lowest expert that has it
    unsigned long long taken = 0ull;                                    // bit i: my expert lane + 64 i is chosen already
    float wsum = 0.f;
    for (int j = 0; j < K; ++j) {
        float bv = -INFINITY; int be = 0x7fffffff;
        for (int e = lane, i = 0; e < E; e += 64, ++i) {
            const float c = cv[e];
            if (!((taken >> i) & 1ull) && (c > bv || be == 0x7fffffff)) { bv = c; be = e; }
        }
        const float top = wave_max(bv);
        int cand = (be != 0x7fffffff && bv == top) ? be : 0x7fffffff;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o));
        if (lane == (cand & 63)) taken |= 1ull << (cand >> 6);
        if (lane == 0) {
            ids[(size_t)t * KS + j] = cand;
            wts[(size_t)t * KS + j] = sc[cand] * scale;
            wsum += sc[cand];
        }
    }
    if (normalise && lane == 0) {
        const float inv = 1.f / (wsum + 1e-20f);
        for (int j = 0; j < K; ++j) wts[(size_t)t * KS + j] *= inv;
    }
}

// Grouping on the device, one workgroup: counts per expert, whole blocks of `bm` rows per expert, then every pair takes the next free
// row of its expert's blocks (rows are independent, so the order inside an expert does not reach any result).
__global__ __launch_bounds__(1024) void moe_group_kernel(int32_t* pos, int32_t* row_token, int32_t* table, const int32_t* ids, int pairs, int top,
                                                         int E, int bm, int n_blocks) {
    extern __shared__ int gsm[];
    int* cnt = gsm;                 // [E]
    int* blk0 = cnt + E;            // [E + 1]
    int* cur = blk0 + E + 1;        // [E]
    for (int e = threadIdx.x; e < E; e += blockDim.x) { cnt[e] = 0; cur[e] = 0; }
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        int e = ids[p];
        e = e < 0 ? 0 : (e >= E ? E - 1 : e);
        atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        blk0[0] = 0;
        for (int e = 0; e < E; ++e) blk0[e + 1] = blk0[e] + (cnt[e] + bm - 1) / bm;
    }
    __syncthreads();
    for (int b = threadIdx.x; b < n_blocks; b += blockDim.x) {
        int lo = 0, hi = E;                                             // the expert e with blk0[e] <= b < blk0[e + 1]
        if (b >= blk0[E]) { table[2 * b] = 0; table[2 * b + 1] = 0; continue; }
        while (hi - lo > 1) { const int mid = (lo + hi) >> 1; if (blk0[mid] <= b) lo = mid; else hi = mid; }
        table[2 * b] = lo;
        table[2 * b + 1] = bm * blk0[lo] + cnt[lo];
    }
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        int e = ids[p];
        e = e < 0 ? 0 : (e >= E ? E - 1 : e);
        const int r = bm * blk0[e] + atomicAdd(&cur[e], 1);
        pos[p] = r;
        row_token[r] = p / top;
    }
}

template <typename TO> __global__ void silu_glu_kernel(TO* out, const float* gu, int64_t n, int ff, const int32_t* table, int bm) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t t = i / ff; const int j = (int)(i - t * ff);
    if (table && t >= table[2 * (t / bm) + 1]) return;                  // a row that no pair landed in
    st<TO>(out, (size_t)i, siluf_(gu[t * 2 * ff + j]) * gu[t * 2 * ff + ff + j]);
}

// y[t] = sum_j wts[t, j] rows[pos[t top + j]] + gate[t] shared[t];  x[t] += y / rms(y) * w.  One workgroup per token; the token's row
// indices and weights go through LDS first (so that the row loads do not wait on them one after the other); y stays in registers
// between the two passes (width <= 256 x 16).  VEC: 16-byte accesses (width a multiple of 4).
template <bool VEC> __global__ __launch_bounds__(256) void moe_combine_norm_add_kernel(float* __restrict__ x, uint16_t* __restrict__ xcopy,
                                                                                       const float* __restrict__ rows, const int32_t* __restrict__ pos,
                                                                                       const float* __restrict__ wts, const float* __restrict__ shared,
                                                                                       const float* __restrict__ sgate, const float* __restrict__ w,
                                                                                       int width, int top, float eps) {
    __shared__ float red[4];
    extern __shared__ int csm[];
    int* sp = csm;                                      // [top] rows of the token's pairs
    float* sw = reinterpret_cast<float*>(csm + top);    // [top] their weights
    const int t = blockIdx.x;
    for (int j = threadIdx.x; j < top; j += blockDim.x) { sp[j] = pos[(size_t)t * top + j]; sw[j] = wts[(size_t)t * top + j]; }
    __syncthreads();
    constexpr int E = VEC ? 4 : 1, U = 16 / E;
    float y[16];
    float ss = 0.f;
    const float sg = shared ? (sgate ? sgate[t] : 1.f) : 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int i = (threadIdx.x + 256 * u) * E;
        float a[E];
#pragma unroll
        for (int e = 0; e < E; ++e) a[e] = 0.f;
        if (i < width) {
            for (int j = 0; j < top; ++j) {
                const float* r = rows + (size_t)sp[j] * width + i;
                if (VEC) { const float4 v = *reinterpret_cast<const float4*>(r); a[0] = fmaf(sw[j], v.x, a[0]); a[E > 1 ? 1 : 0] = fmaf(sw[j], v.y, a[E > 1 ? 1 : 0]);
                           a[E > 1 ? 2 : 0] = fmaf(sw[j], v.z, a[E > 1 ? 2 : 0]); a[E > 1 ? 3 : 0] = fmaf(sw[j], v.w, a[E > 1 ? 3 : 0]); }
                else a[0] = fmaf(sw[j], r[0], a[0]);
            }
            if (shared)
#pragma unroll
                for (int e = 0; e < E; ++e) a[e] = fmaf(sg, shared[(size_t)t * width + i + e], a[e]);
        }
#pragma unroll
        for (int e = 0; e < E; ++e) { y[u * E + e] = a[e]; ss += a[e] * a[e]; }
    }
    ss = block_sum(ss, red);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int i = (threadIdx.x + 256 * u) * E;
        if (i >= width) continue;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float v = x[(size_t)t * width + i + e] + y[u * E + e] * inv * w[i + e];
            x[(size_t)t * width + i + e] = v;
            if (xcopy) xcopy[(size_t)t * width + i + e] = f32_to_bf16(v);
        }
    }
}
__global__ void scale_f32_kernel(float* x, float s, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] *= s;
}

int g_attn_wider = 1;           // A/B: twelve waves per (token, head) for the smallest decoding batches
int g_attn_group = 1;           // 0: grouped-query prompt steps take the kernel with one wave per head (A/B, tests of both paths)
int g_attn_mfma = 1;            // mi355_hyb_set_attention_mfma(0): prompt steps take the generic kernel too (A/B, tests of both paths)


}  // namespace

extern "C" {

// sequence index of every token row (device helper of the host layer and of the standalone entry points)
int mi355_hyb_token_seq(int32_t* tok_seq, const uint32_t* cu_seqlens_q, int32_t num_seqs, int64_t stream) {
    if (num_seqs <= 0) return 0;
    token_seq_kernel<<<num_seqs, 64, 0, to_stream(stream)>>>(tok_seq, cu_seqlens_q, num_seqs);
    LAUNCH_OK(); return 0;
}
void mi355_hyb_set_attention_mfma(int32_t on) { g_attn_mfma = on ? 1 : 0; g_attn_group = on == 2 ? 0 : 1; g_attn_wider = on == 3 ? 0 : 1; }
int mi355_hyb_bf16_to_f32(float* out, const uint16_t* in, int64_t n, int64_t stream) {
    if (n <= 0) return 0;
    bf16_to_f32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, to_stream(stream)>>>(out, in, n);
    LAUNCH_OK(); return 0;
}
int mi355_hyb_copy_f32(float* out, const float* in, int64_t n, int64_t stream) {
    if (n <= 0) return 0;
    copy_f32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, to_stream(stream)>>>(out, in, n);
    LAUNCH_OK(); return 0;
}
int mi355_hyb_fill_f32(float* out, float v, int64_t n, int64_t stream) {
    if (n <= 0) return 0;
    fill_f32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, to_stream(stream)>>>(out, v, n);
    LAUNCH_OK(); return 0;
}

static int linear_launch(float* out, int32_t ldo, int64_t o_bs, const void* a, int32_t a_dtype, int32_t lda, int64_t a_bs, const void* w,
                         int64_t w_bs, const float* bias, int32_t T, int32_t n, int32_t k, int32_t batch, int32_t dtype, int64_t stream) {
    if (!out || !a || !w || T < 0 || n <= 0 || k <= 0 || ldo < n || lda < k || batch <= 0 || batch > 65535 || !is_dt(dtype) || !is_dt(a_dtype)) return -1;
    if (T == 0) return 0;
    LinArgs p{out, ldo, a, lda, w, bias, T, n, k, 0, 0, a_bs, w_bs, o_bs};
    hipStream_t st_ = to_stream(stream);
    const unsigned nz = (unsigned)batch;
    if (dtype == MI355_DTYPE_F32) {
        if (a_dtype != MI355_DTYPE_F32) return -1;
        linear_f32_kernel<<<dim3((n + 63) / 64, (T + 63) / 64, nz), 256, 0, st_>>>(p);
        LAUNCH_OK(); return 0;
    }
    const int a_bytes = a_dtype == MI355_DTYPE_F32 ? 4 : 2;
    p.w_vec = (k % 8 == 0) && ((uintptr_t)w % 16 == 0) && (w_bs % 8 == 0);
    p.a_vec = ((size_t)lda * a_bytes % 16 == 0) && ((uintptr_t)a % 16 == 0) && ((size_t)a_bs * a_bytes % 16 == 0);
    const bool af = a_dtype == MI355_DTYPE_F32;
    if (T <= 16) {
        const dim3 grid((n + 15) / 16, 1, nz);
        if (k >= 2048) { if (af) linear_bf16_stream_kernel<float, 4, 4><<<grid, 256, 0, st_>>>(p); else linear_bf16_stream_kernel<uint16_t, 4, 4><<<grid, 256, 0, st_>>>(p); }
        else { if (af) linear_bf16_stream_kernel<float, 2, 2><<<grid, 128, 0, st_>>>(p); else linear_bf16_stream_kernel<uint16_t, 2, 2><<<grid, 128, 0, st_>>>(p); }
    } else if (T > 32 && !af && p.a_vec && p.w_vec && k % 32 == 0) {
        linear_bf16_lds_kernel<<<dim3((n + 127) / 128, (T + 127) / 128, nz), 256, 0, st_>>>(p);
    } else if (T <= 32) {
        const dim3 grid((n + 63) / 64, (T + 31) / 32, nz);
        if (af) linear_bf16_tile_kernel<float, 2><<<grid, 256, 0, st_>>>(p); else linear_bf16_tile_kernel<uint16_t, 2><<<grid, 256, 0, st_>>>(p);
    } else {
        const dim3 grid((n + 63) / 64, (T + 63) / 64, nz);
        if (af) linear_bf16_tile_kernel<float, 4><<<grid, 256, 0, st_>>>(p); else linear_bf16_tile_kernel<uint16_t, 4><<<grid, 256, 0, st_>>>(p);
    }
    LAUNCH_OK(); return 0;
}

int mi355_hyb_linear(float* out, int32_t ldo, const void* a, int32_t a_dtype, int32_t lda, const void* w, const float* bias,
                     int32_t T, int32_t n, int32_t k, int32_t dtype, int64_t stream) {
    return linear_launch(out, ldo, 0, a, a_dtype, lda, 0, w, 0, bias, T, n, k, 1, dtype, stream);
}
int mi355_hyb_linear_batched(float* out, int32_t ldo, int64_t o_bs, const void* a, int32_t a_dtype, int32_t lda, int64_t a_bs,
                             const void* w, int64_t w_bs, int32_t T, int32_t n, int32_t k, int32_t batch, int32_t dtype, int64_t stream) {
    if (o_bs < 0 || a_bs < 0 || w_bs < 0) return -1;
    return linear_launch(out, ldo, o_bs, a, a_dtype, lda, a_bs, w, w_bs, nullptr, T, n, k, batch, dtype, stream);
}

int mi355_hyb_embed(float* x, void* xcopy, const void* table, const uint32_t* ids, int32_t T, int32_t width, int32_t vocab, int32_t dtype,
                    int64_t stream) {
    if (!x || !table || !ids || !is_dt(dtype) || width <= 0) return -1;
    if (T <= 0) return 0;
    if (dtype == MI355_DTYPE_F32) embed_kernel<float><<<T, 256, 0, to_stream(stream)>>>(x, (uint16_t*)xcopy, (const float*)table, ids, width, vocab);
    else embed_kernel<uint16_t><<<T, 256, 0, to_stream(stream)>>>(x, (uint16_t*)xcopy, (const uint16_t*)table, ids, width, vocab);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_norm_add(float* x, void* xcopy, const float* y, int32_t ldy, const float* w, int32_t T, int32_t width, float eps,
                       int64_t stream) {
    if (!x || !y || !w || width <= 0 || ldy < width) return -1;
    if (T <= 0) return 0;
    norm_add_kernel<<<T, 256, 0, to_stream(stream)>>>(x, (uint16_t*)xcopy, y, ldy, w, width, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_gather_norm(void* out, int32_t out_dtype, const float* x, const int32_t* rows, const float* w, int32_t n_rows, int32_t width,
                          float eps, int64_t stream) {
    if (!out || !x || !rows || !w || !is_dt(out_dtype)) return -1;
    if (n_rows <= 0) return 0;
    if (out_dtype == MI355_DTYPE_F32) gather_norm_kernel<float><<<n_rows, 256, 0, to_stream(stream)>>>((float*)out, x, rows, w, width, eps);
    else gather_norm_kernel<uint16_t><<<n_rows, 256, 0, to_stream(stream)>>>((uint16_t*)out, x, rows, w, width, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_clamped_glu(void* out, int32_t out_dtype, const float* gu, int32_t T, int32_t ff, float limit, float alpha, int64_t stream) {
    if (!out || !gu || ff <= 0 || !is_dt(out_dtype)) return -1;
    const int64_t n = (int64_t)T * ff;
    if (n <= 0) return 0;
    const unsigned grid = (unsigned)((n + 255) / 256);
    if (out_dtype == MI355_DTYPE_F32) clamped_glu_kernel<float><<<grid, 256, 0, to_stream(stream)>>>((float*)out, gu, n, ff, limit, alpha);
    else clamped_glu_kernel<uint16_t><<<grid, 256, 0, to_stream(stream)>>>((uint16_t*)out, gu, n, ff, limit, alpha);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_attn_prepare(void* q_out, void* k_pages, void* v_pages, const float* proj, int32_t ldp, int32_t q_off, int32_t k_off,
                           int32_t v_off, const float* q_norm_w, const float* k_norm_w, const float* cos_t, const float* sin_t,
                           const int64_t* positions, const int64_t* slot_mapping, int32_t T, int32_t heads, int32_t kv_heads,
                           int32_t dim, int32_t vdim, int32_t rot_dims, float eps, int32_t dtype, int64_t stream) {
    // (the plain form: a norm only where weights are given, before the rotation; rotate-half pairs)
    return mi355_hyb_attn_prepare_ex(q_out, k_pages, v_pages, proj, ldp, q_off, k_off, v_off, q_norm_w, k_norm_w, cos_t, sin_t, positions,
                                     slot_mapping, T, heads, kv_heads, dim, vdim, rot_dims, 0, (q_norm_w || k_norm_w) ? 1 : 0, nullptr, eps,
                                     dtype, stream);
}

int mi355_hyb_attn_prepare_ex(void* q_out, void* k_pages, void* v_pages, const float* proj, int32_t ldp, int32_t q_off, int32_t k_off,
                              int32_t v_off, const float* q_norm_w, const float* k_norm_w, const float* cos_t, const float* sin_t,
                              const int64_t* positions, const int64_t* slot_mapping, int32_t T, int32_t heads, int32_t kv_heads,
                              int32_t dim, int32_t vdim, int32_t rot_dims, int32_t interleaved, int32_t norm_mode,
                              const float* q_head_scale, float eps, int32_t dtype, int64_t stream) {
    if (norm_mode < 0 || norm_mode > 2) return -1;
    if (!q_out || !k_pages || !v_pages || !proj || !positions || !slot_mapping || !is_dt(dtype)) return -1;
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0 || rot_dims < 0 || rot_dims > dim || (rot_dims & 1)) return -1;
    if (rot_dims > 0 && (!cos_t || !sin_t)) return -1;
    if (T <= 0) return 0;
    PrepArgs p{q_out, k_pages, v_pages, proj, ldp, q_off, k_off, v_off, q_norm_w, k_norm_w, cos_t, sin_t, positions, slot_mapping,
               heads, kv_heads, dim, vdim, rot_dims, eps, interleaved, norm_mode, q_head_scale};
    const dim3 grid(T, heads + 2 * kv_heads);
    if (dtype == MI355_DTYPE_F32) attn_prepare_kernel<float><<<grid, 64, 2 * dim * sizeof(float), to_stream(stream)>>>(p);
    else attn_prepare_kernel<uint16_t><<<grid, 64, 2 * dim * sizeof(float), to_stream(stream)>>>(p);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_window_attention(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const void* q, const void* k_pages,
                                   const void* v_pages, const uint32_t* block_tables, const uint32_t* context_lens,
                                   const uint32_t* cu_seqlens_q, const int32_t* tok_seq, const float* sink, int32_t num_seqs,
                                   int32_t T, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, int32_t block_size,
                                   int32_t max_blocks, int32_t window, float scale, float out_scale, int32_t dtype, int64_t stream) {
    return mi355_hyb_window_attention_ex(out, out_dtype, ldo, out_off, q, k_pages, v_pages, block_tables, context_lens, cu_seqlens_q, tok_seq,
                                         sink, num_seqs, T, heads, kv_heads, dim, vdim, block_size, max_blocks, window, scale, out_scale,
                                         0, 0, 0.f, 0, dtype, stream);
}

int mi355_hyb_window_attention_ex(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const void* q, const void* k_pages,
                                   const void* v_pages, const uint32_t* block_tables, const uint32_t* context_lens,
                                   const uint32_t* cu_seqlens_q, const int32_t* tok_seq, const float* sink, int32_t num_seqs,
                                   int32_t T, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, int32_t block_size,
                                   int32_t max_blocks, int32_t window, float scale, float out_scale, int32_t k_ld, int32_t v_ld,
                                   float softcap, int32_t cross_values, int32_t dtype, int64_t stream) {
    return mi355_hyb_masked_attention(out, out_dtype, ldo, out_off, q, k_pages, v_pages, block_tables, context_lens, cu_seqlens_q, tok_seq,
                                      sink, num_seqs, T, heads, kv_heads, dim, vdim, block_size, max_blocks, window, 0, scale, out_scale,
                                      k_ld, v_ld, softcap, cross_values, dtype, stream);
}

int mi355_hyb_masked_attention(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const void* q, const void* k_pages,
                               const void* v_pages, const uint32_t* block_tables, const uint32_t* context_lens,
                               const uint32_t* cu_seqlens_q, const int32_t* tok_seq, const float* sink, int32_t num_seqs,
                               int32_t T, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, int32_t block_size,
                               int32_t max_blocks, int32_t window, int32_t keep_first, float scale, float out_scale, int32_t k_ld,
                               int32_t v_ld, float softcap, int32_t cross_values, int32_t dtype, int64_t stream) {
    return mi355_hyb_biased_attention(out, out_dtype, ldo, out_off, q, k_pages, v_pages, block_tables, context_lens, cu_seqlens_q, tok_seq, sink,
                                      nullptr, num_seqs, T, heads, kv_heads, dim, vdim, block_size, max_blocks, window, keep_first, scale,
                                      out_scale, k_ld, v_ld, softcap, cross_values, dtype, stream);
}

int mi355_hyb_biased_attention(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const void* q, const void* k_pages,
                               const void* v_pages, const uint32_t* block_tables, const uint32_t* context_lens,
                               const uint32_t* cu_seqlens_q, const int32_t* tok_seq, const float* sink, const float* dist,
                               int32_t num_seqs, int32_t T, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim,
                               int32_t block_size, int32_t max_blocks, int32_t window, int32_t keep_first, float scale, float out_scale,
                               int32_t k_ld, int32_t v_ld, float softcap, int32_t cross_values, int32_t dtype, int64_t stream) {
    if (keep_first < 0) return -1;
    if (!out || !q || !k_pages || !v_pages || !block_tables || !context_lens || !cu_seqlens_q || !tok_seq) return -1;
    if (!is_dt(dtype) || !is_dt(out_dtype) || heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0) return -1;
    if (block_size <= 0 || max_blocks <= 0 || window < 0 || softcap < 0.f) return -1;
    if (k_ld == 0) k_ld = kv_heads * dim;
    if (v_ld == 0) v_ld = kv_heads * vdim;
    if (k_ld < kv_heads * dim || v_ld < kv_heads * vdim) return -1;
    if (T <= 0) return 0;
    const bool f = dtype == MI355_DTYPE_F32;
    const int cross = cross_values ? 1 : 0, nz = cross ? kv_heads : 1;
    AttnArgs p{out, ldo, out_off, q, k_pages, v_pages, block_tables, context_lens, cu_seqlens_q, tok_seq, sink,
               num_seqs, heads, kv_heads, dim, vdim, block_size, max_blocks, window, scale, out_scale, 64, out_dtype == MI355_DTYPE_F32,
               k_ld, v_ld, softcap, cross};
    hipStream_t s_ = to_stream(stream);
    const int epv = f ? 4 : 8;
    const bool vec = dim % epv == 0 && vdim % epv == 0 && vdim / epv <= 64 && dim / epv <= 64 && (uintptr_t)k_pages % 16 == 0 && (uintptr_t)v_pages % 16 == 0 &&
                     k_ld % epv == 0 && v_ld % epv == 0;
    p.cpk = 64;
    p.keep = window > 0 ? keep_first : 0;
    p.dist = dist;
    if (vec) { int c = 1; while (c < vdim / epv) c <<= 1; p.cp2 = c; c = 1; while (c < dim / epv) c <<= 1; p.cpk = c; }
    else if (vdim > 512) return -1;
    // prompt-sized steps over bf16 pages: the matrix-core kernel (a tile of 16 tokens never spans two sequences)
    if (!f && T >= 64 && dim % 32 == 0 && dim <= 256 && vdim % 16 == 0 && vdim <= 256 && (uintptr_t)q % 16 == 0 && (uintptr_t)k_pages % 16 == 0 &&
        (uintptr_t)v_pages % 16 == 0 && k_ld % 8 == 0 && v_ld % 8 == 0 && g_attn_mfma) {
        const int dk = dim / 32, vt = vdim / 16;
        // grouped-query attention: the query heads of a key/value head share a workgroup and its staged rows
        const int hpk = heads / kv_heads, hpg = cross ? 1 : (hpk % 4 == 0 ? 4 : hpk % 3 == 0 ? 3 : hpk % 2 == 0 ? 2 : 1);
        if (hpg > 1 && dk <= 4 && vt <= 8 && vt % 2 == 0 && g_attn_group) {
            const dim3 ggrid((T + 15) / 16 + num_seqs, heads / hpg, 1);
#define WG2(DK, VT) do { if (hpg == 4) window_attention_group_kernel<DK, VT, 4><<<ggrid, 256, 0, s_>>>(p); \
                         else if (hpg == 3) window_attention_group_kernel<DK, VT, 3><<<ggrid, 192, 0, s_>>>(p); \
                         else window_attention_group_kernel<DK, VT, 2><<<ggrid, 128, 0, s_>>>(p); } while (0)
#define WGV(DK) do { switch (vt) { case 2: WG2(DK, 2); break; case 4: WG2(DK, 4); break; case 6: WG2(DK, 6); break; default: WG2(DK, 8); break; } } while (0)
            switch (dk) { case 1: WGV(1); break; case 2: WGV(2); break; case 3: WGV(3); break; default: WGV(4); break; }
#undef WGV
#undef WG2
            LAUNCH_OK(); return 0;
        }
        // cross mode: 2 value heads per block where the head sizes have such a build (dim <= 128, vdim <= 128), the rest of the
        // key/value heads along z (4 per block: one wave per SIMD, measured 1.4 x slower)
        const int nv = (cross && dk <= 4 && vt <= 8) ? (kv_heads % 2 == 0 ? 2 : 1) : 1;
        const dim3 mgrid((T + 15) / 16 + num_seqs, heads, nz / nv);
#define WM1(DK, VT) window_attention_mfma_kernel<DK, VT, 1><<<mgrid, 64, 0, s_>>>(p)
#define WMN(DK, VT) do { if (nv == 2) window_attention_mfma_kernel<DK, VT, 2><<<mgrid, 64, 0, s_>>>(p); else WM1(DK, VT); } while (0)
#define WMV(DK, WM) do { switch (vt) { case 1: WM(DK, 1); break; case 2: WM(DK, 2); break; case 3: WM(DK, 3); break; case 4: WM(DK, 4); break; \
                                        case 5: WM(DK, 5); break; case 6: WM(DK, 6); break; case 7: WM(DK, 7); break; case 8: WM(DK, 8); break; \
                                        default: ok_shape = false; } } while (0)
        // value rows wider than 128 (latent attention: the latent itself is the value row): 16-column steps up to 256
#define WMW(DK) do { switch (vt) { case 10: WM1(DK, 10); break; case 12: WM1(DK, 12); break; case 14: WM1(DK, 14); break; case 16: WM1(DK, 16); break; \
                                   default: ok_shape = false; } } while (0)
        bool ok_shape = true;
        if (vt > 8) {
            switch (dk) { case 4: WMW(4); break; case 5: WMW(5); break; case 6: WMW(6); break; case 7: WMW(7); break; case 8: WMW(8); break;
                          default: ok_shape = false; }
        } else {
            switch (dk) { case 1: WMV(1, WMN); break; case 2: WMV(2, WMN); break; case 3: WMV(3, WMN); break; case 4: WMV(4, WMN); break;
                          case 6: WMV(6, WM1); break; case 8: WMV(8, WM1); break; default: ok_shape = false; }
        }
#undef WMW
#undef WMV
#undef WMN
#undef WM1
        if (ok_shape) { LAUNCH_OK(); return 0; }
    }
    // few (token, head) pairs (decoding batches): eight waves share a window instead of four
    const bool wide = (int64_t)T * heads < 2048;
    // a handful of sequences: twelve waves (a window of a thousand keys plus kept tokens is two rounds of 64-key chunks instead of three)
    const bool wider = (int64_t)T * heads <= 256 && g_attn_wider;
    // cross mode with 16-byte rows: 4 or 2 value heads per workgroup, the rest of the key/value heads along z
    int nv = (cross && vec) ? (kv_heads % 4 == 0 ? 4 : kv_heads % 2 == 0 ? 2 : 1) : 1;
    if ((size_t)(wider ? 12 : 8) * nv * vdim * sizeof(float) > 32768) nv = 1;          // the waves' partial sums must fit the workgroup's LDS
    while (nv > 1 && (int64_t)T * heads * (nz / nv) < 512) nv >>= 1;    // decoding batches: rather more workgroups than shared scores
    const dim3 ggrid(T, heads, nz / nv);
#define WA4(TC, NW, VEC, DQ, NV) window_attention_kernel<TC, NW, VEC, DQ, NV><<<ggrid, 64 * NW, (size_t)(((dim + 3) & ~3) + 2 * NW + NW * NV * vdim) * sizeof(float), s_>>>(p)
#define WA3(TC, NW, VEC, DQ) do { if (nv == 4) WA4(TC, NW, VEC, DQ, 4); else if (nv == 2) WA4(TC, NW, VEC, DQ, 2); else WA4(TC, NW, VEC, DQ, 1); } while (0)
#define WA2(TC, NW) do { if (!vec) WA4(TC, NW, false, 0, 1); else WA3(TC, NW, true, 0); } while (0)
#define WA(TC) do { if (wider) WA2(TC, 12); else if (wide) WA2(TC, 8); else WA2(TC, 4); } while (0)
    if (f) WA(float); else WA(uint16_t);
#undef WA
#undef WA2
#undef WA3
#undef WA4
    LAUNCH_OK(); return 0;
}

int mi355_hyb_conv_silu(float* out, const float* proj, int32_t ldp, int32_t off, const float* w, const float* conv_state,
                            int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                            const int32_t* state_slots, const int32_t* tok_seq, int32_t num_seqs, int32_t T, int32_t channels,
                            int32_t taps, int64_t stream) {
    return mi355_hyb_conv(out, proj, ldp, off, w, conv_state, state_stride, context_lens, cu_seqlens_q, state_slots, tok_seq, num_seqs, T,
                          channels, taps, 1, stream);
}

int mi355_hyb_conv(float* out, const float* proj, int32_t ldp, int32_t off, const float* w, const float* conv_state,
                   int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                   const int32_t* tok_seq, int32_t num_seqs, int32_t T, int32_t channels, int32_t taps, int32_t act, int64_t stream) {
    return mi355_hyb_conv_bias(out, proj, ldp, off, w, nullptr, conv_state, state_stride, context_lens, cu_seqlens_q, state_slots, tok_seq,
                               num_seqs, T, channels, taps, act, stream);
}
int mi355_hyb_conv_bias(float* out, const float* proj, int32_t ldp, int32_t off, const float* w, const float* bias, const float* conv_state,
                        int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                        const int32_t* tok_seq, int32_t num_seqs, int32_t T, int32_t channels, int32_t taps, int32_t act, int64_t stream) {
    if (act != 0 && act != 1) return -1;
    if (!out || !proj || !w || !conv_state || !context_lens || !cu_seqlens_q || !state_slots || !tok_seq) return -1;
    if (channels <= 0 || taps < 1 || taps > 16) return -1;
    if (T <= 0) return 0;
    ConvArgs p{out, proj, ldp, off, w, const_cast<float*>(conv_state), state_stride, context_lens, cu_seqlens_q, state_slots, tok_seq, channels, taps, T, act, 0, nullptr, bias};
    const int64_t n = (int64_t)T * channels;
    conv_silu_kernel<<<(unsigned)((n + 255) / 256), 256, 0, to_stream(stream)>>>(p);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_conv_residual(void* out, int32_t out_dtype, const float* in, int32_t ld, int32_t off, const float* w, const float* conv_state,
                            int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                            const int32_t* tok_seq, int32_t num_seqs, int32_t T, int32_t channels, int32_t taps, int64_t stream) {
    if (!out || !in || !w || !conv_state || !context_lens || !cu_seqlens_q || !state_slots || !tok_seq || !is_dt(out_dtype)) return -1;
    if (channels <= 0 || taps < 1 || taps > 16 || ld < off + channels) return -1;
    if (T <= 0) return 0;
    const bool f = out_dtype == MI355_DTYPE_F32;
    ConvArgs p{f ? (float*)out : nullptr, in, ld, off, w, const_cast<float*>(conv_state), state_stride, context_lens, cu_seqlens_q, state_slots,
               tok_seq, channels, taps, T, 0, 1, f ? nullptr : (uint16_t*)out};
    const int64_t n = (int64_t)T * channels;
    conv_silu_kernel<<<(unsigned)((n + 255) / 256), 256, 0, to_stream(stream)>>>(p);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_conv_state_update(float* conv_state, int64_t state_stride, const float* proj, int32_t ldp, int32_t off,
                                const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                                int32_t num_seqs, int32_t channels, int32_t taps, int64_t stream) {
    if (!conv_state || !proj || !context_lens || !cu_seqlens_q || !state_slots || channels <= 0 || taps < 1 || taps > 16) return -1;
    if (num_seqs <= 0 || taps == 1) return 0;
    ConvArgs p{nullptr, proj, ldp, off, nullptr, conv_state, state_stride, context_lens, cu_seqlens_q, state_slots, nullptr, channels, taps, 0, 0, 0, nullptr};
    const int n = num_seqs * channels;
    conv_state_update_kernel<<<(n + 255) / 256, 256, 0, to_stream(stream)>>>(p, num_seqs);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_delta_rule_scratch_floats(int32_t num_tokens, int32_t heads, int32_t kv_heads, int32_t dim, int32_t decay_channels) {
    return num_tokens * (2 * kv_heads * dim + heads * (decay_channels ? dim : 1) + heads);
}

int mi355_hyb_delta_rule(float* o, float* state, int64_t state_stride, const float* qkv, int32_t ldq, const float* proj, int32_t ldp,
                         int32_t b_off, const float* decay_in, int32_t ldd, int32_t decay_channels, const float* a_log,
                         const float* dt_bias, const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                         int32_t num_seqs, int32_t num_tokens, int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, float unit_eps,
                         float* scratch, int64_t stream) {
    if (!o || !state || !qkv || !proj || !decay_in || !a_log || !dt_bias || !context_lens || !cu_seqlens_q || !state_slots || !scratch) return -1;
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || dim > 256 || vdim <= 0) return -1;
    if (num_seqs <= 0 || num_tokens <= 0) return 0;
    DeltaArgs p{o, state, state_stride, qkv, ldq, proj, ldp, b_off, decay_in, ldd, decay_channels, a_log, dt_bias,
                context_lens, cu_seqlens_q, state_slots, heads, kv_heads, dim, vdim, unit_eps};
    hipStream_t s_ = to_stream(stream);
    const int P = 2 * kv_heads * dim + heads * (decay_channels ? dim : 1) + heads;
    delta_prep_kernel<<<dim3(num_tokens, heads), 64, 0, s_>>>(p, scratch, P, num_tokens);
    LAUNCH_OK();
    if (dim < 64) {
        const dim3 grid(num_seqs, heads, (vdim + 63) / 64);
        if (dim <= 16) delta_scan_kernel<4, 4, 8><<<grid, 256, 0, s_>>>(p, scratch, P);
        else if (dim <= 32) delta_scan_kernel<8, 4, 8><<<grid, 256, 0, s_>>>(p, scratch, P);
        else delta_scan_kernel<16, 4, 8><<<grid, 256, 0, s_>>>(p, scratch, P);
    } else {
        const dim3 grid(num_seqs, heads, (vdim + 15) / 16);
        if (dim <= 64) delta_scan_kernel<4, 16, 8><<<grid, 256, 0, s_>>>(p, scratch, P);
        else if (dim <= 128) delta_scan_kernel<8, 16, 8><<<grid, 256, 0, s_>>>(p, scratch, P);
        else delta_scan_kernel<16, 16, 8><<<grid, 256, 0, s_>>>(p, scratch, P);
    }
    LAUNCH_OK(); return 0;
}

int mi355_hyb_gated_norm(void* out, int32_t out_dtype, int32_t ldo, int32_t out_off, const float* o, const float* w,
                         const float* gate_in, int32_t ldg, int32_t gate, int32_t T, int32_t heads, int32_t vdim, float eps,
                         float out_scale, int64_t stream) {
    if (!out || !o || !w || !gate_in || !is_dt(out_dtype) || heads <= 0 || vdim <= 0) return -1;
    if (T <= 0) return 0;
    const dim3 grid(T, heads);
    if (out_dtype == MI355_DTYPE_F32) gated_norm_kernel<float><<<grid, 64, 0, to_stream(stream)>>>((float*)out, ldo, out_off, o, w, gate_in, ldg, gate, heads, vdim, eps, out_scale);
    else gated_norm_kernel<uint16_t><<<grid, 64, 0, to_stream(stream)>>>((uint16_t*)out, ldo, out_off, o, w, gate_in, ldg, gate, heads, vdim, eps, out_scale);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_mingru(void* out, int32_t out_dtype, float* state, int64_t state_stride, const float* proj, int32_t ldp, int32_t z_off,
                     int32_t x_off, int32_t g_off, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                     const int32_t* state_slots, int32_t num_seqs, int32_t num_tokens, int32_t width, int64_t stream) {
    if (!out || !state || !proj || !context_lens || !cu_seqlens_q || !state_slots || !is_dt(out_dtype) || width <= 0) return -1;
    if (num_seqs <= 0) return 0;
    GruArgs p{out, state, state_stride, proj, ldp, z_off, x_off, g_off, context_lens, cu_seqlens_q, state_slots, width};
    const dim3 grid((width + 63) / 64, num_seqs);
    if (num_tokens >= 256) {                            // some portion may be long: segmented scan
        if (out_dtype == MI355_DTYPE_F32) mingru_seg_kernel<float, 16, 4><<<grid, 1024, 0, to_stream(stream)>>>(p);
        else mingru_seg_kernel<uint16_t, 16, 4><<<grid, 1024, 0, to_stream(stream)>>>(p);
        LAUNCH_OK(); return 0;
    }
    if (out_dtype == MI355_DTYPE_F32) mingru_kernel<float, 8><<<grid, 64, 0, to_stream(stream)>>>(p);
    else mingru_kernel<uint16_t, 8><<<grid, 64, 0, to_stream(stream)>>>(p);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_resid_norm(float* x, void* xcopy, const float* y, int32_t ldy, const float* w, int32_t T, int32_t width, int32_t groups,
                         float alpha, float eps, int64_t stream) {
    if (groups <= 0) groups = 1;
    if (!x || !y || !w || width <= 0 || ldy < width || width % groups) return -1;
    if (T <= 0) return 0;
    resid_norm_kernel<<<T, 256, 0, to_stream(stream)>>>(x, (uint16_t*)xcopy, y, ldy, w, width, groups, alpha, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_gather_group_norm(void* out, int32_t out_dtype, const float* x, const int32_t* rows, const float* w, int32_t n_rows,
                                int32_t width, int32_t groups, float eps, int64_t stream) {
    if (groups <= 0) groups = 1;
    if (!out || !x || !rows || !w || !is_dt(out_dtype) || width <= 0 || width % groups) return -1;
    if (n_rows <= 0) return 0;
    if (out_dtype == MI355_DTYPE_F32) gather_group_norm_kernel<float><<<n_rows, 256, 0, to_stream(stream)>>>((float*)out, x, rows, w, width, groups, eps);
    else gather_group_norm_kernel<uint16_t><<<n_rows, 256, 0, to_stream(stream)>>>((uint16_t*)out, x, rows, w, width, groups, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_gelu_glu(void* out, int32_t out_dtype, const float* gu, int32_t T, int32_t ff, int64_t stream) {
    if (!out || !gu || ff <= 0 || !is_dt(out_dtype)) return -1;
    const int64_t n = (int64_t)T * ff;
    if (n <= 0) return 0;
    const unsigned grid = (unsigned)((n + 255) / 256);
    if (out_dtype == MI355_DTYPE_F32) gelu_glu_kernel<float><<<grid, 256, 0, to_stream(stream)>>>((float*)out, gu, n, ff);
    else gelu_glu_kernel<uint16_t><<<grid, 256, 0, to_stream(stream)>>>((uint16_t*)out, gu, n, ff);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_attn_prepare_whole(void* q_out, void* k_pages, void* v_pages, const float* src, int32_t ld, int32_t q_off, int32_t k_off,
                                 int32_t v_off, const float* q_norm_w, const float* k_norm_w, const int64_t* slot_mapping, int32_t T,
                                 int32_t heads, int32_t kv_heads, int32_t dim, int32_t vdim, int32_t v_unit, float eps, int32_t dtype,
                                 int64_t stream) {
    if (!q_out || !k_pages || !v_pages || !src || !slot_mapping || !is_dt(dtype)) return -1;
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0) return -1;
    if (T <= 0) return 0;
    WholePrepArgs p{q_out, k_pages, v_pages, src, ld, q_off, k_off, v_off, q_norm_w, k_norm_w, slot_mapping, heads, kv_heads, dim, vdim,
                    v_unit ? 1 : 0, eps};
    if (dtype == MI355_DTYPE_F32) attn_prepare_whole_kernel<float><<<T, 256, 0, to_stream(stream)>>>(p);
    else attn_prepare_whole_kernel<uint16_t><<<T, 256, 0, to_stream(stream)>>>(p);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_latent_prepare(void* q_out, void* pages, const float* proj, int32_t ldp, int32_t q_off, int32_t c_off, const float* q_abs,
                             const float* c_norm_w, const float* cos_t, const float* sin_t, const int64_t* positions,
                             const int64_t* slot_mapping, int32_t T, int32_t heads, int32_t dim, int32_t rot_dim, int32_t kv_rank,
                             int32_t rot_dims, int32_t interleaved, float eps, int32_t dtype, int64_t stream) {
    if (!pages) return -1;
    return mi355_hyb_latent_prepare_ex(q_out, pages, proj, ldp, q_off, proj, ldp, c_off, q_abs, c_norm_w, cos_t, sin_t, positions, slot_mapping, T,
                                       heads, dim, rot_dim, kv_rank, rot_dims, interleaved, eps, dtype, stream);
}
int mi355_hyb_latent_prepare_ex(void* q_out, void* pages, const float* q_src, int32_t ldq, int32_t q_off, const float* c_src, int32_t ldc,
                                int32_t c_off, const float* q_abs, const float* c_norm_w, const float* cos_t, const float* sin_t,
                                const int64_t* positions, const int64_t* slot_mapping, int32_t T, int32_t heads, int32_t dim,
                                int32_t rot_dim, int32_t kv_rank, int32_t rot_dims, int32_t interleaved, float eps, int32_t dtype,
                                int64_t stream) {
    if (!q_out || !q_src || !q_abs || !positions || !slot_mapping || !is_dt(dtype) || (pages && (!c_src || !c_norm_w))) return -1;
    if (heads <= 0 || dim <= 0 || rot_dim < 0 || kv_rank <= 0 || rot_dims < 0 || rot_dims > rot_dim || (rot_dims & 1)) return -1;
    if (rot_dims > 0 && (!cos_t || !sin_t)) return -1;
    if (T <= 0) return 0;
    LatentPrepArgs p{q_out, pages, q_src, ldq, q_off, c_src, ldc, c_off, q_abs, c_norm_w, cos_t, sin_t, positions, slot_mapping,
                     heads, dim, rot_dim, kv_rank, rot_dims, interleaved ? 1 : 0, eps};
    if (dtype == MI355_DTYPE_F32) latent_prepare_kernel<float><<<T, 256, 0, to_stream(stream)>>>(p);
    else latent_prepare_kernel<uint16_t><<<T, 256, 0, to_stream(stream)>>>(p);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_head_mix(void* out, int32_t out_dtype, const float* a, const float* talk, int32_t T, int32_t heads, int32_t kv_heads,
                       int32_t vdim, int64_t stream) {
    if (!out || !a || !talk || !is_dt(out_dtype) || heads <= 0 || kv_heads <= 0 || heads % kv_heads || vdim <= 0) return -1;
    const int64_t n = (int64_t)T * heads * vdim;
    if (n <= 0) return 0;
    const unsigned grid = (unsigned)((n + 255) / 256);
    if (out_dtype == MI355_DTYPE_F32) head_mix_kernel<float><<<grid, 256, 0, to_stream(stream)>>>((float*)out, a, talk, n, heads, kv_heads, vdim);
    else head_mix_kernel<uint16_t><<<grid, 256, 0, to_stream(stream)>>>((uint16_t*)out, a, talk, n, heads, kv_heads, vdim);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_head_gate(void* out, int32_t out_dtype, const float* in, const float* gate_in, int32_t ldg, int32_t T, int32_t heads,
                        int32_t vdim, int64_t stream) {
    if (!out || !in || !is_dt(out_dtype) || heads <= 0 || vdim <= 0 || (gate_in && ldg < heads)) return -1;
    const int64_t n = (int64_t)T * heads * vdim;
    if (n <= 0) return 0;
    const unsigned grid = (unsigned)((n + 255) / 256);
    if (out_dtype == MI355_DTYPE_F32) head_gate_kernel<float><<<grid, 256, 0, to_stream(stream)>>>((float*)out, in, gate_in, ldg, n, heads, vdim);
    else head_gate_kernel<uint16_t><<<grid, 256, 0, to_stream(stream)>>>((uint16_t*)out, in, gate_in, ldg, n, heads, vdim);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_pre_norm(void* out, int32_t out_dtype, const float* x, const float* w, int32_t T, int32_t width, float eps, int64_t stream) {
    if (!out || !x || !w || !is_dt(out_dtype) || width <= 0) return -1;
    if (T <= 0) return 0;
    if (out_dtype == MI355_DTYPE_F32) gather_norm_kernel<float><<<T, 256, 0, to_stream(stream)>>>((float*)out, x, nullptr, w, width, eps);
    else gather_norm_kernel<uint16_t><<<T, 256, 0, to_stream(stream)>>>((uint16_t*)out, x, nullptr, w, width, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_scale_f32(float* x, float s, int64_t n, int64_t stream) {
    if (!x) return -1;
    if (n <= 0) return 0;
    scale_f32_kernel<<<(unsigned)((n + 255) / 256), 256, 0, to_stream(stream)>>>(x, s, n);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_moe_route(int32_t* expert_ids, float* weights, float* shared_gate, void* xn, int32_t out_dtype, const float* x,
                        const float* norm_w, const float* router, const float* correction, const float* gate_row, int32_t T,
                        int32_t width, int32_t experts, int32_t top, float scale, float eps, int32_t append_shared, int64_t stream) {
    return mi355_hyb_moe_route_ex(expert_ids, weights, shared_gate, xn, out_dtype, x, norm_w, router, correction, gate_row, T, width, experts, top,
                                  scale, eps, append_shared, 0, 0, 0, 0, stream);
}
int mi355_hyb_moe_route_ex(int32_t* expert_ids, float* weights, float* shared_gate, void* xn, int32_t out_dtype, const float* x,
                           const float* norm_w, const float* router, const float* correction, const float* gate_row, int32_t T,
                           int32_t width, int32_t experts, int32_t top, float scale, float eps, int32_t append_shared,
                           int32_t sigmoid_scores, int32_t groups, int32_t keep_groups, int32_t normalise, int64_t stream) {
    if (groups < 0 || (groups > 0 && (experts % groups || keep_groups < 1 || keep_groups > groups || (experts / groups) * keep_groups < top))) return -1;
    if (!expert_ids || !weights || !x || !router || width <= 0 || experts < 1 || experts > 4096 || top < 1 || top > experts) return -1;
    if ((gate_row && !shared_gate && !append_shared) || (append_shared && !gate_row) || (xn && !is_dt(out_dtype))) return -1;
    if (T <= 0) return 0;
    const size_t lds = (size_t)(width + 4 * experts + 1) * sizeof(float);
    if (lds > 60000) return -1;
    // few tokens (decoding batches): sixteen waves per token, about one router row each; prompts: four
    const bool bf = xn && out_dtype == MI355_DTYPE_BF16;
#define ROUTE(TO, NW) moe_route_kernel<TO, NW><<<T, 64 * NW, lds, to_stream(stream)>>>(expert_ids, weights, shared_gate, (TO*)xn, x, norm_w, router, \
                                                                                       correction, gate_row, width, experts, top, scale, eps, append_shared ? 1 : 0, \
                                                                                       sigmoid_scores ? 1 : 0, groups, keep_groups, normalise ? 1 : 0)
    if (T <= 256) { if (bf) ROUTE(uint16_t, 16); else ROUTE(float, 16); }
    else { if (bf) ROUTE(uint16_t, 4); else ROUTE(float, 4); }
#undef ROUTE
    LAUNCH_OK(); return 0;
}

int32_t mi355_hyb_moe_block_rows(int32_t pairs, int32_t experts, int32_t n, int32_t k, int32_t dtype) {
    if (dtype == MI355_DTYPE_F32) return 64;                            // the f32 product's tile
    if (experts < 1) experts = 1;
    const int avg = pairs / experts;
    if (avg <= 16) return 16;
    if (avg <= 96 || k % 32 != 0) return 64;
    return 128;
}

int mi355_hyb_moe_group(int32_t* pos, int32_t* row_token, int32_t* block_table, const int32_t* expert_ids, int32_t pairs, int32_t top,
                        int32_t experts, int32_t block_rows, int32_t n_blocks, int64_t stream) {
    if (pairs <= 0) return 0;
    if (!pos || !row_token || !block_table || !expert_ids || top < 1 || experts < 1 || experts > 4096 || block_rows < 1) return -1;
    if (n_blocks < (pairs + block_rows - 1) / block_rows + experts) return -1;
    moe_group_kernel<<<1, 1024, (size_t)(3 * experts + 1) * sizeof(int), to_stream(stream)>>>(pos, row_token, block_table, expert_ids, pairs, top,
                                                                                              experts, block_rows, n_blocks);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_linear_grouped(float* out, int32_t ldo, const void* a, int32_t a_dtype, int32_t lda, const int32_t* row_token, const void* w,
                             int64_t w_bs, const int32_t* block_table, int32_t block_rows, int32_t n_blocks, int32_t n, int32_t k,
                             int32_t dtype, int64_t stream) {
    if (!out || !a || !w || !block_table || n <= 0 || k <= 0 || ldo < n || lda < k || w_bs < 0 || !is_dt(dtype) || !is_dt(a_dtype)) return -1;
    if (n_blocks <= 0) return 0;
    if (n_blocks > 65535) return -1;
    LinArgs p{out, ldo, a, lda, w, nullptr, n_blocks * block_rows, n, k, 0, 0, 0, w_bs, 0, block_table, row_token, block_rows};
    hipStream_t st_ = to_stream(stream);
    if (dtype == MI355_DTYPE_F32) {
        if (a_dtype != MI355_DTYPE_F32 || block_rows != 64) return -1;
        linear_f32_kernel<<<dim3((n + 63) / 64, n_blocks, 1), 256, 0, st_>>>(p);
        LAUNCH_OK(); return 0;
    }
    const int a_bytes = a_dtype == MI355_DTYPE_F32 ? 4 : 2;
    p.w_vec = (k % 8 == 0) && ((uintptr_t)w % 16 == 0) && (w_bs % 8 == 0);
    p.a_vec = ((size_t)lda * a_bytes % 16 == 0) && ((uintptr_t)a % 16 == 0);
    const bool af = a_dtype == MI355_DTYPE_F32;
    if (block_rows == 16) {
        const dim3 grid((n + 15) / 16, n_blocks, 1);
        if (k >= 2048) { if (af) linear_bf16_stream_kernel<float, 4, 4><<<grid, 256, 0, st_>>>(p); else linear_bf16_stream_kernel<uint16_t, 4, 4><<<grid, 256, 0, st_>>>(p); }
        else { if (af) linear_bf16_stream_kernel<float, 2, 2><<<grid, 128, 0, st_>>>(p); else linear_bf16_stream_kernel<uint16_t, 2, 2><<<grid, 128, 0, st_>>>(p); }
    } else if (block_rows == 64) {
        const dim3 grid((n + 63) / 64, n_blocks, 1);
        if (af) linear_bf16_tile_kernel<float, 4><<<grid, 256, 0, st_>>>(p); else linear_bf16_tile_kernel<uint16_t, 4><<<grid, 256, 0, st_>>>(p);
    } else if (block_rows == 128 && !af && p.a_vec && p.w_vec && k % 32 == 0) {
        linear_bf16_lds_kernel<<<dim3((n + 127) / 128, n_blocks, 1), 256, 0, st_>>>(p);
    } else {
        return -1;
    }
    LAUNCH_OK(); return 0;
}

int mi355_hyb_silu_glu(void* out, int32_t out_dtype, const float* gu, int32_t rows, int32_t ff, const int32_t* block_table,
                       int32_t block_rows, int64_t stream) {
    if (!out || !gu || ff <= 0 || !is_dt(out_dtype) || (block_table && block_rows < 1)) return -1;
    const int64_t n = (int64_t)rows * ff;
    if (n <= 0) return 0;
    const unsigned grid = (unsigned)((n + 255) / 256);
    if (out_dtype == MI355_DTYPE_F32) silu_glu_kernel<float><<<grid, 256, 0, to_stream(stream)>>>((float*)out, gu, n, ff, block_table, block_rows);
    else silu_glu_kernel<uint16_t><<<grid, 256, 0, to_stream(stream)>>>((uint16_t*)out, gu, n, ff, block_table, block_rows);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_moe_combine_norm_add(float* x, void* xcopy, const float* y_rows, const int32_t* pos, const float* weights,
                                   const float* y_shared, const float* shared_gate, const float* w, int32_t T, int32_t width, int32_t top,
                                   float eps, int64_t stream) {
    if (!x || !y_rows || !pos || !weights || !w || width <= 0 || width > 4096 || top < 1) return -1;
    if (T <= 0) return 0;
    const size_t lds = (size_t)top * 8;
    if (top > 4096) return -1;
    if (width % 4 == 0 && (uintptr_t)y_rows % 16 == 0)
        moe_combine_norm_add_kernel<true><<<T, 256, lds, to_stream(stream)>>>(x, (uint16_t*)xcopy, y_rows, pos, weights, y_shared, shared_gate, w, width, top, eps);
    else
        moe_combine_norm_add_kernel<false><<<T, 256, lds, to_stream(stream)>>>(x, (uint16_t*)xcopy, y_rows, pos, weights, y_shared, shared_gate, w, width, top, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_norm_conv(void* out, int32_t out_dtype, float* hn, const float* x, const float* norm_w, const float* conv_w, float* conv_state,
                        int64_t state_stride, const uint32_t* context_lens, const uint32_t* cu_seqlens_q, const int32_t* state_slots,
                        const int32_t* tok_seq, int32_t num_seqs, int32_t T, int32_t width, int32_t taps, int32_t update_state, float eps,
                        int64_t stream) {
    if (!out || !x || !conv_w || !conv_state || !context_lens || !cu_seqlens_q || !state_slots || !tok_seq || !is_dt(out_dtype)) return -1;
    if (width <= 0 || taps < 1 || taps > 8) return -1;
    if (update_state && T != num_seqs) return -1;                       // a workgroup moves its slot's rows only when it is the portion
    if (T <= 0) return 0;
    const bool f = out_dtype == MI355_DTYPE_F32;
    NormConvArgs p{f ? (float*)out : nullptr, f ? nullptr : (uint16_t*)out, hn, x, norm_w, conv_w, conv_state, state_stride, context_lens,
                   cu_seqlens_q, state_slots, tok_seq, width, update_state ? 1 : 0, eps};
    hipStream_t s_ = to_stream(stream);
    // few tokens (decoding batches): sixteen waves per token, so that a thread walks one or two channels instead of eight
#define NC(TAPS) do { if (T <= 64) norm_conv_kernel<TAPS, 16><<<T, 1024, 0, s_>>>(p); else norm_conv_kernel<TAPS, 4><<<T, 256, 0, s_>>>(p); } while (0)
    switch (taps) {
        case 1: NC(1); break; case 2: NC(2); break; case 3: NC(3); break; case 4: NC(4); break;
        case 5: NC(5); break; case 6: NC(6); break; case 7: NC(7); break; default: NC(8); break;
    }
#undef NC
    LAUNCH_OK(); return 0;
}

}  // extern "C"
