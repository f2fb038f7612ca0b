// More kernels of the layer-list host layer (include/mi355_hybrid.h): the mechanisms of designs whose layers read ONE norm and add
// mixer and feed-forward side by side -- layer norm, the state-space scan (scalar decay per head) with its gated group norm, the
// per-layer token input, the weighted average over the depth of the stack, the experts' sum without a norm, and small elementwise
// glue.  Numerics as in hybrid_kernels.hip: residual stream, norms, recurrent state and everything that enters the recurrence are f32.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>

#include "common.h"
#include "hybrid_device.h"
#include "../../include/mi355_hybrid.h"

namespace {

__device__ __forceinline__ float gelu_tanhf_(float z) { return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

template <typename TW> __global__ void embed_scaled_kernel(float* x, const TW* table, const uint32_t* ids, int width, int vocab, float scale) {
    const int t = blockIdx.x;
    const uint32_t id = min(ids[t], (uint32_t)(vocab - 1));
    for (int i = threadIdx.x; i < width; i += blockDim.x) x[(size_t)t * width + i] = ld<TW>(table, (size_t)id * width + i) * scale;
}

// One workgroup per row.  kind 0: x / sqrt(mean(x^2) + eps) w;  kind 1: (x - mean) / sqrt(mean((x - mean)^2) + eps) w (the mean is
// taken off before the squares are summed: two passes over a row that stays in cache).  rows != NULL: row r of the output is row
// rows[r] of x.
template <typename TO> __global__ __launch_bounds__(1024) void norm_rows_kernel(TO* out, float* out_f32, const float* x, int ldx, const int32_t* rows,
                                                                             const float* w, int width, int kind, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : r) * ldx;
    float mean = 0.f;
    if (kind == 1) {
        float s = 0.f;
        for (int i = threadIdx.x; i < width; i += blockDim.x) s += xr[i];
        mean = block_sum(s, red) / (float)width;
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) { const float d = xr[i] - mean; ss = fmaf(d, d, ss); }
    const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = (xr[i] - mean) * inv * w[i];
        st<TO>(out, (size_t)r * width + i, v);
        if (out_f32) out_f32[(size_t)r * width + i] = v;
    }
}

__global__ void add2_kernel(float* x, const float* a, const float* b, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] += b ? a[i] + b[i] : a[i];
}

// x[t] += y[t] + sum_j wts[t, j] rows[pos[t top + j]]; a workgroup per token, the token's rows and weights through LDS first
__global__ __launch_bounds__(1024) void moe_combine_add_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ rows,
                                                              const int32_t* __restrict__ pos, const float* __restrict__ wts, int width, int top) {
    extern __shared__ int csm[];
    int* sp = csm;
    float* sw = reinterpret_cast<float*>(csm + top);
    const int t = blockIdx.x;
    for (int j = threadIdx.x; j < top; j += blockDim.x) { sp[j] = pos[(size_t)t * top + j]; sw[j] = wts[(size_t)t * top + j]; }
    __syncthreads();
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float a = 0.f;
        for (int j = 0; j < top; ++j) a = fmaf(sw[j], rows[(size_t)sp[j] * width + i], a);
        x[(size_t)t * width + i] += y ? y[(size_t)t * width + i] + a : a;
    }
}

template <typename TO> __global__ void relu2_kernel(TO* out, const float* u, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) { const float v = fmaxf(u[i], 0.f); st<TO>(out, (size_t)i, v * v); }
}

__global__ void tanh_cap_kernel(float* x, float cap, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

template <typename TO> __global__ void elem_gate_kernel(TO* out, const float* in, const float* gate_in, int ldg, int64_t total, int n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int64_t t = i / n;
    st<TO>(out, (size_t)i, in[i] * sigmoidf_(gate_in[(size_t)t * ldg + (i - t * n)]));
}

template <typename TO, typename TW> __global__ void side_act_kernel(TO* out, const float* g, const TW* table, int ldt, int col, const uint32_t* ids,
                                                                    int64_t total, int dim, int vocab) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int64_t t = i / dim;
    const int k = (int)(i - t * dim);
    const uint32_t id = min(ids[t], (uint32_t)(vocab - 1));
    st<TO>(out, (size_t)i, gelu_tanhf_(g[i]) * ld<TW>(table, (size_t)id * ldt + col + k));
}

// xs[terms - 1] <- x, x <- sum_j w[j] xs[j]
__global__ void depth_average_kernel(float* x, float* xs, const float* w, int terms, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float cur = x[i];
    xs[(size_t)(terms - 1) * n + i] = cur;
    float acc = 0.f;
    for (int j = 0; j + 1 < terms; ++j) acc = fmaf(w[j], xs[(size_t)j * n + i], acc);
    x[i] = fmaf(w[terms - 1], cur, acc);
}

// The end of a layer and the start of the next in one launch, a workgroup per token row (a thread reads back only what it wrote):
//   x += y / rms(y) * sw            (y != NULL: the token's side input)
//   xs[terms - 1] <- x;  x <- sum_j dw[j] xs[j]      (dw != NULL: the average over the depth)
//   out = norm(x) * nw              (nw != NULL: the norm the next layer's sublayers read; out_f32: a second copy in f32)
template <typename TO> __global__ __launch_bounds__(1024) void layer_tail_kernel(float* x, const float* y, const float* sw, float* xs, const float* dw,
                                                                               int terms, int64_t n, TO* out, float* out_f32, const float* nw, int width,
                                                                               int kind, float eps) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    float* xr = x + (size_t)t * width;
    float inv_y = 0.f;
    if (y) {
        const float* yr = y + (size_t)t * width;
        float ss = 0.f;
        for (int i = threadIdx.x; i < width; i += blockDim.x) ss = fmaf(yr[i], yr[i], ss);
        inv_y = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
    }
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float v = xr[i];
        if (y) v += y[(size_t)t * width + i] * inv_y * sw[i];
        if (dw) {
            const size_t at = (size_t)t * width + i;
            float acc = 0.f;
            for (int j = 0; j + 1 < terms; ++j) acc = fmaf(dw[j], xs[(size_t)j * n + at], acc);
            xs[(size_t)(terms - 1) * n + at] = v;
            v = fmaf(dw[terms - 1], v, acc);
        }
        xr[i] = v;
        sum += v;
    }
    if (!nw) return;
    const float mean = kind == 1 ? block_sum(sum, red) / (float)width : 0.f;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) { const float d = xr[i] - mean; ss = fmaf(d, d, ss); }
    const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = (xr[i] - mean) * inv * nw[i];
        st<TO>(out, (size_t)t * width + i, v);
        if (out_f32) out_f32[(size_t)t * width + i] = v;
    }
}

// out = (y silu(z)) / rms over the part * w: a workgroup of 256 per (token, part)
template <typename TO> __global__ __launch_bounds__(256) void gate_group_norm_kernel(TO* out, const float* y, const float* gate_in, int ldg, const float* w,
                                                                                    int n, int groups, float eps) {
    __shared__ float red[16];
    const int t = blockIdx.x, g = blockIdx.y, per = n / groups, c0 = g * per;
    const float* yr = y + (size_t)t * n + c0;
    const float* zr = gate_in + (size_t)t * ldg + c0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < per; i += blockDim.x) { const float v = yr[i] * siluf_(zr[i]); ss = fmaf(v, v, ss); }
    const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)per + eps);
    for (int i = threadIdx.x; i < per; i += blockDim.x) st<TO>(out, (size_t)t * n + c0 + i, yr[i] * siluf_(zr[i]) * inv * w[c0 + i]);
}

// ------------------------------------------------------------------------------------------------------------ state-space scan
struct SsdArgs {
    float* y; float* state; int64_t state_stride;
    const float* xbc; int ldx; const float* dt_in; int ldd;
    const float* a_log; const float* dt_bias; const float* skip;
    const uint32_t* ctx; const uint32_t* cu_q; const int32_t* slots;
    int H, G, N, vd;
};
// A workgroup of 256 threads owns 256 / LPC columns of one (sequence, head)'s state S [N, vd]; LPC neighbouring lanes share a column,
// each holding DP = ceil(N / LPC) of its rows in registers, and walk the new tokens in order:
//   S <- decay S + (dt x[col]) B;  y[col] = sum_n S[n] C[n] + skip x[col]
// The update of a row depends on the row alone and the sum over n (lane exchanges among the LPC lanes) is off the chain, so the time
// per token is a multiply-add per row and the LDS reads of B and C.  B, C of CH tokens at a time sit in LDS (rows padded so that the
// parts fall into different banks), the step sizes and decays of those tokens are made by the first CH threads while they are staged;
// the next CH tokens are fetched into registers while the current ones are used.
template <int DP, int LPC, int CH> __global__ __launch_bounds__(256) void ssd_scan_kernel(SsdArgs p) {
    constexpr int RS = DP + 4, ROW = LPC * DP, TOT = CH * ROW, NPT = (TOT + 255) / 256, CPB = 256 / LPC;
    __shared__ __align__(16) float sB[2][CH][LPC][RS], sC[2][CH][LPC][RS];
    __shared__ float sdt[2][CH], sdec[2][CH];
    const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int col = blockIdx.z * CPB + tid / LPC, part = tid % LPC;
    const int N = p.N, vd = p.vd, g = h / (p.H / p.G);
    const int tb = (int)p.cu_q[s], te = (int)p.cu_q[s + 1];
    if (te <= tb) return;
    const int start_pos = (int)p.ctx[s] - (te - tb);
    const bool own = col < vd;
    float* stt = p.state + (size_t)p.slots[s] * p.state_stride + (size_t)h * N * vd;
    float S[DP];
#pragma unroll
    for (int r = 0; r < DP; ++r) { const int i = part * DP + r; S[r] = (own && i < N && start_pos > 0) ? stt[(size_t)i * vd + col] : 0.f; }
    const int x_col = h * vd + col, b_off = p.H * vd + g * N, c_off = p.H * vd + p.G * N + g * N;
    const float a_rate = expf(p.a_log[h]), dtb = p.dt_bias[h], skip = p.skip ? p.skip[h] : 0.f;
    float rB[NPT], rC[NPT], rv[CH], rdt = 0.f, rdec = 1.f;
    auto fetch = [&](int t0) {
#pragma unroll
        for (int n = 0; n < NPT; ++n) {
            const int idx = tid + n * 256, c = idx / ROW, ii = idx - c * ROW, t = t0 + c;
            const bool ok_ = idx < TOT && t < te && ii < N;
            const float* row = p.xbc + (size_t)(ok_ ? t : tb) * p.ldx;
            rB[n] = ok_ ? row[b_off + ii] : 0.f;
            rC[n] = ok_ ? row[c_off + ii] : 0.f;
        }
#pragma unroll
        for (int c = 0; c < CH; ++c) rv[c] = (own && t0 + c < te) ? p.xbc[(size_t)(t0 + c) * p.ldx + x_col] : 0.f;
        if (tid < CH && t0 + tid < te) {
            rdt = softplusf_(p.dt_in[(size_t)(t0 + tid) * p.ldd + h] + dtb);
            rdec = expf(-a_rate * rdt);
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int n = 0; n < NPT; ++n) {
            const int idx = tid + n * 256;
            if (idx < TOT) {
                const int c = idx / ROW, ii = idx - c * ROW, pp = ii / DP, r = ii - pp * DP;
                sB[buf][c][pp][r] = rB[n]; sC[buf][c][pp][r] = rC[n];
            }
        }
        if (tid < CH) { sdt[buf][tid] = rdt; sdec[buf][tid] = rdec; }
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
        auto token = [&](int c) {
            const float dec = sdec[buf][c], dx = sdt[buf][c] * vc[c];
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < DP; ++r) {
                S[r] = fmaf(dec, S[r], dx * sB[buf][c][part][r]);
                o = fmaf(S[r], sC[buf][c][part][r], o);
            }
            o = column_sum<LPC>(o);
            if (own && part == 0) p.y[((size_t)(t0 + c) * p.H + h) * vd + col] = fmaf(skip, vc[c], o);
        };
        if (cn == CH) {                                          // a whole chunk: no branch between the tokens, their LDS reads run ahead
#pragma unroll
            for (int c = 0; c < CH; ++c) token(c);
        } else {
            for (int c = 0; c < cn; ++c) token(c);
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
    }
    if (own)
#pragma unroll
        for (int r = 0; r < DP; ++r) { const int i = part * DP + r; if (i < N) stt[(size_t)i * vd + col] = S[r]; }
}

inline unsigned blocks_of(int64_t n) { return (unsigned)((n + 255) / 256); }

}  // namespace

extern "C" {

int mi355_hyb_embed_scaled(float* x, const void* table, const uint32_t* ids, int32_t T, int32_t width, int32_t vocab, float scale,
                           int32_t dtype, int64_t stream) {
    if (!x || !table || !ids || width <= 0 || vocab <= 0 || !is_dt(dtype)) return -1;
    if (T <= 0) return 0;
    if (dtype == MI355_DTYPE_F32) embed_scaled_kernel<float><<<T, 256, 0, to_stream(stream)>>>(x, (const float*)table, ids, width, vocab, scale);
    else embed_scaled_kernel<uint16_t><<<T, 256, 0, to_stream(stream)>>>(x, (const uint16_t*)table, ids, width, vocab, scale);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_pre_norm_ex(void* out, int32_t out_dtype, float* out_f32, const float* x, int32_t ldx, const float* w, int32_t T, int32_t width,
                          int32_t kind, float eps, int64_t stream) {
    if (!out || !x || !w || !is_dt(out_dtype) || width <= 0 || ldx < width || kind < 0 || kind > 1) return -1;
    if (T <= 0) return 0;
    const int nt = (T <= 64 && width > 256) ? 1024 : 256;
    if (out_dtype == MI355_DTYPE_F32) norm_rows_kernel<float><<<T, nt, 0, to_stream(stream)>>>((float*)out, out_f32, x, ldx, nullptr, w, width, kind, eps);
    else norm_rows_kernel<uint16_t><<<T, nt, 0, to_stream(stream)>>>((uint16_t*)out, out_f32, x, ldx, nullptr, w, width, kind, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_gather_norm_ex(void* out, int32_t out_dtype, const float* x, const int32_t* rows, const float* w, int32_t n_rows, int32_t width,
                             int32_t kind, float eps, int64_t stream) {
    if (!out || !x || !rows || !w || !is_dt(out_dtype) || width <= 0 || kind < 0 || kind > 1) return -1;
    if (n_rows <= 0) return 0;
    if (out_dtype == MI355_DTYPE_F32) norm_rows_kernel<float><<<n_rows, 256, 0, to_stream(stream)>>>((float*)out, nullptr, x, width, rows, w, width, kind, eps);
    else norm_rows_kernel<uint16_t><<<n_rows, 256, 0, to_stream(stream)>>>((uint16_t*)out, nullptr, x, width, rows, w, width, kind, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_add2(float* x, const float* a, const float* b, int64_t n, int64_t stream) {
    if (!x || !a) return -1;
    if (n <= 0) return 0;
    add2_kernel<<<blocks_of(n), 256, 0, to_stream(stream)>>>(x, a, b, n);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_moe_combine_add(float* x, const float* y, const float* y_rows, const int32_t* pos, const float* weights, int32_t T, int32_t width,
                              int32_t top, int64_t stream) {
    if (!x || !y_rows || !pos || !weights || width <= 0 || top < 1 || top > 4096) return -1;
    if (T <= 0) return 0;
    moe_combine_add_kernel<<<T, (T <= 64 && width > 256) ? 1024 : 256, (size_t)top * 8, to_stream(stream)>>>(x, y, y_rows, pos, weights, width, top);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_relu2(void* out, int32_t out_dtype, const float* u, int64_t n, int64_t stream) {
    if (!out || !u || !is_dt(out_dtype)) return -1;
    if (n <= 0) return 0;
    if (out_dtype == MI355_DTYPE_F32) relu2_kernel<float><<<blocks_of(n), 256, 0, to_stream(stream)>>>((float*)out, u, n);
    else relu2_kernel<uint16_t><<<blocks_of(n), 256, 0, to_stream(stream)>>>((uint16_t*)out, u, n);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_tanh_cap(float* x, float cap, int64_t n, int64_t stream) {
    if (!x || !(cap > 0.f)) return -1;
    if (n <= 0) return 0;
    tanh_cap_kernel<<<blocks_of(n), 256, 0, to_stream(stream)>>>(x, cap, n);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_elem_gate(void* out, int32_t out_dtype, const float* in, const float* gate_in, int32_t ldg, int32_t T, int32_t n, int64_t stream) {
    if (!out || !in || !gate_in || !is_dt(out_dtype) || n <= 0 || ldg < n) return -1;
    if (T <= 0) return 0;
    const int64_t total = (int64_t)T * n;
    if (out_dtype == MI355_DTYPE_F32) elem_gate_kernel<float><<<blocks_of(total), 256, 0, to_stream(stream)>>>((float*)out, in, gate_in, ldg, total, n);
    else elem_gate_kernel<uint16_t><<<blocks_of(total), 256, 0, to_stream(stream)>>>((uint16_t*)out, in, gate_in, ldg, total, n);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_side_act(void* out, int32_t out_dtype, const float* g, const void* table, int32_t ldt, int32_t col, const uint32_t* ids, int32_t T,
                       int32_t dim, int32_t vocab, int32_t dtype, int64_t stream) {
    if (!out || !g || !table || !ids || !is_dt(out_dtype) || !is_dt(dtype) || dim <= 0 || col < 0 || ldt < col + dim || vocab <= 0) return -1;
    if (T <= 0) return 0;
    const int64_t total = (int64_t)T * dim;
    hipStream_t s_ = to_stream(stream);
    const bool of = out_dtype == MI355_DTYPE_F32, tf = dtype == MI355_DTYPE_F32;
    if (of && tf) side_act_kernel<float, float><<<blocks_of(total), 256, 0, s_>>>((float*)out, g, (const float*)table, ldt, col, ids, total, dim, vocab);
    else if (of) side_act_kernel<float, uint16_t><<<blocks_of(total), 256, 0, s_>>>((float*)out, g, (const uint16_t*)table, ldt, col, ids, total, dim, vocab);
    else if (tf) side_act_kernel<uint16_t, float><<<blocks_of(total), 256, 0, s_>>>((uint16_t*)out, g, (const float*)table, ldt, col, ids, total, dim, vocab);
    else side_act_kernel<uint16_t, uint16_t><<<blocks_of(total), 256, 0, s_>>>((uint16_t*)out, g, (const uint16_t*)table, ldt, col, ids, total, dim, vocab);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_depth_average(float* x, float* xs, const float* w, int32_t terms, int64_t n, int64_t stream) {
    if (!x || !xs || !w || terms < 1) return -1;
    if (n <= 0) return 0;
    depth_average_kernel<<<blocks_of(n), 256, 0, to_stream(stream)>>>(x, xs, w, terms, n);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_layer_tail(float* x, const float* y, const float* side_w, float* xs, const float* depth_w, int32_t terms, void* out, int32_t out_dtype,
                         float* out_f32, const float* norm_w, int32_t T, int32_t width, int32_t kind, float eps, int64_t stream) {
    if (!x || width <= 0 || (y && !side_w) || (depth_w && (!xs || terms < 1)) || (norm_w && (!out || !is_dt(out_dtype))) || kind < 0 || kind > 1) return -1;
    if (T <= 0) return 0;
    const int64_t n = (int64_t)T * width;
    // a row's passes are chains of loads: few rows (decoding batches) take 1024 threads a row so that a thread walks a quarter of the chain
    const int nt = (T <= 64 && width > 256) ? 1024 : 256;
    if (!norm_w || out_dtype == MI355_DTYPE_F32)
        layer_tail_kernel<float><<<T, nt, 0, to_stream(stream)>>>(x, y, side_w, xs, depth_w, terms, n, (float*)out, out_f32, norm_w, width, kind, eps);
    else
        layer_tail_kernel<uint16_t><<<T, nt, 0, to_stream(stream)>>>(x, y, side_w, xs, depth_w, terms, n, (uint16_t*)out, out_f32, norm_w, width, kind, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_gate_group_norm(void* out, int32_t out_dtype, const float* y, const float* gate_in, int32_t ldg, const float* w, int32_t T,
                              int32_t n, int32_t groups, float eps, int64_t stream) {
    if (!out || !y || !gate_in || !w || !is_dt(out_dtype) || n <= 0 || groups < 1 || n % groups || ldg < n) return -1;
    if (T <= 0) return 0;
    const dim3 grid(T, groups);
    if (out_dtype == MI355_DTYPE_F32) gate_group_norm_kernel<float><<<grid, 256, 0, to_stream(stream)>>>((float*)out, y, gate_in, ldg, w, n, groups, eps);
    else gate_group_norm_kernel<uint16_t><<<grid, 256, 0, to_stream(stream)>>>((uint16_t*)out, y, gate_in, ldg, w, n, groups, eps);
    LAUNCH_OK(); return 0;
}

int mi355_hyb_ssd_scan(float* y, float* state, int64_t state_stride, const float* xbc, int32_t ldx, const float* dt_in, int32_t ldd,
                       const float* a_log, const float* dt_bias, const float* skip, const uint32_t* context_lens,
                       const uint32_t* cu_seqlens_q, const int32_t* state_slots, int32_t num_seqs, int32_t num_tokens, int32_t heads,
                       int32_t groups, int32_t n_state, int32_t vdim, int64_t stream) {
    if (!y || !state || !xbc || !dt_in || !a_log || !dt_bias || !context_lens || !cu_seqlens_q || !state_slots) return -1;
    if (heads <= 0 || groups <= 0 || heads % groups || n_state <= 0 || n_state > 512 || vdim <= 0) return -1;
    if (ldx < heads * vdim + 2 * groups * n_state || ldd < heads) return -1;
    if (num_seqs <= 0 || num_tokens <= 0) return 0;
    SsdArgs p{y, state, state_stride, xbc, ldx, dt_in, ldd, a_log, dt_bias, skip, context_lens, cu_seqlens_q, state_slots, heads, groups, n_state, vdim};
    hipStream_t s_ = to_stream(stream);
    if (n_state < 64) {
        const dim3 grid(num_seqs, heads, (vdim + 63) / 64);
        if (n_state <= 16) ssd_scan_kernel<4, 4, 8><<<grid, 256, 0, s_>>>(p);
        else if (n_state <= 32) ssd_scan_kernel<8, 4, 8><<<grid, 256, 0, s_>>>(p);
        else ssd_scan_kernel<16, 4, 8><<<grid, 256, 0, s_>>>(p);
    } else {
        const dim3 grid(num_seqs, heads, (vdim + 15) / 16);
        // portions of prompts: 16 tokens per stage (the wait for a stage's rows is paid half as often); decoding batches: 8
        const bool longer = num_tokens > 8 * num_seqs;
        if (n_state <= 64) { if (longer) ssd_scan_kernel<4, 16, 16><<<grid, 256, 0, s_>>>(p); else ssd_scan_kernel<4, 16, 8><<<grid, 256, 0, s_>>>(p); }
        else if (n_state <= 128) { if (longer) ssd_scan_kernel<8, 16, 16><<<grid, 256, 0, s_>>>(p); else ssd_scan_kernel<8, 16, 8><<<grid, 256, 0, s_>>>(p); }
        else if (n_state <= 256) ssd_scan_kernel<16, 16, 8><<<grid, 256, 0, s_>>>(p);
        else ssd_scan_kernel<32, 16, 4><<<grid, 256, 0, s_>>>(p);       // (stages of 4 tokens: two stages of B and C rows of 512 states fill LDS)
    }
    LAUNCH_OK(); return 0;
}

}  // extern "C"
