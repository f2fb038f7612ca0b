// Host layer of the layer-list ("hybrid") models (include/mi355_hybrid.h): a model is a list of layers, each with one token mixer
// (sliding-window attention with a sink, gated delta rule, minGRU, attention and delta rule side by side, latent attention, or
// attention behind a short convolution with mixed head weights) and an optional feed-forward; x <- x + norm(mixer(x)),
// x <- x + norm(ff(x)) -- or, with residual_form 1, x <- norm(alpha x + mixer(x)), x <- norm(alpha x + ff(x)) -- the sublayers read
// x itself; residual_form 2 puts a norm on both sides, x <- x + norm(sub(pre_norm(x))), optionally with a short causal convolution
// added to the mixer's input; residual_form 3 has ONE norm per layer that mixer and feed-forward both read, x <- x + mixer(h) + ff(h),
// then the token's side input and the average over the depth (a state-space mixer and an ungated feed-forward belong to that form's
// design).  The feed-forward is a dense gate/up form or a mixture of experts (router, grouped expert products over
// device-built blocks, shared expert).  A layer may run on another layer's weights (share_with) and still owns its pages and state.  Like the llama-family host layers
// (host_model.cpp, dense_model.cpp) it owns the weights, the K/V pages and the activation buffers and enqueues one step on a
// stream; unlike them it owns a pool of recurrent state (one slot per live sequence, handed out by the block engine) and runs
// prompts, portions of prompts and decoded tokens through the same launches.
// Kernels: hybrid_kernels.hip.  Every projection that reads a mixer's input is one matrix (rows concatenated at load time), the
// output projections of a parallel mixer are one matrix along k (the branch scales are applied to the operands, not the weights).
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <map>
#include <vector>

#include "../../include/mi355_hybrid.h"

#define MI355_DTYPE_F32 0
#define MI355_DTYPE_BF16 2

extern "C" {
int mi355_hyb_token_seq(int32_t*, const uint32_t*, int32_t, int64_t);
int mi355_hyb_bf16_to_f32(float*, const uint16_t*, int64_t, int64_t);
int mi355_hyb_fill_f32(float*, float, int64_t, int64_t);
int mi355_hyb_embed(float*, void*, const void*, const uint32_t*, int32_t, int32_t, int32_t, int32_t, int64_t);
int mi355_hyb_gather_norm(void*, int32_t, const float*, const int32_t*, const float*, int32_t, int32_t, float, int64_t);
}
#define MOE_MAX_BLOCK_ROWS 128

namespace {

#define HCHECK(expr) do { const int rc_ = (expr); if (rc_ != 0) return rc_; } while (0)
#define HHIP(expr) do { const hipError_t e_ = (expr); if (e_ != hipSuccess) return (int)e_; } while (0)

enum { P_AQ = 0, P_AK, P_AV, P_DQ, P_DK, P_DV, P_B, P_A, P_G, P_COUNT };   // parts of the input projection (minGRU: z, x, g in 0..2)

struct Weight { void* p = nullptr; int64_t n = 0; };

struct HLayer {
    mi355_hybrid_layer c{};
    Weight w[MI355_HW_COUNT];
    int32_t off[P_COUNT];
    int32_t in_rows = 0, out_k = 0;
    float *cos_t = nullptr, *sin_t = nullptr; int n_pos = 0;
    void *k_pages = nullptr, *v_pages = nullptr;
    int64_t conv_off = 0, state_off = 0;          // floats from the start of a slot
    int64_t in_conv_off = 0;                      // the input convolution's last rows
    bool has_attn() const { return c.mixer == MI355_HYB_MIX_PARALLEL || c.mixer == MI355_HYB_MIX_ATTENTION; }
    bool has_delta() const { return c.mixer == MI355_HYB_MIX_PARALLEL || c.mixer == MI355_HYB_MIX_DELTA; }
    bool is_latent() const { return c.mixer == MI355_HYB_MIX_LATENT; }
    bool is_conv_attn() const { return c.mixer == MI355_HYB_MIX_CONV_ATTENTION; }
    bool is_ssd() const { return c.mixer == MI355_HYB_MIX_SSD; }
    bool uses_pages() const { return has_attn() || is_latent() || is_conv_attn(); }
    bool owns_pages() const { return uses_pages() && !c.kv_from; }       // a layer with kv_from reads another layer's pages
    int ssd_inner() const { return c.d_heads * c.d_vdim; }
    int ssd_channels() const { return c.d_heads * c.d_vdim + 2 * c.d_kv_heads * c.d_dim; }   // x | B | C: what the convolution sees
    bool rotates() const { return (has_attn() || is_latent()) && c.a_rot_dims > 0; }
    int conv_channels() const { return 2 * c.d_kv_heads * c.d_dim + c.d_heads * c.d_vdim; }
    int a_conv_channels() const { return (c.a_heads + c.a_kv_heads) * c.a_dim + c.a_kv_heads * c.a_vdim; }
    // elements of a token's row in the key / value pages (latent attention: one row [latent | rotated key part], no value pages)
    // a shared expert of the experts' size runs as one more group of the grouped products (and one more pair of every token)
    bool shared_merged() const { return c.mlp_kind == 3 && c.moe_shared_ff > 0 && c.moe_shared_ff == c.mlp_ff; }
    int k_row() const { return is_latent() ? c.a_kv_rank + c.a_rot_dim : c.a_kv_heads * c.a_dim; }
    int v_row() const { return is_latent() ? 0 : c.a_kv_heads * c.a_vdim; }
};

struct HModel {
    mi355_hybrid_config cfg{};
    std::vector<HLayer> layers;
    Weight embed, final_norm, head;
    int64_t slot_floats = 0;
    float* state = nullptr;
    int num_blocks = 0;
    // activations (grow-only)
    int cap_t = 0, cap_out = 0;
    float *prep = nullptr, *x = nullptr, *proj = nullptr, *aux1 = nullptr, *aux2 = nullptr, *conv = nullptr, *o = nullptr, *y = nullptr, *gu = nullptr;
    void *xcopy = nullptr, *q = nullptr, *mix = nullptr, *act = nullptr, *xn = nullptr, *att = nullptr;
    int32_t* tok_seq = nullptr;
    // residual form 2 / input convolution: what the sublayer's first product reads; mixture of experts: routing and the gathered rows
    void *pre = nullptr, *moe_act = nullptr;
    // form 3 / depth average / token side input / query latent
    float *y2 = nullptr, *hf = nullptr, *xs = nullptr, *side_g = nullptr;
    void *side_a = nullptr, *cq = nullptr;
    Weight side_table;
    bool need_hf = false, need_xs = false;
    int max_side = 0, max_q_rank = 0;
    float *moe_gu = nullptr, *moe_y = nullptr, *moe_wts = nullptr, *moe_sgate = nullptr;
    int32_t *moe_ids = nullptr, *moe_pos = nullptr, *moe_row_token = nullptr, *moe_table = nullptr;
    bool need_pre = false;
    int max_moe_top = 0, max_moe_experts = 0, max_moe_ff = 0;
    int max_in_rows = 0, max_aux1 = 0, max_aux2 = 0, max_conv = 0, max_o = 0, max_q = 0, max_mix = 0, max_ff = 0, max_prep = 0, max_att = 0;
    // captured steps (mi355_hybrid_forward_graph): one hipGraph per (device input pointers, counts); whatever re-allocates a buffer a
    // step touches drops them all
    struct StepGraph { hipGraph_t graph = nullptr; hipGraphExec_t exec = nullptr; };
    std::map<std::vector<int64_t>, StepGraph> graphs;
    int64_t graph_captures = 0, graph_replays = 0;
    bool bf16() const { return cfg.dtype == MI355_DTYPE_BF16; }
    size_t esize() const { return bf16() ? 2 : 4; }
};

void drop_graphs(HModel* m) {
    for (auto& kv : m->graphs) {
        if (kv.second.exec) (void)hipGraphExecDestroy(kv.second.exec);
        if (kv.second.graph) (void)hipGraphDestroy(kv.second.graph);
    }
    m->graphs.clear();
}

int in_proj_parts(const mi355_hybrid_layer& c, int32_t* off) {
    for (int i = 0; i < P_COUNT; ++i) off[i] = -1;
    int r = 0;
    if (c.mixer == MI355_HYB_MIX_MINGRU) {
        off[0] = 0; off[1] = c.g_width; off[2] = 2 * c.g_width;
        return 3 * c.g_width;
    }
    if (c.mixer == MI355_HYB_MIX_LATENT) {
        off[P_AQ] = r; r += c.a_q_rank > 0 ? c.a_q_rank : c.a_heads * (c.a_dim + c.a_rot_dim);
        if (!c.kv_from) { off[P_AK] = r; r += c.a_kv_rank + c.a_rot_dim; }
        if (c.a_out_gate) { off[P_G] = r; r += c.a_heads * c.a_vdim; }
        else if (c.a_head_gate) { off[P_G] = r; r += c.a_heads; }
        return r;
    }
    if (c.mixer == MI355_HYB_MIX_SSD) {                                  // [gate z | x | B | C | dt]
        const int inner = c.d_heads * c.d_vdim, gn = c.d_kv_heads * c.d_dim;
        off[P_G] = 0; off[P_DV] = inner; off[P_DK] = 2 * inner; off[P_DQ] = 2 * inner + gn; off[P_A] = 2 * inner + 2 * gn;
        return 2 * inner + 2 * gn + c.d_heads;
    }
    if (c.mixer == MI355_HYB_MIX_PARALLEL || c.mixer == MI355_HYB_MIX_ATTENTION || c.mixer == MI355_HYB_MIX_CONV_ATTENTION) {
        off[P_AQ] = r; r += c.a_heads * c.a_dim;
        off[P_AK] = r; r += c.a_kv_heads * c.a_dim;
        off[P_AV] = r; r += c.a_kv_heads * c.a_vdim;
    }
    if (c.mixer == MI355_HYB_MIX_PARALLEL || c.mixer == MI355_HYB_MIX_DELTA) {
        off[P_DQ] = r; r += c.d_kv_heads * c.d_dim;
        off[P_DK] = r; r += c.d_kv_heads * c.d_dim;
        off[P_DV] = r; r += c.d_heads * c.d_vdim;
        off[P_B] = r; r += c.d_heads;
        off[P_A] = r; r += c.d_decay_channels ? c.d_a_rank : c.d_heads;
        off[P_G] = r; r += c.d_gate == MI355_HYB_GATE_SIGMOID_LR ? c.d_g_rank : c.d_heads * c.d_vdim;
    }
    return r;
}

bool layer_ok(const mi355_hybrid_layer& c) {
    const bool attn = c.mixer == MI355_HYB_MIX_PARALLEL || c.mixer == MI355_HYB_MIX_ATTENTION;
    const bool delta = c.mixer == MI355_HYB_MIX_PARALLEL || c.mixer == MI355_HYB_MIX_DELTA;
    if (c.mixer < 0 || c.mixer > MI355_HYB_MIX_SSD || c.share_with < 0) return false;
    if (c.mixer == MI355_HYB_MIX_SSD) {
        if (c.d_heads <= 0 || c.d_kv_heads <= 0 || c.d_heads % c.d_kv_heads || c.d_dim <= 0 || c.d_dim > 512 || c.d_vdim <= 0) return false;
        if (c.d_conv < 1 || c.d_conv > 16 || c.d_norm_groups < 1 || (c.d_heads * c.d_vdim) % c.d_norm_groups) return false;
    }
    if (c.a_q_rank < 0 || c.kv_from < 0 || c.side_dim < 0 || c.side_col < 0 || c.depth_terms < 0 || c.moe_groups < 0) return false;
    if ((c.a_q_rank || c.a_out_gate || c.kv_from) && c.mixer != MI355_HYB_MIX_LATENT) return false;
    if (c.a_out_gate && c.a_head_gate) return false;
    if (c.a_dist_bias && c.mixer != MI355_HYB_MIX_CONV_ATTENTION) return false;
    if (c.moe_groups > 0 && (c.mlp_kind != 3 || c.moe_experts % c.moe_groups || c.moe_keep_groups < 1 || c.moe_keep_groups > c.moe_groups ||
                             (c.moe_experts / c.moe_groups) * c.moe_keep_groups < c.moe_top)) return false;
    if (c.mixer == MI355_HYB_MIX_LATENT) {
        if (c.a_heads <= 0 || c.a_dim <= 0 || c.a_vdim <= 0 || c.a_kv_rank <= 0 || c.a_rot_dim < 0 || c.a_window < 0) return false;
        if (c.a_rot_dims < 0 || c.a_rot_dims > c.a_rot_dim || (c.a_rot_dims & 1) || c.a_softcap < 0.f) return false;
    }
    if (c.mixer == MI355_HYB_MIX_CONV_ATTENTION) {
        if (c.a_heads <= 0 || c.a_kv_heads <= 0 || c.a_heads % c.a_kv_heads || c.a_dim <= 0 || c.a_vdim <= 0 || c.a_window < 0) return false;
        if (c.a_conv < 1 || c.a_conv > 16 || c.a_softcap < 0.f || c.a_rot_dims != 0) return false;
        if (c.a_qk_norm && !c.a_norm_whole) return false;
    }
    if (attn) {
        if (c.a_heads <= 0 || c.a_kv_heads <= 0 || c.a_heads % c.a_kv_heads || c.a_dim <= 0 || c.a_vdim <= 0 || c.a_vdim > 512) return false;
        if (c.a_window < 0 || c.a_rot_dims < 0 || c.a_rot_dims > c.a_dim || (c.a_rot_dims & 1)) return false;
    }
    if (delta) {
        if (c.d_heads <= 0 || c.d_kv_heads <= 0 || c.d_heads % c.d_kv_heads || c.d_dim <= 0 || c.d_dim > 256 || c.d_vdim <= 0) return false;
        if (c.d_conv < 1 || c.d_conv > 16) return false;
        if (c.d_decay_channels && c.d_a_rank <= 0) return false;
        if (c.d_gate == MI355_HYB_GATE_SIGMOID_LR && c.d_g_rank <= 0) return false;
        if (c.d_gate != MI355_HYB_GATE_SIGMOID_LR && c.d_gate != MI355_HYB_GATE_SILU) return false;
    }
    if (c.mixer == MI355_HYB_MIX_MINGRU && c.g_width <= 0) return false;
    if (c.mlp_kind < 0 || c.mlp_kind > 4 || (c.mlp_kind && c.mlp_ff <= 0)) return false;
    if (c.mlp_kind == 3 && (c.moe_experts < 1 || c.moe_experts > 4096 || c.moe_top < 1 || c.moe_top > c.moe_experts || c.moe_shared_ff < 0)) return false;
    if (c.a_keep_first < 0 || c.in_conv < 0 || c.in_conv > 16) return false;
    if ((c.a_keep_first || c.a_norm_after_rot || c.a_head_temp) && !attn) return false;      // switches of the plain attention branch
    return true;
}

// what a slot holds and in which type: matrices follow the model dtype, vectors and small tables are f32
bool is_matrix(int which) {
    switch (which) {
        case MI355_HW_EMBED: case MI355_HW_HEAD: case MI355_HW_IN_PROJ: case MI355_HW_OUT_PROJ: case MI355_HW_D_A2: case MI355_HW_D_G2:
        case MI355_HW_MLP_GATE_UP: case MI355_HW_MLP_DOWN: case MI355_HW_L_UKT: case MI355_HW_L_UV:
        case MI355_HW_MOE_GATE_UP: case MI355_HW_MOE_DOWN: case MI355_HW_L_UQ: case MI355_HW_SIDE_GATE: case MI355_HW_SIDE_PROJ:
        case MI355_HW_SIDE_TABLE: return true;
        default: return false;
    }
}

int64_t expected_elems(const HModel* m, int layer, int which) {
    const int W = m->cfg.width;
    if (layer < 0) {
        if (which == MI355_HW_EMBED) return (int64_t)m->cfg.vocab * W;
        if (which == MI355_HW_HEAD) return m->cfg.tie_head ? -1 : (int64_t)m->cfg.vocab * W;
        if (which == MI355_HW_FINAL_NORM) return W;
        if (which == MI355_HW_SIDE_TABLE) return m->cfg.side_cols > 0 ? (int64_t)m->cfg.vocab * m->cfg.side_cols : -1;
        return -1;
    }
    const HLayer& L = m->layers[layer];
    const mi355_hybrid_layer& c = L.c;
    if (c.share_with) return -1;                               // a layer that runs on another layer's weights holds none
    switch (which) {
        case MI355_HW_NORM1: return W;
        case MI355_HW_NORM2: return c.mlp_kind && m->cfg.residual_form != 3 ? W : -1;
        case MI355_HW_D_SKIP: return L.is_ssd() ? c.d_heads : -1;
        case MI355_HW_CONV_BIAS: return L.is_ssd() ? L.ssd_channels() : -1;
        case MI355_HW_A_DIST: return L.is_conv_attn() && c.a_dist_bias ? 2 * c.a_heads : -1;
        case MI355_HW_L_QNORM: return L.is_latent() && c.a_q_rank ? c.a_q_rank : -1;
        case MI355_HW_L_UQ: return L.is_latent() && c.a_q_rank ? (int64_t)c.a_heads * (c.a_dim + c.a_rot_dim) * c.a_q_rank : -1;
        case MI355_HW_SIDE_GATE: case MI355_HW_SIDE_PROJ: return c.side_dim ? (int64_t)c.side_dim * W : -1;
        case MI355_HW_SIDE_NORM: return c.side_dim ? W : -1;
        case MI355_HW_DEPTH_W: return c.depth_terms ? c.depth_terms : -1;
        case MI355_HW_IN_PROJ: return (int64_t)L.in_rows * W;
        case MI355_HW_IN_BIAS: return L.in_rows;
        case MI355_HW_OUT_PROJ: return (int64_t)W * L.out_k;
        case MI355_HW_A_QNORM: if (L.is_conv_attn()) return c.a_qk_norm ? c.a_heads * c.a_dim : -1;
                               return L.has_attn() && c.a_qk_norm && !c.a_norm_after_rot ? c.a_dim : -1;
        case MI355_HW_A_KNORM: if (L.is_conv_attn()) return c.a_qk_norm ? c.a_kv_heads * c.a_dim : -1;
                               return L.has_attn() && c.a_qk_norm && !c.a_norm_after_rot ? c.a_dim : -1;
        case MI355_HW_A_TEMP: return L.has_attn() && c.a_head_temp ? c.a_heads : -1;
        case MI355_HW_PRE_NORM1: return m->cfg.residual_form == 2 ? W : -1;
        case MI355_HW_PRE_NORM2: return m->cfg.residual_form == 2 && c.mlp_kind ? W : -1;
        case MI355_HW_IN_CONV: return c.in_conv ? (int64_t)W * c.in_conv : -1;
        case MI355_HW_MOE_ROUTER: return c.mlp_kind == 3 ? (int64_t)(c.moe_experts + (c.moe_shared_ff ? 1 : 0)) * W : -1;
        case MI355_HW_MOE_CORRECTION: return c.mlp_kind == 3 ? c.moe_experts : -1;
        case MI355_HW_MOE_GATE_UP: return c.mlp_kind == 3 ? (int64_t)(c.moe_experts + L.shared_merged()) * 2 * c.mlp_ff * W : -1;
        case MI355_HW_MOE_DOWN: return c.mlp_kind == 3 ? (int64_t)(c.moe_experts + L.shared_merged()) * W * c.mlp_ff : -1;
        case MI355_HW_A_SINK: return (L.has_attn() || L.is_latent()) && c.a_has_sink ? c.a_heads : -1;
        case MI355_HW_A_CONV: return L.is_conv_attn() ? (int64_t)L.a_conv_channels() * c.a_conv : -1;
        case MI355_HW_A_TALK: return L.is_conv_attn() && c.a_talk ? c.a_heads * c.a_heads : -1;
        case MI355_HW_L_UKT: return L.is_latent() ? (int64_t)c.a_heads * c.a_kv_rank * c.a_dim : -1;
        case MI355_HW_L_UV: return L.is_latent() ? (int64_t)c.a_heads * c.a_vdim * c.a_kv_rank : -1;
        case MI355_HW_L_CNORM: return L.is_latent() && !c.kv_from ? c.a_kv_rank : -1;
        case MI355_HW_D_CONV: if (L.is_ssd()) return (int64_t)L.ssd_channels() * c.d_conv;
                              return L.has_delta() ? (int64_t)L.conv_channels() * c.d_conv : -1;
        case MI355_HW_D_A_LOG: return L.has_delta() || L.is_ssd() ? c.d_heads : -1;
        case MI355_HW_D_DT_BIAS: if (L.is_ssd()) return c.d_heads;
                                 return L.has_delta() ? (c.d_decay_channels ? c.d_heads * c.d_dim : c.d_heads) : -1;
        case MI355_HW_D_NORM: if (L.is_ssd()) return L.ssd_inner();
                              return L.has_delta() ? c.d_vdim : -1;
        case MI355_HW_D_A2: return L.has_delta() && c.d_decay_channels ? (int64_t)c.d_heads * c.d_dim * c.d_a_rank : -1;
        case MI355_HW_D_G2: return L.has_delta() && c.d_gate == MI355_HYB_GATE_SIGMOID_LR ? (int64_t)c.d_heads * c.d_vdim * c.d_g_rank : -1;
        case MI355_HW_MLP_GATE_UP: if (c.mlp_kind == 3) return c.moe_shared_ff && !L.shared_merged() ? (int64_t)2 * c.moe_shared_ff * W : -1;
                                   if (c.mlp_kind == 4) return (int64_t)c.mlp_ff * W;
                                   return c.mlp_kind ? (int64_t)2 * c.mlp_ff * W : -1;
        case MI355_HW_MLP_DOWN: if (c.mlp_kind == 3) return c.moe_shared_ff && !L.shared_merged() ? (int64_t)W * c.moe_shared_ff : -1;
                                return c.mlp_kind ? (int64_t)W * c.mlp_ff : -1;
        default: return -1;
    }
}

Weight* slot_of(HModel* m, int layer, int which) {
    if (layer < 0) return which == MI355_HW_EMBED ? &m->embed : which == MI355_HW_FINAL_NORM ? &m->final_norm : which == MI355_HW_HEAD ? &m->head :
                          which == MI355_HW_SIDE_TABLE ? &m->side_table : nullptr;
    if (layer >= (int)m->layers.size() || which < MI355_HW_NORM1 || which >= MI355_HW_COUNT) return nullptr;
    return &m->layers[layer].w[which];
}

// device bf16 bits -> the slot's storage
int store_weight(HModel* m, int layer, int which, const uint16_t* dev_bits, int64_t n, int64_t stream) {
    Weight* w = slot_of(m, layer, which);
    if (!w || n != expected_elems(m, layer, which)) return -2;
    const bool as_bf16 = is_matrix(which) && m->bf16();
    drop_graphs(m);
    if (w->p) { (void)hipFree(w->p); w->p = nullptr; }
    HHIP(hipMalloc(&w->p, (size_t)n * (as_bf16 ? 2 : 4)));
    w->n = n;
    if (as_bf16) HHIP(hipMemcpyAsync(w->p, dev_bits, (size_t)n * 2, hipMemcpyDeviceToDevice, reinterpret_cast<hipStream_t>(stream)));
    else HCHECK(mi355_hyb_bf16_to_f32(static_cast<float*>(w->p), dev_bits, n, stream));
    return 0;
}

template <typename T> int grow(T*& p, size_t bytes) {
    if (p) (void)hipFree(p);
    p = nullptr;
    void* q = nullptr;
    const hipError_t e = hipMalloc(&q, bytes ? bytes : 16);
    if (e != hipSuccess) return (int)e;
    p = static_cast<T*>(q);
    return 0;
}

int ensure_capacity(HModel* m, int T, int n_out) {
    if (T > m->cap_t) {
        const size_t t = (size_t)T, W = (size_t)m->cfg.width;
        HHIP(hipDeviceSynchronize());
        drop_graphs(m);
        HCHECK(grow(m->x, t * W * 4));
        HCHECK(grow(m->proj, t * m->max_in_rows * 4));
        HCHECK(grow(m->aux1, t * (size_t)m->max_aux1 * 4));
        HCHECK(grow(m->aux2, t * (size_t)m->max_aux2 * 4));
        HCHECK(grow(m->conv, t * (size_t)m->max_conv * 4));
        HCHECK(grow(m->o, t * (size_t)m->max_o * 4));
        HCHECK(grow(m->prep, t * (size_t)m->max_prep * 4));
        HCHECK(grow(m->y, t * W * 4));
        HCHECK(grow(m->gu, t * (size_t)m->max_ff * 2 * 4));
        HCHECK(grow(m->xcopy, t * W * 2));
        HCHECK(grow(m->q, t * (size_t)m->max_q * m->esize()));
        HCHECK(grow(m->mix, t * (size_t)m->max_mix * m->esize()));
        HCHECK(grow(m->act, t * (size_t)m->max_ff * m->esize()));
        HCHECK(grow(m->att, t * (size_t)m->max_att * m->esize()));
        HCHECK(grow(m->tok_seq, t * 4));
        if (m->need_pre) HCHECK(grow(m->pre, t * W * m->esize()));
        if (m->cfg.residual_form == 3) HCHECK(grow(m->y2, t * W * 4));
        if (m->need_hf) HCHECK(grow(m->hf, t * W * 4));
        if (m->need_xs) HCHECK(grow(m->xs, (m->layers.size() + 1) * t * W * 4));
        if (m->max_side) { HCHECK(grow(m->side_g, t * (size_t)m->max_side * 4)); HCHECK(grow(m->side_a, t * (size_t)m->max_side * m->esize())); }
        if (m->max_q_rank) HCHECK(grow(m->cq, t * (size_t)m->max_q_rank * m->esize()));
        if (m->max_moe_experts) {
            const size_t pairs = t * m->max_moe_top, rows = pairs + (size_t)(m->max_moe_experts + 1) * MOE_MAX_BLOCK_ROWS;
            HCHECK(grow(m->moe_ids, pairs * 4));
            HCHECK(grow(m->moe_pos, pairs * 4));
            HCHECK(grow(m->moe_wts, pairs * 4));
            HCHECK(grow(m->moe_sgate, t * 4));
            HCHECK(grow(m->moe_row_token, rows * 4));
            HCHECK(grow(m->moe_table, (pairs / 16 + m->max_moe_experts + 2) * 2 * 4));
            HCHECK(grow(m->moe_gu, rows * 2 * m->max_moe_ff * 4));
            HCHECK(grow(m->moe_act, rows * m->max_moe_ff * m->esize()));
            HCHECK(grow(m->moe_y, rows * W * 4));
        }
        m->cap_t = T;
    }
    if (n_out > m->cap_out) {
        HHIP(hipDeviceSynchronize());
        drop_graphs(m);
        HCHECK(grow(m->xn, (size_t)n_out * m->cfg.width * m->esize()));
        m->cap_out = n_out;
    }
    return 0;
}

}  // namespace

extern "C" {

int32_t mi355_hybrid_in_proj_rows(const mi355_hybrid_layer* layer, int32_t* offsets) {
    int32_t off[P_COUNT];
    if (!layer) return -1;
    const int r = in_proj_parts(*layer, off);
    if (offsets) std::memcpy(offsets, off, sizeof(off));
    return r;
}

void* mi355_hybrid_create(const mi355_hybrid_config* cfg, const mi355_hybrid_layer* layers) {
    if (!cfg || !layers || cfg->width <= 0 || cfg->vocab <= 0 || cfg->n_layers <= 0 || cfg->block_size <= 0 || cfg->state_slots <= 0) return nullptr;
    if (cfg->dtype != MI355_DTYPE_F32 && cfg->dtype != MI355_DTYPE_BF16) return nullptr;
    for (int i = 0; i < cfg->n_layers; ++i) {
        if (!layer_ok(layers[i])) return nullptr;
        const int sw = layers[i].share_with;                   // the lender has weights of its own and the same shape
        if (sw && (sw > cfg->n_layers || sw - 1 == i || layers[sw - 1].share_with)) return nullptr;
        if (sw) {
            mi355_hybrid_layer a = layers[i], b = layers[sw - 1];
            a.share_with = b.share_with = 0;
            if (std::memcmp(&a, &b, sizeof(a)) != 0) return nullptr;
        }
    }
    if (cfg->embed_scale != 0.f && cfg->embed_scale != 1.f && cfg->residual_form < 2) return nullptr;     // forms 0 / 1 read a bf16 copy of x
    if (cfg->norm_kind < 0 || cfg->norm_kind > 1 || (cfg->norm_kind == 1 && cfg->residual_form != 3) || cfg->side_cols < 0 || cfg->logit_softcap < 0.f) return nullptr;
    for (int i = 0; i < cfg->n_layers; ++i) {
        const mi355_hybrid_layer& c = layers[i];
        if (c.side_dim && c.side_col + c.side_dim > cfg->side_cols) return nullptr;
        if (c.depth_terms && c.depth_terms != i + 2) return nullptr;
        if (c.mlp_kind == 4 && cfg->residual_form != 3) return nullptr;
        if (cfg->residual_form == 3 && (c.in_conv || c.share_with || c.moe_shared_ff || c.mlp_kind == 1 || c.mlp_kind == 2)) return nullptr;
        if (c.kv_from) {                                            // the lender: an earlier latent layer with pages of its own and the same row
            if (c.kv_from > i) return nullptr;
            const mi355_hybrid_layer& b = layers[c.kv_from - 1];
            if (b.mixer != MI355_HYB_MIX_LATENT || b.kv_from || b.a_kv_rank != c.a_kv_rank || b.a_rot_dim != c.a_rot_dim) return nullptr;
        }
    }
    if (cfg->residual_form < 0 || cfg->residual_form > 3 || cfg->norm_groups < 0 || (cfg->norm_groups > 1 && cfg->width % cfg->norm_groups)) return nullptr;
    for (int i = 0; i < cfg->n_layers; ++i)                        // the experts' outputs are combined in front of an output norm
        if (layers[i].mlp_kind == 3 && (cfg->residual_form == 1 || (cfg->residual_form != 3 && cfg->width > 4096))) return nullptr;
    HModel* m = new HModel();
    m->cfg = *cfg;
    m->need_pre = cfg->residual_form == 2 || cfg->residual_form == 3;
    m->layers.resize(cfg->n_layers);
    int64_t off = 0;
    for (int i = 0; i < cfg->n_layers; ++i) {
        HLayer& L = m->layers[i];
        L.c = layers[i];
        const mi355_hybrid_layer& c = L.c;
        L.in_rows = in_proj_parts(c, L.off);
        L.out_k = 0;
        if (L.uses_pages()) L.out_k += c.a_heads * c.a_vdim;
        if (L.has_delta()) L.out_k += c.d_heads * c.d_vdim;
        if (c.mixer == MI355_HYB_MIX_MINGRU) L.out_k = c.g_width;
        m->max_in_rows = std::max(m->max_in_rows, L.in_rows);
        m->max_mix = std::max(m->max_mix, L.out_k);
        if (L.has_attn() || L.is_conv_attn()) m->max_q = std::max(m->max_q, c.a_heads * c.a_dim);
        if (L.is_ssd()) {
            L.out_k = L.ssd_inner();
            m->max_mix = std::max(m->max_mix, L.out_k);
            m->max_conv = std::max(m->max_conv, L.ssd_channels());
            m->max_o = std::max(m->max_o, L.ssd_inner());
            L.conv_off = off; off += (int64_t)L.ssd_channels() * (c.d_conv - 1);
            L.state_off = off; off += (int64_t)c.d_heads * c.d_dim * c.d_vdim;
        }
        if (c.side_dim) m->max_side = std::max(m->max_side, c.side_dim);
        if (c.depth_terms) m->need_xs = true;
        if (c.mlp_kind == 3 && cfg->residual_form == 3 && cfg->dtype == MI355_DTYPE_BF16) m->need_hf = true;
        if (L.is_latent() && c.a_q_rank) {
            m->max_q_rank = std::max(m->max_q_rank, c.a_q_rank);
            m->max_aux2 = std::max(m->max_aux2, c.a_heads * (c.a_dim + c.a_rot_dim));
        }
        if (L.is_latent()) {
            m->max_q = std::max(m->max_q, c.a_heads * (c.a_kv_rank + c.a_rot_dim));
            m->max_aux1 = std::max(m->max_aux1, c.a_heads * c.a_kv_rank);
            m->max_att = std::max(m->max_att, c.a_heads * c.a_kv_rank);
            m->max_o = std::max(m->max_o, c.a_heads * c.a_vdim);
        }
        if (L.is_conv_attn()) {
            m->max_conv = std::max(m->max_conv, L.a_conv_channels());
            m->max_o = std::max(m->max_o, c.a_heads * (c.a_talk ? c.a_kv_heads : 1) * c.a_vdim);
            L.conv_off = off; off += (int64_t)L.a_conv_channels() * (c.a_conv - 1);
        }
        if (L.has_delta()) {
            if (c.d_decay_channels) m->max_aux1 = std::max(m->max_aux1, c.d_heads * c.d_dim);
            if (c.d_gate == MI355_HYB_GATE_SIGMOID_LR) m->max_aux2 = std::max(m->max_aux2, c.d_heads * c.d_vdim);
            m->max_conv = std::max(m->max_conv, L.conv_channels());
            m->max_o = std::max(m->max_o, c.d_heads * c.d_vdim);
            m->max_prep = std::max(m->max_prep, 2 * c.d_kv_heads * c.d_dim + c.d_heads * (c.d_decay_channels ? c.d_dim : 1) + c.d_heads);
            L.conv_off = off; off += (int64_t)L.conv_channels() * (c.d_conv - 1);
            L.state_off = off; off += (int64_t)c.d_heads * c.d_dim * c.d_vdim;
        }
        if (c.mixer == MI355_HYB_MIX_MINGRU) { L.state_off = off; off += c.g_width; }
        if (c.in_conv) { L.in_conv_off = off; off += (int64_t)cfg->width * (c.in_conv - 1); m->need_pre = true; }
        if (c.mlp_kind == 3) {
            m->max_moe_experts = std::max(m->max_moe_experts, c.moe_experts + 1);
            m->max_moe_top = std::max(m->max_moe_top, c.moe_top + 1);
            m->max_moe_ff = std::max(m->max_moe_ff, c.mlp_ff);
            m->max_ff = std::max(m->max_ff, c.moe_shared_ff);
        } else if (c.mlp_kind) m->max_ff = std::max(m->max_ff, c.mlp_ff);
    }
    m->slot_floats = std::max<int64_t>(off, 1);
    return m;
}

void mi355_hybrid_destroy(void* mp) {
    HModel* m = static_cast<HModel*>(mp);
    if (!m) return;
    (void)hipDeviceSynchronize();
    drop_graphs(m);
    for (HLayer& L : m->layers) {
        for (Weight& w : L.w) if (w.p) (void)hipFree(w.p);
        for (void* p : {(void*)L.cos_t, (void*)L.sin_t, L.owns_pages() ? L.k_pages : nullptr, L.owns_pages() ? L.v_pages : nullptr}) if (p) (void)hipFree(p);
    }
    for (void* p : {m->embed.p, m->final_norm.p, m->head.p, (void*)m->state, (void*)m->prep, (void*)m->x, (void*)m->proj, (void*)m->aux1, (void*)m->aux2,
                    (void*)m->conv, (void*)m->o, (void*)m->y, (void*)m->gu, m->xcopy, m->q, m->mix, m->act, m->xn, m->att, (void*)m->tok_seq,
                    m->pre, m->moe_act, (void*)m->y2, (void*)m->hf, (void*)m->xs, (void*)m->side_g, m->side_a, m->cq, m->side_table.p, (void*)m->moe_gu, (void*)m->moe_y, (void*)m->moe_wts, (void*)m->moe_sgate, (void*)m->moe_ids,
                    (void*)m->moe_pos, (void*)m->moe_row_token, (void*)m->moe_table})
        if (p) (void)hipFree(p);
    delete m;
}

int mi355_hybrid_set_weight(void* mp, int32_t layer, int32_t which, const uint16_t* host_bf16, int64_t n) {
    HModel* m = static_cast<HModel*>(mp);
    if (!m || !host_bf16 || n <= 0) return -1;
    if (n != expected_elems(m, layer, which)) return -2;
    uint16_t* tmp = nullptr;
    HHIP(hipMalloc(reinterpret_cast<void**>(&tmp), (size_t)n * 2));
    int rc = (int)hipMemcpy(tmp, host_bf16, (size_t)n * 2, hipMemcpyHostToDevice);
    if (rc == 0) rc = store_weight(m, layer, which, tmp, n, 0);
    if (rc == 0) rc = (int)hipDeviceSynchronize();
    (void)hipFree(tmp);
    return rc;
}

int mi355_hybrid_set_weight_dev(void* mp, int32_t layer, int32_t which, const uint16_t* dev_bf16, int64_t n, int64_t stream) {
    HModel* m = static_cast<HModel*>(mp);
    if (!m || !dev_bf16 || n <= 0) return -1;
    return store_weight(m, layer, which, dev_bf16, n, stream);
}

int mi355_hybrid_set_rope_tables(void* mp, int32_t layer, const float* cos_t, const float* sin_t, int32_t n_positions) {
    HModel* m = static_cast<HModel*>(mp);
    if (!m || layer < 0 || layer >= (int)m->layers.size() || !cos_t || !sin_t || n_positions <= 0) return -1;
    HLayer& L = m->layers[layer];
    if (!L.rotates() || L.c.share_with) return -2;
    drop_graphs(m);
    const size_t bytes = (size_t)n_positions * (L.c.a_rot_dims / 2) * 4;
    HHIP(hipDeviceSynchronize());
    HCHECK(grow(L.cos_t, bytes));
    HCHECK(grow(L.sin_t, bytes));
    HHIP(hipMemcpy(L.cos_t, cos_t, bytes, hipMemcpyHostToDevice));
    HHIP(hipMemcpy(L.sin_t, sin_t, bytes, hipMemcpyHostToDevice));
    L.n_pos = n_positions;
    return 0;
}

int64_t mi355_hybrid_state_floats_per_slot(void* mp) { return mp ? static_cast<HModel*>(mp)->slot_floats : -1; }
void* mi355_hybrid_state_ptr(void* mp) { return mp ? static_cast<HModel*>(mp)->state : nullptr; }

int64_t mi355_hybrid_cache_bytes(void* mp, int32_t num_blocks) {
    HModel* m = static_cast<HModel*>(mp);
    if (!m || num_blocks < 0) return -1;
    int64_t b = m->slot_floats * 4 * m->cfg.state_slots;
    for (const HLayer& L : m->layers)
        if (L.owns_pages()) b += (int64_t)num_blocks * m->cfg.block_size * (L.k_row() + L.v_row()) * (int64_t)m->esize();
    return b;
}

int mi355_hybrid_alloc_cache(void* mp, int32_t num_blocks) {
    HModel* m = static_cast<HModel*>(mp);
    if (!m || num_blocks <= 0) return -1;
    HHIP(hipDeviceSynchronize());
    drop_graphs(m);
    for (HLayer& L : m->layers) {
        if (!L.owns_pages()) continue;
        const size_t rows = (size_t)num_blocks * m->cfg.block_size;
        HCHECK(grow(L.k_pages, rows * L.k_row() * m->esize()));
        HHIP(hipMemset(L.k_pages, 0, rows * L.k_row() * m->esize()));
        if (L.v_row() > 0) {
            HCHECK(grow(L.v_pages, rows * L.v_row() * m->esize()));
            HHIP(hipMemset(L.v_pages, 0, rows * L.v_row() * m->esize()));
        }
    }
    for (HLayer& L : m->layers) if (L.c.kv_from) L.k_pages = m->layers[L.c.kv_from - 1].k_pages;
    const size_t sb = (size_t)m->slot_floats * 4 * m->cfg.state_slots;
    HCHECK(grow(m->state, sb));
    HHIP(hipMemset(m->state, 0, sb));
    HHIP(hipDeviceSynchronize());
    m->num_blocks = num_blocks;
    return 0;
}

static int forward_check(HModel* m, const uint32_t* tokens, const int64_t* positions, const int64_t* slot_mapping,
                         const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                         const int32_t* state_slots, const int32_t* out_rows, int32_t n_out, int32_t num_seqs, int32_t T,
                         int32_t max_blocks, int32_t max_context_len, float* logits) {
    if (!m || !tokens || !positions || !slot_mapping || !block_tables || !context_lens || !cu_seqlens_q || !state_slots) return -1;
    if (num_seqs <= 0 || T <= 0 || n_out < 0 || (n_out > 0 && (!out_rows || !logits)) || max_blocks <= 0) return -1;
    if (!m->state || !m->embed.p || !m->final_norm.p || (!m->head.p && !m->cfg.tie_head) || (m->cfg.side_cols > 0 && !m->side_table.p)) return -3;
    if ((int64_t)max_blocks * m->cfg.block_size < max_context_len) return -4;
    for (const HLayer& L : m->layers) {
        const HLayer& WL = L.c.share_with ? m->layers[L.c.share_with - 1] : L;
        if (!L.c.share_with) {
            const int need[] = {MI355_HW_NORM1, MI355_HW_IN_PROJ, MI355_HW_OUT_PROJ};
            for (int s : need) if (!L.w[s].p) return -3;
            for (int s = MI355_HW_NORM2; s < MI355_HW_COUNT; ++s)
                if (s != MI355_HW_IN_BIAS && s != MI355_HW_MOE_CORRECTION && s != MI355_HW_CONV_BIAS && expected_elems(m, (int)(&L - m->layers.data()), s) > 0 && !L.w[s].p) return -3;
        }
        if (L.uses_pages() && (!L.k_pages || (L.rotates() && WL.n_pos < max_context_len))) return -4;
    }
    return ensure_capacity(m, T, n_out);
}

static int forward_enqueue(HModel* m, const uint32_t* tokens, const int64_t* positions, const int64_t* slot_mapping,
                           const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                           const int32_t* state_slots, const int32_t* out_rows, int32_t n_out, int32_t num_seqs, int32_t T,
                           int32_t max_blocks, float* logits, float* layer_trace, int64_t stream) {
    const int W = m->cfg.width, dt = m->cfg.dtype;
    const float eps = m->cfg.norm_eps;
    const bool bf = m->bf16();
    const bool sandwich = m->cfg.residual_form == 2;                // a norm in front of every sublayer: nothing reads a copy of x
    const bool parallel = m->cfg.residual_form == 3;                // one norm per layer, both sublayers read it
    void* xcopy = (bf && !sandwich && !parallel) ? m->xcopy : nullptr;
    void* xin = (sandwich || parallel) ? m->pre : (bf ? m->xcopy : (void*)m->x);  // what the sublayers' first product reads
    const int xin_dt = bf ? MI355_DTYPE_BF16 : MI355_DTYPE_F32;
    const int64_t TW = (int64_t)T * W;
    HCHECK(mi355_hyb_token_seq(m->tok_seq, cu_seqlens_q, num_seqs, stream));
    if (m->cfg.embed_scale != 0.f && m->cfg.embed_scale != 1.f)
        HCHECK(mi355_hyb_embed_scaled(m->x, m->embed.p, tokens, T, W, m->cfg.vocab, m->cfg.embed_scale, dt, stream));
    else
        HCHECK(mi355_hyb_embed(m->x, xcopy, m->embed.p, tokens, T, W, m->cfg.vocab, dt, stream));
    if (m->need_xs) HCHECK(mi355_hyb_copy_f32(m->xs, m->x, TW, stream));         // X_0 of the depth average
    for (size_t li = 0; li < m->layers.size(); ++li) {
        HLayer& L = m->layers[li];
        const mi355_hybrid_layer& c = L.c;
        const HLayer& WL = c.share_with ? m->layers[c.share_with - 1] : L;          // whose weights (and rope tables) the layer runs on
        auto f = [&](int which) { return static_cast<const float*>(WL.w[which].p); };
        const int ldp = L.in_rows;
        const void* min_ = xin;                                         // the mixer's input
        if (c.in_conv) {
            // h + conv(h): h = the normed x (form 2) or x itself.  Up to 8 taps: norm, convolution (and, when every sequence brings one
            // token, the move of the slot's rows) are one launch; else the normed rows go through m->y (free until the output projection)
            float* cst = m->state + L.in_conv_off;
            const float* nw = sandwich ? f(MI355_HW_PRE_NORM1) : nullptr;
            if (c.in_conv <= 8) {
                const int self_update = T == num_seqs;
                HCHECK(mi355_hyb_norm_conv(m->pre, dt, (sandwich && !self_update) ? m->y : nullptr, m->x, nw, f(MI355_HW_IN_CONV), cst, m->slot_floats,
                                           context_lens, cu_seqlens_q, state_slots, m->tok_seq, num_seqs, T, W, c.in_conv, self_update, eps, stream));
                if (!self_update)
                    HCHECK(mi355_hyb_conv_state_update(cst, m->slot_floats, sandwich ? m->y : m->x, W, 0, context_lens, cu_seqlens_q, state_slots,
                                                       num_seqs, W, c.in_conv, stream));
            } else {
                const float* h = m->x;
                if (sandwich) { HCHECK(mi355_hyb_pre_norm(m->y, MI355_DTYPE_F32, m->x, nw, T, W, eps, stream)); h = m->y; }
                HCHECK(mi355_hyb_conv_residual(m->pre, dt, h, W, 0, f(MI355_HW_IN_CONV), cst, m->slot_floats, context_lens, cu_seqlens_q,
                                               state_slots, m->tok_seq, num_seqs, T, W, c.in_conv, stream));
                HCHECK(mi355_hyb_conv_state_update(cst, m->slot_floats, h, W, 0, context_lens, cu_seqlens_q, state_slots, num_seqs, W, c.in_conv,
                                                   stream));
            }
            min_ = m->pre;
        } else if (sandwich) {
            HCHECK(mi355_hyb_pre_norm(m->pre, dt, m->x, f(MI355_HW_PRE_NORM1), T, W, eps, stream));
        } else if (parallel && li == 0) {                              // (the router wants the norm's output in f32; the later layers'
                                                                       //  norms are made at the end of the layer before them)
            HCHECK(mi355_hyb_pre_norm_ex(m->pre, dt, (c.mlp_kind == 3 && bf) ? m->hf : nullptr, m->x, W, f(MI355_HW_NORM1), T, W, m->cfg.norm_kind,
                                         eps, stream));
        }
        HCHECK(mi355_hyb_linear(m->proj, ldp, min_, xin_dt, W, WL.w[MI355_HW_IN_PROJ].p, f(MI355_HW_IN_BIAS), T, L.in_rows, W, dt, stream));
        int mix_col = 0;
        if (L.has_attn()) {
            const int norm_mode = c.a_qk_norm ? (c.a_norm_after_rot ? 2 : 1) : 0;
            HCHECK(mi355_hyb_attn_prepare_ex(m->q, L.k_pages, L.v_pages, m->proj, ldp, L.off[P_AQ], L.off[P_AK], L.off[P_AV],
                                             norm_mode == 1 ? f(MI355_HW_A_QNORM) : nullptr, norm_mode == 1 ? f(MI355_HW_A_KNORM) : nullptr,
                                             WL.cos_t, WL.sin_t, positions, slot_mapping, T, c.a_heads, c.a_kv_heads, c.a_dim, c.a_vdim,
                                             c.a_rot_dims, c.a_rot_interleaved, norm_mode, c.a_head_temp ? f(MI355_HW_A_TEMP) : nullptr, eps,
                                             dt, stream));
            HCHECK(mi355_hyb_masked_attention(m->mix, dt, L.out_k, 0, m->q, L.k_pages, L.v_pages, block_tables, context_lens, cu_seqlens_q,
                                              m->tok_seq, c.a_has_sink ? f(MI355_HW_A_SINK) : nullptr, num_seqs, T, c.a_heads,
                                              c.a_kv_heads, c.a_dim, c.a_vdim, m->cfg.block_size, max_blocks, c.a_window, c.a_keep_first,
                                              c.a_scale, c.mixer == MI355_HYB_MIX_PARALLEL ? c.a_out_scale : 1.f, 0, 0, 0.f, 0, dt, stream));
            mix_col = c.a_heads * c.a_vdim;
        }
        if (L.is_latent()) {
            // absorbed form: q_abs[t, h] = W_uk,h^T q_h (one launch over the heads), attention over the latent rows themselves with
            // ONE shared key/value head (keys [latent | rotated part], values = the latent part of the same page row), then W_uv,h
            // on every head's latent-sized output, the head gate, and the output projection
            // (queries through a latent: the q part of the projection is W_dq h; its RMS norm, then W_uq gives the heads' rows)
            const int R = c.a_kv_rank, dq = R + c.a_rot_dim, H = c.a_heads;
            const float* qsrc = m->proj;
            int ldq = ldp, q_off = L.off[P_AQ];
            if (c.a_q_rank) {
                HCHECK(mi355_hyb_pre_norm_ex(m->cq, dt, nullptr, m->proj + L.off[P_AQ], ldp, f(MI355_HW_L_QNORM), T, c.a_q_rank, 0, eps, stream));
                ldq = H * (c.a_dim + c.a_rot_dim); q_off = 0; qsrc = m->aux2;
                HCHECK(mi355_hyb_linear(m->aux2, ldq, m->cq, dt, c.a_q_rank, WL.w[MI355_HW_L_UQ].p, nullptr, T, ldq, c.a_q_rank, dt, stream));
            }
            HCHECK(mi355_hyb_linear_batched(m->aux1, H * R, R, qsrc + q_off, MI355_DTYPE_F32, ldq, c.a_dim + c.a_rot_dim,
                                            WL.w[MI355_HW_L_UKT].p, (int64_t)R * c.a_dim, T, R, c.a_dim, H, dt, stream));
            HCHECK(mi355_hyb_latent_prepare_ex(m->q, c.kv_from ? nullptr : L.k_pages, qsrc, ldq, q_off, m->proj, ldp, c.kv_from ? 0 : L.off[P_AK],
                                               m->aux1, c.kv_from ? nullptr : f(MI355_HW_L_CNORM), WL.cos_t, WL.sin_t, positions, slot_mapping, T, H,
                                               c.a_dim, c.a_rot_dim, R, c.a_rot_dims, c.a_rot_interleaved, eps, dt, stream));
            HCHECK(mi355_hyb_window_attention_ex(m->att, dt, H * R, 0, m->q, L.k_pages, L.k_pages, block_tables, context_lens, cu_seqlens_q,
                                                 m->tok_seq, c.a_has_sink ? f(MI355_HW_A_SINK) : nullptr, num_seqs, T, H, 1, dq, R,
                                                 m->cfg.block_size, max_blocks, c.a_window, c.a_scale, 1.f, dq, dq, c.a_softcap, 0, dt, stream));
            HCHECK(mi355_hyb_linear_batched(m->o, H * c.a_vdim, c.a_vdim, m->att, dt, H * R, R, WL.w[MI355_HW_L_UV].p,
                                            (int64_t)c.a_vdim * R, T, c.a_vdim, R, H, dt, stream));
            if (c.a_out_gate) HCHECK(mi355_hyb_elem_gate(m->mix, dt, m->o, m->proj + L.off[P_G], ldp, T, H * c.a_vdim, stream));
            else if (c.a_head_gate) HCHECK(mi355_hyb_head_gate(m->mix, dt, m->o, m->proj + L.off[P_G], ldp, T, H, c.a_vdim, stream));
            else HCHECK(mi355_hyb_head_gate(m->mix, dt, m->o, nullptr, 0, T, H, c.a_vdim, stream));
        }
        if (L.is_conv_attn()) {
            const int C = L.a_conv_channels(), H = c.a_heads, G = c.a_kv_heads;
            float* conv_state = m->state + L.conv_off;
            HCHECK(mi355_hyb_conv(m->conv, m->proj, ldp, L.off[P_AQ], f(MI355_HW_A_CONV), conv_state, m->slot_floats, context_lens,
                                  cu_seqlens_q, state_slots, m->tok_seq, num_seqs, T, C, c.a_conv, 0, stream));
            HCHECK(mi355_hyb_conv_state_update(conv_state, m->slot_floats, m->proj, ldp, L.off[P_AQ], context_lens, cu_seqlens_q,
                                               state_slots, num_seqs, C, c.a_conv, stream));
            HCHECK(mi355_hyb_attn_prepare_whole(m->q, L.k_pages, L.v_pages, m->conv, C, 0, H * c.a_dim, (H + G) * c.a_dim,
                                                c.a_qk_norm ? f(MI355_HW_A_QNORM) : nullptr, c.a_qk_norm ? f(MI355_HW_A_KNORM) : nullptr,
                                                slot_mapping, T, H, G, c.a_dim, c.a_vdim, c.a_v_unit, eps, dt, stream));
            if (c.a_talk) {
                // mixed head weights: every head's weights against the values of every key/value head, then the mix of those outputs
                HCHECK(mi355_hyb_window_attention_ex(m->o, MI355_DTYPE_F32, H * G * c.a_vdim, 0, m->q, L.k_pages, L.v_pages, block_tables,
                                                     context_lens, cu_seqlens_q, m->tok_seq, c.a_has_sink ? f(MI355_HW_A_SINK) : nullptr,
                                                     num_seqs, T, H, G, c.a_dim, c.a_vdim, m->cfg.block_size, max_blocks, c.a_window,
                                                     c.a_scale, 1.f, 0, 0, c.a_softcap, 1, dt, stream));
                HCHECK(mi355_hyb_head_mix(m->mix, dt, m->o, f(MI355_HW_A_TALK), T, H, G, c.a_vdim, stream));
            } else {
                HCHECK(mi355_hyb_biased_attention(m->mix, dt, L.out_k, 0, m->q, L.k_pages, L.v_pages, block_tables, context_lens,
                                                  cu_seqlens_q, m->tok_seq, c.a_has_sink ? f(MI355_HW_A_SINK) : nullptr,
                                                  c.a_dist_bias ? f(MI355_HW_A_DIST) : nullptr, num_seqs, T, H, G, c.a_dim, c.a_vdim,
                                                  m->cfg.block_size, max_blocks, c.a_window, 0, c.a_scale, 1.f, 0, 0, c.a_softcap, 0, dt, stream));
            }
        }
        if (L.is_ssd()) {
            // x | B | C through the convolution (bias, silu), the scan over the state slot, then the gate, the group norm and W_o
            const int C = L.ssd_channels();
            float* conv_state = m->state + L.conv_off;
            HCHECK(mi355_hyb_conv_bias(m->conv, m->proj, ldp, L.off[P_DV], f(MI355_HW_D_CONV), f(MI355_HW_CONV_BIAS), conv_state, m->slot_floats,
                                       context_lens, cu_seqlens_q, state_slots, m->tok_seq, num_seqs, T, C, c.d_conv, 1, stream));
            HCHECK(mi355_hyb_conv_state_update(conv_state, m->slot_floats, m->proj, ldp, L.off[P_DV], context_lens, cu_seqlens_q, state_slots,
                                               num_seqs, C, c.d_conv, stream));
            HCHECK(mi355_hyb_ssd_scan(m->o, m->state + L.state_off, m->slot_floats, m->conv, C, m->proj + L.off[P_A], ldp, f(MI355_HW_D_A_LOG),
                                      f(MI355_HW_D_DT_BIAS), f(MI355_HW_D_SKIP), context_lens, cu_seqlens_q, state_slots, num_seqs, T, c.d_heads,
                                      c.d_kv_heads, c.d_dim, c.d_vdim, stream));
            HCHECK(mi355_hyb_gate_group_norm(m->mix, dt, m->o, m->proj + L.off[P_G], ldp, f(MI355_HW_D_NORM), T, L.ssd_inner(), c.d_norm_groups,
                                             eps, stream));
        }
        if (L.has_delta()) {
            const int C = L.conv_channels();
            float* conv_state = m->state + L.conv_off;
            HCHECK(mi355_hyb_conv_silu(m->conv, m->proj, ldp, L.off[P_DQ], f(MI355_HW_D_CONV), conv_state, m->slot_floats, context_lens,
                                       cu_seqlens_q, state_slots, m->tok_seq, num_seqs, T, C, c.d_conv, stream));
            HCHECK(mi355_hyb_conv_state_update(conv_state, m->slot_floats, m->proj, ldp, L.off[P_DQ], context_lens, cu_seqlens_q,
                                               state_slots, num_seqs, C, c.d_conv, stream));
            const float* decay_in = m->proj + L.off[P_A];
            int ldd = ldp;
            if (c.d_decay_channels) {
                HCHECK(mi355_hyb_linear(m->aux1, c.d_heads * c.d_dim, m->proj + L.off[P_A], MI355_DTYPE_F32, ldp, WL.w[MI355_HW_D_A2].p,
                                        nullptr, T, c.d_heads * c.d_dim, c.d_a_rank, dt, stream));
                decay_in = m->aux1; ldd = c.d_heads * c.d_dim;
            }
            const float* gate_in = m->proj + L.off[P_G];
            int ldg = ldp;
            if (c.d_gate == MI355_HYB_GATE_SIGMOID_LR) {
                HCHECK(mi355_hyb_linear(m->aux2, c.d_heads * c.d_vdim, m->proj + L.off[P_G], MI355_DTYPE_F32, ldp, WL.w[MI355_HW_D_G2].p,
                                        nullptr, T, c.d_heads * c.d_vdim, c.d_g_rank, dt, stream));
                gate_in = m->aux2; ldg = c.d_heads * c.d_vdim;
            }
            HCHECK(mi355_hyb_delta_rule(m->o, m->state + L.state_off, m->slot_floats, m->conv, C, m->proj, ldp, L.off[P_B], decay_in, ldd,
                                        c.d_decay_channels, f(MI355_HW_D_A_LOG), f(MI355_HW_D_DT_BIAS), context_lens, cu_seqlens_q,
                                        state_slots, num_seqs, T, c.d_heads, c.d_kv_heads, c.d_dim, c.d_vdim, m->cfg.unit_eps, m->prep, stream));
            HCHECK(mi355_hyb_gated_norm(m->mix, dt, L.out_k, mix_col, m->o, f(MI355_HW_D_NORM), gate_in, ldg, c.d_gate, T, c.d_heads,
                                        c.d_vdim, eps, c.mixer == MI355_HYB_MIX_PARALLEL ? c.d_out_scale : 1.f, stream));
        }
        if (c.mixer == MI355_HYB_MIX_MINGRU)
            HCHECK(mi355_hyb_mingru(m->mix, dt, m->state + L.state_off, m->slot_floats, m->proj, ldp, L.off[0], L.off[1], L.off[2],
                                    context_lens, cu_seqlens_q, state_slots, num_seqs, T, c.g_width, stream));
        auto residual = [&](int norm_slot) -> int {
            if (m->cfg.residual_form == 1)
                return mi355_hyb_resid_norm(m->x, xcopy, m->y, W, f(norm_slot), T, W, m->cfg.norm_groups, m->cfg.resid_alpha, eps, stream);
            return mi355_hyb_norm_add(m->x, xcopy, m->y, W, f(norm_slot), T, W, eps, stream);
        };
        HCHECK(mi355_hyb_linear(m->y, W, m->mix, dt, L.out_k, WL.w[MI355_HW_OUT_PROJ].p, nullptr, T, W, L.out_k, dt, stream));
        if (parallel) {
            // x <- x + mixer(h) + ff(h): the feed-forward reads the same h (m->pre) the mixer's projections read
            if (c.mlp_kind == 3) {
                const int E = c.moe_experts, K = c.moe_top, ff = c.mlp_ff, pairs = T * K;
                HCHECK(mi355_hyb_moe_route_ex(m->moe_ids, m->moe_wts, nullptr, nullptr, dt, bf ? m->hf : static_cast<const float*>(m->pre), nullptr,
                                              f(MI355_HW_MOE_ROUTER), f(MI355_HW_MOE_CORRECTION), nullptr, T, W, E, K,
                                              c.moe_scale != 0.f ? c.moe_scale : 1.f, eps, 0, c.moe_sigmoid, c.moe_groups, c.moe_keep_groups,
                                              c.moe_normalise, stream));
                const int bm = std::min(mi355_hyb_moe_block_rows(pairs, E, 2 * ff, W, dt), mi355_hyb_moe_block_rows(pairs, E, W, ff, dt));
                const int nb = (pairs + bm - 1) / bm + E;
                HCHECK(mi355_hyb_moe_group(m->moe_pos, m->moe_row_token, m->moe_table, m->moe_ids, pairs, K, E, bm, nb, stream));
                HCHECK(mi355_hyb_linear_grouped(m->moe_gu, 2 * ff, xin, xin_dt, W, m->moe_row_token, WL.w[MI355_HW_MOE_GATE_UP].p, (int64_t)2 * ff * W,
                                                m->moe_table, bm, nb, 2 * ff, W, dt, stream));
                HCHECK(mi355_hyb_silu_glu(m->moe_act, dt, m->moe_gu, nb * bm, ff, m->moe_table, bm, stream));
                HCHECK(mi355_hyb_linear_grouped(m->moe_y, W, m->moe_act, dt, ff, nullptr, WL.w[MI355_HW_MOE_DOWN].p, (int64_t)W * ff, m->moe_table, bm,
                                                nb, W, ff, dt, stream));
                HCHECK(mi355_hyb_moe_combine_add(m->x, m->y, m->moe_y, m->moe_pos, m->moe_wts, T, W, K, stream));
            } else if (c.mlp_kind == 4) {
                HCHECK(mi355_hyb_linear(m->gu, c.mlp_ff, xin, xin_dt, W, WL.w[MI355_HW_MLP_GATE_UP].p, nullptr, T, c.mlp_ff, W, dt, stream));
                HCHECK(mi355_hyb_relu2(m->act, dt, m->gu, (int64_t)T * c.mlp_ff, stream));
                HCHECK(mi355_hyb_linear(m->y2, W, m->act, dt, c.mlp_ff, WL.w[MI355_HW_MLP_DOWN].p, nullptr, T, W, c.mlp_ff, dt, stream));
                HCHECK(mi355_hyb_add2(m->x, m->y, m->y2, TW, stream));
            } else {
                HCHECK(mi355_hyb_add2(m->x, m->y, nullptr, TW, stream));
            }
        } else {
        HCHECK(residual(MI355_HW_NORM1));
        if (c.mlp_kind == 3) {
            // mixture of experts: route (with the norm in front of it in form 2), group the (token, expert) pairs into whole blocks per
            // expert, one grouped product for all gate/up matrices, silu, one for all down matrices; the shared expert as one more
            // group of every token (when it has the experts' size) or as dense products; the weighted sum, the shared expert's gate and
            // the output norm in one launch
            const bool merged = L.shared_merged();
            const int E = c.moe_experts + merged, K = c.moe_top + merged, ff = c.mlp_ff, fs = merged ? 0 : c.moe_shared_ff, pairs = T * K;
            const float* router = f(MI355_HW_MOE_ROUTER);
            HCHECK(mi355_hyb_moe_route(m->moe_ids, m->moe_wts, m->moe_sgate, sandwich ? m->pre : nullptr, dt, m->x,
                                       sandwich ? f(MI355_HW_PRE_NORM2) : nullptr, router, f(MI355_HW_MOE_CORRECTION),
                                       c.moe_shared_ff ? router + (size_t)c.moe_experts * W : nullptr, T, W, c.moe_experts, c.moe_top, c.moe_scale,
                                       eps, merged, stream));
            const int bm = std::min(mi355_hyb_moe_block_rows(pairs, E, 2 * ff, W, dt), mi355_hyb_moe_block_rows(pairs, E, W, ff, dt));
            const int nb = (pairs + bm - 1) / bm + E;
            HCHECK(mi355_hyb_moe_group(m->moe_pos, m->moe_row_token, m->moe_table, m->moe_ids, pairs, K, E, bm, nb, stream));
            HCHECK(mi355_hyb_linear_grouped(m->moe_gu, 2 * ff, xin, xin_dt, W, m->moe_row_token, WL.w[MI355_HW_MOE_GATE_UP].p, (int64_t)2 * ff * W,
                                            m->moe_table, bm, nb, 2 * ff, W, dt, stream));
            HCHECK(mi355_hyb_silu_glu(m->moe_act, dt, m->moe_gu, nb * bm, ff, m->moe_table, bm, stream));
            HCHECK(mi355_hyb_linear_grouped(m->moe_y, W, m->moe_act, dt, ff, nullptr, WL.w[MI355_HW_MOE_DOWN].p, (int64_t)W * ff, m->moe_table, bm,
                                            nb, W, ff, dt, stream));
            if (fs) {
                HCHECK(mi355_hyb_linear(m->gu, 2 * fs, xin, xin_dt, W, WL.w[MI355_HW_MLP_GATE_UP].p, nullptr, T, 2 * fs, W, dt, stream));
                HCHECK(mi355_hyb_silu_glu(m->act, dt, m->gu, T, fs, nullptr, 0, stream));
                HCHECK(mi355_hyb_linear(m->y, W, m->act, dt, fs, WL.w[MI355_HW_MLP_DOWN].p, nullptr, T, W, fs, dt, stream));
            }
            HCHECK(mi355_hyb_moe_combine_norm_add(m->x, xcopy, m->moe_y, m->moe_pos, m->moe_wts, fs ? m->y : nullptr, fs ? m->moe_sgate : nullptr,
                                                  f(MI355_HW_NORM2), T, W, K, eps, stream));
        } else if (c.mlp_kind) {
            if (sandwich) HCHECK(mi355_hyb_pre_norm(m->pre, dt, m->x, f(MI355_HW_PRE_NORM2), T, W, eps, stream));
            HCHECK(mi355_hyb_linear(m->gu, 2 * c.mlp_ff, xin, xin_dt, W, WL.w[MI355_HW_MLP_GATE_UP].p, nullptr, T, 2 * c.mlp_ff, W, dt, stream));
            if (c.mlp_kind == 2) HCHECK(mi355_hyb_gelu_glu(m->act, dt, m->gu, T, c.mlp_ff, stream));
            else HCHECK(mi355_hyb_clamped_glu(m->act, dt, m->gu, T, c.mlp_ff, c.mlp_limit, c.mlp_alpha, stream));
            HCHECK(mi355_hyb_linear(m->y, W, m->act, dt, c.mlp_ff, WL.w[MI355_HW_MLP_DOWN].p, nullptr, T, W, c.mlp_ff, dt, stream));
            HCHECK(residual(MI355_HW_NORM2));
        }
        }
        if (c.side_dim) {
            // the token's own input to this layer: x <- x + RMSnorm(W_proj (gelu_tanh(W_gate x) * e)) w, e = the token's columns of the side table
            HCHECK(mi355_hyb_linear(m->side_g, c.side_dim, m->x, MI355_DTYPE_F32, W, WL.w[MI355_HW_SIDE_GATE].p, nullptr, T, c.side_dim, W, dt, stream));
            HCHECK(mi355_hyb_side_act(m->side_a, dt, m->side_g, m->side_table.p, m->cfg.side_cols, c.side_col, tokens, T, c.side_dim, m->cfg.vocab,
                                      dt, stream));
            HCHECK(mi355_hyb_linear(m->y, W, m->side_a, dt, c.side_dim, WL.w[MI355_HW_SIDE_PROJ].p, nullptr, T, W, c.side_dim, dt, stream));
            if (!parallel) HCHECK(mi355_hyb_norm_add(m->x, xcopy, m->y, W, f(MI355_HW_SIDE_NORM), T, W, eps, stream));
        }
        if (parallel) {
            // the side input's norm and sum, the average over the depth and the norm that the next layer reads, in one launch
            const bool more = li + 1 < m->layers.size();
            const mi355_hybrid_layer* nx = more ? &m->layers[li + 1].c : nullptr;
            HCHECK(mi355_hyb_layer_tail(m->x, c.side_dim ? m->y : nullptr, c.side_dim ? f(MI355_HW_SIDE_NORM) : nullptr, m->xs,
                                        c.depth_terms ? f(MI355_HW_DEPTH_W) : nullptr, c.depth_terms, m->pre, dt,
                                        (more && nx->mlp_kind == 3 && bf) ? m->hf : nullptr,
                                        more ? static_cast<const float*>(m->layers[li + 1].w[MI355_HW_NORM1].p) : nullptr, T, W, m->cfg.norm_kind, eps,
                                        stream));
            if (!c.depth_terms && m->need_xs) HCHECK(mi355_hyb_copy_f32(m->xs + (li + 1) * (size_t)TW, m->x, TW, stream));
        } else {
            if (c.depth_terms) HCHECK(mi355_hyb_depth_average(m->x, m->xs, f(MI355_HW_DEPTH_W), c.depth_terms, TW, stream));
            else if (m->need_xs) HCHECK(mi355_hyb_copy_f32(m->xs + (li + 1) * (size_t)TW, m->x, TW, stream));
        }
        if (layer_trace)
            HHIP(hipMemcpyAsync(layer_trace + li * (size_t)T * W, m->x, (size_t)T * W * 4, hipMemcpyDeviceToDevice, reinterpret_cast<hipStream_t>(stream)));
    }
    if (n_out > 0) {
        if (m->cfg.norm_kind == 1)
            HCHECK(mi355_hyb_gather_norm_ex(m->xn, dt, m->x, out_rows, static_cast<const float*>(m->final_norm.p), n_out, W, 1, eps, stream));
        else
            HCHECK(mi355_hyb_gather_group_norm(m->xn, dt, m->x, out_rows, static_cast<const float*>(m->final_norm.p), n_out, W,
                                               m->cfg.norm_groups, eps, stream));
        HCHECK(mi355_hyb_linear(logits, m->cfg.vocab, m->xn, dt, W, m->cfg.tie_head ? m->embed.p : m->head.p, nullptr, n_out, m->cfg.vocab, W, dt,
                                stream));
        if (m->cfg.logit_scale != 0.f && m->cfg.logit_scale != 1.f)
            HCHECK(mi355_hyb_scale_f32(logits, m->cfg.logit_scale, (int64_t)n_out * m->cfg.vocab, stream));
        if (m->cfg.logit_softcap > 0.f) HCHECK(mi355_hyb_tanh_cap(logits, m->cfg.logit_softcap, (int64_t)n_out * m->cfg.vocab, stream));
    }
    return 0;
}

int mi355_hybrid_forward(void* mp, const uint32_t* tokens, const int64_t* positions, const int64_t* slot_mapping,
                         const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                         const int32_t* state_slots, const int32_t* out_rows, int32_t n_out, int32_t num_seqs, int32_t T,
                         int32_t max_blocks, int32_t max_context_len, float* logits, float* layer_trace, int64_t stream) {
    HModel* m = static_cast<HModel*>(mp);
    HCHECK(forward_check(m, tokens, positions, slot_mapping, block_tables, context_lens, cu_seqlens_q, state_slots, out_rows, n_out,
                         num_seqs, T, max_blocks, max_context_len, logits));
    return forward_enqueue(m, tokens, positions, slot_mapping, block_tables, context_lens, cu_seqlens_q, state_slots, out_rows, n_out,
                           num_seqs, T, max_blocks, logits, layer_trace, stream);
}

// The same step replayed from a hipGraph: the launches of a step depend on the counts and on the device pointers only (positions,
// block tables and slots are read on the device), so a caller that keeps its step inputs in static device buffers -- as the llama
// host layers' greedy loops do -- pays one graph launch per step instead of one launch per kernel.  `stream` must be a capturing-
// capable (non-default) stream.  The first step of a shape runs eagerly inside the capture's instantiate-and-launch.
int mi355_hybrid_forward_graph(void* mp, const uint32_t* tokens, const int64_t* positions, const int64_t* slot_mapping,
                               const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_seqlens_q,
                               const int32_t* state_slots, const int32_t* out_rows, int32_t n_out, int32_t num_seqs, int32_t T,
                               int32_t max_blocks, int32_t max_context_len, float* logits, int64_t stream) {
    HModel* m = static_cast<HModel*>(mp);
    if (stream == 0) return -5;
    HCHECK(forward_check(m, tokens, positions, slot_mapping, block_tables, context_lens, cu_seqlens_q, state_slots, out_rows, n_out,
                         num_seqs, T, max_blocks, max_context_len, logits));
    const std::vector<int64_t> key = {(int64_t)(intptr_t)tokens, (int64_t)(intptr_t)positions, (int64_t)(intptr_t)slot_mapping,
                                      (int64_t)(intptr_t)block_tables, (int64_t)(intptr_t)context_lens, (int64_t)(intptr_t)cu_seqlens_q,
                                      (int64_t)(intptr_t)state_slots, (int64_t)(intptr_t)out_rows, (int64_t)(intptr_t)logits,
                                      n_out, num_seqs, T, max_blocks};
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    auto it = m->graphs.find(key);
    if (it == m->graphs.end()) {
        if (m->graphs.size() >= 256) drop_graphs(m);
        HModel::StepGraph g;
        HHIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        const int rc = forward_enqueue(m, tokens, positions, slot_mapping, block_tables, context_lens, cu_seqlens_q, state_slots, out_rows,
                                       n_out, num_seqs, T, max_blocks, logits, nullptr, stream);
        const hipError_t e = hipStreamEndCapture(st, &g.graph);
        if (rc != 0 || e != hipSuccess) { if (g.graph) (void)hipGraphDestroy(g.graph); return rc != 0 ? rc : (int)e; }
        const hipError_t ei = hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0);
        if (ei != hipSuccess) { (void)hipGraphDestroy(g.graph); return (int)ei; }
        it = m->graphs.emplace(key, g).first;
        ++m->graph_captures;
    } else {
        ++m->graph_replays;
    }
    HHIP(hipGraphLaunch(it->second.exec, st));
    return 0;
}

int64_t mi355_hybrid_graph_captures(void* mp) { return mp ? static_cast<HModel*>(mp)->graph_captures : -1; }
int64_t mi355_hybrid_graph_replays(void* mp) { return mp ? static_cast<HModel*>(mp)->graph_replays : -1; }

}  // extern "C"
