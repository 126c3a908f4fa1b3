// ifa_engine_layered.hip -- the layer-list worker: a decoder given layer by layer, each layer with its own sequence mixer
// (windowed softmax attention beside decayed linear attention, or the gated delta rule), one norm feeding mixer and
// feed-forward in parallel, layer scales, a 32-bit residual stream and bfloat16 weights.  It answers the same ifa_model_*
// entry points as the standard network (ifa_model_vtbl) so that the engine above drives both alike.
//
// Slots: what the standard network calls a KV slot holds, per query, ALL per-sequence memory of the stack in one arena:
//   windowed attention   K rows (normed keys) and V rows [max_ctx][kv_heads * dim] fp32, addressed by position
//   linear attention     S [heads][dk][dv] fp32
//   gated delta rule     S [heads][dk][dv] fp32 + the last conv - 1 inputs of the short convolutions
// An arena is allocated when its slot is first used; a sequence that starts at position 0 ignores what the slot held.
//
// A step = a list of sequences (ifa_seq_desc): forward() is one sequence of n tokens from position prefix_len,
// decode_batch() n sequences of one token, decode() one sequence advanced token by token with the argmax fed back
// on the device (the step's tables live in device memory, so the captured step replays for every token).
// Per layer: norm1 -> ONE product for every projection that reads it (mixer inputs, gates, FFN gate | up; biases in the
// epilogue) -> mixer kernels -> output products that add into the fp32 residual with layer scale and branch scale
// in their epilogue -> GELU-gated FFN the same way.
// Layers wired IFA_BLOCK_POSTNORM read the residual itself through a short causal convolution (x' = x + conv(x), its last taps - 1
// inputs in the slot), put a grouped RMS norm on each sub-layer's OUTPUT (x <- x + norm(sub(x'))), mix with latent attention (cache row
// [latent | rotated key part] per position; single tokens take the absorbed form, prompts expanded keys / values and the tiled
// kernel), feed forward through a mixture of experts, and hand the next layer a learned average over the depth of the stack.
// Layers wired IFA_BLOCK_SANDWICH carry an RMS norm with weight (1 + w) before and after each sub-layer (x <- x + norm1b(mixer(norm1(x))),
// x <- x + norm2b(ffn(norm2(x)))), mix with softmax attention over rotated queries and keys (IFA_MIX_ROTARY: K rows normed and rotated,
// V rows of their own size; a layer may read the rows an earlier layer has written instead of projecting keys and values), and feed
// forward through the clamped gated form or a mixture of gated experts with a router on the logits and a shared, sigmoid-gated expert.
// Stem 2 adds a hashed token-pair embedding whose previous token lives in the slot.
// Layers wired IFA_BLOCK_PRENORM put a Dynamic Tanh norm (tanh(alpha x) w + b) in front of each sub-layer (x <- x + mixer(norm1(x)),
// x <- x + ffn(norm2(x))), mix with the rotary attention (here with a learned sink per head, a sliding window, scaled frequencies, normed
// values that enter the cache turned by their position and an output turned back) or with the generalized delta rule (IFA_MIX_CHAN_DELTA:
// state S [dim][dim] per head in the slot), and feed forward through a mixture of clamped gated experts chosen by sigmoid scores.
// A looped layer group runs several times with the same weights: every pass has cache rows and states of its own (a layer's part of the
// arena is repeated per pass), so the stack is walked as a list of RUNS (layer, pass); stem 3 keeps the embedding output for the passes.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <string>
#include <vector>
#include "ifa_engine_state.h"
#include "ifa_f32_common.h"

using ifa32::bf16_t;

namespace {

struct LTensor { void *data = nullptr; int dtype = -1; size_t rows = 0, cols = 0; bool present() const { return data != nullptr; } };

struct LLayer {
    ifa_layer_spec spec;
    LTensor t[IFA_LT_END - IFA_LT_NORM1];
    // fused input projection: rows of every matrix that reads norm1's output, and its bias vector
    bf16_t *w_in = nullptr, *b_in = nullptr; size_t n_in = 0;
    size_t c_aq = 0, c_ak = 0, c_lq = 0, c_lk = 0, c_lv = 0, c_lg = 0, c_dq = 0, c_db = 0, c_da = 0, c_dg = 0, c_fg = 0;   // column offsets in the product
    bf16_t *w_conv = nullptr; int conv_ch = 0;       // [q | k | v channels][taps]
    int *bucket_of = nullptr;                         // distance -> bias row
    // arena offsets (floats)
    size_t o_k = 0, o_v = 0, o_lin = 0, o_rec = 0, o_conv = 0;
    // latent attention: column offsets of q (or its latent), [latent | key part] and the head gates in the fused product; cache and
    // convolution tails in the arena; rotation frequencies (double, device) and the factor on cos / sin
    size_t c_mq = 0, c_mkv = 0, c_mg = 0, o_c = 0, o_cv1 = 0, o_cv2 = 0;
    double *freq = nullptr; float rot_mult = 1.0f;
    // SANDWICH: column of the values in the first product; the second product (what reads norm2: dense gate | up, or router | shared
    // expert's gate logit | shared gate | shared up) with its bias vector and column offsets
    size_t c_av = 0;
    bf16_t *w_in2 = nullptr, *b_in2 = nullptr; size_t n_in2 = 0, c2_fg = 0, c2_router = 0, c2_sg = 0, c2_shg = 0;
    // PRENORM: frequencies of the rotated values; generalized delta rule: columns of r | k | v | g | a | bottleneck in the fused product;
    // a layer of a looped group repeats its part of the arena per pass, pass_stride floats apart
    double *freq_v = nullptr;
    size_t c_cr = 0, c_ck = 0, c_cv = 0, c_cg = 0, c_ca = 0, c_cw = 0, pass_stride = 0;
    LTensor &T(int id) { return t[id - IFA_LT_NORM1]; }
    const LTensor &T(int id) const { return t[id - IFA_LT_NORM1]; }
};

constexpr int MAX_SLOTS = 4096;

} // namespace

struct LayeredNet {
    ifa_layered_config cfg;
    std::vector<LLayer> layers;
    LTensor embd, out_norm, lm_head, embd_norm, bigram, out_norm_b, out_norm_alpha, loop_step;
    std::vector<std::pair<int, int>> runs;          // the stack as it is walked: (layer, pass of the looped group or 0)
    float *x0 = nullptr, *cg_decay = nullptr, *cg_unit = nullptr, *cg_rem = nullptr; size_t chan_max = 0;      // embedding output (looped group); gates of the generalized delta rule
    size_t arena_floats = 0, o_prev = 0;          // (o_prev: the cell of the sequence's last token, stem 2)
    std::vector<float *> slot_ptr;       // host copy of the table (null: not allocated yet)
    float **slot_base_dev = nullptr;
    int n_slots = 1, cur_slot = 0;
    // step tables: pinned staging + device
    int *tab_pin = nullptr, *tab_dev = nullptr; size_t tab_rows = 0, tab_seqs = 0;
    int *tokens_dev = nullptr, *pos_dev = nullptr, *row_seq_dev = nullptr; ifa_seq_desc *seqs_dev = nullptr;
    int *excl_dev = nullptr, *next_dev = nullptr, *ring_dev = nullptr;
    // activations (fp32), sized for scratch_rows
    size_t scratch_rows = 0, n_in_max = 0, mix_max = 0, ffn_max = 0, heads_max = 0;
    float *x = nullptr, *h = nullptr, *proj = nullptr, *m1 = nullptr, *m2 = nullptr, *m3 = nullptr, *beta = nullptr, *decay = nullptr, *logits = nullptr;
    size_t logits_rows = 0, logits_cap = 0;
    float *taps = nullptr; size_t taps_rows = 0; int opt_tap_layers = 0;
    int opt_graph = 1;
    // steps of at most 8 rows: bit 0: the layer norm inside the product that reads it, bit 1: the gated GELU inside the down-projection.
    // Measured slower than the separate launches at width 2048 (decode 1149 tok/s without, 1068 / 1083 / 1012 with bit 0 / bit 1 / both; every
    // wave repeats the element-wise work for its rows) and within 1 % at width 1024: off by default
    int opt_fuse_rows = 0;
    int opt_fuse_post = 1;                 // POSTNORM layers, steps of at most 8 rows: norm-add, depth average, next input convolution and its tail in one launch
                                           // SANDWICH layers, every step size: the norm behind a sub-layer and the norm in front of the next one in one launch
                                           // PRENORM layers: the start of a looped pass inside the norm's launch; steps of at most 8 rows: the norm inside the router's launch
    float *attn_ws = nullptr; size_t attn_ws_bytes = 0;      // partial results of the windowed attention when a (row, head)'s keys are shared out
    int opt_attn_tile_min = 16;            // steps of at least this many rows run the windowed attention through the tiled kernel
    std::vector<ifa_seq_desc> seqs_host;   // the current step's sequences (the tiled attention's grid is sized from them)
    // POSTNORM layers: two more mixer buffers, the planes of the depth average ([layers + 1][scratch_rows * width]), the router's choices,
    // the experts' workspace, and -- prompts through latent attention -- keys / values expanded for every position of the step's sequences
    float *m4 = nullptr, *m5 = nullptr, *stack = nullptr, *moe_wgt = nullptr, *kx = nullptr, *vx = nullptr;
    int *moe_idx = nullptr, *ctx0_dev = nullptr; void *moe_ws = nullptr; size_t moe_ws_bytes = 0, expand_rows = 0, kx_max = 0, vx_max = 0, top_max = 0;
    bool any_depth_avg = false, any_latent = false, any_moe = false, latent_tile_ok = true, step_expand = false;
    std::vector<int> ctx0_host; size_t step_ctx_rows = 0;
    hipGraphExec_t step_exec = nullptr; hipGraph_t step_graph = nullptr; int step_slot = -1;
};

namespace {

int lay_free(void *p) { if (p) (void)hipFree(p); return 0; }

void drop_step_graph(LayeredNet *n)
{
    if (n->step_exec) { (void)hipGraphExecDestroy(n->step_exec); n->step_exec = nullptr; }
    if (n->step_graph) { (void)hipGraphDestroy(n->step_graph); n->step_graph = nullptr; }
    n->step_slot = -1;
}

// rows x cols a tensor of this layer must have; false: the tensor does not belong to the layer's mixer
bool has_moe(const ifa_layer_spec &s) { return s.ffn_kind == IFA_FFN_MOE && s.x_experts + s.x_identity > 0; }

bool expected_shape(const LayeredNet *n, const ifa_layer_spec &s, int li, int id, size_t &r, size_t &c, bool &vec)
{
    const size_t W = (size_t)n->cfg.width;
    vec = false;
    const bool par = s.mixer == IFA_MIX_WINDOW_LINEAR, del = s.mixer == IFA_MIX_GATED_DELTA, lat = s.mixer == IFA_MIX_LATENT, rot = s.mixer == IFA_MIX_ROTARY;
    const bool post = s.block == IFA_BLOCK_POSTNORM, sand = s.block == IFA_BLOCK_SANDWICH, pre = s.block == IFA_BLOCK_PRENORM, moe = has_moe(s);
    const bool chan = s.mixer == IFA_MIX_CHAN_DELTA;
    const size_t CH = (size_t)s.c_heads * s.c_dim;
    const bool own_kv = rot && s.a_kv_layer == 0, gated = s.ffn > 0 && s.ffn_kind == IFA_FFN_GATED, any_ffn = s.ffn > 0 || moe;
    const size_t SF = (size_t)s.x_shared_ff;
    const size_t MH = (size_t)s.m_heads, MQ = MH * (size_t)(s.m_dim + s.m_rot_dim), MR = (size_t)s.m_kv_rank, XA = (size_t)(s.x_experts + s.x_identity);
    switch (id) {
    case IFA_LT_NORM1: r = 1; c = W; vec = true; return true;
    case IFA_LT_LS1: r = 1; c = W; vec = true; return !post && !sand && !pre;
    case IFA_LT_NORM2: r = 1; c = W; vec = true; return (post && moe) || ((sand || pre) && any_ffn);
    case IFA_LT_NORM1_B: r = 1; c = W; vec = true; return pre;
    case IFA_LT_NORM1_ALPHA: r = 1; c = 1; vec = true; return pre;
    case IFA_LT_NORM2_B: r = 1; c = W; vec = true; return pre && any_ffn;
    case IFA_LT_NORM2_ALPHA: r = 1; c = 1; vec = true; return pre && any_ffn;
    case IFA_LT_C_R: case IFA_LT_C_K: case IFA_LT_C_V: case IFA_LT_C_G: case IFA_LT_C_A: r = CH; c = W; return chan;
    case IFA_LT_C_A_B: case IFA_LT_C_W0: case IFA_LT_C_NORM: r = 1; c = CH; vec = true; return chan;
    case IFA_LT_C_W1: r = (size_t)s.c_rank; c = W; return chan;
    case IFA_LT_C_W2: r = CH; c = (size_t)s.c_rank; return chan;
    case IFA_LT_C_O: r = W; c = CH; return chan;
    case IFA_LT_NORM1B: r = 1; c = W; vec = true; return sand;
    case IFA_LT_NORM2B: r = 1; c = W; vec = true; return sand && any_ffn;
    case IFA_LT_A_V: r = (size_t)s.a_kv_heads * s.a_vdim; c = W; return own_kv;
    case IFA_LT_A_Q_B: r = 1; c = (size_t)s.a_heads * s.a_dim; vec = true; return rot;
    case IFA_LT_A_K_B: r = 1; c = (size_t)s.a_kv_heads * s.a_dim; vec = true; return own_kv;
    case IFA_LT_A_V_B: r = 1; c = (size_t)s.a_kv_heads * s.a_vdim; vec = true; return own_kv;
    case IFA_LT_A_Q_NORM: r = 1; c = (size_t)s.a_dim; vec = true; return rot;
    case IFA_LT_A_K_NORM: r = 1; c = (size_t)s.a_dim; vec = true; return own_kv;
    case IFA_LT_X_ROUTER_B: r = 1; c = XA; vec = true; return moe && s.x_route == 1;
    case IFA_LT_X_SH_GATE: case IFA_LT_X_SH_UP: r = SF; c = W; return moe && SF > 0;
    case IFA_LT_X_SH_DOWN: r = W; c = SF; return moe && SF > 0;
    case IFA_LT_X_SH_SG: r = 1; c = W; vec = true; return moe && SF > 0;
    case IFA_LT_CANON1: r = W; c = (size_t)s.canon_taps; return post && s.canon_taps > 0;
    case IFA_LT_CANON2: r = W; c = (size_t)s.canon_taps; return post && s.canon_taps > 0 && moe;
    case IFA_LT_DWA: r = 1; c = (size_t)li + 2; vec = true; return post && s.depth_avg;
    case IFA_LT_M_Q: r = MQ; c = W; return lat && s.m_q_rank == 0;
    case IFA_LT_M_DQ: r = (size_t)s.m_q_rank; c = W; return lat && s.m_q_rank > 0;
    case IFA_LT_M_DQ_NORM: r = 1; c = (size_t)s.m_q_rank; vec = true; return lat && s.m_q_rank > 0;
    case IFA_LT_M_UQ: r = MQ; c = (size_t)s.m_q_rank; return lat && s.m_q_rank > 0;
    case IFA_LT_M_DKV: r = MR + (size_t)s.m_rot_dim; c = W; return lat;
    case IFA_LT_M_DKV_NORM: r = 1; c = MR; vec = true; return lat;
    case IFA_LT_M_UK: r = MH * (size_t)s.m_dim; c = MR; return lat;
    case IFA_LT_M_UV: r = MH * (size_t)s.m_vdim; c = MR; return lat;
    case IFA_LT_M_G: r = MH; c = W; return lat && s.m_gate;
    case IFA_LT_M_O: r = W; c = MH * (size_t)s.m_vdim; return lat;
    case IFA_LT_X_ROUTER: r = XA; c = W; return moe;
    case IFA_LT_X_CORR: r = 1; c = XA; vec = true; return moe && s.x_route == 0;
    case IFA_LT_X_UP: r = (size_t)s.x_experts * s.x_ff * (s.x_gated ? 2 : 1); c = W; return moe && s.x_experts > 0;
    case IFA_LT_X_DOWN: r = (size_t)s.x_experts * W; c = (size_t)s.x_ff; return moe && s.x_experts > 0;
    case IFA_LT_LS2: case IFA_LT_FFN_DOWN_B: r = 1; c = W; vec = true; return gated;
    case IFA_LT_FFN_GATE: case IFA_LT_FFN_UP: r = (size_t)s.ffn; c = W; return s.ffn > 0;
    case IFA_LT_FFN_GATE_B: case IFA_LT_FFN_UP_B: r = 1; c = (size_t)s.ffn; vec = true; return gated;
    case IFA_LT_FFN_DOWN: r = W; c = (size_t)s.ffn; return s.ffn > 0;
    case IFA_LT_A_Q: r = (size_t)s.a_heads * s.a_dim; c = W; return par || rot;
    case IFA_LT_A_K: r = (size_t)s.a_kv_heads * s.a_dim; c = W; return par || own_kv;
    case IFA_LT_A_REL: r = (size_t)s.a_buckets; c = (size_t)s.a_heads; return par;
    case IFA_LT_A_SINK: r = 1; c = (size_t)s.a_heads; vec = true; return par || (rot && s.a_sink == 2);
    case IFA_LT_A_O: r = W; c = (size_t)s.a_heads * (rot ? s.a_vdim : s.a_dim); return par || rot;
    case IFA_LT_L_Q: case IFA_LT_L_K: r = (size_t)s.l_heads * s.l_dim; c = W; return par;
    case IFA_LT_L_V: case IFA_LT_L_G: r = (size_t)s.l_heads * s.l_vdim; c = W; return par;
    case IFA_LT_L_O: r = W; c = (size_t)s.l_heads * s.l_vdim; return par;
    case IFA_LT_L_NORM: r = 1; c = (size_t)s.l_heads * s.l_vdim; vec = true; return par;
    case IFA_LT_L_DECAY: r = 1; c = (size_t)s.l_heads; vec = true; return par;
    case IFA_LT_D_Q: case IFA_LT_D_K: r = (size_t)s.d_kv_heads * s.d_dim; c = W; return del;
    case IFA_LT_D_V: case IFA_LT_D_G: r = (size_t)s.d_heads * s.d_vdim; c = W; return del;
    case IFA_LT_D_QCONV: case IFA_LT_D_KCONV: r = (size_t)s.d_kv_heads * s.d_dim; c = (size_t)s.d_conv; return del;
    case IFA_LT_D_VCONV: r = (size_t)s.d_heads * s.d_vdim; c = (size_t)s.d_conv; return del;
    case IFA_LT_D_B: case IFA_LT_D_A: r = (size_t)s.d_heads; c = W; return del;
    case IFA_LT_D_ALOG: case IFA_LT_D_DTBIAS: r = 1; c = (size_t)s.d_heads; vec = true; return del;
    case IFA_LT_D_NORM: r = 1; c = (size_t)s.d_vdim; vec = true; return del;
    case IFA_LT_D_O: r = W; c = (size_t)s.d_heads * s.d_vdim; return del;
    default: return false;
    }
}

size_t align4(size_t v) { return (v + 3) & ~(size_t)3; }

// distance -> row of the bias table: n for n < B / 2, then logarithmic up to bias_max, the last row beyond (formed in double)
void build_buckets(std::vector<int> &out, int max_ctx, int B, int Dmax)
{
    out.resize((size_t)max_ctx);
    const int half = B / 2;
    for (int d = 0; d < max_ctx; d++) {
        int b;
        if (d < half || half <= 0) b = std::min(d, B - 1);
        else if (Dmax <= half) b = B - 1;
        else {
            const double f = std::log((double)d / (double)half) / std::log((double)Dmax / (double)half) * (double)(B - half);
            b = std::min(B - 1, half + (int)std::floor(f));
        }
        out[(size_t)d] = b;
    }
}

int ensure_slot(ifa_model *m, int slot)
{
    LayeredNet *n = m->lay;
    IFA_REQUIRE(slot >= 0 && slot < n->n_slots, "layer-list worker: slot %d of %d", slot, n->n_slots);
    if (n->slot_ptr[(size_t)slot]) return IFA_OK;
    float *p = nullptr;
    IFA_HIP_CHECK(hipMalloc((void **)&p, std::max<size_t>(n->arena_floats, 4) * 4));
    n->slot_ptr[(size_t)slot] = p;
    IFA_HIP_CHECK(hipMemcpyAsync(n->slot_base_dev + slot, &n->slot_ptr[(size_t)slot], sizeof(float *), hipMemcpyHostToDevice, m->stream));
    IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
    return IFA_OK;
}

int ensure_rows(ifa_model *m, size_t T, size_t nseq)
{
    LayeredNet *n = m->lay;
    if (T > n->tab_rows || nseq > n->tab_seqs) {
        IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
        drop_step_graph(n);
        if (n->tab_pin) (void)hipHostFree(n->tab_pin);
        lay_free(n->tab_dev);
        n->tab_pin = nullptr; n->tab_dev = nullptr;
        const size_t R = std::max(T, n->tab_rows), S = std::max(nseq, n->tab_seqs);
        const size_t ints = 3 * R + 5 * S;
        IFA_HIP_CHECK(hipHostMalloc((void **)&n->tab_pin, ints * 4, hipHostMallocDefault));
        IFA_HIP_CHECK(hipMalloc((void **)&n->tab_dev, ints * 4));
        n->tab_rows = R; n->tab_seqs = S;
        n->tokens_dev = n->tab_dev; n->pos_dev = n->tab_dev + R; n->row_seq_dev = n->tab_dev + 2 * R; n->seqs_dev = (ifa_seq_desc *)(n->tab_dev + 3 * R);
        n->ctx0_dev = n->tab_dev + 3 * R + 4 * S;
    }
    if (T > n->scratch_rows) {
        IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
        drop_step_graph(n);
        float **bufs[] = {&n->x, &n->h, &n->proj, &n->m1, &n->m2, &n->m3, &n->beta, &n->decay};
        for (float **b : bufs) { lay_free(*b); *b = nullptr; }
        const size_t W = (size_t)n->cfg.width;
        const size_t sz[] = {W, W, n->n_in_max, n->mix_max, n->mix_max, std::max<size_t>(n->ffn_max, 4), std::max<size_t>(n->heads_max, 4), std::max<size_t>(n->heads_max, 4)};
        for (size_t i = 0; i < 8; i++) IFA_HIP_CHECK(hipMalloc((void **)bufs[i], T * sz[i] * 4));
        {   // the single-row latent attention leaves at least one partial result per (row, head) in the workspace
            size_t need = 0;
            for (const LLayer &L : n->layers)
                if (L.spec.mixer == IFA_MIX_LATENT) need = std::max(need, T * (size_t)L.spec.m_heads * ((size_t)L.spec.m_kv_rank + 2) * 4);
            if (need > n->attn_ws_bytes) {
                lay_free(n->attn_ws); n->attn_ws = nullptr;
                IFA_HIP_CHECK(hipMalloc((void **)&n->attn_ws, need));
                n->attn_ws_bytes = need;
            }
        }
        lay_free(n->m4); lay_free(n->m5); lay_free(n->stack); lay_free(n->moe_wgt); lay_free(n->moe_idx); lay_free(n->moe_ws);
        n->m4 = n->m5 = n->stack = n->moe_wgt = nullptr; n->moe_idx = nullptr; n->moe_ws = nullptr; n->moe_ws_bytes = 0;
        lay_free(n->x0); lay_free(n->cg_decay); lay_free(n->cg_unit); lay_free(n->cg_rem);
        n->x0 = n->cg_decay = n->cg_unit = n->cg_rem = nullptr;
        if (n->cfg.loop_times > 1) IFA_HIP_CHECK(hipMalloc((void **)&n->x0, T * W * 4));
        if (n->chan_max) {
            float **gb[] = {&n->cg_decay, &n->cg_unit, &n->cg_rem};
            for (float **b : gb) IFA_HIP_CHECK(hipMalloc((void **)b, T * n->chan_max * 4));
        }
        if (n->any_latent) { IFA_HIP_CHECK(hipMalloc((void **)&n->m4, T * n->mix_max * 4)); IFA_HIP_CHECK(hipMalloc((void **)&n->m5, T * n->mix_max * 4)); }
        if (n->any_depth_avg) IFA_HIP_CHECK(hipMalloc((void **)&n->stack, (n->layers.size() + 1) * T * W * 4));
        if (n->any_moe) {
            IFA_HIP_CHECK(hipMalloc((void **)&n->moe_wgt, T * n->top_max * 4));
            IFA_HIP_CHECK(hipMalloc((void **)&n->moe_idx, T * n->top_max * 4));
            for (const LLayer &L : n->layers)
                if (has_moe(L.spec)) n->moe_ws_bytes = std::max(n->moe_ws_bytes, ifa_moe_workspace_bytes(T, L.spec.x_top, (int)W, std::max(L.spec.x_ff, 1) * (L.spec.x_gated ? 3 : 1), L.spec.x_experts));
            IFA_HIP_CHECK(hipMalloc(&n->moe_ws, n->moe_ws_bytes));
        }
        n->scratch_rows = T;
    }
    return IFA_OK;
}

int ensure_logits(ifa_model *m, size_t rows)
{
    LayeredNet *n = m->lay;
    if (rows > n->logits_cap) {
        IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
        drop_step_graph(n);
        lay_free(n->logits); n->logits = nullptr;
        IFA_HIP_CHECK(hipMalloc((void **)&n->logits, rows * (size_t)n->cfg.vocab * 4));
        n->logits_cap = rows;
    }
    return IFA_OK;
}

int linear(ifa_model *m, const bf16_t *W, size_t N, size_t K, const float *A, size_t lda, size_t T, const bf16_t *bias, const bf16_t *mul, float alpha,
           int accumulate, float *C, size_t ldc, int silu0 = 0, int silu1 = 0)
{
    return ifa_linear_bf16w(W, N, K, A, lda, T, bias, mul, alpha, accumulate, m->lay->cfg.ops32, C, ldc, silu0, silu1, (ifa_stream)m->stream);
}

// What lies between two sub-layers of a POSTNORM block: x += gnorm(sub) * norm_w; [depth average]; [h = x + conv(x), tail advanced].
// Steps of a few rows run it as ONE launch (ifa_norm_add_conv_rows_f32), larger steps as the separate row-parallel ops.
int post_step(ifa_model *m, size_t T, int nseq, bool fused, const float *sub, const void *norm_w, const LLayer *depth_of, size_t li, const void *conv_w, int taps,
              size_t conv_off)
{
    LayeredNet *n = m->lay;
    const ifa_layered_config &c = n->cfg;
    const size_t W = (size_t)c.width, plane = n->scratch_rows * W;
    ifa_stream s = (ifa_stream)m->stream;
    void *const *slots = (void *const *)n->slot_base_dev;
    int rc;
    if (fused)
        return ifa_norm_add_conv_rows_f32(n->x, T, W, sub, W, norm_w, c.norm_groups, c.eps, depth_of ? n->stack : nullptr, plane, (int)li + 2,
                                          depth_of ? depth_of->T(IFA_LT_DWA).data : nullptr, conv_w, taps, n->seqs_dev, nseq, n->row_seq_dev, slots, conv_off, n->h, s);
    if (sub && (rc = ifa_group_rmsnorm_f32(sub, W, T, W, c.norm_groups, norm_w, c.eps, 1, n->x, W, s))) return rc;
    if (depth_of && (rc = ifa_depth_average_f32(n->x, T, W, n->stack, plane, (int)li + 2, depth_of->T(IFA_LT_DWA).data, s))) return rc;
    if (conv_w) {
        if ((rc = ifa_shortconv_residual_f32(n->x, W, (int)W, taps, conv_w, n->seqs_dev, n->row_seq_dev, T, slots, conv_off, n->h, W, s))) return rc;
        if ((rc = ifa_shortconv_tail_f32(n->x, W, (int)W, taps, n->seqs_dev, nseq, slots, conv_off, s))) return rc;
    }
    return IFA_OK;
}

// one POSTNORM layer over T rows: x <- x + norm1(mixer(x + conv1(x))); x <- x + norm2(experts(x + conv2(x))); depth average.
// h_ready: the layer before has already left x + conv1(x) in n->h (its closing step ran this layer's input convolution);
// next: the layer after, whose input convolution this layer's closing step runs when both are wired alike (*next_h_ready says so).
int run_postnorm_layer(ifa_model *m, LLayer &L, size_t li, size_t T, int nseq, bool h_ready, const LLayer *next, bool *next_h_ready)
{
    LayeredNet *n = m->lay;
    const ifa_layered_config &c = n->cfg;
    const ifa_layer_spec &sp = L.spec;
    const size_t W = (size_t)c.width, NI = L.n_in;
    ifa_stream s = (ifa_stream)m->stream;
    void *const *slots = (void *const *)n->slot_base_dev;
    const bool fused = T <= 8 && n->opt_fuse_post && !n->opt_tap_layers;
    const bool moe = has_moe(sp);
    const bool next_conv = fused && next && next->spec.block == IFA_BLOCK_POSTNORM && next->spec.canon_taps > 0;
    *next_h_ready = next_conv;
    int rc;
    // what the mixer reads
    const float *hin = n->x;
    if (sp.canon_taps > 0) {
        if (!h_ready && (rc = post_step(m, T, nseq, fused, nullptr, nullptr, nullptr, li, L.T(IFA_LT_CANON1).data, sp.canon_taps, L.o_cv1))) return rc;
        hin = n->h;
    }
    {   // latent attention
        const int H = sp.m_heads, dn = sp.m_dim, dr = sp.m_rot_dim, dv = sp.m_vdim, R = sp.m_kv_rank;
        const size_t QD = (size_t)H * (dn + dr), CR = (size_t)(R + dr), OV = (size_t)H * dv;
        if ((rc = linear(m, L.w_in, NI, W, hin, W, T, nullptr, nullptr, 1.0f, 0, n->proj, NI))) return rc;
        float *q = n->proj + L.c_mq; size_t ldq = NI;
        if (sp.m_q_rank > 0) {      // queries through their own normed latent
            const size_t QR = (size_t)sp.m_q_rank;
            if ((rc = ifa_layernorm_f32(0, n->proj + L.c_mq, NI, T, QR, L.T(IFA_LT_M_DQ_NORM).data, c.eps, n->m3, QR, s))) return rc;
            if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_M_UQ).data, QD, QR, n->m3, QR, T, nullptr, nullptr, 1.0f, 0, n->m1, QD))) return rc;
            q = n->m1; ldq = QD;
        }
        if ((rc = ifa_latent_prepare_f32(n->proj + L.c_mkv, NI, R, dr, sp.m_rot_dims, L.T(IFA_LT_M_DKV_NORM).data, c.eps, q, ldq, H, dn, L.freq, L.rot_mult,
                                         n->seqs_dev, n->row_seq_dev, T, slots, L.o_c, s))) return rc;
        const float *gate = sp.m_gate ? n->proj + L.c_mg : nullptr;
        if (n->step_expand) {
            // keys and values of every position of the step's sequences from their cached latents, then the tiled kernel
            const size_t ldk = (size_t)H * dn, ldv = OV;
            for (size_t qi = 0; qi < n->seqs_host.size(); qi++) {
                const ifa_seq_desc &sd = n->seqs_host[qi];
                const float *lat = n->slot_ptr[(size_t)sd.slot] + L.o_c;
                const size_t ctx = (size_t)sd.pos0 + sd.n, r0 = (size_t)n->ctx0_host[qi];
                if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_M_UK).data, ldk, (size_t)R, lat, CR, ctx, nullptr, nullptr, 1.0f, 0, n->kx + r0 * ldk, ldk))) return rc;
                if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_M_UV).data, ldv, (size_t)R, lat, CR, ctx, nullptr, nullptr, 1.0f, 0, n->vx + r0 * ldv, ldv))) return rc;
            }
            if ((rc = ifa_attention_latent_tile_f32(q, ldq, H, dn, dr, dv, R, sp.m_scale, n->kx, ldk, n->vx, ldv, n->ctx0_dev, gate, NI, n->seqs_dev, n->seqs_host.data(),
                                                    (int)n->seqs_host.size(), slots, L.o_c, n->m5, OV, s))) return rc;
        } else {
            // absorbed form: the cache rows are keys (whole) and values (latent part) of ONE head that all query heads share
            const size_t QA = (size_t)H * CR;
            if ((rc = ifa_latent_absorb_q_f32(q, ldq, H, dn, dr, R, L.T(IFA_LT_M_UK).data, T, n->m2, QA, s))) return rc;
            if ((rc = ifa_attention_latent_rows_f32(n->m2, QA, H, R, dr, sp.m_scale, n->seqs_dev, n->row_seq_dev, T, slots, L.o_c, c.max_ctx, n->attn_ws, n->attn_ws_bytes,
                                                    n->m4, (size_t)H * R, s))) return rc;
            if ((rc = ifa_latent_expand_out_f32(n->m4, (size_t)H * R, R, H, dv, R, L.T(IFA_LT_M_UV).data, gate, NI, T, n->m5, OV, s))) return rc;
        }
        if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_M_O).data, W, OV, n->m5, OV, T, nullptr, nullptr, 1.0f, 0, n->m1, W))) return rc;
    }
    const LLayer *depth_of = sp.depth_avg ? &L : nullptr;
    const void *ncw = next_conv ? next->T(IFA_LT_CANON1).data : nullptr;
    const int ntaps = next_conv ? next->spec.canon_taps : 0;
    const size_t noff = next_conv ? next->o_cv1 : 0;
    if (!moe) return post_step(m, T, nseq, fused, n->m1, L.T(IFA_LT_NORM1).data, depth_of, li, ncw, ntaps, noff);
    {
        // the mixer's output into the residual, then what the experts read
        if ((rc = post_step(m, T, nseq, fused, n->m1, L.T(IFA_LT_NORM1).data, nullptr, li, sp.canon_taps > 0 ? L.T(IFA_LT_CANON2).data : nullptr, sp.canon_taps, L.o_cv2))) return rc;
        hin = sp.canon_taps > 0 ? n->h : n->x;
        const size_t XA = (size_t)(sp.x_experts + sp.x_identity);
        if (fused && XA <= 512) {      // a few rows: the router's product inside the choice's launch
            if ((rc = ifa_moe_route_rows_f32(hin, W, T, (int)W, L.T(IFA_LT_X_ROUTER).data, (int)XA, sp.x_top, L.T(IFA_LT_X_CORR).data, n->moe_idx, n->moe_wgt, s))) return rc;
        } else {
            if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_X_ROUTER).data, XA, W, hin, W, T, nullptr, nullptr, 1.0f, 0, n->m2, XA))) return rc;
            if ((rc = ifa_moe_route_f32(n->m2, XA, T, (int)XA, sp.x_top, L.T(IFA_LT_X_CORR).data, n->moe_idx, n->moe_wgt, s))) return rc;
        }
        if ((rc = ifa_moe_experts_f32(hin, W, T, (int)W, std::max(sp.x_ff, 1), sp.x_experts, sp.x_identity, sp.x_top, 0, L.T(IFA_LT_X_UP).data, L.T(IFA_LT_X_DOWN).data,
                                      n->moe_idx, n->moe_wgt, c.ops32, n->moe_ws, n->moe_ws_bytes, n->m1, W, 0, s))) return rc;
    }
    return post_step(m, T, nseq, fused, n->m1, L.T(IFA_LT_NORM2).data, depth_of, li, ncw, ntaps, noff);
}

// one SANDWICH layer over T rows: x <- x + norm1b(attention(norm1(x))); x <- x + norm2b(ffn(norm2(x))), every norm an RMS norm with
// weight (1 + w).  The keys enter the cache normed and rotated; a layer with a_kv_layer reads the rows that layer has written in this step.
// The norm behind a sub-layer and the norm in front of the next one run as ONE launch (option fuse_post): h_ready says that the layer
// before has left norm1(x) in n->h, *next_h_ready that this layer has done so for `next`.
int run_sandwich_layer(ifa_model *m, LLayer &L, size_t T, int nseq, bool h_ready, const LLayer *next, bool *next_h_ready)
{
    LayeredNet *n = m->lay;
    const ifa_layered_config &c = n->cfg;
    const ifa_layer_spec &sp = L.spec;
    const size_t W = (size_t)c.width, NI = L.n_in;
    ifa_stream s = (ifa_stream)m->stream;
    void *const *slots = (void *const *)n->slot_base_dev;
    const bool fused = n->opt_fuse_post != 0, moe = has_moe(sp), any_ffn = sp.ffn > 0 || moe;
    const void *next_norm = fused && next && next->spec.block == IFA_BLOCK_SANDWICH ? next->T(IFA_LT_NORM1).data : nullptr;
    *next_h_ready = next_norm != nullptr;
    // x += norm_after(sub); h = norm_before(x) for whatever comes next
    auto close_sub = [&](const float *sub, const void *w_after, const void *w_before) -> int {
        if (fused) return ifa_norm_add_norm_f32(n->x, W, T, W, sub, W, w_after, w_before, 1.0f, c.eps, n->h, W, s);
        int r = ifa_rmsnorm_offset_f32(sub, W, T, W, w_after, 1.0f, c.eps, 1, n->x, W, s);
        if (!r && w_before) r = ifa_rmsnorm_offset_f32(n->x, W, T, W, w_before, 1.0f, c.eps, 0, n->h, W, s);
        return r;
    };
    int rc;
    {
        const int H = sp.a_heads, G = sp.a_kv_heads, D = sp.a_dim, DV = sp.a_vdim;
        const size_t OV = (size_t)H * DV;
        const bool own = sp.a_kv_layer == 0;
        const LLayer &KV = own ? L : n->layers[(size_t)sp.a_kv_layer - 1];
        if (!h_ready && (rc = ifa_rmsnorm_offset_f32(n->x, W, T, W, L.T(IFA_LT_NORM1).data, 1.0f, c.eps, 0, n->h, W, s))) return rc;
        if ((rc = linear(m, L.w_in, NI, W, n->h, W, T, L.b_in, nullptr, 1.0f, 0, n->proj, NI))) return rc;
        if ((rc = ifa_qk_rope_store_f32(n->proj + L.c_aq, NI, H, own ? n->proj + L.c_ak : nullptr, NI, own ? n->proj + L.c_av : nullptr, NI, G, D, DV,
                                        L.T(IFA_LT_A_Q_NORM).data, own ? L.T(IFA_LT_A_K_NORM).data : nullptr, c.eps, sp.a_rot_dims, L.freq, n->seqs_dev, n->row_seq_dev, T,
                                        slots, KV.o_k, KV.o_v, s))) return rc;
        if ((rc = ifa_attention_kv_f32(n->proj + L.c_aq, NI, H, G, D, DV, sp.a_scale, sp.a_window, sp.a_keep_first, sp.a_sink, sp.a_sink_score, n->seqs_dev,
                                       n->row_seq_dev, T, slots, KV.o_k, KV.o_v, n->m1, OV, n->seqs_host.data(), (int)n->seqs_host.size(), n->opt_attn_tile_min,
                                       c.max_ctx, n->attn_ws, n->attn_ws_bytes, s))) return rc;
        if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_A_O).data, W, OV, n->m1, OV, T, nullptr, nullptr, 1.0f, 0, n->m2, W))) return rc;
        if ((rc = close_sub(n->m2, L.T(IFA_LT_NORM1B).data, any_ffn ? L.T(IFA_LT_NORM2).data : next_norm))) return rc;
    }
    if (!any_ffn) return IFA_OK;
    const size_t N2 = L.n_in2;
    if ((rc = linear(m, L.w_in2, N2, W, n->h, W, T, L.b_in2, nullptr, 1.0f, 0, n->proj, N2))) return rc;
    if (!moe) {
        const size_t F = (size_t)sp.ffn;
        if ((rc = ifa_glu_ex_f32(3, sp.f_limit, n->proj + L.c2_fg, N2, T, F, nullptr, 0, n->m3, F, s))) return rc;
        if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_FFN_DOWN).data, W, F, n->m3, F, T, nullptr, nullptr, 1.0f, 0, n->m2, W))) return rc;
    } else {
        // the router's logits (bias added by the product) are columns of the second product; the chosen experts read norm2's output
        if ((rc = ifa_moe_route_top_f32(n->proj + L.c2_router, N2, T, sp.x_experts, sp.x_top, nullptr, n->moe_idx, n->moe_wgt, s))) return rc;
        if ((rc = ifa_moe_experts_gated_f32(n->h, W, T, (int)W, sp.x_ff, sp.x_experts, sp.x_top, L.T(IFA_LT_X_UP).data, L.T(IFA_LT_X_DOWN).data, n->moe_idx, n->moe_wgt,
                                            c.ops32, n->moe_ws, n->moe_ws_bytes, n->m2, W, 0, s))) return rc;
        if (sp.x_shared_ff > 0) {      // the shared expert: its gate sigmoid(w_sg . h) multiplies the activations in front of the down-projection
            const size_t SF = (size_t)sp.x_shared_ff;
            if ((rc = ifa_glu_ex_f32(0, 0.0f, n->proj + L.c2_shg, N2, T, SF, n->proj + L.c2_sg, N2, n->m3, SF, s))) return rc;
            if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_X_SH_DOWN).data, W, SF, n->m3, SF, T, nullptr, nullptr, 1.0f, 1, n->m2, W))) return rc;
        }
    }
    return close_sub(n->m2, L.T(IFA_LT_NORM2B).data, next_norm);
}

// one PRENORM layer over T rows: x <- x + mixer(dyt1(x)); x <- x + experts(dyt2(x)), dyt(x) = tanh(alpha x) w + b.  pass: which copy of the
// layer's cache rows / state (a layer of a looped group has one per pass).  The output products and the experts add into the residual themselves.
int run_prenorm_layer(ifa_model *m, LLayer &L, size_t T, int nseq, int pass, bool pass_start)
{
    LayeredNet *n = m->lay;
    const ifa_layered_config &c = n->cfg;
    const ifa_layer_spec &sp = L.spec;
    const size_t W = (size_t)c.width, NI = L.n_in, po = (size_t)pass * L.pass_stride;
    ifa_stream s = (ifa_stream)m->stream;
    void *const *slots = (void *const *)n->slot_base_dev;
    int rc;
    // (the first layer of a looped pass: x += the embedding output, from the second pass on, + the pass's own vector, in the norm's launch)
    const bool fused = n->opt_fuse_post != 0;      // (option fuse_post 0: every element-wise step as a launch of its own)
    if (pass_start && !fused && (rc = ifa_add_rows_vec_f32(n->x, W, T, W, pass > 0 ? n->x0 : nullptr, W, (const bf16_t *)n->loop_step.data + (size_t)pass * W, s))) return rc;
    if (pass_start && fused)
        rc = ifa_add_dyt_f32(n->x, W, T, W, pass > 0 ? n->x0 : nullptr, W, (const bf16_t *)n->loop_step.data + (size_t)pass * W, L.T(IFA_LT_NORM1_ALPHA).data,
                             L.T(IFA_LT_NORM1).data, L.T(IFA_LT_NORM1_B).data, n->h, W, s);
    else rc = ifa_dyt_f32(n->x, W, T, W, L.T(IFA_LT_NORM1_ALPHA).data, L.T(IFA_LT_NORM1).data, L.T(IFA_LT_NORM1_B).data, n->h, W, s);
    if (rc) return rc;
    if ((rc = linear(m, L.w_in, NI, W, n->h, W, T, L.b_in, nullptr, 1.0f, 0, n->proj, NI))) return rc;
    if (sp.mixer == IFA_MIX_ROTARY) {
        const int H = sp.a_heads, G = sp.a_kv_heads, D = sp.a_dim, DV = sp.a_vdim;
        const size_t OV = (size_t)H * DV;
        if ((rc = ifa_qkv_rope_store_f32(n->proj + L.c_aq, NI, H, n->proj + L.c_ak, NI, n->proj + L.c_av, NI, G, D, DV, L.T(IFA_LT_A_Q_NORM).data, L.T(IFA_LT_A_K_NORM).data,
                                         c.eps, sp.a_rot_dims, L.freq, sp.a_vnorm, sp.a_vrot ? L.freq_v : nullptr, n->seqs_dev, n->row_seq_dev, T, slots, L.o_k + po,
                                         L.o_v + po, s))) return rc;
        if (sp.a_sink == 2)
            rc = ifa_attention_kv_sinks_f32(n->proj + L.c_aq, NI, H, G, D, DV, sp.a_scale, sp.a_window, sp.a_keep_first, L.T(IFA_LT_A_SINK).data, n->seqs_dev, n->row_seq_dev, T,
                                            slots, L.o_k + po, L.o_v + po, n->m1, OV, n->seqs_host.data(), (int)n->seqs_host.size(), n->opt_attn_tile_min, c.max_ctx, n->attn_ws,
                                            n->attn_ws_bytes, s);
        else
            rc = ifa_attention_kv_f32(n->proj + L.c_aq, NI, H, G, D, DV, sp.a_scale, sp.a_window, sp.a_keep_first, sp.a_sink, sp.a_sink_score, n->seqs_dev, n->row_seq_dev, T,
                                      slots, L.o_k + po, L.o_v + po, n->m1, OV, n->seqs_host.data(), (int)n->seqs_host.size(), n->opt_attn_tile_min, c.max_ctx, n->attn_ws,
                                      n->attn_ws_bytes, s);
        if (rc) return rc;
        // the sum over values that entered the cache turned by their positions is turned back by the row's own position
        if (sp.a_vrot && (rc = ifa_rotate_heads_f32(n->m1, OV, H, DV, DV & ~1, L.freq_v, -1.0f, n->seqs_dev, n->row_seq_dev, T, s))) return rc;
        if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_A_O).data, W, OV, n->m1, OV, T, nullptr, nullptr, 1.0f, 1, n->x, W))) return rc;
    } else {
        const int H = sp.c_heads, D = sp.c_dim;
        const size_t CH = (size_t)H * D;
        if (T <= 8) {      // a few rows: the bottleneck's second matrix inside the gates' launch
            if ((rc = ifa_chan_delta_gates_f32(n->proj + L.c_cw, NI, sp.c_rank, L.T(IFA_LT_C_W2).data, L.T(IFA_LT_C_W0).data, sp.c_decay_mult, n->proj + L.c_ca, NI,
                                               n->proj + L.c_ck, NI, H, D, sp.c_l2_eps, T, n->cg_decay, n->cg_unit, n->cg_rem, s))) return rc;
        } else {           // the sigmoid's argument as a product on the matrix cores (its bias = w0), left where the decays will be written
            if ((rc = ifa_tanh_f32(n->proj + L.c_cw, NI, T, (size_t)sp.c_rank, s))) return rc;
            // (fp32 operands in both modes: the product is small, and a decay close to one carries an error of its argument through hundreds of tokens)
            if ((rc = ifa_linear_bf16w(L.T(IFA_LT_C_W2).data, CH, (size_t)sp.c_rank, n->proj + L.c_cw, NI, T, L.T(IFA_LT_C_W0).data, nullptr, 1.0f, 0, 1, n->cg_decay, CH, 0, 0, s))) return rc;
            if ((rc = ifa_chan_delta_gates_f32(n->cg_decay, CH, 0, nullptr, nullptr, sp.c_decay_mult, n->proj + L.c_ca, NI, n->proj + L.c_ck, NI, H, D, sp.c_l2_eps, T,
                                               n->cg_decay, n->cg_unit, n->cg_rem, s))) return rc;
        }
        if ((rc = ifa_state_scan_chan_f32(n->proj + L.c_cr, NI, n->proj + L.c_ck, NI, n->proj + L.c_cv, NI, H, D, D, n->cg_decay, n->cg_unit, n->cg_rem, CH, n->seqs_dev, nseq,
                                          slots, L.o_rec + po, n->m1, CH, s))) return rc;
        if ((rc = ifa_gated_groupnorm_f32(n->m1, CH, T, (int)CH, D, L.T(IFA_LT_C_NORM).data, (int)CH, n->proj + L.c_cg, NI, 0, c.eps, n->m1, CH, s))) return rc;
        if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_C_O).data, W, CH, n->m1, CH, T, nullptr, nullptr, 1.0f, 1, n->x, W))) return rc;
    }
    if (!has_moe(sp)) return IFA_OK;
    const int XA = sp.x_experts;
    if (T <= 8 && XA <= 512 && fused) {      // a few rows: the norm and the router's product inside the choice's launch
        if ((rc = ifa_moe_dyt_route_rows_f32(sp.x_score, n->x, W, L.T(IFA_LT_NORM2_ALPHA).data, L.T(IFA_LT_NORM2).data, L.T(IFA_LT_NORM2_B).data, n->h, W, T, (int)W,
                                             L.T(IFA_LT_X_ROUTER).data, XA, sp.x_top, L.T(IFA_LT_X_CORR).data, n->moe_idx, n->moe_wgt, s))) return rc;
    } else if (T <= 8 && XA <= 512) {
        if ((rc = ifa_dyt_f32(n->x, W, T, W, L.T(IFA_LT_NORM2_ALPHA).data, L.T(IFA_LT_NORM2).data, L.T(IFA_LT_NORM2_B).data, n->h, W, s))) return rc;
        if ((rc = ifa_moe_route_rows_scores_f32(sp.x_score, n->h, W, T, (int)W, L.T(IFA_LT_X_ROUTER).data, XA, sp.x_top, L.T(IFA_LT_X_CORR).data, n->moe_idx, n->moe_wgt, s))) return rc;
    } else {
        if ((rc = ifa_dyt_f32(n->x, W, T, W, L.T(IFA_LT_NORM2_ALPHA).data, L.T(IFA_LT_NORM2).data, L.T(IFA_LT_NORM2_B).data, n->h, W, s))) return rc;
        if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_X_ROUTER).data, (size_t)XA, W, n->h, W, T, nullptr, nullptr, 1.0f, 0, n->m2, (size_t)XA))) return rc;
        if ((rc = ifa_moe_route_scores_f32(sp.x_score, n->m2, (size_t)XA, T, XA, sp.x_top, L.T(IFA_LT_X_CORR).data, n->moe_idx, n->moe_wgt, s))) return rc;
    }
    return ifa_moe_experts_glu_f32(sp.x_glu, sp.x_limit, n->h, W, T, (int)W, sp.x_ff, sp.x_experts, sp.x_top, L.T(IFA_LT_X_UP).data, L.T(IFA_LT_X_DOWN).data, n->moe_idx,
                                   n->moe_wgt, c.ops32, n->moe_ws, n->moe_ws_bytes, n->x, W, 1, s);
}

// the layers of one step over T rows / nseq sequences whose tables are already on the device; leaves the residual in n->x
int run_layers(ifa_model *m, size_t T, int nseq)
{
    LayeredNet *n = m->lay;
    const ifa_layered_config &c = n->cfg;
    const size_t W = (size_t)c.width;
    ifa_stream s = (ifa_stream)m->stream;
    void *const *slots = (void *const *)n->slot_base_dev;
    int rc;
    if (c.stem == 1) {
        if ((rc = ifa_embed_rows_f32(n->embd.data, c.vocab, c.width, n->tokens_dev, T, n->h, s))) return rc;
        if ((rc = ifa_group_rmsnorm_f32(n->h, W, T, W, c.norm_groups, n->embd_norm.data, c.eps, 0, n->x, W, s))) return rc;
        if (n->any_depth_avg && (rc = ifa_group_rmsnorm_f32(n->h, W, T, W, c.norm_groups, n->embd_norm.data, c.eps, 0, n->stack, W, s))) return rc;      // plane 0
    } else if (c.stem == 2) {
        if ((rc = ifa_embed_pair_f32(n->embd.data, c.vocab, c.width, c.bigram_buckets > 0 ? n->bigram.data : nullptr, c.bigram_buckets, c.bigram_mul_prev, c.bigram_mul_cur,
                                     n->tokens_dev, n->seqs_dev, n->row_seq_dev, T, slots, n->o_prev, n->x, s))) return rc;
    } else if (c.stem == 3) {
        if ((rc = ifa_embed_pair_scaled_f32(n->embd.data, c.vocab, c.width, c.embed_scale != 0.0f ? c.embed_scale : 1.0f, c.bigram_buckets > 0 ? n->bigram.data : nullptr,
                                            c.bigram_buckets, c.bigram_mul_prev, c.bigram_mul_cur, n->tokens_dev, n->seqs_dev, n->row_seq_dev, T, slots, n->o_prev, n->x,
                                            n->x0, s))) return rc;
    } else if ((rc = ifa_embed_sinpos_f32(n->embd.data, c.vocab, c.width, n->tokens_dev, n->pos_dev, T, c.pos_base, n->x, s))) return rc;
    bool h_ready = false;
    for (size_t ri = 0; ri < n->runs.size(); ri++) {
        const size_t li = (size_t)n->runs[ri].first;
        const int pass = n->runs[ri].second;
        LLayer &L = n->layers[li];
        const ifa_layer_spec &sp = L.spec;
        const LLayer *next_layer = ri + 1 < n->runs.size() ? &n->layers[(size_t)n->runs[ri + 1].first] : nullptr;
        // a pass of the looped group starts from x (+ the embedding output, from the second pass on) + the pass's own vector
        const bool pass_start = c.loop_times > 0 && (int)li == c.loop_start && c.loop_start < c.loop_stop;
        if (sp.block == IFA_BLOCK_PRENORM) {
            if ((rc = run_prenorm_layer(m, L, T, nseq, pass, pass_start))) return rc;
            h_ready = false;
            if (n->opt_tap_layers && n->taps && T <= n->taps_rows)
                IFA_HIP_CHECK(hipMemcpyAsync(n->taps + ri * n->taps_rows * W, n->x, T * W * 4, hipMemcpyDeviceToDevice, m->stream));
            continue;
        }
        if (sp.block == IFA_BLOCK_POSTNORM) {
            bool next_ready = false;
            if ((rc = run_postnorm_layer(m, L, li, T, nseq, h_ready, next_layer, &next_ready))) return rc;
            h_ready = next_ready;
            if (n->opt_tap_layers && n->taps && T <= n->taps_rows)
                IFA_HIP_CHECK(hipMemcpyAsync(n->taps + ri * n->taps_rows * W, n->x, T * W * 4, hipMemcpyDeviceToDevice, m->stream));
            continue;
        }
        if (sp.block == IFA_BLOCK_SANDWICH) {
            bool next_ready = false;
            if ((rc = run_sandwich_layer(m, L, T, nseq, h_ready, next_layer, &next_ready))) return rc;
            h_ready = next_ready;
            if (n->opt_tap_layers && n->taps && T <= n->taps_rows)
                IFA_HIP_CHECK(hipMemcpyAsync(n->taps + ri * n->taps_rows * W, n->x, T * W * 4, hipMemcpyDeviceToDevice, m->stream));
            continue;
        }
        const bf16_t *ls1 = (const bf16_t *)L.T(IFA_LT_LS1).data;
        const size_t NI = L.n_in;
        // (the linear attention's q | k | v leave the product through SiLU: contiguous columns [c_lq, c_lg))
        const bool lin = sp.mixer == IFA_MIX_WINDOW_LINEAR;
        // steps of a few rows: the norm is formed inside the product's read of the residual, the gated GELU inside the down-projection's
        const bool fuse = T <= 8 && W % 8 == 0;
        if (fuse && (n->opt_fuse_rows & 1)) {
            if ((rc = ifa_linear_bf16w_rows(1, L.T(IFA_LT_NORM1).data, c.eps, L.w_in, NI, W, n->x, W, T, L.b_in, nullptr, 1.0f, 0, n->proj, NI,
                                            lin ? (int)L.c_lq : 0, lin ? (int)L.c_lg : 0, s))) return rc;
        } else {
            if ((rc = ifa_layernorm_f32(1, n->x, W, T, W, L.T(IFA_LT_NORM1).data, c.eps, n->h, W, s))) return rc;
            if ((rc = linear(m, L.w_in, NI, W, n->h, W, T, L.b_in, nullptr, 1.0f, 0, n->proj, NI, lin ? (int)L.c_lq : 0, lin ? (int)L.c_lg : 0))) return rc;
        }
        if (sp.mixer == IFA_MIX_WINDOW_LINEAR) {
            const size_t AQ = (size_t)sp.a_heads * sp.a_dim, LV = (size_t)sp.l_heads * sp.l_vdim;
            // windowed attention: the values are the keys as projected; the cache's K rows hold the normed keys
            if ((rc = ifa_kv_store_f32(n->proj + L.c_ak, NI, n->proj + L.c_ak, NI, sp.a_kv_heads, sp.a_dim, 1, c.eps, n->seqs_dev, n->row_seq_dev, T, slots,
                                       L.o_k, L.o_v, s))) return rc;
            if ((rc = ifa_attention_window_f32(n->proj + L.c_aq, NI, sp.a_heads, sp.a_kv_heads, sp.a_dim, 1, c.eps, sp.a_scale, sp.a_softcap, sp.a_window,
                                               sp.a_keep_first, L.T(IFA_LT_A_REL).data, L.bucket_of, sp.a_buckets, L.T(IFA_LT_A_SINK).data, n->seqs_dev,
                                               n->row_seq_dev, T, slots, L.o_k, L.o_v, n->m1, AQ, n->seqs_host.data(), (int)n->seqs_host.size(), n->opt_attn_tile_min, n->attn_ws, n->attn_ws_bytes, s))) return rc;
            if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_A_O).data, W, AQ, n->m1, AQ, T, nullptr, ls1, sp.a_out_scale, 1, n->x, W))) return rc;
            // decayed linear attention
            if ((rc = ifa_state_scan_f32(0, 0, n->proj + L.c_lq, NI, n->proj + L.c_lk, NI, n->proj + L.c_lv, NI, sp.l_heads, sp.l_heads, sp.l_dim, sp.l_vdim,
                                         L.T(IFA_LT_L_DECAY).data, nullptr, nullptr, n->seqs_dev, nseq, slots, L.o_lin, n->m2, LV, s))) return rc;
            if ((rc = ifa_gated_groupnorm_f32(n->m2, LV, T, (int)LV, (int)LV, L.T(IFA_LT_L_NORM).data, (int)LV, n->proj + L.c_lg, NI, 0, c.eps, n->m2, LV, s))) return rc;
            if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_L_O).data, W, LV, n->m2, LV, T, nullptr, ls1, sp.l_out_scale, 1, n->x, W))) return rc;
        } else {
            const size_t QK = (size_t)sp.d_kv_heads * sp.d_dim, DV = (size_t)sp.d_heads * sp.d_vdim, C = (size_t)L.conv_ch;
            if ((rc = ifa_shortconv_silu_f32(n->proj + L.c_dq, NI, (int)C, sp.d_conv, L.w_conv, n->seqs_dev, n->row_seq_dev, T, slots, L.o_conv, (int)(2 * QK),
                                             sp.d_dim, 1e-6f, (int)QK, 1.0f / sqrtf((float)sp.d_dim), n->m1, C, s))) return rc;
            if ((rc = ifa_shortconv_tail_f32(n->proj + L.c_dq, NI, (int)C, sp.d_conv, n->seqs_dev, nseq, slots, L.o_conv, s))) return rc;
            if ((rc = ifa_delta_gates_f32(n->proj + L.c_db, NI, n->proj + L.c_da, NI, sp.d_heads, T, L.T(IFA_LT_D_ALOG).data, L.T(IFA_LT_D_DTBIAS).data,
                                          n->beta, n->decay, s))) return rc;
            if ((rc = ifa_state_scan_f32(1, 0, n->m1, C, n->m1 + QK, C, n->m1 + 2 * QK, C, sp.d_heads, sp.d_kv_heads, sp.d_dim, sp.d_vdim, nullptr, n->decay,
                                         n->beta, n->seqs_dev, nseq, slots, L.o_rec, n->m2, DV, s))) return rc;
            if ((rc = ifa_gated_groupnorm_f32(n->m2, DV, T, (int)DV, sp.d_vdim, L.T(IFA_LT_D_NORM).data, sp.d_vdim, n->proj + L.c_dg, NI, 1, c.eps, n->m2, DV, s))) return rc;
            if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_D_O).data, W, DV, n->m2, DV, T, nullptr, ls1, 1.0f, 1, n->x, W))) return rc;
        }
        if (sp.ffn > 0) {
            const size_t F = (size_t)sp.ffn;
            if (fuse && (n->opt_fuse_rows & 2) && F % 8 == 0 && L.c_fg % 4 == 0) {
                if ((rc = ifa_linear_bf16w_rows(2, nullptr, 0.0f, L.T(IFA_LT_FFN_DOWN).data, W, F, n->proj + L.c_fg, NI, T, L.T(IFA_LT_FFN_DOWN_B).data,
                                                L.T(IFA_LT_LS2).data, 1.0f, 1, n->x, W, 0, 0, s))) return rc;
            } else {
                if ((rc = ifa_glu_f32(1, n->proj + L.c_fg, NI, T, F, n->m3, F, s))) return rc;
                if ((rc = linear(m, (const bf16_t *)L.T(IFA_LT_FFN_DOWN).data, W, F, n->m3, F, T, (const bf16_t *)L.T(IFA_LT_FFN_DOWN_B).data,
                                 (const bf16_t *)L.T(IFA_LT_LS2).data, 1.0f, 1, n->x, W))) return rc;
            }
        }
        if (n->opt_tap_layers && n->taps && T <= n->taps_rows)
            IFA_HIP_CHECK(hipMemcpyAsync(n->taps + ri * n->taps_rows * W, n->x, T * W * 4, hipMemcpyDeviceToDevice, m->stream));
    }
    return IFA_OK;
}

float logit_scale_of(const LayeredNet *n) { return n->cfg.stem == 3 && n->cfg.logit_scale != 0.0f ? n->cfg.logit_scale : 1.0f; }

// the norm in front of lm_head: (stem 3) the Dynamic Tanh norm, layer norm without bias, (stem 1) the grouped RMS norm, or (stem 2) the RMS norm with weight (1 + w)
int out_norm_rows(ifa_model *m, const float *src, size_t rows, float *dst)
{
    LayeredNet *n = m->lay;
    const size_t W = (size_t)n->cfg.width;
    if (n->cfg.stem == 1) return ifa_group_rmsnorm_f32(src, W, rows, W, n->cfg.norm_groups, n->out_norm.data, n->cfg.eps, 0, dst, W, (ifa_stream)m->stream);
    if (n->cfg.stem == 2) return ifa_rmsnorm_offset_f32(src, W, rows, W, n->out_norm.data, 1.0f, n->cfg.eps, 0, dst, W, (ifa_stream)m->stream);
    if (n->cfg.stem == 3) return ifa_dyt_f32(src, W, rows, W, n->out_norm_alpha.data, n->out_norm.data, n->out_norm_b.data, dst, W, (ifa_stream)m->stream);
    return ifa_layernorm_f32(1, src, W, rows, W, n->out_norm.data, n->cfg.eps, dst, W, (ifa_stream)m->stream);
}

// final norm + lm_head over rows [r0, r0 + nr) of the residual -> n->logits rows [0, nr)
int run_head(ifa_model *m, size_t r0, size_t nr)
{
    LayeredNet *n = m->lay;
    const size_t W = (size_t)n->cfg.width, V = (size_t)n->cfg.vocab;
    int rc;
    if ((n->opt_fuse_rows & 1) && nr <= 8 && W % 8 == 0 && n->cfg.stem == 0) {
        if ((rc = ifa_linear_bf16w_rows(1, n->out_norm.data, n->cfg.eps, n->lm_head.data, V, W, n->x + r0 * W, W, nr, nullptr, nullptr, 1.0f, 0, n->logits, V, 0, 0,
                                        (ifa_stream)m->stream))) return rc;
        n->logits_rows = nr;
        return IFA_OK;
    }
    if ((rc = out_norm_rows(m, n->x + r0 * W, nr, n->h))) return rc;
    if ((rc = linear(m, (const bf16_t *)n->lm_head.data, V, W, n->h, W, nr, nullptr, nullptr, logit_scale_of(n), 0, n->logits, V))) return rc;
    if (n->cfg.logit_softcap > 0.0f && (rc = ifa_softcap_f32(n->logits, nr * V, n->cfg.logit_softcap, (ifa_stream)m->stream))) return rc;
    n->logits_rows = nr;
    return IFA_OK;
}

__global__ void k_lay_advance(int *tokens, int *pos, ifa_seq_desc *seqs, const int *next, int *ring, int step)
{
    tokens[0] = next[0]; pos[0] += 1; seqs[0].pos0 += 1; ring[step] = next[0];
}

// ---- the worker class
int lay_destroy(ifa_model *m)
{
    LayeredNet *n = m->lay;
    (void)hipSetDevice(m->cfg.device);
    if (m->stream) (void)hipStreamSynchronize(m->stream);
    drop_step_graph(n);
    for (LLayer &L : n->layers) {
        for (LTensor &t : L.t) lay_free(t.data);
        lay_free(L.w_in); lay_free(L.b_in); lay_free(L.w_conv); lay_free(L.bucket_of); lay_free(L.freq); lay_free(L.w_in2); lay_free(L.b_in2); lay_free(L.freq_v);
    }
    lay_free(n->embd.data); lay_free(n->out_norm.data); lay_free(n->lm_head.data); lay_free(n->embd_norm.data); lay_free(n->bigram.data);
    lay_free(n->out_norm_b.data); lay_free(n->out_norm_alpha.data); lay_free(n->loop_step.data);
    lay_free(n->x0); lay_free(n->cg_decay); lay_free(n->cg_unit); lay_free(n->cg_rem);
    lay_free(n->m4); lay_free(n->m5); lay_free(n->stack); lay_free(n->moe_wgt); lay_free(n->moe_idx); lay_free(n->moe_ws); lay_free(n->kx); lay_free(n->vx);
    for (float *p : n->slot_ptr) lay_free(p);
    lay_free(n->slot_base_dev);
    if (n->tab_pin) (void)hipHostFree(n->tab_pin);
    lay_free(n->attn_ws);
    lay_free(n->tab_dev); lay_free(n->excl_dev); lay_free(n->next_dev); lay_free(n->ring_dev);
    float *bufs[] = {n->x, n->h, n->proj, n->m1, n->m2, n->m3, n->beta, n->decay, n->logits, n->taps};
    for (float *b : bufs) lay_free(b);
    if (m->stream && m->own_stream) (void)hipStreamDestroy(m->stream);
    delete n;
    delete m;
    return IFA_OK;
}

int cat_rows(std::vector<bf16_t> &w, std::vector<bf16_t> &b, const LTensor &t, const LTensor *bias, size_t K, size_t &off, hipStream_t s)
{
    IFA_REQUIRE(t.present() && t.cols == K, "layer-list worker: a projection is missing or has %zu columns instead of %zu", t.cols, K);
    off = b.size();
    const size_t old = w.size();
    w.resize(old + t.rows * K);
    IFA_HIP_CHECK(hipMemcpy(w.data() + old, t.data, t.rows * K * 2, hipMemcpyDeviceToHost));
    b.resize(off + t.rows, 0);
    if (bias && bias->present()) IFA_HIP_CHECK(hipMemcpy(b.data() + off, bias->data, t.rows * 2, hipMemcpyDeviceToHost));
    return IFA_OK;
}

int lay_finalize(ifa_model *m)
{
    LayeredNet *n = m->lay;
    IFA_HIP_CHECK(hipSetDevice(m->cfg.device));
    const size_t W = (size_t)n->cfg.width;
    IFA_REQUIRE(n->embd.present() && n->out_norm.present() && n->lm_head.present(), "layer-list worker: embedding, final norm or lm_head is missing");
    IFA_REQUIRE(n->cfg.stem != 1 || n->embd_norm.present(), "layer-list worker: the norm behind the embedding is missing");
    IFA_REQUIRE((n->cfg.stem != 2 && n->cfg.stem != 3) || n->cfg.bigram_buckets <= 0 || n->bigram.present(), "layer-list worker: the token-pair embedding is missing");
    IFA_REQUIRE(n->cfg.stem != 3 || (n->out_norm_b.present() && n->out_norm_alpha.present()), "layer-list worker: bias or scalar of the final norm is missing");
    const bool looped = n->cfg.loop_times > 0 && n->cfg.loop_start < n->cfg.loop_stop;
    IFA_REQUIRE(!looped || n->loop_step.present(), "layer-list worker: the vectors of the looped group's passes are missing");
    size_t off = 0;
    if (n->cfg.stem == 2 || n->cfg.stem == 3) { n->o_prev = off; off += 4; }
    n->n_in_max = n->mix_max = n->ffn_max = n->heads_max = 4;
    for (size_t li = 0; li < n->layers.size(); li++) {
        LLayer &L = n->layers[li];
        const ifa_layer_spec &sp = L.spec;
        if (L.w_in) continue;          // finalized before
        const size_t off_layer = off;
        for (int id = IFA_LT_NORM1; id < IFA_LT_END; id++) {
            size_t r, c; bool vec;
            if (expected_shape(n, sp, (int)li, id, r, c, vec)) IFA_REQUIRE(L.T(id).present(), "layer-list worker: tensor %d of layer %zu is missing", id, li);
        }
        std::vector<bf16_t> w, b;
        int rc;
        if (sp.mixer == IFA_MIX_LATENT) {
            if ((rc = cat_rows(w, b, L.T(sp.m_q_rank > 0 ? IFA_LT_M_DQ : IFA_LT_M_Q), nullptr, W, L.c_mq, m->stream))
                || (rc = cat_rows(w, b, L.T(IFA_LT_M_DKV), nullptr, W, L.c_mkv, m->stream))
                || (sp.m_gate && (rc = cat_rows(w, b, L.T(IFA_LT_M_G), nullptr, W, L.c_mg, m->stream)))) return rc;
            // rotation frequencies in double: base^(-2i / dims), YaRN: the scaled and the plain frequency blended by a ramp over i
            const int half = sp.m_rot_dims / 2;
            std::vector<double> fr((size_t)std::max(half, 1), 0.0);
            L.rot_mult = 1.0f;
            const double dims = (double)sp.m_rot_dims, base = (double)sp.m_rot_base;
            for (int i = 0; i < half; i++) fr[(size_t)i] = std::pow(base, -2.0 * i / dims);
            if (sp.m_yarn_factor > 0.0f) {
                const double factor = sp.m_yarn_factor, orig = sp.m_yarn_original, two_pi = 6.283185307179586476925;
                auto dim_of = [&](double turns) { return dims * std::log(orig / (two_pi * turns)) / (2.0 * std::log(base)); };
                const double lo = std::max(std::floor(dim_of(sp.m_yarn_fast)), 0.0), hi = std::min(std::ceil(dim_of(sp.m_yarn_slow)), dims - 1.0);
                for (int i = 0; i < half; i++) {
                    const double ramp = std::min(1.0, std::max(0.0, ((double)i - lo) / std::max(hi - lo, 0.001)));
                    fr[(size_t)i] = fr[(size_t)i] / factor * ramp + fr[(size_t)i] * (1.0 - ramp);
                }
                L.rot_mult = (float)(0.1 * std::log(factor) + 1.0);
            }
            IFA_HIP_CHECK(hipMalloc((void **)&L.freq, fr.size() * 8));
            IFA_HIP_CHECK(hipMemcpy(L.freq, fr.data(), fr.size() * 8, hipMemcpyHostToDevice));
            const size_t CR = (size_t)(sp.m_kv_rank + sp.m_rot_dim), H = (size_t)sp.m_heads;
            L.o_c = off; off += align4((size_t)n->cfg.max_ctx * CR);
            if (sp.canon_taps > 1) { L.o_cv1 = off; off += align4((size_t)(sp.canon_taps - 1) * W); }
            n->mix_max = std::max({n->mix_max, H * (size_t)(sp.m_dim + sp.m_rot_dim), H * CR, H * (size_t)sp.m_vdim, W, (size_t)sp.m_q_rank});
            n->ffn_max = std::max(n->ffn_max, (size_t)sp.m_q_rank);
            n->kx_max = std::max(n->kx_max, H * (size_t)sp.m_dim); n->vx_max = std::max(n->vx_max, H * (size_t)sp.m_vdim);
            n->any_latent = true;
            if ((rc = ifa_attention_latent_rows_reserve(sp.m_kv_rank, sp.m_rot_dim))) return rc;      // (the single-token step may be captured)
            if (!ifa_attention_latent_tile_fits(sp.m_dim, sp.m_rot_dim, sp.m_vdim)) n->latent_tile_ok = false;
            if (has_moe(sp)) {
                if (sp.canon_taps > 1) { L.o_cv2 = off; off += align4((size_t)(sp.canon_taps - 1) * W); }
                n->mix_max = std::max(n->mix_max, (size_t)(sp.x_experts + sp.x_identity));
                n->top_max = std::max(n->top_max, (size_t)sp.x_top);
                n->any_moe = true;
            }
            if (sp.depth_avg) n->any_depth_avg = true;
        } else if (sp.mixer == IFA_MIX_ROTARY) {
            const bool own = sp.a_kv_layer == 0;
            if ((rc = cat_rows(w, b, L.T(IFA_LT_A_Q), &L.T(IFA_LT_A_Q_B), W, L.c_aq, m->stream))) return rc;
            while (b.size() % 4) { w.resize(w.size() + W, 0); b.push_back(0); }      // (keys and values start on 16-byte borders of the product's rows)
            if (own && ((rc = cat_rows(w, b, L.T(IFA_LT_A_K), &L.T(IFA_LT_A_K_B), W, L.c_ak, m->stream)))) return rc;
            while (b.size() % 4) { w.resize(w.size() + W, 0); b.push_back(0); }
            if (own && ((rc = cat_rows(w, b, L.T(IFA_LT_A_V), &L.T(IFA_LT_A_V_B), W, L.c_av, m->stream)))) return rc;
            const int half = sp.a_rot_dims / 2;
            std::vector<double> fr((size_t)std::max(half, 1), 0.0);
            for (int i = 0; i < half; i++) fr[(size_t)i] = std::pow((double)sp.a_rot_base, -2.0 * i / (double)sp.a_rot_dims);
            if (sp.a_rot_scale_factor > 0.0f) {
                // by wavelength: short waves keep their frequency, long ones are slowed by the factor, a linear blend between
                const double factor = sp.a_rot_scale_factor, lo = sp.a_rot_scale_low, hi = sp.a_rot_scale_high, orig = sp.a_rot_scale_original, two_pi = 6.283185307179586476925;
                for (int i = 0; i < half; i++) {
                    const double f = fr[(size_t)i], wl = two_pi / f;
                    if (wl < orig / hi) continue;
                    if (wl > orig / lo) { fr[(size_t)i] = f / factor; continue; }
                    const double sm = (orig / wl - lo) / (hi - lo);
                    fr[(size_t)i] = (1.0 - sm) * f / factor + sm * f;
                }
            }
            IFA_HIP_CHECK(hipMalloc((void **)&L.freq, fr.size() * 8));
            IFA_HIP_CHECK(hipMemcpy(L.freq, fr.data(), fr.size() * 8, hipMemcpyHostToDevice));
            if (sp.a_vrot) {      // the values turn over their whole head with the plain frequencies
                const int vh = sp.a_vdim / 2;
                std::vector<double> fv((size_t)std::max(vh, 1), 0.0);
                for (int i = 0; i < vh; i++) fv[(size_t)i] = std::pow((double)sp.a_rot_base, -2.0 * i / (double)sp.a_vdim);
                IFA_HIP_CHECK(hipMalloc((void **)&L.freq_v, fv.size() * 8));
                IFA_HIP_CHECK(hipMemcpy(L.freq_v, fv.data(), fv.size() * 8, hipMemcpyHostToDevice));
            }
            if (own) {
                L.o_k = off; off += align4((size_t)n->cfg.max_ctx * sp.a_kv_heads * sp.a_dim);
                L.o_v = off; off += align4((size_t)n->cfg.max_ctx * sp.a_kv_heads * sp.a_vdim);
            }
            n->mix_max = std::max({n->mix_max, (size_t)sp.a_heads * sp.a_dim, (size_t)sp.a_heads * sp.a_vdim, W});
            // the second product and the sizes of the feed-forward's buffers
            std::vector<bf16_t> w2, b2;
            size_t dummy;
            if (sp.block == IFA_BLOCK_PRENORM) {      // (the router stays a product of its own: its choice takes it in for steps of a few rows)
                if (has_moe(sp)) {
                    n->mix_max = std::max(n->mix_max, (size_t)sp.x_experts);
                    n->top_max = std::max(n->top_max, (size_t)sp.x_top);
                    n->any_moe = true;
                }
            } else
            if (has_moe(sp)) {
                if ((rc = cat_rows(w2, b2, L.T(IFA_LT_X_ROUTER), sp.x_route == 1 ? &L.T(IFA_LT_X_ROUTER_B) : nullptr, W, L.c2_router, m->stream))) return rc;
                if (sp.x_shared_ff > 0) {
                    LTensor sg = L.T(IFA_LT_X_SH_SG); sg.rows = 1; sg.cols = W;
                    if ((rc = cat_rows(w2, b2, sg, nullptr, W, L.c2_sg, m->stream))) return rc;
                    while (b2.size() % 4) { w2.resize(w2.size() + W, 0); b2.push_back(0); }
                    if ((rc = cat_rows(w2, b2, L.T(IFA_LT_X_SH_GATE), nullptr, W, L.c2_shg, m->stream)) || (rc = cat_rows(w2, b2, L.T(IFA_LT_X_SH_UP), nullptr, W, dummy, m->stream))) return rc;
                    n->ffn_max = std::max(n->ffn_max, (size_t)sp.x_shared_ff);
                }
                n->top_max = std::max(n->top_max, (size_t)sp.x_top);
                n->any_moe = true;
            } else if (sp.ffn > 0) {
                if ((rc = cat_rows(w2, b2, L.T(IFA_LT_FFN_GATE), nullptr, W, L.c2_fg, m->stream)) || (rc = cat_rows(w2, b2, L.T(IFA_LT_FFN_UP), nullptr, W, dummy, m->stream))) return rc;
                n->ffn_max = std::max(n->ffn_max, (size_t)sp.ffn);
            }
            if (!b2.empty()) {
                while (b2.size() % 4) { w2.resize(w2.size() + W, 0); b2.push_back(0); }
                L.n_in2 = b2.size();
                IFA_HIP_CHECK(hipMalloc((void **)&L.w_in2, w2.size() * 2));
                IFA_HIP_CHECK(hipMalloc((void **)&L.b_in2, b2.size() * 2));
                IFA_HIP_CHECK(hipMemcpy(L.w_in2, w2.data(), w2.size() * 2, hipMemcpyHostToDevice));
                IFA_HIP_CHECK(hipMemcpy(L.b_in2, b2.data(), b2.size() * 2, hipMemcpyHostToDevice));
                n->n_in_max = std::max(n->n_in_max, L.n_in2);
            }
        } else if (sp.mixer == IFA_MIX_CHAN_DELTA) {
            if ((rc = cat_rows(w, b, L.T(IFA_LT_C_R), nullptr, W, L.c_cr, m->stream)) || (rc = cat_rows(w, b, L.T(IFA_LT_C_K), nullptr, W, L.c_ck, m->stream))
                || (rc = cat_rows(w, b, L.T(IFA_LT_C_V), nullptr, W, L.c_cv, m->stream)) || (rc = cat_rows(w, b, L.T(IFA_LT_C_G), nullptr, W, L.c_cg, m->stream))
                || (rc = cat_rows(w, b, L.T(IFA_LT_C_A), &L.T(IFA_LT_C_A_B), W, L.c_ca, m->stream)) || (rc = cat_rows(w, b, L.T(IFA_LT_C_W1), nullptr, W, L.c_cw, m->stream))) return rc;
            const size_t CH = (size_t)sp.c_heads * sp.c_dim;
            L.o_rec = off; off += align4((size_t)sp.c_heads * sp.c_dim * sp.c_dim);
            n->mix_max = std::max({n->mix_max, CH, W});
            n->chan_max = std::max(n->chan_max, CH);
            if (has_moe(sp)) {
                n->mix_max = std::max(n->mix_max, (size_t)sp.x_experts);
                n->top_max = std::max(n->top_max, (size_t)sp.x_top);
                n->any_moe = true;
            }
        } else if (sp.mixer == IFA_MIX_WINDOW_LINEAR) {
            if ((rc = cat_rows(w, b, L.T(IFA_LT_A_Q), nullptr, W, L.c_aq, m->stream)) || (rc = cat_rows(w, b, L.T(IFA_LT_A_K), nullptr, W, L.c_ak, m->stream))
                || (rc = cat_rows(w, b, L.T(IFA_LT_L_Q), nullptr, W, L.c_lq, m->stream)) || (rc = cat_rows(w, b, L.T(IFA_LT_L_K), nullptr, W, L.c_lk, m->stream))
                || (rc = cat_rows(w, b, L.T(IFA_LT_L_V), nullptr, W, L.c_lv, m->stream)) || (rc = cat_rows(w, b, L.T(IFA_LT_L_G), nullptr, W, L.c_lg, m->stream))) return rc;
            std::vector<int> bk;
            build_buckets(bk, n->cfg.max_ctx, sp.a_buckets, sp.a_bias_max);
            IFA_HIP_CHECK(hipMalloc((void **)&L.bucket_of, bk.size() * 4));
            IFA_HIP_CHECK(hipMemcpy(L.bucket_of, bk.data(), bk.size() * 4, hipMemcpyHostToDevice));
            const size_t kv = align4((size_t)n->cfg.max_ctx * sp.a_kv_heads * sp.a_dim);
            L.o_k = off; off += kv; L.o_v = off; off += kv;
            L.o_lin = off; off += align4((size_t)sp.l_heads * sp.l_dim * sp.l_vdim);
            n->mix_max = std::max({n->mix_max, (size_t)sp.a_heads * sp.a_dim, (size_t)sp.l_heads * sp.l_vdim});
            n->heads_max = std::max(n->heads_max, (size_t)std::max(sp.a_heads, sp.l_heads));
        } else {
            size_t dk_off, dv_off;
            if ((rc = cat_rows(w, b, L.T(IFA_LT_D_Q), nullptr, W, L.c_dq, m->stream)) || (rc = cat_rows(w, b, L.T(IFA_LT_D_K), nullptr, W, dk_off, m->stream))
                || (rc = cat_rows(w, b, L.T(IFA_LT_D_V), nullptr, W, dv_off, m->stream)) || (rc = cat_rows(w, b, L.T(IFA_LT_D_B), nullptr, W, L.c_db, m->stream))
                || (rc = cat_rows(w, b, L.T(IFA_LT_D_A), nullptr, W, L.c_da, m->stream)) || (rc = cat_rows(w, b, L.T(IFA_LT_D_G), nullptr, W, L.c_dg, m->stream))) return rc;
            const size_t QK = (size_t)sp.d_kv_heads * sp.d_dim, DV = (size_t)sp.d_heads * sp.d_vdim;
            L.conv_ch = (int)(2 * QK + DV);
            std::vector<bf16_t> cw((size_t)L.conv_ch * sp.d_conv);
            IFA_HIP_CHECK(hipMemcpy(cw.data(), L.T(IFA_LT_D_QCONV).data, QK * sp.d_conv * 2, hipMemcpyDeviceToHost));
            IFA_HIP_CHECK(hipMemcpy(cw.data() + QK * sp.d_conv, L.T(IFA_LT_D_KCONV).data, QK * sp.d_conv * 2, hipMemcpyDeviceToHost));
            IFA_HIP_CHECK(hipMemcpy(cw.data() + 2 * QK * sp.d_conv, L.T(IFA_LT_D_VCONV).data, DV * sp.d_conv * 2, hipMemcpyDeviceToHost));
            IFA_HIP_CHECK(hipMalloc((void **)&L.w_conv, cw.size() * 2));
            IFA_HIP_CHECK(hipMemcpy(L.w_conv, cw.data(), cw.size() * 2, hipMemcpyHostToDevice));
            L.o_rec = off; off += align4((size_t)sp.d_heads * sp.d_dim * sp.d_vdim);
            L.o_conv = off; off += align4((size_t)std::max(sp.d_conv - 1, 0) * L.conv_ch);
            n->mix_max = std::max({n->mix_max, (size_t)L.conv_ch, DV});
            n->heads_max = std::max(n->heads_max, (size_t)sp.d_heads);
        }
        // a layer of a looped group: its part of the arena once per pass
        if (looped && (int)li >= n->cfg.loop_start && (int)li < n->cfg.loop_stop && n->cfg.loop_times > 1) {
            L.pass_stride = off - off_layer;
            off += (size_t)(n->cfg.loop_times - 1) * L.pass_stride;
        }
        if (sp.ffn > 0 && sp.block != IFA_BLOCK_SANDWICH) {
            size_t up_off;
            if ((rc = cat_rows(w, b, L.T(IFA_LT_FFN_GATE), &L.T(IFA_LT_FFN_GATE_B), W, L.c_fg, m->stream))
                || (rc = cat_rows(w, b, L.T(IFA_LT_FFN_UP), &L.T(IFA_LT_FFN_UP_B), W, up_off, m->stream))) return rc;
            n->ffn_max = std::max(n->ffn_max, (size_t)sp.ffn);
        }
        L.n_in = b.size();
        // the product's row stride: a multiple of 4 floats so that every row of it starts 16-byte aligned
        while (L.n_in % 4) { w.resize(w.size() + W, 0); b.push_back(0); L.n_in++; }
        IFA_HIP_CHECK(hipMalloc((void **)&L.w_in, w.size() * 2));
        IFA_HIP_CHECK(hipMalloc((void **)&L.b_in, b.size() * 2));
        IFA_HIP_CHECK(hipMemcpy(L.w_in, w.data(), w.size() * 2, hipMemcpyHostToDevice));
        IFA_HIP_CHECK(hipMemcpy(L.b_in, b.data(), b.size() * 2, hipMemcpyHostToDevice));
        n->n_in_max = std::max(n->n_in_max, L.n_in);
        // the separate copies of what the fused product now holds are no longer needed
        for (int id : {IFA_LT_A_Q, IFA_LT_A_K, IFA_LT_L_Q, IFA_LT_L_K, IFA_LT_L_V, IFA_LT_L_G, IFA_LT_D_Q, IFA_LT_D_K, IFA_LT_D_V, IFA_LT_D_B, IFA_LT_D_A,
                       IFA_LT_D_G, IFA_LT_FFN_GATE, IFA_LT_FFN_UP, IFA_LT_M_Q, IFA_LT_M_DQ, IFA_LT_M_DKV, IFA_LT_M_G, IFA_LT_A_V, IFA_LT_A_Q_B, IFA_LT_A_K_B,
                       IFA_LT_A_V_B, IFA_LT_X_ROUTER_B, IFA_LT_X_SH_GATE, IFA_LT_X_SH_UP, IFA_LT_X_SH_SG, IFA_LT_C_R, IFA_LT_C_K, IFA_LT_C_V, IFA_LT_C_G, IFA_LT_C_A,
                       IFA_LT_C_A_B, IFA_LT_C_W1}) {
            LTensor &t = L.T(id);
            if (t.data) { lay_free(t.data); t.data = nullptr; }
        }
        if (sp.block == IFA_BLOCK_SANDWICH) { LTensor &t = L.T(IFA_LT_X_ROUTER); if (t.data) { lay_free(t.data); t.data = nullptr; } }
    }
    if (!n->attn_ws) {
        size_t per_row = 0;
        for (const LLayer &L : n->layers)
            if (L.spec.mixer == IFA_MIX_WINDOW_LINEAR) per_row = std::max(per_row, (size_t)L.spec.a_heads * 32 * ((size_t)L.spec.a_dim + 2) * 4);
            else if (L.spec.mixer == IFA_MIX_ROTARY) per_row = std::max(per_row, (size_t)L.spec.a_heads * 32 * ((size_t)L.spec.a_vdim + 2) * 4);
            else if (L.spec.mixer == IFA_MIX_LATENT) per_row = std::max(per_row, (size_t)L.spec.m_heads * 16 * ((size_t)L.spec.m_kv_rank + 2) * 4);
        n->attn_ws_bytes = per_row * 64;
        if (n->attn_ws_bytes) IFA_HIP_CHECK(hipMalloc((void **)&n->attn_ws, n->attn_ws_bytes));
    }
    // the stack as it is walked: the layers before the looped group, the group once per pass, the layers behind it
    n->runs.clear();
    for (int li = 0; li < (int)n->layers.size(); li++) {
        if (looped && li == n->cfg.loop_start) {
            for (int t = 0; t < n->cfg.loop_times; t++)
                for (int lj = n->cfg.loop_start; lj < n->cfg.loop_stop; lj++) n->runs.push_back({lj, t});
            li = n->cfg.loop_stop - 1;
            continue;
        }
        n->runs.push_back({li, 0});
    }
    if (!n->slot_base_dev) {
        n->arena_floats = off;
        n->slot_ptr.assign((size_t)MAX_SLOTS, nullptr);
        IFA_HIP_CHECK(hipMalloc((void **)&n->slot_base_dev, sizeof(float *) * MAX_SLOTS));
        IFA_HIP_CHECK(hipMemset(n->slot_base_dev, 0, sizeof(float *) * MAX_SLOTS));
        IFA_HIP_CHECK(hipMalloc((void **)&n->excl_dev, 4 * sizeof(int)));
        IFA_HIP_CHECK(hipMemset(n->excl_dev, 0, 4 * sizeof(int)));
        IFA_HIP_CHECK(hipMalloc((void **)&n->next_dev, sizeof(int) * ifa_model::RING));
        IFA_HIP_CHECK(hipMalloc((void **)&n->ring_dev, sizeof(int) * ifa_model::RING));
    }
    m->finalized = true;
    return IFA_OK;
}

int lay_reset(ifa_model *m) { IFA_REQUIRE(m->finalized, "ifa_model_reset: model not finalized"); return IFA_OK; }      // (position 0 restarts every state)

int lay_kv_slots(ifa_model *m, int n_slots)
{
    IFA_REQUIRE(m->finalized, "ifa_model_kv_slots: model not finalized");
    IFA_REQUIRE(n_slots >= 1 && n_slots <= MAX_SLOTS, "ifa_model_kv_slots: n_slots %d", n_slots);
    IFA_REQUIRE(n_slots >= m->lay->n_slots, "ifa_model_kv_slots: cannot shrink below %d slots", m->lay->n_slots);
    m->lay->n_slots = n_slots;
    return IFA_OK;
}

int lay_select_kv(ifa_model *m, int slot)
{
    IFA_REQUIRE(m->finalized, "ifa_model_select_kv: model not finalized");
    IFA_REQUIRE(slot >= 0 && slot < m->lay->n_slots, "ifa_model_select_kv: slot %d of %d", slot, m->lay->n_slots);
    m->lay->cur_slot = slot; m->cur_slot = slot;
    return IFA_OK;
}

int lay_set_option(ifa_model *m, const char *name, int value)
{
    LayeredNet *n = m->lay;
    if (!strcmp(name, "tap_layers")) { n->opt_tap_layers = value; drop_step_graph(n); return IFA_OK; }
    if (!strcmp(name, "fuse_rows")) { n->opt_fuse_rows = value; drop_step_graph(n); return IFA_OK; }
    if (!strcmp(name, "fuse_post")) { n->opt_fuse_post = value; drop_step_graph(n); return IFA_OK; }
    if (!strcmp(name, "attn_tile_min")) { n->opt_attn_tile_min = value; return IFA_OK; }
    if (!strcmp(name, "graph")) { n->opt_graph = value; drop_step_graph(n); return IFA_OK; }
    if (!strcmp(name, "ops32")) { IFA_HIP_CHECK(hipStreamSynchronize(m->stream)); n->cfg.ops32 = value ? 1 : 0; drop_step_graph(n); return IFA_OK; }
    return ifa_fail(IFA_ERR_ARG, "ifa_model_set_option: unknown option '%s' (layer-list model: tap_layers, graph, ops32, attn_tile_min, fuse_rows, fuse_post)", name);
}

int lay_set_excluded(ifa_model *m, const int *ids_host, int cnt)
{
    IFA_REQUIRE(m->finalized, "ifa_model_set_excluded_tokens: model not finalized");
    IFA_REQUIRE(cnt >= 0 && cnt <= 3 && (cnt == 0 || ids_host), "ifa_model_set_excluded_tokens: n %d (0..3)", cnt);
    int v[4] = {cnt, -1, -1, -1};
    for (int i = 0; i < cnt; i++) v[1 + i] = ids_host[i];
    IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
    IFA_HIP_CHECK(hipMemcpy(m->lay->excl_dev, v, sizeof(v), hipMemcpyHostToDevice));
    return IFA_OK;
}

int lay_get_buffer(ifa_model *m, const char *name, int layer, void **dptr, size_t *bytes)
{
    LayeredNet *n = m->lay;
    size_t b = 0; void *p = nullptr;
    if (!strcmp(name, "logits")) { p = n->logits; b = n->logits_rows * (size_t)n->cfg.vocab * 4; }
    else if (!strcmp(name, "x")) { p = n->x; b = n->scratch_rows * (size_t)n->cfg.width * 4; }
    else if (!strcmp(name, "layer_taps")) {      // [layer runs][taps_rows][width] fp32: the residual after every layer run of the last step (option tap_layers;
                                                 // a layer of a looped group counts once per pass)
        IFA_REQUIRE(n->taps, "ifa_model_get_buffer: no taps (set option tap_layers before the step)");
        IFA_REQUIRE(layer >= 0 && layer < (int)n->runs.size(), "ifa_model_get_buffer: layer run %d", layer);
        p = n->taps + (size_t)layer * n->taps_rows * n->cfg.width; b = n->taps_rows * (size_t)n->cfg.width * 4;
    } else if (!strcmp(name, "slot")) {          // the arena of slot `layer`
        IFA_REQUIRE(layer >= 0 && layer < n->n_slots, "ifa_model_get_buffer: slot %d", layer);
        p = n->slot_ptr[(size_t)layer]; b = p ? n->arena_floats * 4 : 0;
    } else return ifa_fail(IFA_ERR_ARG, "ifa_model_get_buffer: unknown buffer '%s'", name);
    *dptr = p;
    if (bytes) *bytes = b;
    return IFA_OK;
}

// tables of a step -> device
int upload_tables(ifa_model *m, const std::vector<int> &tokens, const std::vector<int> &pos, const std::vector<int> &row_seq, const std::vector<ifa_seq_desc> &seqs)
{
    LayeredNet *n = m->lay;
    const size_t T = tokens.size(), S = seqs.size(), R = n->tab_rows;
    memcpy(n->tab_pin, tokens.data(), T * 4);
    memcpy(n->tab_pin + R, pos.data(), T * 4);
    memcpy(n->tab_pin + 2 * R, row_seq.data(), T * 4);
    memcpy(n->tab_pin + 3 * R, seqs.data(), S * sizeof(ifa_seq_desc));
    n->seqs_host = seqs;
    // first row of every sequence in the expanded key / value scratch (its position 0), for steps that take the tiled latent attention
    n->ctx0_host.assign(S, 0);
    size_t ctx_rows = 0;
    for (size_t q = 0; q < S; q++) { n->ctx0_host[q] = (int)ctx_rows; ctx_rows += (size_t)seqs[q].pos0 + seqs[q].n; }
    n->step_ctx_rows = ctx_rows;
    memcpy(n->tab_pin + 3 * R + 4 * n->tab_seqs, n->ctx0_host.data(), S * 4);
    IFA_HIP_CHECK(hipMemcpyAsync(n->tab_dev, n->tab_pin, (3 * R + 4 * n->tab_seqs + S) * 4, hipMemcpyHostToDevice, m->stream));
    return IFA_OK;
}

int check_span(ifa_model *m, int n_tokens, int start, const int *tokens)
{
    const ifa_layered_config &c = m->lay->cfg;
    IFA_REQUIRE(n_tokens >= 1 && start >= 0 && start + n_tokens <= c.max_ctx, "layer-list worker: tokens [%d, %d) exceed the context of %d", start, start + n_tokens, c.max_ctx);
    for (int i = 0; tokens && i < n_tokens; i++) IFA_REQUIRE(tokens[i] >= 0 && tokens[i] < c.vocab, "layer-list worker: token id %d out of range", tokens[i]);
    return IFA_OK;
}

int ensure_taps(ifa_model *m, size_t T)
{
    LayeredNet *n = m->lay;
    if (!n->opt_tap_layers || T <= n->taps_rows) return IFA_OK;
    IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
    lay_free(n->taps); n->taps = nullptr;
    IFA_HIP_CHECK(hipMalloc((void **)&n->taps, std::max(n->runs.size(), n->layers.size()) * T * (size_t)n->cfg.width * 4));
    n->taps_rows = T;
    return IFA_OK;
}

// One step over several sequences: sequence q brings lens[q] tokens (concatenated in tokens_host) at positions [pos0[q], pos0[q] + lens[q])
// of the query in slot slots[q].  logits_mode 0: only the last row of every sequence goes through the head (rows of n->logits = sequences),
// 1: every row does.  next_tokens_host[q] = greedy token after the last row of sequence q.
int lay_step(ifa_model *m, int nseq, const int *tokens_host, const int *lens, const int *pos0, const int *slots, int logits_mode, int *next_tokens_host)
{
    LayeredNet *n = m->lay;
    IFA_REQUIRE(nseq >= 1 && nseq <= ifa_model::RING && tokens_host && lens && pos0 && slots, "layer-list step: bad arguments");
    IFA_HIP_CHECK(hipSetDevice(m->cfg.device));
    int rc;
    size_t T = 0;
    for (int q = 0; q < nseq; q++) {
        if ((rc = check_span(m, lens[q], pos0[q], tokens_host + T)) || (rc = ensure_slot(m, slots[q]))) return rc;
        for (int b = 0; b < q; b++) IFA_REQUIRE(slots[q] != slots[b], "layer-list step: slot %d used twice", slots[q]);
        T += (size_t)lens[q];
    }
    const size_t V = (size_t)n->cfg.vocab, W = (size_t)n->cfg.width;
    const bool all = logits_mode != 0 || T == (size_t)nseq;
    if ((rc = ensure_rows(m, T, (size_t)nseq)) || (rc = ensure_taps(m, T)) || (rc = ensure_logits(m, all ? T : (size_t)nseq))) return rc;
    std::vector<int> tok(tokens_host, tokens_host + T), pos(T), rs(T), last((size_t)nseq);
    std::vector<ifa_seq_desc> sq((size_t)nseq);
    size_t r = 0;
    for (int q = 0; q < nseq; q++) {
        sq[(size_t)q] = ifa_seq_desc{(int)r, lens[q], pos0[q], slots[q]};
        for (int i = 0; i < lens[q]; i++, r++) { pos[r] = pos0[q] + i; rs[r] = q; }
        last[(size_t)q] = (int)r - 1;
    }
    if ((rc = upload_tables(m, tok, pos, rs, sq))) return rc;
    // prompts through latent attention: expanded keys / values + the tiled kernel when a sequence brings enough rows
    n->step_expand = false;
    if (n->any_latent && n->latent_tile_ok) {
        int longest = 0;
        for (int q = 0; q < nseq; q++) longest = std::max(longest, lens[q]);
        n->step_expand = longest >= n->opt_attn_tile_min;
    }
    if (n->step_expand && n->step_ctx_rows > n->expand_rows) {
        IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
        lay_free(n->kx); lay_free(n->vx); n->kx = n->vx = nullptr;
        IFA_HIP_CHECK(hipMalloc((void **)&n->kx, n->step_ctx_rows * n->kx_max * 4));
        IFA_HIP_CHECK(hipMalloc((void **)&n->vx, n->step_ctx_rows * n->vx_max * 4));
        n->expand_rows = n->step_ctx_rows;
    }
    if ((rc = run_layers(m, T, nseq))) return rc;
    ifa_stream s = (ifa_stream)m->stream;
    if (all) {
        if ((rc = run_head(m, 0, T))) return rc;
        for (int q = 0; q < nseq; q++)
            if ((rc = ifa_argmax_rows_f32(n->logits + (size_t)last[(size_t)q] * V, V, V, 1, n->excl_dev, n->next_dev + q, s))) return rc;
    } else {
        // the sequences' last rows, normed one by one into consecutive rows of h, then one product
        for (int q = 0; q < nseq; q++)
            if ((rc = out_norm_rows(m, n->x + (size_t)last[(size_t)q] * W, 1, n->h + (size_t)q * W))) return rc;
        if ((rc = linear(m, (const bf16_t *)n->lm_head.data, V, W, n->h, W, (size_t)nseq, nullptr, nullptr, logit_scale_of(n), 0, n->logits, V))) return rc;
        if (n->cfg.logit_softcap > 0.0f && (rc = ifa_softcap_f32(n->logits, (size_t)nseq * V, n->cfg.logit_softcap, s))) return rc;
        n->logits_rows = (size_t)nseq;
        if ((rc = ifa_argmax_rows_f32(n->logits, V, V, (size_t)nseq, n->excl_dev, n->next_dev, s))) return rc;
    }
    std::vector<int> next((size_t)nseq, -1);
    IFA_HIP_CHECK(hipMemcpyAsync(next.data(), n->next_dev, (size_t)nseq * 4, hipMemcpyDeviceToHost, m->stream));
    IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
    if (next_tokens_host) memcpy(next_tokens_host, next.data(), (size_t)nseq * 4);
    return IFA_OK;
}

int lay_forward(ifa_model *m, const int *tokens_host, int n_tokens, int prefix_len, void *logits_out_dev, int *next_token_host)
{
    LayeredNet *n = m->lay;
    IFA_REQUIRE(tokens_host, "ifa_model_forward: null tokens");
    int rc = lay_step(m, 1, tokens_host, &n_tokens, &prefix_len, &n->cur_slot, logits_out_dev ? 1 : 0, next_token_host);
    if (rc || !logits_out_dev) return rc;
    if ((rc = ifa_convert_f32_f16(n->logits, (size_t)n_tokens * n->cfg.vocab, logits_out_dev, (ifa_stream)m->stream))) return rc;
    IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
    return IFA_OK;
}

int lay_decode_batch(ifa_model *m, int cnt, const int *tokens_host, const int *positions_host, const int *kv_slots_host, int *next_tokens_host,
                     void *logits_out_dev)
{
    LayeredNet *n = m->lay;
    IFA_REQUIRE(cnt >= 1 && cnt <= ifa_model::RING, "ifa_model_decode_batch: bad arguments");
    std::vector<int> ones((size_t)cnt, 1);
    int rc = lay_step(m, cnt, tokens_host, ones.data(), positions_host, kv_slots_host, 1, next_tokens_host);
    if (rc || !logits_out_dev) return rc;
    if ((rc = ifa_convert_f32_f16(n->logits, (size_t)cnt * n->cfg.vocab, logits_out_dev, (ifa_stream)m->stream))) return rc;
    IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
    return IFA_OK;
}

// one token of the current slot's sequence, everything it depends on in device memory: capturable
int enqueue_decode_step(ifa_model *m)
{
    LayeredNet *n = m->lay;
    const size_t V = (size_t)n->cfg.vocab;
    int rc;
    if ((rc = run_layers(m, 1, 1)) || (rc = run_head(m, 0, 1))) return rc;
    return ifa_argmax_rows_f32(n->logits, V, V, 1, n->excl_dev, n->next_dev, (ifa_stream)m->stream);
}

int lay_decode(ifa_model *m, int first_token, int start_pos, int n_steps, int *out_tokens_host, float *elapsed_ms, bool prepare_only)
{
    LayeredNet *n = m->lay;
    IFA_REQUIRE(m->finalized, "ifa_model_decode: model not finalized");
    IFA_REQUIRE(n_steps >= 1 && n_steps <= ifa_model::RING, "ifa_model_decode: n_steps %d (1..%d)", n_steps, ifa_model::RING);
    IFA_HIP_CHECK(hipSetDevice(m->cfg.device));
    int rc;
    if ((rc = check_span(m, n_steps, start_pos, nullptr)) || (rc = ensure_slot(m, n->cur_slot)) || (rc = ensure_rows(m, 1, 1)) || (rc = ensure_logits(m, 1))) return rc;
    if (n->opt_graph && !n->opt_tap_layers && !n->step_exec) {      // (the slot is read from the device tables: one capture serves every slot)
        drop_step_graph(n);
        n->step_expand = false;
        IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
        IFA_HIP_CHECK(hipStreamBeginCapture(m->stream, hipStreamCaptureModeThreadLocal));
        rc = enqueue_decode_step(m);
        hipGraph_t g = nullptr;
        const hipError_t e = hipStreamEndCapture(m->stream, &g);
        if (rc) { if (g) (void)hipGraphDestroy(g); return rc; }
        if (e != hipSuccess) return ifa_fail(IFA_ERR_HIP, "capture of the decode step: %s", hipGetErrorString(e));
        n->step_graph = g;
        IFA_HIP_CHECK(hipGraphInstantiate(&n->step_exec, g, nullptr, nullptr, 0));
        n->step_slot = n->cur_slot;
    }
    if (prepare_only) return IFA_OK;
    IFA_REQUIRE(out_tokens_host, "ifa_model_decode: null output");
    if ((rc = check_span(m, 1, start_pos, &first_token))) return rc;
    std::vector<int> tok(1, first_token), pos(1, start_pos), rs(1, 0);
    std::vector<ifa_seq_desc> sq(1); sq[0] = ifa_seq_desc{0, 1, start_pos, n->cur_slot};
    if ((rc = upload_tables(m, tok, pos, rs, sq))) return rc;
    n->step_expand = false;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (elapsed_ms) { IFA_HIP_CHECK(hipEventCreate(&e0)); IFA_HIP_CHECK(hipEventCreate(&e1)); IFA_HIP_CHECK(hipEventRecord(e0, m->stream)); }
    for (int st = 0; st < n_steps; st++) {
        if (n->step_exec && n->opt_graph && !n->opt_tap_layers) IFA_HIP_CHECK(hipGraphLaunch(n->step_exec, m->stream));
        else if ((rc = enqueue_decode_step(m))) return rc;
        hipLaunchKernelGGL(k_lay_advance, dim3(1), dim3(1), 0, m->stream, n->tokens_dev, n->pos_dev, n->seqs_dev, n->next_dev, n->ring_dev, st);
        IFA_LAUNCH_CHECK();
    }
    if (elapsed_ms) IFA_HIP_CHECK(hipEventRecord(e1, m->stream));
    IFA_HIP_CHECK(hipMemcpyAsync(out_tokens_host, n->ring_dev, (size_t)n_steps * 4, hipMemcpyDeviceToHost, m->stream));
    IFA_HIP_CHECK(hipStreamSynchronize(m->stream));
    if (elapsed_ms) { IFA_HIP_CHECK(hipEventElapsedTime(elapsed_ms, e0, e1)); (void)hipEventDestroy(e0); (void)hipEventDestroy(e1); }
    return IFA_OK;
}

const ifa_model_vtbl kLayeredVtbl = {lay_destroy, lay_finalize, lay_reset, lay_kv_slots, lay_select_kv, lay_set_option, lay_set_excluded, lay_get_buffer,
                                     lay_forward, lay_decode, lay_decode_batch};

} // namespace

extern "C" {

int ifa_model_create_layered(const ifa_layered_config *cfg, const ifa_layer_spec *layers, ifa_model **out)
{
    IFA_REQUIRE(cfg && layers && out, "ifa_model_create_layered: null pointer");
    IFA_REQUIRE(cfg->width > 0 && cfg->vocab > 0 && cfg->max_ctx > 0 && cfg->n_layers > 0, "ifa_model_create_layered: bad hyper-parameters");
    for (int l = 0; l < cfg->n_layers; l++) {
        const ifa_layer_spec &s = layers[l];
        IFA_REQUIRE(s.ffn >= 0, "ifa_model_create_layered: layer %d: ffn %d", l, s.ffn);
        if (s.mixer == IFA_MIX_WINDOW_LINEAR) {
            IFA_REQUIRE(s.a_heads > 0 && s.a_kv_heads > 0 && s.a_heads % s.a_kv_heads == 0 && s.a_dim > 0 && s.a_dim <= 256 && s.a_window >= 1 && s.a_keep_first >= 0
                        && s.a_buckets >= 1 && s.a_bias_max >= 1, "ifa_model_create_layered: layer %d: bad windowed-attention sizes", l);
            IFA_REQUIRE(s.l_heads > 0 && s.l_dim > 0 && s.l_dim <= 256 && s.l_vdim > 0, "ifa_model_create_layered: layer %d: bad linear-attention sizes", l);
        } else if (s.mixer == IFA_MIX_GATED_DELTA) {
            IFA_REQUIRE(s.d_heads > 0 && s.d_kv_heads > 0 && s.d_heads % s.d_kv_heads == 0 && s.d_dim > 0 && s.d_dim <= 256 && s.d_vdim > 0 && s.d_conv >= 1 && s.d_conv <= 64,
                        "ifa_model_create_layered: layer %d: bad delta-rule sizes", l);
        } else if (s.mixer == IFA_MIX_LATENT) {
            IFA_REQUIRE(s.m_heads > 0 && s.m_dim > 0 && s.m_rot_dim >= 0 && s.m_vdim > 0 && s.m_kv_rank > 0 && s.m_q_rank >= 0 && s.m_kv_rank + s.m_rot_dim <= 1024
                        && s.m_rot_dims >= 0 && s.m_rot_dims <= s.m_rot_dim && s.m_rot_dims % 2 == 0 && (s.m_rot_dims == 0 || s.m_rot_base > 1.0f),
                        "ifa_model_create_layered: layer %d: bad latent-attention sizes", l);
            IFA_REQUIRE(s.m_yarn_factor == 0.0f || (s.m_yarn_factor > 0.0f && s.m_yarn_original > 0.0f && s.m_yarn_fast > 0.0f && s.m_yarn_slow > 0.0f),
                        "ifa_model_create_layered: layer %d: bad frequency scaling", l);
        } else if (s.mixer == IFA_MIX_ROTARY) {
            IFA_REQUIRE(s.a_heads > 0 && s.a_kv_heads > 0 && s.a_heads % s.a_kv_heads == 0 && s.a_dim > 0 && s.a_dim <= 1024 && s.a_vdim > 0 && s.a_vdim <= 1024
                        && s.a_window >= 0 && s.a_keep_first >= 0 && s.a_rot_dims >= 0 && s.a_rot_dims <= s.a_dim && s.a_rot_dims % 2 == 0
                        && (s.a_rot_dims == 0 || s.a_rot_base > 1.0f), "ifa_model_create_layered: layer %d: bad attention sizes", l);
            if (s.a_kv_layer != 0) {
                IFA_REQUIRE(s.a_kv_layer >= 1 && s.a_kv_layer <= l, "ifa_model_create_layered: layer %d reads the keys and values of layer %d, which is not an earlier layer", l, s.a_kv_layer - 1);
                const ifa_layer_spec &o = layers[s.a_kv_layer - 1];
                IFA_REQUIRE(o.mixer == IFA_MIX_ROTARY && o.a_kv_layer == 0 && o.a_kv_heads == s.a_kv_heads && o.a_dim == s.a_dim && o.a_vdim == s.a_vdim,
                            "ifa_model_create_layered: layer %d: layer %d has no keys and values of its own in this layer's shape", l, s.a_kv_layer - 1);
            }
            IFA_REQUIRE(s.a_sink >= 0 && s.a_sink <= 2 && (s.a_rot_scale_factor == 0.0f || (s.a_rot_scale_factor > 0.0f && s.a_rot_scale_original > 0.0f
                        && s.a_rot_scale_low > 0.0f && s.a_rot_scale_high > s.a_rot_scale_low)) && (!s.a_vrot || (s.a_vdim % 2 == 0 && s.a_rot_base > 1.0f)),
                        "ifa_model_create_layered: layer %d: bad sink, frequency scaling or rotated values of an odd size", l);
        } else if (s.mixer == IFA_MIX_CHAN_DELTA) {
            IFA_REQUIRE(s.c_heads > 0 && s.c_dim > 0 && s.c_dim <= 256 && s.c_rank >= 1 && s.c_rank <= 8192 && s.c_decay_mult > 0.0f && s.c_l2_eps >= 0.0f,
                        "ifa_model_create_layered: layer %d: bad sizes of the generalized delta rule", l);
        } else return ifa_fail(IFA_ERR_ARG, "ifa_model_create_layered: layer %d: unknown mixer %d", l, s.mixer);
        const bool wired = s.mixer == IFA_MIX_LATENT ? s.block == IFA_BLOCK_POSTNORM
                           : s.mixer == IFA_MIX_ROTARY ? (s.block == IFA_BLOCK_SANDWICH || s.block == IFA_BLOCK_PRENORM)
                           : s.mixer == IFA_MIX_CHAN_DELTA ? s.block == IFA_BLOCK_PRENORM : s.block == IFA_BLOCK_PARALLEL;
        IFA_REQUIRE(wired, "ifa_model_create_layered: layer %d: mixer %d is not wired for block kind %d", l, s.mixer, s.block);
        if (s.block == IFA_BLOCK_PRENORM) {
            IFA_REQUIRE(s.ffn == 0 && s.a_kv_layer == 0, "ifa_model_create_layered: layer %d: this wiring takes a mixture of experts or no feed-forward, and keys of its own", l);
            if (s.ffn_kind == IFA_FFN_MOE && s.x_experts + s.x_identity > 0)
                IFA_REQUIRE(s.x_identity == 0 && s.x_gated == 1 && s.x_route == 0 && s.x_shared_ff == 0 && s.x_experts >= 1 && s.x_experts <= 4096 && s.x_top >= 1
                            && s.x_top <= s.x_experts && s.x_ff > 0 && (s.x_score == 0 || s.x_score == 1) && (s.x_glu == 0 || (s.x_glu == 3 && s.x_limit > 0.0f)),
                            "ifa_model_create_layered: layer %d: bad mixture-of-experts sizes", l);
        } else
        if (s.block == IFA_BLOCK_SANDWICH) {
            if (s.ffn_kind == IFA_FFN_MOE && s.x_experts + s.x_identity > 0)
                IFA_REQUIRE(s.ffn == 0 && s.x_identity == 0 && s.x_gated == 1 && s.x_route == 1 && s.x_experts >= 1 && s.x_experts <= 4096 && s.x_top >= 1 && s.x_top <= s.x_experts
                            && s.x_ff > 0 && s.x_shared_ff >= 0, "ifa_model_create_layered: layer %d: bad mixture-of-experts sizes", l);
            else IFA_REQUIRE(s.ffn == 0 || (s.ffn_kind == IFA_FFN_CLAMPED && s.f_limit > 0.0f), "ifa_model_create_layered: layer %d: this wiring takes the clamped feed-forward or a mixture", l);
        } else
        if (s.block == IFA_BLOCK_POSTNORM) {
            IFA_REQUIRE(s.ffn == 0 && s.canon_taps >= 0 && s.canon_taps <= 64 && cfg->norm_groups >= 1 && cfg->width % cfg->norm_groups == 0,
                        "ifa_model_create_layered: layer %d: bad block sizes (norm in %d parts of width %d)", l, cfg->norm_groups, cfg->width);
            if (s.ffn_kind == IFA_FFN_MOE && s.x_experts + s.x_identity > 0)
                IFA_REQUIRE(s.x_experts >= 0 && s.x_identity >= 0 && s.x_experts + s.x_identity <= 4096 && s.x_top >= 1 && s.x_top <= s.x_experts + s.x_identity
                            && (s.x_experts == 0 || s.x_ff > 0), "ifa_model_create_layered: layer %d: bad mixture-of-experts sizes", l);
        } else IFA_REQUIRE(s.ffn_kind == IFA_FFN_GATED, "ifa_model_create_layered: layer %d: this wiring takes the gated feed-forward with biases", l);
    }
    IFA_REQUIRE(cfg->stem == 0 || (cfg->stem == 1 && cfg->norm_groups >= 1 && cfg->width % cfg->norm_groups == 0)
                || ((cfg->stem == 2 || cfg->stem == 3) && cfg->bigram_buckets >= 0 && cfg->bigram_buckets < (1 << 30)), "ifa_model_create_layered: bad stem");
    if (cfg->loop_times > 0 && cfg->loop_start < cfg->loop_stop) {
        IFA_REQUIRE(cfg->loop_start >= 0 && cfg->loop_stop <= cfg->n_layers && cfg->loop_times <= 1024, "ifa_model_create_layered: looped group [%d, %d) x %d of %d layers",
                    cfg->loop_start, cfg->loop_stop, cfg->loop_times, cfg->n_layers);
        for (int l = cfg->loop_start; l < cfg->loop_stop; l++)
            IFA_REQUIRE(layers[l].block == IFA_BLOCK_PRENORM, "ifa_model_create_layered: layer %d of the looped group is not wired with norms in front of its sub-layers", l);
        IFA_REQUIRE(cfg->loop_times == 1 || cfg->stem == 3, "ifa_model_create_layered: a looped group of several passes needs the stem that keeps the embedding output");
    }
    IFA_HIP_CHECK(hipSetDevice(cfg->device));
    ifa_model *m = new ifa_model();
    memset(&m->cfg, 0, sizeof(m->cfg));
    m->cfg.dim = cfg->width; m->cfg.layers = cfg->n_layers; m->cfg.vocab = cfg->vocab; m->cfg.max_ctx = cfg->max_ctx; m->cfg.device = cfg->device;
    m->cfg.eps = cfg->eps; m->cfg.tp_size = 1;
    LayeredNet *n = new LayeredNet();
    n->cfg = *cfg;
    if (n->cfg.eps <= 0) n->cfg.eps = 1e-5f;
    if (n->cfg.pos_base <= 1.0f) n->cfg.pos_base = 10000.0f;
    n->layers.resize((size_t)cfg->n_layers);
    for (int l = 0; l < cfg->n_layers; l++) n->layers[(size_t)l].spec = layers[l];
    m->lay = n; m->vt = &kLayeredVtbl;
    hipError_t e = hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking);
    if (e != hipSuccess) { delete n; delete m; return ifa_fail(IFA_ERR_HIP, "hipStreamCreate: %s", hipGetErrorString(e)); }
    *out = m;
    return IFA_OK;
}

int ifa_model_set_tensor_host(ifa_model *m, int layer, int tensor_id, int dtype, const void *host_src, size_t rows, size_t cols)
{
    IFA_REQUIRE(m && m->lay && host_src, "ifa_model_set_tensor_host: not a layer-list model / null pointer");
    LayeredNet *n = m->lay;
    IFA_REQUIRE(!m->finalized, "ifa_model_set_tensor_host: the model is finalized");
    IFA_REQUIRE(rows > 0 && cols > 0, "ifa_model_set_tensor_host: empty tensor");
    LTensor *t = nullptr;
    size_t er = 0, ec = 0; bool vec = false;
    const size_t W = (size_t)n->cfg.width, V = (size_t)n->cfg.vocab;
    if (layer < 0) {
        if (tensor_id == IFA_T_EMBD) { t = &n->embd; er = V; ec = W; }
        else if (tensor_id == IFA_T_LM_HEAD) { t = &n->lm_head; er = V; ec = W; }
        else if (tensor_id == IFA_T_OUT_NORM) { t = &n->out_norm; er = 1; ec = W; vec = true; }
        else if (tensor_id == IFA_T_EMBD_NORM) { t = &n->embd_norm; er = 1; ec = W; vec = true; }
        else if (tensor_id == IFA_T_BIGRAM && (n->cfg.stem == 2 || n->cfg.stem == 3) && n->cfg.bigram_buckets > 0) { t = &n->bigram; er = (size_t)n->cfg.bigram_buckets + 1; ec = W; }
        else if (tensor_id == IFA_T_OUT_NORM_B && n->cfg.stem == 3) { t = &n->out_norm_b; er = 1; ec = W; vec = true; }
        else if (tensor_id == IFA_T_OUT_NORM_ALPHA && n->cfg.stem == 3) { t = &n->out_norm_alpha; er = 1; ec = 1; vec = true; }
        else if (tensor_id == IFA_T_LOOP_STEP && n->cfg.loop_times > 0) { t = &n->loop_step; er = (size_t)n->cfg.loop_times; ec = W; }
        else return ifa_fail(IFA_ERR_ARG, "ifa_model_set_tensor_host: global tensor id %d", tensor_id);
    } else {
        IFA_REQUIRE(layer < (int)n->layers.size() && tensor_id >= IFA_LT_NORM1 && tensor_id < IFA_LT_END, "ifa_model_set_tensor_host: layer %d / tensor id %d", layer, tensor_id);
        LLayer &L = n->layers[(size_t)layer];
        IFA_REQUIRE(expected_shape(n, L.spec, layer, tensor_id, er, ec, vec), "ifa_model_set_tensor_host: tensor %d does not belong to layer %d's mixer", tensor_id, layer);
        t = &L.T(tensor_id);
    }
    const int want = tensor_id == IFA_LT_L_DECAY ? IFA_F32 : IFA_BF16;
    IFA_REQUIRE(dtype == want, "ifa_model_set_tensor_host: tensor %d takes dtype %d, got %d", tensor_id, want, dtype);
    if (vec) IFA_REQUIRE(rows * cols == er * ec, "ifa_model_set_tensor_host: tensor %d of layer %d holds %zu values, the model needs %zu", tensor_id, layer, rows * cols, er * ec);
    else IFA_REQUIRE(rows == er && cols == ec, "ifa_model_set_tensor_host: tensor %d of layer %d is %zu x %zu, the model needs %zu x %zu", tensor_id, layer, rows, cols, er, ec);
    IFA_HIP_CHECK(hipSetDevice(m->cfg.device));
    lay_free(t->data); t->data = nullptr;
    const size_t bytes = rows * cols * (dtype == IFA_F32 ? 4 : 2);
    IFA_HIP_CHECK(hipMalloc(&t->data, bytes));
    IFA_HIP_CHECK(hipMemcpy(t->data, host_src, bytes, hipMemcpyHostToDevice));
    t->dtype = dtype; t->rows = rows; t->cols = cols;
    return IFA_OK;
}

int ifa_model_logits_f32(ifa_model *m, void **dptr, size_t *rows, size_t *cols)
{
    IFA_REQUIRE(m && m->lay && dptr, "ifa_model_logits_f32: not a layer-list model / null pointer");
    *dptr = m->lay->logits;
    if (rows) *rows = m->lay->logits_rows;
    if (cols) *cols = (size_t)m->lay->cfg.vocab;
    return IFA_OK;
}

int ifa_model_step_seqs(ifa_model *m, int n_seqs, const int *tokens_host, const int *seq_lens, const int *seq_pos0, const int *seq_slots, int all_logits,
                        int *next_tokens_host)
{
    IFA_REQUIRE(m && m->lay && m->finalized, "ifa_model_step_seqs: not a finalized layer-list model");
    return lay_step(m, n_seqs, tokens_host, seq_lens, seq_pos0, seq_slots, all_logits, next_tokens_host);
}

int ifa_model_is_layered(const ifa_model *m) { return m && m->vt ? 1 : 0; }

} // extern "C"
