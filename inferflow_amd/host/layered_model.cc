// layered_model.cc -- models described layer by layer in their own config.json ("architecture": <name>, "layers": [...]),
// served by the layer-list worker (ifa_model_create_layered).  The registry below maps an architecture name to the reader of
// its configuration and to its tensor names; a model directory holds config.json + model.safetensors (bfloat16 weights).
//
// Gelarax: width / vocab / norm.eps; every layer has one layer norm (no bias) feeding its mixer and its GELU-gated
// feed-forward in parallel, layer scales ls1 / ls2, and a mixer of type
//   "parallel"  windowed softmax attention with kept first tokens, soft cap, distance-bucket bias and sink ("left") beside
//               decayed linear attention ("right"), summed with left_scale / right_scale
//   "delta"     gated delta rule behind short causal convolutions
//
// Muzopel: width / vocab / norm.eps / norm.groups / canon.taps / logit_softcap; the embedding and the output pass a grouped RMS norm;
// every layer reads the residual through a short causal convolution, puts a grouped RMS norm on each sub-layer's output, feeds
// forward through a mixture of experts (with identity experts and a correction on the choice scores) and ends in a learned average
// over the depth of the stack; mixer types
//   "latent_attention"    queries through a normed latent (q_rank), YaRN-scaled rotation when rot.scaling is given, sigmoid gate per head
//   "latent_attention_2"  queries straight from the input, plain rotation, no gate
// both with one cached row [kv_rank latent | rot_dim rotated key part] per position.
//
// Sopulorn: width / vocab / norm.eps / embedding.bigram {buckets, mul_prev, mul_cur}; the token embedding plus a hashed embedding of the
// (previous token, token) pair; every layer has an RMS norm with weight (1 + w) before and after each sub-layer; mixer type
//   "attention"  causal softmax attention with grouped queries, biases on q / k / v, weighted RMS norm of q and k per head, rotation of
//                the first rot.dims dimensions of a head (pairs i, i + dims / 2), values of size vdim, one added to the softmax's
//                denominator; "kv_from": j = the layer has no key / value tensors and reads the cache rows of layer j
// and a feed-forward of kind "dense" (clamped: min(gate, limit) * sigmoid(1.702 .) * (clamp(up) + 1)) or "moe" (router on logits + bias,
// softmax over the chosen, gated SiLU experts, a shared expert times sigmoid(sg . h)), or none.
//
// Bogupel: width / vocab / norm.eps / embedding {scale, bigram {buckets, mul_prev, mul_cur}} / logit_scale / loop {start, stop, times}; the token
// embedding times embedding.scale plus the hashed pair embedding; Dynamic Tanh norms (tanh(alpha x) w + b) in front of each sub-layer and of the
// head; layers [loop.start, loop.stop) run loop.times times with the same weights, every pass on a cache of its own; mixer types
//   "attention"      grouped queries, biases on q / k / v, weighted RMS norm of q and k per head, rotation of the first rot.dims dimensions with
//                    frequencies scaled by wavelength (rot.scaling {factor, low, high, original}), values divided by their root mean square and
//                    turned by their position over all of vdim (the head's output turned back), sliding window mask.size, a learned sink per head
//   "general_delta"  generalized delta rule with a decay and a removal rate per head and key channel, per-head RMS norm, sigmoid gate
// and a mixture of clamped gated experts (sigmoid scores, choice by score + correction, weights = the scores), or no feed-forward.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>

#include "inferflow_amd.h"
#include "inference_engine.h"
#include "ifa_json.h"

namespace inferflow_amd {

bool IndexSafetensorsFile(const std::string &path, std::map<std::string, StTensorEntry> &index);      // model_loader.cc

namespace {

bool ReadText(const std::string &path, std::string &out)
{
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    std::stringstream ss; ss << f.rdbuf();
    out = ss.str();
    return true;
}

struct LayeredDesc {
    ifa_layered_config cfg;
    std::vector<ifa_layer_spec> layers;
    std::vector<std::vector<float>> decays;        // per layer: decay per linear-attention head
};

template <typename T> bool Need(const JsonValue &o, const char *key, T &out, const char *where)
{
    if (o.GetNumber(key, out)) return true;
    EngineSetError("config.json: %s.%s is missing", where, key);
    return false;
}

// ---- Gelarax
bool ParseGelarax(const JsonValue &root, LayeredDesc &d)
{
    memset(&d.cfg, 0, sizeof(d.cfg));
    if (!Need(root, "width", d.cfg.width, "config") || !Need(root, "vocab", d.cfg.vocab, "config")) return false;
    const JsonValue *norm = root.Get("norm");
    if (!norm || !Need(*norm, "eps", d.cfg.eps, "norm")) { if (!norm) EngineSetError("config.json: norm is missing"); return false; }
    d.cfg.pos_base = 10000.0f;
    const JsonValue *layers = root.Get("layers");
    if (!layers || layers->type != JsonValue::Array || layers->arr.empty()) { EngineSetError("config.json: layers is missing or empty"); return false; }
    for (size_t li = 0; li < layers->arr.size(); li++) {
        const JsonValue &L = layers->arr[li];
        ifa_layer_spec s; memset(&s, 0, sizeof(s));
        std::vector<float> decay;
        std::string type;
        const JsonValue *mx = L.Get("mixer");
        if (!L.GetString("type", type) || !mx || mx->type != JsonValue::Object) { EngineSetError("config.json: layer %zu has no type / mixer", li); return false; }
        const std::string where = "layers[" + std::to_string(li) + "].mixer";
        if (type == "parallel") {
            s.mixer = IFA_MIX_WINDOW_LINEAR;
            const JsonValue *a = mx->Get("left"), *r = mx->Get("right");
            if (!a || !r) { EngineSetError("config.json: %s needs left and right", where.c_str()); return false; }
            int vdim = 0;
            const JsonValue *mask = a->Get("mask");
            if (!mask) { EngineSetError("config.json: %s.left.mask is missing", where.c_str()); return false; }
            if (!Need(*a, "heads", s.a_heads, "left") || !Need(*a, "kv_heads", s.a_kv_heads, "left") || !Need(*a, "dim", s.a_dim, "left") || !Need(*a, "vdim", vdim, "left")
                || !Need(*a, "scale", s.a_scale, "left") || !Need(*a, "softcap", s.a_softcap, "left") || !Need(*a, "bias_max", s.a_bias_max, "left")
                || !Need(*mask, "size", s.a_window, "left.mask") || !Need(*mask, "keep_first", s.a_keep_first, "left.mask")
                || !Need(*mx, "left_scale", s.a_out_scale, "mixer") || !Need(*mx, "right_scale", s.l_out_scale, "mixer")
                || !Need(*r, "heads", s.l_heads, "right") || !Need(*r, "dim", s.l_dim, "right") || !Need(*r, "vdim", s.l_vdim, "right")) return false;
            if (vdim != s.a_dim) { EngineSetError("config.json: %s.left: the values are the keys, so vdim (%d) must equal dim (%d)", where.c_str(), vdim, s.a_dim); return false; }
            const JsonValue *dc = r->Get("decay");
            if (!dc || dc->type != JsonValue::Array || (int)dc->arr.size() != s.l_heads) { EngineSetError("config.json: %s.right.decay needs one value per head", where.c_str()); return false; }
            for (const JsonValue &v : dc->arr) decay.push_back((float)v.num);
        } else if (type == "delta") {
            s.mixer = IFA_MIX_GATED_DELTA;
            if (!Need(*mx, "heads", s.d_heads, "mixer") || !Need(*mx, "kv_heads", s.d_kv_heads, "mixer") || !Need(*mx, "dim", s.d_dim, "mixer")
                || !Need(*mx, "vdim", s.d_vdim, "mixer") || !Need(*mx, "conv", s.d_conv, "mixer")) return false;
        } else { EngineSetError("config.json: layer %zu: unknown type \"%s\"", li, type.c_str()); return false; }
        const JsonValue *mlp = L.Get("mlp");
        if (mlp && mlp->type == JsonValue::Object) {
            std::string kind;
            if (!mlp->GetString("kind", kind) || kind != "dense") { EngineSetError("config.json: layer %zu: mlp.kind \"%s\" is not supported (dense)", li, kind.c_str()); return false; }
            if (!Need(*mlp, "ff", s.ffn, "mlp")) return false;
        }
        d.layers.push_back(s);
        d.decays.push_back(decay);
    }
    d.cfg.n_layers = (int)d.layers.size();
    return true;
}

// ---- Muzopel
bool ParseMuzopel(const JsonValue &root, LayeredDesc &d)
{
    memset(&d.cfg, 0, sizeof(d.cfg));
    if (!Need(root, "width", d.cfg.width, "config") || !Need(root, "vocab", d.cfg.vocab, "config")) return false;
    const JsonValue *norm = root.Get("norm");
    if (!norm) { EngineSetError("config.json: norm is missing"); return false; }
    if (!Need(*norm, "eps", d.cfg.eps, "norm") || !Need(*norm, "groups", d.cfg.norm_groups, "norm")) return false;
    d.cfg.stem = 1;
    root.GetNumber("logit_softcap", d.cfg.logit_softcap);
    int taps = 0;
    if (const JsonValue *canon = root.Get("canon")) canon->GetNumber("taps", taps);
    const JsonValue *layers = root.Get("layers");
    if (!layers || layers->type != JsonValue::Array || layers->arr.empty()) { EngineSetError("config.json: layers is missing or empty"); return false; }
    for (size_t li = 0; li < layers->arr.size(); li++) {
        const JsonValue &L = layers->arr[li];
        ifa_layer_spec s; memset(&s, 0, sizeof(s));
        std::string type;
        const JsonValue *mx = L.Get("mixer");
        if (!L.GetString("type", type) || !mx || mx->type != JsonValue::Object) { EngineSetError("config.json: layer %zu has no type / mixer", li); return false; }
        if (type != "latent_attention" && type != "latent_attention_2") { EngineSetError("config.json: layer %zu: unknown type \"%s\"", li, type.c_str()); return false; }
        const bool first = type == "latent_attention";
        s.mixer = IFA_MIX_LATENT; s.block = IFA_BLOCK_POSTNORM; s.canon_taps = taps; s.depth_avg = 1;
        if (!Need(*mx, "heads", s.m_heads, "mixer") || !Need(*mx, "dim", s.m_dim, "mixer") || !Need(*mx, "rot_dim", s.m_rot_dim, "mixer") || !Need(*mx, "vdim", s.m_vdim, "mixer")
            || !Need(*mx, "kv_rank", s.m_kv_rank, "mixer") || !Need(*mx, "scale", s.m_scale, "mixer")) return false;
        if (first && !Need(*mx, "q_rank", s.m_q_rank, "mixer")) return false;
        s.m_gate = first ? 1 : 0;
        const JsonValue *rot = mx->Get("rot");
        if (!rot || !Need(*rot, "base", s.m_rot_base, "mixer.rot") || !Need(*rot, "dims", s.m_rot_dims, "mixer.rot")) { if (!rot) EngineSetError("config.json: layer %zu: mixer.rot is missing", li); return false; }
        const JsonValue *sc = rot->Get("scaling");
        if (first && sc && sc->type == JsonValue::Object
            && (!Need(*sc, "factor", s.m_yarn_factor, "rot.scaling") || !Need(*sc, "original", s.m_yarn_original, "rot.scaling")
                || !Need(*sc, "fast", s.m_yarn_fast, "rot.scaling") || !Need(*sc, "slow", s.m_yarn_slow, "rot.scaling"))) return false;
        const JsonValue *mlp = L.Get("mlp");
        if (mlp && mlp->type == JsonValue::Object) {
            std::string kind;
            if (!mlp->GetString("kind", kind) || kind != "moe") { EngineSetError("config.json: layer %zu: mlp.kind \"%s\" is not supported (moe)", li, kind.c_str()); return false; }
            const JsonValue *ex = mlp->Get("expert"), *ro = mlp->Get("router");
            if (!ex || !ro) { EngineSetError("config.json: layer %zu: mlp needs expert and router", li); return false; }
            s.ffn_kind = IFA_FFN_MOE;
            if (!Need(*ex, "ff", s.x_ff, "mlp.expert") || !Need(*ro, "experts", s.x_experts, "mlp.router") || !Need(*ro, "top", s.x_top, "mlp.router")) return false;
            ro->GetNumber("identity", s.x_identity);
        }
        d.layers.push_back(s);
        d.decays.push_back(std::vector<float>());
    }
    d.cfg.n_layers = (int)d.layers.size();
    return true;
}

// ---- Sopulorn
bool ParseSopulorn(const JsonValue &root, LayeredDesc &d)
{
    memset(&d.cfg, 0, sizeof(d.cfg));
    if (!Need(root, "width", d.cfg.width, "config") || !Need(root, "vocab", d.cfg.vocab, "config")) return false;
    const JsonValue *norm = root.Get("norm");
    if (!norm || !Need(*norm, "eps", d.cfg.eps, "norm")) { if (!norm) EngineSetError("config.json: norm is missing"); return false; }
    d.cfg.stem = 2;
    const JsonValue *emb = root.Get("embedding");
    const JsonValue *bg = emb ? emb->Get("bigram") : nullptr;
    if (bg && bg->type == JsonValue::Object
        && (!Need(*bg, "buckets", d.cfg.bigram_buckets, "embedding.bigram") || !Need(*bg, "mul_prev", d.cfg.bigram_mul_prev, "embedding.bigram")
            || !Need(*bg, "mul_cur", d.cfg.bigram_mul_cur, "embedding.bigram"))) return false;
    const JsonValue *layers = root.Get("layers");
    if (!layers || layers->type != JsonValue::Array || layers->arr.empty()) { EngineSetError("config.json: layers is missing or empty"); return false; }
    for (size_t li = 0; li < layers->arr.size(); li++) {
        const JsonValue &L = layers->arr[li];
        ifa_layer_spec s; memset(&s, 0, sizeof(s));
        std::string type;
        const JsonValue *mx = L.Get("mixer");
        if (!L.GetString("type", type) || !mx || mx->type != JsonValue::Object) { EngineSetError("config.json: layer %zu has no type / mixer", li); return false; }
        if (type != "attention") { EngineSetError("config.json: layer %zu: unknown type \"%s\"", li, type.c_str()); return false; }
        s.mixer = IFA_MIX_ROTARY; s.block = IFA_BLOCK_SANDWICH;
        s.a_sink = 1; s.a_sink_score = 0.0f;          // one added to the denominator = a sink of score 0
        if (!Need(*mx, "heads", s.a_heads, "mixer") || !Need(*mx, "kv_heads", s.a_kv_heads, "mixer") || !Need(*mx, "dim", s.a_dim, "mixer")
            || !Need(*mx, "vdim", s.a_vdim, "mixer") || !Need(*mx, "scale", s.a_scale, "mixer")) return false;
        const JsonValue *rot = mx->Get("rot");
        if (rot && rot->type == JsonValue::Object && (!Need(*rot, "base", s.a_rot_base, "mixer.rot") || !Need(*rot, "dims", s.a_rot_dims, "mixer.rot"))) return false;
        int from = -1;
        if (mx->GetNumber("kv_from", from)) {
            if (from < 0 || from >= (int)li) { EngineSetError("config.json: layer %zu: kv_from %d is not an earlier layer", li, from); return false; }
            s.a_kv_layer = from + 1;
        }
        const JsonValue *mlp = L.Get("mlp");
        if (mlp && mlp->type == JsonValue::Object) {
            std::string kind;
            mlp->GetString("kind", kind);
            if (kind == "dense") {
                s.ffn_kind = IFA_FFN_CLAMPED;
                if (!Need(*mlp, "ff", s.ffn, "mlp") || !Need(*mlp, "limit", s.f_limit, "mlp")) return false;
            } else if (kind == "moe") {
                const JsonValue *ex = mlp->Get("expert"), *ro = mlp->Get("router"), *sh = mlp->Get("shared");
                if (!ex || !ro) { EngineSetError("config.json: layer %zu: mlp needs expert and router", li); return false; }
                s.ffn_kind = IFA_FFN_MOE; s.x_gated = 1; s.x_route = 1;
                if (!Need(*ex, "ff", s.x_ff, "mlp.expert") || !Need(*ro, "experts", s.x_experts, "mlp.router") || !Need(*ro, "top", s.x_top, "mlp.router")) return false;
                if (sh && sh->type == JsonValue::Object && !Need(*sh, "ff", s.x_shared_ff, "mlp.shared")) return false;
            } else { EngineSetError("config.json: layer %zu: mlp.kind \"%s\" is not supported (dense, moe)", li, kind.c_str()); return false; }
        }
        d.layers.push_back(s);
        d.decays.push_back(std::vector<float>());
    }
    d.cfg.n_layers = (int)d.layers.size();
    return true;
}

// ---- Bogupel
bool ParseBogupel(const JsonValue &root, LayeredDesc &d)
{
    memset(&d.cfg, 0, sizeof(d.cfg));
    if (!Need(root, "width", d.cfg.width, "config") || !Need(root, "vocab", d.cfg.vocab, "config")) return false;
    const JsonValue *norm = root.Get("norm");
    if (!norm || !Need(*norm, "eps", d.cfg.eps, "norm")) { if (!norm) EngineSetError("config.json: norm is missing"); return false; }
    d.cfg.stem = 3;
    d.cfg.embed_scale = 1.0f; d.cfg.logit_scale = 1.0f;
    root.GetNumber("logit_scale", d.cfg.logit_scale);
    if (const JsonValue *emb = root.Get("embedding")) {
        emb->GetNumber("scale", d.cfg.embed_scale);
        const JsonValue *bg = emb->Get("bigram");
        if (bg && bg->type == JsonValue::Object
            && (!Need(*bg, "buckets", d.cfg.bigram_buckets, "embedding.bigram") || !Need(*bg, "mul_prev", d.cfg.bigram_mul_prev, "embedding.bigram")
                || !Need(*bg, "mul_cur", d.cfg.bigram_mul_cur, "embedding.bigram"))) return false;
    }
    const JsonValue *loop = root.Get("loop");
    if (loop && loop->type == JsonValue::Object
        && (!Need(*loop, "start", d.cfg.loop_start, "loop") || !Need(*loop, "stop", d.cfg.loop_stop, "loop") || !Need(*loop, "times", d.cfg.loop_times, "loop"))) return false;
    const JsonValue *layers = root.Get("layers");
    if (!layers || layers->type != JsonValue::Array || layers->arr.empty()) { EngineSetError("config.json: layers is missing or empty"); return false; }
    for (size_t li = 0; li < layers->arr.size(); li++) {
        const JsonValue &L = layers->arr[li];
        ifa_layer_spec s; memset(&s, 0, sizeof(s));
        std::string type;
        const JsonValue *mx = L.Get("mixer");
        if (!L.GetString("type", type) || !mx || mx->type != JsonValue::Object) { EngineSetError("config.json: layer %zu has no type / mixer", li); return false; }
        s.block = IFA_BLOCK_PRENORM;
        if (type == "attention") {
            s.mixer = IFA_MIX_ROTARY;
            s.a_sink = 2; s.a_vnorm = 1; s.a_vrot = 1;
            if (!Need(*mx, "heads", s.a_heads, "mixer") || !Need(*mx, "kv_heads", s.a_kv_heads, "mixer") || !Need(*mx, "dim", s.a_dim, "mixer")
                || !Need(*mx, "vdim", s.a_vdim, "mixer") || !Need(*mx, "scale", s.a_scale, "mixer")) return false;
            const JsonValue *rot = mx->Get("rot");
            if (!rot || rot->type != JsonValue::Object || !Need(*rot, "base", s.a_rot_base, "mixer.rot") || !Need(*rot, "dims", s.a_rot_dims, "mixer.rot")) {
                if (!rot) EngineSetError("config.json: layer %zu: mixer.rot is missing", li);
                return false;
            }
            const JsonValue *sc = rot->Get("scaling");
            if (sc && sc->type == JsonValue::Object
                && (!Need(*sc, "factor", s.a_rot_scale_factor, "rot.scaling") || !Need(*sc, "low", s.a_rot_scale_low, "rot.scaling")
                    || !Need(*sc, "high", s.a_rot_scale_high, "rot.scaling") || !Need(*sc, "original", s.a_rot_scale_original, "rot.scaling"))) return false;
            const JsonValue *mask = mx->Get("mask");
            if (mask && mask->type == JsonValue::Object && !Need(*mask, "size", s.a_window, "mixer.mask")) return false;
        } else if (type == "general_delta") {
            s.mixer = IFA_MIX_CHAN_DELTA;
            s.c_decay_mult = 0.60653065971263342f;      // exp(-1/2)
            s.c_l2_eps = 1e-6f;
            if (!Need(*mx, "heads", s.c_heads, "mixer") || !Need(*mx, "dim", s.c_dim, "mixer")) return false;
        } else { EngineSetError("config.json: layer %zu: unknown type \"%s\"", li, type.c_str()); return false; }
        const JsonValue *mlp = L.Get("mlp");
        if (mlp && mlp->type == JsonValue::Object) {
            std::string kind;
            if (!mlp->GetString("kind", kind) || kind != "moe") { EngineSetError("config.json: layer %zu: mlp.kind \"%s\" is not supported (moe)", li, kind.c_str()); return false; }
            const JsonValue *ex = mlp->Get("expert"), *ro = mlp->Get("router");
            if (!ex || !ro) { EngineSetError("config.json: layer %zu: mlp needs expert and router", li); return false; }
            s.ffn_kind = IFA_FFN_MOE; s.x_gated = 1; s.x_route = 0; s.x_score = 1; s.x_glu = 3;
            if (!Need(*ex, "ff", s.x_ff, "mlp.expert") || !Need(*ex, "limit", s.x_limit, "mlp.expert") || !Need(*ro, "experts", s.x_experts, "mlp.router")
                || !Need(*ro, "top", s.x_top, "mlp.router")) return false;
        }
        d.layers.push_back(s);
        d.decays.push_back(std::vector<float>());
    }
    d.cfg.n_layers = (int)d.layers.size();
    return true;
}

// the decay's bottleneck has the size its first matrix gives
bool BogupelSizesFromTensors(const std::map<std::string, StTensorEntry> &index, LayeredDesc &d)
{
    for (size_t li = 0; li < d.layers.size(); li++) {
        if (d.layers[li].mixer != IFA_MIX_CHAN_DELTA) continue;
        const std::string name = "l" + std::to_string(li) + ".mix.w1";
        auto it = index.find(name);
        if (it == index.end() || it->second.shape.size() != 2 || it->second.shape[0] < 1) { EngineSetError("tensor %s is missing or not a matrix", name.c_str()); return false; }
        d.layers[li].c_rank = (int)it->second.shape[0];
    }
    return true;
}

void BogupelNames(const LayeredDesc &d, std::vector<std::pair<std::string, std::pair<int, int>>> &out)
{
    out.push_back({"embed", {-1, IFA_T_EMBD}});
    if (d.cfg.bigram_buckets > 0) out.push_back({"bigram", {-1, IFA_T_BIGRAM}});
    if (d.cfg.loop_times > 0 && d.cfg.loop_start < d.cfg.loop_stop) out.push_back({"loop.step", {-1, IFA_T_LOOP_STEP}});
    out.push_back({"final.norm", {-1, IFA_T_OUT_NORM}}); out.push_back({"final.norm.b", {-1, IFA_T_OUT_NORM_B}}); out.push_back({"final.norm.alpha", {-1, IFA_T_OUT_NORM_ALPHA}});
    out.push_back({"head", {-1, IFA_T_LM_HEAD}});
    for (size_t li = 0; li < d.layers.size(); li++) {
        const ifa_layer_spec &s = d.layers[li];
        const std::string p = "l" + std::to_string(li) + ".";
        const int l = (int)li;
        out.push_back({p + "norm1", {l, IFA_LT_NORM1}}); out.push_back({p + "norm1.b", {l, IFA_LT_NORM1_B}}); out.push_back({p + "norm1.alpha", {l, IFA_LT_NORM1_ALPHA}});
        if (s.mixer == IFA_MIX_ROTARY) {
            out.push_back({p + "mix.q", {l, IFA_LT_A_Q}}); out.push_back({p + "mix.q.b", {l, IFA_LT_A_Q_B}}); out.push_back({p + "mix.q.norm", {l, IFA_LT_A_Q_NORM}});
            out.push_back({p + "mix.k", {l, IFA_LT_A_K}}); out.push_back({p + "mix.k.b", {l, IFA_LT_A_K_B}}); out.push_back({p + "mix.k.norm", {l, IFA_LT_A_K_NORM}});
            out.push_back({p + "mix.v", {l, IFA_LT_A_V}}); out.push_back({p + "mix.v.b", {l, IFA_LT_A_V_B}});
            out.push_back({p + "mix.sink", {l, IFA_LT_A_SINK}}); out.push_back({p + "mix.o", {l, IFA_LT_A_O}});
        } else {
            out.push_back({p + "mix.r", {l, IFA_LT_C_R}}); out.push_back({p + "mix.k", {l, IFA_LT_C_K}}); out.push_back({p + "mix.v", {l, IFA_LT_C_V}});
            out.push_back({p + "mix.g", {l, IFA_LT_C_G}}); out.push_back({p + "mix.a", {l, IFA_LT_C_A}}); out.push_back({p + "mix.a.b", {l, IFA_LT_C_A_B}});
            out.push_back({p + "mix.w1", {l, IFA_LT_C_W1}}); out.push_back({p + "mix.w2", {l, IFA_LT_C_W2}}); out.push_back({p + "mix.w0", {l, IFA_LT_C_W0}});
            out.push_back({p + "mix.norm", {l, IFA_LT_C_NORM}}); out.push_back({p + "mix.o", {l, IFA_LT_C_O}});
        }
        if (!(s.ffn_kind == IFA_FFN_MOE && s.x_experts > 0)) continue;
        out.push_back({p + "norm2", {l, IFA_LT_NORM2}}); out.push_back({p + "norm2.b", {l, IFA_LT_NORM2_B}}); out.push_back({p + "norm2.alpha", {l, IFA_LT_NORM2_ALPHA}});
        out.push_back({p + "mlp.router", {l, IFA_LT_X_ROUTER}}); out.push_back({p + "mlp.correction", {l, IFA_LT_X_CORR}});
        for (int e = 0; e < s.x_experts; e++) {      // per expert: its gate rows, then its up rows
            out.push_back({p + "mlp.e" + std::to_string(e) + ".gate", {l, IFA_LT_X_UP}});
            out.push_back({p + "mlp.e" + std::to_string(e) + ".up", {l, IFA_LT_X_UP}});
        }
        for (int e = 0; e < s.x_experts; e++) out.push_back({p + "mlp.e" + std::to_string(e) + ".down", {l, IFA_LT_X_DOWN}});
    }
}

void SopulornNames(const LayeredDesc &d, std::vector<std::pair<std::string, std::pair<int, int>>> &out)
{
    out.push_back({"embed", {-1, IFA_T_EMBD}});
    if (d.cfg.bigram_buckets > 0) out.push_back({"bigram", {-1, IFA_T_BIGRAM}});
    out.push_back({"final.norm", {-1, IFA_T_OUT_NORM}});
    out.push_back({"head", {-1, IFA_T_LM_HEAD}});
    for (size_t li = 0; li < d.layers.size(); li++) {
        const ifa_layer_spec &s = d.layers[li];
        const std::string p = "l" + std::to_string(li) + ".";
        const int l = (int)li;
        out.push_back({p + "norm1", {l, IFA_LT_NORM1}}); out.push_back({p + "norm1b", {l, IFA_LT_NORM1B}});
        out.push_back({p + "mix.q", {l, IFA_LT_A_Q}}); out.push_back({p + "mix.q.b", {l, IFA_LT_A_Q_B}}); out.push_back({p + "mix.q.norm", {l, IFA_LT_A_Q_NORM}});
        if (s.a_kv_layer == 0) {
            out.push_back({p + "mix.k", {l, IFA_LT_A_K}}); out.push_back({p + "mix.k.b", {l, IFA_LT_A_K_B}}); out.push_back({p + "mix.k.norm", {l, IFA_LT_A_K_NORM}});
            out.push_back({p + "mix.v", {l, IFA_LT_A_V}}); out.push_back({p + "mix.v.b", {l, IFA_LT_A_V_B}});
        }
        out.push_back({p + "mix.o", {l, IFA_LT_A_O}});
        const bool moe = s.ffn_kind == IFA_FFN_MOE && s.x_experts > 0;
        if (!moe && s.ffn <= 0) continue;
        out.push_back({p + "norm2", {l, IFA_LT_NORM2}}); out.push_back({p + "norm2b", {l, IFA_LT_NORM2B}});
        if (!moe) {
            out.push_back({p + "mlp.gate", {l, IFA_LT_FFN_GATE}}); out.push_back({p + "mlp.up", {l, IFA_LT_FFN_UP}}); out.push_back({p + "mlp.down", {l, IFA_LT_FFN_DOWN}});
            continue;
        }
        out.push_back({p + "mlp.router", {l, IFA_LT_X_ROUTER}}); out.push_back({p + "mlp.router.b", {l, IFA_LT_X_ROUTER_B}});
        for (int e = 0; e < s.x_experts; e++) {      // per expert: its gate rows, then its up rows
            out.push_back({p + "mlp.e" + std::to_string(e) + ".gate", {l, IFA_LT_X_UP}});
            out.push_back({p + "mlp.e" + std::to_string(e) + ".up", {l, IFA_LT_X_UP}});
        }
        for (int e = 0; e < s.x_experts; e++) out.push_back({p + "mlp.e" + std::to_string(e) + ".down", {l, IFA_LT_X_DOWN}});
        if (s.x_shared_ff > 0) {
            out.push_back({p + "mlp.shared.gate", {l, IFA_LT_X_SH_GATE}}); out.push_back({p + "mlp.shared.up", {l, IFA_LT_X_SH_UP}});
            out.push_back({p + "mlp.shared.down", {l, IFA_LT_X_SH_DOWN}}); out.push_back({p + "mlp.shared.sg", {l, IFA_LT_X_SH_SG}});
        }
    }
}

// tensor name -> (layer, id).  Names that share (layer, id) are parts of ONE tensor, stacked row-wise in the order given (the experts).
void MuzopelNames(const LayeredDesc &d, std::vector<std::pair<std::string, std::pair<int, int>>> &out)
{
    out.push_back({"embed", {-1, IFA_T_EMBD}});
    out.push_back({"embed.norm", {-1, IFA_T_EMBD_NORM}});
    out.push_back({"final.norm", {-1, IFA_T_OUT_NORM}});
    out.push_back({"head", {-1, IFA_T_LM_HEAD}});
    for (size_t li = 0; li < d.layers.size(); li++) {
        const ifa_layer_spec &s = d.layers[li];
        const std::string p = "l" + std::to_string(li) + ".";
        const int l = (int)li;
        const bool moe = s.ffn_kind == IFA_FFN_MOE && s.x_experts + s.x_identity > 0;
        out.push_back({p + "norm1", {l, IFA_LT_NORM1}});
        if (s.canon_taps > 0) out.push_back({p + "canon1", {l, IFA_LT_CANON1}});
        out.push_back({p + "dwa", {l, IFA_LT_DWA}});
        if (s.m_q_rank > 0) {
            out.push_back({p + "mix.dq", {l, IFA_LT_M_DQ}}); out.push_back({p + "mix.dq.norm", {l, IFA_LT_M_DQ_NORM}}); out.push_back({p + "mix.uq", {l, IFA_LT_M_UQ}});
        } else out.push_back({p + "mix.q", {l, IFA_LT_M_Q}});
        out.push_back({p + "mix.dkv", {l, IFA_LT_M_DKV}}); out.push_back({p + "mix.dkv.norm", {l, IFA_LT_M_DKV_NORM}});
        out.push_back({p + "mix.uk", {l, IFA_LT_M_UK}}); out.push_back({p + "mix.uv", {l, IFA_LT_M_UV}});
        if (s.m_gate) out.push_back({p + "mix.g", {l, IFA_LT_M_G}});
        out.push_back({p + "mix.o", {l, IFA_LT_M_O}});
        if (!moe) continue;
        out.push_back({p + "norm2", {l, IFA_LT_NORM2}});
        if (s.canon_taps > 0) out.push_back({p + "canon2", {l, IFA_LT_CANON2}});
        out.push_back({p + "mlp.router", {l, IFA_LT_X_ROUTER}}); out.push_back({p + "mlp.correction", {l, IFA_LT_X_CORR}});
        for (int e = 0; e < s.x_experts; e++) out.push_back({p + "mlp.e" + std::to_string(e) + ".up", {l, IFA_LT_X_UP}});
        for (int e = 0; e < s.x_experts; e++) out.push_back({p + "mlp.e" + std::to_string(e) + ".down", {l, IFA_LT_X_DOWN}});
    }
}

bool NoSizesFromTensors(const std::map<std::string, StTensorEntry> &, LayeredDesc &) { return true; }

struct NameId { const char *suffix; int id; };
const NameId kGelaraxCommon[] = {{"norm1", IFA_LT_NORM1}, {"ls1", IFA_LT_LS1}, {"ls2", IFA_LT_LS2}, {"mlp.gate", IFA_LT_FFN_GATE}, {"mlp.gate.b", IFA_LT_FFN_GATE_B},
                                 {"mlp.up", IFA_LT_FFN_UP}, {"mlp.up.b", IFA_LT_FFN_UP_B}, {"mlp.down", IFA_LT_FFN_DOWN}, {"mlp.down.b", IFA_LT_FFN_DOWN_B}};
const NameId kGelaraxParallel[] = {{"mix.left.q", IFA_LT_A_Q}, {"mix.left.k", IFA_LT_A_K}, {"mix.left.rel", IFA_LT_A_REL}, {"mix.left.sink", IFA_LT_A_SINK},
                                   {"mix.left.o", IFA_LT_A_O}, {"mix.right.q", IFA_LT_L_Q}, {"mix.right.k", IFA_LT_L_K}, {"mix.right.v", IFA_LT_L_V},
                                   {"mix.right.g", IFA_LT_L_G}, {"mix.right.o", IFA_LT_L_O}, {"mix.right.norm", IFA_LT_L_NORM}};
const NameId kGelaraxDelta[] = {{"mix.q", IFA_LT_D_Q}, {"mix.k", IFA_LT_D_K}, {"mix.v", IFA_LT_D_V}, {"mix.q.conv", IFA_LT_D_QCONV}, {"mix.k.conv", IFA_LT_D_KCONV},
                                {"mix.v.conv", IFA_LT_D_VCONV}, {"mix.b", IFA_LT_D_B}, {"mix.a", IFA_LT_D_A}, {"mix.A_log", IFA_LT_D_ALOG},
                                {"mix.dt_bias", IFA_LT_D_DTBIAS}, {"mix.g", IFA_LT_D_G}, {"mix.norm", IFA_LT_D_NORM}, {"mix.o", IFA_LT_D_O}};

// tensor name -> (layer, id) for Gelarax: "embed", "final.norm", "head", "l<i>.<suffix>"
void GelaraxNames(const LayeredDesc &d, std::vector<std::pair<std::string, std::pair<int, int>>> &out)
{
    out.push_back({"embed", {-1, IFA_T_EMBD}});
    out.push_back({"final.norm", {-1, IFA_T_OUT_NORM}});
    out.push_back({"head", {-1, IFA_T_LM_HEAD}});
    for (size_t li = 0; li < d.layers.size(); li++) {
        const std::string p = "l" + std::to_string(li) + ".";
        for (const NameId &n : kGelaraxCommon) {
            const bool ffn_part = n.id != IFA_LT_NORM1 && n.id != IFA_LT_LS1;
            if (ffn_part && d.layers[li].ffn <= 0) continue;
            out.push_back({p + n.suffix, {(int)li, n.id}});
        }
        if (d.layers[li].mixer == IFA_MIX_WINDOW_LINEAR) for (const NameId &n : kGelaraxParallel) out.push_back({p + n.suffix, {(int)li, n.id}});
        else for (const NameId &n : kGelaraxDelta) out.push_back({p + n.suffix, {(int)li, n.id}});
    }
}

// sizes that only a tensor's shape gives: the number of rows of a layer's distance-bias table
bool GelaraxSizesFromTensors(const std::map<std::string, StTensorEntry> &index, LayeredDesc &d)
{
    for (size_t li = 0; li < d.layers.size(); li++) {
        if (d.layers[li].mixer != IFA_MIX_WINDOW_LINEAR) continue;
        const std::string name = "l" + std::to_string(li) + ".mix.left.rel";
        auto it = index.find(name);
        if (it == index.end() || it->second.shape.size() != 2 || it->second.shape[0] < 1) { EngineSetError("tensor %s is missing or not a matrix", name.c_str()); return false; }
        d.layers[li].a_buckets = (int)it->second.shape[0];
    }
    return true;
}

struct ArchEntry {
    const char *name;
    bool (*parse)(const JsonValue &root, LayeredDesc &d);
    bool (*sizes_from_tensors)(const std::map<std::string, StTensorEntry> &index, LayeredDesc &d);
    void (*names)(const LayeredDesc &d, std::vector<std::pair<std::string, std::pair<int, int>>> &out);
};
const ArchEntry kArchitectures[] = {{"Gelarax", ParseGelarax, GelaraxSizesFromTensors, GelaraxNames},
                                    {"Muzopel", ParseMuzopel, NoSizesFromTensors, MuzopelNames},
                                    {"Sopulorn", ParseSopulorn, NoSizesFromTensors, SopulornNames},
                                    {"Bogupel", ParseBogupel, BogupelSizesFromTensors, BogupelNames}};

const ArchEntry *FindArch(const std::string &name)
{
    for (const ArchEntry &a : kArchitectures) if (name == a.name) return &a;
    return nullptr;
}

bool ParseDir(const ModelSpec &spec, LayeredDesc &d, const ArchEntry **arch)
{
    std::string text;
    const std::string path = spec.dir + (spec.config_file.empty() ? "config.json" : spec.config_file);
    if (!ReadText(path, text)) { EngineSetError("Cannot open %s", path.c_str()); return false; }
    JsonValue root; JsonParser jp; std::string err;
    if (!jp.Parse(text, root, &err) || root.type != JsonValue::Object) { EngineSetError("%s: %s", path.c_str(), err.c_str()); return false; }
    std::string name;
    root.GetString("architecture", name);
    *arch = FindArch(name);
    if (!*arch) { EngineSetError("%s: architecture \"%s\" is not registered", path.c_str(), name.c_str()); return false; }
    return (*arch)->parse(root, d);
}

} // namespace

bool LayeredArchitectureOf(const std::string &dir, std::string &arch)
{
    std::string text;
    if (!ReadText(dir + "config.json", text)) return false;
    JsonValue root; JsonParser jp;
    if (!jp.Parse(text, root) || root.type != JsonValue::Object) return false;
    return root.GetString("architecture", arch) && FindArch(arch) != nullptr;
}

// fills the spec of a layer-list model from its config.json (hyper-parameters for model_info; format "layered")
bool LoadLayeredSpec(ModelSpec &spec)
{
    LayeredDesc d; const ArchEntry *arch = nullptr;
    if (!ParseDir(spec, d, &arch)) return false;
    spec.architecture = arch->name;
    spec.network_structure = std::string("layered.") + arch->name;
    spec.model_file_format = "layered";
    if (spec.model_files.empty()) spec.model_files.push_back("model.safetensors");
    spec.hyper_params.vocab_size = d.cfg.vocab; spec.hyper_params.embd_dims = d.cfg.width; spec.hyper_params.decoder_layers = d.cfg.n_layers;
    spec.unk_token_id = -1;          // no vocabulary file: no id is withheld from selection
    return true;
}

bool LoadLayered(std::vector<WorkerPlan> &plans, ModelSpec &spec)
{
    if (plans.size() != 1 || plans[0].n_stages > 1 || plans[0].tp_size > 1) { EngineSetError("model %s: layer-list models run on one device", spec.sid.c_str()); return false; }
    LayeredDesc d; const ArchEntry *arch = nullptr;
    if (!ParseDir(spec, d, &arch)) return false;
    WorkerPlan &w = plans[0];
    d.cfg.device = w.device;
    d.cfg.max_ctx = spec.max_context_len > 0 ? spec.max_context_len : ModelSpec::DEFAULT_MAX_CONTEXT_LEN;
    d.cfg.ops32 = spec.exact_fp32 ? 1 : 0;
    w.layer0 = 0; w.layer1 = d.cfg.n_layers;
    std::map<std::string, StTensorEntry> index;
    for (const std::string &f : spec.model_files) if (!IndexSafetensorsFile(spec.dir + f, index)) return false;
    if (!arch->sizes_from_tensors(index, d)) return false;
    if (ifa_model_create_layered(&d.cfg, d.layers.data(), &w.model) != IFA_OK) { EngineSetError("ifa_model_create_layered: %s", ifa_last_error()); return false; }
    std::vector<std::pair<std::string, std::pair<int, int>>> names;
    arch->names(d, names);
    std::vector<uint8_t> raw, stacked;
    size_t stacked_rows = 0, stacked_cols = 0;
    for (size_t ni = 0; ni < names.size(); ni++) {
        const auto &nm = names[ni];
        auto it = index.find(nm.first);
        if (it == index.end()) { EngineSetError("tensor %s is missing in %s", nm.first.c_str(), spec.dir.c_str()); return false; }
        const StTensorEntry &e = it->second;
        if (e.dtype != "BF16") { EngineSetError("tensor %s: dtype %s (bfloat16 expected)", nm.first.c_str(), e.dtype.c_str()); return false; }
        size_t cnt = 1; for (size_t x : e.shape) cnt *= x;
        if (e.end - e.begin != cnt * 2 || cnt == 0) { EngineSetError("tensor %s: %zu bytes for %zu values", nm.first.c_str(), e.end - e.begin, cnt); return false; }
        raw.resize(cnt * 2);
        FILE *fp = fopen(e.file.c_str(), "rb");
        if (!fp) { EngineSetError("Failed to open file %s", e.file.c_str()); return false; }
        fseek(fp, (long)(e.data_off + e.begin), SEEK_SET);
        const bool ok = fread(raw.data(), 1, raw.size(), fp) == raw.size();
        fclose(fp);
        if (!ok) { EngineSetError("%s is truncated (tensor %s)", e.file.c_str(), nm.first.c_str()); return false; }
        size_t rows = e.shape.size() >= 2 ? e.shape[0] : 1, cols = e.shape.size() >= 2 ? cnt / e.shape[0] : cnt;
        // consecutive names with the same (layer, id) are parts of one tensor, stacked row-wise
        const bool more = ni + 1 < names.size() && names[ni + 1].second == nm.second, part = more || !stacked.empty();
        if (part) {
            if (!stacked.empty() && cols != stacked_cols) { EngineSetError("tensor %s: %zu columns, the parts before it have %zu", nm.first.c_str(), cols, stacked_cols); return false; }
            stacked.insert(stacked.end(), raw.begin(), raw.end());
            stacked_rows += rows; stacked_cols = cols;
            if (more) continue;
            rows = stacked_rows;
        }
        const int rc = ifa_model_set_tensor_host(w.model, nm.second.first, nm.second.second, IFA_BF16, part ? stacked.data() : raw.data(), rows, cols);
        stacked.clear(); stacked_rows = 0;
        if (rc != IFA_OK) { EngineSetError("tensor %s: %s", nm.first.c_str(), ifa_last_error()); return false; }
    }
    for (size_t li = 0; li < d.layers.size(); li++)
        if (d.layers[li].mixer == IFA_MIX_WINDOW_LINEAR
            && ifa_model_set_tensor_host(w.model, (int)li, IFA_LT_L_DECAY, IFA_F32, d.decays[li].data(), 1, d.decays[li].size()) != IFA_OK) {
            EngineSetError("layer %zu decay: %s", li, ifa_last_error()); return false;
        }
    return true;
}

} // namespace inferflow_amd
