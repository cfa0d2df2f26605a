// model_registry.cpp — architecture name of a configuration file -> the model family that runs it and that family's description.
// Dense decoder graphs (Qwen3Config, reference src/models/qwen3.rs:26-125) fill an nvr_model_config; layer-list designs fill a LayeredSpec.
#include <cmath>
#include <cstring>
#include "common.h"
#include "layered_model.h"

namespace nvr {

namespace {

struct Reader {                                            // typed access with the path of the key in the error text
    std::string err;
    const Json *need(const Json &o, const char *key, const std::string &where) {
        const Json *v = o.get(key);
        if (!v && err.empty()) err = "config: '" + where + key + "' is missing";
        return v;
    }
    double num(const Json &o, const char *key, const std::string &where) {
        const Json *v = need(o, key, where);
        if (!v) return 0;
        if (v->kind != Json::Num) { if (err.empty()) err = "config: '" + where + key + "' is not a number"; return 0; }
        return v->num;
    }
    int64_t integer(const Json &o, const char *key, const std::string &where) {
        const double d = num(o, key, where);
        if (d != std::floor(d) && err.empty()) err = "config: '" + where + key + "' is not an integer";
        return (int64_t)d;
    }
};

int parse_qwen3(const Json &c, nvr_model_spec *out) {
    nvr_model_config &m = out->dense;
    nvr_model_config_default(&m);
    Reader rd;
    m.vocab_size = (uint64_t)rd.integer(c, "vocab_size", ""); m.hidden_size = (uint64_t)rd.integer(c, "hidden_size", "");
    m.intermediate_size = (uint64_t)rd.integer(c, "intermediate_size", ""); m.num_hidden_layers = (uint64_t)rd.integer(c, "num_hidden_layers", "");
    m.num_attention_heads = (uint64_t)rd.integer(c, "num_attention_heads", "");
    if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
    auto opt = [&](const char *k, double d) { const Json *v = c.get(k); return v && v->kind == Json::Num ? v->num : d; };
    auto flag = [&](const char *k, bool d) { const Json *v = c.get(k); return v && v->kind == Json::Bool ? v->b : d; };
    m.num_key_value_heads = (uint64_t)opt("num_key_value_heads", (double)m.num_attention_heads);
    m.head_dim = (uint64_t)opt("head_dim", 0);
    m.max_position_embeddings = (uint64_t)opt("max_position_embeddings", 32768);
    m.rms_norm_eps = (float)opt("rms_norm_eps", 1e-6); m.rope_theta = opt("rope_theta", 10000.0);
    m.tie_word_embeddings = flag("tie_word_embeddings", false);
    m.qk_norm = flag("qk_norm", true);                      // checkpoints of this architecture carry q_norm / k_norm
    m.use_bias = flag("attention_bias", false);
    out->family = 0;
    return NVR_OK;
}

int parse_rugudra_spec(const Json &c, nvr_model_spec *out) {
    out->family = 1;
    return LayeredSpec::parse_rugudra(c, &out->layered);
}

int parse_pusunex_spec(const Json &c, nvr_model_spec *out) {
    out->family = 1;
    return LayeredSpec::parse_pusunex(c, &out->layered);
}

int parse_sosutar_spec(const Json &c, nvr_model_spec *out) {
    out->family = 1;
    return LayeredSpec::parse_sosutar(c, &out->layered);
}

int parse_sokalorn_spec(const Json &c, nvr_model_spec *out) {
    out->family = 1;
    return LayeredSpec::parse_sokalorn(c, &out->layered);
}

struct Entry { const char *name; int (*parse)(const Json &, nvr_model_spec *); };
const Entry kRegistry[] = {
    {"Qwen3ForCausalLM", parse_qwen3},
    {"Rugudra", parse_rugudra_spec},
    {"Pusunex", parse_pusunex_spec},
    {"Sosutar", parse_sosutar_spec},
    {"Sokalorn", parse_sokalorn_spec},
};

}  // namespace

// Rugudra: every sublayer reads norm(x) through a short causal convolution; the mixer is softmax attention with a logarithmic distance
// penalty and a sink, or retention; x <- x + m * (mixer + feed-forward); a range of layers may run several times.
int LayeredSpec::parse_rugudra(const Json &c, LayeredSpec *s) {
    Reader rd;
    s->vocab = rd.integer(c, "vocab", ""); s->width = rd.integer(c, "width", "");
    s->residual_mult = rd.num(c, "residual_mult", "");
    if (const Json *e = rd.need(c, "embedding", "")) s->embedding_scale = rd.num(*e, "scale", "embedding.");
    if (const Json *n = rd.need(c, "norm", "")) s->eps = rd.num(*n, "eps", "norm.");
    if (const Json *k = rd.need(c, "canon", "")) s->taps = rd.integer(*k, "taps", "canon.");
    const Json *layers = rd.need(c, "layers", "");
    if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
    if (layers->kind != Json::Arr || layers->arr.empty()) return fail(NVR_ERR_INVALID_ARG, "config: 'layers' is not a list of layers");
    s->layers.clear();
    for (size_t i = 0; i < layers->arr.size(); ++i) {
        const Json &lj = layers->arr[i];
        const std::string w = "layers[" + std::to_string(i) + "].";
        Layer L;
        const Json *type = rd.need(lj, "type", w), *mx = rd.need(lj, "mixer", w);
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (type->kind != Json::Str) return fail(NVR_ERR_INVALID_ARG, "config: '%stype' is not a string", w.c_str());
        L.heads = rd.integer(*mx, "heads", w + "mixer."); L.dim = rd.integer(*mx, "dim", w + "mixer."); L.vdim = rd.integer(*mx, "vdim", w + "mixer.");
        if (type->str == "attention") {
            L.mixer = ATTENTION;
            L.kv_heads = rd.integer(*mx, "kv_heads", w + "mixer."); L.scale = rd.num(*mx, "scale", w + "mixer.");
        } else if (type->str == "retention") {
            L.mixer = RETENTION; L.kv_heads = L.heads;
            const Json *d = rd.need(*mx, "decay", w + "mixer.");
            if (d) {
                if (d->kind != Json::Arr) return fail(NVR_ERR_INVALID_ARG, "config: '%smixer.decay' is not a list", w.c_str());
                for (const Json &v : d->arr) L.decay.push_back(v.num);
            }
            const Json *rot = mx->get("rot");
            if (rot && !rot->is_null()) { L.rot_dims = rd.integer(*rot, "dims", w + "mixer.rot."); L.rot_base = rd.num(*rot, "base", w + "mixer.rot."); }
        } else return fail(NVR_ERR_UNSUPPORTED, "config: layer type '%s' (attention or retention)", type->str.c_str());
        const Json *mlp = lj.get("mlp");
        if (mlp && !mlp->is_null()) {
            const Json *kind = mlp->get("kind");
            if (kind && !(kind->kind == Json::Str && kind->str == "dense")) return fail(NVR_ERR_UNSUPPORTED, "config: '%smlp.kind' (dense)", w.c_str());
            L.has_mlp = true; L.ff = rd.integer(*mlp, "ff", w + "mlp."); L.limit = rd.num(*mlp, "limit", w + "mlp.");
        }
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (L.heads < 1 || L.dim < 1 || L.vdim < 1 || L.kv_heads < 1 || L.heads % L.kv_heads)
            return fail(NVR_ERR_INVALID_ARG, "config: %s %ld heads over %ld key/value heads of %ld / %ld", w.c_str(), (long)L.heads, (long)L.kv_heads, (long)L.dim, (long)L.vdim);
        if (L.mixer == RETENTION && ((int64_t)L.decay.size() != L.heads || L.rot_dims % 2 || L.rot_dims > L.dim || L.rot_dims < 0))
            return fail(NVR_ERR_INVALID_ARG, "config: %s needs one decay per head and an even number of rotated coordinates <= dim", w.c_str());
        if (L.has_mlp && L.ff < 1) return fail(NVR_ERR_INVALID_ARG, "config: '%smlp.ff' must be positive", w.c_str());
        s->layers.push_back(L);
    }
    const int64_t n = (int64_t)s->layers.size();
    s->runs.clear();
    const Json *loop = c.get("loop");
    if (loop && !loop->is_null()) {
        const int64_t a = rd.integer(*loop, "start", "loop."), b = rd.integer(*loop, "stop", "loop."), t = rd.integer(*loop, "times", "loop.");
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (a < 0 || b < a || b > n || t < 1) return fail(NVR_ERR_INVALID_ARG, "config: loop [%ld, %ld) x %ld over %ld layers", (long)a, (long)b, (long)t, (long)n);
        for (int64_t i = 0; i < a; ++i) s->runs.push_back((int)i);
        for (int64_t k = 0; k < t; ++k) for (int64_t i = a; i < b; ++i) s->runs.push_back((int)i);
        for (int64_t i = b; i < n; ++i) s->runs.push_back((int)i);
    } else
        for (int64_t i = 0; i < n; ++i) s->runs.push_back((int)i);
    if (s->vocab < 1 || s->width < 1 || s->taps < 1) return fail(NVR_ERR_INVALID_ARG, "config: vocab, width and canon.taps must be positive");
    return NVR_OK;
}

// Pusunex: x <- x + nb(mixer(n(x))), x <- x + nb(ff(n(x))) with RMS norms in groups; mixers 'latent_attention' (cached latent, optional 'kv_from' an earlier
// layer, output gate), 'latent_attention_2' (latent queries, a rotated key part shared by the heads) and 'gla' (gated linear attention); feed-forward 'dense'
// (polynomial-norm activation) or 'moe' (sigmoid router, top-k, shared expert); a per-layer token input ('token_side') and a weighted average over depth.
int LayeredSpec::parse_pusunex(const Json &c, LayeredSpec *s) {
    Reader rd;
    s->layout = SEQUENTIAL; s->taps = 1; s->embedding_scale = 1.0; s->residual_mult = 1.0;
    s->vocab = rd.integer(c, "vocab", ""); s->width = rd.integer(c, "width", "");
    if (const Json *n = rd.need(c, "norm", "")) { s->eps = rd.num(*n, "eps", "norm."); s->norm_groups = rd.integer(*n, "groups", "norm."); }
    const Json *side = c.get("token_side");
    s->side_dim = (side && !side->is_null()) ? rd.integer(*side, "dim", "token_side.") : 0;
    const Json *layers = rd.need(c, "layers", "");
    if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
    if (layers->kind != Json::Arr || layers->arr.empty()) return fail(NVR_ERR_INVALID_ARG, "config: 'layers' is not a list of layers");
    if (s->vocab < 1 || s->width < 1 || s->norm_groups < 1 || s->width % s->norm_groups || s->side_dim < 0)
        return fail(NVR_ERR_INVALID_ARG, "config: vocab and width must be positive, and norm.groups must divide the width");
    s->layers.clear(); s->runs.clear();
    for (size_t i = 0; i < layers->arr.size(); ++i) {
        const Json &lj = layers->arr[i];
        const std::string w = "layers[" + std::to_string(i) + "].", wm = w + "mixer.";
        Layer L;
        const Json *type = rd.need(lj, "type", w), *mx = rd.need(lj, "mixer", w);
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (type->kind != Json::Str) return fail(NVR_ERR_INVALID_ARG, "config: '%stype' is not a string", w.c_str());
        L.heads = rd.integer(*mx, "heads", wm); L.dim = rd.integer(*mx, "dim", wm); L.vdim = rd.integer(*mx, "vdim", wm);
        if (type->str == "latent_attention" || type->str == "latent_attention_2") {
            L.mixer = LATENT; L.kv_heads = 1;
            L.kv_rank = rd.integer(*mx, "kv_rank", wm); L.scale = rd.num(*mx, "scale", wm);
            if (type->str == "latent_attention") {
                L.out_gate = true;
                const Json *from = mx->get("kv_from");
                if (from && !from->is_null()) {
                    L.kv_from = rd.integer(*mx, "kv_from", wm);
                    if (L.kv_from < 0 || L.kv_from >= (int64_t)i) return fail(NVR_ERR_INVALID_ARG, "config: '%skv_from' must name an earlier layer", w.c_str());
                    const Layer &src = s->layers[(size_t)L.kv_from];
                    if (src.mixer != LATENT || src.kv_from >= 0 || src.kv_rank != L.kv_rank || src.rot_dim != 0)
                        return fail(NVR_ERR_INVALID_ARG, "config: '%skv_from' must name a latent-attention layer with a latent of its own and the same kv_rank", w.c_str());
                }
            } else {
                L.q_rank = rd.integer(*mx, "q_rank", wm); L.rot_dim = rd.integer(*mx, "rot_dim", wm);
                const Json *rot = rd.need(*mx, "rot", wm);
                if (rot) {
                    L.rot_dims = rd.integer(*rot, "dims", wm + "rot."); L.rot_base = rd.num(*rot, "base", wm + "rot.");
                    if (rd.err.empty() && (L.rot_dims != L.rot_dim || L.rot_dim % 2 || L.rot_dim < 0 || L.q_rank < 1))
                        return fail(NVR_ERR_INVALID_ARG, "config: %s rotates rot.dims = rot_dim coordinates, an even number, and needs a q_rank", w.c_str());
                }
            }
            if (rd.err.empty() && L.kv_rank < 1) return fail(NVR_ERR_INVALID_ARG, "config: '%skv_rank' must be positive", w.c_str());
        } else if (type->str == "gla") {
            L.mixer = GLA; L.kv_heads = L.heads; L.tau = rd.num(*mx, "tau", wm);
            if (rd.err.empty() && !(L.tau > 0)) return fail(NVR_ERR_INVALID_ARG, "config: '%stau' must be positive", w.c_str());
        } else return fail(NVR_ERR_UNSUPPORTED, "config: layer type '%s' (latent_attention, latent_attention_2 or gla)", type->str.c_str());
        const Json *mlp = lj.get("mlp");
        if (mlp && !mlp->is_null()) {
            const Json *kind = rd.need(*mlp, "kind", w + "mlp.");
            if (kind && kind->kind == Json::Str && kind->str == "dense") { L.ff_kind = FF_POLY; L.ff = rd.integer(*mlp, "ff", w + "mlp."); }
            else if (kind && kind->kind == Json::Str && kind->str == "moe") {
                L.ff_kind = FF_MOE;
                const Json *ex = rd.need(*mlp, "expert", w + "mlp."), *ro = rd.need(*mlp, "router", w + "mlp."), *sh = mlp->get("shared");
                if (ex) L.expert_ff = rd.integer(*ex, "ff", w + "mlp.expert.");
                if (ro) { L.experts = rd.integer(*ro, "experts", w + "mlp.router."); L.top = rd.integer(*ro, "top", w + "mlp.router."); }
                if (sh && !sh->is_null()) L.shared_ff = rd.integer(*sh, "ff", w + "mlp.shared.");
                if (rd.err.empty() && (L.expert_ff < 1 || L.experts < 1 || L.top < 1 || L.top > L.experts || L.shared_ff < 0))
                    return fail(NVR_ERR_INVALID_ARG, "config: %smlp needs positive expert sizes and 1 <= top <= experts", w.c_str());
            } else if (kind) return fail(NVR_ERR_UNSUPPORTED, "config: '%smlp.kind' (dense or moe)", w.c_str());
            L.has_mlp = true;
            if (rd.err.empty() && L.ff_kind == FF_POLY && L.ff < 1) return fail(NVR_ERR_INVALID_ARG, "config: '%smlp.ff' must be positive", w.c_str());
        }
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (L.heads < 1 || L.dim < 1 || L.vdim < 1) return fail(NVR_ERR_INVALID_ARG, "config: %s heads, dim and vdim must be positive", w.c_str());
        s->layers.push_back(L); s->runs.push_back((int)i);
    }
    return NVR_OK;
}

// Sosutar: x <- x + ls1 * mixer(n1(x)), x <- x + ls2 * ff(n2(x)); learned positions; mixers 'mlstm' (matrix memory with exponential gates capped by gate_cap) and
// 'parallel' (mixer.left: attention with mask.size, q_temp.{coef, every}, scale; mixer.right: a gated recurrence of 'width' channels); feed-forward 'dense'
// (squared ReLU) or none; 'weights_of': j gives a layer the tensors of layer j and a cache / state of its own.
int LayeredSpec::parse_sosutar(const Json &c, LayeredSpec *s) {
    Reader rd;
    s->layout = SCALED; s->taps = 1; s->residual_mult = 1.0; s->norm_groups = 1;
    s->vocab = rd.integer(c, "vocab", ""); s->width = rd.integer(c, "width", "");
    s->max_positions = rd.integer(c, "max_positions", ""); s->logit_scale = rd.num(c, "logit_scale", "");
    if (const Json *e = rd.need(c, "embedding", "")) s->embedding_scale = rd.num(*e, "scale", "embedding.");
    if (const Json *n = rd.need(c, "norm", "")) s->eps = rd.num(*n, "eps", "norm.");
    const Json *layers = rd.need(c, "layers", "");
    if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
    if (layers->kind != Json::Arr || layers->arr.empty()) return fail(NVR_ERR_INVALID_ARG, "config: 'layers' is not a list of layers");
    if (s->vocab < 1 || s->width < 1 || s->max_positions < 1) return fail(NVR_ERR_INVALID_ARG, "config: vocab, width and max_positions must be positive");
    s->layers.clear(); s->runs.clear();
    for (size_t i = 0; i < layers->arr.size(); ++i) {
        const Json &lj = layers->arr[i];
        const std::string w = "layers[" + std::to_string(i) + "].", wm = w + "mixer.";
        Layer L;
        const Json *type = rd.need(lj, "type", w), *mx = rd.need(lj, "mixer", w);
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (type->kind != Json::Str) return fail(NVR_ERR_INVALID_ARG, "config: '%stype' is not a string", w.c_str());
        if (type->str == "mlstm") {
            L.mixer = MLSTM;
            L.heads = rd.integer(*mx, "heads", wm); L.dim = rd.integer(*mx, "dim", wm); L.vdim = rd.integer(*mx, "vdim", wm); L.kv_heads = L.heads;
            L.gate_cap = rd.num(*mx, "gate_cap", wm);
            if (rd.err.empty() && !(L.gate_cap > 0)) return fail(NVR_ERR_INVALID_ARG, "config: '%sgate_cap' must be positive", wm.c_str());
        } else if (type->str == "parallel") {
            L.mixer = ATTN_GRU;
            const Json *lf = rd.need(*mx, "left", wm), *rt = rd.need(*mx, "right", wm);
            if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
            const std::string wl = wm + "left.";
            L.heads = rd.integer(*lf, "heads", wl); L.kv_heads = rd.integer(*lf, "kv_heads", wl); L.dim = rd.integer(*lf, "dim", wl); L.vdim = rd.integer(*lf, "vdim", wl);
            L.scale = rd.num(*lf, "scale", wl);
            if (const Json *m = rd.need(*lf, "mask", wl)) L.window = rd.integer(*m, "size", wl + "mask.");
            if (const Json *t = rd.need(*lf, "q_temp", wl)) { L.temp_coef = rd.num(*t, "coef", wl + "q_temp."); L.temp_every = rd.integer(*t, "every", wl + "q_temp."); }
            L.gru_width = rd.integer(*rt, "width", wm + "right.");
            if (rd.err.empty() && (L.window < 1 || L.temp_every < 1 || L.gru_width < 1))
                return fail(NVR_ERR_INVALID_ARG, "config: %s mask.size, q_temp.every and right.width must be positive", wm.c_str());
        } else return fail(NVR_ERR_UNSUPPORTED, "config: layer type '%s' (mlstm or parallel)", type->str.c_str());
        const Json *mlp = lj.get("mlp");
        if (mlp && !mlp->is_null()) {
            const Json *kind = rd.need(*mlp, "kind", w + "mlp.");
            if (kind && !(kind->kind == Json::Str && kind->str == "dense")) return fail(NVR_ERR_UNSUPPORTED, "config: '%smlp.kind' (dense)", w.c_str());
            L.has_mlp = true; L.ff_kind = FF_RELU2; L.ff = rd.integer(*mlp, "ff", w + "mlp.");
            if (rd.err.empty() && L.ff < 1) return fail(NVR_ERR_INVALID_ARG, "config: '%smlp.ff' must be positive", w.c_str());
        }
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (L.heads < 1 || L.dim < 1 || L.vdim < 1 || L.kv_heads < 1 || L.heads % L.kv_heads)
            return fail(NVR_ERR_INVALID_ARG, "config: %s %ld heads over %ld key/value heads of %ld / %ld", w.c_str(), (long)L.heads, (long)L.kv_heads, (long)L.dim, (long)L.vdim);
        const Json *wof = lj.get("weights_of");
        if (wof && !wof->is_null()) {
            L.weights_of = rd.integer(lj, "weights_of", w);
            if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        }
        s->layers.push_back(L);
    }
    // a layer may name any other layer (also a later one, or one that borrows itself): the tensors are those of the layer the chain ends at
    const int64_t n = (int64_t)s->layers.size();
    std::vector<int64_t> src((size_t)n);
    for (int64_t i = 0; i < n; ++i) {
        int64_t j = i, hops = 0;
        while (s->layers[(size_t)j].weights_of >= 0 || s->layers[(size_t)j].weights_of < -1) {
            const int64_t k = s->layers[(size_t)j].weights_of;
            if (k < 0 || k >= n || k == j || ++hops > n) return fail(NVR_ERR_INVALID_ARG, "config: 'layers[%ld].weights_of' must name another layer that leads to tensors", (long)i);
            j = k;
        }
        src[(size_t)i] = j;
        const Layer &o = s->layers[(size_t)j], &L = s->layers[(size_t)i];
        if (o.mixer != L.mixer || o.heads != L.heads || o.kv_heads != L.kv_heads || o.dim != L.dim || o.vdim != L.vdim || o.gru_width != L.gru_width || o.has_mlp != L.has_mlp || o.ff != L.ff)
            return fail(NVR_ERR_INVALID_ARG, "config: 'layers[%ld].weights_of' names a layer of other sizes", (long)i);
    }
    for (int64_t i = 0; i < n; ++i) {
        if (src[(size_t)i] != i) s->layers[(size_t)i].weights_of = src[(size_t)i];
        s->runs.push_back((int)src[(size_t)i]);
    }
    return NVR_OK;
}

// Sokalorn: x <- x + mixer(shift(n(x))) + ff(n(x)) with one RMS norm per layer; mixers 'mamba2' (mixer.{heads, vdim, state, groups, conv, norm_groups}) and 'parallel'
// (mixer.left: attention with rot.{dims, base, scaling.factor}, scale, softcap, mask.size — a chunk —, sigmoid weights; mixer.right: time mixing with heads x dim);
// feed-forward 'moe' (expert.{ff, limit}, router.{experts, top}, optional shared.{ff, limit}) or none; 'loop': layers start .. stop-1 run `times` times, every pass
// behind a product over [x ; embedding output].
int LayeredSpec::parse_sokalorn(const Json &c, LayeredSpec *s) {
    Reader rd;
    s->layout = JOINT; s->taps = 1; s->residual_mult = 1.0; s->norm_groups = 1; s->embedding_scale = 1.0;
    s->vocab = rd.integer(c, "vocab", ""); s->width = rd.integer(c, "width", "");
    if (const Json *n = rd.need(c, "norm", "")) s->eps = rd.num(*n, "eps", "norm.");
    const Json *layers = rd.need(c, "layers", "");
    if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
    if (layers->kind != Json::Arr || layers->arr.empty()) return fail(NVR_ERR_INVALID_ARG, "config: 'layers' is not a list of layers");
    if (s->vocab < 1 || s->width < 1) return fail(NVR_ERR_INVALID_ARG, "config: vocab and width must be positive");
    s->layers.clear(); s->runs.clear(); s->pass_start.clear(); s->has_loop = false;
    for (size_t i = 0; i < layers->arr.size(); ++i) {
        const Json &lj = layers->arr[i];
        const std::string w = "layers[" + std::to_string(i) + "].", wm = w + "mixer.";
        Layer L;
        const Json *type = rd.need(lj, "type", w), *mx = rd.need(lj, "mixer", w);
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (type->kind != Json::Str) return fail(NVR_ERR_INVALID_ARG, "config: '%stype' is not a string", w.c_str());
        if (type->str == "mamba2") {
            L.mixer = SSM;
            L.heads = rd.integer(*mx, "heads", wm); L.vdim = rd.integer(*mx, "vdim", wm); L.dim = rd.integer(*mx, "state", wm); L.kv_heads = rd.integer(*mx, "groups", wm);
            L.conv_taps = rd.integer(*mx, "conv", wm); L.mix_norm_groups = rd.integer(*mx, "norm_groups", wm);
            if (rd.err.empty() && (L.conv_taps < 1 || L.mix_norm_groups < 1 || L.heads < 1 || L.vdim < 1 || (L.heads * L.vdim) % L.mix_norm_groups))
                return fail(NVR_ERR_INVALID_ARG, "config: %s conv must be positive and norm_groups must divide heads * vdim", wm.c_str());
        } else if (type->str == "parallel") {
            L.mixer = ATTN_TMIX;
            const Json *lf = rd.need(*mx, "left", wm), *rt = rd.need(*mx, "right", wm);
            if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
            const std::string wl = wm + "left.";
            L.heads = rd.integer(*lf, "heads", wl); L.kv_heads = rd.integer(*lf, "kv_heads", wl); L.dim = rd.integer(*lf, "dim", wl); L.vdim = rd.integer(*lf, "vdim", wl);
            L.scale = rd.num(*lf, "scale", wl);
            const Json *cap = lf->get("softcap");
            if (cap && !cap->is_null()) L.softcap = rd.num(*lf, "softcap", wl);
            const Json *mask = lf->get("mask");
            if (mask && !mask->is_null()) L.chunk = rd.integer(*mask, "size", wl + "mask.");
            const Json *rot = lf->get("rot");
            if (rot && !rot->is_null()) {
                L.rot_dims = rd.integer(*rot, "dims", wl + "rot."); L.rot_base = rd.num(*rot, "base", wl + "rot.");
                const Json *sc = rot->get("scaling");
                if (sc && !sc->is_null()) L.rot_factor = rd.num(*sc, "factor", wl + "rot.scaling.");
            }
            L.t_heads = rd.integer(*rt, "heads", wm + "right."); L.t_dim = rd.integer(*rt, "dim", wm + "right.");
            if (rd.err.empty() && (L.chunk < 0 || L.softcap < 0 || L.rot_dims < 0 || L.rot_dims % 2 || L.rot_dims > L.dim || !(L.rot_factor > 0) || L.t_heads < 1 || L.t_dim < 1))
                return fail(NVR_ERR_INVALID_ARG, "config: %s needs an even rot.dims <= dim, a positive scaling factor and positive right.heads / right.dim", wm.c_str());
        } else return fail(NVR_ERR_UNSUPPORTED, "config: layer type '%s' (mamba2 or parallel)", type->str.c_str());
        const Json *mlp = lj.get("mlp");
        if (mlp && !mlp->is_null()) {
            const Json *kind = rd.need(*mlp, "kind", w + "mlp.");
            if (kind && !(kind->kind == Json::Str && kind->str == "moe")) return fail(NVR_ERR_UNSUPPORTED, "config: '%smlp.kind' (moe)", w.c_str());
            L.has_mlp = true; L.ff_kind = FF_MOE_GLU;
            const Json *ex = rd.need(*mlp, "expert", w + "mlp."), *ro = rd.need(*mlp, "router", w + "mlp."), *sh = mlp->get("shared");
            if (ex) { L.expert_ff = rd.integer(*ex, "ff", w + "mlp.expert."); L.limit = rd.num(*ex, "limit", w + "mlp.expert."); }
            if (ro) { L.experts = rd.integer(*ro, "experts", w + "mlp.router."); L.top = rd.integer(*ro, "top", w + "mlp.router."); }
            if (sh && !sh->is_null()) { L.shared_ff = rd.integer(*sh, "ff", w + "mlp.shared."); L.shared_limit = rd.num(*sh, "limit", w + "mlp.shared."); }
            if (rd.err.empty() && (L.expert_ff < 1 || L.experts < 1 || L.top < 1 || L.top > L.experts || L.shared_ff < 0))
                return fail(NVR_ERR_INVALID_ARG, "config: %smlp needs positive expert sizes and 1 <= top <= experts", w.c_str());
        }
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (L.heads < 1 || L.dim < 1 || L.vdim < 1 || L.kv_heads < 1 || L.heads % L.kv_heads)
            return fail(NVR_ERR_INVALID_ARG, "config: %s %ld heads over %ld groups of %ld / %ld", w.c_str(), (long)L.heads, (long)L.kv_heads, (long)L.dim, (long)L.vdim);
        s->layers.push_back(L);
    }
    const int64_t n = (int64_t)s->layers.size();
    const Json *loop = c.get("loop");
    if (loop && !loop->is_null()) {
        const int64_t a = rd.integer(*loop, "start", "loop."), b = rd.integer(*loop, "stop", "loop."), t = rd.integer(*loop, "times", "loop.");
        if (!rd.err.empty()) return fail(NVR_ERR_INVALID_ARG, "%s", rd.err.c_str());
        if (a < 0 || b < a || b > n || t < 1) return fail(NVR_ERR_INVALID_ARG, "config: loop [%ld, %ld) x %ld over %ld layers", (long)a, (long)b, (long)t, (long)n);
        s->has_loop = true;
        for (int64_t i = 0; i < a; ++i) { s->runs.push_back((int)i); s->pass_start.push_back(0); }
        for (int64_t k = 0; k < t; ++k) for (int64_t i = a; i < b; ++i) { s->runs.push_back((int)i); s->pass_start.push_back(i == a ? 1 : 0); }
        for (int64_t i = b; i < n; ++i) { s->runs.push_back((int)i); s->pass_start.push_back(0); }
    } else
        for (int64_t i = 0; i < n; ++i) { s->runs.push_back((int)i); s->pass_start.push_back(0); }
    return NVR_OK;
}

}  // namespace nvr

extern "C" {

size_t nvr_model_registry_size(void) { return sizeof(nvr::kRegistry) / sizeof(nvr::kRegistry[0]); }
const char *nvr_model_registry_name(size_t i) { return i < nvr_model_registry_size() ? nvr::kRegistry[i].name : nullptr; }

nvr_model_spec_t *nvr_model_spec_from_json(const char *text) {
    try {
        if (!text) { nvr::fail(NVR_ERR_INVALID_ARG, "config: no text"); return nullptr; }
        nvr::Json c; std::string err;
        if (!nvr::Json::parse(text, &c, &err)) { nvr::fail(NVR_ERR_INVALID_ARG, "config: %s", err.c_str()); return nullptr; }
        std::string arch;
        if (const nvr::Json *a = c.get("architecture")) { if (a->kind == nvr::Json::Str) arch = a->str; }
        if (arch.empty())
            if (const nvr::Json *a = c.get("architectures")) if (a->kind == nvr::Json::Arr && !a->arr.empty() && a->arr[0].kind == nvr::Json::Str) arch = a->arr[0].str;
        if (arch.empty()) { nvr::fail(NVR_ERR_INVALID_ARG, "config: no 'architecture' (or 'architectures') entry"); return nullptr; }
        for (const auto &e : nvr::kRegistry)
            if (arch == e.name) {
                std::unique_ptr<nvr_model_spec> sp(new nvr_model_spec());
                sp->arch = arch;
                if (e.parse(c, sp.get()) != NVR_OK) return nullptr;
                return sp.release();
            }
        nvr::fail(NVR_ERR_UNSUPPORTED, "config: architecture '%s' is not registered", arch.c_str());
        return nullptr;
    } catch (...) { nvr::fail(NVR_ERR_INVARIANT, "config: out of memory"); return nullptr; }
}
void nvr_model_spec_destroy(nvr_model_spec_t *s) { delete s; }
const char *nvr_model_spec_architecture(const nvr_model_spec_t *s) { return s->arch.c_str(); }
int32_t nvr_model_spec_family(const nvr_model_spec_t *s) { return s->family; }
int nvr_model_spec_dense(const nvr_model_spec_t *s, nvr_model_config *out) {
    if (s->family != 0) return nvr::fail(NVR_ERR_INVALID_ARG, "architecture '%s' is not a dense graph", s->arch.c_str());
    *out = s->dense;
    return NVR_OK;
}
uint64_t nvr_model_spec_vocab(const nvr_model_spec_t *s) { return s->family == 0 ? s->dense.vocab_size : (uint64_t)s->layered.vocab; }
uint64_t nvr_model_spec_num_layer_runs(const nvr_model_spec_t *s) { return s->family == 0 ? s->dense.num_hidden_layers : (uint64_t)s->layered.runs.size(); }

}  // extern "C"
