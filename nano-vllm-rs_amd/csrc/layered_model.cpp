// layered_model.cpp — see layered_model.h.
#include "layered_model.h"
#include <algorithm>
#include <cmath>
#include <cstring>
#include "common.h"
#include "model_runner.h"
#include "kernels/kernels.h"

#define RC(expr) do { int _rc = (expr); if (_rc) return _rc; } while (0)

namespace nvr {

namespace {
template <class T> int dmalloc(T **p, size_t bytes) {
    NVR_HIP_CHECK(hipMalloc((void **)p, bytes ? bytes : 16));
    return NVR_OK;
}
inline float bf16_to_f(uint16_t b) { uint32_t u = (uint32_t)b << 16; float f; std::memcpy(&f, &u, 4); return f; }
inline uint16_t f_to_bf16(float f) {
    uint32_t u; std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
inline float f16_to_f(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000) << 16, exp = (h >> 10) & 0x1f, man = h & 0x3ff;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) u = sign;
        else { int e = -1; uint32_t m = man; do { ++e; m <<= 1; } while (!(m & 0x400)); u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3ff) << 13); }
    } else if (exp == 31) u = sign | 0x7f800000u | (man << 13);
    else u = sign | ((exp + 112) << 23) | (man << 13);
    float f; std::memcpy(&f, &u, 4); return f;
}
inline float src_at(int dtype, const void *src, size_t i) {
    return dtype == 2 ? ((const float *)src)[i] : dtype == 1 ? bf16_to_f(((const uint16_t *)src)[i]) : f16_to_f(((const uint16_t *)src)[i]);
}
}  // namespace

LayeredModel::~LayeredModel() {
    for (auto &g : graphs) if (g.second) (void)hipGraphExecDestroy(g.second);
    for (auto &w : lw) for (void *p : {w.mix, w.gu, w.out, (void *)w.canon1, (void *)w.canon2, (void *)w.r1, (void *)w.r2, (void *)w.sink, (void *)w.decay, (void *)w.freq, (void *)w.sin_t, (void *)w.pen})
        if (p) (void)hipFree(p);
    for (auto &s : rs) for (void *p : {s.kc, s.vc, (void *)s.state, (void *)s.hist}) if (p && !s.borrowed) (void)hipFree(p);
    if (attn_ws) (void)hipFree(attn_ws);
    for (void *p : {embed, head, (void *)x, (void *)proj, (void *)gu, (void *)tmp, (void *)ret_o, a1, a2, cat, xsel, (void *)in_dev}) if (p) (void)hipFree(p);
    if (in_host) (void)hipHostFree(in_host);
    for (void *p : owned) if (p) (void)hipFree(p);
}


int LayeredModel::init(nvr_model_runner &r) {
    r.env = nvr::Env::read();
    if (r.cfg.tensor_parallel_size != 1) return fail(NVR_ERR_UNSUPPORTED, "layer-list models run on one GPU (tensor_parallel_size 1)");
    r.bf16 = std::strcmp(r.cfg.dtype, "bfloat16") == 0; r.f32 = std::strcmp(r.cfg.dtype, "float32") == 0;
    if (!r.bf16 && !r.f32) return fail(NVR_ERR_UNSUPPORTED, "layer-list models: dtype '%s' (bfloat16 or float32)", r.cfg.dtype);
    bf16 = r.bf16; esz = bf16 ? 2 : 4; r.em = bf16 ? 1 : 2;
    r.tp = 1; r.rank = 0; r.tiled_weights = false; r.lm_fused = false;
    const int64_t W = spec.width, V = spec.vocab;
    r.Hd = W; r.V = r.Vl = V; r.vocab_start = 0; r.L = (int64_t)spec.runs.size();
    r.block_size = (int64_t)r.cfg.kvcache_block_size; r.max_tokens = (int64_t)r.cfg.max_num_batched_tokens; r.max_seqs = (int64_t)r.cfg.max_num_seqs;
    r.max_pos = std::max<int64_t>((int64_t)r.cfg.max_model_len, 1);
    if (spec.max_positions > 0) r.max_pos = std::min(r.max_pos, spec.max_positions);     // (learned positions: the table ends there)
    r.max_blocks_per_seq = (r.max_pos + r.block_size - 1) / r.block_size + 1;
    slots = r.cfg.num_state_slots ? (int64_t)r.cfg.num_state_slots : r.max_seqs;
    slot_par.assign((size_t)slots, 0);
    r.device = r.cfg.device_ordinal;
    NVR_HIP_CHECK(hipSetDevice(r.device));
    NVR_HIP_CHECK(hipStreamCreateWithFlags(&r.stream, hipStreamNonBlocking));
    RC(kl::prepare()); RC(kl::prepare_blocks());
    if (r.f32) RC(nvr::kf::prepare());
    else { RC(nvr::kb::linear_stream_prepare()); RC(nvr::kb::gemm_tiled_prepare()); }
    { int v = 0; if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, r.device) == hipSuccess && v > 0) r.num_cus = v; }

    if (spec.layout == LayeredSpec::SEQUENTIAL) RC(init_sequential(r));
    else if (spec.layout == LayeredSpec::SCALED) RC(init_scaled(r));
    else if (spec.layout == LayeredSpec::JOINT) RC(init_joint(r));
    else {
    // weights (zero until loaded)
    const int64_t taps = spec.taps;
    int64_t max_nmix = 0, max_ff = 0, max_kcat = 0, max_hv = 0;
    lw.resize(spec.layers.size());
    for (size_t i = 0; i < spec.layers.size(); ++i) {
        const LayeredSpec::Layer &L = spec.layers[i]; LayerW &w = lw[i];
        const int64_t qn = L.heads * L.dim, kn = L.kv_heads * L.dim, vn = L.kv_heads * L.vdim, hv = L.heads * L.vdim;
        w.qcol = 0; w.kcol = qn; w.vcol = qn + kn; w.gcol = qn + kn + vn;
        w.nmix = qn + kn + vn + (L.mixer == LayeredSpec::RETENTION ? hv : 0);
        w.mixcols = hv; w.kcat = hv + (L.has_mlp ? L.ff : 0);
        RC(dmalloc(&w.mix, (size_t)(w.nmix * W * esz))); NVR_HIP_CHECK(hipMemset(w.mix, 0, (size_t)(w.nmix * W * esz)));
        RC(dmalloc(&w.out, (size_t)(W * w.kcat * esz))); NVR_HIP_CHECK(hipMemset(w.out, 0, (size_t)(W * w.kcat * esz)));
        if (L.has_mlp) { RC(dmalloc(&w.gu, (size_t)(2 * L.ff * W * esz))); NVR_HIP_CHECK(hipMemset(w.gu, 0, (size_t)(2 * L.ff * W * esz))); }
        RC(dmalloc(&w.canon1, (size_t)(W * taps * 4))); NVR_HIP_CHECK(hipMemset(w.canon1, 0, (size_t)(W * taps * 4)));
        RC(dmalloc(&w.canon2, (size_t)(W * taps * 4))); NVR_HIP_CHECK(hipMemset(w.canon2, 0, (size_t)(W * taps * 4)));
        if (L.mixer == LayeredSpec::ATTENTION) {
            if (std::find(attn_groups.begin(), attn_groups.end(), L.heads / L.kv_heads) == attn_groups.end()) attn_groups.push_back(L.heads / L.kv_heads);
            w.flash = bf16 && L.dim == L.vdim && nvr::kb::flash_prefill_ok((int)L.dim, (int)L.heads, (int)L.kv_heads) && w.nmix % 8 == 0 && w.kcat % 4 == 0;
            if (w.flash && std::find(flash_groups.begin(), flash_groups.end(), L.heads / L.kv_heads) == flash_groups.end()) flash_groups.push_back(L.heads / L.kv_heads);
            for (float **p : {&w.r1, &w.r2, &w.sink}) { RC(dmalloc(p, (size_t)L.heads * 4)); NVR_HIP_CHECK(hipMemset(*p, 0, (size_t)L.heads * 4)); }
        } else {
            std::vector<float> d(L.heads);
            for (int64_t h = 0; h < L.heads; ++h) d[(size_t)h] = (float)L.decay[(size_t)h];
            RC(dmalloc(&w.decay, d.size() * 4)); NVR_HIP_CHECK(hipMemcpy(w.decay, d.data(), d.size() * 4, hipMemcpyHostToDevice));
            // rotation table: the angle is the f32 product of the position and the f32 frequency; its cosine and sine are rounded once from f64
            const int64_t half = L.rot_dims / 2;
            std::vector<float> cs((size_t)std::max<int64_t>(r.max_pos * half, 1)), sn(cs.size());
            for (int64_t j = 0; j < half; ++j) {
                const float f = (float)std::pow(L.rot_base, -2.0 * (double)j / (double)L.rot_dims);
                for (int64_t p = 0; p < r.max_pos; ++p) {
                    const float ang = (float)p * f;
                    cs[(size_t)(p * half + j)] = (float)std::cos((double)ang); sn[(size_t)(p * half + j)] = (float)std::sin((double)ang);
                }
            }
            RC(dmalloc(&w.freq, cs.size() * 4)); NVR_HIP_CHECK(hipMemcpy(w.freq, cs.data(), cs.size() * 4, hipMemcpyHostToDevice));
            RC(dmalloc(&w.sin_t, sn.size() * 4)); NVR_HIP_CHECK(hipMemcpy(w.sin_t, sn.data(), sn.size() * 4, hipMemcpyHostToDevice));
        }
        max_nmix = std::max(max_nmix, w.nmix); max_kcat = std::max(max_kcat, w.kcat); max_hv = std::max(max_hv, hv);
        if (L.has_mlp) max_ff = std::max(max_ff, L.ff);
    }
    RC(dmalloc(&embed, (size_t)(V * W * esz))); NVR_HIP_CHECK(hipMemset(embed, 0, (size_t)(V * W * esz)));
    RC(dmalloc(&head, (size_t)(V * W * esz))); NVR_HIP_CHECK(hipMemset(head, 0, (size_t)(V * W * esz)));

    // K/V pages and per-sequence state, one set per layer RUN (a looped layer keeps a cache / state per pass)
    size_t block_bytes = 0;
    for (int li : spec.runs) {
        const LayeredSpec::Layer &L = spec.layers[(size_t)li];
        if (L.mixer == LayeredSpec::ATTENTION) block_bytes += (size_t)(r.block_size * L.kv_heads * (L.dim + L.vdim) * esz);
    }
    if (r.cfg.num_kvcache_blocks >= 0) r.num_blocks = r.cfg.num_kvcache_blocks;
    else if (r.cfg.num_kvcache_blocks == -1) r.num_blocks = 1000;
    else {
        size_t free_b = 0, total_b = 0;
        NVR_HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        const double budget = (double)free_b - (1.0 - r.cfg.gpu_memory_utilization) * (double)total_b;
        const int64_t nb = block_bytes ? (int64_t)(budget * 0.9 / (double)block_bytes) : 1000;
        if (nb < 1) return fail(NVR_ERR_HIP, "not enough free HBM for one KV block");
        r.num_blocks = nb;
    }
    rs.resize(spec.runs.size());
    for (size_t ri = 0; ri < spec.runs.size(); ++ri) {
        const LayeredSpec::Layer &L = spec.layers[(size_t)spec.runs[ri]]; RunState &s = rs[ri];
        if (L.mixer == LayeredSpec::ATTENTION) {
            const size_t kb = (size_t)(r.num_blocks * r.block_size * L.kv_heads * L.dim * esz), vb = (size_t)(r.num_blocks * r.block_size * L.kv_heads * L.vdim * esz);
            RC(dmalloc(&s.kc, kb)); NVR_HIP_CHECK(hipMemset(s.kc, 0, kb));
            RC(dmalloc(&s.vc, vb)); NVR_HIP_CHECK(hipMemset(s.vc, 0, vb));
        } else {
            const size_t sb = (size_t)(slots * L.heads * L.dim * L.vdim * 4);
            RC(dmalloc(&s.state, sb)); NVR_HIP_CHECK(hipMemset(s.state, 0, sb));
        }
        const size_t hb = (size_t)(2 * slots * (taps - 1) * W * 4);
        RC(dmalloc(&s.hist, hb)); NVR_HIP_CHECK(hipMemset(s.hist, 0, hb ? hb : 16));
    }

    // activations
    const int64_t MT = r.max_tokens;
    RC(dmalloc(&x, (size_t)(MT * W * 4))); RC(dmalloc(&tmp, (size_t)(MT * W * esz)));
    RC(dmalloc(&proj, (size_t)(MT * max_nmix * esz))); RC(dmalloc(&gu, (size_t)(MT * 2 * max_ff * esz))); RC(dmalloc(&ret_o, (size_t)(MT * max_hv * 4)));
    RC(dmalloc(&a1, (size_t)(MT * W * esz))); RC(dmalloc(&a2, (size_t)(MT * W * esz))); RC(dmalloc(&cat, (size_t)(MT * max_kcat * esz)));
    }
    const int64_t MT = r.max_tokens;
    logit_rows_cap = std::max<int64_t>(r.max_seqs, 64);
    RC(dmalloc(&xsel, (size_t)(std::max(MT, logit_rows_cap) * W * esz)));
    RC(dmalloc(&r.logits, (size_t)(logit_rows_cap * V * 4)));

    // step inputs: ids | row_seq | want | cu | start | slot | par | block tables
    in_bytes = (size_t)(MT * 8 + MT * 4 * 2 + (r.max_seqs + 1) * 4 + r.max_seqs * 4 * 3 + r.max_seqs * r.max_blocks_per_seq * 4 + 256) +
               (attn_groups.size() + 2 * flash_groups.size()) * (size_t)((MT + r.max_seqs) * sizeof(kl::AttnTile) + 16);
    attn_ws_bytes = kl::sink_attention_workspace_bytes(4 * r.num_cus);
    NVR_HIP_CHECK(hipMalloc(&attn_ws, attn_ws_bytes));
    NVR_HIP_CHECK(hipHostMalloc((void **)&in_host, in_bytes, hipHostMallocDefault));
    NVR_HIP_CHECK(hipMalloc((void **)&in_dev, in_bytes));

    // sampling (Sampler::sample, sampler.rs:71-218: the runner's own samplers read r.logits)
    NVR_HIP_CHECK(hipMalloc((void **)&r.d_tok, (size_t)r.max_seqs * 8)); NVR_HIP_CHECK(hipMalloc((void **)&r.d_maxval, (size_t)r.max_seqs * 4));
    NVR_HIP_CHECK(hipHostMalloc((void **)&r.h_tok, (size_t)r.max_seqs * 8, hipHostMallocDefault));
    NVR_HIP_CHECK(hipMalloc((void **)&r.d_temp, (size_t)r.max_seqs * 4)); NVR_HIP_CHECK(hipMalloc((void **)&r.d_topk, (size_t)r.max_seqs * 8));
    NVR_HIP_CHECK(hipMalloc((void **)&r.d_topp, (size_t)r.max_seqs * 4)); NVR_HIP_CHECK(hipMalloc((void **)&r.d_keys, (size_t)r.max_seqs * 8));
    NVR_HIP_CHECK(hipHostMalloc((void **)&r.samp_host, (size_t)r.max_seqs * 24, hipHostMallocDefault));
    NVR_HIP_CHECK(hipMalloc(&r.sample_ws, nvr::kb::sample_workspace_bytes(r.max_seqs, V)));
    NVR_HIP_CHECK(hipDeviceSynchronize());
    return NVR_OK;
}

// src [rows][cols] (row-major, dtype 0 f16 / 1 bf16 / 2 f32) -> dst rows of dst_ld elements: the operand type, or f32
int LayeredModel::put(nvr_model_runner &r, void *dst, int64_t dst_ld, int64_t rows, int64_t cols, int dtype, const void *src, bool as_operand) {
    const size_t n = (size_t)(rows * cols);
    const int64_t e = (as_operand && bf16) ? 2 : 4;
    std::vector<char> buf(n * (size_t)e);
    if (e == 2) {
        uint16_t *o = (uint16_t *)buf.data();
        if (dtype == 1) std::memcpy(o, src, n * 2);
        else for (size_t i = 0; i < n; ++i) o[i] = f_to_bf16(src_at(dtype, src, i));
    } else {
        float *o = (float *)buf.data();
        for (size_t i = 0; i < n; ++i) o[i] = src_at(dtype, src, i);
    }
    NVR_HIP_CHECK(hipSetDevice(r.device));
    NVR_HIP_CHECK(hipMemcpy2D(dst, (size_t)(dst_ld * e), buf.data(), (size_t)(cols * e), (size_t)(cols * e), (size_t)rows, hipMemcpyHostToDevice));
    return NVR_OK;
}

// Tensors by the names of the checkpoint: "embed", "head", "final.norm", and per layer i "l<i>.norm1" / "norm2" (one number each), "l<i>.canon1" / "canon2"
// [width][taps], "l<i>.mix.{q,k,v,g,o}" (+ "r1", "r2", "sink" per head for attention), "l<i>.mlp.{gate,up,down}".  Linear weights are [out][in].
int LayeredModel::load_tensor(nvr_model_runner &r, const char *name_in, int dtype, const int64_t *shape, int ndim, const void *data) {
    if (dtype < 0 || dtype > 2) return fail(NVR_ERR_INVALID_ARG, "load_tensor: dtype %d", dtype);
    const std::string name(name_in);
    if (spec.layout == LayeredSpec::SEQUENTIAL) return load_sequential(r, name, dtype, shape, ndim, data);
    if (spec.layout == LayeredSpec::SCALED) return load_scaled(r, name, dtype, shape, ndim, data);
    if (spec.layout == LayeredSpec::JOINT) return load_joint(r, name, dtype, shape, ndim, data);
    const int64_t W = spec.width, V = spec.vocab;
    auto is2 = [&](int64_t a, int64_t b) { return ndim == 2 && shape[0] == a && shape[1] == b; };
    auto bad = [&]() { return fail(NVR_ERR_LEN_MISMATCH, "load_tensor: '%s' has the wrong shape", name_in); };
    auto scalar = [&](float *out) { int64_t n = 1; for (int i = 0; i < ndim; ++i) n *= shape[i]; if (n != 1) return bad(); *out = src_at(dtype, data, 0); return (int)NVR_OK; };
    if (name == "embed") return is2(V, W) ? put(r, embed, W, V, W, dtype, data, true) : bad();
    if (name == "head") return is2(V, W) ? put(r, head, W, V, W, dtype, data, true) : bad();
    if (name == "final.norm") return scalar(&gfinal);
    if (name.size() < 3 || name[0] != 'l') return fail(NVR_ERR_UNSUPPORTED, "load_tensor: unknown tensor '%s'", name_in);
    size_t dot = name.find('.');
    if (dot == std::string::npos || dot < 2) return fail(NVR_ERR_UNSUPPORTED, "load_tensor: unknown tensor '%s'", name_in);
    int64_t li = 0;
    for (size_t i = 1; i < dot; ++i) { if (name[i] < '0' || name[i] > '9') return fail(NVR_ERR_UNSUPPORTED, "load_tensor: unknown tensor '%s'", name_in); li = li * 10 + (name[i] - '0'); }
    if (li >= (int64_t)spec.layers.size()) return fail(NVR_ERR_UNSUPPORTED, "load_tensor: '%s' names a layer the model does not have", name_in);
    const LayeredSpec::Layer &L = spec.layers[(size_t)li]; LayerW &w = lw[(size_t)li];
    const std::string rest = name.substr(dot + 1);
    const int64_t qn = L.heads * L.dim, kn = L.kv_heads * L.dim, vn = L.kv_heads * L.vdim, hv = L.heads * L.vdim;
    auto rows_at = [&](void *base, int64_t row0, int64_t ld) { return (void *)((char *)base + (size_t)(row0 * ld * esz)); };
    auto vec = [&](float *dst, int64_t n) { return (ndim == 1 && shape[0] == n) ? put(r, dst, n, 1, n, dtype, data, false) : bad(); };
    if (rest == "norm1") return scalar(&w.g1);
    if (rest == "norm2") return scalar(&w.g2);
    if (rest == "canon1") return is2(W, spec.taps) ? put(r, w.canon1, spec.taps, W, spec.taps, dtype, data, false) : bad();
    if (rest == "canon2") return is2(W, spec.taps) ? put(r, w.canon2, spec.taps, W, spec.taps, dtype, data, false) : bad();
    if (rest == "mix.q") return is2(qn, W) ? put(r, rows_at(w.mix, w.qcol, W), W, qn, W, dtype, data, true) : bad();
    if (rest == "mix.k") return is2(kn, W) ? put(r, rows_at(w.mix, w.kcol, W), W, kn, W, dtype, data, true) : bad();
    if (rest == "mix.v") return is2(vn, W) ? put(r, rows_at(w.mix, w.vcol, W), W, vn, W, dtype, data, true) : bad();
    if (rest == "mix.o") return is2(W, hv) ? put(r, w.out, w.kcat, W, hv, dtype, data, true) : bad();
    if (L.mixer == LayeredSpec::RETENTION && rest == "mix.g") return is2(hv, W) ? put(r, rows_at(w.mix, w.gcol, W), W, hv, W, dtype, data, true) : bad();
    if (L.mixer == LayeredSpec::ATTENTION) {
        if (rest == "mix.r1") { w.pen_dirty = true; return vec(w.r1, L.heads); }
        if (rest == "mix.r2") { w.pen_dirty = true; return vec(w.r2, L.heads); }
        if (rest == "mix.sink") return vec(w.sink, L.heads);
    }
    if (L.has_mlp) {
        if (rest == "mlp.gate") return is2(L.ff, W) ? put(r, w.gu, W, L.ff, W, dtype, data, true) : bad();
        if (rest == "mlp.up") return is2(L.ff, W) ? put(r, rows_at(w.gu, L.ff, W), W, L.ff, W, dtype, data, true) : bad();
        if (rest == "mlp.down") return is2(W, L.ff) ? put(r, (char *)w.out + (size_t)(hv * esz), w.kcat, W, L.ff, dtype, data, true) : bad();
    }
    return fail(NVR_ERR_UNSUPPORTED, "load_tensor: unknown tensor '%s'", name_in);
}

// y = a . w^T in the operand type (bf16: f32 accumulation on the matrix cores, one rounding at the store; the dense graph's GEMM routing), or, for the
// logits, in f32
int LayeredModel::gemm(nvr_model_runner &r, const void *a, int64_t lda, const void *w, int64_t T, int64_t K, int64_t N, void *y, bool y_f32) {
    if (!bf16) return nvr::kf::linear((const float *)a, lda, (const float *)w, T, K, N, nullptr, (float *)y, r.stream);
    if (K % 32 == 0 && N % 16 == 0 && lda % 8 == 0) return nvr::kb::linear((const uint16_t *)a, lda, (const uint16_t *)w, T, K, N, y, y_f32, r.stream);
    return kl::gemm_any(a, lda, w, T, K, N, y, y_f32, true, r.stream);
}

// One step over a batch of chunks: sequence i contributes its tokens [chunk_start, chunk_start + chunk_len).  want: rows of the step (in batch
// order) whose logits are produced, or null for the last row of every sequence.
int LayeredModel::execute(nvr_model_runner &r, nvr_seq *const *seqs, size_t nseq, const int32_t *want, size_t nwant) {
    NVR_HIP_CHECK(hipSetDevice(r.device));
    if (nseq == 0) return fail(NVR_ERR_INVALID_ARG, "execute_model: empty batch");
    if ((int64_t)nseq > r.max_seqs) return fail(NVR_ERR_INVALID_ARG, "execute_model: %zu sequences exceed max_num_seqs %ld", nseq, (long)r.max_seqs);
    int64_t T = 0, max_ctx = 0, max_rows = 0;
    for (size_t i = 0; i < nseq; ++i) {
        const nvr_seq *s = seqs[i];
        if (s->chunk_len == 0 || s->chunk_start + s->chunk_len > s->num_tokens)
            return fail(NVR_ERR_INVALID_ARG, "execute_model: sequence %lu has no valid chunk (%zu + %zu of %zu tokens)", (unsigned long)s->seq_id, s->chunk_start, s->chunk_len, s->num_tokens);
        if (s->state_slot < 0 || s->state_slot >= slots) return fail(NVR_ERR_NOT_ALLOCATED, "execute_model: sequence %lu holds no state slot", (unsigned long)s->seq_id);
        const int64_t end = (int64_t)(s->chunk_start + s->chunk_len);
        if (end > r.max_pos) return fail(NVR_ERR_INVALID_ARG, "execute_model: sequence %lu reaches position %ld (max_model_len %ld)", (unsigned long)s->seq_id, (long)end, (long)r.max_pos);
        if ((int64_t)s->block_table.size() * r.block_size < end) return fail(NVR_ERR_NOT_ALLOCATED, "execute_model: sequence %lu has blocks for %zu tokens, needs %ld", (unsigned long)s->seq_id, s->block_table.size() * (size_t)r.block_size, (long)end);
        for (size_t j = 0; j < nseq; ++j) if (j != i && seqs[j]->state_slot == s->state_slot) return fail(NVR_ERR_INVARIANT, "execute_model: two sequences of the batch share state slot %d", s->state_slot);
        T += (int64_t)s->chunk_len; max_ctx = std::max(max_ctx, end); max_rows = std::max<int64_t>(max_rows, (int64_t)s->chunk_len);
    }
    if (T > r.max_tokens) return fail(NVR_ERR_INVALID_ARG, "execute_model: %ld tokens exceed max_num_batched_tokens %ld", (long)T, (long)r.max_tokens);
    const size_t R = want ? nwant : nseq;
    if ((int64_t)R > std::max(r.max_tokens, logit_rows_cap)) return fail(NVR_ERR_INVALID_ARG, "execute_model: %zu rows of logits asked of a step of %ld tokens", R, (long)T);
    if ((int64_t)R > logit_rows_cap) {                                   // (grown outside any capture: an allocation synchronises)
        NVR_HIP_CHECK(hipStreamSynchronize(r.stream));
        (void)hipFree(r.logits); r.logits = nullptr;
        for (auto &g : graphs) if (g.second) (void)hipGraphExecDestroy(g.second);   // (they hold the old address)
        graphs.clear();
        logit_rows_cap = (int64_t)R;
        NVR_HIP_CHECK(hipMalloc((void **)&r.logits, (size_t)(logit_rows_cap * spec.vocab * 4)));
    }
    // arena
    const int64_t MB = r.max_blocks_per_seq;
    size_t off = 0;
    auto carve = [&](size_t bytes) { size_t o = off; off += (bytes + 15) / 16 * 16; return o; };
    const size_t o_ids = carve((size_t)T * 8), o_rs = carve((size_t)T * 4), o_want = carve(std::max<size_t>(R, 1) * 4), o_cu = carve((nseq + 1) * 4), o_st = carve(nseq * 4),
                 o_sl = carve(nseq * 4), o_par = carve(nseq * 4), o_bt = carve(nseq * (size_t)MB * 4);
    // query tiles of the matrix-core attention, one list per distinct group size g = H / G: 64 / g positions of one sequence each
    std::vector<size_t> o_tiles(attn_groups.size()); std::vector<int32_t> n_tiles(attn_groups.size(), 0);
    for (size_t gi = 0; gi < attn_groups.size(); ++gi) {
        const int64_t pw = std::max<int64_t>(1, 64 / attn_groups[gi]);
        size_t cnt = 0;
        for (size_t i = 0; i < nseq; ++i) cnt += (seqs[i]->chunk_len + (size_t)pw - 1) / (size_t)pw;
        o_tiles[gi] = carve(cnt * sizeof(kl::AttnTile)); n_tiles[gi] = (int32_t)cnt;
    }
    std::vector<size_t> o_ftiles(flash_groups.size()); std::vector<int32_t> n_ftiles(flash_groups.size(), 0);
    for (size_t gi = 0; gi < flash_groups.size(); ++gi) {
        const int64_t pw = nvr::kb::flash_tile_positions((int)flash_groups[gi], 1);
        size_t cnt = 0;
        for (size_t i = 0; i < nseq; ++i) cnt += (seqs[i]->chunk_len + (size_t)pw - 1) / (size_t)pw;
        o_ftiles[gi] = carve(cnt * sizeof(nvr::kt::FlashTile)); n_ftiles[gi] = (int32_t)cnt;
    }
    if (off > in_bytes) return fail(NVR_ERR_INVARIANT, "execute_model: step inputs of %zu bytes exceed the arena", off);
    for (size_t gi = 0; gi < flash_groups.size(); ++gi) {
        const int64_t pw = nvr::kb::flash_tile_positions((int)flash_groups[gi], 1);
        nvr::kt::FlashTile *tl = (nvr::kt::FlashTile *)(in_host + o_ftiles[gi]);
        int64_t row = 0;
        for (size_t i = 0; i < nseq; ++i) {
            for (int64_t r0 = 0; r0 < (int64_t)seqs[i]->chunk_len; r0 += pw)
                *tl++ = nvr::kt::FlashTile{(int32_t)(row + r0), (int32_t)std::min<int64_t>(pw, (int64_t)seqs[i]->chunk_len - r0), (int32_t)((int64_t)seqs[i]->chunk_start + r0), flash_contiguous ? (int32_t)row : (int32_t)i};
            row += (int64_t)seqs[i]->chunk_len;
        }
    }
    for (size_t gi = 0; gi < attn_groups.size(); ++gi) {
        const int64_t pw = std::max<int64_t>(1, 64 / attn_groups[gi]);
        kl::AttnTile *tl = (kl::AttnTile *)(in_host + o_tiles[gi]);
        for (size_t i = 0; i < nseq; ++i)
            for (int64_t r0 = 0; r0 < (int64_t)seqs[i]->chunk_len; r0 += pw) *tl++ = kl::AttnTile{(int32_t)i, (int32_t)r0};
    }
    int64_t *ids = (int64_t *)(in_host + o_ids); int32_t *rowseq = (int32_t *)(in_host + o_rs), *wnt = (int32_t *)(in_host + o_want), *cu = (int32_t *)(in_host + o_cu),
            *stt = (int32_t *)(in_host + o_st), *sl = (int32_t *)(in_host + o_sl), *par = (int32_t *)(in_host + o_par), *bt = (int32_t *)(in_host + o_bt);
    int64_t t = 0;
    for (size_t i = 0; i < nseq; ++i) {
        const nvr_seq *s = seqs[i];
        cu[i] = (int32_t)t; stt[i] = (int32_t)s->chunk_start; sl[i] = s->state_slot;
        if (s->chunk_start == 0) slot_par[(size_t)s->state_slot] = 0;     // a sequence's first tokens read no history: whatever the slot held is dead
        par[i] = slot_par[(size_t)s->state_slot];
        for (size_t j = 0; j < s->chunk_len; ++j, ++t) {
            const int64_t id = s->token_ids[s->chunk_start + j];
            if ((uint64_t)id >= (uint64_t)spec.vocab) return fail(NVR_ERR_INVALID_ARG, "execute_model: token id %ld outside the vocabulary [0, %ld)", (long)id, (long)spec.vocab);
            ids[t] = id; rowseq[t] = (int32_t)i;
        }
        for (int64_t j = 0; j < MB; ++j) bt[i * (size_t)MB + (size_t)j] = j < (int64_t)s->block_table.size() ? s->block_table[(size_t)j] : -1;
        if (!want) wnt[i] = (int32_t)t - 1;
    }
    cu[nseq] = (int32_t)t;
    if (want) for (size_t i = 0; i < R; ++i) { if (want[i] < 0 || want[i] >= T) return fail(NVR_ERR_INVALID_ARG, "execute_model: logits row %d of a step of %ld rows", want[i], (long)T); wnt[i] = want[i]; }
    NVR_HIP_CHECK(hipMemcpyAsync(in_dev, in_host, off, hipMemcpyHostToDevice, r.stream));
    kl::Batch b{};
    b.ids = (const int64_t *)(in_dev + o_ids); b.row_seq = (const int32_t *)(in_dev + o_rs); b.cu = (const int32_t *)(in_dev + o_cu);
    b.start = (const int32_t *)(in_dev + o_st); b.slot = (const int32_t *)(in_dev + o_sl); b.par = (const int32_t *)(in_dev + o_par);
    b.block_tables = (const int32_t *)(in_dev + o_bt); b.max_blocks = (int32_t)MB; b.block_size = (int32_t)r.block_size;
    b.T = (int32_t)T; b.B = (int32_t)nseq; b.max_ctx = (int32_t)max_ctx; b.max_rows = (int32_t)max_rows;
    const int32_t *d_want = (const int32_t *)(in_dev + o_want);

    bool decode_sized = true;
    for (size_t i = 0; i < nseq && decode_sized; ++i) decode_sized = seqs[i]->chunk_len == 1;
    StepPlan plan{b, d_want, (int64_t)R, T, max_ctx, o_tiles, n_tiles, o_ftiles, n_ftiles, decode_sized};
    plan.whole_prompts = !decode_sized;
    for (size_t i = 0; i < nseq && plan.whole_prompts; ++i) plan.whole_prompts = seqs[i]->chunk_start == 0;
    if (decode_sized && !r.cfg.enforce_eager) {
        const int64_t bucket = (max_ctx + 255) / 256 * 256;
        plan.max_ctx = plan.b.max_ctx = (int32_t)bucket;
        const uint64_t key = ((uint64_t)nseq << 40) | ((uint64_t)R << 20) | (uint64_t)(bucket / 256);
        auto it = graphs.find(key);
        if (it == graphs.end()) {
            if (graphs.size() >= (size_t)r.env.max_graphs) {
                NVR_HIP_CHECK(hipStreamSynchronize(r.stream));
                for (auto &g : graphs) if (g.second) (void)hipGraphExecDestroy(g.second);
                graphs.clear();
            }
            graphs.emplace(key, nullptr);                                  // seen once: this step runs eagerly
            RC(forward(r, plan));
        } else {
            if (!it->second) {
                hipGraph_t g = nullptr; hipGraphExec_t ge = nullptr;
                NVR_HIP_CHECK(hipStreamBeginCapture(r.stream, hipStreamCaptureModeThreadLocal));
                int rc = forward(r, plan);
                hipError_t e = hipStreamEndCapture(r.stream, &g);
                if (!rc && e != hipSuccess) rc = fail(NVR_ERR_HIP, "hipStreamEndCapture failed: %s", hipGetErrorString(e));
                if (!rc && hipGraphInstantiate(&ge, g, nullptr, nullptr, 0) != hipSuccess) rc = fail(NVR_ERR_HIP, "hipGraphInstantiate failed");
                if (g) (void)hipGraphDestroy(g);
                if (rc) return rc;
                it->second = ge;
            }
            NVR_HIP_CHECK(hipGraphLaunch(it->second, r.stream));
            ++graph_replays;
        }
    } else
        RC(forward(r, plan));
    for (size_t i = 0; i < nseq; ++i) slot_par[(size_t)seqs[i]->state_slot] ^= 1;
    r.last_rows = R; r.last_tokens = T;
    return NVR_OK;
}

int LayeredModel::forward(nvr_model_runner &r, const StepPlan &p) {
    if (spec.layout == LayeredSpec::SEQUENTIAL) return forward_sequential(r, p);
    if (spec.layout == LayeredSpec::SCALED) return forward_scaled(r, p);
    if (spec.layout == LayeredSpec::JOINT) return forward_joint(r, p);
    const kl::Batch &b = p.b;
    const int32_t *d_want = p.d_want;
    const int64_t T = p.T, R = p.R, max_ctx = p.max_ctx;
    const std::vector<size_t> &o_tiles = p.o_tiles; const std::vector<int32_t> &n_tiles = p.n_tiles;
    hipStream_t s = r.stream;
    const int64_t W = spec.width;
    const float eps = (float)spec.eps;
    RC(kl::embed_scale(embed, bf16, b.ids, T, W, (float)spec.embedding_scale, x, s));
    for (size_t ri = 0; ri < spec.runs.size(); ++ri) {
        const size_t li = (size_t)spec.runs[ri];
        const LayeredSpec::Layer &L = spec.layers[li]; const LayerW &w = lw[li]; RunState &st = rs[ri];
        RC(kl::norm_canon(x, b, W, eps, (int)spec.taps, w.g1, w.canon1, a1, w.g2, w.canon2, L.has_mlp ? a2 : nullptr, bf16, st.hist, slots, s));
        RC(gemm(r, a1, W, w.mix, T, W, w.nmix, proj));
        if (L.mixer == LayeredSpec::ATTENTION) {
            kl::SinkAttnArgs a{};
            a.q = (const char *)proj + (size_t)(w.qcol * esz); a.ldq = w.nmix; a.kc = st.kc; a.vc = st.vc; a.r1 = w.r1; a.r2 = w.r2; a.sink = w.sink;
            a.H = (int32_t)L.heads; a.G = (int32_t)L.kv_heads; a.D = (int32_t)L.dim; a.Dv = (int32_t)L.vdim; a.scale = (float)L.scale;
            a.out = cat; a.ldo = w.kcat;
            a.v_grouped = w.flash ? 0 : 1;                                          // (a property of the layer: the pages keep one layout)
            const bool tiled = kl::sink_attention_tiled_ok(a, bf16, (int)r.block_size);   // (a property of the layer's shape: the same answer every step)
            RC(kl::kv_store(proj, w.nmix, w.kcol, w.vcol, b, L.kv_heads, L.dim, L.vdim, st.kc, st.vc, bf16, tiled && !w.flash, s));
            if (w.flash && !p.decode_sized) {
                // prompts and portions: the dense graph's flash kernel in its penalty / sink form (K and V through the block tables, the step's own rows included)
                const size_t gi = (size_t)(std::find(flash_groups.begin(), flash_groups.end(), L.heads / L.kv_heads) - flash_groups.begin());
                nvr::kt::FlashArgs f{};
                f.q = (const uint16_t *)a.q; f.ldq = w.nmix; f.k = (const uint16_t *)st.kc; f.v = (const uint16_t *)st.vc; f.ldkv = 0;
                f.block_tables = b.block_tables; f.max_blocks = b.max_blocks; f.block_size = b.block_size;
                f.tiles = (const nvr::kt::FlashTile *)(in_dev + p.o_ftiles[gi]); f.ntiles = p.n_ftiles[gi];
                f.H = (int32_t)L.heads; f.KVH = (int32_t)L.kv_heads; f.D = (int32_t)L.dim; f.scale = (float)L.scale; f.out = (uint16_t *)cat;
                f.r1 = w.r1; f.r2 = w.r2; f.sink = w.sink; f.ldo = w.kcat;
                RC(nvr::kb::flash_prefill(f, true, s));
            } else if (tiled) {
                LayerW &wm = lw[li];
                if (!wm.pen || wm.pen_dirty) {                                      // the penalties by distance, once per set of r1 / r2
                    if (!wm.pen) RC(dmalloc(&wm.pen, (size_t)(L.heads * r.max_pos * 4)));
                    RC(kl::penalty_table(w.r1, w.r2, L.heads, r.max_pos, wm.pen, s));
                    wm.pen_dirty = false;
                }
                a.pen = wm.pen; a.pen_n = (int32_t)r.max_pos;
                const size_t gi = (size_t)(std::find(attn_groups.begin(), attn_groups.end(), L.heads / L.kv_heads) - attn_groups.begin());
                // decode-sized steps over long contexts: few tiles, many keys each — spread every tile's keys over several workgroups
                const int64_t wgs = (int64_t)n_tiles[gi] * L.kv_heads;
                int64_t nsplit = 1;
                if (wgs < r.num_cus && max_ctx >= 512) nsplit = std::max<int64_t>(1, std::min<int64_t>({(2 * r.num_cus) / wgs, (max_ctx + 255) / 256, 16}));
                RC(kl::sink_attention_tiled(a, b, (const kl::AttnTile *)(in_dev + o_tiles[gi]), n_tiles[gi], (int)nsplit, attn_ws, attn_ws_bytes, s));
            } else
                RC(kl::sink_attention(a, b, bf16, s));
        } else {
            kl::RetentionArgs a{};
            a.proj = proj; a.ld = w.nmix; a.qcol = w.qcol; a.kcol = w.kcol; a.vcol = w.vcol; a.decay = w.decay; a.cos_t = w.freq; a.sin_t = w.sin_t; a.rot_dims = (int32_t)L.rot_dims;
            a.az = nullptr; a.ldz = 0; a.abias = nullptr; a.inv_tau = 1.f; a.qscale = 1.f;
            a.kscale = 1.0f / std::sqrt((float)L.dim); a.H = (int32_t)L.heads; a.D = (int32_t)L.dim; a.Dv = (int32_t)L.vdim; a.state = st.state; a.o = ret_o;
            RC(kl::retention(a, b, bf16, s));
            RC(kl::head_norm_gate(ret_o, proj, w.nmix, w.gcol, T, L.heads, L.vdim, eps, nullptr, cat, w.kcat, bf16, s));
        }
        if (L.has_mlp) {
            RC(gemm(r, a2, W, w.gu, T, W, 2 * L.ff, gu));
            RC(kl::clamped_glu(gu, T, L.ff, (float)L.limit, 1.702f, (char *)cat + (size_t)(w.mixcols * esz), w.kcat, bf16, s));
        }
        RC(gemm(r, cat, w.kcat, w.out, T, w.kcat, W, tmp));
        RC(kl::axpy(x, tmp, bf16, (float)spec.residual_mult, T * W, s));
    }
    RC(kl::norm_rows(x, d_want, (int64_t)R, W, eps, gfinal, xsel, bf16, s));
    return gemm(r, xsel, W, head, (int64_t)R, W, spec.vocab, r.logits, true);
}

// ===================================================================================================================================================
// Sequential layout: x <- x + nb(mixer(n(x))); x <- x + nb(ff(n(x))); token input; weighted average over depth.

int LayeredModel::init_sequential(nvr_model_runner &r) {
    const int64_t W = spec.width, V = spec.vocab, MT = r.max_tokens, nL = (int64_t)spec.layers.size();
    auto named = [&](void **p, size_t bytes) {              // (the buffers the destructor frees by name)
        RC(dmalloc((char **)p, bytes));
        NVR_HIP_CHECK(hipMemset(*p, 0, bytes ? bytes : 16));
        return (int)NVR_OK;
    };
    lw.resize(spec.layers.size());
    int64_t max_kvx = 0, max_experts = 0, max_f = 0;
    int64_t max_nmix = 0, max_q2 = 0, max_qabs = 0, max_ctx = 0, max_hv = 0, max_qlat = 0, max_hd = 0, max_ff = 0, max_rows_e = 0, max_e2f = 0, max_ef = 0;
    size_t block_bytes = 0;
    for (size_t i = 0; i < spec.layers.size(); ++i) {
        const LayeredSpec::Layer &L = spec.layers[i]; LayerW &w = lw[i];
        const int64_t hv = L.heads * L.vdim, hd = L.heads * L.dim;
        for (float **p : {&w.n1, &w.n1b}) RC(own(p, (size_t)W * 4));
        if (L.has_mlp) for (float **p : {&w.n2, &w.n2b}) RC(own(p, (size_t)W * 4));
        if (L.mixer == LayeredSpec::LATENT) {
            const int64_t R = L.rot_dim, own_kv = L.kv_from < 0 ? L.kv_rank + R : 0;
            // mix rows: queries (or their latent), the output gate's rows, the cached row's source
            w.qcol = 0; const int64_t qn = L.q_rank ? L.q_rank : hd;
            w.gcol = qn; w.dcol = qn + (L.out_gate ? hv : 0); w.nmix = w.dcol + own_kv;
            if (L.q_rank) { RC(own(&w.uq, (size_t)(L.heads * (L.dim + R) * L.q_rank * esz))); RC(own(&w.dqn, (size_t)L.q_rank * 4)); max_q2 = std::max(max_q2, L.heads * (L.dim + R)); max_qlat = std::max(max_qlat, L.q_rank); }
            if (own_kv) { RC(own(&w.dkvn, (size_t)L.kv_rank * 4)); block_bytes += (size_t)(r.block_size * own_kv * esz); }
            RC(own(&w.ukt, (size_t)(L.heads * L.kv_rank * L.dim * esz))); RC(own(&w.uv, (size_t)(hv * L.kv_rank * esz)));
            std::vector<float> f((size_t)std::max<int64_t>(R / 2, 1));
            for (int64_t j = 0; j < R / 2; ++j) f[(size_t)j] = (float)std::pow(L.rot_base, -2.0 * (double)j / (double)L.rot_dims);
            RC(own(&w.rfreq, f.size() * 4)); NVR_HIP_CHECK(hipMemcpy(w.rfreq, f.data(), f.size() * 4, hipMemcpyHostToDevice));
            max_qabs = std::max(max_qabs, L.heads * (L.kv_rank + R)); max_ctx = std::max(max_ctx, L.heads * L.kv_rank);
            // whole prompts (every key is a row of the step): keys and values expanded by one product and the dense graph's flash kernel, one key/value head per query head
            w.flash = bf16 && L.dim + R == L.vdim && nvr::kb::flash_prefill_ok((int)L.vdim, (int)L.heads, (int)L.heads) && (L.kv_rank + R) % 32 == 0 && (2 * hv) % 16 == 0 &&
                      w.nmix % 8 == 0 && (L.heads * (L.dim + R)) % 8 == 0;
            if (w.flash) {
                RC(own(&w.wx, (size_t)(2 * hv * (L.kv_rank + R) * esz)));
                std::vector<uint16_t> one((size_t)1, f_to_bf16(1.0f));
                for (int64_t h = 0; h < L.heads; ++h)           // the shared rotated key part is copied into every head's keys by rows of the identity
                    for (int64_t j = 0; j < R; ++j)
                        NVR_HIP_CHECK(hipMemcpy((char *)w.wx + (size_t)(((h * L.vdim + L.dim + j) * (L.kv_rank + R) + L.kv_rank + j) * esz), one.data(), 2, hipMemcpyHostToDevice));
                if (std::find(flash_groups.begin(), flash_groups.end(), (int64_t)1) == flash_groups.end()) flash_groups.push_back(1);
                flash_contiguous = true;
                max_kvx = std::max(max_kvx, 2 * hv);
            }
            // the matrix-core attention takes up to 16 query heads per key/value row: the heads go in equal shares of the largest divisor of H up to 16
            int64_t g = std::min<int64_t>(L.heads, 16);
            while (L.heads % g) --g;
            w.head_share = g;
            if (std::find(attn_groups.begin(), attn_groups.end(), g) == attn_groups.end()) attn_groups.push_back(g);
        } else if (L.mixer == LayeredSpec::GLA) {
            w.qcol = 0; w.kcol = hd; w.vcol = 2 * hd; w.gcol = 2 * hd + hv; w.nmix = 2 * hd + 2 * hv;
            RC(own(&w.a2b, (size_t)hd * 4)); RC(own(&w.hnorm, (size_t)L.vdim * 4));
            max_hd = std::max(max_hd, hd);
        } else return fail(NVR_ERR_UNSUPPORTED, "layer %zu: this mixer does not belong to the sequential layout", i);
        RC(named(&w.mix, (size_t)(w.nmix * W * esz))); RC(own(&w.wo, (size_t)(W * hv * esz)));
        if (L.ff_kind == LayeredSpec::FF_POLY) {
            RC(own(&w.up, (size_t)(L.ff * W * esz))); RC(own(&w.down, (size_t)(W * L.ff * esz))); RC(own(&w.act, 16));
            max_ff = std::max(max_ff, L.ff);
        } else if (L.ff_kind == LayeredSpec::FF_MOE) {
            const int64_t f = L.expert_ff, fs = L.shared_ff;
            RC(own(&w.router, (size_t)(L.experts * W * 4)));
            RC(own(&w.egu, (size_t)(L.experts * 2 * f * W * esz))); RC(own(&w.edown, (size_t)(L.experts * W * f * esz)));
            if (fs) { RC(own(&w.sgu, (size_t)(2 * fs * W * esz))); RC(own(&w.sdown, (size_t)(W * fs * esz))); }
            max_ff = std::max(max_ff, 2 * fs); max_rows_e = std::max(max_rows_e, L.top); max_e2f = std::max(max_e2f, L.top * 2 * f); max_ef = std::max(max_ef, L.top * f); max_experts = std::max(max_experts, L.experts); max_f = std::max(max_f, f);
        } else if (L.has_mlp) return fail(NVR_ERR_UNSUPPORTED, "layer %zu: this feed-forward does not belong to the sequential layout", i);
        if (spec.side_dim) { RC(own(&w.sgate, (size_t)(spec.side_dim * W * esz))); RC(own(&w.sproj, (size_t)(W * spec.side_dim * esz))); RC(own(&w.snorm, (size_t)W * 4)); }
        RC(own(&w.dwa, (size_t)(i + 2) * 4));                   // (until loaded: the layer's own output passes)
        { const float one = 1.f; NVR_HIP_CHECK(hipMemcpy(w.dwa + i + 1, &one, 4, hipMemcpyHostToDevice)); }
        max_nmix = std::max(max_nmix, w.nmix); max_hv = std::max(max_hv, hv);
    }
    RC(named(&embed, (size_t)(V * W * esz))); RC(named(&head, (size_t)(V * W * esz))); RC(own(&wfinal, (size_t)W * 4));
    if (spec.side_dim) RC(own(&side_embed, (size_t)(V * nL * spec.side_dim * esz)));

    // pages: one row of kv_rank + rot_dim numbers per token for every latent-attention layer with a latent of its own; state per slot for gated linear attention
    if (r.cfg.num_kvcache_blocks >= 0) r.num_blocks = r.cfg.num_kvcache_blocks;
    else if (r.cfg.num_kvcache_blocks == -1) r.num_blocks = 1000;
    else {
        size_t free_b = 0, total_b = 0;
        NVR_HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        const double budget = (double)free_b - (1.0 - r.cfg.gpu_memory_utilization) * (double)total_b - (double)((nL + 8) * MT * W * 4);
        const int64_t nb = block_bytes ? (int64_t)(budget * 0.9 / (double)block_bytes) : 1000;
        if (nb < 1) return fail(NVR_ERR_HIP, "not enough free HBM for one KV block");
        r.num_blocks = nb;
    }
    rs.resize(spec.layers.size());
    for (size_t i = 0; i < spec.layers.size(); ++i) {
        const LayeredSpec::Layer &L = spec.layers[i];
        if (L.mixer == LayeredSpec::LATENT && L.kv_from < 0) {
            RC(named(&rs[i].kc, (size_t)(r.num_blocks * r.block_size * (L.kv_rank + L.rot_dim) * esz)));
            RC(own(&rs[i].rows, (size_t)(MT * (L.kv_rank + L.rot_dim) * esz)));                 // the step's own cached rows, in step order
        }
        else if (L.mixer == LayeredSpec::GLA) RC(named((void **)&rs[i].state, (size_t)(slots * L.heads * L.dim * L.vdim * 4)));
    }
    for (size_t i = 0; i < spec.layers.size(); ++i) {                           // a layer without a latent of its own reads its source's pages
        const LayeredSpec::Layer &L = spec.layers[i];
        if (L.mixer == LayeredSpec::LATENT && L.kv_from >= 0) { rs[i].kc = rs[(size_t)L.kv_from].kc; rs[i].rows = rs[(size_t)L.kv_from].rows; rs[i].borrowed = true; }
    }

    // activations
    RC(named((void **)&x, (size_t)(MT * W * 4))); RC(own(&kept, (size_t)((nL + 1) * MT * W * 4)));
    RC(named(&a1, (size_t)(MT * W * esz))); RC(named(&a2, (size_t)(MT * W * esz))); RC(named(&tmp, (size_t)(MT * W * esz)));
    RC(named(&proj, (size_t)(MT * max_nmix * esz))); RC(named(&cat, (size_t)(MT * max_hv * esz)));
    RC(own(&qlat, (size_t)(MT * max_qlat * esz))); RC(own(&q2, (size_t)(MT * max_q2 * esz))); RC(own(&qabs, (size_t)(MT * max_qabs * esz))); RC(own(&ctx, (size_t)(MT * max_ctx * esz)));
    RC(named((void **)&ret_o, (size_t)(MT * max_hv * 4))); RC(own(&az, (size_t)(MT * max_hd * esz)));
    RC(named(&gu, (size_t)(MT * max_ff * esz))); RC(own(&act, (size_t)(MT * max_ff * esz))); RC(own(&shared_y, (size_t)(MT * W * esz)));
    const int64_t pad_rows = (max_experts + 1) * 256;       // (experts' rows padded to whole blocks of 256)
    RC(own(&e_gu, (size_t)(MT * max_e2f * esz))); RC(own(&e_act, (size_t)((MT * max_ef + pad_rows * max_f) * esz))); RC(own(&e_y, (size_t)((MT * max_rows_e + pad_rows) * W * esz)));
    RC(own(&e_x, (size_t)((MT * max_rows_e + pad_rows) * W * esz)));
    RC(own(&kvx, (size_t)(MT * max_kvx * esz)));
    RC(own(&side_z, (size_t)(MT * std::max<int64_t>(spec.side_dim, 1) * esz))); RC(own(&side_g, (size_t)(MT * std::max<int64_t>(spec.side_dim, 1) * esz)));
    RC(own(&moe_i, (size_t)((3 * MT * std::max<int64_t>(max_rows_e, 1) + max_experts + 1 + MT * std::max<int64_t>(max_rows_e, 1) / 256 + max_experts + 1024 + 8) * 4))); RC(own(&moe_score, (size_t)(MT * std::max<int64_t>(max_rows_e, 1) * 4)));
    return NVR_OK;
}

// Tensors by the names of the checkpoint: "embed", "head", "final.norm" [W], "side.embed" [vocab][layers * side]; per layer i "l<i>.norm1" / "norm1b" / "norm2" / "norm2b" [W],
// "l<i>.mix.*" (latent attention: q | dq, dq.norm, uq; dkv, dkv.norm; uk, uv; g; o — gated linear attention: q, k, v, g, o, norm, a1, a2, a2.b), "l<i>.mlp.*" (dense: up, down,
// act — experts: router, e<j>.{gate,up,down}, shared.{gate,up,down}), "l<i>.side.{gate,proj,norm}", "l<i>.dwa" [i + 2].  Linear weights are [out][in].
int LayeredModel::load_sequential(nvr_model_runner &r, const std::string &name, int dtype, const int64_t *shape, int ndim, const void *data) {
    const int64_t W = spec.width, V = spec.vocab, nL = (int64_t)spec.layers.size();
    const char *name_in = name.c_str();
    auto is2 = [&](int64_t a, int64_t b) { return ndim == 2 && shape[0] == a && shape[1] == b; };
    auto bad = [&]() { return fail(NVR_ERR_LEN_MISMATCH, "load_tensor: '%s' has the wrong shape", name_in); };
    auto unknown = [&]() { return fail(NVR_ERR_UNSUPPORTED, "load_tensor: unknown tensor '%s'", name_in); };
    auto vec = [&](float *dst, int64_t n) { return (dst && ndim == 1 && shape[0] == n) ? put(r, dst, n, 1, n, dtype, data, false) : bad(); };
    auto mat = [&](void *dst, int64_t ld, int64_t rows, int64_t cols) { return (dst && is2(rows, cols)) ? put(r, dst, ld, rows, cols, dtype, data, true) : bad(); };
    auto rows_at = [&](void *base, int64_t row0, int64_t ld) { return (void *)((char *)base + (size_t)(row0 * ld * esz)); };
    if (name == "embed") return mat(embed, W, V, W);
    if (name == "head") return mat(head, W, V, W);
    if (name == "final.norm") return vec(wfinal, W);
    if (name == "side.embed") return spec.side_dim ? mat(side_embed, nL * spec.side_dim, V, nL * spec.side_dim) : unknown();
    size_t dot = name.find('.');
    if (name.size() < 3 || name[0] != 'l' || dot == std::string::npos || dot < 2) return unknown();
    int64_t li = 0;
    for (size_t i = 1; i < dot; ++i) { if (name[i] < '0' || name[i] > '9') return unknown(); li = li * 10 + (name[i] - '0'); }
    if (li >= nL) return fail(NVR_ERR_UNSUPPORTED, "load_tensor: '%s' names a layer the model does not have", name_in);
    const LayeredSpec::Layer &L = spec.layers[(size_t)li]; LayerW &w = lw[(size_t)li];
    const std::string rest = name.substr(dot + 1);
    const int64_t hd = L.heads * L.dim, hv = L.heads * L.vdim, R = L.rot_dim;
    if (rest == "norm1") return vec(w.n1, W);
    if (rest == "norm1b") return vec(w.n1b, W);
    if (rest == "norm2") return L.has_mlp ? vec(w.n2, W) : unknown();
    if (rest == "norm2b") return L.has_mlp ? vec(w.n2b, W) : unknown();
    if (rest == "dwa") return vec(w.dwa, li + 2);
    if (spec.side_dim) {
        if (rest == "side.gate") return mat(w.sgate, W, spec.side_dim, W);
        if (rest == "side.proj") return mat(w.sproj, spec.side_dim, W, spec.side_dim);
        if (rest == "side.norm") return vec(w.snorm, W);
    }
    if (rest == "mix.o") return mat(w.wo, hv, W, hv);
    if (L.mixer == LayeredSpec::LATENT) {
        if (rest == "mix.q" && !L.q_rank) return mat(w.mix, W, hd, W);
        if (rest == "mix.dq" && L.q_rank) return mat(w.mix, W, L.q_rank, W);
        if (rest == "mix.dq.norm" && L.q_rank) return vec(w.dqn, L.q_rank);
        if (rest == "mix.uq" && L.q_rank) return mat(w.uq, L.q_rank, L.heads * (L.dim + R), L.q_rank);
        if (rest == "mix.g" && L.out_gate) return mat(rows_at(w.mix, w.gcol, W), W, hv, W);
        if (rest == "mix.dkv" && L.kv_from < 0) return mat(rows_at(w.mix, w.dcol, W), W, L.kv_rank + R, W);
        if (rest == "mix.dkv.norm" && L.kv_from < 0) return vec(w.dkvn, L.kv_rank);
        if (rest == "mix.uv") {
            if (w.flash && is2(hv, L.kv_rank)) RC(put(r, (char *)w.wx + (size_t)(hv * (L.kv_rank + R) * esz), L.kv_rank + R, hv, L.kv_rank, dtype, data, true));
            return mat(w.uv, L.kv_rank, hv, L.kv_rank);
        }
        if (rest == "mix.uk") {                             // [H D][kv_rank] -> per head its transpose [kv_rank][D]: the expansion folds into the queries
            if (!is2(hd, L.kv_rank)) return bad();
            std::vector<float> t((size_t)(hd * L.kv_rank));
            for (int64_t h = 0; h < L.heads; ++h)
                for (int64_t k = 0; k < L.dim; ++k)
                    for (int64_t n = 0; n < L.kv_rank; ++n) t[(size_t)((h * L.kv_rank + n) * L.dim + k)] = src_at(dtype, data, (size_t)((h * L.dim + k) * L.kv_rank + n));
            if (w.flash)                                    // head h's key rows sit at h * (D + R) of the expansion (the rotated part's rows follow them)
                for (int64_t h = 0; h < L.heads; ++h)
                    RC(put(r, (char *)w.wx + (size_t)(h * L.vdim * (L.kv_rank + R) * esz), L.kv_rank + R, L.dim, L.kv_rank, dtype,
                           (const char *)data + (size_t)(h * L.dim * L.kv_rank) * (dtype == 2 ? 4 : 2), true));
            return put(r, w.ukt, L.dim, L.heads * L.kv_rank, L.dim, 2, t.data(), true);
        }
    } else {
        if (rest == "mix.q") return mat(rows_at(w.mix, w.qcol, W), W, hd, W);
        if (rest == "mix.k") return mat(rows_at(w.mix, w.kcol, W), W, hd, W);
        if (rest == "mix.v") return mat(rows_at(w.mix, w.vcol, W), W, hv, W);
        if (rest == "mix.g") return mat(rows_at(w.mix, w.gcol, W), W, hv, W);
        if (rest == "mix.norm") return vec(w.hnorm, L.vdim);
        if (rest == "mix.a2.b") return vec(w.a2b, hd);
        if (rest == "mix.a1") {                             // the rank of the decay projection is the tensor's
            if (ndim != 2 || shape[1] != W || shape[0] < 1 || (w.a_rank && w.a_rank != shape[0])) return bad();
            w.a_rank = shape[0];
            if (!w.wa1) RC(own(&w.wa1, (size_t)(w.a_rank * W * esz)));
            if (w.a_rank > alow_cap) { RC(own(&alow, (size_t)(r.max_tokens * w.a_rank * esz))); alow_cap = w.a_rank; }   // (a smaller one before it stays owned)
            return put(r, w.wa1, W, w.a_rank, W, dtype, data, true);
        }
        if (rest == "mix.a2") {
            if (ndim != 2 || shape[0] != hd || shape[1] < 1 || (w.a_rank && w.a_rank != shape[1])) return bad();
            w.a_rank = shape[1];
            if (!w.wa2) RC(own(&w.wa2, (size_t)(hd * w.a_rank * esz)));
            return put(r, w.wa2, w.a_rank, hd, w.a_rank, dtype, data, true);
        }
    }
    if (L.ff_kind == LayeredSpec::FF_POLY) {
        if (rest == "mlp.up") return mat(w.up, W, L.ff, W);
        if (rest == "mlp.down") return mat(w.down, L.ff, W, L.ff);
        if (rest == "mlp.act") return vec(w.act, 4);
    } else if (L.ff_kind == LayeredSpec::FF_MOE) {
        const int64_t f = L.expert_ff, fs = L.shared_ff;
        if (rest == "mlp.router") return (is2(L.experts, W)) ? put(r, w.router, W, L.experts, W, dtype, data, false) : bad();
        if (fs && rest == "mlp.shared.gate") return mat(w.sgu, W, fs, W);
        if (fs && rest == "mlp.shared.up") return mat(rows_at(w.sgu, fs, W), W, fs, W);
        if (fs && rest == "mlp.shared.down") return mat(w.sdown, fs, W, fs);
        if (rest.compare(0, 5, "mlp.e") == 0) {
            size_t d2 = rest.find('.', 5);
            if (d2 == std::string::npos || d2 == 5) return unknown();
            int64_t e = 0;
            for (size_t i = 5; i < d2; ++i) { if (rest[i] < '0' || rest[i] > '9') return unknown(); e = e * 10 + (rest[i] - '0'); }
            if (e >= L.experts) return fail(NVR_ERR_UNSUPPORTED, "load_tensor: '%s' names an expert the layer does not have", name_in);
            const std::string part = rest.substr(d2 + 1);
            if (part == "gate") return mat(rows_at(w.egu, e * 2 * f, W), W, f, W);
            if (part == "up") return mat(rows_at(w.egu, e * 2 * f + f, W), W, f, W);
            if (part == "down") return mat(rows_at(w.edown, e * W, f), f, W, f);
        }
    }
    return unknown();
}

int LayeredModel::forward_sequential(nvr_model_runner &r, const StepPlan &p) {
    const kl::Batch &b = p.b;
    const int64_t T = p.T, R = p.R, W = spec.width, nL = (int64_t)spec.layers.size(), MT = r.max_tokens;
    const float eps = (float)spec.eps; const int groups = (int)spec.norm_groups;
    hipStream_t s = r.stream;
    auto at = [&](void *base, int64_t col) { return (void *)((char *)base + (size_t)(col * esz)); };
    RC(kl::embed_keep(embed, bf16, b.ids, T, W, x, kept, s));
    {   // the first layer's input; every later one leaves the end of the layer before it
        kl::GroupNormArgs n{}; n.in = x; n.ldi = W; n.in_f32 = true; n.rows_n = T; n.W = W; n.groups = groups; n.eps = eps; n.w = lw[0].n1; n.out = a1; n.ldo = W;
        RC(kl::group_norm(n, bf16, s));
    }
    for (int64_t i = 0; i < nL; ++i) {
        const LayeredSpec::Layer &L = spec.layers[(size_t)i]; const LayerW &w = lw[(size_t)i]; RunState &st = rs[(size_t)i];
        const int64_t hv = L.heads * L.vdim;
        RC(gemm(r, a1, W, w.mix, T, W, w.nmix, proj));
        if (L.mixer == LayeredSpec::LATENT) {
            const int64_t Rr = L.rot_dim, rank = L.kv_rank, Dq = rank + Rr;
            const void *qsrc = proj; int64_t ldq = w.nmix, qstride = L.dim;
            if (L.q_rank) {                                 // queries through their own normed latent
                kl::GroupNormArgs n{}; n.in = proj; n.ldi = w.nmix; n.rows_n = T; n.W = L.q_rank; n.groups = 1; n.eps = eps; n.w = w.dqn; n.out = qlat; n.ldo = L.q_rank;
                RC(kl::group_norm(n, bf16, s));
                RC(gemm(r, qlat, L.q_rank, w.uq, T, L.q_rank, L.heads * (L.dim + Rr), q2));
                qsrc = q2; ldq = L.heads * (L.dim + Rr); qstride = L.dim + Rr;
            }
            if (L.kv_from < 0) RC(kl::latent_store(proj, w.nmix, w.dcol, b, rank, Rr, eps, w.dkvn, w.rfreq, st.kc, st.rows, bf16, s));
            if (w.flash && p.whole_prompts) {
                // every key is a row of this step: K (with the rotated part) and V of all heads by one product from the step's cached rows, then the flash kernel
                RC(kl::rotate_heads(qsrc, ldq, qstride, L.dim, b, L.heads, Rr, w.rfreq, (void *)qsrc, ldq, qstride, L.dim, bf16, s));   // (in place: a thread reads a pair, then writes it)
                RC(gemm(r, st.rows, Dq, w.wx, T, Dq, 2 * hv, kvx));
                const size_t gi = (size_t)(std::find(flash_groups.begin(), flash_groups.end(), (int64_t)1) - flash_groups.begin());
                nvr::kt::FlashArgs f{};
                f.q = (const uint16_t *)qsrc; f.ldq = ldq; f.k = (const uint16_t *)kvx; f.v = (const uint16_t *)kvx + hv; f.ldkv = 2 * hv;
                f.tiles = (const nvr::kt::FlashTile *)(in_dev + p.o_ftiles[gi]); f.ntiles = p.n_ftiles[gi];
                f.H = (int32_t)L.heads; f.KVH = (int32_t)L.heads; f.D = (int32_t)L.vdim; f.scale = (float)L.scale; f.out = (uint16_t *)cat; f.ldo = hv;
                RC(nvr::kb::flash_prefill(f, false, s));
                if (L.out_gate) RC(kl::sigmoid_gate(cat, hv, at(proj, w.gcol), w.nmix, T, hv, bf16, s));
            } else {
            // the key expansion folded into the queries: per head q' = Wuk_h^T q (kv_rank numbers), then the rotated part
            kl::HeadLinearArgs ha{}; ha.a = qsrc; ha.lda = ldq; ha.ha = qstride; ha.w = w.ukt; ha.y = qabs; ha.ldy = L.heads * Dq; ha.hy = Dq;
            ha.T = (int32_t)T; ha.H = (int32_t)L.heads; ha.K = (int32_t)L.dim; ha.N = (int32_t)rank;
            RC(kl::head_linear(ha, bf16, s));
            RC(kl::rotate_heads(qsrc, ldq, qstride, L.dim, b, L.heads, Rr, w.rfreq, qabs, L.heads * Dq, Dq, rank, bf16, s));
            kl::SinkAttnArgs a{};
            a.q = qabs; a.ldq = L.heads * Dq; a.kc = st.kc; a.vc = st.kc; a.vld = Dq; a.H = (int32_t)L.heads; a.G = 1; a.D = (int32_t)Dq; a.Dv = (int32_t)rank;
            a.scale = (float)L.scale; a.out = ctx; a.ldo = L.heads * rank;
            kl::SinkAttnArgs a1s = a; a1s.H = (int32_t)w.head_share;
            if (kl::sink_attention_tiled_ok(a1s, bf16, (int)r.block_size)) {
                const size_t gi = (size_t)(std::find(attn_groups.begin(), attn_groups.end(), w.head_share) - attn_groups.begin());
                const int64_t wgs = (int64_t)p.n_tiles[gi];
                int64_t nsplit = 1;
                if (wgs * (L.heads / w.head_share) < r.num_cus && p.max_ctx >= 512) nsplit = std::max<int64_t>(1, std::min<int64_t>({(2 * r.num_cus) / (wgs * (L.heads / w.head_share)), (p.max_ctx + 127) / 128, 16}));
                const size_t share_ws = attn_ws_bytes / (size_t)(L.heads / w.head_share);
                for (int64_t h0 = 0; h0 < L.heads; h0 += w.head_share) {       // one launch per share of the heads, all on the same cached rows
                    kl::SinkAttnArgs as = a1s;
                    as.q = (const char *)qabs + (size_t)(h0 * Dq * esz); as.out = (char *)ctx + (size_t)(h0 * rank * esz);
                    RC(kl::sink_attention_tiled(as, b, (const kl::AttnTile *)(in_dev + p.o_tiles[gi]), p.n_tiles[gi], (int)nsplit, (char *)attn_ws + (size_t)(h0 / w.head_share) * share_ws, share_ws, s));
                }
            } else
                RC(kl::sink_attention(a, b, bf16, s));
            // the value expansion of the attended latent, and the output gate
            kl::HeadLinearArgs hu{}; hu.a = ctx; hu.lda = L.heads * rank; hu.ha = rank; hu.w = w.uv; hu.y = cat; hu.ldy = hv; hu.hy = L.vdim;
            hu.T = (int32_t)T; hu.H = (int32_t)L.heads; hu.K = (int32_t)rank; hu.N = (int32_t)L.vdim;
            if (L.out_gate) { hu.gate = at(proj, w.gcol); hu.ldg = w.nmix; hu.hg = L.vdim; }
            RC(kl::head_linear(hu, bf16, s));
            }
        } else {
            if (!w.wa1 || !w.wa2) return fail(NVR_ERR_NOT_ALLOCATED, "layer %ld: the decay projections were not loaded", (long)i);
            RC(gemm(r, a1, W, w.wa1, T, W, w.a_rank, alow));
            RC(gemm(r, alow, w.a_rank, w.wa2, T, w.a_rank, L.heads * L.dim, az));
            kl::RetentionArgs a{};
            a.proj = proj; a.ld = w.nmix; a.qcol = w.qcol; a.kcol = w.kcol; a.vcol = w.vcol; a.rot_dims = 0; a.kscale = 1.0f;
            a.H = (int32_t)L.heads; a.D = (int32_t)L.dim; a.Dv = (int32_t)L.vdim; a.state = st.state; a.o = ret_o;
            a.az = az; a.ldz = L.heads * L.dim; a.abias = w.a2b; a.inv_tau = (float)(1.0 / L.tau); a.qscale = 1.0f / std::sqrt((float)L.dim);
            RC(kl::retention(a, b, bf16, s));
            RC(kl::head_norm_gate(ret_o, proj, w.nmix, w.gcol, T, L.heads, L.vdim, eps, w.hnorm, cat, hv, bf16, s));
        }
        RC(gemm(r, cat, hv, w.wo, T, hv, W, tmp));
        {   // the mixer's output joins the stream; the feed-forward's input leaves in the same pass
            kl::GroupNormArgs n{}; n.in = tmp; n.ldi = W; n.rows_n = T; n.W = W; n.groups = groups; n.eps = eps; n.w = w.n1b; n.xres = x;
            if (L.has_mlp) { n.w2 = w.n2; n.out = a2; n.ldo = W; }
            else if (spec.side_dim && bf16) { n.out_plain = true; n.out = a2; n.ldo = W; }       // (the token input's projection reads the stream in the operand type)
            RC(kl::group_norm(n, bf16, s));
        }
        if (L.ff_kind == LayeredSpec::FF_POLY) {
            RC(gemm(r, a2, W, w.up, T, W, L.ff, gu));
            RC(kl::poly_norm(gu, L.ff, T, L.ff, eps, w.act, act, L.ff, bf16, s));
            RC(gemm(r, act, L.ff, w.down, T, L.ff, W, tmp));
        } else if (L.ff_kind == LayeredSpec::FF_MOE) {
            const int64_t f = L.expert_ff, fs = L.shared_ff, n = T * L.top;
            int32_t *sel = moe_i, *order = sel + MT * L.top, *place_of = order + MT * L.top, *off = place_of + MT * L.top, *row_w = off + L.experts + 1;
            // many rows: every expert's rows padded to whole blocks of 256, brought together once, and the dense graph's 256 x 256 product with a matrix per row block
            const int64_t nblocks = n / 256 + L.experts;
            const bool blocks = bf16 && n >= 2048 && nvr::kb::gemm256_silu_ok(nblocks * 256, W, f, W) && nvr::kb::gemm256_ok(nblocks * 256, f, W, f);
            RC(kl::moe_route(a2, W, T, W, w.router, L.experts, L.top, sel, moe_score, off, order, place_of, blocks ? 256 : 1, blocks ? row_w : nullptr, nblocks, bf16, s));
            if (blocks) {
                RC(kl::moe_gather(a2, W, T, W, L.top, place_of, moe_score, e_x, bf16, s));
                RC(nvr::kb::gemm256_grouped_silu_mul((const uint16_t *)e_x, W, (const uint16_t *)w.egu, 2 * f * W, row_w, nblocks * 256, W, f, (uint16_t *)e_act, s));
                RC(nvr::kb::gemm256_grouped((const uint16_t *)e_act, f, (const uint16_t *)w.edown, W * f, row_w, nblocks * 256, f, W, (uint16_t *)e_y, s));
            } else {
                kl::GroupedLinearArgs g{}; g.a = a2; g.lda = W; g.w = w.egu; g.y = e_gu; g.ldy = 2 * f; g.off = off; g.groups = (int32_t)L.experts; g.K = (int32_t)W; g.N = (int32_t)(2 * f);
                g.max_rows = (int32_t)n; g.src = order; g.rscale = moe_score; g.src_div = (int32_t)L.top;
                RC(kl::grouped_linear(g, bf16, s));
                RC(kl::silu_mul(e_gu, n, f, e_act, f, bf16, s));
                kl::GroupedLinearArgs d{}; d.a = e_act; d.lda = f; d.w = w.edown; d.y = e_y; d.ldy = W; d.off = off; d.groups = (int32_t)L.experts; d.K = (int32_t)f; d.N = (int32_t)W; d.max_rows = (int32_t)n;
                RC(kl::grouped_linear(d, bf16, s));
            }
            if (fs) {
                if (bf16 && nvr::kb::gemm256_silu_ok(T, W, fs, W)) RC(nvr::kb::gemm256_silu_mul((const uint16_t *)a2, W, (const uint16_t *)w.sgu, T, W, fs, (uint16_t *)act, s));   // (gate, up and SiLU in one launch)
                else {
                    RC(gemm(r, a2, W, w.sgu, T, W, 2 * fs, gu));
                    RC(kl::silu_mul(gu, T, fs, act, fs, bf16, s));
                }
                RC(gemm(r, act, fs, w.sdown, T, fs, W, shared_y));
            }
            RC(kl::moe_combine(e_y, place_of, T, L.top, fs ? shared_y : nullptr, W, tmp, bf16, s));
        }
        if (L.has_mlp) {
            kl::GroupNormArgs n{}; n.in = tmp; n.ldi = W; n.rows_n = T; n.W = W; n.groups = groups; n.eps = eps; n.w = w.n2b; n.xres = x;
            if (spec.side_dim && bf16) { n.out_plain = true; n.out = a2; n.ldo = W; }
            RC(kl::group_norm(n, bf16, s));
        }
        kl::LayerTailArgs t{}; t.x = x; t.T = (int32_t)T; t.W = (int32_t)W; t.eps = eps;
        if (spec.side_dim) {                                // the token input: two products around the gate, its norm at the end of the layer
            RC(gemm(r, bf16 ? a2 : (void *)x, W, w.sgate, T, W, spec.side_dim, side_z));
            RC(kl::side_gate(side_z, b.ids, side_embed, nL * spec.side_dim, i * spec.side_dim, spec.side_dim, T, side_g, bf16, s));
            RC(gemm(r, side_g, spec.side_dim, w.sproj, T, spec.side_dim, W, tmp));
            t.side_y = tmp; t.side_norm = w.snorm;
        }
        t.kept = kept; t.kept_rows = MT; t.nx = (int32_t)(i + 2); t.mix = w.dwa;
        if (i + 1 < nL) { t.wnext = lw[(size_t)(i + 1)].n1; t.groups = groups; t.out = a1; }
        RC(kl::layer_tail(t, bf16, s));
    }
    kl::GroupNormArgs n{}; n.in = x; n.ldi = W; n.in_f32 = true; n.rows = p.d_want; n.rows_n = R; n.W = W; n.groups = groups; n.eps = eps; n.w = wfinal; n.out = xsel; n.ldo = W;
    RC(kl::group_norm(n, bf16, s));
    return gemm(r, xsel, W, head, R, W, spec.vocab, r.logits, true);
}

// ===================================================================================================================================================
// Scaled layout: x <- x + ls1 * mixer(n1(x)); x <- x + ls2 * ff(n2(x)); learned positions; a layer run uses the weights of layer spec.runs[run] and a
// cache / state of its own.

namespace { inline int64_t pad16(int64_t n) { return (n + 15) / 16 * 16; } }

int LayeredModel::init_scaled(nvr_model_runner &r) {
    const int64_t W = spec.width, V = spec.vocab, MT = r.max_tokens;
    auto named = [&](void **p, size_t bytes) {              // (the buffers the destructor frees by name)
        RC(dmalloc((char **)p, bytes));
        NVR_HIP_CHECK(hipMemset(*p, 0, bytes ? bytes : 16));
        return (int)NVR_OK;
    };
    lw.resize(spec.layers.size());
    int64_t max_nmix = 0, max_hv = 0, max_ro = 0, max_ff = 0, max_gw = 0, max_gpad = 16, max_h = 1;
    for (size_t i = 0; i < spec.layers.size(); ++i) {
        const LayeredSpec::Layer &L = spec.layers[i]; LayerW &w = lw[i];
        if (L.weights_of >= 0) continue;                    // (its runs read the source's LayerW)
        const int64_t hd = L.heads * L.dim, hv = L.heads * L.vdim;
        RC(own(&w.n1, (size_t)W * 4)); RC(own(&w.ls1, (size_t)W * 4));
        if (L.has_mlp) {
            RC(own(&w.n2, (size_t)W * 4)); RC(own(&w.ls2, (size_t)W * 4));
            RC(own(&w.up, (size_t)(L.ff * W * esz))); RC(own(&w.down, (size_t)(W * L.ff * esz)));
            max_ff = std::max(max_ff, L.ff);
        }
        if (L.mixer == LayeredSpec::MLSTM) {
            w.qcol = 0; w.kcol = pad16(hd); w.vcol = w.kcol + pad16(hd); w.gcol = w.vcol + pad16(hv); w.nmix = w.gcol + pad16(hv);
            w.gpad = pad16(2 * L.heads);
            RC(own(&w.wgates, (size_t)(w.gpad * W * esz))); RC(own(&w.bi, (size_t)L.heads * 4)); RC(own(&w.bfg, (size_t)L.heads * 4)); RC(own(&w.hnorm, (size_t)hv * 4));
            max_ro = std::max(max_ro, L.heads * (L.vdim + 1)); max_gpad = std::max(max_gpad, w.gpad); max_h = std::max(max_h, L.heads);
        } else if (L.mixer == LayeredSpec::ATTN_GRU) {
            const int64_t kn = L.kv_heads * L.dim, vn = L.kv_heads * L.vdim, gw = L.gru_width;
            w.qcol = 0; w.kcol = pad16(hd); w.vcol = w.kcol + pad16(kn); w.gcol = w.vcol + pad16(vn); w.zcol = w.gcol + pad16(hv); w.ucol = w.zcol + pad16(gw); w.rgcol = w.ucol + pad16(gw);
            w.nmix = w.rgcol + pad16(gw);
            RC(own(&w.qn, (size_t)hd * 4)); RC(own(&w.kn, (size_t)kn * 4)); RC(named((void **)&w.sink, (size_t)L.heads * 4));
            RC(own(&w.bz, (size_t)gw * 4)); RC(own(&w.bu, (size_t)gw * 4)); RC(own(&w.outl, (size_t)W * 4)); RC(own(&w.outr, (size_t)W * 4));
            RC(own(&w.wo2, (size_t)(W * gw * esz)));
            std::vector<float> sl((size_t)L.heads);
            for (int64_t h = 0; h < L.heads; ++h) sl[(size_t)h] = (float)std::exp2(-8.0 * (double)(h + 1) / (double)L.heads);
            RC(own(&w.slope, sl.size() * 4)); NVR_HIP_CHECK(hipMemcpy(w.slope, sl.data(), sl.size() * 4, hipMemcpyHostToDevice));
            if (std::find(attn_groups.begin(), attn_groups.end(), L.heads / L.kv_heads) == attn_groups.end()) attn_groups.push_back(L.heads / L.kv_heads);
            w.flash = bf16 && L.dim == L.vdim && nvr::kb::flash_prefill_ok((int)L.dim, (int)L.heads, (int)L.kv_heads) && hv % 8 == 0;
            if (w.flash && std::find(flash_groups.begin(), flash_groups.end(), L.heads / L.kv_heads) == flash_groups.end()) flash_groups.push_back(L.heads / L.kv_heads);
            if (bf16) {                                     // the matrix-core attention takes the slopes as its table of penalties by distance (the window bounds the distance)
                const int64_t n = std::min<int64_t>(r.max_pos, L.window) + 1;
                RC(dmalloc(&w.pen, (size_t)(L.heads * n * 4)));
                RC(kl::linear_penalty_table(w.slope, L.heads, n, w.pen, r.stream)); w.pen_dirty = false;
            }
            max_gw = std::max(max_gw, gw);
        } else return fail(NVR_ERR_UNSUPPORTED, "layer %zu: this mixer does not belong to the scaled layout", i);
        RC(named(&w.mix, (size_t)(w.nmix * W * esz))); RC(own(&w.wo, (size_t)(W * hv * esz)));
        max_nmix = std::max(max_nmix, w.nmix); max_hv = std::max(max_hv, hv);
    }
    RC(named(&embed, (size_t)(V * W * esz))); RC(named(&head, (size_t)(V * W * esz))); RC(own(&wfinal, (size_t)W * 4));
    RC(own(&pos, (size_t)(spec.max_positions * W * esz)));

    // pages for every run with attention; per slot the matrix memory (with the column of the keys' running sum and the running maxima) or the recurrence's state
    size_t block_bytes = 0;
    for (int li : spec.runs) {
        const LayeredSpec::Layer &L = spec.layers[(size_t)li];
        if (L.mixer == LayeredSpec::ATTN_GRU) block_bytes += (size_t)(r.block_size * L.kv_heads * (L.dim + L.vdim) * esz);
    }
    if (r.cfg.num_kvcache_blocks >= 0) r.num_blocks = r.cfg.num_kvcache_blocks;
    else if (r.cfg.num_kvcache_blocks == -1) r.num_blocks = 1000;
    else {
        size_t free_b = 0, total_b = 0;
        NVR_HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        const double budget = (double)free_b - (1.0 - r.cfg.gpu_memory_utilization) * (double)total_b - (double)(MT * (8 * W + 2 * max_nmix + 2 * max_ro + 4 * max_ff) * 4);
        const int64_t nb = block_bytes ? (int64_t)(budget * 0.9 / (double)block_bytes) : 1000;
        if (nb < 1) return fail(NVR_ERR_HIP, "not enough free HBM for one KV block");
        r.num_blocks = nb;
    }
    rs.resize(spec.runs.size());
    for (size_t ri = 0; ri < spec.runs.size(); ++ri) {
        const LayeredSpec::Layer &L = spec.layers[(size_t)spec.runs[ri]]; RunState &st = rs[ri];
        if (L.mixer == LayeredSpec::ATTN_GRU) {
            RC(named(&st.kc, (size_t)(r.num_blocks * r.block_size * L.kv_heads * L.dim * esz))); RC(named(&st.vc, (size_t)(r.num_blocks * r.block_size * L.kv_heads * L.vdim * esz)));
            RC(named((void **)&st.state, (size_t)(slots * L.gru_width * 4)));
        } else {
            RC(named((void **)&st.state, (size_t)(slots * L.heads * L.dim * (L.vdim + 1) * 4))); RC(own(&st.mstate, (size_t)(slots * L.heads * 4)));
        }
    }

    // activations
    RC(named((void **)&x, (size_t)(MT * W * 4)));
    RC(named(&a1, (size_t)(MT * W * esz))); RC(named(&a2, (size_t)(MT * W * esz))); RC(named(&tmp, (size_t)(MT * W * esz))); RC(own(&tmp2, (size_t)(MT * W * esz)));
    RC(named(&proj, (size_t)(MT * max_nmix * esz))); RC(named(&cat, (size_t)(MT * max_hv * esz))); RC(own(&gy, (size_t)(MT * max_gw * esz)));
    RC(named((void **)&ret_o, (size_t)(MT * max_ro * 4)));
    RC(own(&gpre, (size_t)(MT * max_gpad * 4))); RC(own(&tokg, (size_t)(MT * max_h * 2 * 4))); RC(own(&gfloor, (size_t)(MT * max_h * 4)));
    RC(named(&gu, (size_t)(MT * max_ff * esz))); RC(own(&act, (size_t)(MT * max_ff * esz)));
    return NVR_OK;
}

// Tensors by the names of the checkpoint: "embed", "pos" [positions][W], "head", "final.norm" [W]; per layer i with tensors of its own "l<i>.norm1" / "norm2" / "ls1" / "ls2" [W],
// matrix memory "l<i>.mix.{q,k,v,g,o,norm,i,i.b,f,f.b}", side by side "l<i>.mix.left.{q,k,v,g,o,q.norm,k.norm,sink,out}" and "l<i>.mix.right.{z,z.b,x,x.b,g,o,out}",
// "l<i>.mlp.{up,down}".  Linear weights are [out][in].
int LayeredModel::load_scaled(nvr_model_runner &r, const std::string &name, int dtype, const int64_t *shape, int ndim, const void *data) {
    const int64_t W = spec.width, V = spec.vocab, nL = (int64_t)spec.layers.size();
    const char *name_in = name.c_str();
    auto is2 = [&](int64_t a, int64_t b) { return ndim == 2 && shape[0] == a && shape[1] == b; };
    auto bad = [&]() { return fail(NVR_ERR_LEN_MISMATCH, "load_tensor: '%s' has the wrong shape", name_in); };
    auto unknown = [&]() { return fail(NVR_ERR_UNSUPPORTED, "load_tensor: unknown tensor '%s'", name_in); };
    auto vec = [&](float *dst, int64_t n) { return (dst && ndim == 1 && shape[0] == n) ? put(r, dst, n, 1, n, dtype, data, false) : bad(); };
    auto mat = [&](void *dst, int64_t ld, int64_t rows, int64_t cols) { return (dst && is2(rows, cols)) ? put(r, dst, ld, rows, cols, dtype, data, true) : bad(); };
    auto rows_at = [&](void *base, int64_t row0, int64_t ld) { return (void *)((char *)base + (size_t)(row0 * ld * esz)); };
    if (name == "embed") return mat(embed, W, V, W);
    if (name == "head") return mat(head, W, V, W);
    if (name == "pos") return mat(pos, W, spec.max_positions, W);
    if (name == "final.norm") return vec(wfinal, W);
    size_t dot = name.find('.');
    if (name.size() < 3 || name[0] != 'l' || dot == std::string::npos || dot < 2) return unknown();
    int64_t li = 0;
    for (size_t i = 1; i < dot; ++i) { if (name[i] < '0' || name[i] > '9') return unknown(); li = li * 10 + (name[i] - '0'); }
    if (li >= nL) return fail(NVR_ERR_UNSUPPORTED, "load_tensor: '%s' names a layer the model does not have", name_in);
    const LayeredSpec::Layer &L = spec.layers[(size_t)li]; LayerW &w = lw[(size_t)li];
    if (L.weights_of >= 0) return fail(NVR_ERR_UNSUPPORTED, "load_tensor: '%s' names a layer that uses the tensors of layer %ld", name_in, (long)L.weights_of);
    const std::string rest = name.substr(dot + 1);
    const int64_t hd = L.heads * L.dim, hv = L.heads * L.vdim;
    if (rest == "norm1") return vec(w.n1, W);
    if (rest == "ls1") return vec(w.ls1, W);
    if (L.has_mlp) {
        if (rest == "norm2") return vec(w.n2, W);
        if (rest == "ls2") return vec(w.ls2, W);
        if (rest == "mlp.up") return mat(w.up, W, L.ff, W);
        if (rest == "mlp.down") return mat(w.down, L.ff, W, L.ff);
    }
    if (L.mixer == LayeredSpec::MLSTM) {
        if (rest == "mix.q") return mat(rows_at(w.mix, w.qcol, W), W, hd, W);
        if (rest == "mix.k") return mat(rows_at(w.mix, w.kcol, W), W, hd, W);
        if (rest == "mix.v") return mat(rows_at(w.mix, w.vcol, W), W, hv, W);
        if (rest == "mix.g") return mat(rows_at(w.mix, w.gcol, W), W, hv, W);
        if (rest == "mix.o") return mat(w.wo, hv, W, hv);
        if (rest == "mix.norm") return vec(w.hnorm, hv);
        if (rest == "mix.i") return mat(w.wgates, W, L.heads, W);
        if (rest == "mix.f") return mat(rows_at(w.wgates, L.heads, W), W, L.heads, W);
        if (rest == "mix.i.b") return vec(w.bi, L.heads);
        if (rest == "mix.f.b") return vec(w.bfg, L.heads);
    } else {
        const int64_t kn = L.kv_heads * L.dim, vn = L.kv_heads * L.vdim, gw = L.gru_width;
        if (rest == "mix.left.q") return mat(rows_at(w.mix, w.qcol, W), W, hd, W);
        if (rest == "mix.left.k") return mat(rows_at(w.mix, w.kcol, W), W, kn, W);
        if (rest == "mix.left.v") return mat(rows_at(w.mix, w.vcol, W), W, vn, W);
        if (rest == "mix.left.g") return mat(rows_at(w.mix, w.gcol, W), W, hv, W);
        if (rest == "mix.left.o") return mat(w.wo, hv, W, hv);
        if (rest == "mix.left.q.norm") return vec(w.qn, hd);
        if (rest == "mix.left.k.norm") return vec(w.kn, kn);
        if (rest == "mix.left.sink") return vec(w.sink, L.heads);
        if (rest == "mix.left.out") return vec(w.outl, W);
        if (rest == "mix.right.z") return mat(rows_at(w.mix, w.zcol, W), W, gw, W);
        if (rest == "mix.right.x") return mat(rows_at(w.mix, w.ucol, W), W, gw, W);
        if (rest == "mix.right.g") return mat(rows_at(w.mix, w.rgcol, W), W, gw, W);
        if (rest == "mix.right.z.b") return vec(w.bz, gw);
        if (rest == "mix.right.x.b") return vec(w.bu, gw);
        if (rest == "mix.right.o") return mat(w.wo2, gw, W, gw);
        if (rest == "mix.right.out") return vec(w.outr, W);
    }
    return unknown();
}

int LayeredModel::forward_scaled(nvr_model_runner &r, const StepPlan &p) {
    const kl::Batch &b = p.b;
    const int64_t T = p.T, R = p.R, W = spec.width, nR = (int64_t)spec.runs.size();
    const float eps = (float)spec.eps;
    hipStream_t s = r.stream;
    auto at = [&](void *base, int64_t col) { return (void *)((char *)base + (size_t)(col * esz)); };
    RC(kl::embed_pos(embed, pos, bf16, b, W, (float)spec.embedding_scale, x, s));
    {   // the first layer's input; every later one leaves the join before it
        kl::GroupNormArgs n{}; n.in = x; n.ldi = W; n.in_f32 = true; n.rows_n = T; n.W = W; n.groups = 1; n.eps = eps; n.w = lw[(size_t)spec.runs[0]].n1; n.out = a1; n.ldo = W;
        RC(kl::group_norm(n, bf16, s));
    }
    for (int64_t ri = 0; ri < nR; ++ri) {
        const size_t li = (size_t)spec.runs[(size_t)ri];
        const LayeredSpec::Layer &L = spec.layers[li]; const LayerW &w = lw[li]; RunState &st = rs[(size_t)ri];
        const int64_t hv = L.heads * L.vdim;
        const float *next_n1 = ri + 1 < nR ? lw[(size_t)spec.runs[(size_t)ri + 1]].n1 : nullptr;
        kl::JoinArgs j{}; j.x = x; j.T = T; j.W = W; j.eps = eps; j.ls = w.ls1; j.y1 = tmp; j.ld1 = W;
        if (L.has_mlp) { j.wn = w.n2; j.out = a2; } else { j.wn = next_n1; j.out = a1; }
        j.ldo = W;
        RC(gemm(r, a1, W, w.mix, T, W, w.nmix, proj));
        if (L.mixer == LayeredSpec::MLSTM) {
            RC(gemm(r, a1, W, w.wgates, T, W, w.gpad, gpre, true));                  // the gates' pre-activations leave the product in f32
            RC(kl::exp_gates(gpre, w.gpad, w.bi, w.bfg, (float)L.gate_cap, b, L.heads, st.mstate, tokg, gfloor, s));
            kl::RetentionArgs a{};
            a.proj = proj; a.ld = w.nmix; a.qcol = w.qcol; a.kcol = w.kcol; a.vcol = w.vcol; a.rot_dims = 0; a.kscale = 1.0f; a.qscale = 1.0f / std::sqrt((float)L.dim);
            a.H = (int32_t)L.heads; a.D = (int32_t)L.dim; a.Dv = (int32_t)L.vdim + 1; a.v_ones = 1; a.tok_gate = tokg; a.state = st.state; a.o = ret_o; a.inv_tau = 1.f;
            RC(kl::retention(a, b, bf16, s));
            RC(kl::memory_readout(ret_o, gfloor, proj, w.nmix, w.gcol, T, L.heads, L.vdim, eps, w.hnorm, cat, hv, bf16, s));
            RC(gemm(r, cat, hv, w.wo, T, hv, W, tmp));
        } else {
            kl::SinkAttnArgs a{};
            a.q = at(proj, w.qcol); a.ldq = w.nmix; a.kc = st.kc; a.vc = st.vc; a.sink = w.sink; a.slope = w.slope; a.window = (int32_t)L.window;
            a.H = (int32_t)L.heads; a.G = (int32_t)L.kv_heads; a.D = (int32_t)L.dim; a.Dv = (int32_t)L.vdim; a.scale = (float)L.scale;
            a.out = cat; a.ldo = hv;
            a.v_grouped = w.flash ? 0 : 1;                                           // (a property of the layer: the pages keep one layout)
            const bool tiled = kl::sink_attention_tiled_ok(a, bf16, (int)r.block_size);
            kl::QkvNormArgs qa{};
            qa.proj = proj; qa.ld = w.nmix; qa.qcol = w.qcol; qa.kcol = w.kcol; qa.vcol = w.vcol; qa.H = a.H; qa.G = a.G; qa.D = a.D; qa.Dv = a.Dv; qa.eps = eps;
            qa.wq = w.qn; qa.wk = w.kn; qa.v_unit = true; qa.temp_coef = (float)L.temp_coef; qa.temp_every = (int32_t)L.temp_every;
            qa.kc = st.kc; qa.vc = st.vc; qa.v_grouped = tiled && !w.flash;
            RC(kl::qkv_norm_store(qa, b, bf16, s));
            if (w.flash && !p.decode_sized) {
                // prompts and portions: the dense graph's flash kernel in its penalty / sink form, linear in the distance and windowed
                const size_t gi = (size_t)(std::find(flash_groups.begin(), flash_groups.end(), L.heads / L.kv_heads) - flash_groups.begin());
                nvr::kt::FlashArgs f{};
                f.q = (const uint16_t *)a.q; f.ldq = w.nmix; f.k = (const uint16_t *)st.kc; f.v = (const uint16_t *)st.vc; f.ldkv = 0;
                f.block_tables = b.block_tables; f.max_blocks = b.max_blocks; f.block_size = b.block_size;
                f.tiles = (const nvr::kt::FlashTile *)(in_dev + p.o_ftiles[gi]); f.ntiles = p.n_ftiles[gi];
                f.H = (int32_t)L.heads; f.KVH = (int32_t)L.kv_heads; f.D = (int32_t)L.dim; f.scale = (float)L.scale; f.out = (uint16_t *)cat;
                f.r1 = w.slope; f.r2 = nullptr; f.sink = w.sink; f.ldo = hv; f.window = (int32_t)L.window;
                RC(nvr::kb::flash_prefill(f, true, s));
            } else if (tiled) {
                a.pen = w.pen; a.pen_n = (int32_t)(std::min<int64_t>(r.max_pos, L.window) + 1);
                const size_t gi = (size_t)(std::find(attn_groups.begin(), attn_groups.end(), L.heads / L.kv_heads) - attn_groups.begin());
                const int64_t wgs = (int64_t)p.n_tiles[gi] * L.kv_heads, keys = std::min<int64_t>(p.max_ctx, L.window + 64);
                int64_t nsplit = 1;
                if (wgs < r.num_cus && keys >= 512) nsplit = std::max<int64_t>(1, std::min<int64_t>({(2 * r.num_cus) / wgs, (keys + 255) / 256, 16}));
                RC(kl::sink_attention_tiled(a, b, (const kl::AttnTile *)(in_dev + p.o_tiles[gi]), p.n_tiles[gi], (int)nsplit, attn_ws, attn_ws_bytes, s));
            } else
                RC(kl::sink_attention(a, b, bf16, s));
            RC(kl::sigmoid_gate(cat, hv, at(proj, w.gcol), w.nmix, T, hv, bf16, s));
            RC(gemm(r, cat, hv, w.wo, T, hv, W, tmp));
            RC(kl::gated_unit(proj, w.nmix, w.zcol, w.ucol, w.rgcol, w.bz, w.bu, b, L.gru_width, st.state, gy, L.gru_width, bf16, s));
            RC(gemm(r, gy, L.gru_width, w.wo2, T, L.gru_width, W, tmp2));
            j.w1 = w.outl; j.y2 = tmp2; j.ld2 = W; j.w2 = w.outr;
        }
        RC(kl::residual_join(j, bf16, s));
        if (L.has_mlp) {
            if (bf16 && nvr::kb::gemm256_preferred(T, W, L.ff, W)) RC(nvr::kb::gemm256_relu2((const uint16_t *)a2, W, (const uint16_t *)w.up, T, W, L.ff, (uint16_t *)act, s));   // (the squared ReLU in the product's epilogue)
            else {
                RC(gemm(r, a2, W, w.up, T, W, L.ff, gu));
                RC(kl::relu_squared(gu, L.ff, T, L.ff, act, L.ff, bf16, s));
            }
            RC(gemm(r, act, L.ff, w.down, T, L.ff, W, tmp));
            kl::JoinArgs j2{}; j2.x = x; j2.T = T; j2.W = W; j2.eps = eps; j2.ls = w.ls2; j2.y1 = tmp; j2.ld1 = W; j2.wn = next_n1; j2.out = a1; j2.ldo = W;
            RC(kl::residual_join(j2, bf16, s));
        }
    }
    kl::GroupNormArgs n{}; n.in = x; n.ldi = W; n.in_f32 = true; n.rows = p.d_want; n.rows_n = R; n.W = W; n.groups = 1; n.eps = eps; n.w = wfinal; n.out = xsel; n.ldo = W;
    RC(kl::group_norm(n, bf16, s));
    RC(gemm(r, xsel, W, head, R, W, spec.vocab, r.logits, true));
    if (spec.logit_scale != 1.0) RC(kl::scale_f32(r.logits, R * spec.vocab, (float)spec.logit_scale, s));
    return NVR_OK;
}

}  // namespace nvr
