// layered_joint.cpp — the joint layout of layer-list models (layered_model.h): x <- x + mixer(shift(n(x))) + ff(n(x)) with one norm per layer, a state-space mixer or an
// attention without softmax beside a time-mixing recurrence, a mixture of clamped gated experts, and passes over a looped range of layers that each start with a
// product over [x ; embedding output].  A layer run uses the weights of layer spec.runs[run] and a cache / state of its own.
#include <algorithm>
#include <cmath>
#include <cstring>
#include "layered_model.h"
#include "model_runner.h"
#include "kernels/kernels.h"

#define RC(expr) do { int _rc = (expr); if (_rc) return _rc; } while (0)

namespace nvr {

namespace {
inline int64_t pad16(int64_t n) { return (n + 15) / 16 * 16; }
}

int LayeredModel::init_joint(nvr_model_runner &r) {
    const int64_t W = spec.width, V = spec.vocab, MT = r.max_tokens;
    auto named = [&](void **p, size_t bytes) {              // (the buffers the destructor frees by name)
        NVR_HIP_CHECK(hipMalloc(p, bytes ? bytes : 16));
        NVR_HIP_CHECK(hipMemset(*p, 0, bytes ? bytes : 16));
        return (int)NVR_OK;
    };
    lw.resize(spec.layers.size());
    int64_t max_nmix = 0, max_cat = 0, max_ro = 0, max_conv = 0, max_h = 1, max_t4 = 0, max_tn = 0, max_fs = 0, max_top = 0, max_e2f = 0, max_ef = 0, max_experts = 0, max_f = 0;
    const bool loops = spec.has_loop;
    for (size_t i = 0; i < spec.layers.size(); ++i) {
        const LayeredSpec::Layer &L = spec.layers[i]; LayerW &w = lw[i];
        RC(own(&w.n1, (size_t)W * 4)); RC(own(&w.shift, (size_t)W * 4));
        if (L.mixer == LayeredSpec::SSM) {
            const int64_t inner = L.heads * L.vdim, gn = L.kv_heads * L.dim;
            w.conv_c = inner + 2 * gn; w.ccol = inner; w.dtcol = inner + w.conv_c;
            w.nmix = pad16(w.dtcol + L.heads);               // z | x | B | C | dt, as the checkpoint's one tensor has them (zero rows behind)
            RC(own(&w.convw, (size_t)(w.conv_c * L.conv_taps) * 4)); RC(own(&w.convb, (size_t)w.conv_c * 4));
            RC(own(&w.dtb, (size_t)L.heads * 4)); RC(own(&w.alog, (size_t)L.heads * 4)); RC(own(&w.skip, (size_t)L.heads * 4)); RC(own(&w.hnorm, (size_t)inner * 4));
            RC(own(&w.wo, (size_t)(W * inner * esz)));
            max_cat = std::max(max_cat, inner); max_ro = std::max(max_ro, inner); max_conv = std::max(max_conv, w.conv_c); max_h = std::max(max_h, L.heads);
        } else if (L.mixer == LayeredSpec::ATTN_TMIX) {
            const int64_t hd = L.heads * L.dim, kn = L.kv_heads * L.dim, vn = L.kv_heads * L.vdim, hv = L.heads * L.vdim, tn = L.t_heads * L.t_dim;
            w.qcol = 0; w.kcol = pad16(hd); w.vcol = w.kcol + pad16(kn); w.gcol = w.vcol + pad16(vn); w.nmix = w.gcol + pad16(hv);
            RC(own(&w.pb, (size_t)L.heads * 4)); RC(own(&w.outl, (size_t)W * 4)); RC(own(&w.outr, (size_t)W * 4)); RC(own(&w.wo, (size_t)(W * hv * esz)));
            std::vector<float> f((size_t)std::max<int64_t>(L.rot_dims / 2, 1));
            for (int64_t j = 0; j < L.rot_dims / 2; ++j) f[(size_t)j] = (float)(std::pow(L.rot_base, -2.0 * (double)j / (double)L.rot_dims) / L.rot_factor);
            RC(own(&w.rfreq, f.size() * 4)); NVR_HIP_CHECK(hipMemcpy(w.rfreq, f.data(), f.size() * 4, hipMemcpyHostToDevice));
            RC(own(&w.mu, (size_t)(5 * W) * 4)); RC(own(&w.w4, (size_t)(4 * tn * W * esz))); RC(own(&w.wo2, (size_t)(W * tn * esz)));
            RC(own(&w.w0, (size_t)tn * 4)); RC(own(&w.bonus, (size_t)tn * 4)); RC(own(&w.tnorm, (size_t)tn * 4));
            if (std::find(attn_groups.begin(), attn_groups.end(), L.heads / L.kv_heads) == attn_groups.end()) attn_groups.push_back(L.heads / L.kv_heads);
            // prompts and portions on the dense graph's flash kernel in its gated form (row-major value pages)
            w.flash = bf16 && L.dim == L.vdim && nvr::kb::flash_prefill_ok((int)L.dim, (int)L.heads, (int)L.kv_heads) && hv % 8 == 0;
            if (w.flash && std::find(flash_groups.begin(), flash_groups.end(), L.heads / L.kv_heads) == flash_groups.end()) flash_groups.push_back(L.heads / L.kv_heads);
            max_cat = std::max(max_cat, hv); max_ro = std::max(max_ro, tn); max_t4 = std::max(max_t4, 4 * tn); max_tn = std::max(max_tn, tn);
        } else return fail(NVR_ERR_UNSUPPORTED, "layer %zu: this mixer does not belong to the joint layout", i);
        RC(named(&w.mix, (size_t)(w.nmix * W * esz)));         // (freed by name with the model)
        if (L.ff_kind == LayeredSpec::FF_MOE_GLU) {
            const int64_t f = L.expert_ff, fs = L.shared_ff;
            RC(own(&w.router_op, (size_t)(pad16(L.experts + 1) * W * esz)));      // the router's rows, then the shared expert's gate, in the operand type (zero rows behind)
            RC(own(&w.egu, (size_t)(L.experts * 2 * f * W * esz))); RC(own(&w.edown, (size_t)(L.experts * W * f * esz)));
            if (fs) { RC(own(&w.sgu, (size_t)(2 * fs * W * esz))); RC(own(&w.sdown, (size_t)(W * fs * esz))); }
            max_fs = std::max(max_fs, fs); max_top = std::max(max_top, L.top); max_e2f = std::max(max_e2f, L.top * 2 * f); max_ef = std::max(max_ef, L.top * f);
            max_experts = std::max(max_experts, L.experts); max_f = std::max(max_f, f);
        } else if (L.has_mlp) return fail(NVR_ERR_UNSUPPORTED, "layer %zu: this feed-forward does not belong to the joint layout", i);
        max_nmix = std::max(max_nmix, w.nmix);
    }
    RC(named(&embed, (size_t)(V * W * esz))); RC(named(&head, (size_t)(V * W * esz))); RC(own(&wfinal, (size_t)W * 4));
    if (loops) { RC(own(&loop_in, (size_t)(W * 2 * W * esz))); RC(own(&pair, (size_t)(MT * 2 * W * esz))); if (bf16) RC(own(&lm_part, (size_t)(MT * ((W + 255) / 256) * 2) * 4)); }

    // pages for every run with attention; per slot the recurrent states and the rows before a step that the shifts and the convolution read
    size_t block_bytes = 0;
    for (int li : spec.runs) {
        const LayeredSpec::Layer &L = spec.layers[(size_t)li];
        if (L.mixer == LayeredSpec::ATTN_TMIX) block_bytes += (size_t)(r.block_size * L.kv_heads * (L.dim + L.vdim) * esz);
    }
    if (r.cfg.num_kvcache_blocks >= 0) r.num_blocks = r.cfg.num_kvcache_blocks;
    else if (r.cfg.num_kvcache_blocks == -1) r.num_blocks = 1000;
    else {
        size_t free_b = 0, total_b = 0;
        NVR_HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        const double act = (double)MT * (double)(12 * W + 2 * max_nmix + 2 * max_cat + 2 * max_ro + 2 * max_conv + 3 * max_t4 + 6 * max_e2f + 4 * max_fs) * 4.0;
        const double budget = (double)free_b - (1.0 - r.cfg.gpu_memory_utilization) * (double)total_b - act;
        const int64_t nb = block_bytes ? (int64_t)(budget * 0.9 / (double)block_bytes) : 1000;
        if (nb < 1) return fail(NVR_ERR_HIP, "not enough free HBM for one KV block");
        r.num_blocks = nb;
    }
    rs.resize(spec.runs.size());
    for (size_t ri = 0; ri < spec.runs.size(); ++ri) {
        const LayeredSpec::Layer &L = spec.layers[(size_t)spec.runs[ri]]; const LayerW &w = lw[(size_t)spec.runs[ri]]; RunState &st = rs[ri];
        RC(named((void **)&st.hist, (size_t)(2 * slots * W) * 4));
        if (L.mixer == LayeredSpec::SSM) {
            RC(named((void **)&st.state, (size_t)(slots * L.heads * L.dim * L.vdim) * 4));
            RC(own(&st.chist, (size_t)(2 * slots * std::max<int64_t>(L.conv_taps - 1, 1) * w.conv_c) * 4));
        } else {
            RC(named(&st.kc, (size_t)(r.num_blocks * r.block_size * L.kv_heads * L.dim * esz))); RC(named(&st.vc, (size_t)(r.num_blocks * r.block_size * L.kv_heads * L.vdim * esz)));
            RC(named((void **)&st.state, (size_t)(slots * L.t_heads * L.t_dim * L.t_dim) * 4));
            RC(own(&st.shist, (size_t)(2 * slots * W) * 4));
        }
    }

    // activations
    RC(named((void **)&x, (size_t)(MT * W * 4))); RC(own(&x0, (size_t)(MT * W * 4)));
    RC(named(&a1, (size_t)(MT * W * esz))); RC(named(&a2, (size_t)(MT * W * esz))); RC(named(&tmp, (size_t)(MT * W * esz))); RC(own(&tmp2, (size_t)(MT * W * esz)));
    RC(named(&proj, (size_t)(MT * max_nmix * esz))); RC(named(&cat, (size_t)(MT * max_cat * esz))); RC(named((void **)&ret_o, (size_t)(MT * max_ro * 4)));
    RC(own(&conv_o, (size_t)(MT * max_conv * esz))); RC(own(&tokg, (size_t)(MT * max_h * 2) * 4));
    RC(own(&mixes, (size_t)(MT * 5 * W * esz))); RC(own(&tproj, (size_t)(MT * max_t4 * esz))); RC(own(&tz, (size_t)(MT * max_tn * esz))); RC(own(&tcat, (size_t)(MT * max_tn * esz)));
    RC(named(&gu, (size_t)(MT * 2 * max_fs * esz))); RC(own(&act, (size_t)(MT * max_fs * esz))); RC(own(&shared_y, (size_t)(MT * W * esz))); RC(own(&shared_g, (size_t)MT * 4));
    const int64_t rows_e = MT * std::max<int64_t>(max_top, 1), pad_rows = (max_experts + 1) * 256;     // (experts' rows padded to whole blocks of 256)
    RC(own(&e_gu, (size_t)((MT * max_e2f + pad_rows * 2 * max_f) * esz))); RC(own(&e_act, (size_t)((MT * max_ef + pad_rows * max_f) * esz)));
    RC(own(&e_y, (size_t)((rows_e + pad_rows) * W * esz))); RC(own(&e_x, (size_t)((rows_e + pad_rows) * W * esz)));
    RC(own(&rlogits, (size_t)(MT * pad16(max_experts + 1)) * 4));
    RC(own(&moe_i, (size_t)(3 * rows_e + max_experts + 1 + rows_e / 256 + max_experts + 1024 + 8) * 4)); RC(own(&moe_score, (size_t)rows_e * 4));
    {   // the experts' inputs are the rows as they are: a scale of one per (token, choice)
        std::vector<float> one((size_t)std::max<int64_t>(rows_e, 1), 1.0f);
        RC(own(&gfloor, one.size() * 4)); NVR_HIP_CHECK(hipMemcpy(gfloor, one.data(), one.size() * 4, hipMemcpyHostToDevice));
    }
    return NVR_OK;
}

// Tensors by the names of the checkpoint: "embed", "head", "final.norm" [W], "loop.in" [W][2 W]; per layer i "l<i>.norm1" and "l<i>.shift" [W];
// state-space mixer "l<i>.mix.{in,conv,conv.b,dt_bias,A_log,D,norm,o}"; side by side "l<i>.mix.left.{q,k,v,g,o,pb,out}" and
// "l<i>.mix.right.{mu.r,mu.k,mu.v,mu.g,mu.w,r,k,v,g,w1,w2,w0,u,norm,o,out}"; experts "l<i>.mlp.{router,e<j>.{gate,up,down},shared.{gate,up,down,sg}}".  Linear weights are [out][in].
int LayeredModel::load_joint(nvr_model_runner &r, const std::string &name, int dtype, const int64_t *shape, int ndim, const void *data) {
    const int64_t W = spec.width, V = spec.vocab, nL = (int64_t)spec.layers.size();
    const char *name_in = name.c_str();
    auto is2 = [&](int64_t a, int64_t b) { return ndim == 2 && shape[0] == a && shape[1] == b; };
    auto bad = [&]() { return fail(NVR_ERR_LEN_MISMATCH, "load_tensor: '%s' has the wrong shape", name_in); };
    auto unknown = [&]() { return fail(NVR_ERR_UNSUPPORTED, "load_tensor: unknown tensor '%s'", name_in); };
    auto vec = [&](float *dst, int64_t n) { return (dst && ndim == 1 && shape[0] == n) ? put(r, dst, n, 1, n, dtype, data, false) : bad(); };
    auto mat = [&](void *dst, int64_t ld, int64_t rows, int64_t cols) { return (dst && is2(rows, cols)) ? put(r, dst, ld, rows, cols, dtype, data, true) : bad(); };
    auto fmat = [&](float *dst, int64_t rows, int64_t cols) { return (dst && is2(rows, cols)) ? put(r, dst, cols, rows, cols, dtype, data, false) : bad(); };
    auto rows_at = [&](void *base, int64_t row0, int64_t ld) { return (void *)((char *)base + (size_t)(row0 * ld * esz)); };
    // the decay's low-rank pair in 16 bits is kept with its rank padded by zero rows / columns to whole 256-column tiles: a product with 64 columns over many rows
    // leaves most of the chip idle, the padded one takes the 256 x 256 tiles (tanh(0) = 0 keeps the padding out of the second product)
    auto rank_rows = [&](int64_t rank) { return (bf16 && W % 32 == 0) ? (rank + 255) / 256 * 256 : rank; };
    if (name == "embed") return mat(embed, W, V, W);
    if (name == "head") return mat(head, W, V, W);
    if (name == "final.norm") return vec(wfinal, W);
    if (name == "loop.in") return loop_in ? mat(loop_in, 2 * W, W, 2 * W) : unknown();
    size_t dot = name.find('.');
    if (name.size() < 3 || name[0] != 'l' || dot == std::string::npos || dot < 2) return unknown();
    int64_t li = 0;
    for (size_t i = 1; i < dot; ++i) { if (name[i] < '0' || name[i] > '9') return unknown(); li = li * 10 + (name[i] - '0'); }
    if (li >= nL) return fail(NVR_ERR_UNSUPPORTED, "load_tensor: '%s' names a layer the model does not have", name_in);
    const LayeredSpec::Layer &L = spec.layers[(size_t)li]; LayerW &w = lw[(size_t)li];
    const std::string rest = name.substr(dot + 1);
    if (rest == "norm1") return vec(w.n1, W);
    if (rest == "shift") return vec(w.shift, W);
    if (L.mixer == LayeredSpec::SSM) {
        const int64_t inner = L.heads * L.vdim;
        if (rest == "mix.in") return mat(w.mix, W, w.dtcol + L.heads, W);
        if (rest == "mix.conv") return fmat(w.convw, w.conv_c, L.conv_taps);
        if (rest == "mix.conv.b") return vec(w.convb, w.conv_c);
        if (rest == "mix.dt_bias") return vec(w.dtb, L.heads);
        if (rest == "mix.A_log") return vec(w.alog, L.heads);
        if (rest == "mix.D") return vec(w.skip, L.heads);
        if (rest == "mix.norm") return vec(w.hnorm, inner);
        if (rest == "mix.o") return mat(w.wo, inner, W, inner);
    } else {
        const int64_t hd = L.heads * L.dim, kn = L.kv_heads * L.dim, vn = L.kv_heads * L.vdim, hv = L.heads * L.vdim, tn = L.t_heads * L.t_dim;
        if (rest == "mix.left.q") return mat(rows_at(w.mix, w.qcol, W), W, hd, W);
        if (rest == "mix.left.k") return mat(rows_at(w.mix, w.kcol, W), W, kn, W);
        if (rest == "mix.left.v") return mat(rows_at(w.mix, w.vcol, W), W, vn, W);
        if (rest == "mix.left.g") return mat(rows_at(w.mix, w.gcol, W), W, hv, W);
        if (rest == "mix.left.o") return mat(w.wo, hv, W, hv);
        if (rest == "mix.left.pb") return vec(w.pb, L.heads);
        if (rest == "mix.left.out") return vec(w.outl, W);
        if (rest == "mix.right.out") return vec(w.outr, W);
        static const char *const kMix[5] = {"mix.right.mu.r", "mix.right.mu.k", "mix.right.mu.v", "mix.right.mu.g", "mix.right.mu.w"};
        for (int k = 0; k < 5; ++k) if (rest == kMix[k]) return vec(w.mu + k * W, W);
        static const char *const kProj[4] = {"mix.right.r", "mix.right.k", "mix.right.v", "mix.right.g"};
        for (int k = 0; k < 4; ++k) if (rest == kProj[k]) return mat(rows_at(w.w4, k * tn, W), W, tn, W);
        if (rest == "mix.right.w0") return vec(w.w0, tn);
        if (rest == "mix.right.norm") return vec(w.tnorm, tn);
        if (rest == "mix.right.u") return is2(L.t_heads, L.t_dim) ? put(r, w.bonus, L.t_dim, L.t_heads, L.t_dim, dtype, data, false) : bad();
        if (rest == "mix.right.o") return mat(w.wo2, tn, W, tn);
        if (rest == "mix.right.w1") {                       // the rank of the decay projection is the tensor's
            if (ndim != 2 || shape[1] != W || shape[0] < 1 || (w.t_rank && w.t_rank != shape[0])) return bad();
            w.t_rank = shape[0];
            const int64_t rp = rank_rows(w.t_rank);
            if (!w.w1) RC(own(&w.w1, (size_t)(rp * W * esz)));
            if (rp > tlow_cap) { RC(own(&tlow, (size_t)(r.max_tokens * rp * esz))); tlow_cap = rp; }   // (a smaller one before it stays owned)
            return put(r, w.w1, W, w.t_rank, W, dtype, data, true);
        }
        if (rest == "mix.right.w2") {
            if (ndim != 2 || shape[0] != tn || shape[1] < 1 || (w.t_rank && w.t_rank != shape[1])) return bad();
            w.t_rank = shape[1];
            if (!w.w2) RC(own(&w.w2, (size_t)(tn * rank_rows(w.t_rank) * esz)));
            return put(r, w.w2, rank_rows(w.t_rank), tn, w.t_rank, dtype, data, true);
        }
    }
    if (L.ff_kind == LayeredSpec::FF_MOE_GLU) {
        const int64_t f = L.expert_ff, fs = L.shared_ff;
        if (rest == "mlp.router") return mat(w.router_op, W, L.experts, W);
        if (fs && rest == "mlp.shared.sg") return mat(rows_at(w.router_op, L.experts, W), W, 1, W);
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

int LayeredModel::forward_joint(nvr_model_runner &r, const StepPlan &p) {
    const kl::Batch &b = p.b;
    const int64_t T = p.T, R = p.R, W = spec.width, nR = (int64_t)spec.runs.size(), MT = r.max_tokens;
    const float eps = (float)spec.eps;
    hipStream_t s = r.stream;
    auto at = [&](void *base, int64_t col) { return (void *)((char *)base + (size_t)(col * esz)); };
    RC(kl::embed_keep(embed, bf16, b.ids, T, W, x, loop_in ? x0 : nullptr, s));
    for (int64_t ri = 0; ri < nR; ++ri) {
        const size_t li = (size_t)spec.runs[(size_t)ri];
        const LayeredSpec::Layer &L = spec.layers[li]; const LayerW &w = lw[li]; RunState &st = rs[(size_t)ri];
        if (spec.pass_start[(size_t)ri]) {                   // a pass over the looped range starts from the stream and the embedding output together
            RC(kl::pair_rows(x, x0, T, W, pair, bf16, s));
            if (bf16 && lm_part && nvr::kb::gemm256_lm_head_ok(T, 2 * W, W, 2 * W)) {       // many rows: the 256 x 256 product that leaves in f32 (the LM head's; its arg-max partials are not read)
                int32_t nparts = 0;
                RC(nvr::kb::gemm256_lm_head((const uint16_t *)pair, 2 * W, (const uint16_t *)loop_in, T, 2 * W, W, x, lm_part, (int32_t *)(lm_part + MT * ((W + 255) / 256)), &nparts, s));
            } else
                RC(gemm(r, pair, 2 * W, loop_in, T, 2 * W, W, x, true));
        }
        RC(kl::norm_shift(x, b, W, eps, w.n1, w.shift, L.has_mlp ? a2 : nullptr, a1, st.hist, slots, bf16, s));
        RC(gemm(r, a1, W, w.mix, T, W, w.nmix, proj));
        kl::JoinArgs j{}; j.x = x; j.T = T; j.W = W; j.eps = eps; j.y1 = tmp; j.ld1 = W;
        if (L.mixer == LayeredSpec::SSM) {
            const int64_t inner = L.heads * L.vdim, gn = L.kv_heads * L.dim;
            kl::ConvGateArgs c{}; c.proj = proj; c.ld = w.nmix; c.ccol = w.ccol; c.dcol = w.dtcol; c.C = (int32_t)w.conv_c; c.taps = (int32_t)L.conv_taps; c.H = (int32_t)L.heads;
            c.w = w.convw; c.bias = w.convb; c.dt_bias = w.dtb; c.a_log = w.alog; c.hist = st.chist; c.slots = slots; c.out = conv_o; c.ldo = w.conv_c; c.tok_gate = tokg;
            RC(kl::conv_gates(c, b, bf16, s));
            // the recurrence is retention's token-gated form: keys the input maps B, queries the output maps C (both shared by the heads of a group), values the channels x
            kl::RetentionArgs a{};
            a.proj = conv_o; a.ld = w.conv_c; a.qcol = inner + gn; a.kcol = inner; a.vcol = 0; a.rot_dims = 0; a.kscale = 1.0f; a.qscale = 1.0f; a.inv_tau = 1.f;
            a.H = (int32_t)L.heads; a.D = (int32_t)L.dim; a.Dv = (int32_t)L.vdim; a.tok_gate = tokg; a.qk_share = (int32_t)(L.heads / L.kv_heads); a.state = st.state; a.o = ret_o;
            RC(kl::retention(a, b, bf16, s));
            kl::StateReadoutArgs ro{}; ro.o = ret_o; ro.xs = conv_o; ro.ldx = w.conv_c; ro.z = proj; ro.ldz = w.nmix; ro.skip = w.skip; ro.w = w.hnorm;
            ro.T = (int32_t)T; ro.H = (int32_t)L.heads; ro.Dv = (int32_t)L.vdim; ro.groups = (int32_t)L.mix_norm_groups; ro.eps = eps; ro.out = cat; ro.ldo = inner;
            RC(kl::state_readout(ro, bf16, s));
            RC(gemm(r, cat, inner, w.wo, T, inner, W, tmp));
        } else {
            const int64_t hv = L.heads * L.vdim, tn = L.t_heads * L.t_dim;
            if (!w.w1 || !w.w2) return fail(NVR_ERR_NOT_ALLOCATED, "layer %zu: the decay projections were not loaded", li);
            // left: attention over the chunk's keys with sigmoid weights
            kl::SinkAttnArgs a{};
            a.q = at(proj, w.qcol); a.ldq = w.nmix; a.kc = st.kc; a.vc = st.vc; a.chunk = (int32_t)L.chunk; a.softcap = (float)L.softcap; a.gate_bias = w.pb;
            a.H = (int32_t)L.heads; a.G = (int32_t)L.kv_heads; a.D = (int32_t)L.dim; a.Dv = (int32_t)L.vdim; a.scale = (float)L.scale; a.out = cat; a.ldo = hv;
            a.v_grouped = w.flash ? 0 : 1;                                           // (a property of the layer: the pages keep one layout)
            const bool tiled = kl::sink_attention_tiled_ok(a, bf16, (int)r.block_size);       // (a property of the layer's shape: the pages keep one layout)
            kl::RopeStoreArgs ra{}; ra.proj = proj; ra.ld = w.nmix; ra.qcol = w.qcol; ra.kcol = w.kcol; ra.vcol = w.vcol; ra.H = a.H; ra.G = a.G; ra.D = a.D; ra.Dv = a.Dv;
            ra.rot = (int32_t)L.rot_dims; ra.freq = w.rfreq; ra.kc = st.kc; ra.vc = st.vc; ra.v_grouped = tiled && !w.flash;
            RC(kl::rope_store(ra, b, bf16, s));
            if (w.flash && !p.decode_sized) {
                const size_t gi = (size_t)(std::find(flash_groups.begin(), flash_groups.end(), L.heads / L.kv_heads) - flash_groups.begin());
                nvr::kt::FlashArgs f{};
                f.q = (const uint16_t *)a.q; f.ldq = w.nmix; f.k = (const uint16_t *)st.kc; f.v = (const uint16_t *)st.vc; f.ldkv = 0;
                f.block_tables = b.block_tables; f.max_blocks = b.max_blocks; f.block_size = b.block_size;
                f.tiles = (const nvr::kt::FlashTile *)(in_dev + p.o_ftiles[gi]); f.ntiles = p.n_ftiles[gi];
                f.H = (int32_t)L.heads; f.KVH = (int32_t)L.kv_heads; f.D = (int32_t)L.dim; f.scale = (float)L.scale; f.out = (uint16_t *)cat; f.ldo = hv;
                f.gate_bias = w.pb; f.softcap = (float)L.softcap; f.chunk = (int32_t)L.chunk;
                RC(nvr::kb::flash_prefill(f, true, s));
            } else if (tiled) {
                const size_t gi = (size_t)(std::find(attn_groups.begin(), attn_groups.end(), L.heads / L.kv_heads) - attn_groups.begin());
                // decode-sized steps over long chunks: few tiles, many keys each — a tile's keys go to several workgroups whose partial sums are added up
                const int64_t wgs = (int64_t)p.n_tiles[gi] * L.kv_heads, keys = L.chunk > 0 ? std::min<int64_t>(p.max_ctx, L.chunk + 64) : p.max_ctx;
                int64_t nsplit = 1;
                if (wgs < r.num_cus && keys >= 512) nsplit = std::max<int64_t>(1, std::min<int64_t>({(2 * r.num_cus) / wgs, (keys + 255) / 256, 16}));
                RC(kl::sink_attention_tiled(a, b, (const kl::AttnTile *)(in_dev + p.o_tiles[gi]), p.n_tiles[gi], (int)nsplit, attn_ws, attn_ws_bytes, s));
            } else
                RC(kl::sink_attention(a, b, bf16, s));
            RC(kl::sigmoid_gate(cat, hv, at(proj, w.gcol), w.nmix, T, hv, bf16, s));
            RC(gemm(r, cat, hv, w.wo, T, hv, W, tmp));
            // right: five shifted inputs, their projections (one matrix per input), the decay's two products, retention's gated form with a bonus
            RC(kl::shift_mixes(a1, W, b, W, 5, w.mu, mixes, st.shist, slots, bf16, s));
            // r, k, v, g leave in planes of [max tokens][Ht Dt] each: many rows take the tiled product once per plane, few rows one launch with a matrix per plane
            const int64_t plane = MT * tn;
            if (T >= 128) {
                for (int k = 0; k < 4; ++k) RC(gemm(r, at(mixes, k * W), 5 * W, at(w.w4, k * tn * W), T, W, tn, at(tproj, k * plane)));
            } else {
                kl::HeadLinearArgs ha{}; ha.a = mixes; ha.lda = 5 * W; ha.ha = W; ha.w = w.w4; ha.y = tproj; ha.ldy = tn; ha.hy = plane; ha.T = (int32_t)T; ha.H = 4; ha.K = (int32_t)W; ha.N = (int32_t)tn;
                RC(kl::head_linear(ha, bf16, s));
            }
            const int64_t rp = (bf16 && W % 32 == 0) ? (w.t_rank + 255) / 256 * 256 : w.t_rank;       // (the rank as load_joint padded it)
            RC(gemm(r, at(mixes, 4 * W), 5 * W, w.w1, T, W, rp, tlow));
            RC(kl::tanh_rows(tlow, rp, T, rp, bf16, s));
            RC(gemm(r, tlow, rp, w.w2, T, rp, tn, tz));
            kl::RetentionArgs t{};
            t.proj = tproj; t.ld = tn; t.qcol = 0; t.kcol = plane; t.vcol = 2 * plane; t.rot_dims = 0; t.kscale = 1.0f; t.qscale = 1.0f; t.inv_tau = 1.f;
            t.H = (int32_t)L.t_heads; t.D = (int32_t)L.t_dim; t.Dv = (int32_t)L.t_dim; t.az = tz; t.ldz = tn; t.abias = w.w0; t.decay_exp = true; t.bonus = w.bonus;
            t.state = st.state; t.o = ret_o;
            RC(kl::retention(t, b, bf16, s));
            RC(kl::head_norm_gate(ret_o, tproj, tn, 3 * plane, T, L.t_heads, L.t_dim, eps, w.tnorm, tcat, tn, bf16, s, true));
            RC(gemm(r, tcat, tn, w.wo2, T, tn, W, tmp2));
            j.w1 = w.outl; j.y2 = tmp2; j.ld2 = W; j.w2 = w.outr;
        }
        if (L.ff_kind == LayeredSpec::FF_MOE_GLU) {
            const int64_t f = L.expert_ff, fs = L.shared_ff, n = T * L.top;
            int32_t *sel = moe_i, *order = sel + MT * L.top, *place_of = order + MT * L.top, *off = place_of + MT * L.top, *row_w = off + L.experts + 1;
            // many rows: every expert's rows padded to whole blocks of 256, brought together once, and the dense graph's 256 x 256 product with a matrix per row block
            const int64_t nblocks = n / 256 + L.experts;
            const bool blocks = bf16 && n >= 2048 && nvr::kb::gemm256_ok(nblocks * 256, W, 2 * f, W) && nvr::kb::gemm256_ok(nblocks * 256, f, W, f);
            // router logits (and the shared expert's gate): one product with f32 accumulation that leaves in f32, then the choice per token
            const int64_t ne = pad16(L.experts + 1);
            RC(gemm(r, a2, W, w.router_op, T, W, ne, rlogits, true));
            RC(kl::moe_route(a2, W, T, W, nullptr, L.experts, L.top, sel, moe_score, off, order, place_of, blocks ? 256 : 1, blocks ? row_w : nullptr, nblocks, bf16, s,
                             true, fs ? 1 : 0, fs ? shared_g : nullptr, rlogits, ne));
            if (blocks) {
                RC(kl::moe_gather(a2, W, T, W, L.top, place_of, gfloor, e_x, bf16, s));
                RC(nvr::kb::gemm256_grouped((const uint16_t *)e_x, W, (const uint16_t *)w.egu, 2 * f * W, row_w, nblocks * 256, W, 2 * f, (uint16_t *)e_gu, s));
                RC(kl::clamped_glu(e_gu, nblocks * 256, f, (float)L.limit, 1.702f, e_act, f, bf16, s));
                RC(nvr::kb::gemm256_grouped((const uint16_t *)e_act, f, (const uint16_t *)w.edown, W * f, row_w, nblocks * 256, f, W, (uint16_t *)e_y, s));
            } else {
                kl::GroupedLinearArgs g{}; g.a = a2; g.lda = W; g.w = w.egu; g.y = e_gu; g.ldy = 2 * f; g.off = off; g.groups = (int32_t)L.experts; g.K = (int32_t)W; g.N = (int32_t)(2 * f);
                g.max_rows = (int32_t)n; g.src = order; g.rscale = gfloor; g.src_div = (int32_t)L.top;
                RC(kl::grouped_linear(g, bf16, s));
                RC(kl::clamped_glu(e_gu, n, f, (float)L.limit, 1.702f, e_act, f, bf16, s));
                kl::GroupedLinearArgs d{}; d.a = e_act; d.lda = f; d.w = w.edown; d.y = e_y; d.ldy = W; d.off = off; d.groups = (int32_t)L.experts; d.K = (int32_t)f; d.N = (int32_t)W; d.max_rows = (int32_t)n;
                RC(kl::grouped_linear(d, bf16, s));
            }
            if (fs) {
                RC(gemm(r, a2, W, w.sgu, T, W, 2 * fs, gu));
                RC(kl::clamped_glu(gu, T, fs, (float)L.shared_limit, 1.702f, act, fs, bf16, s));
                RC(gemm(r, act, fs, w.sdown, T, fs, W, shared_y));
            }
            RC(kl::moe_combine(e_y, place_of, T, L.top, fs ? shared_y : nullptr, W, a2, bf16, s, moe_score, fs ? shared_g : nullptr, 1));
            j.add = a2; j.lda = W;
        }
        RC(kl::residual_join(j, bf16, s));
    }
    kl::GroupNormArgs n{}; n.in = x; n.ldi = W; n.in_f32 = true; n.rows = p.d_want; n.rows_n = R; n.W = W; n.groups = 1; n.eps = eps; n.w = wfinal; n.out = xsel; n.ldo = W;
    RC(kl::group_norm(n, bf16, s));
    return gemm(r, xsel, W, head, R, W, spec.vocab, r.logits, true);
}

}  // namespace nvr
