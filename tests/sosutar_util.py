"""Helpers of the Sosutar tests: small configurations, random tensors by the checkpoint's names (float32 on the bfloat16 grid), and weights turned so that
one key decides a row.  The expected values come from tests/sosutar_reference.py."""
import numpy as np

import sosutar_reference as ref
from rugudra_util import bf16_round


def mlstm_layer(heads=2, dim=16, vdim=24, gate_cap=10.0, ff=None, weights_of=None):
    L = {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def side_layer(heads=4, kv_heads=2, dim=16, vdim=16, window=12, scale=None, coef=0.25, every=16, gru=40, ff=48, weights_of=None):
    L = {"type": "parallel",
         "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window}, "q_temp": {"coef": coef, "every": every},
                            "scale": scale if scale is not None else dim ** -0.5},
                   "right": {"width": gru}},
         "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def make_config(layers, vocab=83, width=64, max_positions=512, embedding_scale=3.0, logit_scale=0.5, eps=1e-5):
    return {"architecture": "Sosutar", "vocab": vocab, "width": width, "max_positions": max_positions, "embedding": {"scale": embedding_scale}, "logit_scale": logit_scale,
            "norm": {"eps": eps}, "layers": layers}


def make_weights(cfg, seed=0, pos_gain=1.0):
    rng = np.random.default_rng(seed)
    W, V = cfg["width"], cfg["vocab"]

    def lin(o, i, g=1.0):
        return bf16_round(rng.standard_normal((o, i)) * (g / np.sqrt(i)))

    def gains(n, spread=0.2):
        return bf16_round(1.0 + spread * rng.standard_normal(n))
    w = {"embed": bf16_round(rng.standard_normal((V, W))), "pos": bf16_round(pos_gain * rng.standard_normal((cfg["max_positions"], W))), "head": lin(V, W),
         "final.norm": gains(W)}
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        p, m = "l%d." % i, L["mixer"]
        w[p + "norm1"], w[p + "ls1"] = gains(W), bf16_round(0.6 + 0.2 * rng.standard_normal(W))
        if L["type"] == "mlstm":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"], w[p + "mix.g"] = lin(H * D, W), lin(H * D, W), lin(H * Dv, W), lin(H * Dv, W)
            w[p + "mix.o"], w[p + "mix.norm"] = lin(W, H * Dv), gains(H * Dv)
            w[p + "mix.i"], w[p + "mix.f"] = lin(H, W, 2.0), lin(H, W, 2.0)
            w[p + "mix.i.b"], w[p + "mix.f.b"] = bf16_round(rng.standard_normal(H)), bf16_round(2.0 + rng.standard_normal(H))
        else:
            a, g = m["left"], m["right"]["width"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            w[q + "q"], w[q + "k"], w[q + "v"], w[q + "g"], w[q + "o"] = lin(H * D, W), lin(G * D, W), lin(G * Dv, W), lin(H * Dv, W), lin(W, H * Dv)
            w[q + "q.norm"], w[q + "k.norm"], w[q + "sink"], w[q + "out"] = gains(H * D), gains(G * D), bf16_round(rng.standard_normal(H)), gains(W)
            q = p + "mix.right."
            w[q + "z"], w[q + "x"], w[q + "g"], w[q + "o"] = lin(g, W), lin(g, W), lin(g, W), lin(W, g)
            w[q + "z.b"], w[q + "x.b"], w[q + "out"] = bf16_round(rng.standard_normal(g)), bf16_round(0.5 * rng.standard_normal(g)), gains(W)
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            w[p + "norm2"], w[p + "ls2"] = gains(W), bf16_round(0.6 + 0.2 * rng.standard_normal(W))
            w[p + "mlp.up"], w[p + "mlp.down"] = lin(F, W, 1.5), lin(W, F)
    return w


def make_key_stand_out(cfg, w, qtok, ktok):
    """Layer 0 (attention beside the recurrence; weights made with pos_gain 0, so the layer's input is a property of the token): the query projection is
    replaced so that token qtok's normed queries lie along token ktok's normed keys in every head.  With a score scale of about 12 / dim that pair's score
    exceeds every other by far."""
    a = cfg["layers"][0]["mixer"]["left"]
    H, G, D, eps = a["heads"], a["kv_heads"], a["dim"], cfg["norm"]["eps"]
    w64 = {k: np.asarray(v, np.float64) for k, v in w.items()}
    h = ref.rms(w64["embed"][[qtok, ktok]] * cfg["embedding"]["scale"], eps) * w64["l0.norm1"]
    k = (ref.rms(h[1:] @ w64["l0.mix.left.k"].T, eps) * w64["l0.mix.left.k.norm"]).reshape(G, D)
    want_q = np.concatenate([k[hd // (H // G)] for hd in range(H)]) / w64["l0.mix.left.q.norm"]
    wq = 0.05 * w64["l0.mix.left.q"] + np.outer(want_q, h[0]) / (h[0] @ h[0])
    out = dict(w)
    out["l0.mix.left.q"] = bf16_round(wq)
    return out


def expected_logits(cfg, weights, tokens):
    w64 = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
    return ref.forward(cfg, w64, list(tokens))[0]
