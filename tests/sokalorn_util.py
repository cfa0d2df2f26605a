"""Helpers of the Sokalorn tests: small configurations, random tensors by the checkpoint's names (float32 on the bfloat16 grid), token sequences whose
router decisions are no close calls, and weights turned so that one key decides a row.  The expected values come from tests/sokalorn_reference.py."""
import numpy as np

import sokalorn_reference as ref
from rugudra_util import bf16_round


def moe(experts=6, top=2, ff=24, limit=1.25, shared=40, shared_limit=2.0):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared, "limit": shared_limit}
    return m


def ssm_layer(heads=4, vdim=16, state=24, groups=2, conv=4, norm_groups=2, mlp="default"):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups},
            "mlp": moe() if mlp == "default" else mlp}


def side_layer(heads=4, kv_heads=2, dim=16, vdim=24, chunk=12, scale=None, softcap=15.0, rot=8, base=100.0, factor=2.0, t_heads=2, t_dim=16, mlp="default"):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": chunk}, "scale": scale if scale is not None else dim ** -0.5,
                               "softcap": softcap, "rot": {"dims": rot, "base": base, "scaling": {"factor": factor}}},
                      "right": {"heads": t_heads, "dim": t_dim}},
            "mlp": moe() if mlp == "default" else mlp}


def make_config(layers, vocab=83, width=64, loop=None, eps=1e-5):
    cfg = {"architecture": "Sokalorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


ROUTED = 8      # the routers read the first channels only, where the embeddings are large: see make_weights


def make_weights(cfg, seed=0, t_rank=6):
    """Random tensors.  The first ROUTED channels of the embeddings are large, everything that writes into the residual stream writes little into them, and the
    routers read only these channels: a router's decision is then (nearly) a property of the token — the order of its logits does not change with the norm's
    scale —, 16-bit noise hardly reaches it, and tokens can be drawn so that no decision is a close call (settled_tokens)."""
    rng = np.random.default_rng(seed)
    W, V = cfg["width"], cfg["vocab"]
    quiet = np.ones(W); quiet[:ROUTED] = 0.02

    def lin(o, i, g=1.0):
        return bf16_round(rng.standard_normal((o, i)) * (g / np.sqrt(i)))

    def out(i):                                             # a projection into the residual stream
        return bf16_round(rng.standard_normal((W, i)) * (1.0 / np.sqrt(i)) * quiet[:, None])

    def gains(n, spread=0.2):
        return bf16_round(1.0 + spread * rng.standard_normal(n))
    emb = rng.standard_normal((V, W)); emb[:, :ROUTED] *= 4.0
    w = {"embed": bf16_round(emb), "head": lin(V, W), "final.norm": gains(W)}
    if cfg.get("loop") is not None:
        li = rng.standard_normal((W, 2 * W)) * (0.7 / np.sqrt(W))
        li[:ROUTED] = 0.0
        for c in range(ROUTED):
            li[c, c], li[c, W + c] = 1.0, 0.5
        w["loop.in"] = bf16_round(li)
    for i, L in enumerate(cfg["layers"]):
        p, m = "l%d." % i, L["mixer"]
        w[p + "norm1"], w[p + "shift"] = gains(W), bf16_round(rng.uniform(0.0, 1.0, W))
        if L["type"] == "mamba2":
            H, P, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            C = H * P + 2 * G * N
            w[p + "mix.in"] = lin(2 * H * P + 2 * G * N + H, W, 1.5)
            w[p + "mix.conv"], w[p + "mix.conv.b"] = bf16_round(rng.standard_normal((C, taps)) * 0.5), bf16_round(0.2 * rng.standard_normal(C))
            w[p + "mix.dt_bias"], w[p + "mix.A_log"] = bf16_round(rng.uniform(-3.0, 0.5, H)), bf16_round(rng.uniform(-1.5, 1.0, H))
            w[p + "mix.D"], w[p + "mix.norm"], w[p + "mix.o"] = bf16_round(rng.standard_normal(H)), gains(H * P), out(H * P)
        else:
            a, t = m["left"], m["right"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            w[q + "q"], w[q + "k"], w[q + "v"], w[q + "g"], w[q + "o"] = lin(H * D, W, 2.0), lin(G * D, W, 2.0), lin(G * Dv, W), lin(H * Dv, W), lin(W, H * Dv)
            w[q + "pb"], w[q + "out"] = bf16_round(rng.uniform(-3.0, 0.0, H)), bf16_round(gains(W) * quiet)
            q, tn = p + "mix.right.", t["heads"] * t["dim"]
            for s in "rkvgw":
                w[q + "mu." + s] = bf16_round(rng.uniform(0.0, 1.0, W))
            w[q + "r"], w[q + "k"], w[q + "v"], w[q + "g"], w[q + "o"] = lin(tn, W), lin(tn, W), lin(tn, W), lin(tn, W), lin(W, tn)
            w[q + "w1"], w[q + "w2"], w[q + "w0"] = lin(t_rank, W), lin(tn, t_rank, 2.0), bf16_round(rng.uniform(-4.0, 0.5, tn))
            w[q + "u"], w[q + "norm"], w[q + "out"] = bf16_round(0.5 * rng.standard_normal((t["heads"], t["dim"]))), gains(tn), bf16_round(gains(W) * quiet)
        mlp = L.get("mlp")
        if mlp:
            E = mlp["router"]["experts"]
            rt = np.zeros((E, W)); rt[:, :ROUTED] = rng.standard_normal((E, ROUTED)) * 0.6
            w[p + "mlp.router"] = bf16_round(rt)
            for n in ["e%d" % e for e in range(E)] + (["shared"] if mlp.get("shared") else []):
                fe = mlp["shared"]["ff"] if n == "shared" else mlp["expert"]["ff"]
                w[p + "mlp.%s.gate" % n], w[p + "mlp.%s.up" % n], w[p + "mlp.%s.down" % n] = lin(fe, W, 2.0), lin(fe, W, 2.0), out(fe)
            if mlp.get("shared"):
                w[p + "mlp.shared.sg"] = lin(1, W, 2.0)
    return w


def as64(weights):
    return {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}


def expected_logits(cfg, weights, tokens):
    return ref.forward(cfg, as64(weights), list(tokens))[0]


def settled_tokens(cfg, w, n, seed, gap=0.05, lo=0):
    """n random tokens for which every router decision of the restatement has a gap of at least `gap` between the last chosen and the first rejected logit (a
    bfloat16 engine may otherwise choose another expert than the float64 restatement: no comparison should rest on such a call)."""
    V, w64 = cfg["vocab"], as64(w)
    for k in range(200):
        toks, m = np.random.default_rng(seed + 1000 * k).integers(lo, V, n).tolist(), []
        ref.forward(cfg, w64, toks, margins=m)
        if not m or min(m) > gap:
            return toks
        # drop the tokens whose own decisions are close and draw again among the rest
        per = np.asarray(m).reshape(-1, n).min(axis=0)
        good = sorted({t for t, g in zip(toks, per) if g > 2 * gap})
        if len(good) >= max(4, V // 6):
            for k2 in range(50):
                toks, m = [good[j] for j in np.random.default_rng(seed + 7 * k + k2).integers(0, len(good), n)], []
                ref.forward(cfg, w64, toks, margins=m)
                if min(m) > gap:
                    return toks
    raise AssertionError("no token sequence with settled router decisions")


def make_key_stand_out(cfg, w, qtok, ktok, amount=40.0, bias=-12.0, seed=77):
    """Layer 0 (attention beside time mixing, made without a token shift so that its input is a property of the token; a vocabulary no larger than the width): the
    query and key projections are replaced so that only token qtok has queries and only token ktok has keys to speak of (each projection reads the one direction of
    the input space that is 1 on its token and 0 on every other token), both along the same unrotated direction per key/value head, with a raw score of `amount` —
    the cap's height after the cap —, and the bias of every head is so low that every other pair's weight is next to nothing.  Inside its chunk that one key decides
    the row."""
    a = cfg["layers"][0]["mixer"]["left"]
    H, G, D, R, eps = a["heads"], a["kv_heads"], a["dim"], a["rot"]["dims"], cfg["norm"]["eps"]
    assert cfg["vocab"] <= cfg["width"] and R < D
    out = dict(w)
    out["l0.shift"] = np.zeros_like(w["l0.shift"])
    w64 = as64(out)
    h = ref.rms(w64["embed"], eps) * w64["l0.norm1"]        # [vocab, W]: the layer's input for every token
    pick = np.linalg.pinv(h)                                # [W, vocab]: column t is 1 on token t's input and 0 on the others'
    d = np.random.default_rng(seed).standard_normal((G, D)); d[:, :R] = 0.0
    want_k = d.reshape(-1)
    want_q = np.concatenate([d[hd // (H // G)] * amount / (a["scale"] * (d[hd // (H // G)] @ d[hd // (H // G)])) for hd in range(H)])
    out["l0.mix.left.k"] = bf16_round(0.02 * w64["l0.mix.left.k"] + np.outer(want_k, pick[:, ktok]))
    out["l0.mix.left.q"] = bf16_round(0.02 * w64["l0.mix.left.q"] + np.outer(want_q, pick[:, qtok]))
    out["l0.mix.left.pb"] = np.full_like(w["l0.mix.left.pb"], bias)
    return out
