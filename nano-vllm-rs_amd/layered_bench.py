"""Prefill and decode throughput of the layer-list designs (Rugudra, Pusunex, Sosutar, Sokalorn) beside the dense Qwen3 graph at equal sizes (bench.py --layered-compare).

Random weights, layer shapes that resemble a real model's; both models go through the same engine (scheduler, block manager, runner step).
Per size one JSON object: tokens/s of one prefill step over BATCH prompts of PROMPT tokens and of the decode steps that follow, for both."""
import json
import time

import numpy as np

SIZES = {
    # width, ff, heads, kv_heads, head size, layers (alternating attention / retention for the layer-list model), vocab
    "w1024": dict(width=1024, ff=3072, heads=16, kv_heads=8, dim=128, layers=4, vocab=32768),
    "w2048": dict(width=2048, ff=6144, heads=16, kv_heads=8, dim=128, layers=4, vocab=32768),
    "w4096": dict(width=4096, ff=12288, heads=32, kv_heads=8, dim=128, layers=2, vocab=32768),
}


def rugudra_config(s, loop=False):
    layers = []
    for i in range(s["layers"]):
        if i % 2 == 0:
            layers.append({"type": "attention", "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["dim"], "scale": s["dim"] ** -0.5},
                           "mlp": {"kind": "dense", "ff": s["ff"], "limit": 7.0}})
        else:
            h = s["heads"]
            layers.append({"type": "retention", "mixer": {"heads": h, "dim": s["dim"], "vdim": s["dim"], "decay": [1.0 - 2.0 ** (-5 - 3 * j / max(1, h - 1)) for j in range(h)],
                                                          "rot": {"dims": s["dim"], "base": 10000.0}},
                           "mlp": {"kind": "dense", "ff": s["ff"], "limit": 7.0}})
    cfg = {"architecture": "Rugudra", "vocab": s["vocab"], "width": s["width"], "residual_mult": 0.5, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5},
           "canon": {"taps": 4}, "layers": layers}
    if loop:
        cfg["loop"] = {"start": 0, "stop": len(layers), "times": 2}
    return cfg


def random_weights(cfg, seed=0):
    """Tensors of a Rugudra configuration with values of a size that keeps activations in range (f32 arrays by name)."""
    rng = np.random.default_rng(seed)
    W, V, taps = cfg["width"], cfg["vocab"], cfg["canon"]["taps"]

    def lin(o, i):
        return (rng.standard_normal((o, i), dtype=np.float32) * (1.0 / np.sqrt(i))).astype(np.float32)
    out = {"embed": rng.standard_normal((V, W), dtype=np.float32), "head": lin(V, W), "final.norm": np.float32(1.0)}
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], "l%d." % i
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        G = m.get("kv_heads", H)
        out[p + "norm1"] = np.float32(1.0 + 0.1 * rng.standard_normal())
        out[p + "norm2"] = np.float32(1.0 + 0.1 * rng.standard_normal())
        out[p + "canon1"] = (0.2 * rng.standard_normal((W, taps))).astype(np.float32)
        out[p + "canon2"] = (0.2 * rng.standard_normal((W, taps))).astype(np.float32)
        out[p + "mix.q"], out[p + "mix.k"], out[p + "mix.v"], out[p + "mix.o"] = lin(H * D, W), lin(G * D, W), lin(G * Dv, W), lin(W, H * Dv)
        if L["type"] == "retention":
            out[p + "mix.g"] = lin(H * Dv, W)
        else:
            out[p + "mix.r1"] = rng.uniform(0.1, 1.0, H).astype(np.float32)
            out[p + "mix.r2"] = rng.uniform(0.05, 0.5, H).astype(np.float32)
            out[p + "mix.sink"] = rng.standard_normal(H).astype(np.float32)
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            out[p + "mlp.gate"], out[p + "mlp.up"], out[p + "mlp.down"] = lin(F, W), lin(F, W), lin(W, F)
    return out


def pusunex_config(s):
    """Layers in turn: latent attention with a dense feed-forward, latent attention on the first layer's cached rows with experts, gated linear attention
    with experts, latent attention with latent queries and a rotated key part with experts.  The experts' sizes add up to the dense feed-forward's:
    8 experts of ff / 4, two chosen per token, and a shared one of ff / 2."""
    H, D, W = s["heads"], s["dim"], s["width"]
    experts = {"kind": "moe", "expert": {"ff": s["ff"] // 4}, "router": {"experts": 8, "top": 2}, "shared": {"ff": s["ff"] // 2}}
    layers = []
    for i in range(s["layers"]):
        k = i % 4
        if k == 0:
            layers.append({"type": "latent_attention", "mixer": {"heads": H, "dim": D, "vdim": D, "kv_rank": 256, "scale": D ** -0.5}, "mlp": {"kind": "dense", "ff": s["ff"]}})
        elif k == 1:
            layers.append({"type": "latent_attention", "mixer": {"heads": H, "dim": D, "vdim": D, "kv_rank": 256, "kv_from": i - 1, "scale": D ** -0.5}, "mlp": experts})
        elif k == 2:
            layers.append({"type": "gla", "mixer": {"heads": H, "dim": D, "vdim": D, "tau": 16.0}, "mlp": experts})
        else:
            layers.append({"type": "latent_attention_2", "mixer": {"heads": H, "dim": D - 64, "rot_dim": 64, "vdim": D, "kv_rank": 192, "q_rank": W // 2,
                                                                    "rot": {"dims": 64, "base": 10000.0}, "scale": D ** -0.5}, "mlp": experts})
    return {"architecture": "Pusunex", "vocab": s["vocab"], "width": W, "norm": {"eps": 1e-6, "groups": 4}, "token_side": {"dim": 64}, "layers": layers}


def pusunex_weights(cfg, seed=0):
    rng = np.random.default_rng(seed)
    W, V, nL, side = cfg["width"], cfg["vocab"], len(cfg["layers"]), cfg["token_side"]["dim"]

    def lin(o, i, g=1.0):
        return (rng.standard_normal((o, i), dtype=np.float32) * (g / np.sqrt(i))).astype(np.float32)

    def gains(n):
        return (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32)
    out = {"embed": rng.standard_normal((V, W), dtype=np.float32), "head": lin(V, W), "final.norm": gains(W), "side.embed": rng.standard_normal((V, nL * side), dtype=np.float32)}
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], "l%d." % i
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        out[p + "norm1"], out[p + "norm1b"], out[p + "norm2"], out[p + "norm2b"] = gains(W), gains(W), gains(W), gains(W)
        if L["type"] == "gla":
            out[p + "mix.q"], out[p + "mix.k"], out[p + "mix.v"], out[p + "mix.g"] = lin(H * D, W), lin(H * D, W), lin(H * Dv, W), lin(H * Dv, W)
            out[p + "mix.norm"], out[p + "mix.a1"], out[p + "mix.a2"] = gains(Dv), lin(32, W), lin(H * D, 32)
            out[p + "mix.a2.b"] = (3.0 + rng.standard_normal(H * D)).astype(np.float32)
        else:
            rank, R = m["kv_rank"], m.get("rot_dim", 0)
            if "q_rank" in m:
                out[p + "mix.dq"], out[p + "mix.dq.norm"], out[p + "mix.uq"] = lin(m["q_rank"], W), gains(m["q_rank"]), lin(H * (D + R), m["q_rank"])
            else:
                out[p + "mix.q"], out[p + "mix.g"] = lin(H * D, W), lin(H * Dv, W)
            if m.get("kv_from") is None:
                out[p + "mix.dkv"], out[p + "mix.dkv.norm"] = lin(rank + R, W), gains(rank)
            out[p + "mix.uk"], out[p + "mix.uv"] = lin(H * D, rank), lin(H * Dv, rank)
        out[p + "mix.o"] = lin(W, H * Dv)
        mlp = L["mlp"]
        if mlp["kind"] == "dense":
            out[p + "mlp.up"], out[p + "mlp.down"], out[p + "mlp.act"] = lin(mlp["ff"], W), lin(W, mlp["ff"]), np.array([0.7, 0.4, -0.3, 0.1], np.float32)
        else:
            out[p + "mlp.router"] = lin(mlp["router"]["experts"], W, 2.0)
            for n, f in [("e%d" % e, mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])] + [("shared", mlp["shared"]["ff"])]:
                out[p + "mlp.%s.gate" % n], out[p + "mlp.%s.up" % n], out[p + "mlp.%s.down" % n] = lin(f, W), lin(f, W), lin(W, f)
        out[p + "side.gate"], out[p + "side.proj"], out[p + "side.norm"] = lin(side, W), lin(W, side), (0.3 * gains(W)).astype(np.float32)
        out[p + "dwa"] = np.concatenate([0.1 * rng.standard_normal(i + 1), [1.0]]).astype(np.float32)
    return out


def sosutar_config(s, window=512):
    """Layers in turn: a matrix memory without a feed-forward, then windowed attention beside a gated recurrence of the model's width with a dense feed-forward;
    from the third layer on a matrix-memory layer uses the first one's weights (a state of its own)."""
    H, G, D, W = s["heads"], s["kv_heads"], s["dim"], s["width"]
    layers = []
    for i in range(s["layers"]):
        if i % 2 == 0:
            L = {"type": "mlstm", "mixer": {"heads": H, "dim": D, "vdim": D, "gate_cap": 15.0}, "mlp": None}
            if i >= 2:
                L["weights_of"] = 0
        else:
            L = {"type": "parallel", "mixer": {"left": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "mask": {"size": window}, "q_temp": {"coef": 0.2, "every": 256}, "scale": D ** -0.5},
                                               "right": {"width": W}}, "mlp": {"kind": "dense", "ff": s["ff"]}}
        layers.append(L)
    return {"architecture": "Sosutar", "vocab": s["vocab"], "width": W, "max_positions": 4096, "embedding": {"scale": 4.0}, "logit_scale": 0.5, "norm": {"eps": 1e-5}, "layers": layers}


def sosutar_weights(cfg, seed=0):
    rng = np.random.default_rng(seed)
    W, V = cfg["width"], cfg["vocab"]

    def lin(o, i, g=1.0):
        return (rng.standard_normal((o, i), dtype=np.float32) * (g / np.sqrt(i))).astype(np.float32)

    def gains(n, mean=1.0):
        return (mean + 0.1 * rng.standard_normal(n)).astype(np.float32)
    out = {"embed": rng.standard_normal((V, W), dtype=np.float32), "pos": rng.standard_normal((cfg["max_positions"], W), dtype=np.float32), "head": lin(V, W), "final.norm": gains(W)}
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        m, p = L["mixer"], "l%d." % i
        out[p + "norm1"], out[p + "ls1"] = gains(W), gains(W, 0.5)
        if L["type"] == "mlstm":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            out[p + "mix.q"], out[p + "mix.k"], out[p + "mix.v"], out[p + "mix.g"], out[p + "mix.o"] = lin(H * D, W), lin(H * D, W), lin(H * Dv, W), lin(H * Dv, W), lin(W, H * Dv)
            out[p + "mix.norm"], out[p + "mix.i"], out[p + "mix.f"] = gains(H * Dv), lin(H, W), lin(H, W)
            out[p + "mix.i.b"], out[p + "mix.f.b"] = rng.standard_normal(H).astype(np.float32), (3.0 + rng.standard_normal(H)).astype(np.float32)
        else:
            a, g = m["left"], m["right"]["width"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            out[q + "q"], out[q + "k"], out[q + "v"], out[q + "g"], out[q + "o"] = lin(H * D, W), lin(G * D, W), lin(G * Dv, W), lin(H * Dv, W), lin(W, H * Dv)
            out[q + "q.norm"], out[q + "k.norm"], out[q + "sink"], out[q + "out"] = gains(H * D), gains(G * D), rng.standard_normal(H).astype(np.float32), gains(W)
            q = p + "mix.right."
            out[q + "z"], out[q + "x"], out[q + "g"], out[q + "o"] = lin(g, W), lin(g, W), lin(g, W), lin(W, g)
            out[q + "z.b"], out[q + "x.b"], out[q + "out"] = rng.standard_normal(g).astype(np.float32), (0.5 * rng.standard_normal(g)).astype(np.float32), gains(W)
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            out[p + "norm2"], out[p + "ls2"], out[p + "mlp.up"], out[p + "mlp.down"] = gains(W), gains(W, 0.5), lin(F, W), lin(W, F)
    return out


def sokalorn_config(s, chunk=512):
    """A state-space layer and an attention over chunks beside a time mixing, both with eight experts of ff / 4 (two per token) and a shared expert of ff / 2; the pair
    runs layers / 2 times with the same weights, every pass behind the product over [x ; embedding output]."""
    H, G, D, W = s["heads"], s["kv_heads"], s["dim"], s["width"]
    mlp = {"kind": "moe", "expert": {"ff": s["ff"] // 4, "limit": 7.0}, "router": {"experts": 8, "top": 2}, "shared": {"ff": s["ff"] // 2, "limit": 7.0}}
    layers = [{"type": "mamba2", "mixer": {"heads": H, "vdim": D, "state": 128, "groups": G, "conv": 4, "norm_groups": G}, "mlp": mlp},
              {"type": "parallel", "mixer": {"left": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "mask": {"size": chunk}, "scale": D ** -0.5, "softcap": 30.0,
                                                      "rot": {"dims": D // 2, "base": 10000.0, "scaling": {"factor": 4.0}}},
                                             "right": {"heads": W // 64, "dim": 64}}, "mlp": mlp}]
    return {"architecture": "Sokalorn", "vocab": s["vocab"], "width": W, "norm": {"eps": 1e-5}, "layers": layers, "loop": {"start": 0, "stop": 2, "times": max(1, s["layers"] // 2)}}


def sokalorn_weights(cfg, seed=0, t_rank=64):
    rng = np.random.default_rng(seed)
    W, V = cfg["width"], cfg["vocab"]

    def lin(o, i, g=1.0):
        return (rng.standard_normal((o, i), dtype=np.float32) * (g / np.sqrt(i))).astype(np.float32)

    def gains(n, mean=1.0):
        return (mean + 0.1 * rng.standard_normal(n)).astype(np.float32)
    out = {"embed": rng.standard_normal((V, W), dtype=np.float32), "head": lin(V, W), "final.norm": gains(W), "loop.in": lin(W, 2 * W)}
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], "l%d." % i
        out[p + "norm1"], out[p + "shift"] = gains(W), rng.uniform(0.0, 1.0, W).astype(np.float32)
        if L["type"] == "mamba2":
            H, P, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            C = H * P + 2 * G * N
            out[p + "mix.in"], out[p + "mix.conv"], out[p + "mix.conv.b"] = lin(2 * H * P + 2 * G * N + H, W), (0.5 * rng.standard_normal((C, taps))).astype(np.float32), (0.1 * rng.standard_normal(C)).astype(np.float32)
            out[p + "mix.dt_bias"], out[p + "mix.A_log"] = rng.uniform(-4.0, -1.0, H).astype(np.float32), rng.uniform(-1.0, 1.0, H).astype(np.float32)
            out[p + "mix.D"], out[p + "mix.norm"], out[p + "mix.o"] = rng.standard_normal(H).astype(np.float32), gains(H * P), lin(W, H * P)
        else:
            a, t = m["left"], m["right"]
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            out[q + "q"], out[q + "k"], out[q + "v"], out[q + "g"], out[q + "o"] = lin(H * D, W), lin(G * D, W), lin(G * Dv, W), lin(H * Dv, W), lin(W, H * Dv)
            out[q + "pb"], out[q + "out"] = rng.uniform(-6.0, -3.0, H).astype(np.float32), gains(W)
            q, tn = p + "mix.right.", t["heads"] * t["dim"]
            for c in "rkvgw":
                out[q + "mu." + c] = rng.uniform(0.0, 1.0, W).astype(np.float32)
            out[q + "r"], out[q + "k"], out[q + "v"], out[q + "g"], out[q + "o"] = lin(tn, W), lin(tn, W), lin(tn, W), lin(tn, W), lin(W, tn)
            out[q + "w1"], out[q + "w2"], out[q + "w0"] = lin(t_rank, W), lin(tn, t_rank), rng.uniform(-5.0, -1.0, tn).astype(np.float32)
            out[q + "u"], out[q + "norm"], out[q + "out"] = (0.5 * rng.standard_normal((t["heads"], t["dim"]))).astype(np.float32), gains(tn), gains(W)
        mlp = L.get("mlp")
        if mlp:
            E = mlp["router"]["experts"]
            out[p + "mlp.router"], out[p + "mlp.shared.sg"] = lin(E, W), lin(1, W)
            for n in ["e%d" % e for e in range(E)] + ["shared"]:
                f = mlp["shared"]["ff"] if n == "shared" else mlp["expert"]["ff"]
                out[p + "mlp.%s.gate" % n], out[p + "mlp.%s.up" % n], out[p + "mlp.%s.down" % n] = lin(f, W), lin(f, W), lin(W, f)
    return out


def _run(nvr, engine, vocab, batch, prompt, steps, warmup):
    sp = nvr.SamplingParams(temperature=0.0, max_tokens=steps + warmup + 1, ignore_eos=True)
    for i in range(batch):
        engine.add_request(nvr.synthetic_tokens(prompt, 7, i, vocab).tolist(), sp)
    nvr.synchronize()
    t0 = time.perf_counter()
    rec = engine.step()
    nvr.synchronize()
    t_prefill = time.perf_counter() - t0
    assert rec["is_prefill"] and rec["num_seqs"] == batch, rec
    for _ in range(warmup):
        engine.step()
    nvr.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    nvr.synchronize()
    t_decode = (time.perf_counter() - t0) / steps
    return dict(prefill_tokens_per_s=round(batch * prompt / t_prefill), prefill_ms=round(t_prefill * 1e3, 2),
                decode_tokens_per_s=round(batch / t_decode), decode_ms_per_step=round(t_decode * 1e3, 3))


def compare(nvr, sizes=("w1024", "w2048"), batch=16, prompt=1024, steps=32, warmup=4, dtype="bfloat16", which=("rugudra", "qwen3")):
    out = []
    bs = 256
    for name in sizes:
        s = SIZES[name]
        ecfg = dict(max_num_seqs=batch, max_num_batched_tokens=batch * prompt, max_model_len=prompt + steps + warmup + 8, kvcache_block_size=bs,
                    num_kvcache_blocks=batch * ((prompt + steps + warmup + 8 + bs - 1) // bs + 1), dtype=dtype)
        line = {"size": name, "shape": s, "batch": batch, "prompt_len": prompt, "decode_steps": steps, "dtype": dtype}
        if "rugudra" in which:
            cfg = rugudra_config(s)
            eng = nvr.LLMEngine(nvr.Config(**ecfg), nvr.ModelSpec(cfg))
            for k, v in random_weights(cfg).items():
                eng.model_runner.load_tensor(k, np.asarray(v))
            _run(nvr, eng, s["vocab"], 2, 64, 2, 1)                       # first launches
            line["rugudra"] = _run(nvr, eng, s["vocab"], batch, prompt, steps, warmup)
            del eng
        if "pusunex" in which:
            cfg = pusunex_config(s)
            eng = nvr.LLMEngine(nvr.Config(**ecfg), nvr.ModelSpec(cfg))
            for k, v in pusunex_weights(cfg).items():
                eng.model_runner.load_tensor(k, np.asarray(v))
            _run(nvr, eng, s["vocab"], 2, 64, 2, 1)
            line["pusunex"] = _run(nvr, eng, s["vocab"], batch, prompt, steps, warmup)
            del eng
        if "sosutar" in which:
            cfg = sosutar_config(s)
            eng = nvr.LLMEngine(nvr.Config(**ecfg), nvr.ModelSpec(cfg))
            for k, v in sosutar_weights(cfg).items():
                eng.model_runner.load_tensor(k, np.asarray(v))
            _run(nvr, eng, s["vocab"], 2, 64, 2, 1)
            line["sosutar"] = _run(nvr, eng, s["vocab"], batch, prompt, steps, warmup)
            del eng
        if "sokalorn" in which:
            cfg = sokalorn_config(s)
            eng = nvr.LLMEngine(nvr.Config(**ecfg), nvr.ModelSpec(cfg))
            for k, v in sokalorn_weights(cfg).items():
                eng.model_runner.load_tensor(k, np.asarray(v))
            _run(nvr, eng, s["vocab"], 2, 64, 2, 1)
            line["sokalorn"] = _run(nvr, eng, s["vocab"], batch, prompt, steps, warmup)
            del eng
        if "qwen3" in which:
            m = nvr.ModelConfig(vocab_size=s["vocab"], hidden_size=s["width"], intermediate_size=s["ff"], num_hidden_layers=s["layers"], num_attention_heads=s["heads"],
                                num_key_value_heads=s["kv_heads"], head_dim=s["dim"], max_position_embeddings=8192, tie_word_embeddings=0)
            eng = nvr.LLMEngine(nvr.Config(**ecfg), m)
            _run(nvr, eng, s["vocab"], 2, 64, 2, 1)
            line["qwen3"] = _run(nvr, eng, s["vocab"], batch, prompt, steps, warmup)
            del eng
        out.append(line)
        print(json.dumps(line), flush=True)
    return out
