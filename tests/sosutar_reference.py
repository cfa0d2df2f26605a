"""A plain restatement of the Sosutar design in numpy float64, one function per mechanism, written from the design's equations.  It shares no
code with the library: the GPU tests compare the engine against it.

Notation.  x [T, W] is the residual stream of ONE sequence (positions 0 .. T-1), `cfg` the configuration (the dict of config.json), `wt` a dict
name -> array with the checkpoint's tensor names.  Linear weights are [out, in].

  x_0     =  embed[token] * embedding.scale + pos[p]
  layer:     x <- x + ls1 * mixer(n1(x));   x <- x + ls2 * ff(n2(x))   (a layer without a feed-forward has the first half only)
  n(v)    =  w * v / sqrt(mean(v^2) + eps)
  logits  =  head n_final(x) * logit_scale
A layer with 'weights_of': j reads layer j's tensors (j may come later) and keeps a state / cache of its own.
"""
import math

import numpy as np


def rms(v, eps):
    return v / np.sqrt((v * v).mean(axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def silu(z):
    return z * sigmoid(z)


def soft_cap(z, cap):
    return cap * np.tanh(z / cap)


def mlstm(h, m, wt, p, eps, state=None):
    """Matrix memory with exponential gates, per head: with log gates i_t, f_t and a running maximum m_t = max(f_t + m_(t-1), i_t), m_(-1) = 0,
        S_t = e^(f_t + m_(t-1) - m_t) S_(t-1) + e^(i_t - m_t) k_t v_t^T,   n_t the same with k_t alone,
        o_t = S_t^T q_t / (max(|n_t . q_t|, e^(-m_t)) + 1e-6).
    Each head's o is divided by its root mean square; the heads together times a weight, times sigmoid(W_g h), then W_o.
    state: (S [H, D, Dv], n [H, D], m [H]) carried in, or None for zeros; returns (y, state)."""
    T = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ wt[p + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ wt[p + "k"].T).reshape(T, H, D)
    v = (h @ wt[p + "v"].T).reshape(T, H, Dv)
    gi = soft_cap(h @ wt[p + "i"].T + wt[p + "i.b"], cap)
    gf = log_sigmoid(soft_cap(h @ wt[p + "f"].T + wt[p + "f.b"], cap))
    if state is None:
        S, n, mx = np.zeros((H, D, Dv)), np.zeros((H, D)), np.zeros(H)
    else:
        S, n, mx = (a.copy() for a in state)
    o = np.zeros((T, H, Dv))
    for t in range(T):
        for a in range(H):
            m_new = max(gf[t, a] + mx[a], gi[t, a])
            keep, take = math.exp(gf[t, a] + mx[a] - m_new), math.exp(gi[t, a] - m_new)
            S[a] = keep * S[a] + take * np.outer(k[t, a], v[t, a])
            n[a] = keep * n[a] + take * k[t, a]
            mx[a] = m_new
            o[t, a] = (S[a].T @ q[t, a]) / (max(abs(n[a] @ q[t, a]), math.exp(-m_new)) + 1e-6)
    o = rms(o, eps).reshape(T, H * Dv) * wt[p + "norm"] * sigmoid(h @ wt[p + "g"].T)
    return o @ wt[p + "o"].T, (S, n, mx)


def query_temperature(pos, coef, every):
    """1 + coef * ln(floor((p + 1) / every) + 1)"""
    return 1.0 + coef * np.log(np.floor((pos + 1) / every) + 1.0)


def head_slopes(H):
    return np.array([2.0 ** (-8.0 * (a + 1) / H) for a in range(H)])


def window_attention(h, m, wt, p, eps, pos0=0, past=None):
    """Grouped heads; q and k RMS-normed over their whole projection (all heads at once) with a weight; q times the query temperature of its
    position; every head's value divided by its root mean square; score = q.k * scale - slope_h * (i - j) for 0 <= i - j < window;
    softmax whose denominator also holds e^(sink_h); heads times sigmoid(W_g h); W_o.
    past: (k, v) of the positions before pos0 (already normed), or None; returns (y, (k, v)) with the rows of this call appended."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    window, scale = m["mask"]["size"], m["scale"]
    pos = pos0 + np.arange(T)
    q = rms(h @ wt[p + "q"].T, eps) * wt[p + "q.norm"]
    q = q * query_temperature(pos, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None]
    k = rms(h @ wt[p + "k"].T, eps) * wt[p + "k.norm"]
    v = rms((h @ wt[p + "v"].T).reshape(T, G, Dv), eps)
    q, k = q.reshape(T, H, D), k.reshape(T, G, D)
    if past is not None:
        k, v = np.concatenate([past[0], k]), np.concatenate([past[1], v])
    slopes, sink = head_slopes(H), wt[p + "sink"]
    o = np.zeros((T, H, Dv))
    for t in range(T):
        i = pos0 + t
        j0 = max(0, i - window + 1)
        js = np.arange(j0, i + 1)
        for a in range(H):
            g = a // (H // G)
            s = k[js, g] @ q[t, a] * scale - slopes[a] * (i - js)
            mx = max(s.max(), sink[a])
            e = np.exp(s - mx)
            o[t, a] = (e @ v[js, g]) / (e.sum() + math.exp(sink[a] - mx))
    o = o.reshape(T, H * Dv) * sigmoid(h @ wt[p + "g"].T)
    return o @ wt[p + "o"].T, (k, v)


def min_gru(h, wt, p, state=None):
    """z = sigmoid(W_z h + b_z), u = W_x h + b_x, c = u + 1/2 (u >= 0) or sigmoid(u) (u < 0); S_t = (1 - z) S_(t-1) + z c; y = W_o (S_t silu(W_g h)).
    state [width] or None for zeros."""
    T = h.shape[0]
    z = sigmoid(h @ wt[p + "z"].T + wt[p + "z.b"])
    u = h @ wt[p + "x"].T + wt[p + "x.b"]
    c = np.where(u >= 0, u + 0.5, sigmoid(u))
    S = np.zeros(z.shape[1]) if state is None else state.copy()
    out = np.zeros_like(z)
    for t in range(T):
        S = (1.0 - z[t]) * S + z[t] * c[t]
        out[t] = S
    return (out * silu(h @ wt[p + "g"].T)) @ wt[p + "o"].T, S


def side_by_side(h, m, wt, p, eps, pos0=0, state=None):
    """Windowed attention and the gated recurrence read the same input; each result is RMS-normed over the width with its own weight; half their sum."""
    past, S = state if state is not None else (None, None)
    yl, past = window_attention(h, m["left"], wt, p + "left.", eps, pos0, past)
    yr, S = min_gru(h, wt, p + "right.", S)
    return 0.5 * (rms(yl, eps) * wt[p + "left.out"] + rms(yr, eps) * wt[p + "right.out"]), (past, S)


def relu2_ff(h, wt, p):
    z = np.maximum(h @ wt[p + "up"].T, 0.0)
    return (z * z) @ wt[p + "down"].T


def forward(cfg, wt, tokens, layer_outputs=None, pos0=0, states=None):
    """Logits [T, vocab] of one sequence's tokens at positions pos0 ..; states: the list forward returned for the tokens before (None: a new sequence).
    Returns (logits, states)."""
    eps = cfg["norm"]["eps"]
    tokens = np.asarray(tokens)
    T = len(tokens)
    x = wt["embed"][tokens] * cfg["embedding"]["scale"] + wt["pos"][pos0 + np.arange(T)]
    new_states = []
    for i, L in enumerate(cfg["layers"]):
        src = i
        while cfg["layers"][src].get("weights_of") is not None:     # (a borrowed layer may borrow itself)
            src = cfg["layers"][src]["weights_of"]
        p = "l%d." % src
        st = states[i] if states is not None else None
        h = rms(x, eps) * wt[p + "norm1"]
        if L["type"] == "mlstm":
            y, st = mlstm(h, L["mixer"], wt, p + "mix.", eps, st)
        elif L["type"] == "parallel":
            y, st = side_by_side(h, L["mixer"], wt, p + "mix.", eps, pos0, st)
        else:
            raise ValueError(L["type"])
        new_states.append(st)
        x = x + wt[p + "ls1"] * y
        if L.get("mlp") is not None:
            x = x + wt[p + "ls2"] * relu2_ff(rms(x, eps) * wt[p + "norm2"], wt, p + "mlp.")
        if layer_outputs is not None:
            layer_outputs.append(x.copy())
    logits = (rms(x, eps) * wt["final.norm"]) @ wt["head"].T * cfg["logit_scale"]
    return logits, new_states
