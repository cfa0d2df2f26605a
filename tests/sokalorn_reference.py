"""A plain restatement of the Sokalorn design in numpy float64, one function per mechanism, written from the design's equations.  It shares no
code with the library: the GPU tests compare the engine against it.

Notation.  x [T, W] is the residual stream of ONE sequence, `cfg` the configuration (the dict of config.json), `wt` a dict name -> array with the
checkpoint's tensor names.  Linear weights are [out, in].  Every function takes the state its mechanism carries from the tokens before (None: a
new sequence) and returns it updated, so that a prompt can be cut anywhere.

  x_0      =  embed[token]
  pass:       x <- W_loop [x ; x_0] before the first layer of every pass over the looped range (layers start .. stop-1, `times` passes,
              each pass with states of its own)
  layer:      h = w1 * x / sqrt(mean(x^2) + eps);   m_t = h_t + (h_(t-1) - h_t) * shift   (h_(-1) = 0)
              x <- x + mixer(m) + ff(h)
  logits   =  head (w_f * x / sqrt(mean(x^2) + eps))
"""
import numpy as np


def rms(v, eps):
    return v / np.sqrt((v * v).mean(axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def token_shift(h, mu, prev):
    """m_t = h_t + (h_(t-1) - h_t) * mu; prev: the row before the first one (None: zeros).  Returns (m, last row of h)."""
    before = np.concatenate([np.zeros((1, h.shape[1])) if prev is None else prev[None], h[:-1]])
    return h + (before - h) * mu, h[-1].copy()


def mamba2(h, m, wt, p, eps, state=None):
    """State-space mixer.  W_in h = [z | x | B | C | dt]; x, B, C pass a causal convolution per channel (with bias) and silu;
    dt = softplus(dt + dt_bias); per head a (its B, C those of group a // (heads / groups)):
        S_t = exp(-exp(A_log_a) dt_t) S_(t-1) + dt_t B_t x_t^T,   y_t = S_t^T C_t + D_a x_t;
    y silu(z), RMS-normed in norm_groups equal parts, times a weight, then W_o.
    state: (S [H, N, P], the last taps-1 rows that entered the convolution) or None."""
    T = h.shape[0]
    H, P, N, G, taps, ng = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"], m["norm_groups"]
    inner = H * P
    u = h @ wt[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    C = xbc.shape[1]
    if state is None:
        S, tail = np.zeros((H, N, P)), np.zeros((taps - 1, C))
    else:
        S, tail = state[0].copy(), state[1]
    padded = np.concatenate([tail, xbc])
    cw = wt[p + "conv"]
    conv = sum(padded[j:j + T] * cw[:, j] for j in range(taps)) + wt[p + "conv.b"]
    new_tail = padded[len(padded) - (taps - 1):].copy() if taps > 1 else padded[:0]
    conv = silu(conv)
    xs = conv[:, :inner].reshape(T, H, P)
    Bm = conv[:, inner:inner + G * N].reshape(T, G, N)
    Cm = conv[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + wt[p + "dt_bias"])
    decay = np.exp(-np.exp(wt[p + "A_log"]) * dt)
    y = np.zeros((T, H, P))
    for t in range(T):
        for a in range(H):
            g = a // (H // G)
            S[a] = decay[t, a] * S[a] + dt[t, a] * np.outer(Bm[t, g], xs[t, a])
            y[t, a] = S[a].T @ Cm[t, g] + wt[p + "D"][a] * xs[t, a]
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.reshape(T, ng, inner // ng), eps).reshape(T, inner) * wt[p + "norm"]
    return y @ wt[p + "o"].T, (S, new_tail)


def rotate_half(v, pos, dims, base, factor):
    """The first `dims` numbers of every head: (u_i, u_(i + dims/2)) turned by the angle pos * base^(-2i/dims) / factor."""
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims) / factor
    ang = pos[:, None] * f[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    out = v.copy()
    a, b = v[..., :half], v[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def chunk_sigmoid_attention(h, m, wt, p, pos0=0, past=None):
    """Grouped heads, rotated q and k, score = cap tanh(q.k scale / cap); position i sees j <= i of its own chunk of mask.size positions (chunks
    count from position 0); the weight of a visible key is sigmoid(score + pb_h), not normalised; heads times sigmoid(W_g h); W_o.
    past: (k, v) of the positions before pos0 or None."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size, scale, cap = m["mask"]["size"], m["scale"], m["softcap"]
    rot = m["rot"]
    pos = pos0 + np.arange(T)
    q = rotate_half((h @ wt[p + "q"].T).reshape(T, H, D), pos, rot["dims"], rot["base"], rot["scaling"]["factor"])
    k = rotate_half((h @ wt[p + "k"].T).reshape(T, G, D), pos, rot["dims"], rot["base"], rot["scaling"]["factor"])
    v = (h @ wt[p + "v"].T).reshape(T, G, Dv)
    if past is not None:
        k, v = np.concatenate([past[0], k]), np.concatenate([past[1], v])
    o = np.zeros((T, H, Dv))
    for t in range(T):
        i = pos0 + t
        js = np.arange(i // size * size, i + 1)
        for a in range(H):
            g = a // (H // G)
            s = k[js, g] @ q[t, a] * scale
            s = cap * np.tanh(s / cap)
            o[t, a] = sigmoid(s + wt[p + "pb"][a]) @ v[js, g]
    o = o.reshape(T, H * Dv) * sigmoid(h @ wt[p + "g"].T)
    return o @ wt[p + "o"].T, (k, v)


def receptance_mixing(h, m, wt, p, eps, state=None):
    """Time mixing with a decay per token and key channel.  Each of r, k, v, g, w reads h_t + (h_(t-1) - h_t) mu_s;
        w_t = exp(-exp(W_w2 tanh(W_w1 .) + w0));   o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t;   S_t = diag(w_t) S_(t-1) + k_t v_t^T;
    each head's o divided by its root mean square, times a weight, times silu(W_g .), then W_o.
    state: (S [H, D, D], the last row of h) or None."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    S, prev = (np.zeros((H, D, D)), None) if state is None else (state[0].copy(), state[1])
    mix = {}
    for s in "rkvgw":
        mix[s], last = token_shift(h, wt[p + "mu." + s], prev)
    r = (mix["r"] @ wt[p + "r"].T).reshape(T, H, D)
    k = (mix["k"] @ wt[p + "k"].T).reshape(T, H, D)
    v = (mix["v"] @ wt[p + "v"].T).reshape(T, H, D)
    gate = silu(mix["g"] @ wt[p + "g"].T)
    w = np.exp(-np.exp(np.tanh(mix["w"] @ wt[p + "w1"].T) @ wt[p + "w2"].T + wt[p + "w0"])).reshape(T, H, D)
    u = wt[p + "u"]
    o = np.zeros((T, H, D))
    for t in range(T):
        for a in range(H):
            kv = np.outer(k[t, a], v[t, a])
            o[t, a] = (S[a] + u[a][:, None] * kv).T @ r[t, a]
            S[a] = w[t, a][:, None] * S[a] + kv
    o = rms(o, eps).reshape(T, H * D) * wt[p + "norm"] * gate
    return o @ wt[p + "o"].T, (S, last)


def side_by_side(h, m, wt, p, eps, pos0=0, state=None):
    """Attention and time mixing read the same input; each result is RMS-normed over the width with its own weight; half their sum."""
    past, rs = state if state is not None else (None, None)
    yl, past = chunk_sigmoid_attention(h, m["left"], wt, p + "left.", pos0, past)
    yr, rs = receptance_mixing(h, m["right"], wt, p + "right.", eps, rs)
    return 0.5 * (rms(yl, eps) * wt[p + "left.out"] + rms(yr, eps) * wt[p + "right.out"]), (past, rs)


def clamped_expert(h, wt, p, limit):
    g = np.minimum(h @ wt[p + "gate"].T, limit)
    u = np.clip(h @ wt[p + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ wt[p + "down"].T


def route(h, wt, p, top, margins=None):
    """Softmax over all experts; the `top` largest; their scores divided by their sum.  Returns (chosen [T, top], weights [T, top]).
    margins (a list) collects, per token, the gap between the last chosen and the first rejected logit."""
    z = h @ wt[p + "router"].T
    if margins is not None and top < z.shape[1]:
        zs = np.sort(z, axis=-1)[:, ::-1]
        margins.extend((zs[:, top - 1] - zs[:, top]).tolist())
    z = z - z.max(axis=-1, keepdims=True)
    s = np.exp(z)
    s /= s.sum(axis=-1, keepdims=True)
    chosen = np.argsort(-s, axis=-1, kind="stable")[:, :top]
    w = np.take_along_axis(s, chosen, axis=-1)
    return chosen, w / (w.sum(axis=-1, keepdims=True) + 1e-20)


def expert_ff(h, f, wt, p, margins=None):
    """Mixture of experts with an optional shared expert that every token uses, times sigmoid(W_sg h)."""
    chosen, w = route(h, wt, p, f["router"]["top"], margins)
    y = np.zeros((h.shape[0], wt[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for c, wc in zip(chosen[t], w[t]):
            y[t] += wc * clamped_expert(h[t:t + 1], wt, p + "e%d." % c, f["expert"]["limit"])[0]
    if f.get("shared") is not None:
        y = y + clamped_expert(h, wt, p + "shared.", f["shared"]["limit"]) * sigmoid(h @ wt[p + "shared.sg"].T)
    return y


def layer_runs(cfg):
    """[(layer, first of a pass over the looped range)] in the order the layers run."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if loop is None:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        runs += [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, False) for i in range(loop["stop"], n)]


def forward(cfg, wt, tokens, layer_outputs=None, pos0=0, states=None, margins=None):
    """Logits [T, vocab] of one sequence's tokens at positions pos0 ..; states: the list forward returned for the tokens before (None: a new
    sequence).  Returns (logits, states)."""
    eps = cfg["norm"]["eps"]
    tokens = np.asarray(tokens)
    x = wt["embed"][tokens].astype(np.float64)
    x0 = x.copy()
    new_states = []
    for ri, (i, first) in enumerate(layer_runs(cfg)):
        L, p = cfg["layers"][i], "l%d." % i
        st = states[ri] if states is not None else (None, None)
        if first:
            x = np.concatenate([x, x0], axis=1) @ wt["loop.in"].T
        h = rms(x, eps) * wt[p + "norm1"]
        m, last = token_shift(h, wt[p + "shift"], st[0])
        if L["type"] == "mamba2":
            y, ms = mamba2(m, L["mixer"], wt, p + "mix.", eps, st[1])
        elif L["type"] == "parallel":
            y, ms = side_by_side(m, L["mixer"], wt, p + "mix.", eps, pos0, st[1])
        else:
            raise ValueError(L["type"])
        new_states.append((last, ms))
        if L.get("mlp") is not None:
            y = y + expert_ff(h, L["mlp"], wt, p + "mlp.", margins)
        x = x + y
        if layer_outputs is not None:
            layer_outputs.append(x.copy())
    logits = (rms(x, eps) * wt["final.norm"]) @ wt["head"].T
    return logits, new_states
