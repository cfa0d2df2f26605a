"""Host side of the Sokalorn design, no GPU: the model registry's reading of a configuration and its refusals, and the plain restatement's own consistency
(a state carried over a cut gives the rows of the whole prompt; the recurrences in their one-shot forms; the probe the GPU tests rely on does decide its row)."""
import copy

import numpy as np
import pytest

import nvr_import
import sokalorn_reference as ref
from sokalorn_util import as64, expected_logits, make_config, make_key_stand_out, make_weights, moe, settled_tokens, side_layer, ssm_layer

nvr = nvr_import.load()


def small():
    return make_config([ssm_layer(), side_layer(), side_layer(mlp=None), ssm_layer(heads=2, vdim=8, state=8, groups=1, mlp=moe(experts=3, top=1, ff=8, shared=None))],
                       vocab=53, width=48, loop=(1, 3, 3))


def test_registry_reads_the_design():
    assert "Sokalorn" in nvr.registered_architectures()
    s = nvr.ModelSpec(small())
    assert (s.architecture, s.family, s.vocab_size, s.num_layer_runs) == ("Sokalorn", 1, 53, 8)
    cfg = small(); cfg.pop("loop")
    assert nvr.ModelSpec(cfg).num_layer_runs == 4
    cfg = small(); cfg["loop"] = {"start": 2, "stop": 2, "times": 5}
    assert nvr.ModelSpec(cfg).num_layer_runs == 4


@pytest.mark.parametrize("breakage, message", [
    (lambda c: c.pop("width"), "'width' is missing"),
    (lambda c: c.pop("norm"), "'norm' is missing"),
    (lambda c: c["layers"][0].update(type="attention"), "layer type 'attention'"),
    (lambda c: c["layers"][0]["mixer"].pop("state"), "mixer.state' is missing"),
    (lambda c: c["layers"][0]["mixer"].update(groups=3), "4 heads over 3 groups"),
    (lambda c: c["layers"][0]["mixer"].update(norm_groups=5), "norm_groups must divide"),
    (lambda c: c["layers"][0]["mixer"].update(conv=0), "conv must be positive"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "4 heads over 3 groups"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=7), "even rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=64), "even rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"]["scaling"].update(factor=0.0), "positive scaling factor"),
    (lambda c: c["layers"][1]["mixer"].pop("right"), "mixer.right' is missing"),
    (lambda c: c["layers"][1]["mixer"]["right"].pop("dim"), "right.dim' is missing"),
    (lambda c: c["layers"][1]["mlp"].update(kind="dense"), "mlp.kind"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "1 <= top <= experts"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"), "expert.limit' is missing"),
    (lambda c: c["loop"].update(stop=9), r"loop \[1, 9\)"),
    (lambda c: c["loop"].update(times=0), "loop"),
])
def test_registry_refuses_a_broken_configuration(breakage, message):
    cfg = copy.deepcopy(small())
    breakage(cfg)
    with pytest.raises(nvr.NvrError, match=message):
        nvr.ModelSpec(cfg)


def test_a_carried_state_gives_the_rows_of_the_whole_prompt():
    cfg = small()
    w = as64(make_weights(cfg, seed=1))
    toks = np.random.default_rng(2).integers(0, cfg["vocab"], 45).tolist()
    whole, _ = ref.forward(cfg, w, toks)
    rows, states, at = [], None, 0
    for n in (7, 1, 14, 2, 21):
        lg, states = ref.forward(cfg, w, toks[at:at + n], pos0=at, states=states)
        rows.append(lg); at += n
    assert np.abs(np.concatenate(rows) - whole).max() < 1e-9


def test_the_state_space_recurrence_is_a_decayed_sum():
    """y_t = sum_(s <= t) (prod_(s < r <= t) decay_r) dt_s (C_t . B_s) x_s + D x_t, written out without a state."""
    rng = np.random.default_rng(3)
    m = {"heads": 2, "vdim": 3, "state": 4, "groups": 1, "conv": 1, "norm_groups": 1}
    W, T, inner, N = 8, 9, 6, 4
    wt = {"in": rng.standard_normal((2 * inner + 2 * N + 2, W)), "conv": np.ones((inner + 2 * N, 1)), "conv.b": np.zeros(inner + 2 * N), "dt_bias": rng.standard_normal(2),
          "A_log": rng.standard_normal(2), "D": rng.standard_normal(2), "norm": np.ones(inner), "o": np.eye(inner)}
    h = rng.standard_normal((T, W))
    got, _ = ref.mamba2(h, m, wt, "", 1e-5)
    u = h @ wt["in"].T
    z, xbc, dt = u[:, :inner], ref.silu(u[:, inner:2 * inner + 2 * N]), ref.softplus(u[:, 2 * inner + 2 * N:] + wt["dt_bias"])
    x, B, C = xbc[:, :inner].reshape(T, 2, 3), xbc[:, inner:inner + N], xbc[:, inner + N:]
    la = -np.exp(wt["A_log"]) * dt
    y = np.zeros((T, 2, 3))
    for t in range(T):
        for a in range(2):
            for s in range(t + 1):
                y[t, a] += np.exp(la[s + 1:t + 1, a].sum()) * dt[s, a] * (C[t] @ B[s]) * x[s, a]
            y[t, a] += wt["D"][a] * x[t, a]
    want = ref.rms(y.reshape(T, inner) * ref.silu(z), 1e-5)
    assert np.abs(got - want).max() < 1e-9


def test_the_bonus_reaches_the_current_token_only():
    """With decays of (nearly) zero the time mixing's output is the bonus term alone: o_t = (r_t . (u k_t)) v_t."""
    cfg = make_config([side_layer(t_heads=1, t_dim=8, mlp=None)], vocab=11, width=16)
    w = as64(make_weights(cfg, seed=4))
    w["l0.mix.right.w0"] = np.full(8, 5.0)
    h = np.random.default_rng(5).standard_normal((6, 16))
    p = "l0.mix.right."
    got, _ = ref.receptance_mixing(h, cfg["layers"][0]["mixer"]["right"], w, p, 1e-5)
    mix = {s: ref.token_shift(h, w[p + "mu." + s], None)[0] for s in "rkvg"}
    r, k, v = mix["r"] @ w[p + "r"].T, mix["k"] @ w[p + "k"].T, mix["v"] @ w[p + "v"].T
    o = ((r * w[p + "u"][0] * k).sum(axis=1, keepdims=True)) * v
    o[1:] += ((r[1:] * k[:-1]).sum(axis=1, keepdims=True)) * v[:-1]          # (the token before is still in the state, undecayed, when the next one reads it)
    want = (ref.rms(o, 1e-5) * w[p + "norm"] * ref.silu(mix["g"] @ w[p + "g"].T)) @ w[p + "o"].T
    assert np.abs(got - want).max() < 1e-6


def test_the_probe_key_decides_its_row_inside_the_chunk_only():
    cfg = make_config([side_layer(heads=4, kv_heads=2, dim=16, vdim=16, chunk=20, scale=0.25, softcap=24.0, t_heads=1, t_dim=8, mlp=None)], vocab=31, width=48)
    Q, K = 0, 1
    w = make_key_stand_out(cfg, make_weights(cfg, seed=4), Q, K)
    w["l0.mix.right.out"] = np.zeros_like(w["l0.mix.right.out"]); w["l0.mix.right.mu.r"] = np.zeros_like(w["l0.mix.right.mu.r"])
    w64 = as64(w)
    rng = np.random.default_rng(5)
    for n, back, decides in ((60, 1, True), (60, 19, True), (60, 20, False), (60, 33, False), (41, 1, False), (42, 1, True)):
        toks = rng.integers(2, cfg["vocab"], n).tolist(); toks[-1] = Q; toks[n - 1 - back] = K
        gone = list(toks); gone[n - 1 - back] = 2
        h = [ref.rms(w64["embed"][t], 1e-5) * w64["l0.norm1"] for t in (toks, gone)]
        a, b = (ref.chunk_sigmoid_attention(x, cfg["layers"][0]["mixer"]["left"], w64, "l0.mix.left.")[0][-1] for x in h)
        moved = np.sqrt(((a - b) ** 2).mean()) / np.sqrt((a ** 2).mean())
        assert (moved > 0.5) == decides, (n, back, moved)


def test_settled_tokens_are_no_close_calls():
    cfg = small(); w = make_weights(cfg, seed=6)
    toks = settled_tokens(cfg, w, 50, 7)
    m = []
    ref.forward(cfg, as64(w), toks, margins=m)
    assert len(m) > 0 and min(m) > 0.05
