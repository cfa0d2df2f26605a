"""Host side of the Sosutar design, no GPU: the model registry's reading of a configuration and its refusals, and the plain restatement's own consistency
(a state carried over a cut gives the rows of the whole prompt; the probes the GPU tests rely on do decide their rows)."""
import copy

import numpy as np
import pytest

import nvr_import
import sosutar_reference as ref
from sosutar_util import expected_logits, make_config, make_key_stand_out, make_weights, mlstm_layer, side_layer

nvr = nvr_import.load()


def small():
    return make_config([mlstm_layer(), side_layer(), side_layer(ff=None), mlstm_layer(weights_of=0), side_layer(weights_of=1), mlstm_layer(heads=1, dim=8, vdim=8, ff=24)], vocab=53, width=48)


def test_registry_reads_the_design():
    assert "Sosutar" in nvr.registered_architectures()
    s = nvr.ModelSpec(small())
    assert (s.architecture, s.family, s.vocab_size, s.num_layer_runs) == ("Sosutar", 1, 53, 6)
    cfg = small()                                                  # a layer may name a later one, or one that borrows itself
    cfg["layers"][0], cfg["layers"][3] = cfg["layers"][3], cfg["layers"][0]
    cfg["layers"][0]["weights_of"] = 3
    cfg["layers"].append(dict(cfg["layers"][0], weights_of=0))
    assert nvr.ModelSpec(cfg).num_layer_runs == 7


@pytest.mark.parametrize("breakage, message", [
    (lambda c: c.pop("width"), "'width' is missing"),
    (lambda c: c.pop("max_positions"), "'max_positions' is missing"),
    (lambda c: c.pop("logit_scale"), "'logit_scale' is missing"),
    (lambda c: c["layers"][0].update(type="attention"), "layer type 'attention'"),
    (lambda c: c["layers"][0]["mixer"].update(gate_cap=0.0), "gate_cap' must be positive"),
    (lambda c: c["layers"][1]["mixer"]["left"].pop("mask"), "left.mask' is missing"),
    (lambda c: c["layers"][1]["mixer"]["left"]["q_temp"].update(every=0), "q_temp.every"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "4 heads over 3 key/value heads"),
    (lambda c: c["layers"][1]["mixer"].pop("right"), "mixer.right' is missing"),
    (lambda c: c["layers"][1]["mlp"].update(kind="moe"), "mlp.kind"),
    (lambda c: c["layers"][3].update(weights_of=3), "must name another layer"),
    (lambda c: c["layers"][3].update(weights_of=9), "must name another layer"),
    (lambda c: (c["layers"][0].update(weights_of=3), c["layers"][3].update(weights_of=0)), "must name another layer"),
    (lambda c: c["layers"][3].update(weights_of=1), "layer of other sizes"),
    (lambda c: c["layers"][4]["mixer"]["right"].update(width=8), "layer of other sizes"),
])
def test_registry_refuses_a_broken_configuration(breakage, message):
    cfg = copy.deepcopy(small())
    breakage(cfg)
    with pytest.raises(nvr.NvrError, match=message.replace("[", r"\[").replace("]", r"\]")):
        nvr.ModelSpec(cfg)


def test_a_carried_state_gives_the_rows_of_the_whole_prompt():
    cfg = small()
    w = {k: np.asarray(v, np.float64) for k, v in make_weights(cfg, seed=1).items()}
    toks = np.random.default_rng(2).integers(0, cfg["vocab"], 45).tolist()
    whole, _ = ref.forward(cfg, w, toks)
    rows, states, at = [], None, 0
    for n in (7, 1, 14, 2, 21):
        lg, states = ref.forward(cfg, w, toks[at:at + n], pos0=at, states=states)
        rows.append(lg); at += n
    assert np.abs(np.concatenate(rows) - whole).max() < 1e-9


def test_the_matrix_memory_does_not_overflow_with_open_gates():
    """Input gates at their cap for hundreds of tokens: the running maximum keeps every exponential at or below one."""
    cfg = make_config([mlstm_layer(heads=1, dim=8, vdim=8, gate_cap=30.0)], vocab=11, width=16)
    w = {k: np.asarray(v, np.float64) for k, v in make_weights(cfg, seed=3).items()}
    w["l0.mix.i.b"] = np.full(1, 200.0); w["l0.mix.f.b"] = np.full(1, 200.0)
    lg, st = ref.forward(cfg, w, [1, 2, 3] * 100)
    assert np.isfinite(lg).all() and st[0][2][0] > 29.0


def test_the_probe_key_decides_its_row_inside_the_window_only():
    cfg = make_config([side_layer(heads=4, kv_heads=2, dim=16, vdim=16, window=20, scale=0.75, ff=None), mlstm_layer()], vocab=31, width=48, embedding_scale=0.7)
    Q, K, n = 0, 1, 60
    w = make_key_stand_out(cfg, make_weights(cfg, seed=4, pos_gain=0.0), Q, K)
    rng = np.random.default_rng(5)
    for back, decides in ((1, True), (19, True), (20, False), (33, False)):
        toks = rng.integers(2, cfg["vocab"], n).tolist(); toks[-1] = Q; toks[n - 1 - back] = K
        gone = list(toks); gone[n - 1 - back] = 2
        a, b = expected_logits(cfg, w, toks)[-1], expected_logits(cfg, w, gone)[-1]
        moved = np.sqrt(((a - b) ** 2).mean()) / a.std()
        assert (moved > 0.2) == decides, (back, moved)
