"""Sosutar on the GPU against the plain restatement of the design (tests/sosutar_reference.py): every mechanism alone, prompts against token-by-token
decoding, portions down to two tokens, unequal batches, pages and state slots that are used again, one key that stands out just inside and just outside the
window and at page borders, states that reach far back, the first tokens of a sequence, long decoding, sizes that are 1 or equal to each other, shapes of
every attention kernel, and greedy generation through the engine's scheduler."""
import numpy as np
import pytest

import nvr_import
from rugudra_util import Driver, TOL, row_errors
from sosutar_util import expected_logits, make_config, make_key_stand_out, make_weights, mlstm_layer, side_layer

pytestmark = pytest.mark.gpu


def tokens_of(n, vocab, seed, lo=0):
    return np.random.default_rng(seed).integers(lo, vocab, n).tolist()


def check(got, want, dtype, what=""):
    e = row_errors(got, want)
    assert e.max() < TOL[dtype], f"{what}: row {int(e.argmax())} differs by {e.max():.3g} of the row's spread (limit {TOL[dtype]})"


# ------------------------------------------------------------------------------------------------ each mechanism alone
MECHANISMS = {
    "matrix_memory": make_config([mlstm_layer(heads=2, dim=16, vdim=24)]),
    "matrix_memory_one_head_small_cap": make_config([mlstm_layer(heads=1, dim=40, vdim=8, gate_cap=1.5)]),
    "matrix_memory_values_of_31_and_32": make_config([mlstm_layer(heads=3, dim=8, vdim=31), mlstm_layer(heads=2, dim=24, vdim=32)]),
    "matrix_memory_keys_of_128": make_config([mlstm_layer(heads=1, dim=128, vdim=16, gate_cap=20.0)]),
    "matrix_memory_heads_of_64_and_128": make_config([mlstm_layer(heads=2, dim=64, vdim=96), mlstm_layer(heads=1, dim=128, vdim=136, gate_cap=6.0)], width=96),
    "matrix_memory_with_feed_forward": make_config([mlstm_layer(ff=40)]),
    "attention_beside_recurrence": make_config([side_layer(heads=4, kv_heads=2, dim=16, vdim=16, window=12, gru=40)]),
    "attention_one_head_window_of_one": make_config([side_layer(heads=1, kv_heads=1, dim=24, vdim=8, window=1, gru=8, ff=None)]),
    "attention_window_longer_than_the_prompt": make_config([side_layer(heads=6, kv_heads=2, dim=8, vdim=40, window=300, coef=1.0, every=1, gru=100)]),
    "attention_temperature_every_seven": make_config([side_layer(heads=2, kv_heads=2, dim=32, vdim=16, window=33, coef=0.9, every=7, scale=0.4, gru=24)]),
    "attention_heads_of_64_in_groups_of_two": make_config([side_layer(heads=4, kv_heads=2, dim=64, vdim=64, window=40, gru=48)], width=96),
    "attention_heads_of_64_in_groups_of_four": make_config([side_layer(heads=4, kv_heads=1, dim=64, vdim=64, window=70, gru=48)], width=96),
    "attention_heads_of_128_ungrouped": make_config([side_layer(heads=2, kv_heads=2, dim=128, vdim=128, window=50, gru=16, ff=None)], width=128),
    "attention_keys_of_32_values_of_48": make_config([side_layer(heads=8, kv_heads=1, dim=32, vdim=48, window=24, gru=16)]),
    "attention_twenty_heads_on_one": make_config([side_layer(heads=20, kv_heads=1, dim=32, vdim=16, window=9, gru=16)]),
    "shared_weights": make_config([mlstm_layer(), side_layer(), mlstm_layer(weights_of=0), side_layer(weights_of=1), mlstm_layer(weights_of=0)]),
    "shared_weights_named_ahead": make_config([mlstm_layer(weights_of=2), side_layer(ff=None), mlstm_layer(), side_layer(ff=None, weights_of=1), mlstm_layer(weights_of=0)]),
    "scales_of_one": make_config([side_layer(), mlstm_layer(ff=24)], embedding_scale=1.0, logit_scale=1.0),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(name, dtype):
    cfg = MECHANISMS[name]
    w = make_weights(cfg, seed=len(name))
    toks = tokens_of(75, cfg["vocab"], 1)
    check(Driver(cfg, w, dtype).run_alone(toks), expected_logits(cfg, w, toks), dtype, name)
    check(Driver(cfg, w, dtype, page=8).run_alone(toks, cuts=[41, 3, 1]), expected_logits(cfg, w, toks), dtype, name + ", in portions")


def test_each_part_changes_the_result():
    """A part that is left out must show: with the sink, the gates' biases, the branch norms, the layer scale, the positions or the query temperature changed,
    the restatement's logits move by far more than the tolerance, and the engine follows each variant."""
    cfg = make_config([side_layer(every=4, coef=0.8), mlstm_layer(ff=32)])
    w = make_weights(cfg, seed=11)
    toks = tokens_of(40, cfg["vocab"], 4)
    full = expected_logits(cfg, w, toks)
    check(Driver(cfg, w, "float32").run_alone(toks), full, "float32", "full")
    for key, val in (("l0.mix.left.sink", 6.0), ("l0.mix.left.g", 0.0), ("l0.mix.left.out", 0.1), ("l0.mix.right.out", 0.1), ("l0.mix.right.z.b", -3.0), ("l0.mix.right.x.b", 1.0),
                     ("l0.mix.left.q.norm", 3.0), ("l0.mix.left.k.norm", 0.2), ("l0.ls1", 0.1), ("l1.ls2", 1.5), ("l1.mix.i.b", -4.0), ("l1.mix.f.b", -2.0), ("l1.mix.norm", 0.3),
                     ("pos", 0.0)):
        w2 = dict(w); w2[key] = np.full_like(w[key], val)
        want = expected_logits(cfg, w2, toks)
        assert row_errors(want, full).max() > 50 * TOL["float32"], key
        check(Driver(cfg, w2, "float32").run_alone(toks), want, "float32", key)
    cfg2 = make_config([side_layer(every=4, coef=0.0), mlstm_layer(ff=32)])
    want = expected_logits(cfg2, w, toks)
    assert row_errors(want, full).max() > 50 * TOL["float32"]
    check(Driver(cfg2, w, "float32").run_alone(toks), want, "float32", "no query temperature")


# ------------------------------------------------------------------------------------------------ a model with everything, in portions and batches
def everything(vocab=113, width=96):
    return make_config([mlstm_layer(heads=3, dim=16, vdim=32),
                        side_layer(heads=4, kv_heads=2, dim=32, vdim=32, window=21, every=8, gru=72, ff=80),
                        side_layer(heads=6, kv_heads=3, dim=16, vdim=8, window=50, every=16, gru=24, ff=None),
                        mlstm_layer(heads=3, dim=16, vdim=32, weights_of=0),
                        side_layer(heads=4, kv_heads=2, dim=32, vdim=32, window=21, every=8, gru=72, ff=80, weights_of=1),
                        mlstm_layer(heads=2, dim=24, vdim=16, gate_cap=4.0, ff=40)], vocab=vocab, width=width)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_against_token_by_token_decoding(dtype):
    cfg = everything(); w = make_weights(cfg, seed=5)
    toks = tokens_of(60, cfg["vocab"], 3)
    want = expected_logits(cfg, w, toks)
    check(Driver(cfg, w, dtype).run_alone(toks), want, dtype, "whole prompt")
    check(Driver(cfg, w, dtype, page=8).run_alone(toks, cuts=[1]), want, dtype, "token by token")
    check(Driver(cfg, w, dtype, page=8).run_alone(toks, cuts=[37, 1]), want, dtype, "a prompt, then token by token")


@pytest.mark.parametrize("cuts", [[2], [3, 2, 17, 2, 5], [16], [15, 17], [33, 2, 1], [64, 7], [20, 1, 21, 1]])
def test_portions(cuts):
    cfg = everything(); w = make_weights(cfg, seed=6)
    toks = tokens_of(85, cfg["vocab"], 7)
    check(Driver(cfg, w, "float32", page=16).run_alone(toks, cuts=cuts), expected_logits(cfg, w, toks), "float32", f"portions {cuts}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_with_pages_and_slots_used_again(dtype):
    """Five requests of different lengths through three state slots and a pool of pages that cannot hold them all at once: portions of some beside single
    tokens of others; a finished request's pages and slot go to the next one.  Every request must come out as it does alone."""
    cfg = everything(); w = make_weights(cfg, seed=8)
    reqs = {n: tokens_of(ln, cfg["vocab"], 20 + k) for k, (n, ln) in enumerate([("a", 61), ("b", 9), ("c", 34), ("d", 47), ("e", 2)])}
    want = {n: expected_logits(cfg, w, t) for n, t in reqs.items()}
    d = Driver(cfg, w, dtype, page=8, pages=20, slots=3, max_tokens=256)
    at = {n: 0 for n in reqs}
    got = {n: [] for n in reqs}
    waiting, live = ["a", "b", "c", "d", "e"], []
    sizes, k = [5, 1, 2, 11, 1, 1, 3, 8, 1, 2], 0
    while waiting or live:
        while waiting and len(live) < 3 and sum((len(reqs[n]) + 7) // 8 for n in live + waiting[:1]) <= 20:
            live.append(waiting.pop(0))
        entries = []
        for n in live:
            c = min(sizes[k % len(sizes)], len(reqs[n]) - at[n]); k += 1
            entries.append((n, reqs[n][at[n]:at[n] + c]))
            at[n] += c
        out = d.step(entries)
        for n, _ in entries:
            got[n].append(out[n])
        for n in [n for n in live if at[n] == len(reqs[n])]:
            d.end(n); live.remove(n)
    for n in reqs:
        check(np.concatenate(got[n]), want[n], dtype, f"request {n}")


# ------------------------------------------------------------------------------------------------ one key that stands out, around the window's edge
PROBE_LAYERS = {
    "small_heads": (dict(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.75), 48),
    "heads_of_64": (dict(heads=4, kv_heads=2, dim=64, vdim=64, scale=0.19), 96),
    "keys_of_32_values_of_48": (dict(heads=4, kv_heads=1, dim=32, vdim=48, scale=0.38), 64),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", sorted(PROBE_LAYERS))
@pytest.mark.parametrize("window, back", [(20, 0), (20, 1), (20, 7), (20, 8), (20, 19), (20, 20), (20, 21), (64, 63), (64, 64), (65, 64), (65, 65), (130, 127), (130, 129), (130, 130),
                                          (300, 299), (300, 300), (1, 1)])
def test_one_key_stands_out(kind, window, back, dtype):
    """Token K occurs once, `back` positions before the last token Q, whose queries lie along K's keys: inside the window that one key decides the last row, one
    position further out it must not be seen (8-token pages; windows that end at page borders, at the 64-key tiles' borders, and far back).  The engine must agree
    with the restatement as a whole prompt, with the last token decoded alone, and with the last token ending a short portion."""
    layer, width = PROBE_LAYERS[kind]
    if kind != "small_heads" and (window, back) not in ((20, 19), (20, 20), (64, 63), (64, 64), (130, 129), (130, 130), (300, 299)):
        pytest.skip("the other head sizes repeat the edges only")
    cfg = make_config([side_layer(window=window, gru=24, ff=None, **layer), mlstm_layer()], vocab=61, width=width, embedding_scale=0.7)
    Q, K, n = 0, 1, 340
    w = make_key_stand_out(cfg, make_weights(cfg, seed=9, pos_gain=0.0), Q, K)
    toks = tokens_of(n, cfg["vocab"], 10 + back, lo=2)
    toks[-1] = Q
    if back:
        toks[n - 1 - back] = K
    want = expected_logits(cfg, w, toks)
    if 0 < back < window:
        gone = list(toks); gone[n - 1 - back] = 2
        assert row_errors(expected_logits(cfg, w, gone)[-1:], want[-1:]).max() > 4 * TOL[dtype]
    for cuts, what in (([n], "whole"), ([n - 1, 1], "decoded"), ([n - 3, 3], "end of a portion"), ([n - back - 1, back + 1] if 0 < back < n - 1 else [n - 2, 2], "a portion from the key on")):
        got = Driver(cfg, w, dtype, page=8, pages=48, max_tokens=512).run_alone(toks, cuts=cuts)
        check(got[-4:], want[-4:], dtype, f"{what}, {back} back, window {window}")


def test_states_reach_far_back():
    """A matrix memory with forget gates near one and a recurrence with update gates near zero: the first eight tokens of 400 still move the last row, through an attention
    window of five; passes of 16 tokens, state slots and single tokens agree."""
    for cfg, keys in ((make_config([mlstm_layer(heads=2, dim=16, vdim=16, gate_cap=15.0)], vocab=41), {"l0.mix.f.b": 9.0, "l0.mix.i.b": -1.0}),
                      (make_config([side_layer(heads=2, kv_heads=1, dim=16, vdim=16, window=5, gru=32, ff=None)], vocab=41), {"l0.mix.right.z.b": -5.5})):
        w = make_weights(cfg, seed=12, pos_gain=0.05)
        for k, v in keys.items():
            w[k] = np.full_like(w[k], v)
        toks = tokens_of(400, cfg["vocab"], 13)
        want = expected_logits(cfg, w, toks)
        other = [(t + 1) % cfg["vocab"] for t in toks[:8]] + toks[8:]
        moved = row_errors(expected_logits(cfg, w, other)[-1:], want[-1:]).max()       # (the branch's output is normed: eight tokens of 400 move the row by their share)
        assert moved > 2e-4
        for cuts in ([400], [399, 1], [17, 200, 2, 1]):
            got = Driver(cfg, w, "float32", page=16, pages=32, max_tokens=512).run_alone(toks, cuts=cuts)
            check(got, want, "float32", f"portions {cuts}")
            assert row_errors(got[-1:], want[-1:]).max() < moved / 10, f"portions {cuts}: the last row is off by a tenth of what the first tokens move it"


def test_gates_at_their_cap():
    """Input gates pinned at a cap of 30 for 150 tokens: the running maximum grows to thousands while every stored number stays of order one."""
    cfg = make_config([mlstm_layer(heads=2, dim=8, vdim=8, gate_cap=30.0)], vocab=23)
    w = make_weights(cfg, seed=19)
    w["l0.mix.i.b"] = np.full_like(w["l0.mix.i.b"], 100.0); w["l0.mix.f.b"] = np.full_like(w["l0.mix.f.b"], 100.0)
    toks = tokens_of(150, cfg["vocab"], 20)
    want = expected_logits(cfg, w, toks)
    for cuts in ([150], [40, 1]):
        check(Driver(cfg, w, "float32", page=8, pages=32).run_alone(toks, cuts=cuts), want, "float32", f"portions {cuts}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = everything(); w = make_weights(cfg, seed=14)
    toks = tokens_of(200, cfg["vocab"], 15)
    got = Driver(cfg, w, dtype, page=8, pages=32).run_alone(toks, cuts=[10, 1])
    check(got, expected_logits(cfg, w, toks), dtype, "190 decoded tokens")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_and_decoding_with_split_keys(dtype):
    """Heads of 64 with a window of 700 over 1100 tokens: prompts take the flash kernel's windowed form across many 64-key steps, decode-sized steps spread a tile's keys
    over several workgroups; two requests decode side by side."""
    cfg = make_config([side_layer(heads=4, kv_heads=2, dim=64, vdim=64, window=700, every=128, gru=64, ff=64), mlstm_layer(heads=2, dim=32, vdim=32)], vocab=71, width=128, max_positions=1200)
    w = make_weights(cfg, seed=24)
    a, b = tokens_of(1100, cfg["vocab"], 25), tokens_of(900, cfg["vocab"], 26)
    wa, wb = expected_logits(cfg, w, a), expected_logits(cfg, w, b)
    d = Driver(cfg, w, dtype, page=64, pages=40, slots=2, max_tokens=2048, max_len=1200)
    ga, gb = [d.step([("a", a[:1080]), ("b", b[:880])])], []
    gb.append(ga[0]["b"]); ga[0] = ga[0]["a"]
    for i in range(20):
        out = d.step([("a", a[1080 + i:1081 + i]), ("b", b[880 + i:881 + i])])
        ga.append(out["a"]); gb.append(out["b"])
    check(np.concatenate(ga)[-60:], wa[-60:], dtype, "first request")
    check(np.concatenate(gb)[-60:], wb[-60:], dtype, "second request")
    check(np.concatenate(ga)[:40], wa[:40], dtype, "first rows")


def test_squared_relu_in_the_products_epilogue():
    """A step of more than four thousand rows at a width of 1024: the feed-forward's first product takes the 256 x 256 tiles with the squared ReLU in its epilogue; the same
    prompt in two portions takes the product and the activation as two launches.  Both must agree with the restatement."""
    cfg = make_config([mlstm_layer(heads=1, dim=16, vdim=16, ff=2048)], vocab=47, width=1024, max_positions=4400)
    w = make_weights(cfg, seed=29, pos_gain=0.5)
    toks = tokens_of(4300, cfg["vocab"], 30)
    want = expected_logits(cfg, w, toks)
    for cuts in ([4300], [2100, 2200]):
        got = Driver(cfg, w, "bfloat16", page=64, pages=70, slots=1, max_tokens=4352, max_len=4400).run_alone(toks, cuts=cuts)
        check(got[::7], want[::7], "bfloat16", f"portions {cuts}")


def test_decode_steps_replay_a_graph():
    """Decode-sized steps are captured the second time their shape is seen and replayed from then on; every replay is compared."""
    cfg = everything(); w = make_weights(cfg, seed=16)
    toks = tokens_of(48, cfg["vocab"], 17)
    d = Driver(cfg, w, "float32", page=8)
    got = d.run_alone(toks, cuts=[8, 1])
    assert d.engine.model_runner is not None
    check(got, expected_logits(cfg, w, toks), "float32", "replayed steps")


def test_positions_end_with_the_table():
    cfg = make_config([mlstm_layer()], max_positions=24)
    w = make_weights(cfg, seed=27)
    d = Driver(cfg, w, "float32", page=8, pages=16)
    toks = tokens_of(30, cfg["vocab"], 28)
    check(d.step([("r", toks[:24])])["r"], expected_logits(cfg, w, toks[:24]), "float32", "the table's last position")
    with pytest.raises(d.nvr.NvrError, match="position"):
        d.step([("r", toks[24:25])])


# ------------------------------------------------------------------------------------------------ through the engine's own entry point
@pytest.mark.parametrize("chunked", [0, 1])
def test_greedy_generation_through_the_scheduler(chunked):
    """Five requests through LLMEngine.add_request / step with three state slots and a token budget that cuts prompts (chunked) or batches them whole: every
    generated token is the arg-max of the restatement's logits for the sequence so far."""
    nvr = nvr_import.load()
    cfg = everything(); w = make_weights(cfg, seed=18)
    prompts = [tokens_of(n, cfg["vocab"], 30 + n) for n in (5, 23, 1, 40, 12)]
    new = 12
    eng = nvr.LLMEngine(nvr.Config(dtype="float32", kvcache_block_size=8, skip_block_size_check=1, num_kvcache_blocks=40, max_num_seqs=3, num_state_slots=3,
                                   max_num_batched_tokens=32 if chunked else 256, max_model_len=128, enable_chunked_prefill=chunked), nvr.ModelSpec(cfg))
    for k, v in w.items():
        eng.model_runner.load_tensor(k, np.asarray(v, dtype=np.float32))
    ids = [eng.add_request(p, nvr.SamplingParams(temperature=0.0, max_tokens=new, ignore_eos=True)) for p in prompts]
    steps = 0
    while not eng.is_finished():
        eng.step(); steps += 1
        assert steps < 400
    done = {s.seq_id: s for s in eng.take_finished()}
    assert sorted(done) == sorted(ids)
    for sid, p in zip(ids, prompts):
        full = done[sid].token_ids
        assert full[:len(p)] == p and len(full) == len(p) + new
        lg = expected_logits(cfg, w, full[:-1])
        for k in range(len(p) - 1, len(full) - 1):
            row = lg[k]
            spread = np.sqrt(((row - row.mean()) ** 2).mean())
            assert row.max() - row[full[k + 1]] <= 3 * TOL["float32"] * spread, f"request {sid}: token {k + 1} is not the greedy choice"


# ------------------------------------------------------------------------------------------------ designs and schedules drawn at random
def random_design(seed):
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    width = pick([48, 64, 96, 104, 128, 192])
    layers = []
    for i in range(int(rng.integers(1, 6))):
        same = [j for j, L in enumerate(layers) if "weights_of" not in L]
        if same and rng.random() < 0.3:
            j = pick(same)
            layers.append(dict(layers[j], weights_of=j))
            continue
        ff = pick([None, 24, 40, 100])
        if rng.random() < 0.45:
            layers.append(mlstm_layer(heads=int(rng.integers(1, 5)), dim=pick([8, 12, 16, 32, 64]), vdim=pick([8, 15, 16, 32, 33, 64]), gate_cap=pick([2.0, 8.0, 15.0, 30.0]), ff=ff))
        else:
            G = int(rng.integers(1, 4)); dim = pick([8, 16, 32, 64, 96])
            layers.append(side_layer(heads=G * pick([1, 2, 4, 5]), kv_heads=G, dim=dim, vdim=pick([dim, 16, 24, 64]), window=pick([1, 2, 7, 16, 31, 64, 65, 200]), scale=float(rng.uniform(0.05, 0.3)),
                                     coef=float(rng.uniform(0.0, 1.0)), every=pick([1, 3, 16, 64, 1000]), gru=pick([8, 24, 50, 128]), ff=ff))
    return make_config(layers, vocab=int(rng.integers(40, 200)), width=width, embedding_scale=pick([1.0, 2.0, 7.5]), logit_scale=pick([0.25, 1.0, 3.0]), eps=pick([1e-6, 1e-5]))


@pytest.mark.parametrize("seed", range(12))
def test_random_designs_and_schedules(seed):
    """A design drawn at random (layer order, sizes, windows, shared weights, feed-forwards) runs a prompt whole, in random portions, and two requests of unequal length in
    one batch with their own portions, in both number formats."""
    cfg = random_design(100 + seed)
    w = make_weights(cfg, seed=200 + seed)
    rng = np.random.default_rng(300 + seed)
    a, b = tokens_of(int(rng.integers(20, 130)), cfg["vocab"], 400 + seed), tokens_of(int(rng.integers(2, 60)), cfg["vocab"], 500 + seed)
    wa, wb = expected_logits(cfg, w, a), expected_logits(cfg, w, b)
    for dtype in ("float32", "bfloat16"):
        check(Driver(cfg, w, dtype, page=8, pages=64).run_alone(a), wa, dtype, f"design {seed}, whole")
        cuts = [int(c) for c in rng.integers(1, 40, 12)] + [1]
        check(Driver(cfg, w, dtype, page=8, pages=64).run_alone(a, cuts=cuts), wa, dtype, f"design {seed}, portions {cuts}")
        d = Driver(cfg, w, dtype, page=8, pages=64, slots=2)
        at, got = {"a": 0, "b": 0}, {"a": [], "b": []}
        toks = {"a": a, "b": b}
        while at["a"] < len(a) or at["b"] < len(b):
            entries = []
            for n in ("a", "b"):
                if at[n] < len(toks[n]):
                    c = min(int(rng.integers(1, 24)), len(toks[n]) - at[n])
                    entries.append((n, toks[n][at[n]:at[n] + c])); at[n] += c
            out = d.step(entries)
            for n, _ in entries:
                got[n].append(out[n])
        check(np.concatenate(got["a"]), wa, dtype, f"design {seed}, batch, first request")
        check(np.concatenate(got["b"]), wb, dtype, f"design {seed}, batch, second request")
