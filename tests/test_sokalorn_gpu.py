"""Sokalorn on the GPU against the plain restatement of the design (tests/sokalorn_reference.py): every mechanism alone, prompts against token-by-token
decoding, portions down to two tokens, unequal batches, pages and state slots that are used again, one key that stands out just inside and just outside its
chunk and at page borders, states that reach far back, the first tokens of a sequence, long decoding, sizes that are 1 or equal to each other, shapes of
every attention kernel, and greedy generation through the engine's scheduler."""
import numpy as np
import pytest

import nvr_import
from rugudra_util import Driver, TOL, row_errors
from sokalorn_util import as64, expected_logits, make_config, make_key_stand_out, make_weights, moe, settled_tokens, side_layer, ssm_layer
import sokalorn_reference as ref

pytestmark = pytest.mark.gpu


def tokens_of(n, vocab, seed, lo=0):
    return np.random.default_rng(seed).integers(lo, vocab, n).tolist()


def check(got, want, dtype, what=""):
    """float32: every row within the tolerance.  bfloat16: a head's output is divided by its root mean square, so a row whose head output nearly cancels carries its
    16-bit noise enlarged (the first rows of a sequence above all, where one token's sign decides); one row in fifty may exceed the tolerance, none five times."""
    e = row_errors(got, want)
    if dtype == "bfloat16":
        over = int((e >= TOL[dtype]).sum())
        assert over <= max(1, len(e) // 50) and e.max() < 5 * TOL[dtype], f"{what}: {over} of {len(e)} rows over the limit {TOL[dtype]}, row {int(e.argmax())} differs by {e.max():.3g}"
        return
    assert e.max() < TOL[dtype], f"{what}: row {int(e.argmax())} differs by {e.max():.3g} of the row's spread (limit {TOL[dtype]})"


# ------------------------------------------------------------------------------------------------ each mechanism alone
MECHANISMS = {
    "state_space": make_config([ssm_layer(heads=4, vdim=16, state=24, groups=2, conv=4, norm_groups=2)]),
    "state_space_one_group_one_norm": make_config([ssm_layer(heads=3, vdim=8, state=40, groups=1, conv=2, norm_groups=1)]),
    "state_space_a_group_per_head_no_convolution": make_config([ssm_layer(heads=2, vdim=32, state=16, groups=2, conv=1, norm_groups=4)]),
    "state_space_five_taps_odd_sizes": make_config([ssm_layer(heads=5, vdim=12, state=10, groups=5, conv=5, norm_groups=3, mlp=None)]),
    "state_space_values_of_33_states_of_64": make_config([ssm_layer(heads=2, vdim=33, state=64, groups=1, conv=3, norm_groups=2)]),
    "state_space_states_of_128": make_config([ssm_layer(heads=8, vdim=64, state=128, groups=2, conv=4, norm_groups=8, mlp=None)], width=96),
    "attention_beside_time_mixing": make_config([side_layer(heads=4, kv_heads=2, dim=16, vdim=24, chunk=12, rot=8, t_heads=2, t_dim=16)]),
    "attention_one_head_chunk_of_one": make_config([side_layer(heads=1, kv_heads=1, dim=24, vdim=8, chunk=1, rot=24, factor=1.0, t_heads=1, t_dim=8, mlp=None)]),
    "attention_chunk_longer_than_the_prompt": make_config([side_layer(heads=6, kv_heads=2, dim=8, vdim=40, chunk=300, rot=2, softcap=3.0, t_heads=3, t_dim=24)]),
    "attention_nothing_rotated_small_cap": make_config([side_layer(heads=2, kv_heads=2, dim=32, vdim=16, chunk=33, rot=0, softcap=0.5, scale=0.4, t_heads=4, t_dim=8)]),
    "attention_heads_of_64_in_groups_of_two": make_config([side_layer(heads=4, kv_heads=2, dim=64, vdim=64, chunk=40, rot=16, t_heads=2, t_dim=32)], width=96),
    "attention_heads_of_64_in_groups_of_four": make_config([side_layer(heads=4, kv_heads=1, dim=64, vdim=64, chunk=70, rot=64, factor=8.0, t_heads=1, t_dim=64)], width=96),
    "attention_heads_of_128_ungrouped": make_config([side_layer(heads=2, kv_heads=2, dim=128, vdim=128, chunk=50, rot=32, t_heads=2, t_dim=16, mlp=None)], width=128),
    "attention_keys_of_32_values_of_48": make_config([side_layer(heads=8, kv_heads=1, dim=32, vdim=48, chunk=24, rot=30, t_heads=2, t_dim=40)]),
    "attention_twenty_heads_on_one": make_config([side_layer(heads=20, kv_heads=1, dim=32, vdim=16, chunk=9, rot=4, t_heads=5, t_dim=12)]),
    "time_mixing_heads_of_64_and_128": make_config([side_layer(heads=2, kv_heads=1, dim=16, vdim=16, chunk=20, t_heads=2, t_dim=64),
                                                    side_layer(heads=2, kv_heads=1, dim=16, vdim=16, chunk=20, t_heads=1, t_dim=128, mlp=None)], width=96),
    "experts_one_of_one": make_config([ssm_layer(mlp=moe(experts=1, top=1, ff=16, shared=None))]),
    "experts_all_chosen": make_config([side_layer(mlp=moe(experts=4, top=4, ff=24, shared=24, shared_limit=1.25))]),
    "experts_one_of_seventy": make_config([ssm_layer(mlp=moe(experts=70, top=1, ff=8, limit=0.5, shared=8))]),
    "experts_five_of_nine_odd_sizes": make_config([side_layer(mlp=moe(experts=9, top=5, ff=20, limit=7.0, shared=12, shared_limit=0.25))], width=72),
    "loop_over_everything": make_config([ssm_layer(), side_layer()], loop=(0, 2, 3)),
    "loop_in_the_middle": make_config([side_layer(), ssm_layer(mlp=None), side_layer(mlp=None), ssm_layer()], loop=(1, 3, 2)),
    "loop_once_at_the_end": make_config([ssm_layer(), side_layer(), ssm_layer()], loop=(2, 3, 1)),
    "loop_over_nothing": make_config([ssm_layer(), side_layer()], loop=(1, 1, 4)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(name, dtype):
    cfg = MECHANISMS[name]
    w = make_weights(cfg, seed=len(name))
    toks = settled_tokens(cfg, w, 75, 1)
    want = expected_logits(cfg, w, toks)
    check(Driver(cfg, w, dtype).run_alone(toks), want, dtype, name)
    check(Driver(cfg, w, dtype, page=8).run_alone(toks, cuts=[41, 3, 1]), want, dtype, name + ", in portions")


def test_each_part_changes_the_result():
    """A part that is left out must show: with one tensor changed, the restatement's logits move by far more than the tolerance, and the engine follows each variant."""
    cfg = make_config([side_layer(), ssm_layer()], loop=(0, 2, 2))
    w = make_weights(cfg, seed=11)
    toks = settled_tokens(cfg, w, 40, 4)
    full = expected_logits(cfg, w, toks)
    check(Driver(cfg, w, "float32").run_alone(toks), full, "float32", "full")
    for key, val in (("l0.shift", 0.0), ("l1.shift", 1.0), ("l0.mix.left.pb", 2.0), ("l0.mix.left.g", 0.0), ("l0.mix.left.out", 0.1), ("l0.mix.right.out", 0.1),
                     ("l0.mix.right.mu.w", 0.0), ("l0.mix.right.mu.g", 1.0), ("l0.mix.right.u", 3.0), ("l0.mix.right.w0", 1.0), ("l0.mix.right.norm", 0.2),
                     ("l1.mix.D", 0.0), ("l1.mix.dt_bias", 2.0), ("l1.mix.A_log", -4.0), ("l1.mix.conv.b", 1.0), ("l1.mix.norm", 0.3),
                     ("l0.mlp.shared.sg", 0.0), ("l1.mlp.shared.down", 0.0), ("loop.in", 0.05)):
        w2 = dict(w); w2[key] = np.full_like(w[key], val)
        if key == "loop.in":
            w2[key] = (np.asarray(w[key]) * 0.5).astype(np.float32)
        want = expected_logits(cfg, w2, toks)
        assert row_errors(want, full).max() > 50 * TOL["float32"], key
        check(Driver(cfg, w2, "float32").run_alone(toks), want, "float32", key)
    for change in (lambda c: c["layers"][0]["mixer"]["left"].update(softcap=0.3), lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(base=3.0),
                   lambda c: c["layers"][0]["mixer"]["left"]["rot"]["scaling"].update(factor=0.25), lambda c: c["layers"][0]["mlp"]["expert"].update(limit=0.2),
                   lambda c: c["layers"][1]["mlp"]["shared"].update(limit=0.1), lambda c: c["layers"][0]["mixer"]["left"]["mask"].update(size=3)):
        import copy
        cfg2 = copy.deepcopy(cfg); change(cfg2)
        want = expected_logits(cfg2, w, toks)
        assert row_errors(want, full).max() > 50 * TOL["float32"]
        check(Driver(cfg2, w, "float32").run_alone(toks), want, "float32", "a constant of the configuration")


# ------------------------------------------------------------------------------------------------ a model with everything, in portions and batches
def everything(vocab=113, width=96):
    return make_config([ssm_layer(heads=3, vdim=16, state=32, groups=1, conv=3, norm_groups=3),
                        side_layer(heads=4, kv_heads=2, dim=32, vdim=32, chunk=21, rot=16, t_heads=3, t_dim=24, mlp=moe(experts=5, top=2, ff=40, shared=24)),
                        side_layer(heads=6, kv_heads=3, dim=16, vdim=8, chunk=50, rot=16, factor=1.0, t_heads=2, t_dim=16, mlp=None),
                        ssm_layer(heads=4, vdim=24, state=16, groups=4, conv=4, norm_groups=1, mlp=moe(experts=3, top=1, ff=56, shared=None))],
                       vocab=vocab, width=width, loop=(1, 3, 2))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_against_token_by_token_decoding(dtype):
    cfg = everything(); w = make_weights(cfg, seed=5)
    toks = settled_tokens(cfg, w, 60, 3)
    want = expected_logits(cfg, w, toks)
    check(Driver(cfg, w, dtype).run_alone(toks), want, dtype, "whole prompt")
    check(Driver(cfg, w, dtype, page=8).run_alone(toks, cuts=[1]), want, dtype, "token by token")
    check(Driver(cfg, w, dtype, page=8).run_alone(toks, cuts=[37, 1]), want, dtype, "a prompt, then token by token")


@pytest.mark.parametrize("cuts", [[2], [3, 2, 17, 2, 5], [16], [15, 17], [33, 2, 1], [64, 7], [20, 1, 21, 1]])
def test_portions(cuts):
    cfg = everything(); w = make_weights(cfg, seed=6)
    toks = settled_tokens(cfg, w, 85, 7)
    check(Driver(cfg, w, "float32", page=16).run_alone(toks, cuts=cuts), expected_logits(cfg, w, toks), "float32", f"portions {cuts}")


def test_first_tokens():
    """One, two and three tokens (shorter than the convolution), alone and as the first portion of a longer prompt."""
    cfg = everything(); w = make_weights(cfg, seed=21)
    toks = settled_tokens(cfg, w, 12, 22)
    want = expected_logits(cfg, w, toks)
    for n in (1, 2, 3):
        check(Driver(cfg, w, "float32", page=8).run_alone(toks[:n]), want[:n], "float32", f"{n} tokens")
        check(Driver(cfg, w, "float32", page=8).run_alone(toks, cuts=[n, 1, 2]), want, "float32", f"{n} tokens first")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_with_pages_and_slots_used_again(dtype):
    """Five requests of different lengths through three state slots and a pool of pages that cannot hold them all at once: portions of some beside single
    tokens of others; a finished request's pages and slot go to the next one.  Every request must come out as it does alone."""
    cfg = everything(); w = make_weights(cfg, seed=8)
    reqs = {n: settled_tokens(cfg, w, ln, 20 + k) for k, (n, ln) in enumerate([("a", 61), ("b", 9), ("c", 34), ("d", 47), ("e", 2)])}
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


def test_a_request_left_out_of_steps():
    """A request that sits out some steps while another goes on keeps its states and history."""
    cfg = everything(); w = make_weights(cfg, seed=31)
    a, b = settled_tokens(cfg, w, 30, 32), settled_tokens(cfg, w, 26, 33)
    d = Driver(cfg, w, "float32", page=8, slots=2)
    ga, gb = [], []
    out = d.step([("a", a[:7]), ("b", b[:3])]); ga.append(out["a"]); gb.append(out["b"])
    for i in range(3, 20):
        gb.append(d.step([("b", b[i:i + 1])])["b"])
    out = d.step([("a", a[7:9]), ("b", b[20:])]); ga.append(out["a"]); gb.append(out["b"])
    ga.append(d.step([("a", a[9:])])["a"])
    check(np.concatenate(ga), expected_logits(cfg, w, a), "float32", "the request that waited")
    check(np.concatenate(gb), expected_logits(cfg, w, b), "float32", "the request that went on")


# ------------------------------------------------------------------------------------------------ one key that stands out, around the chunk's edge
PROBE_LAYERS = {
    "small_heads": (dict(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.25, rot=8), 48),
    "heads_of_64": (dict(heads=4, kv_heads=2, dim=64, vdim=64, scale=0.11, rot=32), 96),
    "keys_of_32_values_of_48": (dict(heads=4, kv_heads=1, dim=32, vdim=48, scale=0.2, rot=4), 64),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", sorted(PROBE_LAYERS))
@pytest.mark.parametrize("chunk, last, back", [(20, 339, 0), (20, 339, 1), (20, 339, 19), (20, 339, 20), (20, 327, 7), (20, 327, 8), (20, 320, 1), (64, 319, 63), (64, 319, 64), (64, 320, 1),
                                               (65, 324, 64), (65, 324, 65), (130, 389, 127), (130, 389, 129), (130, 389, 130), (300, 599, 299), (300, 599, 300), (300, 300, 1), (1, 50, 1)])
def test_one_key_stands_out(kind, chunk, last, back, dtype):
    """Token K occurs once, `back` positions before the last token Q (at position `last`), whose queries lie along K's keys while every other key's weight is next to
    nothing: inside Q's chunk that one key decides the last row, one position before the chunk's first it must not be seen (8-token pages; chunks that start at page
    borders and inside pages, keys at the 64-key tiles' borders and far back).  The engine must agree with the restatement as a whole prompt, with the last token
    decoded alone, with the last token ending a short portion, and with a portion that starts at the key."""
    layer, width = PROBE_LAYERS[kind]
    if kind != "small_heads" and (chunk, back) not in ((20, 19), (20, 20), (64, 63), (64, 64), (130, 129), (130, 130), (300, 299)):
        pytest.skip("the other head sizes repeat the edges only")
    cfg = make_config([side_layer(chunk=chunk, softcap=24.0, t_heads=1, t_dim=8, mlp=None, **layer), ssm_layer(mlp=None)], vocab=31, width=width)
    Q, K, n = 0, 1, last + 1
    w = make_key_stand_out(cfg, make_weights(cfg, seed=9), Q, K)
    w["l0.mix.right.out"] = (np.asarray(w["l0.mix.right.out"]) * 0.05).astype(np.float32)       # (the attention's branch carries the layer)
    toks = tokens_of(n, cfg["vocab"], 10 + back, lo=2)
    toks[-1] = Q
    if back:
        toks[n - 1 - back] = K
    want = expected_logits(cfg, w, toks)
    inside = 0 < back <= last % chunk
    gone = list(toks); gone[n - 1 - back] = 2
    moved = row_errors(expected_logits(cfg, w, gone)[-1:], want[-1:]).max() if back else 0.0
    if inside:
        assert moved > 4 * TOL[dtype], "the key inside the chunk must decide the row"
    for cuts, what in (([n], "whole"), ([n - 1, 1], "decoded"), ([n - 3, 3], "end of a portion"), ([n - back - 1, back + 1] if 0 < back < n - 1 else [n - 2, 2], "a portion from the key on")):
        got = Driver(cfg, w, dtype, page=8, pages=80, max_tokens=640, max_len=640).run_alone(toks, cuts=cuts)
        check(got[-4:], want[-4:], dtype, f"{what}, {back} back, chunk {chunk}")
        if inside:
            assert row_errors(got[-1:], want[-1:]).max() < moved / 4, f"{what}, {back} back, chunk {chunk}: the last row is off by a quarter of what the key moves it"


def test_states_reach_far_back():
    """A state-space layer with decays near one and a time mixing with decays near one: the first eight tokens of 400 still move the last row (the attention beside it
    sees five positions); passes of 16 tokens, state slots and single tokens agree."""
    for cfg, keys in ((make_config([ssm_layer(heads=2, vdim=16, state=16, groups=1, mlp=None)], vocab=41), {"l0.mix.A_log": -7.0, "l0.mix.dt_bias": -1.0}),
                      (make_config([side_layer(heads=2, kv_heads=1, dim=16, vdim=16, chunk=5, t_heads=2, t_dim=16, mlp=None)], vocab=41), {"l0.mix.right.w0": -7.0, "l0.mix.left.out": 0.05})):
        w = make_weights(cfg, seed=12)
        for k, v in keys.items():
            w[k] = np.full_like(w[k], v)
        toks = tokens_of(400, cfg["vocab"], 13)
        want = expected_logits(cfg, w, toks)
        other = [(t + 1) % cfg["vocab"] for t in toks[:8]] + toks[8:]
        moved = row_errors(expected_logits(cfg, w, other)[-1:], want[-1:]).max()
        assert moved > 2e-4
        for cuts in ([400], [399, 1], [17, 200, 2, 1]):
            got = Driver(cfg, w, "float32", page=16, pages=32, max_tokens=512).run_alone(toks, cuts=cuts)
            check(got, want, "float32", f"portions {cuts}")
            assert row_errors(got[-1:], want[-1:]).max() < moved / 10, f"portions {cuts}: the last row is off by a tenth of what the first tokens move it"


def test_fast_decays_and_large_steps():
    """Step sizes of about twenty (past the soft-plus's linear branch) and decays of e^-e^3: nothing overflows and the state forgets at once."""
    cfg = make_config([ssm_layer(mlp=None), side_layer(mlp=None)], vocab=23)
    w = make_weights(cfg, seed=19)
    w["l0.mix.dt_bias"] = np.full_like(w["l0.mix.dt_bias"], 22.0); w["l1.mix.right.w0"] = np.full_like(w["l1.mix.right.w0"], 3.0)
    toks = tokens_of(50, cfg["vocab"], 20)
    want = expected_logits(cfg, w, toks)
    for cuts in ([50], [20, 1]):
        check(Driver(cfg, w, "float32", page=8, pages=32).run_alone(toks, cuts=cuts), want, "float32", f"portions {cuts}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = everything(); w = make_weights(cfg, seed=14)
    toks = settled_tokens(cfg, w, 200, 15)
    got = Driver(cfg, w, dtype, page=8, pages=32).run_alone(toks, cuts=[10, 1])
    check(got, expected_logits(cfg, w, toks), dtype, "190 decoded tokens")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_and_decoding_side_by_side(dtype):
    """Heads of 64 with chunks of 700 over 1100 tokens, twelve experts of which three: prompts cross many 64-key tiles and a chunk's edge, the experts' rows take the
    padded blocks of 256; two requests then decode side by side."""
    cfg = make_config([side_layer(heads=4, kv_heads=2, dim=64, vdim=64, chunk=700, rot=32, t_heads=2, t_dim=32, mlp=moe(experts=12, top=3, ff=64, shared=64)),
                       ssm_layer(heads=4, vdim=32, state=32, groups=2, mlp=None)], vocab=71, width=128)
    w = make_weights(cfg, seed=24)
    a, b = settled_tokens(cfg, w, 1100, 25, gap=0.02), settled_tokens(cfg, w, 900, 26, gap=0.02)
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
    check(np.concatenate(ga)[690:720], wa[690:720], dtype, "across the chunk's edge")


def test_decode_steps_replay_a_graph():
    """Decode-sized steps are captured the second time their shape is seen and replayed from then on; every replay is compared."""
    cfg = everything(); w = make_weights(cfg, seed=16)
    toks = settled_tokens(cfg, w, 48, 17)
    d = Driver(cfg, w, "float32", page=8)
    got = d.run_alone(toks, cuts=[8, 1])
    assert d.engine.model_runner is not None
    check(got, expected_logits(cfg, w, toks), "float32", "replayed steps")


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
    w64 = as64(w)
    for sid, p in zip(ids, prompts):
        full = done[sid].token_ids
        assert full[:len(p)] == p and len(full) == len(p) + new
        m = []
        lg = ref.forward(cfg, w64, full[:-1], margins=m)[0]
        for k in range(len(p) - 1, len(full) - 1):
            row = lg[k]
            spread = np.sqrt(((row - row.mean()) ** 2).mean())
            assert row.max() - row[full[k + 1]] <= 3 * TOL["float32"] * spread or min(m) < 1e-4, f"request {sid}: token {k + 1} is not the greedy choice"


# ------------------------------------------------------------------------------------------------ designs and schedules drawn at random
def random_design(seed):
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    width = pick([48, 64, 72, 96, 104, 128, 160])
    layers = []
    for i in range(int(rng.integers(1, 6))):
        mlp = None if rng.random() < 0.3 else moe(experts=int(rng.integers(1, 12)), top=1, ff=pick([8, 24, 40, 100]), limit=pick([0.5, 1.5, 7.0]),
                                                   shared=pick([None, 16, 40]), shared_limit=pick([0.5, 1.5]))
        if mlp:
            mlp["router"]["top"] = int(rng.integers(1, mlp["router"]["experts"] + 1))
        if rng.random() < 0.45:
            G = int(rng.integers(1, 4)); H = G * pick([1, 2, 3]); P = pick([8, 12, 16, 32, 40])
            ng = pick([g for g in (1, 2, 3, 4, H) if (H * P) % g == 0])
            layers.append(ssm_layer(heads=H, vdim=P, state=pick([8, 16, 24, 48, 64]), groups=G, conv=int(rng.integers(1, 6)), norm_groups=ng, mlp=mlp))
        else:
            G = int(rng.integers(1, 4)); dim = pick([8, 16, 32, 64, 96])
            layers.append(side_layer(heads=G * pick([1, 2, 4, 5]), kv_heads=G, dim=dim, vdim=pick([dim, 16, 24, 64]), chunk=pick([1, 2, 7, 16, 31, 64, 65, 100, 200]),
                                     scale=float(rng.uniform(0.05, 0.3)), softcap=pick([0.7, 5.0, 20.0, 50.0]), rot=pick([0, 2, 4, 8, dim]), base=pick([10.0, 10000.0]),
                                     factor=pick([1.0, 2.0, 4.0]), t_heads=int(rng.integers(1, 5)), t_dim=pick([8, 12, 16, 32, 64]), mlp=mlp))
    n = len(layers)
    loop = None
    if rng.random() < 0.7:
        a = int(rng.integers(0, n)); b = int(rng.integers(a, n + 1))
        loop = (a, b, int(rng.integers(1, 4)))
    return make_config(layers, vocab=int(rng.integers(40, 200)), width=width, loop=loop, eps=pick([1e-6, 1e-5]))


@pytest.mark.parametrize("seed", range(12))
def test_random_designs_and_schedules(seed):
    """A design drawn at random (layer order, sizes, chunks, loops, feed-forwards) runs a prompt whole, in random portions, and two requests of unequal length in
    one batch with their own portions, in both number formats."""
    cfg = random_design(100 + seed)
    w = make_weights(cfg, seed=200 + seed)
    rng = np.random.default_rng(300 + seed)
    a, b = settled_tokens(cfg, w, int(rng.integers(20, 130)), 400 + seed), settled_tokens(cfg, w, int(rng.integers(2, 60)), 500 + seed)
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
