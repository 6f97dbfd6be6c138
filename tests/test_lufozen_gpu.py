"""The batched serving store (kr_serve_*) with the Lufozen design against the plain float64 restatement in tests/oracle_lufozen.py.

Small random models of several shapes; every comparison is between what the store's step function returns (logits, or the residual stream after each
layer run) and the oracle run on the whole sequence.  The f32 store is held to 2e-4 of the stream's scale, the bf16 store to a few percent."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import oracle_lufozen as O

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def engine(cfg, W, dtype="float32", max_tokens=1024, max_slots=4):
    from krasis_amd import model_registry as R
    from krasis_amd.scheduler import BatchEngine
    spec = R.lufozen_spec(cfg)
    spec.fit(spec, lambda name: W[name].shape)
    eng = BatchEngine(spec, dtype=dtype, max_tokens=max_tokens, max_slots=max_slots)
    eng.load_arrays(W)
    return eng


def rel(got, ref):
    """largest row error, relative to the root mean square of the reference rows"""
    d = np.asarray(got, np.float64) - ref
    return float(np.sqrt((d ** 2).mean(-1)).max() / np.sqrt((ref ** 2).mean()))


def tokens(cfg, n, seed):
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


# sizes differ from layer to layer; key / value heads fewer than query heads (three to one, two to one, one to one); value width unlike key width; rotation
# on a part of a head and on all of it, with and without frequency scaling; 2, 3 and 5 taps; state-space heads in three groups; a layer without
# feed-forward; the repeated block in the middle, run twice
def cfg_varied():
    return O.make_config(width=96, vocab=101, embed_scale=1.7, bigram=(31, 13, 7), logit_scale=0.6, loop=(1, 4, 2), layers=[
        O.layer(O.attn(6, 2, 16, 10, scale=0.31, conv=3, rot=O.rot(8, 300.0, factor=3.0, low=1.0, high=5.0, original=48)), O.dense(40)),
        O.layer(O.parallel(O.left(4, 2, 24, 12, scale=0.2, rot=O.rot(24, 50.0)), O.ssd(3, 10, 7, groups=3, conv=2, norm_groups=3), 0.8, 0.45), O.dense(24)),
        O.layer(O.gla(3, 20, 12, tau=4.0), None),
        O.layer(O.attn(4, 4, 8, 8, scale=0.4, conv=5), O.dense(56)),
        O.layer(O.parallel(O.left(3, 3, 10, 14, scale=0.25), O.ssd(4, 6, 9, groups=1, conv=4, norm_groups=1), 1.0, 1.0), None),
    ])


def cfg_wide():
    """rows that are multiples of 16 bytes and head shapes of the matrix-instruction attention (four heads per key head and one, heads of 64 and 128); the
    repeated block opens the model and runs three times; recurrent heads of 64 keys; state-space heads of 32 channels over 16 states"""
    return O.make_config(width=128, vocab=260, eps=1e-6, embed_scale=8.0, bigram=(97, 29, 23), logit_scale=0.8, loop=(0, 2, 3), layers=[
        O.layer(O.attn(8, 2, 64, 64, scale=0.15, conv=4, rot=O.rot(32, 1e4, factor=8.0, low=1.0, high=4.0, original=128)), O.dense(96)),
        O.layer(O.parallel(O.left(8, 2, 128, 64, scale=0.09, rot=O.rot(32, 1e5, factor=4.0, low=1.0, high=4.0, original=256)), O.ssd(4, 32, 16, groups=2, conv=4, norm_groups=2),
                           0.7, 0.4), O.dense(64)),
        O.layer(O.gla(2, 64, 64, tau=12.0), None),
        O.layer(O.attn(16, 16, 32, 32, scale=0.2, conv=2), O.dense(160)),
    ])


@pytest.mark.parametrize("make,n", [(cfg_varied, 75), (cfg_wide, 200)])
def test_every_layer_and_logits_f32(make, n):
    cfg = make(); W = O.random_weights(cfg, 1); toks = tokens(cfg, n, 2)
    ref_logits, ref_streams = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    eng.store.set_capture(True)
    logits, amax = eng.step([("a", toks, list(range(n)))])
    streams = eng.store.read_capture(n)
    assert len(streams) == len(ref_streams)
    for li in range(len(ref_streams)):
        assert rel(streams[li], ref_streams[li]) < 2e-4, f"layer run {li}"
    assert rel(logits, ref_logits) < 2e-4
    assert np.array_equal(amax, logits.argmax(-1))


@pytest.mark.parametrize("make,n", [(cfg_varied, 75), (cfg_wide, 150)])
def test_bf16_store_close_to_oracle(make, n):
    cfg = make(); W = {k: O.bf16_round(v) for k, v in O.random_weights(cfg, 3).items()}; toks = tokens(cfg, n, 4)
    ref_logits, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W, "bfloat16")
    logits, _ = eng.step([("a", toks, list(range(n)))])
    e = np.sqrt(((logits - ref_logits) ** 2).mean(-1)) / np.sqrt((ref_logits ** 2).mean())
    assert np.median(e) < 2e-2 and e.max() < 6e-2


def small_model(layers, **kw):
    kw.setdefault("width", 64); kw.setdefault("vocab", 50)
    return O.make_config(layers=layers, **kw)


def far_below_zero_scores(W):
    """keys that point against the queries: every score is far below the sink's zero, and the sink takes nearly all of the weight"""
    W["l0.mix.k"] = (-3.0 * W["l0.mix.q"][:W["l0.mix.k"].shape[0]]).astype(np.float32)
    W["l0.mix.k.b"] = (-3.0 * W["l0.mix.q.b"][:W["l0.mix.k.b"].shape[0]]).astype(np.float32)


def slow_and_fast_heads(W):
    W["l0.mix.right.A_log"] = np.linspace(-6.0, 2.0, W["l0.mix.right.A_log"].size).astype(np.float32)
    W["l0.mix.right.dt_bias"] = np.linspace(-4.0, 3.0, W["l0.mix.right.dt_bias"].size).astype(np.float32)


def decays_over_the_whole_range(W):
    W["l0.mix.a2.b"] = np.linspace(-4.0, 9.0, W["l0.mix.a2.b"].size).astype(np.float32)


A8 = O.attn(2, 1, 8, 8)
MECHANISMS = [
    ("attention_one_tap", [O.layer(O.attn(2, 1, 8, 8, conv=1), None)], {}, None),
    ("attention_two_taps_three_heads_on_one_key_head", [O.layer(O.attn(3, 1, 8, 12, conv=2), None)], {}, None),
    ("attention_seven_taps", [O.layer(O.attn(4, 4, 16, 4, conv=7), None)], {}, None),
    ("attention_scores_far_below_the_sink", [O.layer(O.attn(4, 4, 16, 16, scale=1.0, conv=1), None)], {}, far_below_zero_scores),
    ("attention_rotation_on_all_of_a_head", [O.layer(O.attn(4, 2, 16, 16, rot=O.rot(16, 100.0)), None)], {}, None),
    ("attention_rotation_in_three_bands", [O.layer(O.attn(4, 2, 16, 8, rot=O.rot(12, 10.0, factor=4.0, low=1.0, high=4.0, original=40)), None)], {}, None),
    ("attention_on_the_matrix_path", [O.layer(O.attn(4, 4, 32, 32, rot=O.rot(32, 1e4, factor=2.0, low=2.0, high=8.0, original=32)), None)], {}, None),
    ("attention_thirty_two_heads_on_one_key_head", [O.layer(O.attn(32, 1, 32, 16, conv=2), None)], {}, None),
    ("parallel_weights_of_one_groups_of_one", [O.layer(O.parallel(O.left(2, 1, 8, 8), O.ssd(2, 8, 4, groups=1, conv=4, norm_groups=1), 1.0, 1.0), None)], {}, None),
    ("parallel_a_group_per_head_one_tap", [O.layer(O.parallel(O.left(2, 2, 8, 4, rot=O.rot(4, 20.0)), O.ssd(4, 5, 6, groups=4, conv=1, norm_groups=4), 0.3, 1.9), None)], {}, None),
    ("parallel_slow_and_fast_heads", [O.layer(O.parallel(O.left(2, 1, 16, 16), O.ssd(6, 20, 3, groups=2, conv=3, norm_groups=6), 0.5, 0.5), None)], {}, slow_and_fast_heads),
    ("parallel_state_of_one_wide_heads", [O.layer(O.parallel(O.left(4, 2, 32, 16, rot=O.rot(32, 500.0, factor=2.0, low=1.0, high=2.0, original=16)),
                                                               O.ssd(1, 72, 1, groups=1, conv=2, norm_groups=3), 0.6, 0.5), O.dense(24))], {}, None),
    ("parallel_states_of_130", [O.layer(O.parallel(O.left(2, 1, 8, 8), O.ssd(2, 16, 130, groups=2, conv=4, norm_groups=1), 0.7, 0.7), None)], {}, None),
    ("gla_root_of_one", [O.layer(O.gla(2, 16, 16, tau=1.0), None)], {}, None),
    ("gla_odd_sizes", [O.layer(O.gla(5, 10, 9, tau=3.0), None)], {}, None),
    ("gla_keys_of_200_wide_values", [O.layer(O.gla(1, 200, 72, tau=16.0), None)], {}, None),
    ("gla_decays_over_the_whole_range", [O.layer(O.gla(3, 12, 20, tau=2.0), O.dense(24))], {}, decays_over_the_whole_range),
    ("no_repeated_block", [O.layer(A8, O.dense(24)), O.layer(O.gla(2, 8, 8), None)], {}, None),
    ("whole_model_runs_once_as_a_block", [O.layer(A8, O.dense(24)), O.layer(O.gla(2, 8, 8), None)], {"loop": (0, 2, 1)}, None),
    ("last_layer_four_times", [O.layer(A8, None), O.layer(O.parallel(O.left(2, 1, 8, 8), O.ssd(2, 8, 4)), O.dense(24))], {"loop": (1, 2, 4)}, None),
    ("every_layer_twice_logits_and_embedding_as_they_are", [O.layer(O.gla(2, 8, 8), None), O.layer(A8, O.dense(16)), O.layer(O.parallel(O.left(2, 1, 8, 8), O.ssd(2, 8, 4)), None)],
     {"loop": (0, 3, 2), "logit_scale": 1.0, "embed_scale": 1.0}, None),
    ("pair_table_of_one_bucket", [O.layer(A8, O.dense(24))], {"bigram": (1, 3, 5)}, None),
    ("pair_hash_beyond_32_bits", [O.layer(A8, O.dense(24))], {"bigram": (1019, 2000003, 1999993), "vocab": 3000}, None),
]


@pytest.mark.parametrize("name,layers,kw,patch", MECHANISMS, ids=[m[0] for m in MECHANISMS])
def test_each_mechanism_alone(name, layers, kw, patch):
    cfg = small_model(layers, **kw)
    W = O.random_weights(cfg, 5)
    if patch:
        patch(W)
    toks = tokens(cfg, 40, 6)
    ref_logits, ref_streams = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    eng.store.set_capture(True)
    logits, _ = eng.step([("a", toks, list(range(40)))])
    got = eng.store.read_capture(40)
    for li in range(len(ref_streams)):
        assert rel(got[li], ref_streams[li]) < 2e-4, (name, li)
    assert rel(logits, ref_logits) < 2e-4, name
    eng.store.set_capture(False)
    # and the same tokens one by one, through the cache and the state
    rows = [eng.step([("d", [t], [0])])[0][0] for t in toks]
    assert rel(np.stack(rows), ref_logits) < 2e-4, name


def test_the_oracle_feels_every_mechanism(monkeypatch):
    """the oracle itself: leaving out the sink, a convolution, the pair table, the vector before a pass, the one in the norm weights, the frequency
    scaling, the skip term, the root of the decay, or putting the gate after the norm moves its result far beyond the tolerance the store is held to"""
    cfg = small_model([O.layer(O.attn(4, 2, 16, 12, scale=0.5, rot=O.rot(12, 10.0, factor=4.0, low=1.0, high=4.0, original=40)), O.dense(24)),
                       O.layer(O.parallel(O.left(2, 1, 16, 8, rot=O.rot(8, 30.0)), O.ssd(3, 8, 5, groups=1, conv=3, norm_groups=3)), None), O.layer(O.gla(2, 8, 12, tau=6.0), None)],
                      loop=(1, 3, 2))
    W = O.random_weights(cfg, 5); toks = tokens(cfg, 30, 6)
    base, _ = O.forward(cfg, W, toks)

    def changed(**patch):
        with monkeypatch.context() as m:
            for k, v in patch.items():
                m.setattr(O, k, v)
            return O.forward(cfg, W, toks)[0]

    def weights(**patch):
        W2 = dict(W); W2.update(patch)
        return O.forward(cfg, W2, toks)[0]

    def config(edit):
        c2 = json.loads(json.dumps(cfg)); edit(c2)
        return O.forward(c2, W, toks)[0]
    soft = O.softmax_attention
    assert rel(changed(softmax_attention=lambda q, k, v, s, g, sink: soft(q, k, v, s, g, False)), base) > 1e-2
    assert rel(changed(causal_conv=lambda u, w, bias=None: u if bias is None else u + bias), base) > 1e-2
    assert rel(changed(bigram_rows=lambda t, b, mp, mc: [b] * len(t)), base) > 1e-2
    assert rel(changed(norm_one_plus=lambda x, w, eps: O.rms_unit(x, eps) * w), base) > 1e-2
    assert rel(changed(rotate=lambda v, pos, r, inter: v), base) > 1e-2
    assert rel(changed(softplus=lambda z: np.maximum(z, 0.0)), base) > 1e-3
    assert rel(weights(**{"loop.step": np.zeros_like(W["loop.step"])}), base) > 1e-2
    assert rel(weights(**{"loop.step": W["loop.step"][::-1]}), base) > 1e-2
    assert rel(weights(**{"l1.mix.right.D": np.zeros_like(W["l1.mix.right.D"])}), base) > 1e-3
    assert rel(weights(**{"l0.mix.o.b": np.zeros_like(W["l0.mix.o.b"])}), base) > 1e-3
    assert rel(weights(**{"l0.mix.v.b": np.zeros_like(W["l0.mix.v.b"])}), base) > 1e-3
    assert rel(config(lambda c: c["layers"][0]["mixer"]["rot"].pop("scaling")), base) > 1e-3
    assert rel(config(lambda c: c["layers"][2]["mixer"].update(tau=1.0)), base) > 1e-3
    assert rel(config(lambda c: c["layers"][1]["mixer"]["right"].update(norm_groups=1)), base) > 1e-3
    assert rel(config(lambda c: c["layers"][1]["mixer"].update(left_scale=0.0)), base) > 1e-2
    assert rel(config(lambda c: c["loop"].update(times=1)), base) > 1e-2
    assert rel(config(lambda c: c.update(logit_scale=1.0)), base) > 1e-2


# ---------------------------------------------------------------------------------------------------------------- one key that decides
def peaked_attention_model(kind, dim=32, width=64, vocab=40):
    """attention that finds ONE key among hundreds: an empty pair table and convolutions that pass the current token only, so that a token's key and
    query depend on the token alone; the query projection is steered so that the query of token 1 points along the key of token 0.  After the
    per-head norms that key scores about 1.2 * dim against O(sqrt(dim)) for any other."""
    if kind == "attention":
        cfg = small_model([O.layer(O.attn(2, 1, dim, dim, scale=1.2, conv=3), None)], width=width, vocab=vocab)
        p = "l0.mix."
    else:
        cfg = small_model([O.layer(O.parallel(O.left(2, 1, dim, dim, scale=1.2), O.ssd(2, 8, 4), 1.0, 0.1), None)], width=width, vocab=vocab)
        p = "l0.mix.left."
    W = O.random_weights(cfg, 11)
    W["bigram"][:] = 0.0
    for n in ("q.b", "k.b"):
        if p + n in W:
            W[p + n][:] = 0.0
    for n in ("q.conv", "k.conv", "v.conv"):
        if p + n in W:
            W[p + n][:] = 0.0; W[p + n][:, -1] = 1.0
    W[p + "q.norm"][:] = 1.0; W[p + "k.norm"][:] = 1.0
    x = O.embed(cfg, {k: v.astype(np.float64) for k, v in W.items()}, [0])      # a first token's row; the pair table is empty, so any token 0 has it
    x1 = O.embed(cfg, {k: v.astype(np.float64) for k, v in W.items()}, [1])
    h0 = O.norm_one_plus(x[0], W["l0.norm1"].astype(np.float64), cfg["norm"]["eps"])
    h1 = O.norm_one_plus(x1[0], W["l0.norm1"].astype(np.float64), cfg["norm"]["eps"])
    k0 = W[p + "k"].astype(np.float64) @ h0
    steer = np.outer(np.concatenate([k0, k0]), h1) / (h1 @ h1)
    W[p + "q"] = (0.3 * W[p + "q"] + 2.0 * steer).astype(np.float32)
    return cfg, W


def needle_sequence(vocab, n, needle_at, query_at, seed):
    """random tokens 2.., token 0 (the needle) once, token 1 (the query) once"""
    t = [int(x) for x in np.random.default_rng(seed).integers(2, vocab, n)]
    t[needle_at] = 0; t[query_at] = 1
    return t


@pytest.mark.parametrize("kind", ["attention", "parallel"])
@pytest.mark.parametrize("needle,query", [(0, 1), (0, 63), (63, 64), (63, 127), (64, 128), (127, 128), (1, 128), (3, 700), (5, 450)])
def test_one_key_far_back_and_at_page_borders_prompt_and_decode(kind, needle, query):
    cfg, W = peaked_attention_model(kind)
    n = query + 3
    toks = needle_sequence(cfg["vocab"], n, needle, query, 19)
    ref, _ = O.forward(cfg, W, toks)
    moved = list(toks); moved[needle] = 7
    ref2, _ = O.forward(cfg, W, moved)
    assert rel(ref2[query:query + 1], ref[query:query + 1]) > 0.05      # the oracle's own sensitivity: that one key carries the query's answer
    eng = engine(cfg, W, max_tokens=1024)
    whole, _ = eng.step([("w", toks, [query - 1, query, query + 1])])
    assert rel(whole, ref[[query - 1, query, query + 1]]) < 2e-4
    eng.finish("w")
    cut = (query // 64) * 64 if query % 64 else query - 1       # the prompt cut at the page border before the query, then decoded
    cut = max(cut, 1)
    eng.step([("a", toks[:cut], [])])
    got = []
    for p in range(cut, query + 1):
        lg, _ = eng.step([("a", [toks[p]], [0])])
        got.append(lg[0])
    assert rel(np.stack(got), ref[cut:query + 1]) < 2e-4


def remembering_model(kind):
    """recurrent layers that keep a token for hundreds of positions: decays next to one"""
    if kind == "gla":
        cfg = small_model([O.layer(O.gla(2, 32, 24, tau=16.0), None)], vocab=12)
        W = O.random_weights(cfg, 12)
        W["l0.mix.a2.b"][:] = 7.0; W["l0.mix.a2"] *= 0.2
    else:
        cfg = small_model([O.layer(O.parallel(O.left(2, 1, 8, 8, scale=0.05), O.ssd(2, 24, 16, groups=1, conv=2, norm_groups=1), 0.05, 2.0), None)], vocab=12)
        W = O.random_weights(cfg, 12)
        W["l0.mix.right.A_log"][:] = -7.0; W["l0.mix.right.dt_bias"][:] = 0.0
    W["l0.mix.o" if kind == "gla" else "l0.mix.right.o"] *= 4.0
    return cfg, W


@pytest.mark.parametrize("kind", ["gla", "ssd"])
def test_far_token_among_hundreds_through_the_state(kind):
    """a token fed 700 positions earlier, in another step, still decides the answer: only the state can have carried it"""
    cfg, W = remembering_model(kind)
    n = 760
    toks = needle_sequence(8, n, 40, 740, 17)                    # fillers 2 .. 7
    ref, _ = O.forward(cfg, W, toks)
    toks_moved = list(toks); toks_moved[40] = 5
    ref_moved, _ = O.forward(cfg, W, toks_moved)
    assert rel(ref_moved[740:741], ref[740:741]) > 4e-3          # 20 times the tolerance below
    eng = engine(cfg, W, max_tokens=1024)
    eng.step([("a", toks[:300], []), ("other", toks_moved[:90], [])])
    eng.step([("a", toks[300:700], [])])
    lg, _ = eng.step([("a", toks[700:], [40]), ("other", toks_moved[90:95], [])])
    assert rel(lg, ref[740:741]) < 2e-4
    eng.finish("a")
    eng.step([("b", toks[:739], [])])
    eng.step([("b", toks[739:740], [])])
    lg, _ = eng.step([("b", toks[740:741], [0])])
    assert rel(lg, ref[740:741]) < 2e-4


def test_first_tokens_of_a_sequence():
    cfg = cfg_varied(); W = O.random_weights(cfg, 21); toks = tokens(cfg, 8, 22)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    one, _ = eng.step([("one", toks[:1], [0])])
    assert rel(one, ref[:1]) < 2e-4
    two, _ = eng.step([("two", toks[:2], [0, 1])])
    assert rel(two, ref[:2]) < 2e-4
    nxt, _ = eng.step([("one", toks[1:2], [0])])
    assert rel(nxt, ref[1:2]) < 2e-4
    rest, _ = eng.step([("one", toks[2:4], [0, 1]), ("two", toks[2:3], [0])])       # the convolutions reach back over three separate steps
    assert rel(rest, np.stack([ref[2], ref[3], ref[2]])) < 2e-4
    last, _ = eng.step([("two", toks[3:8], [0, 1, 2, 3, 4]), ("one", toks[4:5], [0])])
    assert rel(last, np.concatenate([ref[3:8], ref[4:5]])) < 2e-4


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-4), ("bfloat16", 5e-2)])
def test_prefill_equals_token_by_token_decode(dtype, tol):
    cfg = cfg_varied(); W = {k: O.bf16_round(v) for k, v in O.random_weights(cfg, 23).items()}; n = 90; toks = tokens(cfg, n, 24)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W, dtype)
    whole, _ = eng.step([("w", toks, list(range(n)))])
    rows = []
    for p in range(n):
        lg, _ = eng.step([("d", [toks[p]], [0])])
        rows.append(lg[0])
    assert rel(whole, ref) < tol and rel(np.stack(rows), ref) < tol


@pytest.mark.parametrize("sizes", [[2] * 30, [3, 2, 7, 2, 64, 5, 65, 2, 31, 2, 9], [37, 3, 3, 37, 37, 5, 11, 25, 24, 2], [1, 128, 2, 60], [1, 1, 2, 1, 3, 1, 1, 4]])
@pytest.mark.parametrize("make", [cfg_varied, cfg_wide])
def test_portions_of_several_sizes(make, sizes):
    cfg = make(); W = O.random_weights(cfg, 25); n = sum(sizes); toks = tokens(cfg, n, 26)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    at, rows = 0, []
    for s in sizes:
        lg, _ = eng.step([("c", toks[at:at + s], list(range(s)))])
        rows.append(lg); at += s
    assert rel(np.concatenate(rows), ref) < 2e-4


@pytest.mark.parametrize("make", [cfg_varied, cfg_wide])
def test_unequal_requests_in_one_batch_equal_each_alone(make):
    cfg = make(); W = O.random_weights(cfg, 27)
    lens = {"a": 70, "b": 9, "c": 131, "d": 33}
    toks = {k: tokens(cfg, n, 30 + i) for i, (k, n) in enumerate(lens.items())}
    refs = {k: O.forward(cfg, W, t)[0] for k, t in toks.items()}
    eng = engine(cfg, W, max_tokens=512)
    # a schedule that mixes portions with single tokens: every request advances by its own stride; 0 = the request sits this step out
    stride = {"a": [17, 1, 0, 30, 1, 20], "b": [2, 1, 1, 0, 0, 4], "c": [64, 1, 65, 0, 1], "d": [1, 1, 31]}
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    step = 0
    while any(at[k] < lens[k] for k in lens):
        entries, owners = [], []
        for k in lens:
            if at[k] >= lens[k]:
                continue
            s = stride[k][step] if step < len(stride[k]) else 1
            s = min(s, lens[k] - at[k])
            if s == 0:
                continue
            entries.append((k, toks[k][at[k]:at[k] + s], list(range(s)))); owners.append((k, s)); at[k] += s
        lg, _ = eng.step(entries)
        o = 0
        for k, s in owners:
            got[k].append(lg[o:o + s]); o += s
        step += 1
    for k in lens:
        assert rel(np.concatenate(got[k]), refs[k]) < 2e-4, k


def test_pages_and_slots_are_used_again():
    """a pool of five pages and four slots: requests come and go; the later ones run in pages and slots -- cache rows of every pass, convolution rows,
    matrix states, the previous token -- that the earlier ones gave back"""
    cfg = cfg_varied(); W = O.random_weights(cfg, 31)
    eng = engine(cfg, W, max_tokens=320, max_slots=4)
    assert eng.store.free_pages() == 5
    seqs = [tokens(cfg, n, 40 + i) for i, n in enumerate([130, 60, 64, 100, 65, 190, 20, 129])]
    refs = [O.forward(cfg, W, t)[0] for t in seqs]
    a, _ = eng.step([(0, seqs[0], [129]), (1, seqs[1], [59]), (2, seqs[2], [63])])      # 3 + 1 + 1 pages: the pool is full
    assert eng.store.free_pages() == 0
    with pytest.raises(RuntimeError):
        eng.step([(3, seqs[3], [0])])                        # no page left: refused, nothing changed
    assert rel(a, np.stack([refs[0][129], refs[1][59], refs[2][63]])) < 2e-4
    eng.finish(0); eng.finish(3)                            # request 3 was admitted (slot) but holds no page
    assert eng.store.free_pages() == 3
    b, _ = eng.step([(3, seqs[3], [99]), (4, seqs[4][:40], [39])])          # 2 + 1 pages, out of request 0's
    assert rel(b, np.stack([refs[3][99], refs[4][39]])) < 2e-4
    eng.finish(1); eng.finish(2)
    c, _ = eng.step([(4, seqs[4][40:], [24]), (3, [seqs[3][0]], [])])      # request 4 crosses into a second page (one that request 1 or 2 held)
    assert rel(c, refs[4][64:65]) < 2e-4
    eng.finish(3); eng.finish(4)
    assert eng.store.free_pages() == 5
    d, _ = eng.step([(5, seqs[5], [0, 189]), (6, seqs[6], [19])])
    assert rel(d, np.stack([refs[5][0], refs[5][189], refs[6][19]])) < 2e-4
    eng.finish(5)
    e, _ = eng.step([(7, seqs[7][:1], [0])])                # one token into a slot whose state another request filled
    f, _ = eng.step([(7, seqs[7][1:], [127]), (6, [3], [0])])
    assert rel(np.concatenate([e, f[:1]]), np.stack([refs[7][0], refs[7][128]])) < 2e-4


def test_long_decoding_through_pages():
    cfg = cfg_wide(); W = O.random_weights(cfg, 33); n = 330; toks = tokens(cfg, n, 34)
    ref, _ = O.forward(cfg, W, toks)
    eng = engine(cfg, W)
    eng.step([("a", toks[:20], [])])
    rows = []
    for p in range(20, n):
        lg, _ = eng.step([("a", [toks[p]], [0])])
        rows.append(lg[0])
    assert rel(np.stack(rows), ref[20:]) < 2e-4


def greedy_oracle(cfg, W, prompt, n_new):
    seq, out, margins = list(prompt), [], []
    for _ in range(n_new):
        lg = O.forward(cfg, W, seq)[0][-1]
        top = np.sort(lg)[-2:]
        margins.append(float(top[1] - top[0]))
        out.append(int(lg.argmax())); seq.append(out[-1])
    return out, min(margins)


def test_greedy_generation_through_the_scheduler():
    """five prompts, four slots, a pool that cannot hold all at once, a step budget that cuts prompts into portions"""
    cfg = cfg_varied(); W = O.random_weights(cfg, 35)
    prompts = [tokens(cfg, n, 50 + i) for i, n in enumerate([45, 3, 70, 18, 29])]
    eng = engine(cfg, W, max_tokens=256, max_slots=4)
    outs = eng.generate(prompts, 6, token_budget=32)
    assert eng.store.free_pages() == 4 and not eng.live()
    for p, o in zip(prompts, outs):
        want, margin = greedy_oracle(cfg, W, p, 6)
        if margin > 1e-3:                                   # a near-tie of the two best logits may fall either way in f32
            assert o == want
        else:
            assert o[0] == want[0] or margin < 1e-3


def test_sampling_uses_the_frameworks_sampler():
    cfg = cfg_varied(); W = O.random_weights(cfg, 37); p = tokens(cfg, 12, 38)
    eng = engine(cfg, W)
    a = eng.generate([p], 8, temperature=0.8, top_k=5, top_p=0.9, seed=7)
    b = eng.generate([p], 8, temperature=0.8, top_k=5, top_p=0.9, seed=7)
    assert a == b and len(a[0]) == 8
    g = eng.generate([p], 8)
    k1 = eng.generate([p], 8, temperature=1.3, top_k=1, seed=3)      # top_k = 1 is greedy whatever the temperature
    assert g == k1


def test_checkpoint_directory_command_line_and_trace_replay(tmp_path):
    cfg = cfg_varied(); W = {k: O.bf16_round(v) for k, v in O.random_weights(cfg, 39).items()}
    model = str(tmp_path / "model"); O.write_checkpoint(model, cfg, W)
    from krasis_amd import model_registry as R
    assert R.model_family(R.read_config(model)) == "serve:Lufozen"
    p1, p2 = tokens(cfg, 20, 60), tokens(cfg, 7, 61)
    env = dict(os.environ, PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-m", "krasis_amd", "generate", "--model", model, "--dtype", "float32", "--max-new-tokens", "4",
                          "--prompt", ",".join(map(str, p1)), "--prompt", ",".join(map(str, p2))], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [json.loads(x) for x in out.stdout.splitlines() if x.startswith("{")]
    for p, line in zip((p1, p2), lines):
        want, margin = greedy_oracle(cfg, W, p, 4)
        assert line["prompt"] == p and (line["tokens"] == want or margin < 1e-3)
    # trace replay: two requests, portions beside single tokens, one ends early and its slot is used again
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": p1[:11], "want": [10]}, {"id": "y", "tokens": p2[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": p1[11:12], "want": [0]}, {"id": "y", "tokens": p2[2:], "want": [0, 4]}], "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": p1[12:], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "z", "tokens": p2, "want": [6]}], "end": ["x", "z"]}]
    outdir = str(tmp_path / "out")
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", model, "--dtype", "float32", "--out", outdir, "--max-tokens", "128"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [x for x in r.stdout.splitlines() if x.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    r1, r2 = O.forward(cfg, W, p1)[0], O.forward(cfg, W, p2)[0]
    V = cfg["vocab"]
    g0 = np.fromfile(os.path.join(outdir, "0.f32"), "<f4").reshape(-1, V)
    g1 = np.fromfile(os.path.join(outdir, "1.f32"), "<f4").reshape(-1, V)
    g3 = np.fromfile(os.path.join(outdir, "3.f32"), "<f4").reshape(-1, V)
    assert not os.path.exists(os.path.join(outdir, "2.f32"))
    assert rel(g0, r1[10:11]) < 2e-4 and rel(g1, np.stack([r1[11], r2[2], r2[6]])) < 2e-4 and rel(g3, r2[6:7]) < 2e-4


def test_store_refuses_what_it_cannot_run():
    from krasis_amd import serve_store as S
    seq = dict(block_kind=S.BLOCK_SEQUENTIAL, norm_kind=S.NORM_RMS)
    att = dict(heads=4, kv_heads=2, dim=8, vdim=8)
    ssd = dict(ssd_heads=4, ssd_vdim=4, ssd_state=4, ssd_groups=2, ssd_conv=3, ssd_norm_groups=2)
    with pytest.raises(ValueError):          # a layer that uses the tensors of a later layer
        S.ServeStore(50, 32, [S.LayerSpec(**att, weights_of=2), S.LayerSpec(**att)], **seq)
    with pytest.raises(ValueError):          # ... or of a layer described otherwise
        S.ServeStore(50, 32, [S.LayerSpec(**att), S.LayerSpec(heads=4, kv_heads=4, dim=8, vdim=8, weights_of=1)], **seq)
    with pytest.raises(ValueError):          # a state-space mixer beside a recurrent one
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=4, dim=8, vdim=8, mixer_kind=S.MIX_RETENTION, side_mixer=S.MIX_SSD, **ssd)], **seq)
    with pytest.raises(ValueError):          # state-space heads that do not split into their groups
        S.ServeStore(50, 32, [S.LayerSpec(**att, side_mixer=S.MIX_SSD, **{**ssd, "ssd_groups": 3})], **seq)
    with pytest.raises(ValueError):          # gla without the rank of its decay projections
        S.ServeStore(50, 32, [S.LayerSpec(heads=4, kv_heads=4, dim=8, vdim=8, mixer_kind=S.MIX_GLA, decay_tau=2.0, lin_norm_weight=2)], **seq)
    with pytest.raises(ValueError):          # a convolution on projections a layer does not have
        S.ServeStore(50, 32, [S.LayerSpec(**att), S.LayerSpec(**att, kv_from=0, proj_conv=3)], **seq)
    st = S.ServeStore(50, 32, [S.LayerSpec(**att, pre_add=1), S.LayerSpec(**att, weights_of=1, pre_add=1)], **seq)
    with pytest.raises(RuntimeError):
        st.finalize()                                         # tensors missing
    with pytest.raises(ValueError):
        st.set_tensor(1, "q", np.zeros((32, 32), np.float32))   # the second run owns no projection
    st.set_tensor(1, "pre_add", np.zeros(32, np.float32))       # ... but its own vector
    with pytest.raises(ValueError):
        st.set_tensor(0, "ssd_in", np.zeros((4, 32), np.float32))  # no state-space mixer here
    with pytest.raises(ValueError):
        st.set_tensor(0, "v_bias", np.zeros(16, np.float32))    # the layer has no value bias


def test_graph_replays_equal_eager_steps():
    """decode steps replay a captured graph from their second visit on; every replay is compared with a store that runs eagerly, with eager steps of
    other shapes (a prompt portion of a third request) and host synchronisation between the replays"""
    cfg = cfg_wide(); W = O.random_weights(cfg, 41)
    a, b = tokens(cfg, 150, 42), tokens(cfg, 150, 43)
    c = tokens(cfg, 60, 44)
    eng_g, eng_e = engine(cfg, W, "bfloat16"), engine(cfg, W, "bfloat16")
    eng_e.store.set_use_graph(False)
    for eng in (eng_g, eng_e):
        eng.step([("a", a[:30], []), ("b", b[:7], [])])
    for i in range(100):
        entries = [("a", [a[30 + i]], [0]), ("b", [b[7 + i]], [0])]
        lg, am = eng_g.step(entries)
        le, ae = eng_e.step(entries)
        assert np.array_equal(lg, le) and np.array_equal(am, ae), i
        if i % 25 == 10:                                    # an eager step of another shape in between
            part = c[(i // 25) * 15:(i // 25) * 15 + 15]
            lg, _ = eng_g.step([("c", part, [14])]); le, _ = eng_e.step([("c", part, [14])])
            assert np.array_equal(lg, le)
    assert eng_g.store.graph_replays() >= 60 and eng_e.store.graph_replays() == 0
    lg, _ = eng_g.step([("a", [a[130]], [0])])
    ref = O.forward(cfg, {k: O.bf16_round(v) for k, v in W.items()}, a[:131])[0]
    e = np.sqrt(((lg[0] - ref[130]) ** 2).mean()) / np.sqrt((ref ** 2).mean())
    assert e < 5e-2


def test_state_space_mixer_as_a_layers_only_mixer():
    """the store's state-space mixer without an attention beside it (no registered design asks for that; another one may): plain RMS norms, no pair table"""
    from krasis_amd import model_registry as R, serve_store as S
    from krasis_amd.scheduler import BatchEngine
    rng = np.random.default_rng(3)
    width, vocab, m = 48, 30, O.ssd(3, 10, 6, groups=3, conv=3, norm_groups=2)
    cfgw = O.random_weights(small_model([O.layer(O.parallel(O.left(1, 1, 4, 4), m), None)], width=width, vocab=vocab), 9)
    W = {k: v for k, v in cfgw.items() if k.startswith("l0.mix.right.") or k in ("embed", "head")}
    W["l0.norm1"] = (1.0 + 0.1 * rng.standard_normal(width)).astype(np.float32); W["final.norm"] = (1.0 + 0.1 * rng.standard_normal(width)).astype(np.float32)

    def names(spec):
        yield -1, "embed", 0, "embed"
        yield -1, "final_norm_w", 0, "final.norm"
        yield -1, "head", 0, "head"
        yield 0, "norm_w", 0, "l0.norm1"
        for role, n in (("ssd_in", "in"), ("ssd_conv", "conv"), ("ssd_conv_b", "conv.b"), ("ssd_dt_bias", "dt_bias"), ("ssd_a_log", "A_log"), ("ssd_d", "D"), ("ssd_norm", "norm"), ("ssd_o", "o")):
            yield 0, role, 0, "l0.mix.right." + n
    layer = S.LayerSpec(heads=1, kv_heads=1, dim=1, vdim=1, mixer_kind=S.MIX_SSD, ssd_heads=3, ssd_vdim=10, ssd_state=6, ssd_groups=3, ssd_conv=3, ssd_norm_groups=2)
    spec = R.ServeModelSpec(vocab, width, S.NORM_RMS, 1e-5, [layer], names, block_kind=S.BLOCK_SEQUENTIAL, pre_norm=1, post_norm=0, norm_bias=0)
    eng = BatchEngine(spec, dtype="float32", max_tokens=256)
    eng.load_arrays(W)
    toks = [int(t) for t in rng.integers(0, vocab, 50)]
    w64 = {k: v.astype(np.float64) for k, v in W.items()}
    x = w64["embed"][toks]
    x = x + O.mixer_ssd(m, w64, "l0.mix.right.", O.rms_unit(x, 1e-5) * w64["l0.norm1"], 1e-5)
    ref = (O.rms_unit(x, 1e-5) * w64["final.norm"]) @ w64["head"].T
    whole, _ = eng.step([("w", toks, list(range(50)))])
    assert rel(whole, ref) < 2e-4
    rows = [eng.step([("d", toks[:7], [6])])[0][0]] + [eng.step([("d", [t], [0])])[0][0] for t in toks[7:]]
    assert rel(np.stack(rows), ref[6:]) < 2e-4


def test_many_workgroups_take_the_plain_walk_of_the_scan():
    """four prompts in one step, seven heads of 112 value columns: more workgroups than the pipelined form of the prompt scan is launched for, in the gla
    mixer and in a state-space mixer whose 130 states are beyond the block form"""
    cfg = small_model([O.layer(O.gla(7, 8, 112, tau=5.0), None),
                       O.layer(O.parallel(O.left(2, 1, 8, 8), O.ssd(7, 112, 130, groups=7, conv=2, norm_groups=1), 0.5, 0.8), O.dense(24))])
    W = O.random_weights(cfg, 51)
    seqs = {k: tokens(cfg, n, 52 + i) for i, (k, n) in enumerate((("a", 40), ("b", 33), ("c", 57), ("d", 36)))}
    eng = engine(cfg, W, max_tokens=512)
    lg, _ = eng.step([(k, t, [len(t) - 1, 0]) for k, t in seqs.items()])
    ref = np.concatenate([O.forward(cfg, W, t)[0][[len(t) - 1, 0]] for t in seqs.values()])
    assert rel(lg, ref) < 2e-4
    nxt, _ = eng.step([(k, [5], [0]) for k in seqs])        # the states the plain walk left continue in the decode form
    ref = np.stack([O.forward(cfg, W, t + [5])[0][-1] for t in seqs.values()])
    assert rel(nxt, ref) < 2e-4
