"""Host-side parts of the Lufozen design that need no GPU: its config reader (every size and constant from config.json or a tensor's shape), the
expansion of a repeated block into layer runs, its tensor names, the registry's choice, a checkpoint round trip, and the oracle's own mechanisms
against closed forms."""
import math
import os

import numpy as np
import pytest

from krasis_amd import model_registry as R
from krasis_amd import serve_store as S
from tests import oracle_lufozen as O


def small_cfg():
    return O.make_config(width=48, vocab=37, eps=3e-6, embed_scale=2.5, bigram=(29, 5, 3), logit_scale=0.25, loop=(1, 3, 3), layers=[
        O.layer(O.attn(6, 3, 8, 10, scale=0.2, conv=4, rot=O.rot(6, 123.0, factor=2.0, low=0.5, high=3.0, original=40)), O.dense(20)),
        O.layer(O.parallel(O.left(4, 2, 12, 6, scale=0.15, rot=O.rot(12, 77.0)), O.ssd(6, 5, 7, groups=3, conv=2, norm_groups=5), 0.9, 0.3), None),
        O.layer(O.gla(2, 10, 14, tau=5.0), O.dense(16)),
        O.layer(O.attn(4, 4, 12, 12, scale=0.25, conv=1), O.dense(24)),
    ])


def test_config_reader_takes_every_size_and_constant_from_config():
    cfg = small_cfg()
    spec = R.lufozen_spec(cfg)
    assert (spec.vocab, spec.width, spec.norm_kind, spec.norm_eps, spec.embed_scale, spec.logit_scale, spec.bigram) == (37, 48, S.NORM_RMS, 3e-6, 2.5, 0.25, (29, 5, 3))
    assert (spec.block_kind, spec.pre_norm, spec.post_norm, spec.norm_bias, spec.norm_weight_offset, spec.embed_norm) == (S.BLOCK_SEQUENTIAL, 1, 0, 0, 1.0, 1)
    # layer runs: 0 | 1 2 | 1 2 | 1 2 | 3; the repeats use the first run's tensors, every pass opens with its own vector
    assert len(spec.layers) == 8
    assert [l.weights_of for l in spec.layers] == [0, 0, 0, 2, 3, 2, 3, 0]
    assert [l.pre_add for l in spec.layers] == [0, 1, 0, 1, 0, 1, 0, 0]
    a, b, c = spec.layers[0], spec.layers[1], spec.layers[2]
    assert (a.mixer_kind, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.proj_conv, a.proj_bias, a.out_gate, a.has_sink, a.qk_unit_norm) == \
        (S.MIX_ATTENTION, 6, 3, 8, 10, 0.2, 4, 2, S.OGATE_ELEM_SIGMOID, S.SINK_ZERO, S.QKNORM_WEIGHTED)
    assert (a.rot_dims, a.rot_interleaved, a.rot_base, a.rot_scaling, a.rot_factor, a.rot_slow, a.rot_fast, a.rot_original) == (6, 1, 123.0, S.ROT_BANDS, 2.0, 0.5, 3.0, 40.0)
    assert (a.mlp_kind, a.ff, a.dense_act, a.window) == (S.MLP_DENSE, 20, S.ACT_RELU2, 0)
    assert (b.mixer_kind, b.side_mixer, b.heads, b.kv_heads, b.dim, b.vdim, b.scale, b.has_sink, b.proj_bias, b.proj_conv, b.out_gate) == (S.MIX_ATTENTION, S.MIX_SSD, 4, 2, 12, 6, 0.15, 0, 0, 0, 0)
    assert (b.rot_dims, b.rot_interleaved, b.rot_scaling, b.rot_base) == (12, 0, S.ROT_LINEAR, 77.0)
    assert (b.ssd_heads, b.ssd_vdim, b.ssd_state, b.ssd_groups, b.ssd_conv, b.ssd_norm_groups, b.mix_scale, b.side_scale, b.mlp_kind) == (6, 5, 7, 3, 2, 5, 0.9, 0.3, S.MLP_NONE)
    assert (c.mixer_kind, c.heads, c.kv_heads, c.dim, c.vdim, c.decay_tau, c.lin_norm_weight, c.decay_rank) == (S.MIX_GLA, 2, 2, 10, 14, 5.0, 2, 0)
    W = O.random_weights(cfg, 0, rank=9)
    spec.fit(spec, lambda name: W[name].shape)      # the rank of the decay projections is the checkpoint's
    assert [l.decay_rank for l in spec.layers] == [0, 0, 9, 0, 9, 0, 9, 0]
    names = [n for _, _, _, n in spec.tensors(spec)]
    assert [n for n in names if n.startswith("loop.step")] == ["loop.step@0", "loop.step@1", "loop.step@2"]
    assert {n.split("@")[0] for n in names} == set(W)          # the store asks for exactly the checkpoint's tensors, each layer's once
    assert len([n for n in names if n == "l1.mix.left.q"]) == 1
    last = spec.layers[7]
    assert (last.proj_conv, last.rot_dims, last.kv_heads) == (1, 0, 4)


def test_layer_runs_for_every_place_of_the_repeated_block():
    def runs(loop, n=4):
        cfg = small_cfg()
        if loop is None:
            cfg.pop("loop")
        else:
            cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
        spec = R.lufozen_spec(cfg)
        return [(spec.row_of[f"layer{r}"], l.weights_of, spec.row_of.get(f"run{r}")) for r, l in enumerate(spec.layers)]
    assert runs(None) == [(0, 0, None), (1, 0, None), (2, 0, None), (3, 0, None)]
    assert runs((0, 2, 2)) == [(0, 0, 0), (1, 0, None), (0, 1, 1), (1, 2, None), (2, 0, None), (3, 0, None)]
    assert runs((3, 4, 3)) == [(0, 0, None), (1, 0, None), (2, 0, None), (3, 0, 0), (3, 4, 1), (3, 4, 2)]
    assert runs((0, 4, 1)) == [(0, 0, 0), (1, 0, None), (2, 0, None), (3, 0, None)]
    assert runs((2, 2, 5)) == [(0, 0, None), (1, 0, None), (2, 0, None), (3, 0, None)]      # an empty block: nothing runs again, no vector joins
    assert [x[0] for x in runs((1, 3, 2))] == [i for i, _ in O.layer_order({**small_cfg(), "loop": {"start": 1, "stop": 3, "times": 2}})]
    with pytest.raises(ValueError):
        runs((3, 2, 2))
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["type"] = "retention"; R.lufozen_spec(bad)
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["mlp"]["kind"] = "moe"; R.lufozen_spec(bad)


def test_registry_and_checkpoint_roundtrip(tmp_path):
    assert {"Lufozen", "Midisun", "Pamulix", "Lomutar"} <= set(R.architectures())
    cfg = small_cfg(); W = O.random_weights(cfg, 0)
    assert R.model_family(cfg) == "serve:Lufozen"
    O.write_checkpoint(str(tmp_path), cfg, W)
    f = R.SafetensorsFile(os.path.join(tmp_path, "model.safetensors"))
    assert sorted(f.names()) == sorted(W)
    assert f.shape("l2.mix.a1") == (6, 48) and f.shape("loop.step") == (3, 48) and f.shape("bigram") == (30, 48)
    got = f.get("l1.mix.right.A_log")
    assert got.dtype == np.uint16 and np.array_equal((got.astype(np.uint32) << 16).view(np.float32), O.bf16_round(W["l1.mix.right.A_log"]))


def test_oracle_mechanisms_against_closed_forms():
    rng = np.random.default_rng(0)
    # pair rows: the first token takes the last row, later ones the hash of (previous, current)
    assert O.bigram_rows([3, 4, 4], 29, 5, 3) == [29, (3 * 5 + 4 * 3) % 29, (4 * 5 + 4 * 3) % 29]
    # the three bands of the frequency scaling: wavelengths 2 pi / f against original / high and original / low
    r = O.rot(8, 10.0, factor=4.0, low=1.0, high=4.0, original=40)
    f0 = np.array([10.0 ** (-2.0 * i / 8) for i in range(4)])      # wavelengths 6.3, 11.2, 19.9, 35.3, 62.8 ...: below 10 kept, above 40 divided
    f = O.rot_frequencies(r)
    assert f[0] == f0[0]
    mid = [(40 / (2 * math.pi / x) - 1.0) / 3.0 for x in f0[1:4]]
    assert np.allclose(f[1:4], [(1 - s) * x / 4 + s * x for s, x in zip(mid, f0[1:4])]) and all(0 < s < 1 for s in mid)
    r2 = O.rot(4, 1e4, factor=8.0, low=1.0, high=4.0, original=40)
    assert np.allclose(O.rot_frequencies(r2), [1.0, 1e-2 / 8.0])
    # rotation: position 0 leaves a vector alone; pairs (2i, 2i + 1) or (i, i + dims / 2); the tail past dims passes
    x = rng.standard_normal((4, 1, 10))
    for inter, (i0, i1) in ((True, (2, 3)), (False, (1, 4))):
        y = O.rotate(x, range(4), O.rot(6, 50.0), inter)
        assert np.array_equal(y[0], x[0]) and np.array_equal(y[:, :, 6:], x[:, :, 6:])
        ang = 3 * 50.0 ** (-2.0 / 6)
        assert np.allclose(y[3, 0, i0], x[3, 0, i0] * np.cos(ang) - x[3, 0, i1] * np.sin(ang)) and np.allclose(y[3, 0, i1], x[3, 0, i1] * np.cos(ang) + x[3, 0, i0] * np.sin(ang))
    # convolution: the last column is the current token's
    u = rng.standard_normal((5, 2)); w = rng.standard_normal((2, 3))
    y = O.causal_conv(u, w)
    assert np.allclose(y[0], w[:, 2] * u[0]) and np.allclose(y[4], w[:, 0] * u[2] + w[:, 1] * u[3] + w[:, 2] * u[4])
    # the sink: with scores far below zero the weights vanish; without it they sum to one
    q = np.ones((3, 1, 2)); k = -np.ones((3, 1, 2)) * 20; v = np.ones((3, 1, 1))
    assert np.all(O.softmax_attention(q, k, v, 1.0, 1, True) < 1e-15) and np.allclose(O.softmax_attention(q, k, v, 1.0, 1, False), 1.0)
    # gla: o_t = sum_s (prod_{s < r <= t} alpha_r) . k_s . q_t v_s per key channel
    cfg = O.make_config(16, 11, [O.layer(O.gla(1, 3, 2, tau=2.0), None)])
    W = {k_: v_.astype(np.float64) for k_, v_ in O.random_weights(cfg, 1, rank=2).items()}
    h = rng.standard_normal((6, 16))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    got = O.mixer_gla(m, W, p, h, 1e-5)
    qq = (h @ W[p + "q"].T) * 3 ** -0.5; kk = h @ W[p + "k"].T; vv = h @ W[p + "v"].T
    al = np.sqrt(O.sigmoid((h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]))
    o = np.zeros((6, 2))
    for t in range(6):
        for s_ in range(t + 1):
            o[t] += ((qq[t] * kk[s_] * np.prod(al[s_ + 1:t + 1], axis=0)).sum()) * vv[s_]
    want = (O.rms_unit(o, 1e-5) * W[p + "norm"] * O.silu(h @ W[p + "g"].T)) @ W[p + "o"].T
    assert np.allclose(got, want)
