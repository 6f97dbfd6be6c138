"""Host-side parts of the Midisun design that need no GPU: its config reader (every size and constant from config.json, the constants the design fixes
from the code), its tensor names, the registry's choice, a checkpoint round trip, and the oracle's own recurrences against closed forms."""
import os

import numpy as np
import pytest

from krasis_amd import model_registry as R
from krasis_amd import serve_store as S
from tests import oracle_midisun as O


def small_cfg():
    return O.make_config(width=48, vocab=37, eps=3e-6, groups=6, taps=5, embed_scale=2.5, layers=[
        O.layer(O.retention(3, 10, 14, [0.5, 0.75, 0.875], rot_dims=6, base=123.0), O.moe(10, 3, 6, groups=5, keep=2)),
        O.layer(O.attn(6, 3, 8, 9, scale=0.2, softcap=7.5), None),
        O.layer(O.mlstm(2, 8, 12, gate_cap=3.5), O.dense(20)),
        O.layer(O.attn(4, 4, 12, 21, scale=0.25, softcap=50.0), O.moe(7, 7, 9)),
    ])


def test_config_reader_takes_every_size_and_constant_from_config():
    spec = R.midisun_spec(small_cfg())
    assert (spec.vocab, spec.width, spec.norm_kind, spec.norm_eps, spec.norm_groups, spec.canon_taps, spec.embed_scale) == (37, 48, S.NORM_RMS, 3e-6, 6, 5, 2.5)
    assert (spec.block_kind, spec.pre_norm, spec.post_norm, spec.norm_bias, spec.res_gate) == (S.BLOCK_SEQUENTIAL, 1, 0, 0, 1)
    a, b, c, d = spec.layers
    assert (a.mixer_kind, a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims, a.rot_interleaved, a.rot_base) == (S.MIX_RETENTION, 3, 3, 10, 14, 6, 0, 123.0)
    assert np.array_equal(spec.extra["l0.mix.decay"], np.asarray([0.5, 0.75, 0.875], np.float32))
    assert (a.mlp_kind, a.experts, a.top, a.groups, a.keep, a.renorm, a.router_bias, a.router_score, a.group_score, a.expert_ff, a.expert_act) == \
        (S.MLP_MOE, 10, 3, 5, 2, 1, S.RBIAS_CHOICE, S.RSCORE_SIGMOID, S.GSCORE_TOP2, 6, S.ACT_SILU)
    assert (b.mixer_kind, b.heads, b.kv_heads, b.dim, b.vdim, b.window, b.scale, b.softcap, b.rot_dims, b.mlp_kind) == (S.MIX_ATTENTION, 6, 3, 8, 8, 9, 0.2, 7.5, 0, S.MLP_NONE)
    assert (b.has_sink, b.dist_bias, b.dist_bias_exp, b.qk_unit_norm, b.proj_bias, b.v_from_k, b.out_gate) == (S.SINK_TENSOR, 1, 8.0, S.QKNORM_WHOLE, 1, 1, S.OGATE_HEAD_SIGMOID)
    assert (c.mixer_kind, c.heads, c.dim, c.vdim, c.gate_cap, c.lin_norm_weight, c.mlp_kind, c.ff, c.dense_act) == (S.MIX_MLSTM, 2, 8, 12, 3.5, 1, S.MLP_DENSE, 20, S.ACT_SILU)
    assert (d.window, d.softcap, d.top, d.experts, d.groups, d.keep) == (21, 50.0, 7, 7, 1, 1)
    names = [n for _, _, _, n in spec.tensors(spec)]
    assert {"l0.mix.q", "l0.mix.k", "l0.mix.v", "l0.mix.g", "l0.mix.o", "l0.canon1", "l0.rg1", "l0.rg1.b", "l0.rg2", "l0.rg2.b", "l0.norm1", "l0.norm2"} <= set(names)
    assert "l0.mix.norm" not in names and "l2.mix.norm" in names and {"l2.mix.i", "l2.mix.i.b", "l2.mix.f", "l2.mix.f.b"} <= set(names)
    assert "l1.mix.v" not in names and {"l1.mix.q.b", "l1.mix.k.b", "l1.mix.o.b", "l1.mix.q.norm", "l1.mix.k.norm", "l1.mix.sink"} <= set(names)
    assert "l1.norm2" not in names and "l1.rg2" not in names and "l1.rg1" in names
    assert "l0.mlp.correction" in names and "l3.mlp.e6.down" in names and "l3.mlp.e7.down" not in names and "l2.mlp.down" in names
    W = O.random_weights(small_cfg(), 0)
    assert set(names) - set(spec.extra) <= set(W) and set(W) <= set(names)      # the store asks for exactly the checkpoint's tensors plus the decays of the config
    one_tap = small_cfg(); one_tap["canon"]["taps"] = 1
    s1 = R.midisun_spec(one_tap)
    assert s1.canon_taps == 0 and "l0.canon1" not in [n for _, _, _, n in s1.tensors(s1)]
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["type"] = "latent_attention"; R.midisun_spec(bad)
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["mlp"]["kind"] = "gelu"; R.midisun_spec(bad)
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][0]["mixer"]["decay"] = [0.5, 0.6]; R.midisun_spec(bad)
    with pytest.raises(ValueError):
        bad = small_cfg(); bad["layers"][1]["mixer"]["vdim"] = 12; R.midisun_spec(bad)


def test_registry_and_checkpoint_roundtrip(tmp_path):
    assert {"Midisun", "Pamulix", "Lomutar"} <= set(R.architectures())
    cfg = small_cfg(); W = O.random_weights(cfg, 0)
    assert R.model_family(cfg) == "serve:Midisun"
    O.write_checkpoint(str(tmp_path), cfg, W)
    f = R.SafetensorsFile(os.path.join(tmp_path, "model.safetensors"))
    assert sorted(f.names()) == sorted(W)
    got = f.get("l1.mix.sink")
    assert got.dtype == np.uint16 and np.array_equal((got.astype(np.uint32) << 16).view(np.float32), O.bf16_round(W["l1.mix.sink"]))
    assert R.read_config(str(tmp_path))["embedding"]["scale"] == 2.5


def test_oracle_recurrences_against_closed_forms():
    rng = np.random.default_rng(0)
    T, H, d, dv = 9, 2, 5, 3
    q, k, v = rng.standard_normal((T, H, d)), rng.standard_normal((T, H, d)), rng.standard_normal((T, H, dv))
    dec = [0.8, 1.0]
    o = O.retention_recurrence(q, k, v, dec)
    for h in range(H):      # o_t = sum_s decay^(t - s) (q_t . k_s) v_s
        for t in range(T):
            want = sum(dec[h] ** (t - s) * (q[t, h] @ k[s, h]) * v[s, h] for s in range(t + 1))
            assert np.allclose(o[t, h], want)
    li, lf = rng.standard_normal((T, H)) * 3, -np.abs(rng.standard_normal((T, H)))
    o = O.mlstm_recurrence(q, k, v, li, lf)
    for h in range(H):      # the running maximum only rescales numerator and denominator: unstabilised sums, with the floor exp(-m) scaled back
        for t in range(T):
            wgt = [np.exp(li[s, h] + lf[s + 1:t + 1, h].sum()) for s in range(t + 1)]
            num = sum(w * (q[t, h] @ k[s, h]) * v[s, h] for s, w in enumerate(wgt))
            den = sum(w * (q[t, h] @ k[s, h]) for s, w in enumerate(wgt))
            m = 0.0
            for s in range(t + 1):
                m = max(lf[s, h] + m, li[s, h])
            assert np.allclose(o[t, h], num * np.exp(-m) / (max(abs(den) * np.exp(-m), np.exp(-m)) + 1e-6))
    # rotation: position 0 leaves a vector as it is; the pair (i, i + dims / 2) turns by position * base^(-2 i / dims); the tail passes
    x = rng.standard_normal((4, 1, 10))
    y = O.rotate_half_pairs(x, np.arange(4.0), 6, 50.0)
    assert np.array_equal(y[0], x[0]) and np.array_equal(y[:, :, 6:], x[:, :, 6:])
    ang = 3 * 50.0 ** (-2.0 / 6)
    assert np.allclose(y[3, 0, 1], x[3, 0, 1] * np.cos(ang) - x[3, 0, 4] * np.sin(ang)) and np.allclose(y[3, 0, 4], x[3, 0, 4] * np.cos(ang) + x[3, 0, 1] * np.sin(ang))
    # router: the group limit beats a larger score outside the kept groups; weights come from the uncorrected scores
    s = np.array([0.9, 0.1, 0.5, 0.6, 0.2, 0.3]); corr = np.array([0.0, 0.0, 0.0, 0.0, 0.3, 0.0])
    ids, w = O.route(s, corr, 2, 3, 1)
    assert ids == [3, 2] and np.allclose(w, [0.6 / 1.1, 0.5 / 1.1])
    ids, w = O.route(s, corr, 2, 1, 1)
    assert ids == [0, 3]
    ids, w = O.route(s, corr, 3, 3, 2)          # group sums 1.0, 1.1, 0.8: groups 1 and 0 stay; expert 4's corrected 0.5 is out
    assert ids == [0, 3, 2]
