"""Plain float64 restatement of the Midisun design: one function per mechanism, whole sequences, no cache, no state object.

Nothing here is shared with krasis_amd: the serving store keeps a paged key / value cache, a ring of convolution inputs and matrix states per
request slot and runs ragged batches; this file recomputes every position from the whole token list with explicit loops over time.

Notation.  x_t: residual row of token t (position t, counted from 0).  A layer: h = gnorm(x) w1; x += sigmoid(R1 h + r1) * mixer(h + conv(h));
then, when it has a feed-forward, h = gnorm(x) w2; x += sigmoid(R2 h + r2) * ff(h).  Logits: head @ (gnorm(x) w_final)."""
import json
import os
import struct

import numpy as np


# ---------------------------------------------------------------------------------------------------------------- small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def tanh_cap(z, cap):
    return cap * np.tanh(z / cap)


def unit_rms(v, eps):
    """v / sqrt(mean(v^2) + eps) over the last axis"""
    return v / np.sqrt((v * v).mean(-1, keepdims=True) + eps)


def grouped_norm(x, w, groups, eps):
    """the row in `groups` equal consecutive parts, each divided by its own root mean square; then the weight"""
    T, W = x.shape
    return unit_rms(x.reshape(T, groups, W // groups), eps).reshape(T, W) * w


def input_convolution(h, taps_w):
    """h_t + sum_j w[:, j] h_(t - taps + 1 + j), rows before the sequence's start are zero"""
    T, W = h.shape
    taps = taps_w.shape[1]
    out = h.copy()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += taps_w[:, j] * h[s]
    return out


def head_slopes(H):
    return np.array([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])


def rotate_half_pairs(v, positions, dims, base):
    """v [T, heads, dim]: coordinate i < dims / 2 is paired with i + dims / 2; angle = position * base^(-2 i / dims); the rest passes"""
    out = v.copy()
    half = dims // 2
    for i in range(half):
        ang = positions * base ** (-2.0 * i / dims)
        c, s = np.cos(ang)[:, None], np.sin(ang)[:, None]
        a, b = v[:, :, i], v[:, :, i + half]
        out[:, :, i] = a * c - b * s
        out[:, :, i + half] = b * c + a * s
    return out


# ---------------------------------------------------------------------------------------------------------------- mixers
def windowed_sink_attention(q, k, v, scale, softcap, window, sinks, slopes):
    """q [T, H, d], k [T, G, d], v [T, G, dv].  Query i sees keys j with 0 <= i - j < window.  Score: scale * q.k, capped by softcap * tanh(. / softcap),
    minus slope_h * (i - j).  The softmax denominator also holds exp(sink_h), which has no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = max(0, i - window + 1)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            s = tanh_cap(s, softcap) - slopes[h] * (i - np.arange(lo, i + 1))
            m = max(s.max(), sinks[h])
            e = np.exp(s - m)
            out[i, h] = (e @ v[lo:i + 1, g]) / (e.sum() + np.exp(sinks[h] - m))
    return out


def attention_mixer(u, P, p, m, eps):
    T = u.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = u @ P[p + "q"].T + P[p + "q.b"]
    k = u @ P[p + "k"].T + P[p + "k.b"]
    v = k.reshape(T, G, d)                                   # the values are the keys as projected
    q = (unit_rms(q, eps) * P[p + "q.norm"]).reshape(T, H, d)      # one statistic over the whole projection
    k = (unit_rms(k, eps) * P[p + "k.norm"]).reshape(T, G, d)
    o = windowed_sink_attention(q, k, v, m["scale"], m["softcap"], m["mask"]["size"], P[p + "sink"], head_slopes(H))
    o = o * sigmoid(u @ P[p + "g"].T)[:, :, None]            # one gate per head
    return o.reshape(T, -1) @ P[p + "o"].T + P[p + "o.b"]


def retention_recurrence(q, k, v, decays):
    """S_t = decay_h S_(t-1) + k_t v_t^T; o_t = S_t^T q_t"""
    T, H, d = q.shape
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        S = np.zeros((d, v.shape[2]))
        for t in range(T):
            S = decays[h] * S + np.outer(k[t, h], v[t, h])
            out[t, h] = q[t, h] @ S
    return out


def retention_mixer(u, P, p, m, eps):
    T = u.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    pos = np.arange(T, dtype=np.float64)
    q = (u @ P[p + "q"].T).reshape(T, H, d)
    k = (u @ P[p + "k"].T).reshape(T, H, d)
    v = (u @ P[p + "v"].T).reshape(T, H, dv)
    rot = m.get("rot")
    if rot and rot["dims"]:
        q = rotate_half_pairs(q, pos, rot["dims"], rot["base"])
        k = rotate_half_pairs(k, pos, rot["dims"], rot["base"])
    o = retention_recurrence(q, k / np.sqrt(d), v, m["decay"])
    o = unit_rms(o, eps).reshape(T, -1) * silu(u @ P[p + "g"].T)
    return o @ P[p + "o"].T


def mlstm_recurrence(q, k, v, log_i, log_f):
    """running maximum m (starts at 0): m_t = max(f_t + m_(t-1), i_t); S_t = e^(f_t + m_(t-1) - m_t) S_(t-1) + e^(i_t - m_t) k_t v_t^T, n_t alike with k_t;
    o_t = S_t^T q_t / (max(|n_t . q_t|, e^(-m_t)) + 1e-6)"""
    T, H, d = q.shape
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        S = np.zeros((d, v.shape[2])); n = np.zeros(d); m = 0.0
        for t in range(T):
            m_new = max(log_f[t, h] + m, log_i[t, h])
            keep, take = np.exp(log_f[t, h] + m - m_new), np.exp(log_i[t, h] - m_new)
            S = keep * S + take * np.outer(k[t, h], v[t, h])
            n = keep * n + take * k[t, h]
            m = m_new
            out[t, h] = (q[t, h] @ S) / (max(abs(n @ q[t, h]), np.exp(-m)) + 1e-6)
    return out


def mlstm_mixer(u, P, p, m, eps):
    T = u.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (u @ P[p + "q"].T).reshape(T, H, d) / np.sqrt(d)
    k = (u @ P[p + "k"].T).reshape(T, H, d)
    v = (u @ P[p + "v"].T).reshape(T, H, dv)
    log_i = tanh_cap(u @ P[p + "i"].T + P[p + "i.b"], m["gate_cap"])
    log_f = log_sigmoid(tanh_cap(u @ P[p + "f"].T + P[p + "f.b"], m["gate_cap"]))
    o = mlstm_recurrence(q, k, v, log_i, log_f)
    o = unit_rms(o, eps).reshape(T, -1) * P[p + "norm"] * sigmoid(u @ P[p + "g"].T)
    return o @ P[p + "o"].T


# ---------------------------------------------------------------------------------------------------------------- feed-forward
def gated_ff(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def route(scores, correction, top, group_count, group_keep):
    """scores [E] = sigmoid(logits).  Choice scores = scores + correction.  Groups of neighbours; a group's score = the sum of its two largest choice
    scores; only the group_keep best groups stay eligible; the `top` largest eligible choice scores win (lowest index among equals); weights = the
    winners' scores without the correction, over their sum + 1e-20"""
    E = scores.shape[0]
    per = E // group_count
    choice = scores + correction
    gscore = [np.sort(choice[g * per:(g + 1) * per])[-2:].sum() for g in range(group_count)]
    kept = sorted(range(group_count), key=lambda g: (-gscore[g], g))[:group_keep]
    eligible = [e for e in range(E) if e // per in kept]
    ids = sorted(eligible, key=lambda e: (-choice[e], e))[:top]
    w = scores[ids]
    return ids, w / (w.sum() + 1e-20)


def moe_ff(h, P, p, mlp):
    r = mlp["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    out = np.zeros_like(h)
    s = sigmoid(h @ P[p + "router"].T)
    for t in range(h.shape[0]):
        ids, w = route(s[t], P[p + "correction"], r["top"], g["count"], g["keep"])
        for e, we in zip(ids, w):
            out[t] += we * gated_ff(h[t:t + 1], P[f"{p}e{e}.gate"], P[f"{p}e{e}.up"], P[f"{p}e{e}.down"])[0]
    return out


# ---------------------------------------------------------------------------------------------------------------- the model
MIXERS = {"attention": attention_mixer, "retention": retention_mixer, "mlstm": mlstm_mixer}


def forward(cfg, W, tokens):
    """logits [T, vocab] and the residual stream after every layer [layers, T, width]"""
    P = {k: np.asarray(v, np.float64) for k, v in W.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = P["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    streams = []
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = grouped_norm(x, P[p + "norm1"], groups, eps)
        gate = sigmoid(h @ P[p + "rg1"].T + P[p + "rg1.b"])
        u = input_convolution(h, P[p + "canon1"]) if cfg["canon"]["taps"] > 1 else h
        x = x + gate * MIXERS[lc["type"]](u, P, p + "mix.", lc["mixer"], eps)
        mlp = lc.get("mlp")
        if mlp is not None:
            h = grouped_norm(x, P[p + "norm2"], groups, eps)
            gate = sigmoid(h @ P[p + "rg2"].T + P[p + "rg2.b"])
            y = gated_ff(h, P[p + "mlp.gate"], P[p + "mlp.up"], P[p + "mlp.down"]) if mlp["kind"] == "dense" else moe_ff(h, P, p + "mlp.", mlp)
            x = x + gate * y
        streams.append(x.copy())
    return grouped_norm(x, P["final.norm"], groups, eps) @ P["head"].T, np.stack(streams)


# ---------------------------------------------------------------------------------------------------------------- configurations and weights
def attn(heads, kv_heads, dim, window, scale=0.3, softcap=20.0):
    return "attention", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": window}, "scale": scale, "softcap": softcap}


def retention(heads, dim, vdim, decay, rot_dims=None, base=10000.0):
    return "retention", {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay), "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base}}


def mlstm(heads, dim, vdim, gate_cap=10.0):
    return "mlstm", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, groups=1, keep=1):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def make_config(width, vocab, layers, eps=1e-5, groups=2, taps=3, embed_scale=2.0):
    return {"architecture": "Midisun", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups}, "canon": {"taps": taps},
            "embedding": {"scale": embed_scale}, "layers": layers}


def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    sh = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    for i, lc in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        sh[p + "norm1"] = (W,)
        if cfg["canon"]["taps"] > 1:
            sh[p + "canon1"] = (W, cfg["canon"]["taps"])
        sh[p + "rg1"] = (W, W); sh[p + "rg1.b"] = (W,)
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        if lc["type"] == "attention":
            G = m["kv_heads"]
            sh.update({p + "mix.q": (H * d, W), p + "mix.q.b": (H * d,), p + "mix.k": (G * d, W), p + "mix.k.b": (G * d,), p + "mix.q.norm": (H * d,),
                       p + "mix.k.norm": (G * d,), p + "mix.sink": (H,), p + "mix.g": (H, W), p + "mix.o": (W, H * dv), p + "mix.o.b": (W,)})
        else:
            sh.update({p + "mix.q": (H * d, W), p + "mix.k": (H * d, W), p + "mix.v": (H * dv, W), p + "mix.g": (H * dv, W), p + "mix.o": (W, H * dv)})
            if lc["type"] == "mlstm":
                sh.update({p + "mix.norm": (H * dv,), p + "mix.i": (H, W), p + "mix.i.b": (H,), p + "mix.f": (H, W), p + "mix.f.b": (H,)})
        mlp = lc.get("mlp")
        if mlp is not None:
            sh[p + "norm2"] = (W,); sh[p + "rg2"] = (W, W); sh[p + "rg2.b"] = (W,)
            if mlp["kind"] == "dense":
                sh.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
            else:
                E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
                sh[p + "mlp.router"] = (E, W); sh[p + "mlp.correction"] = (E,)
                for e in range(E):
                    sh.update({f"{p}mlp.e{e}.gate": (F, W), f"{p}mlp.e{e}.up": (F, W), f"{p}mlp.e{e}.down": (W, F)})
    return sh


def random_weights(cfg, seed):
    """float32 arrays by checkpoint name; matrices ~ N(0, 1 / fan-in) (a bit livelier for the small projections so that every mechanism moves the result)"""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if name in ("embed",):
            a = rng.standard_normal(shape)
        elif leaf in ("norm1", "norm2", "norm") or name == "final.norm":
            a = 1.0 + 0.2 * rng.standard_normal(shape)
        elif leaf == "canon1":
            a = 0.4 * rng.standard_normal(shape)
        elif leaf == "sink":
            a = rng.standard_normal(shape)
        elif leaf == "correction":
            a = 0.3 * rng.standard_normal(shape)
        elif leaf == "b":
            a = 0.3 * rng.standard_normal(shape)
        elif name.endswith("mlp.router"):
            a = 2.0 * rng.standard_normal(shape) / np.sqrt(shape[1])
        elif name.endswith("mix.i") or name.endswith("mix.f"):
            a = 3.0 * rng.standard_normal(shape) / np.sqrt(shape[1])
        elif len(shape) == 2:
            a = rng.standard_normal(shape) / np.sqrt(shape[1])
        else:
            a = rng.standard_normal(shape)
        out[name] = a.astype(np.float32)
    return out


def bf16_round(a):
    """float32 -> the nearest bfloat16 (ties to even), back as float32"""
    b = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
    return b.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def write_checkpoint(path, cfg, W):
    """config.json + model.safetensors with the weights as bfloat16 (their values rounded: the caller's oracle should use bf16_round of W)"""
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, a in W.items():
        raw = (np.ascontiguousarray(bf16_round(a), np.float32).view(np.uint32) >> 16).astype("<u2").tobytes()
        header[name] = {"dtype": "BF16", "shape": list(np.shape(a)), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw); at += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(path, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj))); f.write(hj)
        for b in blobs:
            f.write(b)
