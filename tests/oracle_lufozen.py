"""Float64 numpy restatement of the Lufozen design, one function per mechanism, whole sequence at once with explicit loops over time.

No cache, no state object, no code shared with the package: the recurrences are written as recurrences, the convolutions as sums over earlier
positions, attention as a full score matrix.  `forward(cfg, w, tokens)` returns the logits of every position and the residual stream after every
layer run.  `w` maps checkpoint tensor names to float arrays; `cfg` is the dictionary of config.json.
"""
import json
import math
import os
import struct

import numpy as np


def rms_unit(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm_one_plus(x, w, eps):
    """weight stored around zero"""
    return rms_unit(x, eps) * (1.0 + w)


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.where(z > 30.0, z, np.log1p(np.exp(np.minimum(z, 30.0))))


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    rows = []
    for i, t in enumerate(tokens):
        rows.append(buckets if i == 0 else (int(tokens[i - 1]) * mul_prev + int(t) * mul_cur) % buckets)
    return rows


def embed(cfg, w, tokens):
    e = cfg["embedding"]
    x = w["embed"][np.asarray(tokens)] * float(e.get("scale", 1.0))
    bg = e.get("bigram")
    if bg:
        x = x + w["bigram"][bigram_rows(tokens, int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"]))]
    return norm_one_plus(x, w["embed.norm"], cfg["norm"]["eps"])


def rot_frequencies(rot):
    """base^(-2i/dims), then the three-band rescaling by wavelength"""
    dims = int(rot["dims"])
    f = np.array([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for fi in f:
            wl = 2.0 * math.pi / fi
            if wl < orig / high:
                out.append(fi)
            elif wl > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = np.array(out)
    return f


def rotate(v, positions, rot, interleaved):
    """v [T, heads, dim]; the first rot.dims coordinates of every head turn, the rest pass"""
    if not rot or int(rot.get("dims", 0)) == 0:
        return v
    dims = int(rot["dims"])
    f = rot_frequencies(rot)
    out = v.copy()
    for t, p in enumerate(positions):
        for i in range(dims // 2):
            a = p * f[i]
            i0, i1 = (2 * i, 2 * i + 1) if interleaved else (i, i + dims // 2)
            u, s = v[t, :, i0], v[t, :, i1]
            out[t, :, i0] = u * math.cos(a) - s * math.sin(a)
            out[t, :, i1] = s * math.cos(a) + u * math.sin(a)
    return out


def causal_conv(u, taps_w, bias=None):
    """u [T, C], taps_w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), nothing before the start"""
    T, C = u.shape
    taps = taps_w.shape[1]
    y = np.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += taps_w[:, j] * u[s]
    if bias is not None:
        y = y + bias
    return y


def softmax_attention(q, k, v, scale, kv_heads, sink_one):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; causal; with sink_one the denominator carries an extra 1"""
    T, H, _ = q.shape
    rep = H // kv_heads
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // rep
        for i in range(T):
            s = (k[: i + 1, g] @ q[i, h]) * scale
            m = max(s.max(), 0.0) if sink_one else s.max()
            e = np.exp(s - m)
            den = e.sum() + (math.exp(-m) if sink_one else 0.0)
            out[i, h] = (e / den) @ v[: i + 1, g]
    return out


def mixer_attention(m, w, p, h, eps):
    """biased projections, a short convolution on q / k / v, per-head q / k norm, interleaved rotation, sink of score 0, element-wise sigmoid gate"""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = h @ w[p + "v"].T + w[p + "v.b"]
    if int(m.get("conv") or 0) > 0:
        q, k, v = causal_conv(q, w[p + "q.conv"]), causal_conv(k, w[p + "k.conv"]), causal_conv(v, w[p + "v.conv"])
    q = rms_unit(q.reshape(T, H, d), eps) * w[p + "q.norm"]
    k = rms_unit(k.reshape(T, G, d), eps) * w[p + "k.norm"]
    pos = list(range(T))
    q, k = rotate(q, pos, m.get("rot"), True), rotate(k, pos, m.get("rot"), True)
    o = softmax_attention(q, k, v.reshape(T, G, dv), float(m["scale"]), G, True).reshape(T, H * dv)
    o = o * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T + w[p + "o.b"]


def mixer_left(m, w, p, h, eps):
    """the attention half of a parallel mixer: no biases, half-split rotation, ordinary softmax"""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms_unit((h @ w[p + "q"].T).reshape(T, H, d), eps) * w[p + "q.norm"]
    k = rms_unit((h @ w[p + "k"].T).reshape(T, G, d), eps) * w[p + "k.norm"]
    v = (h @ w[p + "v"].T).reshape(T, G, dv)
    pos = list(range(T))
    q, k = rotate(q, pos, m.get("rot"), False), rotate(k, pos, m.get("rot"), False)
    o = softmax_attention(q, k, v, float(m["scale"]), G, False).reshape(T, H * dv)
    return o @ w[p + "o"].T


def mixer_ssd(m, w, p, h, eps):
    """selective state space with a scalar decay per head and token"""
    T = h.shape[0]
    nh, dv, N, G, ng = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m.get("norm_groups", 1))
    inner = nh * dv
    zz = h @ w[p + "in"].T
    z, xbc, dt = zz[:, :inner], zz[:, inner:2 * inner + 2 * G * N], zz[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, nh, dv)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    Cm = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[p + "dt_bias"])
    y = np.zeros((T, nh, dv))
    for hd in range(nh):
        g = hd // (nh // G)
        S = np.zeros((N, dv))
        rate = math.exp(float(w[p + "A_log"][hd]))
        for t in range(T):
            S = math.exp(-rate * dt[t, hd]) * S + dt[t, hd] * np.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ Cm[t, g] + w[p + "D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    y = rms_unit(y.reshape(T, ng, inner // ng), eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


def mixer_parallel(m, w, p, h, eps):
    return float(m["left_scale"]) * mixer_left(m["left"], w, p + "left.", h, eps) + float(m["right_scale"]) * mixer_ssd(m["right"], w, p + "right.", h, eps)


def mixer_gla(m, w, p, h, eps):
    """linear attention with a decay per key channel"""
    T = h.shape[0]
    H, d, dv, tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"])
    q = (h @ w[p + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ w[p + "k"].T).reshape(T, H, d)
    v = (h @ w[p + "v"].T).reshape(T, H, dv)
    alpha = sigmoid((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]).reshape(T, H, d) ** (1.0 / tau)
    o = np.zeros((T, H, dv))
    for hd in range(H):
        S = np.zeros((d, dv))
        for t in range(T):
            S = alpha[t, hd][:, None] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = (rms_unit(o, eps) * w[p + "norm"]).reshape(T, H * dv)
    return (o * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def feed_forward(mlp, w, p, h):
    if mlp.get("kind") != "dense":
        raise ValueError(mlp.get("kind"))
    return np.maximum(h @ w[p + "up"].T, 0.0) ** 2 @ w[p + "down"].T


MIXERS = {"attention": mixer_attention, "parallel": mixer_parallel, "gla": mixer_gla}


def layer_order(cfg):
    """(layer index, pass number or None when the run does not open a pass)"""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, None) for i in range(n)]
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    runs = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def forward(cfg, w, tokens):
    w = {k: np.asarray(v, np.float64) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    x = embed(cfg, w, tokens)
    streams = []
    for i, opens in layer_order(cfg):
        lc = cfg["layers"][i]
        if opens is not None:
            x = x + w["loop.step"][opens]
        x = x + MIXERS[lc["type"]](lc["mixer"], w, f"l{i}.mix.", norm_one_plus(x, w[f"l{i}.norm1"], eps), eps)
        if lc.get("mlp"):
            x = x + feed_forward(lc["mlp"], w, f"l{i}.mlp.", norm_one_plus(x, w[f"l{i}.norm2"], eps))
        streams.append(x.copy())
    logits = norm_one_plus(x, w["final.norm"], eps) @ w["head"].T * float(cfg.get("logit_scale", 1.0))
    return logits, np.stack(streams)


# ------------------------------------------------------------------------------------------------------------------------------------
# small configurations and random weights for the tests
# ------------------------------------------------------------------------------------------------------------------------------------
def rot(dims, base=10000.0, factor=None, low=1.0, high=4.0, original=64):
    r = {"dims": dims, "base": base}
    if factor is not None:
        r["scaling"] = {"factor": factor, "low": low, "high": high, "original": original}
    return r


def attn(heads, kv_heads, dim, vdim, scale=0.3, conv=3, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "conv": conv}
    if rot:
        m["rot"] = rot
    return "attention", m


def left(heads, kv_heads, dim, vdim, scale=0.3, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot:
        m["rot"] = rot
    return m


def ssd(heads, vdim, state, groups=1, conv=4, norm_groups=1):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def parallel(a, b, left_scale=0.7, right_scale=0.4):
    return "parallel", {"left": a, "right": b, "left_scale": left_scale, "right_scale": right_scale}


def gla(heads, dim, vdim, tau=8.0):
    return "gla", {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def make_config(width, vocab, layers, eps=1e-5, embed_scale=3.0, bigram=(53, 7, 11), loop=None, logit_scale=0.7):
    cfg = {"architecture": "Lufozen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers, "logit_scale": logit_scale,
           "embedding": {"scale": embed_scale, "bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def random_weights(cfg, seed, rank=6):
    rng = np.random.default_rng(seed)
    W, V = cfg["width"], cfg["vocab"]
    out = {}

    def mat(name, o, i, gain=1.0):
        out[name] = (rng.standard_normal((o, i)) * gain / math.sqrt(i)).astype(np.float32)

    def vec(name, n, mid=0.0, amp=0.1):
        out[name] = (mid + amp * rng.standard_normal(n)).astype(np.float32)
    out["embed"] = (rng.standard_normal((V, W)) * 0.5).astype(np.float32)
    out["bigram"] = (rng.standard_normal((cfg["embedding"]["bigram"]["buckets"] + 1, W)) * 0.8).astype(np.float32)
    vec("embed.norm", W); vec("final.norm", W)
    mat("head", V, W)
    times = int(cfg["loop"]["times"]) if cfg.get("loop") else 1
    out["loop.step"] = (0.4 * rng.standard_normal((times, W))).astype(np.float32)
    for i, lc in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        vec(p + "norm1", W)
        if lc["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(p + "mix.q", H * d, W); mat(p + "mix.k", G * d, W); mat(p + "mix.v", G * dv, W); mat(p + "mix.g", H * dv, W); mat(p + "mix.o", W, H * dv)
            vec(p + "mix.q.b", H * d, amp=0.3); vec(p + "mix.k.b", G * d, amp=0.3); vec(p + "mix.v.b", G * dv, amp=0.3); vec(p + "mix.o.b", W, amp=0.3)
            vec(p + "mix.q.norm", d, 1.0, 0.2); vec(p + "mix.k.norm", d, 1.0, 0.2)
            if m.get("conv"):
                for n, c in (("q", H * d), ("k", G * d), ("v", G * dv)):
                    out[p + f"mix.{n}.conv"] = (rng.standard_normal((c, m["conv"])) * 0.6).astype(np.float32)
        elif lc["type"] == "parallel":
            a, b = m["left"], m["right"]
            H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            mat(q + "q", H * d, W); mat(q + "k", G * d, W); mat(q + "v", G * dv, W); mat(q + "o", W, H * dv)
            vec(q + "q.norm", d, 1.0, 0.2); vec(q + "k.norm", d, 1.0, 0.2)
            nh, sv, N, sg = b["heads"], b["vdim"], b["state"], b["groups"]
            inner, cc = nh * sv, nh * sv + 2 * sg * N
            q = p + "mix.right."
            mat(q + "in", 2 * inner + 2 * sg * N + nh, W); mat(q + "o", W, inner)
            out[q + "conv"] = (rng.standard_normal((cc, b["conv"])) * 0.6).astype(np.float32)
            vec(q + "conv.b", cc, amp=0.2); vec(q + "dt_bias", nh, -0.5, 1.0); vec(q + "A_log", nh, -0.5, 1.0); vec(q + "D", nh, 1.0, 0.3); vec(q + "norm", inner, 1.0, 0.2)
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            q = p + "mix."
            mat(q + "q", H * d, W); mat(q + "k", H * d, W); mat(q + "v", H * dv, W); mat(q + "g", H * dv, W); mat(q + "o", W, H * dv)
            mat(q + "a1", rank, W); mat(q + "a2", H * d, rank, 2.0); vec(q + "a2.b", H * d, 2.0, 1.5); vec(q + "norm", dv, 1.0, 0.2)
        if lc.get("mlp"):
            vec(p + "norm2", W)
            mat(p + "mlp.up", lc["mlp"]["ff"], W); mat(p + "mlp.down", W, lc["mlp"]["ff"])
    return out


def bf16_round(a):
    """float32 -> the nearest bfloat16 (ties to even), back as float32"""
    b = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
    return b.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def write_checkpoint(path, cfg, W):
    """config.json + model.safetensors with the weights as bfloat16 (the caller's oracle should use bf16_round of W)"""
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
