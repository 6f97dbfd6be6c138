"""Float64 numpy restatement of the Lufozen design, one function per mechanism, whole sequence at once with explicit loops over time.

No cache, no state object, no code shared with the package: the recurrences are written as recurrences, the convolutions as sums over earlier
positions, attention as a full score matrix.  `forward(cfg, w, tokens)` returns the logits of every position and the residual stream after every
layer run.  `w` maps checkpoint tensor names to float arrays; `cfg` is the dictionary of config.json.
"""
import math

import numpy as np


def rms_unit(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm_one_plus(x, w, eps):
    """weight stored around zero"""
    return rms_unit(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


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
