"""Model registry: config.json -> the class that serves the checkpoint.

Two families of engines live in this package:
  * `CpuDecoder` (decode_setup.py): the quantized single-request decode graph of the HF model types (`model_type` in config.json);
  * `BatchEngine` (scheduler.py): the batched serving store for designs described layer by layer (`architecture` in config.json), bf16 / f32
    weights, paged cache, several requests per step.
`load_model(model_dir, ...)` picks by config.json.  A new layer-described design registers a function that turns its config.json into
`LayerSpec`s and names its tensors (`register_architecture`); the mechanisms themselves (rotation, unit norm, window, sink, borrowed cache,
group-limited router, clamped gated activation) are parameters of the serving store, not code of the design."""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass
from typing import Callable, Dict, Iterator, List, Optional, Tuple

import numpy as np

from . import serve_store as S


# ------------------------------------------------------------------------------------------------------------------------------------
# safetensors without a tensor library: 8-byte little-endian header length, JSON header (name -> dtype, shape, data_offsets), raw data
# ------------------------------------------------------------------------------------------------------------------------------------
class SafetensorsFile:
    _DT = {"BF16": (np.uint16, 2), "F32": (np.float32, 4), "I32": (np.int32, 4), "F16": (np.float16, 2), "I64": (np.int64, 8)}

    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            (n,) = struct.unpack("<Q", f.read(8))
            if n > (1 << 30):
                raise IOError(f"{path}: header of {n} bytes")
            self.meta = json.loads(f.read(n))
        self.meta.pop("__metadata__", None)
        self._base = 8 + n
        self._map = np.memmap(path, dtype=np.uint8, mode="r")

    def names(self) -> List[str]:
        return list(self.meta)

    def has(self, name: str) -> bool:
        return name in self.meta

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.meta[name]["shape"])

    def get(self, name: str) -> np.ndarray:
        """BF16 tensors come back as uint16 bit patterns, F32 as float32 (what ServeStore.set_tensor takes)"""
        m = self.meta.get(name)
        if m is None:
            raise IOError(f"tensor {name} not found in {self.path}")
        if m["dtype"] not in self._DT:
            raise IOError(f"tensor {name}: dtype {m['dtype']} not handled")
        dt, sz = self._DT[m["dtype"]]
        lo, hi = m["data_offsets"]
        n = int(np.prod(m["shape"])) if m["shape"] else 1
        if hi - lo != n * sz:
            raise IOError(f"tensor {name}: {hi - lo} bytes for shape {m['shape']}")
        a = np.frombuffer(self._map, dtype=dt, count=n, offset=self._base + lo).reshape(m["shape"])
        if m["dtype"] == "F16":
            a = a.astype(np.float32)
        return a


# ------------------------------------------------------------------------------------------------------------------------------------
# layer-described designs
# ------------------------------------------------------------------------------------------------------------------------------------
@dataclass
class ServeModelSpec:
    vocab: int
    width: int
    norm_kind: int
    norm_eps: float
    layers: List[S.LayerSpec]
    tensors: Callable[["ServeModelSpec"], Iterator[Tuple[int, str, int, str]]]      # (layer, role, index, tensor name)
    # how a layer is put together (`kr_serve_config` in include/krasis_hip.h); the defaults are one pre-normed block with mixer and feed-forward side by side
    block_kind: int = S.BLOCK_PARALLEL
    pre_norm: int = 1
    post_norm: int = 0
    norm_bias: Optional[int] = None      # None: layer norms carry a bias, RMS norms do not
    residual_mult: float = 1.0
    norm_groups: int = 0                 # > 1: every norm works on that many equal parts of the row
    embed_scale: float = 0.0             # 0: the embedding row as it is
    canon_taps: int = 0                  # > 1: the mixers read h + a causal convolution of h over the request's positions
    res_gate: int = 0                    # 1: sublayer outputs are gated by sigmoid(W h + b) before they join the stream
    extra: Optional[dict] = None         # per-layer arrays the design's config carries instead of the checkpoint (tensor name -> float32 array)
    norm_weight_offset: float = 0.0      # 1: norm weights are stored around zero
    embed_norm: int = 0                  # the embedding row is normed before the first layer
    bigram: Optional[Tuple[int, int, int]] = None      # (buckets, multiplier of the previous token, multiplier of the token): a hashed pair embedding joins the row
    logit_scale: float = 0.0             # 0: the logits as they are
    row_of: Optional[Dict[str, int]] = None            # a design's own bookkeeping: which config layer / which pass a layer run stands for
    fit: Optional[Callable[["ServeModelSpec", Callable[[str], Tuple[int, ...]]], None]] = None      # completes sizes that only tensor shapes give (called with name -> shape before the store is made)


_ARCHITECTURES: Dict[str, Callable[[dict], ServeModelSpec]] = {}


def register_architecture(name: str, spec_from_config: Callable[[dict], ServeModelSpec]) -> None:
    _ARCHITECTURES[name] = spec_from_config


def architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


# ---- Lomutar: pre-norm layers with ONE layer norm (weight + bias) feeding an attention mixer and a feed-forward in parallel.  Attention: grouped
# key / value heads, interleaved partial rotary with linear position scaling, weightless RMS norm of q and k after the rotation, sliding window,
# a learned per-head sink in the softmax denominator, optional reuse of an earlier layer's cache.  Feed-forward: gated tanh-GELU, or a mixture of
# clamped gated experts behind a softmax router restricted to the best groups, plus a shared expert.
def _lomutar_tensors(spec: ServeModelSpec) -> Iterator[Tuple[int, str, int, str]]:
    yield -1, "embed", 0, "embed"
    yield -1, "final_norm_w", 0, "final.norm"
    yield -1, "final_norm_b", 0, "final.norm.b"
    yield -1, "head", 0, "head"
    for i, l in enumerate(spec.layers):
        p = f"l{i}"
        yield i, "norm_w", 0, f"{p}.norm1"
        yield i, "norm_b", 0, f"{p}.norm1.b"
        yield i, "q", 0, f"{p}.mix.q"
        if l.kv_from < 0:
            yield i, "k", 0, f"{p}.mix.k"
            yield i, "v", 0, f"{p}.mix.v"
        yield i, "o", 0, f"{p}.mix.o"
        if l.has_sink:
            yield i, "sink", 0, f"{p}.mix.sink"
        if l.mlp_kind == S.MLP_DENSE:
            for r in ("gate", "up", "down"):
                yield i, r, 0, f"{p}.mlp.{r}"
        elif l.mlp_kind == S.MLP_MOE:
            yield i, "router", 0, f"{p}.mlp.router"
            for e in range(l.experts):
                for r in ("gate", "up", "down"):
                    yield i, f"expert_{r}", e, f"{p}.mlp.e{e}.{r}"
            if l.shared_ff:
                for r in ("gate", "up", "down"):
                    yield i, f"shared_{r}", 0, f"{p}.mlp.shared.{r}"


def lomutar_spec(cfg: dict) -> ServeModelSpec:
    layers: List[S.LayerSpec] = []
    for i, lc in enumerate(cfg["layers"]):
        if lc.get("type", "attention") != "attention":
            raise ValueError(f"layer {i}: mixer type {lc.get('type')!r} is not part of this design")
        m = lc["mixer"]
        rot = m.get("rot") or {}
        sc = (rot.get("scaling") or {})
        l = S.LayerSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                        rot_dims=int(rot.get("dims", 0)), rot_interleaved=1, rot_base=float(rot.get("base", 10000.0)), rot_factor=float(sc.get("factor", 1.0)),
                        qk_unit_norm=1, scale=float(m["scale"]), window=int((m.get("mask") or {}).get("size", 0)), has_sink=1,
                        kv_from=-1 if m.get("kv_from") is None else int(m["kv_from"]))
        mlp = lc.get("mlp")
        if mlp is not None:
            kind = mlp.get("kind")
            if kind == "dense":
                l.mlp_kind, l.ff, l.dense_act = S.MLP_DENSE, int(mlp["ff"]), S.ACT_GELU_TANH
            elif kind == "moe":
                r, ex = mlp["router"], mlp["expert"]
                g = r.get("groups") or {}
                l.mlp_kind, l.experts, l.top = S.MLP_MOE, int(r["experts"]), int(r["top"])
                l.groups, l.keep, l.renorm = int(g.get("count", 1)), int(g.get("keep", g.get("count", 1))), 0
                l.expert_ff, l.expert_act, l.expert_limit, l.expert_alpha = int(ex["ff"]), S.ACT_CLAMPED_SWIGLU, float(ex["limit"]), 1.702
                sh = mlp.get("shared")
                if sh:
                    l.shared_ff, l.shared_limit = int(sh["ff"]), float(sh["limit"])
            else:
                raise ValueError(f"layer {i}: feed-forward kind {kind!r}")
        layers.append(l)
    return ServeModelSpec(vocab=int(cfg["vocab"]), width=int(cfg["width"]), norm_kind=S.NORM_LAYER, norm_eps=float(cfg["norm"]["eps"]), layers=layers,
                          tensors=_lomutar_tensors)


register_architecture("Lomutar", lomutar_spec)


# ---- Pamulix: x <- x + m * LN(mixer(x)), then x <- x + m * LN(ff(x)): the sublayers read the residual stream itself and a weight-only layer norm sits on
# their OUTPUT.  Two mixers.  'attention': grouped key / value heads, RMS norm of q and k with a weight shared by the heads, no rotation; the score loses
# slope_h * distance with slope_h = 2^(-8 (h + 1) / heads); a query sees the earlier keys of its own block of mask.size positions; the softmax denominator
# carries an extra one; from the second layer marked v_mix on, the values are blended with the first such layer's values of the same token before they
# are cached.  'latent_attention': queries and keys / values through normed low-rank latents, a rotated key part shared by the heads, by-parts scaled
# rotation frequencies, plain causal softmax; the cache holds the latent and the shared part.  Feed-forward: SiLU-gated experts, the `top` largest of
# (router logits + bias), softmax over the chosen logits.
def _pamulix_tensors(spec: ServeModelSpec) -> Iterator[Tuple[int, str, int, str]]:
    yield -1, "embed", 0, "embed"
    yield -1, "final_norm_w", 0, "final.norm"
    yield -1, "head", 0, "head"
    for i, l in enumerate(spec.layers):
        p = f"l{i}"
        yield i, "post1_w", 0, f"{p}.norm1"
        if l.mixer_kind == S.MIX_LATENT:
            for r, n in (("dq", "dq"), ("dq_norm", "dq.norm"), ("uq", "uq"), ("dkv", "dkv"), ("dkv_norm", "dkv.norm"), ("uk", "uk"), ("uv", "uv")):
                yield i, r, 0, f"{p}.mix.{n}"
        else:
            for r, n in (("q", "q"), ("k", "k"), ("v", "v"), ("q_norm", "q.norm"), ("k_norm", "k.norm")):
                yield i, r, 0, f"{p}.mix.{n}"
            if l.v_mix == S.VMIX_BLEND:
                yield i, "vmix", 0, f"{p}.mix.vmix"
        yield i, "o", 0, f"{p}.mix.o"
        if l.mlp_kind == S.MLP_MOE:
            yield i, "post2_w", 0, f"{p}.norm2"
            yield i, "router", 0, f"{p}.mlp.router"
            yield i, "router_bias", 0, f"{p}.mlp.router.b"
            for e in range(l.experts):
                for r in ("gate", "up", "down"):
                    yield i, f"expert_{r}", e, f"{p}.mlp.e{e}.{r}"


def pamulix_spec(cfg: dict) -> ServeModelSpec:
    layers: List[S.LayerSpec] = []
    mixing_seen = False
    for i, lc in enumerate(cfg["layers"]):
        kind, m = lc.get("type"), lc["mixer"]
        if kind == "attention":
            l = S.LayerSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                            qk_unit_norm=S.QKNORM_WEIGHTED, scale=float(m["scale"]), chunk=int((m.get("mask") or {}).get("size", 0)), has_sink=S.SINK_ZERO,
                            dist_bias=1, dist_bias_exp=8.0)
            if m.get("v_mix"):
                l.v_mix = S.VMIX_BLEND if mixing_seen else S.VMIX_FIRST
                mixing_seen = True
        elif kind == "latent_attention":
            rot = m["rot"]
            if int(rot["dims"]) != int(m["rot_dim"]):
                raise ValueError(f"layer {i}: the rotated part has {m['rot_dim']} coordinates, the rotation {rot['dims']}")
            l = S.LayerSpec(heads=int(m["heads"]), kv_heads=1, dim=int(m["dim"]), vdim=int(m["vdim"]), mixer_kind=S.MIX_LATENT, q_rank=int(m["q_rank"]),
                            kv_rank=int(m["kv_rank"]), rot_dims=int(m["rot_dim"]), rot_interleaved=1, rot_base=float(rot["base"]), scale=float(m["scale"]))
            sc = rot.get("scaling")
            if sc:
                l.rot_scaling, l.rot_factor = S.ROT_BY_PARTS, float(sc["factor"])
                l.rot_original, l.rot_fast, l.rot_slow = float(sc["original"]), float(sc["fast"]), float(sc["slow"])
        else:
            raise ValueError(f"layer {i}: mixer type {kind!r} is not part of this design")
        mlp = lc.get("mlp")
        if mlp is not None:
            if mlp.get("kind") != "moe":
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r}")
            r, ex = mlp["router"], mlp["expert"]
            l.mlp_kind, l.experts, l.top, l.groups, l.keep = S.MLP_MOE, int(r["experts"]), int(r["top"]), 1, 1
            l.renorm, l.router_bias = 1, 1      # the softmax over all logits, renormalised over the chosen ones, is the softmax over the chosen ones
            l.expert_ff, l.expert_act = int(ex["ff"]), S.ACT_SILU
        layers.append(l)
    return ServeModelSpec(vocab=int(cfg["vocab"]), width=int(cfg["width"]), norm_kind=S.NORM_LAYER, norm_eps=float(cfg["norm"]["eps"]), layers=layers,
                          tensors=_pamulix_tensors, block_kind=S.BLOCK_SEQUENTIAL, pre_norm=0, post_norm=1, norm_bias=0, residual_mult=float(cfg["residual_mult"]))


register_architecture("Pamulix", pamulix_spec)


# ---- Midisun: pre-normed sequential layers x <- x + gate1 * mixer(h1 + conv(h1)), x <- x + gate2 * ff(h2), h = RMS norm in groups, gate = sigmoid(W h + b)
# element by element, conv = a short causal convolution over the request's positions whose last inputs belong to the request's state.  Three mixers.
# 'attention': biased q / k / o projections, values = the keys before their norm, one RMS statistic over the whole q (k) row with a full-size weight,
# capped scores, a distance bias slope_h * (i - j), a sliding window, a learned sink in the denominator, a per-head sigmoid gate on the output.
# 'retention': rotated q / k (half-split pairs), S <- decay_h S + k v^T with k / sqrt(dim), o = S^T q, per-head unit RMS, times silu(W_g h).
# 'mlstm': S and a normaliser n under exponential input and sigmoid forget gates kept stable by a running maximum, capped gate pre-activations,
# per-head unit RMS with a weight, times sigmoid(W_g h).  Feed-forward: SiLU-gated dense, or SiLU-gated experts behind a sigmoid router whose choice
# (not its weights) is corrected by a bias and limited to the groups with the best top-two sums; weights renormalised over the chosen experts.
def _midisun_tensors(spec: ServeModelSpec) -> Iterator[Tuple[int, str, int, str]]:
    yield -1, "embed", 0, "embed"
    yield -1, "final_norm_w", 0, "final.norm"
    yield -1, "head", 0, "head"
    for i, l in enumerate(spec.layers):
        p = f"l{i}"
        yield i, "norm_w", 0, f"{p}.norm1"
        if spec.canon_taps > 1:
            yield i, "canon", 0, f"{p}.canon1"
        yield i, "res_gate1", 0, f"{p}.rg1"
        yield i, "res_gate1_b", 0, f"{p}.rg1.b"
        yield i, "q", 0, f"{p}.mix.q"
        yield i, "k", 0, f"{p}.mix.k"
        yield i, "out_gate", 0, f"{p}.mix.g"
        yield i, "o", 0, f"{p}.mix.o"
        if l.mixer_kind == S.MIX_ATTENTION:
            for r, n in (("q_bias", "q.b"), ("k_bias", "k.b"), ("o_bias", "o.b"), ("q_norm", "q.norm"), ("k_norm", "k.norm"), ("sink", "sink")):
                yield i, r, 0, f"{p}.mix.{n}"
        else:
            yield i, "v", 0, f"{p}.mix.v"
            if l.mixer_kind == S.MIX_MLSTM:
                for r, n in (("lin_norm", "norm"), ("igate", "i"), ("igate_b", "i.b"), ("fgate", "f"), ("fgate_b", "f.b")):
                    yield i, r, 0, f"{p}.mix.{n}"
            else:
                yield i, "lin_decay", 0, f"{p}.mix.decay"      # from config.json (spec.extra), not from the checkpoint
        if l.mlp_kind != S.MLP_NONE:
            yield i, "norm2_w", 0, f"{p}.norm2"
            yield i, "res_gate2", 0, f"{p}.rg2"
            yield i, "res_gate2_b", 0, f"{p}.rg2.b"
        if l.mlp_kind == S.MLP_DENSE:
            for r in ("gate", "up", "down"):
                yield i, r, 0, f"{p}.mlp.{r}"
        elif l.mlp_kind == S.MLP_MOE:
            yield i, "router", 0, f"{p}.mlp.router"
            yield i, "router_bias", 0, f"{p}.mlp.correction"
            for e in range(l.experts):
                for r in ("gate", "up", "down"):
                    yield i, f"expert_{r}", e, f"{p}.mlp.e{e}.{r}"


def midisun_spec(cfg: dict) -> ServeModelSpec:
    layers: List[S.LayerSpec] = []
    extra: Dict[str, np.ndarray] = {}
    taps = int((cfg.get("canon") or {}).get("taps", 0))      # one tap or none: the mixers read their normed input as it is
    for i, lc in enumerate(cfg["layers"]):
        kind, m = lc.get("type"), lc["mixer"]
        if kind == "attention":
            l = S.LayerSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                            qk_unit_norm=S.QKNORM_WHOLE, scale=float(m["scale"]), window=int((m.get("mask") or {}).get("size", 0)), has_sink=S.SINK_TENSOR, dist_bias=1,
                            dist_bias_exp=8.0, proj_bias=1, v_from_k=1, softcap=float(m.get("softcap") or 0.0), out_gate=S.OGATE_HEAD_SIGMOID)
            if l.vdim != l.dim:
                raise ValueError(f"layer {i}: the values are the keys, so vdim {l.vdim} must equal dim {l.dim}")
        elif kind == "retention":
            rot = m.get("rot") or {}
            l = S.LayerSpec(heads=int(m["heads"]), kv_heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), mixer_kind=S.MIX_RETENTION,
                            rot_dims=int(rot.get("dims", 0)), rot_interleaved=0, rot_base=float(rot.get("base", 10000.0)))
            dec = np.asarray(m["decay"], np.float32)
            if dec.shape != (l.heads,):
                raise ValueError(f"layer {i}: {dec.size} decays for {l.heads} heads")
            extra[f"l{i}.mix.decay"] = dec
        elif kind == "mlstm":
            l = S.LayerSpec(heads=int(m["heads"]), kv_heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), mixer_kind=S.MIX_MLSTM,
                            gate_cap=float(m.get("gate_cap") or 0.0), lin_norm_weight=1)
        else:
            raise ValueError(f"layer {i}: mixer type {kind!r} is not part of this design")
        mlp = lc.get("mlp")
        if mlp is not None:
            if mlp.get("kind") == "dense":
                l.mlp_kind, l.ff, l.dense_act = S.MLP_DENSE, int(mlp["ff"]), S.ACT_SILU
            elif mlp.get("kind") == "moe":
                r, ex = mlp["router"], mlp["expert"]
                g = r.get("groups") or {}
                l.mlp_kind, l.experts, l.top = S.MLP_MOE, int(r["experts"]), int(r["top"])
                l.groups, l.keep = int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))
                l.renorm, l.router_bias, l.router_score, l.group_score = 1, S.RBIAS_CHOICE, S.RSCORE_SIGMOID, S.GSCORE_TOP2
                l.expert_ff, l.expert_act = int(ex["ff"]), S.ACT_SILU
            else:
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r}")
        layers.append(l)
    return ServeModelSpec(vocab=int(cfg["vocab"]), width=int(cfg["width"]), norm_kind=S.NORM_RMS, norm_eps=float(cfg["norm"]["eps"]), layers=layers,
                          tensors=_midisun_tensors, block_kind=S.BLOCK_SEQUENTIAL, pre_norm=1, post_norm=0, norm_bias=0,
                          norm_groups=int(cfg["norm"].get("groups", 1)), embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
                          canon_taps=taps if taps > 1 else 0, res_gate=1, extra=extra)


register_architecture("Midisun", midisun_spec)


# ---- Lufozen: pre-normed sequential layers with RMS norms whose weights are stored around zero.  The embedding row (scaled) plus a hashed pair-of-tokens row is
# normed before the first layer.  A block of consecutive layers may run several times with the same tensors; every pass keeps its own cache and state, and a
# vector of its own joins the stream right before it.  Three mixers.  'attention': biased projections, a short causal convolution on q, k, v, per-head weighted
# q / k norm, interleaved partial rotation with banded frequency scaling, a zero-score sink in the softmax, an element-wise sigmoid gate on the output.
# 'parallel': an un-biased attention (half-split rotation, plain softmax) and a state-space mixer side by side on the same input, their outputs weighted.
# 'gla': linear attention whose state decays per key channel by a low-rank function of the input.  Feed-forward: un-gated, squared relu.  Logits scaled.
def _lufozen_runs(cfg: dict) -> List[Tuple[int, Optional[int]]]:
    """(layer of config.json, pass number if the run opens a pass of the repeated block) for every layer run, in order"""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, None) for i in range(n)]
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    if not 0 <= a <= b <= n or times < 1:
        raise ValueError(f"loop {lp!r} over {n} layers")
    runs: List[Tuple[int, Optional[int]]] = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def _lufozen_rot(l: S.LayerSpec, rot: Optional[dict], interleaved: int) -> None:
    if not rot or not int(rot.get("dims", 0)):
        return
    l.rot_dims, l.rot_interleaved, l.rot_base = int(rot["dims"]), interleaved, float(rot["base"])
    sc = rot.get("scaling")
    if sc:
        l.rot_scaling, l.rot_factor = S.ROT_BANDS, float(sc["factor"])
        l.rot_original, l.rot_fast, l.rot_slow = float(sc["original"]), float(sc["high"]), float(sc["low"])


def _lufozen_tensors(spec: ServeModelSpec) -> Iterator[Tuple[int, str, int, str]]:
    yield -1, "embed", 0, "embed"
    if spec.bigram:
        yield -1, "bigram", 0, "bigram"
    yield -1, "embed_norm", 0, "embed.norm"
    yield -1, "final_norm_w", 0, "final.norm"
    yield -1, "head", 0, "head"
    for r, l in enumerate(spec.layers):
        if l.pre_add:
            yield r, "pre_add", 0, f"loop.step@{spec.row_of[f'run{r}']}"
        if l.weights_of:
            continue
        p = f"l{spec.row_of[f'layer{r}']}"
        yield r, "norm_w", 0, f"{p}.norm1"
        if l.mixer_kind == S.MIX_GLA:
            for role, n in (("q", "q"), ("k", "k"), ("v", "v"), ("out_gate", "g"), ("o", "o"), ("lin_norm", "norm"), ("decay_a1", "a1"), ("decay_a2", "a2"), ("decay_a2_b", "a2.b")):
                yield r, role, 0, f"{p}.mix.{n}"
        elif l.side_mixer == S.MIX_SSD:
            for role, n in (("q", "q"), ("k", "k"), ("v", "v"), ("q_norm", "q.norm"), ("k_norm", "k.norm"), ("o", "o")):
                yield r, role, 0, f"{p}.mix.left.{n}"
            for role, n in (("ssd_in", "in"), ("ssd_conv", "conv"), ("ssd_conv_b", "conv.b"), ("ssd_dt_bias", "dt_bias"), ("ssd_a_log", "A_log"), ("ssd_d", "D"), ("ssd_norm", "norm"),
                            ("ssd_o", "o")):
                yield r, role, 0, f"{p}.mix.right.{n}"
        else:
            for role, n in (("q", "q"), ("k", "k"), ("v", "v"), ("q_bias", "q.b"), ("k_bias", "k.b"), ("v_bias", "v.b"), ("o_bias", "o.b"), ("q_norm", "q.norm"), ("k_norm", "k.norm"),
                            ("out_gate", "g"), ("o", "o")):
                yield r, role, 0, f"{p}.mix.{n}"
            if l.proj_conv:
                for role, n in (("q_conv", "q.conv"), ("k_conv", "k.conv"), ("v_conv", "v.conv")):
                    yield r, role, 0, f"{p}.mix.{n}"
        if l.mlp_kind == S.MLP_DENSE:
            yield r, "norm2_w", 0, f"{p}.norm2"
            yield r, "up", 0, f"{p}.mlp.up"
            yield r, "down", 0, f"{p}.mlp.down"


def lufozen_spec(cfg: dict) -> ServeModelSpec:
    layers: List[S.LayerSpec] = []
    row_of: Dict[str, int] = {}
    first_run: Dict[int, int] = {}
    for r, (i, opens) in enumerate(_lufozen_runs(cfg)):
        lc = cfg["layers"][i]
        kind, m = lc.get("type"), lc["mixer"]
        if kind == "attention":
            l = S.LayerSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                            qk_unit_norm=S.QKNORM_WEIGHTED, scale=float(m["scale"]), has_sink=S.SINK_ZERO, proj_bias=2, proj_conv=int(m.get("conv") or 0),
                            out_gate=S.OGATE_ELEM_SIGMOID)
            _lufozen_rot(l, m.get("rot"), 1)
        elif kind == "parallel":
            a, b = m["left"], m["right"]
            l = S.LayerSpec(heads=int(a["heads"]), kv_heads=int(a.get("kv_heads", a["heads"])), dim=int(a["dim"]), vdim=int(a.get("vdim", a["dim"])),
                            qk_unit_norm=S.QKNORM_WEIGHTED, scale=float(a["scale"]), side_mixer=S.MIX_SSD, ssd_heads=int(b["heads"]), ssd_vdim=int(b["vdim"]),
                            ssd_state=int(b["state"]), ssd_groups=int(b.get("groups", 1)), ssd_conv=int(b.get("conv") or 1), ssd_norm_groups=int(b.get("norm_groups", 1)),
                            mix_scale=float(m.get("left_scale", 1.0)), side_scale=float(m.get("right_scale", 1.0)))
            if l.mix_scale == 0.0 or l.side_scale == 0.0:
                raise ValueError(f"layer {i}: a mixer weighted by zero")
            _lufozen_rot(l, a.get("rot"), 0)
        elif kind == "gla":
            # the rank of the decay's projection pair is the checkpoint's (a1: [rank, width]) unless config.json names it: lufozen_fit_checkpoint
            l = S.LayerSpec(heads=int(m["heads"]), kv_heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), mixer_kind=S.MIX_GLA, lin_norm_weight=2,
                            decay_rank=int(m.get("rank") or 0), decay_tau=float(m["tau"]))
        else:
            raise ValueError(f"layer {i}: mixer type {kind!r} is not part of this design")
        mlp = lc.get("mlp")
        if mlp is not None:
            if mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r}")
            l.mlp_kind, l.ff, l.dense_act = S.MLP_DENSE, int(mlp["ff"]), S.ACT_RELU2
        if i in first_run:
            l.weights_of = first_run[i] + 1
        else:
            first_run[i] = r
        if opens is not None:
            l.pre_add = 1
            row_of[f"run{r}"] = opens
        row_of[f"layer{r}"] = i
        layers.append(l)
    emb = cfg.get("embedding") or {}
    bg = emb.get("bigram")
    return ServeModelSpec(vocab=int(cfg["vocab"]), width=int(cfg["width"]), norm_kind=S.NORM_RMS, norm_eps=float(cfg["norm"]["eps"]), layers=layers,
                          tensors=_lufozen_tensors, block_kind=S.BLOCK_SEQUENTIAL, pre_norm=1, post_norm=0, norm_bias=0, embed_scale=float(emb.get("scale", 1.0)),
                          norm_weight_offset=1.0, embed_norm=1, bigram=(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else None,
                          logit_scale=float(cfg.get("logit_scale", 1.0)), row_of=row_of, fit=lufozen_fit_checkpoint)


def lufozen_fit_checkpoint(spec: ServeModelSpec, shape_of: Callable[[str], Tuple[int, ...]]) -> None:
    """sizes that only the checkpoint gives: the rank of a gla layer's decay projections"""
    for r, l in enumerate(spec.layers):
        if l.mixer_kind == S.MIX_GLA and not l.decay_rank:
            l.decay_rank = int(shape_of(f"l{spec.row_of[f'layer{r}']}.mix.a1")[0])


register_architecture("Lufozen", lufozen_spec)


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def model_family(cfg: dict) -> str:
    """'serve:<architecture>' for a layer-described design, 'decode:<model_type>' for the HF model types of the quantized decode graph"""
    arch = cfg.get("architecture")
    if isinstance(arch, str) and arch in _ARCHITECTURES:
        return "serve:" + arch
    if "model_type" in cfg or "text_config" in cfg or "language_config" in cfg:
        return "decode:" + str(cfg.get("model_type", ""))
    raise ValueError(f"config.json names no known design (architecture {arch!r}; known: {architectures()})")


def load_model(model_dir: str, dtype: str = "bfloat16", max_tokens: int = 4096, max_slots: int = 4, device: int = 0, build: bool = False, **decoder_args):
    """The serving object for a checkpoint directory: a `BatchEngine` (layer-described designs) or a `CpuDecoder` with its weights initialised."""
    cfg = read_config(model_dir)
    fam = model_family(cfg)
    if fam.startswith("serve:"):
        from .scheduler import BatchEngine
        spec = _ARCHITECTURES[fam[6:]](cfg)
        if spec.fit is not None:
            spec.fit(spec, SafetensorsFile(os.path.join(model_dir, "model.safetensors")).shape)
        eng = BatchEngine(spec, dtype=dtype, max_tokens=max_tokens, max_slots=max_slots, device=device, build=build)
        eng.load_safetensors(os.path.join(model_dir, "model.safetensors"))
        return eng
    from .decode_setup import CpuDecoder
    dec = CpuDecoder(model_dir, device=device, **decoder_args)
    dec.init_weights(max_rope_seq=max(max_tokens, 8192))
    return dec
