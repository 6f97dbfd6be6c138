"""ServeStore -- the batched serving store of libkrasis_hip.so (`kr_serve_*`) as a Python object: layer descriptions in, tensors in, then `step`.

A step is a list of entries (slot, tokens); the store appends the tokens to the slots' cache pages and returns the logits of the rows asked for.
Slots and pages are managed by the library (`admit` / `release`); nothing here computes."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, fields
from typing import List, Optional, Sequence, Tuple

import numpy as np

from ._lib import ServeConfigC, ServeLayerC, check_serve, load_serve_library

BF16, F32 = 0, 1
NORM_LAYER, NORM_RMS = 0, 1
MLP_NONE, MLP_DENSE, MLP_MOE = 0, 1, 2
ACT_GELU_TANH, ACT_CLAMPED_SWIGLU, ACT_SILU, ACT_RELU2 = 0, 1, 2, 3
BLOCK_PARALLEL, BLOCK_SEQUENTIAL = 0, 1
MIX_ATTENTION, MIX_LATENT, MIX_RETENTION, MIX_MLSTM, MIX_GLA, MIX_SSD = 0, 1, 2, 3, 4, 5
QKNORM_NONE, QKNORM_AFTER_ROT, QKNORM_WEIGHTED, QKNORM_WHOLE = 0, 1, 2, 3
RBIAS_NONE, RBIAS_LOGIT, RBIAS_CHOICE = 0, 1, 2
RSCORE_SOFTMAX, RSCORE_SIGMOID = 0, 1
GSCORE_MAX, GSCORE_TOP2 = 0, 1
OGATE_NONE, OGATE_HEAD_SIGMOID, OGATE_ELEM_SIGMOID = 0, 1, 2
SINK_NONE, SINK_TENSOR, SINK_ZERO = 0, 1, 2
ROT_LINEAR, ROT_BY_PARTS, ROT_BANDS = 0, 1, 2
VMIX_NONE, VMIX_FIRST, VMIX_BLEND = 0, 1, 2
PAGE_TOKENS = 64
ROLES = {n: i for i, n in enumerate(["embed", "final_norm_w", "final_norm_b", "head", "norm_w", "norm_b", "q", "k", "v", "o", "sink", "gate", "up", "down",
                                     "router", "expert_gate", "expert_up", "expert_down", "shared_gate", "shared_up", "shared_down",
                                     "norm2_w", "norm2_b", "post1_w", "post1_b", "post2_w", "post2_b", "q_norm", "k_norm", "vmix", "router_bias",
                                     "dq", "dq_norm", "uq", "dkv", "dkv_norm", "uk", "uv",
                                     "q_bias", "k_bias", "o_bias", "out_gate", "canon", "res_gate1", "res_gate1_b", "res_gate2", "res_gate2_b",
                                     "lin_norm", "lin_decay", "igate", "igate_b", "fgate", "fgate_b",
                                     "embed_norm", "bigram", "pre_add", "v_bias", "q_conv", "k_conv", "v_conv", "decay_a1", "decay_a2", "decay_a2_b",
                                     "ssd_in", "ssd_conv", "ssd_conv_b", "ssd_dt_bias", "ssd_a_log", "ssd_d", "ssd_norm", "ssd_o"])}


@dataclass
class LayerSpec:
    """One layer: a mixer (attention, attention through latents, or a recurrent matrix state) and a feed-forward, beside or after one another (field meanings: `kr_serve_layer`
    in include/krasis_hip.h)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    rot_dims: int = 0
    rot_interleaved: int = 1
    rot_base: float = 10000.0
    rot_factor: float = 1.0
    qk_unit_norm: int = 0
    scale: float = 1.0
    window: int = 0
    has_sink: int = 0
    kv_from: int = -1
    mlp_kind: int = MLP_NONE
    ff: int = 0
    dense_act: int = ACT_GELU_TANH
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1
    renorm: int = 0
    expert_ff: int = 0
    expert_act: int = ACT_CLAMPED_SWIGLU
    expert_limit: float = 0.0
    expert_alpha: float = 1.702
    shared_ff: int = 0
    shared_limit: float = 0.0
    mixer_kind: int = MIX_ATTENTION
    q_rank: int = 0
    kv_rank: int = 0
    rot_scaling: int = ROT_LINEAR
    rot_original: float = 0.0
    rot_fast: float = 0.0
    rot_slow: float = 0.0
    chunk: int = 0
    dist_bias: int = 0
    dist_bias_exp: float = 8.0
    v_mix: int = VMIX_NONE
    router_bias: int = 0
    proj_bias: int = 0
    v_from_k: int = 0
    softcap: float = 0.0
    out_gate: int = OGATE_NONE
    gate_cap: float = 0.0
    lin_norm_weight: int = 0
    router_score: int = RSCORE_SOFTMAX
    group_score: int = GSCORE_MAX
    weights_of: int = 0                  # 1 + the earlier layer whose tensors this layer uses (a block of layers that runs again); 0: its own
    pre_add: int = 0                     # tensor pre_add [width] joins the stream before the layer
    proj_conv: int = 0                   # taps of the causal convolution on q, k, v
    decay_rank: int = 0                  # gla: rank of the decay's projection pair, and the root taken of its sigmoid
    decay_tau: float = 0.0
    side_mixer: int = 0                  # MIX_SSD: a state-space mixer beside the attention mixer, on the same input
    ssd_heads: int = 0
    ssd_vdim: int = 0
    ssd_state: int = 0
    ssd_groups: int = 0
    ssd_conv: int = 0
    ssd_norm_groups: int = 0
    mix_scale: float = 0.0               # weights of the two mixers' outputs (0 reads as 1)
    side_scale: float = 0.0


class ServeStore:
    def __init__(self, vocab: int, width: int, layers: Sequence[LayerSpec], dtype: int = BF16, norm_kind: int = NORM_LAYER, norm_eps: float = 1e-5,
                 max_slots: int = 4, pool_tokens: int = 4096, page_tokens: int = PAGE_TOKENS, device: int = 0, build: bool = False,
                 block_kind: int = BLOCK_PARALLEL, pre_norm: int = 1, post_norm: int = 0, norm_bias: Optional[int] = None, residual_mult: float = 1.0,
                 norm_groups: int = 0, embed_scale: float = 0.0, canon_taps: int = 0, res_gate: int = 0, norm_weight_offset: float = 0.0, embed_norm: int = 0,
                 bigram: Optional[Tuple[int, int, int]] = None, logit_scale: float = 0.0):
        self._lib = load_serve_library(build=build)
        self.vocab, self.width, self.layers, self.dtype = vocab, width, list(layers), dtype
        self.page_tokens = page_tokens
        pool_tokens = (max(pool_tokens, page_tokens) + page_tokens - 1) // page_tokens * page_tokens
        self.pool_tokens, self.max_slots = pool_tokens, max_slots
        if norm_bias is None:
            norm_bias = int(norm_kind == NORM_LAYER)
        cfg = ServeConfigC(vocab, width, len(self.layers), dtype, norm_kind, norm_eps, max_slots, page_tokens, pool_tokens, block_kind, pre_norm, post_norm, norm_bias,
                           residual_mult, norm_groups, embed_scale, canon_taps, res_gate, norm_weight_offset, embed_norm, *(bigram or (0, 0, 0)), logit_scale)
        arr = (ServeLayerC * len(self.layers))()
        for i, l in enumerate(self.layers):
            for f in fields(LayerSpec):
                setattr(arr[i], f.name, getattr(l, f.name))
        self._h = C.c_void_p()
        check_serve(self._lib.kr_serve_create(device, C.byref(cfg), arr, C.byref(self._h)))

    def close(self) -> None:
        if getattr(self, "_h", None):
            self._lib.kr_serve_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- weights
    def set_tensor(self, layer: int, role: str, array: np.ndarray, index: int = 0) -> None:
        """array: uint16 (bf16 bit patterns) or float32, [rows, cols] or a vector"""
        a = np.ascontiguousarray(array)
        if a.dtype == np.uint16:
            src = BF16
        elif a.dtype == np.float32:
            src = F32
        else:
            raise ValueError(f"tensor dtype {a.dtype}: bf16 bit patterns (uint16) or float32")
        rows, cols = (1, a.size) if a.ndim <= 1 else a.shape
        check_serve(self._lib.kr_serve_set_tensor(self._h, layer, ROLES[role], index, a.ctypes.data, src, rows, cols))

    def fill_synthetic(self, seed: int = 1, amp: float = 1.0) -> None:
        check_serve(self._lib.kr_serve_fill_synthetic(self._h, seed, amp))

    def finalize(self) -> None:
        check_serve(self._lib.kr_serve_finalize(self._h))

    # ---- slots and pages
    def admit(self) -> int:
        s = C.c_int()
        check_serve(self._lib.kr_serve_admit(self._h, C.byref(s)))
        return s.value

    def release(self, slot: int) -> None:
        check_serve(self._lib.kr_serve_release(self._h, slot))

    def slot_len(self, slot: int) -> int:
        n = C.c_int()
        check_serve(self._lib.kr_serve_slot_len(self._h, slot, C.byref(n)))
        return n.value

    def free_pages(self) -> int:
        n = C.c_int()
        check_serve(self._lib.kr_serve_free_pages(self._h, C.byref(n)))
        return n.value

    # ---- the step
    def step(self, entries: Sequence[Tuple[int, Sequence[int]]], want_rows: Sequence[int], logits: bool = True) -> Tuple[Optional[np.ndarray], np.ndarray]:
        """entries: (slot, tokens); want_rows: indices into the entries' tokens laid end to end.  Returns (logits [n_want, vocab] f32 or None, argmax [n_want])."""
        slots = np.asarray([e[0] for e in entries], np.int32)
        counts = np.asarray([len(e[1]) for e in entries], np.int32)
        toks = np.ascontiguousarray(np.concatenate([np.asarray(e[1], np.int32).reshape(-1) for e in entries]) if entries else np.zeros(0, np.int32))
        want = np.asarray(list(want_rows), np.int32)
        out = np.empty((len(want), self.vocab), np.float32) if logits else None
        amax = np.empty(len(want), np.int32)
        check_serve(self._lib.kr_serve_step(self._h, len(entries), slots.ctypes.data, counts.ctypes.data, toks.ctypes.data, len(want), want.ctypes.data if len(want) else None,
                                            out.ctypes.data if (logits and len(want)) else None, amax.ctypes.data if len(want) else None))
        return out, amax

    def sample(self, row: int, temperature: float, top_k: int = 0, top_p: float = 1.0, seed: int = 0) -> int:
        t = C.c_int()
        check_serve(self._lib.kr_serve_sample(self._h, row, temperature, top_k, top_p, seed, C.byref(t)))
        return t.value

    # ---- test / measurement aids
    def set_capture(self, on: bool) -> None:
        check_serve(self._lib.kr_serve_set_capture(self._h, int(on)))

    def read_capture(self, n_tokens: int) -> np.ndarray:
        out = np.empty((len(self.layers), n_tokens, self.width), np.float32)
        check_serve(self._lib.kr_serve_read_capture(self._h, out.ctypes.data, out.size))
        return out

    def set_use_graph(self, on: bool) -> None:
        check_serve(self._lib.kr_serve_set_use_graph(self._h, int(on)))

    def graph_replays(self) -> int:
        return int(self._lib.kr_serve_graph_replays(self._h))

    def device_bytes(self) -> int:
        return int(self._lib.kr_serve_device_bytes(self._h))

    def set_profiling(self, on: bool) -> None:
        check_serve(self._lib.kr_serve_set_profiling(self._h, int(on)))

    def profile(self) -> List[float]:
        ms = (C.c_double * 8)()
        check_serve(self._lib.kr_serve_get_profile(self._h, ms, 8))
        return list(ms)
