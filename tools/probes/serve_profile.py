"""Probe: a layer-described design on the batched serving store at one of bench.py's --arch-compare sizes, random bf16 weights.
    python tools/probes/serve_profile.py <small|large> prefill [design]     three prompt passes of the size's prompt length
    python tools/probes/serve_profile.py <small|large> decode [design]      decode steps of 1 and of 4 requests at the end of such a prompt, graphs on / off
design: lomutar (default), pamulix:<one letter per layer, A = chunked attention, L = attention through latents>, e.g. pamulix:ALAA, or
midisun:<A = windowed attention, R = retention, M = mLSTM>, e.g. midisun:ARMA, or lufozen:<A = attention, P = attention beside a state-space mixer, G = gla>, e.g.
lufozen:APGA (the second and third layer run twice)
Run under `rocprofv3 --kernel-trace --stats` for the kernel tables in profiles/serve_*."""
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
import bench  # noqa: E402
from krasis_amd import model_registry as R, scheduler as SCH, serve_store as S  # noqa: E402

name = sys.argv[1] if len(sys.argv) > 1 else "small"
mode = sys.argv[2] if len(sys.argv) > 2 else "decode"
z = bench.ARCH_SIZES[name]
W, H, G, D, E, k, F, L, V, P = (z[c] for c in ("width", "heads", "kv_heads", "dim", "experts", "top", "ff", "layers", "vocab", "prompt"))
design = sys.argv[3] if len(sys.argv) > 3 else "lomutar"
layers = [S.LayerSpec(heads=H, kv_heads=G, dim=D, vdim=D, rot_dims=D // 2, rot_base=1e6, rot_factor=2.0, qk_unit_norm=1, scale=D ** -0.5, window=z["window"], has_sink=1,
                      mlp_kind=S.MLP_MOE, experts=E, top=k, groups=4, keep=2, expert_ff=F, expert_limit=7.0, shared_ff=F, shared_limit=7.0) for _ in range(L)]
if design.startswith("pamulix:"):
    eng = bench.pamulix_serve_engine(z, design.split(":", 1)[1])
elif design.startswith("midisun:"):
    eng = bench.midisun_serve_engine(z, design.split(":", 1)[1])
elif design.startswith("lufozen:"):
    eng, _ = bench.lufozen_serve_engine(z, design.split(":", 1)[1], k * F)
else:
    eng = SCH.BatchEngine(R.ServeModelSpec(V, W, S.NORM_LAYER, 1e-5, layers, None), dtype="bfloat16", max_tokens=4 * (P + 256), max_slots=4)
    eng.load_synthetic(seed=7, amp=1.0)
rng = np.random.default_rng(3)
toks = lambda n: [int(x) for x in rng.integers(0, V, n)]  # noqa: E731
if mode == "prefill":
    for i in range(3):
        t0 = time.perf_counter()
        eng.step([("p", toks(P), [P - 1])], logits=False)
        print("prompt pass of %d tokens: %.3f ms" % (P, (time.perf_counter() - t0) * 1e3), flush=True)
        eng.finish("p")
    sys.exit(0)
for b in range(4):
    eng.step([(("d", b), toks(P), [])], logits=False)
for graph in (True, False):
    eng.store.set_use_graph(graph)
    for B in (1, 4):
        ent = lambda: [(("d", b), toks(1), [0]) for b in range(B)]  # noqa: E731
        for _ in range(5):
            eng.step(ent(), logits=False)
        n = 40
        t0 = time.perf_counter()
        for _ in range(n):
            eng.step(ent(), logits=False)
        print("graphs %s, %d request(s): %.3f ms / step, %d replays so far" % (graph, B, (time.perf_counter() - t0) / n * 1e3, eng.store.graph_replays()), flush=True)
