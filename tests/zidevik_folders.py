"""Small Zidevik model folders for the tests, written without the engine's code (config.json and a safetensors file made by
`model_folders.write_safetensors_by_hand`), so that the engine's loader reads files it did not write.

Matrices are 0.2 * N(0, 1), which makes scores and logits of order one; norm weights 1 + 0.1 * N(0, 1); biases and the scan's
parameters are of order one so that leaving one out shows.  The configurations differ from one another in every size and option:
value heads smaller and larger than key heads, one and several key/value heads, rotations of a part of the head, of all of it and
none; scans of one state and of seventeen, one tap and five, step sizes of rank one; experts of which one, several or all serve a
row, with and without a shared one; layers without a feed-forward; walks that begin at the first layer and later, over one layer,
several and all, once and several times, and models without walks, without the tokens' second input, without a cap on the logits;
one configuration whose sizes are multiples of nothing and one of the sizes the matrix-core kernels take."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch

from model_folders import write_safetensors_by_hand


def _left(heads, kv_heads, dim, vdim, scale, rot=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot is not None:
        m["rot"] = dict(dims=rot[0], base=rot[1])
    return m


def _right(inner, state, dt_rank, conv):
    return dict(inner=inner, state=state, dt_rank=dt_rank, conv=conv)


def _layer(left, left_scale, right, right_scale, mlp=None):
    return dict(type="parallel", mixer=dict(left=left, left_scale=left_scale, right=right, right_scale=right_scale), mlp=mlp)


def _dense(ff):
    return dict(kind="dense", ff=ff)


def _moe(experts, top, ff, shared=None):
    m = dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=ff))
    if shared is not None:
        m["shared"] = dict(ff=shared)
    return m


ZIDEVIK_A = dict(architecture="Zidevik", vocab=300, width=64, norm=dict(eps=1e-5), logit_softcap=10.0, token_side=dict(dim=6), loop=dict(start=1, stop=3, times=2), layers=[
    _layer(_left(4, 2, 16, 24, 0.2, (8, 100.0)), 0.7, _right(40, 5, 3, 3), 1.3, _moe(5, 2, 24, shared=32)),
    _layer(_left(2, 2, 24, 8, 0.3, (24, 50.0)), 1.1, _right(72, 17, 6, 4), 0.6, _dense(48)),
    _layer(_left(4, 1, 8, 16, 0.5), 0.9, _right(24, 3, 2, 2), 1.0),
    _layer(_left(3, 3, 12, 12, 0.25, (4, 7.0)), 1.0, _right(56, 8, 4, 5), 0.4, _moe(3, 1, 40)),
])
# Sizes the matrix-core kernels take: heads of 64 channels, keys and values alike, everything a multiple of 16.
ZIDEVIK_B = dict(architecture="Zidevik", vocab=512, width=128, norm=dict(eps=1e-6), logit_softcap=30.0, token_side=dict(dim=16), loop=dict(start=0, stop=1, times=3), layers=[
    _layer(_left(4, 2, 64, 64, 0.1, (32, 10000.0)), 1.0, _right(256, 16, 8, 4), 1.0, _moe(8, 2, 64, shared=128)),
    _layer(_left(2, 2, 64, 64, 0.15, (64, 500.0)), 0.5, _right(128, 16, 8, 4), 1.5, _dense(256)),
])
# Sizes that are multiples of nothing; one state, one tap, a step size of rank one; every expert serves every row; no walks, no second input, no cap.
ZIDEVIK_C = dict(architecture="Zidevik", vocab=211, width=50, norm=dict(eps=1e-4), layers=[
    _layer(_left(5, 1, 6, 3, 0.6, (2, 9.0)), 1.2, _right(30, 1, 1, 1), 0.8, _moe(3, 3, 10, shared=7)),
    _layer(_left(1, 1, 10, 7, 0.4, (6, 3.0)), -0.5, _right(17, 33, 5, 3), 2.0, _dense(22)),
    _layer(_left(3, 3, 4, 5, 0.7), 1.0, _right(9, 2, 3, 8), 1.0),
])
# Walks over all layers, and one that is walked once; the cap but no second input.
ZIDEVIK_D = dict(architecture="Zidevik", vocab=128, width=48, norm=dict(eps=1e-5), logit_softcap=5.0, loop=dict(start=0, stop=2, times=2), layers=[
    _layer(_left(2, 1, 24, 16, 0.2, (12, 20.0)), 0.8, _right(48, 4, 2, 4), 1.2, _moe(6, 3, 16)),
    _layer(_left(6, 2, 8, 8, 0.35, (8, 15.0)), 1.0, _right(32, 6, 3, 2), 1.0, _dense(64)),
])
ZIDEVIK_E = dict(architecture="Zidevik", vocab=160, width=32, norm=dict(eps=1e-5), token_side=dict(dim=5), loop=dict(start=1, stop=2, times=1), layers=[
    _layer(_left(2, 2, 16, 16, 0.25, (16, 40.0)), 1.0, _right(20, 9, 2, 3), 1.0, _dense(40)),
    _layer(_left(2, 1, 16, 8, 0.25, (6, 40.0)), 1.0, _right(36, 20, 4, 4), 1.0, _moe(4, 2, 12, shared=20)),
])
CONFIGS = {"A": ZIDEVIK_A, "B": ZIDEVIK_B, "C": ZIDEVIK_C, "D": ZIDEVIK_D, "E": ZIDEVIK_E}
PAGE_SIZE = {"A": 4, "B": 16, "C": 8, "D": 2, "E": 16}


def tensor_layout(cfg):
    d, n = cfg["width"], len(cfg["layers"])
    out = [("embed", (cfg["vocab"], d)), ("final.norm", (d,)), ("head", (cfg["vocab"], d))]
    if cfg.get("loop"):
        out += [("loop.in", (d, 2 * d)), ("loop.step", (cfg["loop"]["times"], d))]
    if cfg.get("token_side"):
        out.append(("side.embed", (cfg["vocab"], n * cfg["token_side"]["dim"])))
    for i, layer in enumerate(cfg["layers"]):
        p, l, r = f"l{i}.", layer["mixer"]["left"], layer["mixer"]["right"]
        x, y = p + "mix.left.", p + "mix.right."
        out += [(p + "norm1", (d,)), (x + "q", (l["heads"] * l["dim"], d)), (x + "k", (l["kv_heads"] * l["dim"], d)), (x + "v", (l["kv_heads"] * l["vdim"], d)),
                (x + "o", (d, l["heads"] * l["vdim"])), (y + "in", (2 * r["inner"], d)), (y + "conv", (r["inner"], r["conv"])), (y + "conv.b", (r["inner"],)),
                (y + "x", (r["dt_rank"] + 2 * r["state"], r["inner"])), (y + "dt", (r["inner"], r["dt_rank"])), (y + "dt.b", (r["inner"],)),
                (y + "A_log", (r["inner"], r["state"])), (y + "D", (r["inner"],)), (y + "o", (d, r["inner"]))]
        three = lambda q, ff: [(q + "gate", (ff, d)), (q + "up", (ff, d)), (q + "down", (d, ff))]
        mlp = layer["mlp"]
        if mlp is not None and mlp["kind"] == "dense":
            out += three(p + "mlp.", mlp["ff"])
        elif mlp is not None:
            out.append((p + "mlp.router", (mlp["router"]["experts"], d)))
            for e in range(mlp["router"]["experts"]):
                out += three(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
            if mlp.get("shared"):
                out += three(p + "mlp.shared.", mlp["shared"]["ff"])
        if cfg.get("token_side"):
            s = cfg["token_side"]["dim"]
            out += [(p + "side.gate", (s, d)), (p + "side.proj", (d, s)), (p + "side.norm", (d,))]
    return out


def random_weights(cfg, seed, std=0.2):
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_layout(cfg):
        z = rng.standard_normal(shape)
        last = name.split(".")[-1]
        if last in ("norm", "norm1"):
            t = 1.0 + 0.1 * z
        elif name.endswith("conv.b") or name.endswith("dt.b") or last == "D" or name == "loop.step":
            t = 0.5 * z
        elif last == "A_log":                                             # decays of order a half a token at step sizes of order one
            t = -0.5 + 0.6 * z
        elif last == "conv":
            t = 0.5 * z
        elif name == "side.embed" or last == "router":
            t = z
        elif last == "dt":
            t = 0.5 * z
        else:
            t = std * z
        w[name] = torch.from_numpy(np.asarray(t, dtype=np.float32))
    return w


def write_model(folder, cfg, seed=0, dtype=torch.bfloat16, std=0.2, weights=None):
    """Writes the folder; returns the float32 weights before rounding to the storage dtype."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg, indent=2))
    w = weights if weights is not None else random_weights(cfg, seed, std)
    write_safetensors_by_hand(folder / "model.safetensors", {n: t.to(dtype) for n, t in w.items()}, shuffle_seed=seed + 5)
    return w


def stored_weights(folder):
    """The folder's tensors as the file holds them (read with the safetensors package, not the engine's reader)."""
    from safetensors.torch import load_file
    return load_file(str(Path(folder) / "model.safetensors"))
