"""Small Mimitar model folders for the tests, written without the engine's code (config.json and a safetensors file made by
`model_folders.write_safetensors_by_hand`), so that the engine's loader reads files it did not write.

Matrices are 0.2 * N(0, 1), which makes scores and logits of order one; norm weights of the layers lie around zero (0.1 * N), those
on queries, keys and latents around one; the weights on the copies of the stream are of order one with a mixing matrix near the
identity, the blend with the token before between -0.5 and 1.5, routers of order one so that the choice is rarely close.  The
configurations differ from one another in every size and option: one, two and three copies of the stream; value heads smaller and
larger than key heads; one and several key/value heads; rotations of a part of the head and of all of it, stretched and plain, and
none; capped scores and free ones; experts of which some or all serve a row, in groups of which some or all are kept, with and
without a shared one; layers without a feed-forward; layers that run with another layer's weights; one configuration whose sizes
are multiples of nothing and one of the sizes the matrix-core kernels take; one folder without the blend and the copies' weights."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch

from model_folders import write_safetensors_by_hand


def _attention(heads, kv_heads, dim, vdim, scale, softcap=None, rot=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if softcap is not None:
        m["softcap"] = softcap
    if rot is not None:
        m["rot"] = rot
    return dict(type="attention", mixer=m)


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, scaling=None):
    rot = dict(dims=rot_dim, base=base)
    if scaling is not None:
        rot["scaling"] = scaling
    return dict(type="latent_attention", mixer=dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale, rot=rot))


def _dense(ff, limit):
    return dict(kind="dense", ff=ff, limit=limit)


def _moe(experts, top, ff, limit, groups=None, shared=None):
    r = dict(experts=experts, top=top)
    if groups is not None:
        r["groups"] = dict(count=groups[0], keep=groups[1])
    m = dict(kind="moe", router=r, expert=dict(ff=ff, limit=limit))
    if shared is not None:
        m["shared"] = dict(ff=shared[0], limit=shared[1])
    return m


def _layer(mixer, mlp=None, weights_of=None):
    out = dict(mixer, mlp=mlp)
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


_A0 = _attention(4, 2, 16, 24, 0.2, softcap=3.0, rot=dict(dims=8, base=100.0, scaling=dict(factor=4.0, low=1.0, high=4.0, original=16)))
_A0_MLP = _moe(6, 2, 24, 1.0, groups=(3, 2), shared=(32, 2.0))
MIMITAR_A = dict(architecture="Mimitar", vocab=300, width=64, norm=dict(eps=1e-5), streams=3, residual_mult=0.6, logit_scale=0.7, layers=[
    _layer(_A0, _A0_MLP),
    _layer(_latent(3, 8, 4, 12, 20, 24, 0.3, 50.0, dict(factor=4.0, original=8, fast=4.0, slow=1.0)), _dense(48, 1.2)),
    _layer(_A0, _A0_MLP, weights_of=0),
    _layer(_attention(2, 1, 24, 8, 0.25, rot=dict(dims=24, base=30.0))),
    _layer(_latent(3, 8, 4, 12, 20, 24, 0.3, 50.0, dict(factor=4.0, original=8, fast=4.0, slow=1.0)), _dense(48, 1.2), weights_of=1),
])
# Sizes the matrix-core kernels take: heads of 64 channels, keys and values alike, everything a multiple of 16.
MIMITAR_B = dict(architecture="Mimitar", vocab=512, width=128, norm=dict(eps=1e-6), streams=2, residual_mult=0.8, logit_scale=1.5, layers=[
    _layer(_attention(4, 2, 64, 64, 0.1, softcap=20.0, rot=dict(dims=32, base=10000.0)), _moe(8, 2, 64, 3.0, groups=(2, 1), shared=(128, 1.5))),
    _layer(_latent(4, 32, 16, 32, 64, 48, 0.15, 1000.0), _dense(256, 2.5)),
    _layer(_attention(2, 2, 64, 64, 0.12, rot=dict(dims=64, base=500.0, scaling=dict(factor=8.0, low=1.0, high=2.0, original=64))), _moe(4, 4, 128, 1.0)),
])
# Sizes that are multiples of nothing; one copy of the stream (with its weights); every expert serves every row; no cap, no scale on the logits.
MIMITAR_C = dict(architecture="Mimitar", vocab=211, width=50, norm=dict(eps=1e-4), layers=[
    _layer(_attention(3, 3, 10, 6, 0.4, softcap=1.5, rot=dict(dims=4, base=7.0)), _moe(5, 5, 14, 0.7)),
    _layer(_latent(1, 6, 2, 10, 9, 11, 0.5, 3.0), None),
    _layer(_attention(6, 2, 6, 14, 0.3), _dense(30, 0.9)),
])
# One copy without weights on it and without the blend with the token before: what is left is a plain pre-norm decoder.
MIMITAR_D = dict(architecture="Mimitar", vocab=150, width=48, norm=dict(eps=1e-5), residual_mult=1.3, layers=[
    _layer(_attention(2, 1, 16, 16, 0.25, softcap=8.0, rot=dict(dims=16, base=40.0)), _dense(64, 1.0)),
    _layer(_latent(2, 8, 8, 8, 16, 16, 0.25, 20.0), _moe(4, 1, 16, 2.0, groups=(4, 2), shared=(16, 1.0))),
])
CONFIGS = {"A": MIMITAR_A, "B": MIMITAR_B, "C": MIMITAR_C, "D": MIMITAR_D}
PAGE_SIZE = {"A": 4, "B": 16, "C": 3, "D": 8}
BARE = {"D"}              # folders written without `l<i>.shift` and `l<i>.hc*`


def tensor_layout(cfg, bare=False):
    """(name, shape) of every tensor of a model, in the model's order."""
    d, n = cfg["width"], cfg.get("streams", 1)
    out = [("embed", (cfg["vocab"], d)), ("final.norm", (d,)), ("head", (cfg["vocab"], d))]
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        x = p + "mix."
        out += [(p + "norm1", (d,))]
        if not bare:
            out += [(p + "shift", (d,)), (p + "hc1.in", (n,)), (p + "hc1.out", (n,)), (p + "hc1.mix", (n, n))]
        if layer["type"] == "attention":
            a, kv = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
            out += [(x + "q", (a, d)), (x + "k", (kv, d)), (x + "v", (m["kv_heads"] * m["vdim"], d)), (x + "q.norm", (a,)), (x + "k.norm", (kv,)),
                    (x + "o", (d, m["heads"] * m["vdim"]))]
        else:
            H = m["heads"]
            out += [(x + "dq", (m["q_rank"], d)), (x + "dq.norm", (m["q_rank"],)), (x + "uq", (H * (m["dim"] + m["rot_dim"]), m["q_rank"])),
                    (x + "dkv", (m["kv_rank"] + m["rot_dim"], d)), (x + "dkv.norm", (m["kv_rank"],)), (x + "uk", (H * m["dim"], m["kv_rank"])),
                    (x + "uv", (H * m["vdim"], m["kv_rank"])), (x + "g", (H, d)), (x + "o", (d, H * m["vdim"]))]
        three = lambda q, ff: [(q + "gate", (ff, d)), (q + "up", (ff, d)), (q + "down", (d, ff))]
        mlp = layer["mlp"]
        if mlp is not None:
            out += [(p + "norm2", (d,))]
            if not bare:
                out += [(p + "hc2.in", (n,)), (p + "hc2.out", (n,)), (p + "hc2.mix", (n, n))]
            if mlp["kind"] == "dense":
                out += three(p + "mlp.", mlp["ff"])
            else:
                out.append((p + "mlp.router", (mlp["router"]["experts"], d)))
                for e in range(mlp["router"]["experts"]):
                    out += three(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
                if mlp.get("shared"):
                    out += three(p + "mlp.shared.", mlp["shared"]["ff"]) + [(p + "mlp.shared.sg", (1, d))]
    return out


def random_weights(cfg, seed, std=0.2, bare=False):
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_layout(cfg, bare):
        z = rng.standard_normal(shape)
        last = name.split(".")[-1]
        if last in ("norm1", "norm2") or name == "final.norm":
            t = 0.1 * z                                       # stored around zero
        elif last == "norm":
            t = 1.0 + 0.1 * z
        elif last == "shift":
            t = 0.5 + 0.5 * z
        elif last in ("in", "out"):
            t = 0.8 + 0.3 * z
        elif last == "mix":
            t = np.eye(shape[0]) + 0.2 * z
        elif last in ("router", "sg", "g"):
            t = z
        else:
            t = std * z
        w[name] = torch.from_numpy(np.asarray(t, dtype=np.float32))
    return w


def write_model(folder, cfg, seed=0, dtype=torch.bfloat16, std=0.2, weights=None, bare=False):
    """Writes the folder; returns the float32 weights before rounding to the storage dtype."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg, indent=2))
    w = weights if weights is not None else random_weights(cfg, seed, std, bare)
    write_safetensors_by_hand(folder / "model.safetensors", {n: t.to(dtype) for n, t in w.items()}, shuffle_seed=seed + 5)
    return w


def stored_weights(folder):
    """The folder's tensors as the file holds them (read with the safetensors package, not the engine's reader)."""
    from safetensors.torch import load_file
    return load_file(str(Path(folder) / "model.safetensors"))
