"""A plain, slow statement of the Mimitar decoder on the CPU, one function per mechanism, for the tests to hold the engine
against.  It shares no code with the engine: every function takes tensors and numbers, works on one whole sequence (rows =
positions 0 .. T-1) in the dtype of its inputs (the tests use float64), and keeps no cache.

A Mimitar model carries several copies of the residual stream (`streams`).  Each half of a layer (mixer, feed-forward) reads a
weighted sum of the copies, norms it, and its result is written back into every copy with a weight of its own while the copies
are mixed among themselves by a small matrix.  The mixer's input is first blended, channel by channel, with the input the token
before had.  Mixers: softmax attention with grouped key/value heads, a norm over the whole query and key projections, a rotation
of a part of every head and capped scores; or attention through low-rank latents with a gate per head.  Feed-forwards: a gated
one with clamped halves, or a mixture of such experts chosen by a softmax router among the best groups of experts, with a
gated shared expert.  A layer may use another layer's weights.

`store`, where a function takes it, is applied to what an engine that computes in bfloat16 would keep in bfloat16 (rows that go
into a matrix product, cached keys and values); the identity by default.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def same(x):
    return x


def to_bfloat16_and_back(x):
    return x.to(torch.bfloat16).to(x.dtype)


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight


def one_plus_norm(x, weight, eps):
    """The norm of the layers and of the model: its weight is stored around zero."""
    return rms_norm(x, 1.0 + weight, eps)


# ------------------------------------------------------------------------------------------------ rotations
def plain_frequencies(dims, base):
    return [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]


def stretched_by_wavelength(freqs, factor, low, high, original):
    """Short waves keep their frequency, long ones are slowed by `factor`, those between are blended."""
    out = []
    for f in freqs:
        wave = 2 * math.pi / f
        if wave < original / high:
            out.append(f)
        elif wave > original / low:
            out.append(f / factor)
        else:
            s = (original / wave - low) / (high - low)
            out.append((1 - s) * f / factor + s * f)
    return out


def stretched_by_ramp(freqs, dims, base, factor, original, fast, slow):
    """A ramp over the pairs between two turning counts; returns the frequencies and what cosines and sines are multiplied by."""
    def pair_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))
    lo, hi = max(math.floor(pair_of(fast)), 0), min(math.ceil(pair_of(slow)), dims - 1)
    out = []
    for i, f in enumerate(freqs):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def angles(T, freqs, dtype, first=0):
    a = torch.arange(first, first + T, dtype=torch.float64)[:, None] * torch.tensor(freqs, dtype=torch.float64)[None, :]
    return torch.cos(a).to(dtype), torch.sin(a).to(dtype)


def turn_halves(x, cos, sin):
    """x [T, heads, channels]: channel i < n and channel i + n are a pair, n = cos.shape[1]; later channels pass."""
    n = cos.shape[1]
    u, v = x[..., :n], x[..., n:2 * n]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:]], dim=-1)


def turn_neighbours(x, cos, sin):
    """x [T, heads, 2n]: channels 2i and 2i + 1 are a pair."""
    u, v = x[..., 0::2], x[..., 1::2]
    c, s = cos[:, None, :], sin[:, None, :]
    out = torch.empty_like(x)
    out[..., 0::2] = u * c - v * s
    out[..., 1::2] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------------ mixers
def causal_softmax_attention(q, k, v, scale, cap=None):
    """q [T, heads, d], k [T, groups, d], v [T, groups, e]; query head a reads group a // (heads / groups).  Scores are
    scaled, then capped by cap * tanh(. / cap)."""
    T, heads, _ = q.shape
    per = heads // k.shape[1]
    seen = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, heads, v.shape[2], dtype=q.dtype)
    for a in range(heads):
        s = (q[:, a] @ k[:, a // per].T) * scale
        if cap is not None:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~seen, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, a // per]
    return out


def attention_mixer(h, w, m, eps, store=same):
    """w: the mixer's tensors by their short names (q, k, v, q.norm, k.norm, o); m: the mixer's entry of the configuration."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w["q"].T, h @ w["k"].T, h @ w["v"].T
    q, k = rms_norm(q, w["q.norm"], eps), rms_norm(k, w["k.norm"], eps)          # over all heads at once
    q, k, v = q.reshape(T, H, d), k.reshape(T, G, d), v.reshape(T, G, e)
    rot = m.get("rot")
    if rot is not None and rot["dims"]:
        f = plain_frequencies(rot["dims"], rot["base"])
        if rot.get("scaling"):
            sc = rot["scaling"]
            f = stretched_by_wavelength(f, sc["factor"], sc["low"], sc["high"], sc["original"])
        cos, sin = angles(T, f, h.dtype)
        q, k = turn_halves(q, cos, sin), turn_halves(k, cos, sin)
    o = causal_softmax_attention(store(q), store(k), store(v), m["scale"], m.get("softcap"))
    return store(o.reshape(T, H * e)) @ w["o"].T


def latent_attention_mixer(h, w, m, eps, store=same):
    """Tensors dq, dq.norm, uq, dkv, dkv.norm, uk, uv, g, o."""
    T = h.shape[0]
    H, d, r, e, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (store(cq) @ w["uq"].T).reshape(T, H, d + r)
    down = h @ w["dkv"].T
    c, k_rot = store(rms_norm(down[:, :rank], w["dkv.norm"], eps)), down[:, rank:].reshape(T, 1, r)
    if r:
        rot = m["rot"]
        f, grow = plain_frequencies(r, rot["base"]), 1.0
        if rot.get("scaling"):
            sc = rot["scaling"]
            f, grow = stretched_by_ramp(f, r, rot["base"], sc["factor"], sc["original"], sc["fast"], sc["slow"])
        cos, sin = angles(T, f, h.dtype)
        cos, sin = cos * grow, sin * grow
        q = torch.cat([q[..., :d], turn_neighbours(q[..., d:], cos, sin)], dim=-1)
        k_rot = turn_neighbours(k_rot, cos, sin)
    k_plain = (c @ w["uk"].T).reshape(T, H, d)
    v = (c @ w["uv"].T).reshape(T, H, e)
    k = torch.cat([k_plain, store(k_rot).expand(T, H, r)], dim=-1)
    o = causal_softmax_attention(store(q), k, v, m["scale"])
    if "g" in w:
        o = o * torch.sigmoid(h @ w["g"].T)[:, :, None]
    return store(o.reshape(T, H * e)) @ w["o"].T


# ------------------------------------------------------------------------------------------------ feed-forwards
def clamped_gated(h, gate, up, down, limit, store=same):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return store(g * torch.sigmoid(1.702 * g) * (u + 1)) @ down.T


def choose_experts(scores, top, n_groups, keep):
    """scores [T, experts] -> (ids [T, top], weights [T, top]): the `top` largest among the experts of the `keep` groups whose
    best expert scores highest; weights are the chosen scores over their sum."""
    T, E = scores.shape
    allowed = scores
    if n_groups > 1 and keep < n_groups:
        best = scores.reshape(T, n_groups, E // n_groups).max(dim=-1).values
        kept = torch.zeros(T, n_groups, dtype=torch.bool)
        kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
        allowed = scores.masked_fill(~kept[:, :, None].expand(T, n_groups, E // n_groups).reshape(T, E), float("-inf"))
    ids = allowed.topk(top, dim=-1).indices
    chosen = scores.gather(1, ids)
    return ids, chosen / (chosen.sum(dim=-1, keepdim=True) + 1e-20)


def feed_forward(h, w, f, store=same):
    """w: the feed-forward's tensors by their short names; f: its entry of the configuration."""
    if f["kind"] == "dense":
        return clamped_gated(h, w["gate"], w["up"], w["down"], f["limit"], store)
    r = f["router"]
    scores = torch.softmax((h @ w["router"].T).double(), dim=-1).to(h.dtype)
    groups = r.get("groups") or {"count": 1, "keep": 1}
    ids, weights = choose_experts(scores, r["top"], groups["count"], groups["keep"])
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(r["top"]):
            e = int(ids[t, j])
            out[t] += weights[t, j] * clamped_gated(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], f["expert"]["limit"], store)[0]
    if f.get("shared"):
        shared = clamped_gated(h, w["shared.gate"], w["shared.up"], w["shared.down"], f["shared"]["limit"], store)
        out = out + torch.sigmoid(h @ w["shared.sg"].T) * shared
    return out


# ------------------------------------------------------------------------------------------------ a layer
def shifted(h, shift):
    """Every row blended with the row before it (zeros before the first): h + (h_before - h) * shift."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (before - h) * shift


def read_streams(xs, w_in):
    """xs [streams, T, width] -> the sublayer's input before its norm."""
    return (w_in[:, None, None] * xs).sum(dim=0)


def write_streams(xs, y, w_mix, w_out, mult):
    """Copy t becomes sum_s mix[s, t] copy_s + mult * out[t] * y, all copies at once from the old ones."""
    return torch.einsum("st,snd->tnd", w_mix, xs) + mult * w_out[:, None, None] * y[None]


def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


class PlainMimitar:
    def __init__(self, folder=None, config=None, tensors=None, dtype=torch.float64, storage=None):
        """From a folder (config.json, model.safetensors) or from a configuration and tensors.  `storage` bfloat16 rounds where an
        engine that computes in bfloat16 stores bfloat16."""
        if folder is not None:
            from safetensors.torch import load_file
            config = json.loads((Path(folder) / "config.json").read_text())
            tensors = load_file(str(Path(folder) / "model.safetensors"))
        self.config = config
        self.w = {k: v.to(dtype) for k, v in tensors.items()}
        self.dtype = dtype
        self.store = to_bfloat16_and_back if storage == torch.bfloat16 else same

    def layer_runs(self, tokens):
        """The sum of the stream's copies after every layer, [layers, T, width], and the logits [T, vocab]."""
        c, w, store = self.config, self.w, self.store
        eps, mult, S = c["norm"]["eps"], c.get("residual_mult", 1.0), c.get("streams", 1)
        x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
        xs = x[None].repeat(S, 1, 1)
        after = []
        for i, layer in enumerate(c["layers"]):
            p = f"l{layer.get('weights_of', i)}."
            for half in (1, 2):
                if half == 2 and layer.get("mlp") is None:
                    continue
                hyper = f"{p}hc{half}.in" in w
                u = read_streams(xs, w[f"{p}hc{half}.in"]) if hyper else xs[0]
                h = one_plus_norm(u, w[f"{p}norm{half}"], eps)
                if half == 1:
                    if f"{p}shift" in w:
                        h = shifted(h, w[f"{p}shift"])
                    mixer = attention_mixer if layer["type"] == "attention" else latent_attention_mixer
                    y = mixer(store(h), sub(w, p + "mix."), layer["mixer"], eps, store)
                else:
                    y = feed_forward(store(h), sub(w, p + "mlp."), layer["mlp"], store)
                if hyper:
                    xs = write_streams(xs, y, w[f"{p}hc{half}.mix"], w[f"{p}hc{half}.out"], mult)
                else:
                    xs = xs + mult * y[None]
            after.append(xs.sum(dim=0))
        x = one_plus_norm(xs.sum(dim=0), w["final.norm"], eps)
        return torch.stack(after), (store(x) @ w["head"].T) * c.get("logit_scale", 1.0)

    def logits(self, tokens):
        return self.layer_runs(tokens)[1]

    def greedy(self, prompt, n):
        tokens, out = list(prompt), []
        for _ in range(n):
            out.append(int(self.logits(tokens)[-1].argmax()))
            tokens.append(out[-1])
        return out
