"""A plain, slow statement of the Zidevik decoder on the CPU, one function per mechanism, for the tests to hold the engine
against.  It shares no code with the engine: every function takes tensors and numbers, works on one whole sequence (rows =
positions 0 .. T-1) in the dtype of its inputs (the tests use float64), and keeps no cache.

A Zidevik layer is "parallel": with h = norm(x), x <- x + mixer(h) + feed_forward(h), and then takes a second, small input
from the token itself (`token_side_input`).  Its mixer is two mixers side by side on the same h, an attention and a selective
scan, whose results are added with a weight each.  The feed-forward is a gated one, or a mixture of such experts with a
sigmoid router.  A run of layers may be walked several times with the same weights (`run_model`), each walk entered through a
product that mixes the stream with the token rows again.

`store`, where a function takes it, is applied to what an engine that computes in bfloat16 would keep in bfloat16 (rows that go
into a matrix product, cached keys and values); the identity by default.
"""
from __future__ import annotations

import math

import torch


def same(x):
    return x


def to_bfloat16_and_back(x):
    return x.to(torch.bfloat16).to(x.dtype)


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def softcap(x, cap):
    return cap * torch.tanh(x / cap)


# ------------------------------------------------------------------------------------------- the left mixer: attention
def rotate_neighbours(x, dims, base):
    """x [T, heads, channels]: channels (2i, 2i + 1), i < dims/2, of every head are turned by position * base^(-2i/dims)."""
    T = x.shape[0]
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    a = torch.arange(T, dtype=torch.float64)[:, None] * f[None, :]
    cos, sin = torch.cos(a).to(x.dtype)[:, None, :], torch.sin(a).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def attention(h, wq, wk, wv, wo, *, heads, kv_heads, dim, vdim, scale, rot_dims, rot_base, eps, store=same, weight=1.0):
    """Causal softmax attention with grouped key/value heads; q and k are turned and then divided by their root mean square.
    `weight` multiplies the result; it is taken in on the values (the result is linear in them), which is where an engine that
    stores them rounded has it."""
    T = h.shape[0]
    q = (h @ wq.T).reshape(T, heads, dim)
    k = (h @ wk.T).reshape(T, kv_heads, dim)
    v = (h @ wv.T).reshape(T, kv_heads, vdim)
    if rot_dims:
        q, k = rotate_neighbours(q, rot_dims, rot_base), rotate_neighbours(k, rot_dims, rot_base)
    q, k, v = store(rms_norm(q, None, eps)), store(rms_norm(k, None, eps)), store(weight * v)
    per = heads // kv_heads
    out = torch.zeros(T, heads, vdim, dtype=h.dtype)
    seen = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for a in range(heads):
        s = (q[:, a] @ k[:, a // per].T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, a // per]
    return store(out.reshape(T, heads * vdim)) @ wo.T


# ------------------------------------------------------------------------------------------ the right mixer: selective scan
def causal_convolution(x, taps, bias):
    """x [T, C], taps [C, K] (the last column is the current row's), zeros before the sequence's start."""
    T, K = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, x.shape[1], dtype=x.dtype), x], dim=0)
    out = torch.zeros_like(x)
    for j in range(K):
        out = out + padded[j:j + T] * taps[:, j]
    return out + bias


def selective_scan(h, w_in, conv, conv_b, w_x, w_dt, dt_b, a_log, d_skip, w_o, *, state, dt_rank, store=same, weight=1.0):
    """S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;  y_c = S[c, :] . C + D_c x_c;  out = W_o (y * silu(z)), times `weight`
    (taken in before the last product)."""
    T = h.shape[0]
    inner = w_in.shape[0] // 2
    xz = h @ w_in.T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_convolution(x, conv, conv_b))
    low = store(x) @ w_x.T
    dt, B, C = low[:, :dt_rank], low[:, dt_rank:dt_rank + state], low[:, dt_rank + state:]
    dt = softplus(dt @ w_dt.T + dt_b)
    A = -torch.exp(a_log)
    S = torch.zeros(inner, state, dtype=h.dtype)
    y = torch.zeros(T, inner, dtype=h.dtype)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + d_skip * x[t]
    return store(weight * y * silu(z)) @ w_o.T


# ------------------------------------------------------------------------------------------------------- feed-forwards
def gated_mlp(h, gate, up, down, store=same):
    return store(silu(h @ gate.T) * (h @ up.T)) @ down.T


def routed_experts(h, router, experts, top, shared=None, store=same):
    """experts: list of (gate, up, down).  Scores are sigmoids of the router's logits; the `top` largest choose the experts, and
    a chosen expert's score multiplies its *input*.  `shared` (gate, up, down) serves every row."""
    s = torch.sigmoid(h @ router.T)
    out = torch.zeros(h.shape[0], experts[0][2].shape[0], dtype=h.dtype)
    chosen = torch.topk(s, top, dim=-1).indices
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            out[t] += gated_mlp(store(s[t, e] * h[t])[None, :], *experts[e], store=store)[0]
    if shared is not None:
        out = out + gated_mlp(h, *shared, store=store)
    return out


def token_side_input(x, tokens, table, lo, hi, gate, proj, norm_w, eps, store=same):
    """x + norm(proj(gelu(gate x) * e)), e the token's own row of `table`, columns lo .. hi - 1."""
    e = table[tokens][:, lo:hi]
    g = gelu_tanh(store(x) @ gate.T) * e
    return x + rms_norm(store(g) @ proj.T, norm_w, eps)


# ------------------------------------------------------------------------------------------------------------ the model
def _mixer(h, cfg, w, p, eps, store):
    left, right = cfg["left"], cfg["right"]
    a = attention(h, w[p + "left.q"], w[p + "left.k"], w[p + "left.v"], w[p + "left.o"], heads=left["heads"], kv_heads=left["kv_heads"],
                  dim=left["dim"], vdim=left["vdim"], scale=left["scale"], rot_dims=left["rot"]["dims"] if left.get("rot") else 0,
                  rot_base=left["rot"]["base"] if left.get("rot") else 1.0, eps=eps, store=store, weight=cfg["left_scale"])
    b = selective_scan(h, w[p + "right.in"], w[p + "right.conv"], w[p + "right.conv.b"], w[p + "right.x"], w[p + "right.dt"], w[p + "right.dt.b"],
                       w[p + "right.A_log"], w[p + "right.D"], w[p + "right.o"], state=right["state"], dt_rank=right["dt_rank"], store=store, weight=cfg["right_scale"])
    return a + b


def _feed_forward(h, cfg, w, p, store):
    three = lambda q: (w[q + "gate"], w[q + "up"], w[q + "down"])
    if cfg["kind"] == "dense":
        return gated_mlp(h, *three(p), store=store)
    n = cfg["router"]["experts"]
    return routed_experts(h, w[p + "router"], [three(f"{p}e{e}.") for e in range(n)], cfg["router"]["top"],
                          three(p + "shared.") if cfg.get("shared") else None, store=store)


def run_order(config):
    """[(layer, number of the walk or None)], the walk's number at its first layer only."""
    n, loop = len(config["layers"]), config.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def run_model(config, w, tokens, store=same, streams=None):
    """Logits [T, vocab] of one sequence.  w: tensors by name in the dtype to compute in.  `streams`, a list, gets the residual
    stream after every layer run."""
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x0 = w["embed"][tokens]
    x = x0
    side = config.get("token_side")
    for i, walk in run_order(config):
        layer, p = config["layers"][i], f"l{i}."
        if walk is not None:
            x = store(torch.cat([x, x0], dim=-1)) @ w["loop.in"].T + w["loop.step"][walk]
        h = store(rms_norm(x, w[p + "norm1"], eps))
        y = _mixer(h, layer["mixer"], w, p + "mix.", eps, store)
        if layer.get("mlp"):
            y = y + _feed_forward(h, layer["mlp"], w, p + "mlp.", store)
        x = x + y
        if side:
            d = side["dim"]
            x = token_side_input(x, tokens, w["side.embed"], i * d, (i + 1) * d, w[p + "side.gate"], w[p + "side.proj"], w[p + "side.norm"], eps, store)
        if streams is not None:
            streams.append(x)
    logits = store(rms_norm(x, w["final.norm"], eps)) @ w["head"].T
    cap = config.get("logit_softcap")
    return softcap(logits, cap) if cap else logits


def forward(config, stored, tokens, dtype=torch.float64, store=same, streams=None):
    """Logits [T, vocab] from tensors as a file stores them, computed in `dtype`."""
    w = {k: v.to(dtype) if v.is_floating_point() else v for k, v in stored.items()}
    return run_model(config, w, tokens, store=store, streams=streams)


def greedy(config, stored, prompt, n_new):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(config, stored, tokens)[-1].argmax()))
    return tokens[len(prompt):]
