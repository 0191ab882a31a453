"""What pins the plain statement of the Zidevik decoder (`plain_zidevik.py`), on the CPU: each mechanism against a second
formulation or a closed form, and the configuration class against the folders the tests write."""
import math

import pytest
import torch

import plain_zidevik as P
from zidevik_folders import CONFIGS, random_weights, tensor_layout


def test_rotation_of_neighbouring_pairs_keeps_lengths_and_depends_on_distance_only():
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(40, 2, 12, generator=g, dtype=torch.float64), torch.randn(40, 2, 12, generator=g, dtype=torch.float64)
    rq, rk = P.rotate_neighbours(q, 8, 30.0), P.rotate_neighbours(k, 8, 30.0)
    assert torch.allclose(rq.norm(dim=-1), q.norm(dim=-1)) and torch.equal(rq[..., 8:], q[..., 8:])
    assert torch.allclose(rq[0], q[0])                                   # position 0 is not turned
    # the same vectors at positions (5, 2) and (25, 22) give the same score
    same_q, same_k = q[:1].expand(40, -1, -1).clone(), k[:1].expand(40, -1, -1).clone()
    a, b = P.rotate_neighbours(same_q, 8, 30.0), P.rotate_neighbours(same_k, 8, 30.0)
    assert torch.allclose((a[5] * b[2]).sum(-1), (a[25] * b[22]).sum(-1))
    # by hand: pair 1 at position 3 turns by 3 * 30^(-2/8)
    angle = 3 * 30.0 ** (-2 / 8)
    u, v = q[3, 0, 2], q[3, 0, 3]
    assert torch.allclose(rq[3, 0, 2], u * math.cos(angle) - v * math.sin(angle)) and torch.allclose(rq[3, 0, 3], v * math.cos(angle) + u * math.sin(angle))


def test_attention_against_the_library_routine():
    g = torch.Generator().manual_seed(1)
    T, d, H, G, dim, vdim = 23, 20, 4, 2, 6, 5
    h = torch.randn(T, d, generator=g, dtype=torch.float64)
    wq, wk, wv = (torch.randn(n, d, generator=g, dtype=torch.float64) for n in (H * dim, G * dim, G * vdim))
    got = P.attention(h, wq, wk, wv, torch.eye(H * vdim, dtype=torch.float64), heads=H, kv_heads=G, dim=dim, vdim=vdim, scale=0.3, rot_dims=4, rot_base=10.0, eps=1e-5)
    unit = lambda z: z / torch.sqrt((z * z).mean(-1, keepdim=True) + 1e-5)
    q = unit(P.rotate_neighbours((h @ wq.T).view(T, H, dim), 4, 10.0)).transpose(0, 1)
    k = unit(P.rotate_neighbours((h @ wk.T).view(T, G, dim), 4, 10.0)).transpose(0, 1).repeat_interleave(H // G, 0)
    v = (h @ wv.T).view(T, G, vdim).transpose(0, 1).repeat_interleave(H // G, 0)
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.3).transpose(0, 1).reshape(T, H * vdim)
    assert torch.allclose(got, want, atol=1e-12)


def test_selective_scan_in_closed_form_and_as_a_convolution():
    g = torch.Generator().manual_seed(2)
    d, inner, N, R, K, T = 6, 4, 3, 2, 3, 9
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    h, w_in, conv, conv_b, w_x, w_dt, dt_b, a_log, D = r(T, d), r(2 * inner, d), r(inner, K), r(inner), r(R + 2 * N, inner), r(inner, R), r(inner), 0.3 * r(inner, N), r(inner)
    got = P.selective_scan(h, w_in, conv, conv_b, w_x, w_dt, dt_b, a_log, D, torch.eye(inner, dtype=torch.float64), state=N, dt_rank=R)
    # unrolled: y_t = sum_{s <= t} C_t . (prod_{s < u <= t} exp(dt_u A)) dt_s x_s B_s + D x_t
    xz = h @ w_in.T
    pre, z = xz[:, :inner], xz[:, inner:]
    x = torch.stack([sum(conv[:, j] * (pre[t - (K - 1 - j)] if t - (K - 1 - j) >= 0 else 0) for j in range(K)) + conv_b for t in range(T)])
    x = x * torch.sigmoid(x)
    low = x @ w_x.T
    dt = torch.log1p(torch.exp(low[:, :R] @ w_dt.T + dt_b))
    B, C, A = low[:, R:R + N], low[:, R + N:], -torch.exp(a_log)
    want = torch.zeros(T, inner, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            decay = torch.exp(A * dt[s + 1:t + 1].sum(0)[:, None])
            want[t] += (decay * (dt[s] * x[s])[:, None] * B[s][None, :]) @ C[t]
        want[t] += D * x[t]
    want = want * (z * torch.sigmoid(z))
    assert torch.allclose(got, want, atol=1e-10)


def test_routed_experts_by_hand():
    g = torch.Generator().manual_seed(3)
    d, ff, E = 5, 4, 4
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    h, router = r(3, d), r(E, d)
    experts = [(r(ff, d), r(ff, d), r(d, ff)) for _ in range(E)]
    shared = (r(7, d), r(7, d), r(d, 7))
    got = P.routed_experts(h, router, experts, 2, shared)
    for t in range(3):
        s = 1 / (1 + torch.exp(-(router @ h[t])))
        best = sorted(range(E), key=lambda e: -float(s[e]))[:2]
        want = sum(P.gated_mlp((s[e] * h[t])[None], *experts[e])[0] for e in best) + P.gated_mlp(h[t][None], *shared)[0]
        assert torch.allclose(got[t], want, atol=1e-12)
    # the weight is on the input: it does not commute with the gate
    assert not torch.allclose(got[0], sum(s_ * P.gated_mlp(h[0][None], *experts[e])[0] for e, s_ in enumerate(torch.sigmoid(router @ h[0]))), atol=1e-3)
    # with every expert chosen nothing depends on the order
    assert torch.allclose(P.routed_experts(h, router, experts, E), sum(P.gated_mlp(torch.sigmoid(h @ router[e])[:, None] * h, *experts[e]) for e in range(E)), atol=1e-12)


def test_activations_and_norm():
    z = torch.tensor([-3.0, -0.5, 0.0, 0.7, 4.0], dtype=torch.float64)
    assert torch.allclose(P.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    assert torch.allclose(P.silu(z), torch.nn.functional.silu(z))
    assert torch.allclose(P.softplus(z), torch.nn.functional.softplus(z))
    x = torch.randn(4, 9, dtype=torch.float64)
    assert torch.allclose(P.rms_norm(x, torch.ones(9, dtype=torch.float64), 1e-5), torch.nn.functional.rms_norm(x, (9,), eps=1e-5))
    assert torch.allclose(P.softcap(torch.tensor([100.0, 0.1]), 5.0), torch.tensor([5.0, 0.1]), atol=1e-4)


def test_the_order_of_layers():
    assert P.run_order(dict(layers=[0] * 4, loop=dict(start=1, stop=3, times=2))) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    assert P.run_order(dict(layers=[0] * 2, loop=dict(start=0, stop=2, times=1))) == [(0, 0), (1, None)]
    assert P.run_order(dict(layers=[0] * 2)) == [(0, None), (1, None)]
    assert P.run_order(dict(layers=[0] * 3, loop=dict(start=2, stop=2, times=4))) == [(0, None), (1, None), (2, None)]


def test_zeroed_output_products_leave_the_token_rows():
    """With every product that writes the stream zeroed (and no walks), the logits are the head of the normed token rows."""
    cfg = CONFIGS["C"]
    w = {k: v.double() for k, v in random_weights(cfg, 3).items()}
    for k in w:
        if k.endswith(".o") or k.endswith("down"):
            w[k] = torch.zeros_like(w[k])
    tokens = [5, 9, 200, 1]
    want = P.rms_norm(w["embed"][torch.tensor(tokens)], w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T
    assert torch.allclose(P.run_model(cfg, w, tokens), want, atol=1e-12)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_configuration_class_reads_the_folders_configurations(name):
    import geneinfer_amd  # noqa: F401
    from geneinfer_amd.config import parse_config
    from geneinfer_amd.parts import model_tensor_needs
    cfg = CONFIGS[name]
    c = parse_config(cfg)
    assert type(c).__name__ == "ZidevikConfig" and parse_config(c.to_dict()) == c
    spec = c.model_spec()
    needs = {n.name: tuple(n.shape) for n in model_tensor_needs(spec)}
    assert needs == {n: tuple(s) for n, s in tensor_layout(cfg)}
    assert [e.layer for e in spec.run_order] == [i for i, _ in P.run_order(cfg)]
    assert [None if e.before is None else e.before.row for e in spec.run_order] == [t for _, t in P.run_order(cfg)]


def test_refusals():
    import copy
    import geneinfer_amd  # noqa: F401
    from geneinfer_amd.config import ConfigError, parse_config
    for change in (lambda c: c["layers"][0].update(type="serial"), lambda c: c["layers"][0]["mixer"]["left"].update(heads=3),
                   lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7), lambda c: c["loop"].update(stop=9),
                   lambda c: c["layers"][0]["mlp"]["router"].update(top=9), lambda c: c["layers"][1]["mlp"].update(kind="sparse"), lambda c: c.pop("norm")):
        cfg = copy.deepcopy(CONFIGS["A"])
        change(cfg)
        with pytest.raises(ConfigError):
            parse_config(cfg)
