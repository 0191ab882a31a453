"""What fixes the plain Mimitar implementation (`plain_mimitar.py`) and the configuration class, on the CPU: each mechanism against a
second formulation or a case worked by hand, the configuration's reading, its refusals and what it writes back, and the list of tensors a
configuration asks for against the folders the tests write."""
import itertools
import math

import pytest
import torch

import plain_mimitar as P
from mimitar_folders import BARE, CONFIGS, random_weights, tensor_layout

torch.manual_seed(0)
F64 = torch.float64


# ------------------------------------------------------------------------------------------------ the plain mechanisms
def test_the_blend_with_the_token_before_by_hand():
    h = torch.tensor([[1.0, 2.0], [3.0, 5.0], [-1.0, 0.0]], dtype=F64)
    w = torch.tensor([0.0, 1.0], dtype=F64)                     # channel 0 keeps the token's own value, channel 1 takes the one before
    assert torch.equal(P.shifted(h, w), torch.tensor([[1.0, 0.0], [3.0, 2.0], [-1.0, 5.0]], dtype=F64))
    half = P.shifted(h, torch.full((2,), 0.5, dtype=F64))
    assert torch.allclose(half[1], (h[0] + h[1]) / 2) and torch.allclose(half[0], h[0] / 2)


def test_copies_of_the_stream_with_unit_weights_are_the_plain_residual():
    xs = torch.randn(1, 5, 8, dtype=F64).repeat(3, 1, 1)
    y = torch.randn(5, 8, dtype=F64)
    first = torch.tensor([1.0, 0.0, 0.0], dtype=F64)
    assert torch.allclose(P.read_streams(xs, first), xs[0])
    out = P.write_streams(xs, y, torch.eye(3, dtype=F64), torch.ones(3, dtype=F64), 0.7)
    assert all(torch.allclose(out[t], xs[t] + 0.7 * y) for t in range(3))
    # the matrix is indexed [from, to]: copy 0 sent to copy 2 only
    mix = torch.zeros(3, 3, dtype=F64)
    mix[0, 2] = 1.0
    xs2 = torch.randn(3, 5, 8, dtype=F64)
    out = P.write_streams(xs2, torch.zeros_like(y), mix, torch.ones(3, dtype=F64), 1.0)
    assert torch.allclose(out[2], xs2[0]) and out[0].abs().max() == 0 and out[1].abs().max() == 0


def test_the_router_s_choice_against_a_search_over_all_subsets():
    g = torch.Generator().manual_seed(3)
    for E, top, groups, keep in ((6, 2, 3, 2), (8, 3, 4, 2), (4, 1, 4, 2), (8, 2, 2, 1), (5, 5, 1, 1), (12, 4, 3, 3)):
        scores = torch.softmax(torch.randn(7, E, generator=g, dtype=F64), dim=-1)
        ids, weights = P.choose_experts(scores, top, groups, keep)
        per = E // groups
        for t in range(7):
            best = sorted(range(groups), key=lambda j: -float(scores[t, j * per:(j + 1) * per].max()))[:keep]
            allowed = [e for e in range(E) if e // per in best]
            want = max(itertools.combinations(allowed, top), key=lambda c: sum(float(scores[t, e]) for e in c))
            assert sorted(ids[t].tolist()) == sorted(want)
            assert abs(float(weights[t].sum()) - 1.0) < 1e-12
            assert torch.allclose(weights[t], scores[t, ids[t]] / scores[t, ids[t]].sum())


def test_the_clamped_gate_by_hand():
    h = torch.eye(3, dtype=F64)
    gate = torch.tensor([[5.0, -5.0, 0.5]], dtype=F64)          # row i of h picks column i
    up = torch.tensor([[0.25, 7.0, -7.0]], dtype=F64)
    down = torch.ones(1, 1, dtype=F64)
    got = P.clamped_gated(h, gate, up, down, 2.0)[:, 0]
    sig = lambda z: 1 / (1 + math.exp(-z))
    want = [2.0 * sig(1.702 * 2.0) * 1.25, -5.0 * sig(1.702 * -5.0) * 3.0, 0.5 * sig(1.702 * 0.5) * -1.0]          # the gate is clamped from above only
    assert torch.allclose(got, torch.tensor(want, dtype=F64))


def test_attention_without_cap_norm_and_rotation_is_the_library_s():
    T, H, G, d, e = 9, 4, 2, 6, 5
    q, k, v = torch.randn(T, H, d, dtype=F64), torch.randn(T, G, d, dtype=F64), torch.randn(T, G, e, dtype=F64)
    got = P.causal_softmax_attention(q, k, v, 0.3)
    want = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1).repeat_interleave(2, 0)[None],
                                                            v.transpose(0, 1).repeat_interleave(2, 0)[None], is_causal=True, scale=0.3)[0].transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-12)
    capped = P.causal_softmax_attention(100 * q, k, v, 0.3, cap=0.01)          # scores squeezed into +-0.01: nearly the mean of the values seen
    mean = torch.stack([v[:t + 1, 0].mean(0) for t in range(T)])
    assert (capped[:, 0] - mean).abs().max() < 0.05


def test_rotations_keep_lengths_and_depend_on_distance_only():
    T, d = 12, 8
    f = P.plain_frequencies(d, 50.0)
    q, k = torch.randn(1, 1, d, dtype=F64).expand(T, 1, d), torch.randn(1, 1, d, dtype=F64).expand(T, 1, d)
    cos, sin = P.angles(T, f, F64)
    for turn in (P.turn_halves, P.turn_neighbours):
        a, b = turn(q, cos, sin), turn(k, cos, sin)
        assert torch.allclose(a.norm(dim=-1), q.norm(dim=-1))
        s = a[:, 0] @ b[:, 0].T
        assert all(abs(float(s[i, j] - s[i + 1, j + 1])) < 1e-9 for i in range(T - 1) for j in range(T - 1))
    part = P.turn_halves(torch.randn(T, 2, d + 3, dtype=F64), cos, sin)
    assert part.shape == (T, 2, d + 3)


def test_stretched_frequencies():
    plain = P.plain_frequencies(16, 100.0)
    got = P.stretched_by_wavelength(plain, 4.0, 1.0, 4.0, 64)
    for f, g in zip(plain, got):
        wave = 2 * math.pi / f
        if wave < 16:
            assert g == f
        elif wave > 64:
            assert g == f / 4
        else:
            assert f / 4 <= g <= f
    assert got[0] == plain[0] and got[-1] == plain[-1] / 4 and any(f / 4 < g < f for f, g in zip(plain, got))
    ramp, grow = P.stretched_by_ramp(plain, 16, 100.0, 4.0, 8, 4.0, 1.0)
    assert grow == pytest.approx(0.1 * math.log(4.0) + 1.0)
    assert ramp[0] == plain[0] and ramp[-1] == pytest.approx(plain[-1] / 4) and all(a >= b for a, b in zip(ramp, ramp[1:]))


def test_the_configuration_s_frequencies_are_the_plain_implementation_s():
    from geneinfer_amd.config.mimitar import RampScaling, WavelengthScaling, ramp_frequencies, wavelength_frequencies
    for dims, base in ((8, 100.0), (32, 10000.0), (4, 7.0)):
        plain = P.plain_frequencies(dims, base)
        assert wavelength_frequencies(dims, base, None) == pytest.approx(plain, rel=1e-15)
        assert wavelength_frequencies(dims, base, WavelengthScaling(4.0, 1.0, 4.0, 16)) == pytest.approx(P.stretched_by_wavelength(plain, 4.0, 1.0, 4.0, 16), rel=1e-14)
        want, grow = P.stretched_by_ramp(plain, dims, base, 8.0, 64, 16.0, 2.0)
        assert ramp_frequencies(dims, base, RampScaling(8.0, 64, 16.0, 2.0)) == pytest.approx(want, rel=1e-14)
        assert RampScaling(8.0, 64, 16.0, 2.0).magnitude() == pytest.approx(grow)


def test_the_plain_model_is_causal_and_a_layer_with_another_s_weights_has_none_of_its_own():
    cfg = CONFIGS["A"]
    w = random_weights(cfg, 4)
    assert not any(n.startswith("l2.") or n.startswith("l4.") for n in w)
    m = P.PlainMimitar(config=cfg, tensors=w)
    tokens = torch.randint(0, cfg["vocab"], (14,), generator=torch.Generator().manual_seed(1)).tolist()
    whole, part = m.logits(tokens), m.logits(tokens[:9])
    assert torch.allclose(whole[:9], part, atol=1e-10)
    layers, _ = m.layer_runs(tokens)
    assert layers.shape == (len(cfg["layers"]), 14, cfg["width"])


def test_without_its_output_products_the_model_is_the_head_of_the_normed_token_rows():
    cfg = CONFIGS["D"]
    w = random_weights(cfg, 2, bare=True)
    for name in w:
        if name.endswith("mix.o") or name.endswith(".down"):
            w[name] = torch.zeros_like(w[name])
    tokens = [3, 17, 149, 0]
    x = w["embed"].double()[torch.tensor(tokens)]
    want = P.one_plus_norm(x, w["final.norm"].double(), cfg["norm"]["eps"]) @ w["head"].double().T
    assert torch.allclose(P.PlainMimitar(config=cfg, tensors=w).logits(tokens), want, atol=1e-12)


# ------------------------------------------------------------------------------------------------ the configuration
@pytest.mark.parametrize("name", list(CONFIGS))
def test_a_configuration_reads_back_and_asks_for_the_folder_s_tensors(name):
    from geneinfer_amd.config import MimitarConfig, parse_config
    from geneinfer_amd.parts import model_tensor_needs
    cfg = CONFIGS[name]
    config = parse_config(cfg)
    assert type(config) is MimitarConfig and MimitarConfig.from_dict(config.to_dict()) == config
    layout = tensor_layout(cfg, bare=name in BARE)
    config = config.fit_to_tensors([n for n, _ in layout])
    assert MimitarConfig.from_dict(config.to_dict()) == config
    needs = {n.name: tuple(n.shape) for n in model_tensor_needs(config.model_spec())}
    assert needs == {n: tuple(s) for n, s in layout}
    spec = config.model_spec()
    assert len(spec.run_order) == len(cfg["layers"]) and spec.n_streams == cfg.get("streams", 1)
    own = [i for i, l in enumerate(cfg["layers"]) if l.get("weights_of") is None]
    assert [e.layer for e in spec.run_order] == [own.index(l.get("weights_of", i) if l.get("weights_of") is not None else i) for i, l in enumerate(cfg["layers"])]


def test_what_the_configuration_refuses():
    import copy
    from geneinfer_amd.config import ConfigError, parse_config
    def broken(change):
        cfg = copy.deepcopy(CONFIGS["A"])
        change(cfg)
        with pytest.raises(ConfigError):
            parse_config(cfg)
    broken(lambda c: c["layers"][0].__setitem__("type", "convolution"))
    broken(lambda c: c["layers"][2].__setitem__("weights_of", 2))
    broken(lambda c: c["layers"][2].__setitem__("weights_of", 9))
    broken(lambda c: c["layers"][2].__setitem__("weights_of", 1))                   # another kind of layer than it says it is
    broken(lambda c: c["layers"][4].__setitem__("weights_of", 2))                   # a layer that has no weights of its own
    broken(lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3))
    broken(lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7))
    broken(lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 18))
    broken(lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 2))         # not the rotated channels
    broken(lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 5))         # more than the kept groups hold
    broken(lambda c: c["layers"][0]["mlp"]["router"]["groups"].__setitem__("count", 4))
    broken(lambda c: c["layers"][0]["mlp"].__setitem__("kind", "sparse"))
    broken(lambda c: c["layers"][1]["mlp"].pop("limit"))
    broken(lambda c: c.pop("norm"))
    broken(lambda c: c.__setitem__("streams", 0))
    broken(lambda c: c.__setitem__("layers", []))


def test_a_layer_may_name_a_later_layer_s_weights():
    import copy
    from geneinfer_amd.config import parse_config
    from geneinfer_amd.parts import model_tensor_needs
    cfg = copy.deepcopy(CONFIGS["A"])
    cfg["layers"][0]["weights_of"] = 2
    del cfg["layers"][2]["weights_of"]
    spec = parse_config(cfg).model_spec()
    assert [e.layer for e in spec.run_order] == [1, 0, 1, 2, 0]
    assert {n.name.split(".")[0] for n in model_tensor_needs(spec)} == {"embed", "final", "head", "l1", "l2", "l3"}
    tokens = [5, 17, 3, 250, 9, 9, 41]
    w = random_weights(cfg, 6)
    assert not any(n.startswith("l0.") for n in w)
    a = P.PlainMimitar(config=cfg, tensors=w).logits(tokens)
    # the same model with the two entries' places in the file swapped back: layer 0 holds the weights and layer 2 names it
    back = copy.deepcopy(CONFIGS["A"])
    w0 = {("l0." + n[3:] if n.startswith("l2.") else n): t for n, t in w.items()}
    b = P.PlainMimitar(config=back, tensors=w0).logits(tokens)
    assert torch.equal(a, b)
