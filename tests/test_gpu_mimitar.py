"""The Mimitar design in the engine against the plain implementation (`plain_mimitar.py`): each kernel alone, then whole models of
four small configurations under every way of cutting the work into steps, and generation through the entry point and the
scheduler.  In float32 the engine's logits must not depend on the cutting at all (equal bits); in bfloat16 they must lie as close
to the exact model as rounding alone explains."""
import math

import pytest
import torch

import plain_mimitar as P
from mimitar_folders import BARE, CONFIGS, PAGE_SIZE, random_weights, stored_weights, write_model
from model_folders import assert_within_bfloat16_noise, relative_error

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64


def _prompt(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("mimitar")
    out = {}
    for name, cfg in CONFIGS.items():
        write_model(root / name, cfg, seed=41 + ord(name), bare=name in BARE)
        out[name] = root / name
    return out


_plain_cache = {}


def plain_logits(folders, name, tokens, rounded=False, dtype=F64):
    key = (str(folders[name]), tuple(tokens), rounded, dtype)
    if key not in _plain_cache:
        _plain_cache[key] = P.PlainMimitar(folders[name], dtype=dtype, storage=torch.bfloat16 if rounded else None).logits(tokens)
    return _plain_cache[key]


def make_runner(folders, name, dtype, **kw):
    from geneinfer_amd.engine import Runner, load_model
    model = load_model(folders[name], dtype, DEV)
    kw.setdefault("page_size", PAGE_SIZE.get(name, 16))
    kw.setdefault("max_tokens", 1024)
    kw.setdefault("max_requests", 4)
    return Runner(model, **kw)


def feed(runner, request, tokens, cuts):
    """The request's tokens in portions of the sizes in `cuts` (the rest one by one); logits of every position, on the host."""
    from geneinfer_amd.engine import StepEntry
    rows, at = [], 0
    sizes = list(cuts) + [1] * (len(tokens) - sum(cuts))
    for n in sizes:
        rows.append(runner.step([StepEntry(request, tokens[at:at + n], tuple(range(n)))]).cpu())
        at += n
    return torch.cat(rows)


def check_against_plain(folders, name, dtype, tokens, got, what):
    exact = plain_logits(folders, name, tokens)
    if dtype == "float32":            # within 4 times what the plain model itself loses in 32-bit
        single = plain_logits(folders, name, tokens, dtype=torch.float32)
        noise = max(relative_error(single[p], exact[p]) for p in range(len(tokens)))
        err = max(relative_error(got[p], exact[p]) for p in range(len(tokens)))
        assert err < 4 * noise + 1e-5, f"{what}: float32 logits differ from the plain implementation by {err:.2e} (the plain model in 32-bit: {noise:.2e})"
    else:
        rounded = plain_logits(folders, name, tokens, rounded=True)
        assert_within_bfloat16_noise({p: got[p] for p in range(len(tokens))}, lambda p: exact[p], lambda p: rounded[p], what)


# =============================================================================================== kernels alone
def _context(seg_len, seg_pos0, seg_slot):
    """Positions and slots of a step's rows on the device, and the longest portion."""
    pos = [p + i for n, p in zip(seg_len, seg_pos0) for i in range(n)]
    slot = [s for n, s in zip(seg_len, seg_slot) for _ in range(n)]
    return torch.tensor(pos, dtype=torch.int32, device=DEV), torch.tensor(slot, dtype=torch.int32, device=DEV), max(seg_len)


@pytest.mark.parametrize("n, width, out_dtype", [(1, 50, torch.float32), (3, 64, torch.float32), (4, 192, torch.bfloat16), (2, 700, torch.float32), (16, 33, torch.float32)])
def test_the_copies_sum_norm_and_blend_with_the_row_before_across_steps(n, width, out_dtype):
    """Three requests whose rows come in portions over four steps, in changing order and slots 2, 0, 5: every row's blend takes the row
    before it from the same step or, at a portion's start, from the slot the step before left; position 0 takes zeros whatever the
    slot holds."""
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(n * width)
    lengths = {"a": 9, "b": 4, "c": 6}
    slot_of = {"a": 2, "b": 0, "c": 5}
    x_all = {r: torch.randn(L, n * width, generator=g) for r, L in lengths.items()}
    read, norm_w, shift = torch.randn(n, generator=g), 1 + 0.1 * torch.randn(width, generator=g), torch.rand(width, generator=g) * 2 - 0.5
    eps = 1e-5
    want = {}
    for r, x in x_all.items():
        u = P.read_streams(x.double().reshape(-1, n, width).transpose(0, 1), read.double())
        want[r] = P.shifted(P.rms_norm(u, norm_w.double(), eps), shift.double())
    state = torch.full((7, width), 99.0, device=DEV)             # what an earlier request left in the slots
    steps = [[("a", 3), ("b", 1)], [("c", 2), ("a", 1)], [("b", 3), ("a", 4), ("c", 1)], [("c", 3), ("a", 1)]]
    at, got = {r: 0 for r in lengths}, {r: [] for r in lengths}
    for step in steps:
        pos, slot, longest = _context([k for _, k in step], [at[r] for r, _ in step], [slot_of[r] for r, _ in step])
        x = torch.cat([x_all[r][at[r]:at[r] + k] for r, k in step]).to(DEV)
        out = torch.empty(x.shape[0], width, dtype=out_dtype, device=DEV)
        kw = dict(read=read.to(DEV), norm_weight=norm_w.to(DEV), eps=eps, shift=shift.to(DEV), state=state, positions=pos, slots=slot)
        if longest == 1:
            ops.streams_norm_shift(x, n, out, mode=3, **kw)
        else:
            ops.streams_norm_shift(x, n, out, mode=1, **kw)
            ops.streams_norm_shift(x, n, out, mode=2, **kw)
        row = 0
        for r, k in step:
            got[r].append(out[row:row + k].float().cpu())
            row, at[r] = row + k, at[r] + k
    tol = 1e-5 if out_dtype == torch.float32 else 6e-3
    for r in lengths:
        assert relative_error(torch.cat(got[r]), want[r]) < tol, r
    # without a blend, and without a norm: the weighted sum alone; without weights: the plain sum
    x = torch.randn(5, n * width, generator=g).to(DEV)
    plain = torch.empty(5, width, device=DEV)
    ops.streams_norm_shift(x, n, plain, read=read.to(DEV))
    assert relative_error(plain, P.read_streams(x.cpu().double().reshape(5, n, width).transpose(0, 1), read.double())) < 1e-6
    ops.streams_norm_shift(x, n, plain)
    assert relative_error(plain, x.cpu().double().reshape(5, n, width).sum(1)) < 1e-6


@pytest.mark.parametrize("n, width", [(1, 50), (3, 64), (4, 300), (16, 7)])
def test_the_copies_written_back_and_the_start(n, width):
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(n + width)
    x, y = torch.randn(6, n * width, generator=g), torch.randn(6, width, generator=g)
    mix, write = torch.eye(n) + 0.3 * torch.randn(n, n, generator=g), torch.randn(n, generator=g)
    want = P.write_streams(x.double().reshape(6, n, width).transpose(0, 1), y.double(), mix.double(), write.double(), 0.7).transpose(0, 1).reshape(6, n * width)
    got = ops.streams_write(x.to(DEV), n, y.to(DEV), mix.to(DEV), write.to(DEV), 0.7)
    assert relative_error(got, want) < 1e-6
    got = ops.streams_write(x.to(DEV), n, y.to(DEV), None, None, 1.3)          # every copy keeps itself and takes the result
    assert relative_error(got, x.double() + 1.3 * y.double().repeat(1, n)) < 1e-6
    x0 = torch.randn(6, width, generator=g).to(DEV)
    assert torch.equal(ops.streams_spread(x0, torch.empty(6, n * width, device=DEV), n), x0.repeat(1, n))


@pytest.mark.parametrize("n, width, out_dtype", [(1, 64, torch.float32), (3, 192, torch.float32), (4, 2048, torch.bfloat16), (8, 36, torch.float32)])
def test_a_result_written_into_the_copies_and_the_next_input_read_out_of_them_in_one_kernel(n, width, out_dtype):
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(n * width + 1)
    x, y = torch.randn(7, n * width, generator=g), torch.randn(7, width, generator=g)
    mix, write, read = torch.eye(n) + 0.3 * torch.randn(n, n, generator=g), torch.randn(n, generator=g), torch.randn(n, generator=g)
    norm_w = 1 + 0.1 * torch.randn(width, generator=g)
    assert ops.streams_write_norm_takes(n, width) and not ops.streams_write_norm_takes(9, width) and not ops.streams_write_norm_takes(n, width + 1)
    new = P.write_streams(x.double().reshape(7, n, width).transpose(0, 1), y.double(), mix.double(), write.double(), 0.7)
    want = P.rms_norm(P.read_streams(new, read.double()), norm_w.double(), 1e-5)
    xd, out = x.to(DEV), torch.empty(7, width, dtype=out_dtype, device=DEV)
    ops.streams_write_norm(xd, n, y.to(DEV), mix.to(DEV), write.to(DEV), 0.7, read.to(DEV), norm_w.to(DEV), 1e-5, out)
    assert relative_error(xd, new.transpose(0, 1).reshape(7, n * width)) < 1e-6
    assert relative_error(out, want) < (1e-5 if out_dtype == torch.float32 else 6e-3)
    # the two kernels it stands for give the same copies, bit for bit, and the same rows up to the order of the sums
    x2 = ops.streams_write(x.to(DEV), n, y.to(DEV), mix.to(DEV), write.to(DEV), 0.7)
    assert torch.equal(x2, xd)
    out2 = ops.streams_norm_shift(x2, n, torch.empty_like(out), read=read.to(DEV), norm_weight=norm_w.to(DEV), eps=1e-5)
    assert relative_error(out2, out) < (1e-6 if out_dtype == torch.float32 else 1e-2)


def test_products_behind_the_experts_come_out_of_the_router_s_kernel():
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(11)
    for dtype in (torch.float32, torch.bfloat16):
        h, router = torch.randn(20, 72, generator=g).to(dtype), torch.randn(6 + 2, 72, generator=g).to(dtype)
        ids, weights = torch.empty(20, 2, dtype=torch.int32, device=DEV), torch.empty(20, 2, device=DEV)
        ids2, weights2, extra = torch.empty_like(ids), torch.empty_like(weights), torch.empty(20, 2, device=DEV)
        ops.route_rows(h.to(DEV), router.to(DEV)[:6], 2, ids, weights, "softmax", True, groups=(3, 2))
        ops.route_rows(h.to(DEV), router.to(DEV), 2, ids2, weights2, "softmax", True, groups=(3, 2), extra=extra)
        assert torch.equal(ids, ids2) and torch.equal(weights, weights2)
        assert relative_error(extra, h.double() @ router.double()[6:].T) < 1e-6


@pytest.mark.parametrize("experts, top, groups, keep", [(6, 2, 3, 2), (16, 4, 4, 3), (8, 2, 2, 1), (4, 1, 4, 2), (64, 8, 8, 4), (130, 4, 10, 3), (12, 12, 3, 3), (9, 2, 1, 1)])
def test_the_router_chooses_among_the_best_groups(experts, top, groups, keep):
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(experts + top)
    logits = 2 * torch.randn(40, experts, generator=g)
    logits[5, 0] = logits[5].max() + 3               # one expert that takes its whole group in, however weak the others of the group are
    scores = torch.softmax(logits.double(), dim=-1)
    want_ids, want_w = P.choose_experts(scores, top, groups, keep)
    ids, weights = torch.empty(40, top, dtype=torch.int32, device=DEV), torch.empty(40, top, device=DEV)
    ops.route_top(logits.to(DEV), top, ids, weights, "softmax", True, groups=(groups, keep), floor=1e-20)
    assert torch.equal(ids.cpu().long().sort(dim=-1).values, want_ids.sort(dim=-1).values)
    order = ids.cpu().long().argsort(dim=-1)
    assert relative_error(weights.cpu().gather(1, order), want_w.gather(1, want_ids.argsort(dim=-1))) < 1e-5
    h, router = torch.randn(40, 56, generator=g), torch.randn(experts, 56, generator=g)
    ids2, weights2 = torch.empty_like(ids), torch.empty_like(weights)
    ops.route_rows(h.to(DEV), router.to(DEV), top, ids2, weights2, "softmax", True, groups=(groups, keep), floor=1e-20)
    w_ids, _ = P.choose_experts(torch.softmax(h.double() @ router.double().T, dim=-1), top, groups, keep)
    assert torch.equal(ids2.cpu().long().sort(dim=-1).values, w_ids.sort(dim=-1).values)
    with pytest.raises(ops.KernelError):
        ops.route_top(logits.to(DEV), top, ids, weights, "softmax", True, groups=(experts + 1, 1))


@pytest.mark.parametrize("rows, d, ff, E, top, dtype", [(7, 50, 10, 3, 3, "float32"), (1, 64, 24, 5, 2, "float32"), (33, 128, 64, 8, 2, "bfloat16"), (300, 64, 48, 6, 1, "float32"),
                                                        (150, 256, 96, 4, 2, "bfloat16"), (2, 128, 64, 8, 2, "bfloat16")])
def test_clamped_experts_and_the_clamped_feed_forward(rows, d, ff, E, top, dtype):
    """The gated feed-forward with clamped halves, alone and as the experts of a mixture, with limits that many values pass."""
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(rows + d)
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    h = torch.randn(rows, d, generator=g).to(td)
    gate, up, down = (0.3 * torch.randn(E, ff, d, generator=g)).to(td), (0.3 * torch.randn(E, ff, d, generator=g)).to(td), (0.3 * torch.randn(E, d, ff, generator=g)).to(td)
    limit = 1.1
    gu = torch.cat([h.double() @ gate[0].double().T, h.double() @ up[0].double().T], dim=1)
    assert float((gu.abs() > limit).double().mean()) > 0.1
    mid = torch.empty(rows, ff, dtype=td, device=DEV)
    ops.act_mul(gu.float().to(DEV), mid, "swish_clamped", limit)
    gg, uu = torch.clamp(gu[:, :ff], max=limit), torch.clamp(gu[:, ff:], -limit, limit)
    assert relative_error(mid, gg * torch.sigmoid(1.702 * gg) * (uu + 1)) < (1e-5 if dtype == "float32" else 6e-3)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(rows)]).to(torch.int32)
    weights = torch.rand(rows, top, generator=g)
    store = P.same if dtype == "float32" else P.to_bfloat16_and_back
    want = torch.zeros(rows, d, dtype=F64)
    for t in range(rows):
        for j in range(top):
            e = int(ids[t, j])
            want[t] += float(weights[t, j]) * P.clamped_gated(h[t:t + 1].double(), gate[e].double(), up[e].double(), down[e].double(), limit, store)[0]
    x = torch.zeros(rows, d, device=DEV)
    if dtype == "bfloat16":
        w_gate, w_up = torch.stack([ops.interleave_gate_up(gate[e], up[e]) for e in range(E)]).to(DEV), None
    else:
        w_gate, w_up = gate.to(DEV), up.to(DEV)
    ops.routed_experts(h.to(DEV), w_gate, w_up, down.to(DEV), ids.to(DEV), weights.to(DEV), x, accumulate=False, weigh="output", activation="swish_clamped", limit=limit)
    assert relative_error(x, want) < (2e-5 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("T, far, dtype", [(300, 3, "float32"), (257, 0, "float32"), (130, 64, "bfloat16"), (70, 1, "float32"), (2, 0, "float32"), (1, 0, "float32"), (200, 15, "bfloat16"),
                                           (200, 16, "bfloat16")])
def test_capped_scores_with_keys_that_would_stand_out(T, far, dtype):
    """Queries and keys made so that the key at `far` scores far above the cap for the last row (it points where that row's queries
    point), and many others above it too: with the cap they weigh the same, without it the far key would be all the last row sees.
    A norm over the whole projections and a rotation of a part of the head come first, by the kernel that stores the keys."""
    from geneinfer_amd.kernels import ops
    H, G, d, e, page, rot, cap, scale, eps = 4, 2, 16, 24, 16, 8, 2.5, 1.0, 1e-5
    if dtype == "bfloat16":
        d = e = 64
    g = torch.Generator().manual_seed(T + far)
    q, k, v = torch.randn(T, H * d, generator=g), torch.randn(T, G * d, generator=g), torch.randn(T, G * e, generator=g)
    k[far] = torch.cat([q[T - 1, (j * (H // G)) * d:(j * (H // G) + 1) * d] for j in range(G)])
    q_w, k_w = 1 + 0.2 * torch.randn(H * d, generator=g), 1 + 0.2 * torch.randn(G * d, generator=g)
    f = P.plain_frequencies(rot, 100.0)
    cos, sin = P.angles(T, f, F64)
    qn, kn = P.rms_norm(q.double(), q_w.double(), eps).reshape(T, H, d), P.rms_norm(k.double(), k_w.double(), eps).reshape(T, G, d)
    store = P.same if dtype == "float32" else P.to_bfloat16_and_back
    qr, kr = store(P.turn_halves(qn, cos, sin)), store(P.turn_halves(kn, cos, sin))
    want = P.causal_softmax_attention(qr, kr, store(v.double().reshape(T, G, e)), scale, cap).reshape(T, H * e)
    free = P.causal_softmax_attention(qr, kr, store(v.double().reshape(T, G, e)), scale).reshape(T, H * e)
    td = torch.float32 if dtype == "float32" else torch.bfloat16
    n_pages = -(-T // page)
    cache = torch.zeros(n_pages + 1, G * page * (d + e), dtype=td, device=DEV)
    table = torch.arange(n_pages, 0, -1, dtype=torch.int32, device=DEV).reshape(1, -1).contiguous()          # the request's pages in falling order
    pos, slot = torch.arange(T, dtype=torch.int32, device=DEV), torch.zeros(T, dtype=torch.int32, device=DEV)
    q_out = torch.empty(T, H * d, dtype=td, device=DEV)
    ops.norm_rope_store(q.to(DEV), k.to(DEV), v.to(DEV), q_w.to(DEV), k_w.to(DEV), eps, cos.float().to(DEV).contiguous(), sin.float().to(DEV).contiguous(), rot, pos, slot, table,
                        q_out, cache, page, H, G, d, e, norm_all=True)
    assert relative_error(q_out, qr.reshape(T, H * d)) < (1e-5 if dtype == "float32" else 5e-3)
    out = torch.empty(T, H * e, dtype=td, device=DEV)
    ops.attention_exact(q_out, cache, out, pos, slot, table, H, G, d, scale=scale, page_size=page, value_dim=e, cap=cap)
    tol = 2e-5 if dtype == "float32" else 1e-2
    assert relative_error(out, want) < tol
    if T > 60:
        assert relative_error(want, free) > 0.05           # the cap matters in this case


def test_the_gate_per_head_and_rows_added_times_their_gate():
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    a, gate = torch.randn(9, 3 * 10, generator=g), torch.randn(9, 5, generator=g)
    want = (a.double().reshape(9, 3, 10) * torch.sigmoid(gate.double()[:, :3, None])).reshape(9, 30)
    assert relative_error(ops.head_gate(a.to(DEV), gate.to(DEV), 3, 10), want) < 1e-6
    assert relative_error(ops.head_gate(a.to(torch.bfloat16).to(DEV), gate.to(DEV), 3, 10), want) < 6e-3
    x, y = torch.randn(9, 70, generator=g), torch.randn(9, 70, generator=g)
    wide = torch.randn(9, 4, generator=g)
    got = ops.add_rows_gated(x.to(DEV), y.to(DEV), wide.to(DEV)[:, 2:3])
    assert relative_error(got, x.double() + torch.sigmoid(wide.double()[:, 2:3]) * y.double()) < 1e-6


# =============================================================================================== whole models
def _portions(n):
    sizes, out = (7, 2, 5, 3, 2, 11, 1, 4), []
    while sum(out) + sizes[len(out) % len(sizes)] <= n:
        out.append(sizes[len(out) % len(sizes)])
    return out


CUTS = {"whole": lambda n: [n], "singly": lambda n: [], "most then singly": lambda n: [n - 9], "portions": _portions, "twos": lambda n: [2] * (n // 2)}


@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_residual_stream_after_every_layer_run(folders, name):
    """Layer by layer, layers that run with another's weights included: the first difference names the layer."""
    tokens = _prompt(CONFIGS[name], 21, 3)
    want, _ = P.PlainMimitar(folders[name]).layer_runs(tokens)
    runner = make_runner(folders, name, "float32")
    runner.open("r")
    last = {}
    runner.model.set_trace(lambda tag, i, rows: last.__setitem__(i, rows.float().cpu()) if tag == "ffn_out" else None)
    try:
        feed(runner, "r", tokens, [len(tokens)])
    finally:
        runner.model.set_trace(None)
    assert len(last) == len(want) == len(CONFIGS[name]["layers"])
    for i in sorted(last):
        assert relative_error(last[i], want[i]) < 2e-5, f"{name}: the stream differs behind layer run {i}"


@pytest.mark.parametrize("name", list(CONFIGS))
def test_float32_logits_match_the_plain_model_and_do_not_depend_on_the_cut(folders, name):
    tokens = _prompt(CONFIGS[name], 75, 5)
    runner = make_runner(folders, name, "float32")
    got = {}
    for what, cuts in CUTS.items():
        runner.open(what)
        got[what] = feed(runner, what, tokens, cuts(len(tokens)))
        runner.close(what)
    check_against_plain(folders, name, "float32", tokens, got["whole"], f"{name} whole")
    for what in CUTS:
        assert torch.equal(got[what], got["whole"]), f"{name}: the logits of '{what}' differ from those of the whole prompt"


@pytest.mark.parametrize("name", list(CONFIGS))
def test_bfloat16_logits_lie_within_rounding_noise(folders, name):
    tokens = _prompt(CONFIGS[name], 90, 6)
    runner = make_runner(folders, name, "bfloat16")
    for what in ("whole", "portions", "most then singly", "twos"):
        runner.open(what)
        got = feed(runner, what, tokens, CUTS[what](len(tokens)))
        runner.close(what)
        check_against_plain(folders, name, "bfloat16", tokens, got, f"{name} {what}")


def test_the_block_s_one_kernel_and_the_parts_one_after_the_other_agree(folders):
    """The copies' sum, norm and blend as one kernel (the block's way) and as the stream's sum, the norm's kernel and the token-shift
    mixer's own blend: the same logits in 32-bit up to the last digits, under a cut that crosses steps."""
    from geneinfer_amd.parts.multistream import MultiStreamBlock
    tokens = _prompt(CONFIGS["A"], 40, 8)
    got = {}
    for fuse in (True, False):
        MultiStreamBlock.FUSE = fuse
        try:
            runner = make_runner(folders, "A", "float32")
            runner.open("r")
            got[fuse] = feed(runner, "r", tokens, [7, 2, 5, 1, 1, 11])
        finally:
            MultiStreamBlock.FUSE = True
    assert relative_error(got[True], got[False]) < 1e-5
    check_against_plain(folders, "A", "float32", tokens, got[False], "A, parts one after the other")


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "float32"), ("C", "float32"), ("D", "float32"), ("A", "bfloat16"), ("B", "bfloat16")])
def test_mixed_batches_on_a_pool_that_is_used_again(folders, name, dtype):
    """Up to four live requests, portions of some beside single tokens of others, through a pool that holds less than all requests
    together and four state slots: pages and slots are freed and used again.  Every request's logits against itself alone."""
    import random
    import traces
    from geneinfer_amd.engine import StepEntry
    cfg = CONFIGS[name]
    rng = random.Random(8)
    requests = {f"q{i}": [rng.randrange(cfg["vocab"]) for _ in range(n)] for i, n in enumerate([50, 1, 33, 77, 40, 9, 2, 61])}
    steps = traces.mixed(requests, seed=5)
    runner = make_runner(folders, name, dtype, max_tokens=traces.peak_tokens(steps, 64), max_requests=4)
    got = {}
    where = traces.wanted_positions(steps)
    for s in steps:
        for e in s["entries"]:
            if not runner.is_open(e["id"]):
                runner.open(e["id"])
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            for key, row in zip(where[s["step"]], logits.cpu()):
                got[key] = row.clone()
        for rid in s["end"]:
            runner.close(rid)
    runner.cache.check_consistency()
    alone = make_runner(folders, name, dtype)
    for rid, tokens in requests.items():
        mine = {p: row for (r, p), row in got.items() if r == rid}
        assert len(mine) == len(tokens)
        if dtype == "float32":
            alone.open(rid)
            ref = feed(alone, rid, tokens, [len(tokens)])
            alone.close(rid)
            assert all(torch.equal(mine[p], ref[p]) for p in mine), f"{name} {rid}: a mixed batch changed the logits"
        else:
            exact, rounded = plain_logits(folders, name, tokens), plain_logits(folders, name, tokens, rounded=True)
            assert_within_bfloat16_noise(mine, lambda p: exact[p], lambda p: rounded[p], f"{name} mixed {rid}")


@pytest.mark.parametrize("name, dtype", [("B", "bfloat16"), ("C", "float32"), ("B", "float32")])
def test_long_portions_beside_single_rows(folders, name, dtype):
    """Steps that hold portions of a hundred rows and more of some requests beside single rows and short portions of others, every
    request at another position; keys hundreds of positions back, across many pages."""
    from geneinfer_amd.engine import StepEntry
    cfg = CONFIGS[name]
    tokens = {r: _prompt(cfg, n, 70 + n) for r, n in (("a", 330), ("b", 150), ("c", 171), ("d", 40))}
    schedule = [[("a", 100), ("c", 70)], [("a", 130), ("b", 1), ("c", 1)], [("b", 140), ("a", 1), ("c", 99), ("d", 3)], [("a", 99), ("b", 2), ("c", 1), ("d", 37)], [("b", 7)]]
    runner = make_runner(folders, name, dtype, max_tokens=1024, max_requests=4)
    at, got = {r: 0 for r in tokens}, {r: [] for r in tokens}
    for step in schedule:
        entries = []
        for r, n in step:
            if not runner.is_open(r):
                runner.open(r)
            entries.append(StepEntry(r, tokens[r][at[r]:at[r] + n], tuple(range(n))))
        logits = runner.step(entries).cpu()
        row = 0
        for r, n in step:
            got[r].append(logits[row:row + n])
            row += n
            at[r] += n
    assert all(at[r] == len(t) for r, t in tokens.items())
    alone = make_runner(folders, name, dtype)
    for r, t in tokens.items():
        mine = torch.cat(got[r])
        if dtype == "float32":
            alone.open(r)
            assert torch.equal(mine, feed(alone, r, t, [len(t)])), f"{name} {r}: a mixed step changed the logits"
            alone.close(r)
        check_against_plain(folders, name, dtype, t, mine, f"{name} {r} in mixed steps")


def test_long_decoding_through_the_captured_step(folders):
    """A short prompt and 300 tokens decoded one by one through the captured decode step: the row before every row comes from the
    request's slot, layer by layer, the layers that share weights each from their own."""
    tokens = _prompt(CONFIGS["A"], 312, 9)
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folders, "A", dtype)
        runner.open("r")
        got = feed(runner, "r", tokens, [12])
        assert runner.steps_replayed > 250
        check_against_plain(folders, "A", dtype, tokens, got, f"A decoding ({dtype})")


def test_a_lost_row_before_or_a_shared_slot_shows(folders, tmp_path):
    """Weights made so that a fault shows: the blend takes all of the row before (shift = 1) in every layer, so each layer's mixer sees
    the token before only, and a slot that is lost between steps, or shared by the layers that run with the same weights, changes
    every logit."""
    cfg = CONFIGS["A"]
    w = random_weights(cfg, 77)
    for name in w:
        if name.endswith(".shift"):
            w[name] = torch.ones_like(w[name])
    folder = tmp_path / "shifted"
    write_model(folder, cfg, weights=w)
    tokens = _prompt(cfg, 60, 12)
    own = {"A": folder}
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(own, "A", dtype, page_size=4)
        runner.open("r")
        got = feed(runner, "r", tokens, [5, 1, 1, 17, 2])
        check_against_plain(own, "A", dtype, tokens, got, f"everything from the row before ({dtype})")
    # the plain model with the blend switched off differs by far more than any tolerance here: the test can see the blend
    off = dict(w)
    for name in w:
        if name.endswith(".shift"):
            off[name] = torch.zeros_like(w[name])
    a = P.PlainMimitar(config=cfg, tensors={k: v.to(torch.bfloat16) for k, v in w.items()}).logits(tokens)
    b = P.PlainMimitar(config=cfg, tensors={k: v.to(torch.bfloat16) for k, v in off.items()}).logits(tokens)
    assert relative_error(a, b) > 0.1


def test_layers_in_another_order_and_a_layer_that_names_a_later_one_s_weights(folders, tmp_path):
    """Configuration A's layers backwards, so that the first layer runs with the weights of the fourth and attention through latents
    comes before the layer whose weights it uses: order and ownership are the configuration's, nothing of them is fixed."""
    import copy
    cfg = copy.deepcopy(CONFIGS["A"])
    layers = cfg["layers"][::-1]
    n = len(layers)
    for l in layers:
        if "weights_of" in l:
            l["weights_of"] = n - 1 - l["weights_of"]
    cfg["layers"] = layers
    assert [l.get("weights_of") for l in layers] == [3, None, 4, None, None]
    write_model(tmp_path / "m", cfg, seed=19)
    own = {"A": tmp_path / "m"}
    tokens = _prompt(cfg, 50, 14)
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(own, "A", dtype)
        runner.open("r")
        got = feed(runner, "r", tokens, [13, 2, 20, 1])
        check_against_plain(own, "A", dtype, tokens, got, f"layers backwards ({dtype})")


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point_and_the_scheduler(folders, name):
    """Greedy tokens of several prompts, one by one through `LLM.generate` and together through the scheduler (more requests than
    it runs at once, prompts in portions), against the plain model's, as far as the plain model's two best logits are clearly apart."""
    import geneinfer_amd as gi
    from geneinfer_amd.engine import EngineConfig, EngineRequest
    from geneinfer_amd.sampling import SamplerConfig
    cfg = CONFIGS[name]
    plain = P.PlainMimitar(folders[name])
    prompts = [_prompt(cfg, n, 30 + n) for n in (5, 23, 1, 40)]
    want, sure = [], []
    for p in prompts:
        tokens = plain.greedy(p, 8)
        top2 = torch.topk(plain.logits(p + tokens)[len(p) - 1:-1], 2, dim=-1).values
        clear = [bool(c) for c in (top2[:, 0] - top2[:, 1] > 1e-3)]
        want.append(tokens)
        sure.append(clear.index(False) if False in clear else len(clear))
    assert sum(sure) >= 24
    llm = gi.LLM(str(folders[name]), dtype="float32", page_size=PAGE_SIZE[name], max_tokens=512, max_running=2)
    assert type(llm.model.config).__name__ == "MimitarConfig"
    for p, t, n in zip(prompts, want, sure):
        assert llm.generate(p, steps=len(p) + 7, temperature=0.0).generated_tokens[:n] == t[:n]
    eng = llm.engine(EngineConfig(max_running=2, step_rows=16, prefill_chunk=6))
    ids = [eng.submit(EngineRequest(p, len(p) + 7, SamplerConfig(0.0))) for p in prompts]
    eng.run_until_idle()
    for i, t, n in zip(ids, want, sure):
        assert eng.result(i).generated_tokens[:n] == t[:n]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_through_the_command_line(folders, tmp_path, dtype):
    """bin/trace_run as a child process on a Mimitar folder: up to four live requests, portions beside single tokens, a pool that
    holds less than all requests together, so that pages and state slots are used again."""
    import json
    import random
    import subprocess
    from pathlib import Path
    import numpy as np
    import traces
    root = Path(__file__).resolve().parent.parent
    cfg = CONFIGS["B"]
    rng = random.Random(4)
    requests = {f"q{i}": [rng.randrange(cfg["vocab"]) for _ in range(n)] for i, n in enumerate([50, 1, 33, 77, 40, 9])}
    steps = traces.mixed(requests, seed=3)
    out = tmp_path / "out"
    cmd = [str(root / "bin" / "trace_run"), "--model", str(folders["B"]), "--dtype", dtype, "--out", str(out), "--max-tokens", str(traces.peak_tokens(steps, 64))]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {s['step']}", (line, proc.stderr.read() if proc.poll() is not None else "")
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0, proc.stderr.read()
    finally:
        if proc.poll() is None:
            proc.kill()
    got = {}
    for step, rows in traces.wanted_positions(steps).items():
        data = np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"])
        for key, row in zip(rows, data):
            got[key] = torch.from_numpy(row.copy())
    for rid, tokens in requests.items():
        mine = {p: row for (r, p), row in got.items() if r == rid}
        assert len(mine) > 0
        exact = plain_logits(folders, "B", tokens)
        if dtype == "float32":
            single = plain_logits(folders, "B", tokens, dtype=torch.float32)
            noise = max(relative_error(single[p], exact[p]) for p in mine)
            assert max(relative_error(row, exact[p]) for p, row in mine.items()) < 4 * noise + 1e-5
        else:
            rounded = plain_logits(folders, "B", tokens, rounded=True)
            assert_within_bfloat16_noise(mine, lambda p: exact[p], lambda p: rounded[p], f"replay {rid}")


def test_generation_from_the_command_line_on_random_weights():
    """bin/gi_generate on the shipped example configuration, random weights, greedy: runs, and twice the same."""
    import subprocess
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    cmd = [str(root / "bin" / "gi_generate"), "--config", str(root / "configs" / "mimitar-small.json"), "--random-seed", "3", "--prompt-ids", "5 17 3 999 4",
           "--steps", "24", "--temperature", "0"]
    runs = [subprocess.run(cmd, capture_output=True, text=True, timeout=280) for _ in range(2)]
    assert all(r.returncode == 0 for r in runs), runs[0].stderr[-2000:]
    assert runs[0].stdout == runs[1].stdout and len(runs[0].stdout.split()) >= 20


def test_the_new_parts_serve_other_designs():
    """The token-shift mixer under the ordinary pre-norm block around a Llama attention, and a norm with weights stored around zero:
    built from specs alone, without a Mimitar configuration, and run under two cuts with equal bits."""
    from geneinfer_amd.config.spec import AttentionSpec, LayerSpec, ModelSpec, RmsNormSpec, RotarySpec, RunEntry, SwiGluSpec, TokenShiftSpec
    from geneinfer_amd.engine import Runner
    from geneinfer_amd.engine.model import DecoderModel
    from geneinfer_amd.parts import model_tensor_needs
    from geneinfer_amd.weights import random_tensors
    d = 32
    attention = AttentionSpec(hidden_size=d, n_heads=2, n_kv_heads=1, head_dim=16, q_proj="q", k_proj="k", v_proj="v", o_proj="o", position=RotarySpec(16, 100.0))
    layer = LayerSpec(mixer=TokenShiftSpec(d, "shift", attention), feed_forward=SwiGluSpec(d, 48, "gate", "up", "down"),
                      mixer_norm=RmsNormSpec(d, 1e-5, "n1", weight_offset=1.0), feed_forward_norm=RmsNormSpec(d, 1e-5, "n2"))
    spec = ModelSpec(architecture="test", vocab_size=90, hidden_size=d, max_positions=256, embedding="embed", final_norm=RmsNormSpec(d, 1e-5, "nf"), lm_head="embed",
                     layers=(layer,), run_order=(RunEntry(0), RunEntry(0)))
    tensors = {k: v.to(DEV) for k, v in random_tensors(model_tensor_needs(spec), 3, torch.float32, 0.2).items()}
    model = DecoderModel(spec, tensors, torch.float32, DEV)
    tokens = list(range(3, 40))
    got = []
    for cuts in ([len(tokens)], [5, 2, 9, 1, 1, 3]):
        runner = Runner(model, page_size=4, max_tokens=256, max_requests=2)
        runner.open("r")
        got.append(feed(runner, "r", tokens, cuts))
    assert torch.equal(got[0], got[1])
    # against a statement of the same model in the plain implementation's functions
    w = {k: v.double().cpu() for k, v in tensors.items()}
    x = w["embed"][torch.tensor(tokens)]
    for _ in range(2):
        h = P.shifted(P.one_plus_norm(x, w["n1"], 1e-5), w["shift"])
        T = len(tokens)
        q, k, v = (h @ w["q"].T).reshape(T, 2, 16), (h @ w["k"].T).reshape(T, 1, 16), (h @ w["v"].T).reshape(T, 1, 16)
        cos, sin = P.angles(T, P.plain_frequencies(16, 100.0), F64)
        o = P.causal_softmax_attention(P.turn_halves(q, cos, sin), P.turn_halves(k, cos, sin), v, 16 ** -0.5)
        x = x + o.reshape(T, 32) @ w["o"].T
        h = P.rms_norm(x, w["n2"], 1e-5)
        g = h @ w["gate"].T
        x = x + (g * torch.sigmoid(g) * (h @ w["up"].T)) @ w["down"].T
    want = P.rms_norm(x, w["nf"], 1e-5) @ w["embed"].T
    assert relative_error(got[0], want) < 2e-5


@pytest.mark.parametrize("case", range(10))
def test_capped_scores_in_the_matrix_core_kernels(case):
    """Steps drawn at random through the bfloat16 attention kernels with a cap on the scores (both prompt kernels, the decode kernel,
    keys shared out over workgroups) against a dense 64-bit computation: single rows, short portions and up to 900 rows on top of up
    to 2,000 cached positions, scores several times the cap, pages on scrambled numbers between pages of NaN."""
    import random
    from geneinfer_amd.kernels import ops
    from geneinfer_amd.parts import StepContext
    rng = random.Random(300 + case)
    torch.manual_seed(case)
    hd = (64, 128)[case % 2]
    KV = rng.choice([1, 2, 4])
    H = KV * rng.choice([1, 2, 4])
    page = rng.choice([16, 32, 64])
    cap, scale = rng.choice([1.5, 5.0, 30.0]), rng.choice([0.125, 0.5])
    segs = []
    for s in range(rng.randrange(1, 5)):
        kind = rng.random()
        start = rng.choice([0, 0, rng.randrange(1, 2000)])
        segs.append((s, start, 1 if kind < 0.3 else rng.randrange(2, 60) if kind < 0.5 else rng.randrange(65, 900)))
    R, ctxs = len(segs), [st + n for _, st, n in segs]
    per = [-(-c // page) for c in ctxs]
    n_pages = sum(per) + 3
    cache = torch.full((n_pages, 2, KV, page, hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    perm = iter(torch.randperm(n_pages)[:sum(per)].tolist())
    table = torch.full((R, max(per)), -1, dtype=torch.int32)
    K, V = [], []
    for s, c in enumerate(ctxs):
        k, v = torch.randn(c, KV, hd, device=DEV).bfloat16(), torch.randn(c, KV, hd, device=DEV).bfloat16()
        K.append(k)
        V.append(v)
        for pi in range(per[s]):
            pg = next(perm)
            table[s, pi] = pg
            lo, hi = pi * page, min(c, (pi + 1) * page)
            bk, bv = torch.zeros(page, KV, hd, dtype=torch.bfloat16, device=DEV), torch.zeros(page, KV, hd, dtype=torch.bfloat16, device=DEV)
            bk[:hi - lo], bv[:hi - lo] = k[lo:hi], v[lo:hi]
            cache[pg, 0] = bk.permute(1, 0, 2)
            cache[pg, 1].view(KV, hd, page).copy_(bv.permute(1, 2, 0))
    table = table.to(DEV)
    rows, seg_start, seg_len, seg_pos0, seg_slot = [], [], [], [], []
    for s, st, n in segs:
        seg_start.append(len(rows)); seg_len.append(n); seg_pos0.append(st); seg_slot.append(s)
        rows += [(s, st + i) for i in range(n)]
    T = len(rows)
    q = torch.randn(T, H * hd, device=DEV).bfloat16()
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32, device=DEV)
    slots = torch.tensor([s for s, _ in rows], dtype=torch.int32, device=DEV)
    ctx = StepContext(n_rows=T, dtype=torch.bfloat16, device=torch.device(DEV), tokens=pos, row_pos=pos, row_slot=slots, seg_slot=seg_slot, seg_start=seg_start,
                      seg_len=seg_len, seg_pos0=seg_pos0)
    out = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attention_general(q, cache, out, ctx, table, H, KV, hd, page_size=page, scale=scale, cap=cap)
    want = torch.zeros(T, H * hd, dtype=F64)
    at = 0
    for s, st, n in segs:
        qq = q[at:at + n].double().cpu().reshape(n, H, hd)
        k, v = K[s].double().cpu(), V[s].double().cpu()
        for a in range(H):
            sc = cap * torch.tanh((qq[:, a] @ k[:, a // (H // KV)].T) * scale / cap)
            seen = torch.arange(k.shape[0])[None, :] <= (st + torch.arange(n))[:, None]
            want[at:at + n, a * hd:(a + 1) * hd] = torch.softmax(sc.masked_fill(~seen, float("-inf")), dim=-1) @ v[:, a // (H // KV)]
        at += n
    err = relative_error(out, want)
    assert bool(torch.isfinite(out.float()).all()) and err < 8e-3, f"case {case}: hd {hd} heads {H}:{KV} page {page} cap {cap} scale {scale} segments {segs}: {err}"
    exact = torch.empty_like(out)
    ops.attention_exact(q, cache.view(n_pages, -1), exact, pos, slots, table, H, KV, hd, scale=scale, page_size=page, cap=cap)
    assert relative_error(exact, want) < 8e-3
