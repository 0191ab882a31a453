"""The Zidevik design in the engine against the plain implementation (`plain_zidevik.py`): each kernel alone, then whole models
of five small configurations under every way of cutting the work into steps, and generation through the entry point and the
scheduler.  In float32 the engine's logits must not depend on the cutting at all (equal bits); in bfloat16 they must lie as close
to the exact model as rounding alone explains."""
import math

import pytest
import torch

import plain_zidevik as P
from model_folders import assert_within_bfloat16_noise, relative_error
from zidevik_folders import CONFIGS, PAGE_SIZE, random_weights, stored_weights, write_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _prompt(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("zidevik")
    out = {}
    for name, cfg in CONFIGS.items():
        write_model(root / name, cfg, seed=23 + ord(name))
        out[name] = root / name
    return out


_plain_cache = {}


def plain_logits(folders, name, tokens, rounded=False, dtype=torch.float64):
    key = (name, tuple(tokens), rounded, dtype)
    if key not in _plain_cache:
        _plain_cache[key] = P.forward(CONFIGS[name], stored_weights(folders[name]), tokens, dtype, store=P.to_bfloat16_and_back if rounded else P.same)
    return _plain_cache[key]


def make_runner(folders, name, dtype, **kw):
    from geneinfer_amd.engine import Runner, load_model
    model = load_model(folders[name], dtype, DEV)
    kw.setdefault("page_size", PAGE_SIZE[name])
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
def test_the_library_and_the_planner_agree_on_the_state_size():
    from geneinfer_amd.kernels import ops
    for inner, n, taps in ((1, 1, 1), (40, 5, 3), (72, 17, 4), (9, 2, 8), (4096, 16, 4)):
        assert ops.lib().gi_ssm_state_floats(inner, n, taps) == ops.ssm_state_floats(inner, n, taps)
    assert ops.lib().gi_ssm_max_taps() == ops.SSM_MAX_TAPS and ops.lib().gi_ssm_max_states() == ops.SSM_MAX_STATES


def _segs(seg_lens, slots, pos0):
    starts = [sum(seg_lens[:i]) for i in range(len(seg_lens))]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    row_slot = i32([s for s, m in zip(slots, seg_lens) for _ in range(m)])
    row_pos = i32([p + i for p, m in zip(pos0, seg_lens) for i in range(m)])
    return i32(starts), i32(seg_lens), row_slot, row_pos


@pytest.mark.parametrize("inner, N, taps", [(40, 5, 3), (72, 17, 4), (30, 1, 1), (17, 33, 3), (9, 2, 8), (256, 16, 4), (64, 100, 2), (20, 130, 5), (24, 7, 13)])
def test_selective_scan_kernels(inner, N, taps):
    """Two requests of unequal length in one step; then the longer one again from a fresh slot in steps down to one and two rows:
    the states and the convolutions' tails carry, and the bits do not change.  One channel barely decays, so that what the first
    rows left is still in the read-out of the last."""
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(inner + taps)
    lens = [29, 90]
    n = sum(lens)
    pre, z, dt_pre = torch.randn(n, inner + 3, generator=g), torch.randn(n, inner, generator=g), torch.randn(n, inner, generator=g)
    low = torch.randn(n, 2 + 2 * N + 1, generator=g)                     # B at column 2, C behind it
    w_taps, conv_b = 0.6 * torch.randn(inner, taps, generator=g), 0.5 * torch.randn(inner, generator=g)
    a_log, dt_b, D = -0.5 + 0.6 * torch.randn(inner, N, generator=g), 0.5 * torch.randn(inner, generator=g), torch.randn(inner, generator=g)
    a_log[0] = -9.0

    def plain(rows):
        x = P.silu(P.causal_convolution(pre[rows, 3:].double(), w_taps.double(), conv_b.double()))
        dt = P.softplus(dt_pre[rows].double() + dt_b.double())
        B, C, A = low[rows, 2:2 + N].double(), low[rows, 2 + N:2 + 2 * N].double(), -torch.exp(a_log.double())
        S, y = torch.zeros(inner, N, dtype=torch.float64), []
        for t in range(x.shape[0]):
            S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
            y.append(S @ C[t] + D.double() * x[t])
        return x, torch.stack(y) * P.silu(z[rows].double()), S

    first, second = slice(0, lens[0]), slice(lens[0], n)
    (x1, y1, S1), (x2, y2, S2) = plain(first), plain(second)
    width = ops.ssm_state_floats(inner, N, taps)
    state = torch.zeros(5, width + 3, device=DEV)
    dev = lambda t: t.to(DEV)
    d_taps, d_cb, d_al, d_db, d_D = dev(w_taps), dev(conv_b), dev(a_log), dev(dt_b), dev(D)

    def run(rows, seg_lens, slots, pos0):
        m = rows.stop - rows.start
        seg_start, seg_len, row_slot, row_pos = _segs(seg_lens, slots, pos0)
        p = dev(pre[rows])[:, 3:]
        x, out = torch.empty(m, inner, device=DEV), torch.empty(m, inner, device=DEV)
        single = max(seg_lens) == 1
        ops.ssm_conv(p, d_taps, d_cb, row_slot, row_pos, state, x, None, N, move_tail=single)
        if not single:
            ops.ssm_tail(p, taps, seg_start, seg_len, row_slot, state, inner, N)
        ops.ssm_scan(x, dev(dt_pre[rows]), d_db, dev(low[rows]), 2, 2 + N, dev(z[rows]), d_al, d_D, seg_start, seg_len, row_slot, state, out, N,
                     rows_per_request=seg_lens)
        return x.cpu(), out.cpu()

    x, y = run(slice(0, n), lens, [2, 0], [0, 0])
    assert relative_error(x, torch.cat([x1, x2])) < 1e-6 and relative_error(y, torch.cat([y1, y2])) < 3e-5
    assert relative_error(y[n - 1, 0], y2[-1, 0]) < 3e-5
    assert relative_error(state[0, :inner * N].view(inner, N), S2) < 3e-5 and relative_error(state[2, :inner * N].view(inner, N), S1) < 3e-5
    if taps > 1:
        assert torch.equal(state[0, inner * N:width].view(taps - 1, inner).cpu(), pre[n - (taps - 1):, 3:])
    assert (state[:, width:] == 0).all() and (state[1] == 0).all()
    # the second request again, cut small; a half-precision copy of x on the way
    cuts, pieces, at = [2, 1, 1, 40, 1, 2, 3, 38, 2], [], 0
    for c in cuts:
        pieces.append(run(slice(lens[0] + at, lens[0] + at + c), [c], [4], [at])[1])
        at += c
    assert at == lens[1] and torch.equal(torch.cat(pieces), y[lens[0]:]) and torch.equal(state[4], state[0])
    # two requests that both go on, side by side in one step, each from its own slot; then both as single rows
    for portion in ([4, 7], [1, 1]):
        state[1], state[3] = state[2], state[4]
        k = sum(portion)
        both = run(slice(0, k), portion, [1, 3], [lens[0], lens[1]])[1]
        alone = torch.cat([run(slice(0, portion[0]), [portion[0]], [2], [lens[0]])[1], run(slice(portion[0], k), [portion[1]], [4], [lens[1]])[1]])
        assert torch.equal(both, alone) and torch.equal(state[1], state[2]) and torch.equal(state[3], state[4])
    # results stored as bfloat16 (the kernel's quick exponentials): as close as their 8 bits allow
    state[1] = 0
    seg_start, seg_len, row_slot, row_pos = _segs([lens[0]], [1], [0])
    half = torch.empty(lens[0], inner, device=DEV, dtype=torch.bfloat16)
    ops.ssm_scan(dev(x1.float()), dev(dt_pre[first]), d_db, dev(low[first]), 2, 2 + N, dev(z[first]), d_al, d_D, seg_start, seg_len, row_slot, state, half, N)
    assert relative_error(half, y1) < 4e-3 and relative_error(state[1, :inner * N].view(inner, N), S1) < 3e-5
    # steps of single rows: the step sizes' product inside the scan's kernel against the same product made in front of it
    seg_start, seg_len, row_slot, _ = _segs([1, 1, 1], [2, 0, 4], [0, 0, 0])
    rows3 = slice(0, 3)
    for R in (7, 64, 96):             # (a rank the lanes take one by one, and ranks they take in pieces of eight)
        w_dt, low_dt = (0.3 * torch.randn(inner, R, generator=g)).to(torch.bfloat16), torch.randn(3, -(-(R + 2 * N) // 4) * 4, generator=g)
        made = (low_dt[:, :R].double() @ w_dt.double().T).float()
        results = []
        for dt_pre, dt_proj in ((dev(made), None), (None, (dev(w_dt), 0))):
            state[:] = 0.25
            out3 = torch.empty(3, inner, device=DEV, dtype=torch.bfloat16)
            ops.ssm_scan(dev(x1.float()[rows3]), dt_pre, d_db, dev(low_dt), R, R + N, dev(z[rows3]), d_al, d_D, seg_start, seg_len, row_slot, state, out3, N, dt_proj=dt_proj,
                         rows_per_request=[1, 1, 1])
            results.append((out3.float().cpu(), state[:, :inner * N].cpu().clone()))
        assert relative_error(results[1][0], results[0][0].double()) < 4e-3 and relative_error(results[1][1], results[0][1].double()) < 1e-5
    low_copy = torch.empty(5, inner, device=DEV, dtype=torch.bfloat16)
    seg_start, seg_len, row_slot, row_pos = _segs([5], [1], [0])
    state[1] = 0
    xf = torch.empty(5, inner, device=DEV)
    ops.ssm_conv(dev(pre[:5])[:, 3:], d_taps, d_cb, row_slot, row_pos, state, xf, low_copy, N)
    assert torch.equal(low_copy.cpu(), xf.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("inner, N, lens", [(40, 5, [300, 70, 129]), (72, 17, [128, 1, 64]), (16, 40, [513]), (33, 16, [2, 200, 191])])
def test_selective_scan_of_long_runs_cut_into_chunks(inner, N, lens):
    """Results stored as bfloat16, requests of a hundred rows and more beside short ones: the runs are cut into chunks that run at
    once.  Every request starts from a state that holds something, and one channel barely decays, so that a chunk that started from
    a wrong state would show in all rows behind it."""
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(inner + N)
    n = sum(lens)
    assert max(lens) >= ops.SSM_CHUNKS_FROM
    x, z, dt_pre = torch.randn(n, inner, generator=g), torch.randn(n, inner, generator=g), torch.randn(n, inner, generator=g) - 1.0
    low = torch.randn(n, 2 * N, generator=g)
    a_log, dt_b, D = -0.5 + 0.6 * torch.randn(inner, N, generator=g), 0.5 * torch.randn(inner, generator=g), torch.randn(inner, generator=g)
    a_log[0] = -9.0
    slots = [3, 0, 2, 1][:len(lens)]
    start = torch.randn(4, inner * N, generator=g)
    want, ends, at = [], {}, 0
    for m, slot in zip(lens, slots):
        rows = slice(at, at + m)
        dt = P.softplus(dt_pre[rows].double() + dt_b.double())
        B, C, A = low[rows, :N].double(), low[rows, N:].double(), -torch.exp(a_log.double())
        S = start[slot].double().view(inner, N).clone()
        for t in range(m):
            S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[at + t].double())[:, None] * B[t][None, :]
            want.append((S @ C[t] + D.double() * x[at + t].double()) * P.silu(z[at + t].double()))
        ends[slot] = S
        at += m
    want = torch.stack(want)
    dev = lambda t: t.to(DEV)
    seg_start, seg_len, row_slot, _ = _segs(lens, slots, [0] * len(lens))
    outs = {}
    for how in ("chunks", "in a row"):
        state = dev(start).clone()
        out = torch.empty(n, inner, device=DEV, dtype=torch.bfloat16)
        ops.ssm_scan(dev(x), dev(dt_pre), dev(dt_b), dev(low), 0, N, dev(z), dev(a_log), dev(D), seg_start, seg_len, row_slot, state, out, N,
                     rows_per_request=lens if how == "chunks" else None)
        outs[how] = out.float().cpu()
        assert relative_error(out, want) < 4e-3, how
        for slot, S in ends.items():
            assert relative_error(state[slot].view(inner, N), S) < 3e-5, (how, slot)
        assert all(torch.equal(state[s].cpu(), start[s]) for s in range(4) if s not in slots)
    assert relative_error(outs["chunks"], outs["in a row"].double()) < 2e-3            # (either is one rounding to 8 bits away from the same 32-bit number)
    assert relative_error(outs["chunks"][:, 0], want[:, 0]) < 4e-3


@pytest.mark.parametrize("experts, top", [(5, 2), (16, 1), (3, 3), (64, 8), (130, 4), (1, 1)])
def test_the_router_s_choice(experts, top):
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(experts)
    logits = 2 * torch.randn(50, experts + 2, generator=g)
    if experts > 2:
        logits[3, 1] = logits[3, 2] = logits[3].max() + 1                  # equals: the lower index first
        logits[4, :] = 0.25
    z = logits[:, :experts].double()
    for score, renorm in (("sigmoid", False), ("sigmoid", True), ("softmax", False), ("softmax", True)):
        s = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, -1)
        order = torch.sort(z, dim=-1, descending=True, stable=True).indices[:, :top]
        want = torch.gather(s, 1, order)
        if renorm:
            want = want / want.sum(-1, keepdim=True)
        ids, weights = torch.empty(50, top, dtype=torch.int32, device=DEV), torch.empty(50, top, device=DEV)
        ops.route_top(logits.to(DEV)[:, :experts], top, ids, weights, score, renorm)
        assert torch.equal(ids.cpu().long(), order) and relative_error(weights, want) < 1e-6
    # the product and the choice in one launch: the same choice from the same logits, whatever rows lie beside a row
    for dtype in (torch.float32, torch.bfloat16):
        h, router = torch.randn(50, 72, generator=g).to(dtype), torch.randn(experts, 72, generator=g).to(dtype)
        ids2, weights2, kept = torch.empty_like(ids), torch.empty_like(weights), torch.empty(50, experts, device=DEV)
        ops.route_rows(h.to(DEV), router.to(DEV), top, ids2, weights2, "softmax", True, logits=kept)
        assert relative_error(kept, h.double() @ router.double().T) < 1e-6
        ops.route_top(kept, top, ids, weights, "softmax", True)
        assert torch.equal(ids, ids2) and torch.equal(weights, weights2)
        one_i, one_w = torch.empty(1, top, dtype=torch.int32, device=DEV), torch.empty(1, top, device=DEV)
        ops.route_rows(h.to(DEV)[17:18], router.to(DEV), top, one_i, one_w, "softmax", True)
        assert torch.equal(one_i[0], ids2[17]) and torch.equal(one_w[0], weights2[17])


@pytest.mark.parametrize("rows, d, ff, E, top, dtype", [(7, 50, 10, 3, 3, "float32"), (1, 64, 24, 5, 2, "float32"), (33, 128, 64, 8, 2, "bfloat16"), (300, 64, 48, 6, 1, "float32"),
                                                        (150, 256, 96, 4, 2, "bfloat16"), (65, 40, 130, 9, 4, "float32"), (300, 128, 128, 16, 4, "bfloat16"),
                                                        (5, 192, 64, 3, 2, "bfloat16"), (2, 128, 64, 4, 2, "bfloat16"), (700, 192, 320, 5, 1, "bfloat16")])
def test_routed_experts_against_the_plain_statement(rows, d, ff, E, top, dtype):
    """Few rows and many (every expert's rows together), the score on an expert's input or on its output; the second time onto rows
    that hold something."""
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(rows + d)
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    r = lambda *s: (0.3 * torch.randn(*s, generator=g)).to(store)
    h, router = r(rows, d) * 3, torch.randn(E, d, generator=g)
    wg, wu, wd = r(E, ff, d), r(E, d, ff).transpose(1, 2).contiguous(), r(E, d, ff)
    logits = (h.float() @ router.T).contiguous()
    rounding = P.to_bfloat16_and_back if dtype == "bfloat16" else P.same
    want_in = P.routed_experts(h.double(), router.double(), [(wg[e].double(), wu[e].double(), wd[e].double()) for e in range(E)], top, store=rounding)
    s = torch.sigmoid(logits.double())
    chosen = torch.topk(s, top, dim=-1).indices
    want_out = torch.stack([sum(s[t, e] * P.gated_mlp(h[t].double()[None], wg[e].double(), wu[e].double(), wd[e].double(), store=rounding)[0] for e in chosen[t].tolist())
                            for t in range(rows)])
    dev = lambda t: t.to(DEV)
    ids, weights = torch.empty(rows, top, dtype=torch.int32, device=DEV), torch.empty(rows, top, device=DEV)
    ops.route_top(dev(logits), top, ids, weights)
    tol = 2e-2 if dtype == "bfloat16" else 3e-5
    d_h, d_wg, d_wu, d_wd = dev(h), dev(wg), dev(wu), dev(wd)
    if dtype == "bfloat16":           # as the part keeps them: an expert's gates and up products in one matrix
        d_wg, d_wu = torch.stack([ops.interleave_gate_up(d_wg[e], d_wu[e]) for e in range(E)]).contiguous(), None
        assert ops.experts_grouped_supported(d_h, d_wg, d_wu, d_wd) == (ff % 64 == 0)
    for weigh, want in (("input", want_in), ("output", want_out)):
        x = torch.full((rows, d), 0.5, device=DEV)
        ops.routed_experts(d_h, d_wg, d_wu, d_wd, ids, weights, x, accumulate=True, weigh=weigh)
        assert relative_error(x - 0.5, want) < tol, weigh
        y = torch.full((rows, d), 7.0, device=DEV)
        ops.routed_experts(d_h, d_wg, d_wu, d_wd, ids, weights, y, accumulate=False, weigh=weigh)
        assert relative_error(y, want) < tol
        if rows > 1:                                                      # a row's result does not depend on the rows beside it
            k = rows // 2
            alone = torch.zeros(1, d, device=DEV)
            ops.routed_experts(d_h[k:k + 1], d_wg, d_wu, d_wd, ids[k:k + 1].contiguous(), weights[k:k + 1].contiguous(), alone, accumulate=False, weigh=weigh)
            if dtype == "float32":
                assert relative_error(alone[0], y[k]) < 1e-6
            else:
                assert relative_error(alone[0], y[k]) < tol


def _paged(T, page, n_numbers, dtype, seed):
    """Pages for one request of T positions in slot 1, in a shuffled order, and its table."""
    n_pages = -(-T // page)
    order = torch.randperm(n_pages + 3, generator=torch.Generator().manual_seed(seed))[:n_pages]
    table = torch.full((3, n_pages + 2), -1, dtype=torch.int32)
    table[1, :n_pages] = order.to(torch.int32)
    cache = torch.zeros(n_pages + 3, page * n_numbers, dtype=dtype, device=DEV)
    return cache, table.to(DEV)


def _ctx(T, pos0=0, slot=1):
    from geneinfer_amd.parts import StepContext
    pos = torch.arange(pos0, pos0 + T, dtype=torch.int32, device=DEV)
    slots = torch.full((T,), slot, dtype=torch.int32, device=DEV)
    return StepContext(n_rows=T, dtype=torch.float32, device=torch.device(DEV), tokens=slots, row_pos=pos, row_slot=slots, seg_slot=[slot], seg_start=[0],
                       seg_len=[T], seg_pos0=[pos0])


@pytest.mark.parametrize("T, far, alone", [(300, 3, 1), (300, 0, 0), (257, 255, 1), (257, 256, 0), (256, 0, 1), (261, 4, 3), (129, 127, 2), (70, 1, 1), (2, 0, 1), (1, 0, 0)])
def test_attention_behind_turned_neighbours_and_unit_heads_with_one_key_that_stands_out(T, far, alone):
    """The last row's query points at the key of position `far`, hundreds of rows back or at a page's edge, whose channels behind the
    turned ones are lined up with it, so that it takes nearly all the weight.  Pairs of neighbouring channels are turned, then every
    head is divided by its root mean square.  The last `alone` rows come in a step of their own, from the pages."""
    from geneinfer_amd.kernels import ops
    heads, kv, dk, dv, rot, page, scale, eps, base = 4, 2, 24, 10, 8, 4, 1.0, 1e-5, 30.0
    g = torch.Generator().manual_seed(T + far)
    q, k, v = torch.randn(T, heads * dk, generator=g), torch.randn(T, kv * dk, generator=g), torch.randn(T, kv * dv, generator=g)
    k.view(T, kv, dk)[:, :, rot:] *= 0.2
    k.view(T, kv, dk)[far, :, rot:] = 3.0
    q.view(T, heads, dk)[T - 1, :, rot:] = 3.0
    unit = lambda x: x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    qd, kd = unit(P.rotate_neighbours(q.double().view(T, heads, dk), rot, base)), unit(P.rotate_neighbours(k.double().view(T, kv, dk), rot, base))
    scores = torch.einsum("thd,shd->hts", qd, kd.repeat_interleave(heads // kv, 1)) * scale
    pr = torch.softmax(scores.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool))[None], float("-inf")), -1)
    want = torch.einsum("hts,shd->thd", pr, v.double().view(T, kv, dv).repeat_interleave(heads // kv, 1))
    assert T < 3 or (pr[:, T - 1, far] > 0.9).all()                                    # (the test's premise)

    cache, table = _paged(T, page, kv * (dk + dv), torch.float32, seed=far)
    f = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float64, device=DEV)
    dev = lambda t: t.to(DEV)
    outs = []
    for lo, hi in ((0, T - alone), (T - alone, T)):
        if hi == lo:
            continue
        n, ctx = hi - lo, _ctx(hi - lo, pos0=lo)
        cos, sin = torch.empty(n, rot // 2, device=DEV), torch.empty(n, rot // 2, device=DEV)
        ops.rope_cos_sin(ctx.row_pos, f, cos, sin)
        q_ready = torch.empty(n, heads * dk, device=DEV)
        ops.norm_rope_store(dev(q[lo:hi]), dev(k[lo:hi]), dev(v[lo:hi]), None, None, eps, cos, sin, rot, ctx.row_pos, ctx.row_slot, table, q_ready, cache, page, heads, kv, dk, dv,
                            neighbours=True, unit_rms=True, norm_last=True)
        assert relative_error(q_ready.view(n, heads, dk), qd[lo:hi]) < 2e-6
        out = torch.empty(n, heads * dv, device=DEV)
        ops.attention_general(q_ready, cache, out, ctx, table, heads, kv, dk, page_size=page, value_dim=dv, scale=scale)
        outs.append(out)
    got = torch.cat(outs).view(T, heads, dv)
    assert relative_error(got, want) < 2e-5 and relative_error(got[T - 1], want[T - 1]) < 2e-5


def test_rows_side_by_side_weighted_sums_vectors_and_gated_token_columns():
    from geneinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    a, b, x = torch.randn(9, 37, generator=g), torch.randn(9, 300, generator=g), torch.randn(9, 37, generator=g)
    for dtype in (torch.float32, torch.bfloat16):
        out = torch.empty(9, 337, device=DEV, dtype=dtype)
        ops.concat_rows(a.to(DEV), b.to(DEV), out)
        assert torch.equal(out.cpu(), torch.cat([a, b], 1).to(dtype))
        out = torch.empty(9, 37, device=DEV, dtype=dtype)
        ops.concat_rows(a.to(DEV), None, out)
        assert torch.equal(out.cpu(), a.to(dtype))
    y = x.to(DEV)
    ops.add_weighted(y, a.to(DEV), 1.2, (2 * a).to(DEV), -0.5)
    assert relative_error(y, x.double() + 1.2 * a.double() - 0.5 * 2 * a.double()) < 1e-6
    y = x.to(DEV)
    ops.add_weighted(y, a.to(DEV), 0.7)
    assert relative_error(y, x.double() + 0.7 * a.double()) < 1e-6
    for v in (torch.randn(37, generator=g), torch.randn(37, generator=g).to(torch.bfloat16)):
        y = x.to(DEV)
        ops.add_vector(y, v.to(DEV))
        assert relative_error(y, x.double() + v.double()) < 1e-6
    table, tokens = torch.randn(20, 50, generator=g), torch.tensor([3, 19, 0, 3, 7, 7, 1, 2, 11], dtype=torch.int32)
    u = 3 * torch.randn(9, 6, generator=g)
    for act, fn in (("gelu_tanh", P.gelu_tanh), ("silu", P.silu)):
        for first in (0, 12, 44):
            out = torch.empty(9, 6, device=DEV)
            ops.gate_token_columns(u.to(DEV), table.to(DEV), first, tokens.to(DEV), out, act)
            assert relative_error(out, fn(u.double()) * table.double()[tokens.long()][:, first:first + 6]) < 1e-6
    with pytest.raises(ops.KernelError):
        ops.gate_token_columns(u.to(DEV), table.to(DEV), 45, tokens.to(DEV), out)
    # a few rows: the product in front of the gate in the same kernel, the rows rounded as a bfloat16 product reads them
    for width in (37, 300, 1024):
        rows, w = torch.randn(9, width, generator=g), 0.1 * torch.randn(6, width, generator=g)
        for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 6e-3)):
            read = rows.to(dtype).double()
            want = P.gelu_tanh(read @ w.to(dtype).double().T) * table.to(dtype).double()[tokens.long()][:, 12:18]
            out = torch.empty(9, 6, device=DEV, dtype=dtype)
            ops.gate_token_columns_rows(rows.to(DEV), w.to(DEV, dtype), table.to(DEV, dtype), 12, tokens.to(DEV), out)
            assert relative_error(out, want) < tol


# =============================================================================================== whole models
def _portions(n, sizes=(7, 2, 5, 3, 2, 11, 1, 4, 2, 19)):
    out, i = [], 0
    while sum(out) + sizes[i % len(sizes)] <= n:
        out.append(sizes[i % len(sizes)])
        i += 1
    return out


CUTS = {"whole": lambda n: [n], "singly": lambda n: [], "most then singly": lambda n: [n - 9], "portions": _portions, "twos": lambda n: [2] * (n // 2)}


@pytest.mark.parametrize("name", list(CONFIGS))
def test_the_residual_stream_after_every_layer_run(folders, name):
    """Layer by layer, walks included: the first difference names the layer."""
    cfg, tokens = CONFIGS[name], _prompt(CONFIGS[name], 21, 3)
    want = []
    P.forward(cfg, stored_weights(folders[name]), tokens, streams=want)
    runner = make_runner(folders, name, "float32")
    runner.open("r")
    last = {}                                      # per run-order entry, the stream as the entry leaves it: behind the block, or behind what follows it
    runner.model.set_trace(lambda tag, i, rows: last.__setitem__(i, rows.float().cpu()) if tag in ("ffn_out", "layer_out") else None)
    try:
        feed(runner, "r", tokens, [len(tokens)])
    finally:
        runner.model.set_trace(None)
    got = [last[i] for i in sorted(last)]
    assert len(got) == len(want) == len(P.run_order(cfg))
    for i, (g, w) in enumerate(zip(got, want)):
        assert relative_error(g, w) < 2e-5, f"{name}: the stream differs behind layer run {i} (layer {P.run_order(cfg)[i][0]})"


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


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "float32"), ("C", "float32"), ("D", "float32"), ("E", "float32"), ("A", "bfloat16"), ("B", "bfloat16")])
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


@pytest.mark.parametrize("name, dtype", [("B", "bfloat16"), ("C", "float32"), ("B", "float32"), ("A", "float32")])
def test_long_portions_beside_single_rows(folders, name, dtype):
    """Steps that hold portions of a hundred rows and more of some requests (the kernels that take the rows of prompts tile by tile,
    the experts that take their rows together) beside single rows and short portions of others, every request at another position."""
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


def test_long_decoding_carries_state(folders):
    """A short prompt and 300 tokens decoded one by one through the captured decode step: the scans' states and the convolutions'
    tails carry, in every walk's own slot."""
    tokens = _prompt(CONFIGS["A"], 312, 9)
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folders, "A", dtype)
        runner.open("r")
        got = feed(runner, "r", tokens, [12])
        assert runner.steps_replayed > 250
        check_against_plain(folders, "A", dtype, tokens, got, f"A decoding ({dtype})")


def test_a_state_that_is_lost_or_a_walk_that_shares_one_shows(folders, tmp_path):
    """Weights made so that a fault shows: the scans hardly decay and outweigh the attention, so the last logits rest on what the
    first tokens left in every walk's state."""
    import copy
    cfg = copy.deepcopy(CONFIGS["D"])
    w = random_weights(cfg, 77)
    for i, layer in enumerate(cfg["layers"]):
        layer["mixer"]["left_scale"], layer["mixer"]["right_scale"] = 0.05, 2.0
        w[f"l{i}.mix.right.A_log"] = torch.full_like(w[f"l{i}.mix.right.A_log"], -7.0)
    write_model(tmp_path / "m", cfg, weights=w)
    from geneinfer_amd.engine import Runner, load_model
    tokens = _prompt(cfg, 150, 4)
    stored = stored_weights(tmp_path / "m")
    want = P.forward(cfg, stored, tokens)
    without = P.forward(cfg, stored, tokens[40:])                            # the premise: the first tokens matter at the end
    assert relative_error(without[-1], want[-1]) > 0.05
    runner = Runner(load_model(tmp_path / "m", "float32", DEV), page_size=4, max_tokens=512, max_requests=2)
    for what, cuts in (("whole", [150]), ("cut", [40, 2, 70]), ("singly", [3])):
        runner.open(what)
        got = feed(runner, what, tokens, cuts)
        runner.close(what)
        assert relative_error(got, want) < 5e-5, what


def test_layers_in_another_order_and_a_walk_elsewhere(folders, tmp_path):
    import copy
    cfg = copy.deepcopy(CONFIGS["A"])
    cfg["layers"] = [cfg["layers"][i] for i in (2, 0, 3, 1)]
    cfg["loop"] = dict(start=2, stop=4, times=3)
    write_model(tmp_path / "m", cfg, seed=4)
    from geneinfer_amd.engine import Runner, load_model
    tokens = _prompt(cfg, 40, 2)
    want = P.forward(cfg, stored_weights(tmp_path / "m"), tokens)
    runner = Runner(load_model(tmp_path / "m", "float32", DEV), page_size=8, max_tokens=256, max_requests=2)
    runner.open("r")
    got = feed(runner, "r", tokens, [13, 2])
    assert relative_error(got, want) < 5e-5


# =============================================================================================== entry points
@pytest.mark.parametrize("name", ["A", "E"])
def test_greedy_generation_through_the_entry_point_and_the_scheduler(folders, name):
    """Greedy tokens of several prompts, one by one through `LLM.generate` and together through the scheduler (more requests than
    it runs at once, prompts in portions), against the plain model's, as far as the plain model's two best logits are clearly apart."""
    import geneinfer_amd as gi
    from geneinfer_amd.engine import EngineConfig, EngineRequest
    from geneinfer_amd.sampling import SamplerConfig
    cfg, w = CONFIGS[name], stored_weights(folders[name])
    prompts = [_prompt(cfg, n, 30 + n) for n in (5, 23, 1, 40)]
    want, sure = [], []
    for p in prompts:
        tokens = P.greedy(cfg, w, p, 8)
        top2 = torch.topk(P.forward(cfg, w, p + tokens)[len(p) - 1:-1], 2, dim=-1).values
        clear = [bool(c) for c in (top2[:, 0] - top2[:, 1] > 1e-3)]
        want.append(tokens)
        sure.append(clear.index(False) if False in clear else len(clear))
    assert sum(sure) >= 24
    llm = gi.LLM(str(folders[name]), dtype="float32", page_size=PAGE_SIZE[name], max_tokens=512, max_running=2)
    assert type(llm.model.config).__name__ == "ZidevikConfig"
    for p, t, n in zip(prompts, want, sure):
        assert llm.generate(p, steps=len(p) + 7, temperature=0.0).generated_tokens[:n] == t[:n]
    eng = llm.engine(EngineConfig(max_running=2, step_rows=16, prefill_chunk=6))
    ids = [eng.submit(EngineRequest(p, len(p) + 7, SamplerConfig(0.0))) for p in prompts]
    eng.run_until_idle()
    for i, t, n in zip(ids, want, sure):
        assert eng.result(i).generated_tokens[:n] == t[:n]


@pytest.mark.parametrize("dtype, mode", [("float32", "mixed"), ("bfloat16", "mixed"), ("float32", "portions")])
def test_replay_through_the_command_line(folders, tmp_path, dtype, mode):
    """bin/trace_run as a child process on a Zidevik folder: up to four live requests, portions beside single tokens, a pool that
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
    steps = traces.mixed(requests, seed=3) if mode == "mixed" else traces.portions(requests)
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
            assert_within_bfloat16_noise(mine, lambda p: exact[p], lambda p: rounded[p], f"replay {mode} {rid}")


def test_generation_from_the_command_line_on_random_weights():
    """bin/gi_generate on the shipped example configuration, random weights, greedy: runs, and twice the same."""
    import subprocess
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    cmd = [str(root / "bin" / "gi_generate"), "--config", str(root / "configs" / "zidevik-small.json"), "--random-seed", "3", "--prompt-ids", "5 17 3 999 4",
           "--steps", "24", "--temperature", "0"]
    runs = [subprocess.run(cmd, capture_output=True, text=True, timeout=280) for _ in range(2)]
    assert all(r.returncode == 0 for r in runs), runs[0].stderr[-2000:]
    assert runs[0].stdout == runs[1].stdout and len(runs[0].stdout.split()) >= 20


def test_the_new_parts_serve_other_designs():
    """The parts are not Zidevik's own: a model put together by hand, a pre-norm layer whose mixer is a Llama attention beside a
    selective scan and whose feed-forward is a mixture with a softmax router, renormalised scores on the experts' outputs and no
    shared expert, then a parallel layer around a selective scan alone with a SiLU-gated token input behind it, entered through a
    product with the token rows without a vector; against a plain computation from the plain implementations' functions."""
    from geneinfer_amd.config import (AttentionSpec, LayerSpec, ModelSpec, RejoinSpec, RmsNormSpec, RotarySpec, RoutedExpertsSpec, RunEntry, SelectiveScanSpec,
                                      SideBySideSpec, SwiGluSpec, TokenSideInputSpec)
    from geneinfer_amd.engine import Runner
    from geneinfer_amd.engine.model import DecoderModel
    from geneinfer_amd.parts import model_tensor_needs
    from geneinfer_amd.weights import random_tensors
    from plain_llama import causal_attention, rms_norm, rope_inverse_frequencies, rope_rotate, swiglu
    d, vocab, eps, E = 64, 100, 1e-5, 4
    norm = lambda name: RmsNormSpec(d, eps, name)
    scan = lambda p, inner, n, r, taps: SelectiveScanSpec(d, inner, n, r, taps, p + "in", p + "c", p + "cb", p + "x", p + "dt", p + "db", p + "al", p + "D", p + "o")
    att = AttentionSpec(d, 4, 2, 16, "a.q", "a.k", "a.v", "a.o", RotarySpec(16, 10000.0))
    moe = RoutedExpertsSpec(d, 24, E, 2, "r", tuple(f"e{j}.g" for j in range(E)), tuple(f"e{j}.u" for j in range(E)), tuple(f"e{j}.d" for j in range(E)),
                            score="softmax", renormalize=True, weigh="output")
    side = TokenSideInputSpec(d, vocab, 5, "tab", 9, 3, "s.g", "s.p", norm("s.n"), activation="silu")
    spec = ModelSpec(architecture="by hand", vocab_size=vocab, hidden_size=d, max_positions=256, embedding="emb", final_norm=norm("fn"), lm_head="head", layers=(
        LayerSpec(mixer=SideBySideSpec(d, (att, scan("m.", 48, 6, 3, 3)), (0.8, -1.1)), feed_forward=moe, mixer_norm=norm("p1"), feed_forward_norm=norm("p2"), block="prenorm"),
        LayerSpec(mixer=scan("n.", 32, 4, 2, 2), feed_forward=SwiGluSpec(d, 80, "g.g", "g.u", "g.d"), mixer_norm=norm("n1"), feed_forward_norm=None, block="parallel", after=(side,))),
        run_order=(RunEntry(0), RunEntry(1, before=RejoinSpec(d, "join"))))
    host = random_tensors(model_tensor_needs(spec), seed=5, dtype="float32", std=0.2)
    model = DecoderModel(spec, {k: v.to(DEV) for k, v in host.items()}, torch.float32, DEV)
    runner = Runner(model, page_size=4, max_tokens=256, max_requests=2)
    tokens = _prompt(dict(vocab=vocab), 45, 2)
    got = {}
    for what, cuts in (("whole", [45]), ("cut", [3, 20, 2])):
        runner.open(what)
        got[what] = feed(runner, what, tokens, cuts)
        runner.close(what)
    assert torch.equal(got["whole"], got["cut"])

    w = {k: v.double() for k, v in host.items()}
    T, pos = len(tokens), torch.arange(len(tokens))
    x0 = w["emb"][torch.tensor(tokens)]
    h = rms_norm(x0, w["p1"], eps)
    f = rope_inverse_frequencies(16, 10000.0)
    q, k = rope_rotate((h @ w["a.q"].T).view(T, 4, 16), pos, f), rope_rotate((h @ w["a.k"].T).view(T, 2, 16), pos, f)
    left = causal_attention(q, k, (h @ w["a.v"].T).view(T, 2, 16)).reshape(T, 64) @ w["a.o"].T
    run_scan = lambda rows, p, n, r: P.selective_scan(rows, w[p + "in"], w[p + "c"], w[p + "cb"], w[p + "x"], w[p + "dt"], w[p + "db"], w[p + "al"], w[p + "D"], w[p + "o"],
                                                      state=n, dt_rank=r)
    x = x0 + 0.8 * left - 1.1 * run_scan(h, "m.", 6, 3)
    h = rms_norm(x, w["p2"], eps)
    s = torch.softmax(h @ w["r"].T, -1)
    best = torch.topk(s, 2, dim=-1)
    share = best.values / best.values.sum(-1, keepdim=True)
    x = x + torch.stack([sum(share[t, j] * swiglu(h[t][None], w[f"e{e}.g"], w[f"e{e}.u"], w[f"e{e}.d"])[0] for j, e in enumerate(best.indices[t].tolist())) for t in range(T)])
    x = torch.cat([x, x0], -1) @ w["join"].T
    h = rms_norm(x, w["n1"], eps)
    x = x + run_scan(h, "n.", 4, 2) + swiglu(h, w["g.g"], w["g.u"], w["g.d"])
    g = P.silu(x @ w["s.g"].T) * w["tab"][torch.tensor(tokens)][:, 3:8]
    x = x + rms_norm(g @ w["s.p"].T, w["s.n"], eps)
    want = rms_norm(x, w["fn"], eps) @ w["head"].T
    assert relative_error(got["whole"], want) < 5e-5
