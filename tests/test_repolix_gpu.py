"""Repolix on the GPU against the plain implementation (tests/plain_repolix.py): each mechanism's kernels alone, with
inputs made so that a lost state, a far token, a window that is one token off or a wrong expert shows; then whole
models of four small configurations in 32-bit and in bfloat16: whole prompts, portions, token by token, unequal
batches, slots and pages used again, long decoding, the first tokens, and greedy generation through the pipeline."""
import math

import pytest
import torch

import plain_repolix as P
from repolix_cases import CONFIGS, cases, model_folder, plain_logits, plain_model, tokens_for
from helpers import assert_logits_close

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
DEV = "cuda:0"
F64 = torch.float64


@pytest.fixture(scope="module", autouse=True)
def need_gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")


def engine(name, dtype, max_tokens=1024, max_slots=None):
    from synaptix_amd import Engine
    return Engine.load(model_folder(name), dtype=dtype, max_tokens=max_tokens, max_slots=max_slots)


def dev(t, dtype=torch.float32):
    return t.to(device=DEV, dtype=dtype).contiguous()


def ints(xs):
    return torch.tensor(list(xs), dtype=torch.int32, device=DEV)


def randn(g, *shape):
    return torch.randn(*shape, generator=g, dtype=F64)


class Step:
    """The device arrays of a step over sequences (slot, tokens cached before, new tokens)."""

    def __init__(self, seqs):
        self.slots, self.past, self.new = zip(*seqs)
        starts = [0]
        for n in self.new:
            starts.append(starts[-1] + n)
        self.starts = starts
        self.seq_start, self.seq_past, self.seq_slot = ints(starts), ints(self.past), ints(self.slots)
        self.tok_seq = ints(b for b, n in enumerate(self.new) for _ in range(n))
        self.tok_pos = ints(p + i for p, n in zip(self.past, self.new) for i in range(n))
        self.N = starts[-1]


# ----------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("taps,bias,silu", [(1, False, False), (2, True, True), (4, False, True), (5, True, False), (16, False, False)])
def test_short_convolution_carries_its_last_inputs(taps, bias, silu):
    """Three sequences in portions of unequal sizes (down to one token, shorter and longer than the filter) in state rows
    of their own; a row is then taken by a new sequence after it was zeroed; a negative slot writes the last row."""
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(taps)
    C, width, rows = 70, 90, 5
    w, b = randn(g, C, taps), randn(g, C) if bias else None
    seqs = {0: randn(g, 40, width), 3: randn(g, 23, width), 1: randn(g, 9, width)}
    want = {s: P.short_conv(u[:, 11:11 + C], w, b) for s, u in seqs.items()}
    if silu:
        want = {s: P.silu(y) for s, y in want.items()}
    state = torch.zeros((rows, taps - 1, C), dtype=torch.float32, device=DEV)
    state[4] = 7.0
    fed = {s: 0 for s in seqs}
    got = {s: [] for s in seqs}
    plan = [{0: 1, 3: 5, 1: 2}, {0: 2, 3: 1}, {0: 17, 1: 1, 3: 16}, {1: 6, 0: 1}, {0: 1, 3: 1}, {0: 18}]      # (one step of single tokens only)
    for portion in plan:
        st = Step([(s, fed[s], n) for s, n in portion.items()])
        u = dev(torch.cat([seqs[s][fed[s]:fed[s] + n] for s, n in portion.items()]))
        out = torch.empty((st.N, C), dtype=torch.float32, device=DEV)
        ops.short_conv(u[:, 11:11 + C], dev(w), None if b is None else dev(b), state, st.tok_seq, st.tok_pos, st.seq_start,
                       st.seq_past, st.seq_slot, out, silu=silu)
        for i, (s, n) in enumerate(portion.items()):
            got[s].append(out[st.starts[i]:st.starts[i + 1]].cpu().double())
            fed[s] += n
    for s in seqs:
        assert fed[s] == len(seqs[s])
        assert float((torch.cat(got[s]) - want[s]).abs().max()) < 1e-4, f"sequence in row {s}"
    if taps > 1:
        assert float((state[4] - 7.0).abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0     # rows of nobody
    # a row used again: zeroed (as the cache does when a slot is taken), then a new sequence; and the spare row
    state[0].zero_()
    u2 = randn(g, 6, width)
    st = Step([(0, 0, 6), (-1, 0, 1)])
    out = torch.empty((7, C), dtype=torch.float32, device=DEV)
    ops.short_conv(dev(torch.cat([u2, u2[:1]]))[:, 11:11 + C], dev(w), None if b is None else dev(b), state, st.tok_seq,
                   st.tok_pos, st.seq_start, st.seq_past, st.seq_slot, out, silu=silu)
    y = P.short_conv(u2[:, 11:11 + C], w, b)
    assert float((out[:6].cpu().double() - (P.silu(y) if silu else y)).abs().max()) < 1e-4
    if taps > 1:
        assert float((state[4, -1].cpu().double() - u2[0, 11:11 + C]).abs().max()) < 1e-6


@pytest.mark.parametrize("H,Pv,G,N", [(4, 16, 2, 24), (3, 10, 1, 7), (2, 70, 2, 130), (6, 64, 3, 64), (1, 5, 1, 256)])
def test_state_space_scan_keeps_far_tokens(H, Pv, G, N):
    """Decays close to one, so that a token hundreds back still carries a tenth of its weight: two sequences in portions
    (17 tokens, one token, the rest) from states in given rows, against the plain cell over the whole sequences."""
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(H * 100 + N)
    T = [150, 40]
    a_log, bias, d = randn(g, H) * 0.3 - 3.5, randn(g, H) * 0.2 - 1.0, randn(g, H)
    data, want = [], []
    for t in T:
        x, B, C, dt = randn(g, t, H, Pv), randn(g, t, G, N) * N ** -0.5, randn(g, t, G, N), randn(g, t, H) * 0.5
        data.append((x, B, C, dt))
        want.append(P.state_space_cell(x, B, C, dt, bias, a_log, d))
    # the first token still counts at the end
    x, B, C, dt = [t.clone() for t in data[0]]
    x[0] += 30.0
    moved = P.state_space_cell(x, B, C, dt, bias, a_log, d)
    assert float((moved[-1] - want[0][-1]).abs().max()) > 1e-2
    state = torch.zeros((4, H, N, Pv), dtype=torch.float32, device=DEV)
    got, fed = [[], []], [0, 0]
    for portion in ([17, 1], [1, 1], [132, 38]):
        st = Step([(3, fed[0], portion[0]), (1, fed[1], portion[1])])
        xbc = torch.cat([torch.cat([data[i][0][fed[i]:fed[i] + n].reshape(n, -1), data[i][1][fed[i]:fed[i] + n].reshape(n, -1),
                                    data[i][2][fed[i]:fed[i] + n].reshape(n, -1)], 1) for i, n in enumerate(portion)])
        dts = torch.cat([data[i][3][fed[i]:fed[i] + n] for i, n in enumerate(portion)])
        wide = torch.zeros((st.N, H + 9), dtype=torch.float32, device=DEV)
        wide[:, 9:] = dev(dts)
        out = torch.empty((st.N, H * Pv), dtype=torch.float32, device=DEV)
        ops.state_space_scan(dev(xbc), wide[:, 9:], dev(bias), dev(a_log), dev(d), state, st.seq_start, st.seq_slot, out,
                             H, Pv, N, G, single_tokens=all(n == 1 for n in portion))
        for i, n in enumerate(portion):
            got[i].append(out[st.starts[i]:st.starts[i + 1]].cpu().double().view(n, H, Pv))
            fed[i] += n
    for i in range(2):
        scale = max(1.0, float(want[i].abs().max()))
        assert float((torch.cat(got[i]) - want[i]).abs().max()) < 2e-4 * scale, f"sequence {i}"
    assert float(state[0].abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0


@pytest.mark.parametrize("H,K,D,E", [(4, 2, 16, 24), (3, 1, 12, 20), (2, 2, 130, 70), (4, 4, 64, 64), (1, 1, 256, 5)])
def test_channel_delta_scan(H, K, D, E):
    """Slow decays (far tokens count), steps near one (the rule overwrites what a key held): two sequences in portions
    from states in given rows, against the plain cell; the decays arrive as a piece of longer rows."""
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(H * 100 + D)
    T = [120, 35]
    a_log, a_bias = randn(g, H) * 0.3 - 3.0, randn(g, H, D) * 0.3 - 1.0
    data, want = [], []
    for t in T:
        q, k, v = randn(g, t, K, D), randn(g, t, K, D), randn(g, t, H, E)
        beta, a = randn(g, t, H) * 2.0 + 1.0, randn(g, t, H, D) * 0.5
        data.append((q, k, v, beta, a))
        want.append(P.delta_cell(q, k, v, beta, a, a_bias, a_log))
    q, k, v, beta, a = [t.clone() for t in data[0]]
    v[0] += 30.0
    assert float((P.delta_cell(q, k, v, beta, a, a_bias, a_log)[-1] - want[0][-1]).abs().max()) > 1e-3
    state = torch.zeros((3, H, D, E), dtype=torch.float32, device=DEV)
    got, fed = [[], []], [0, 0]
    for portion in ([16, 2], [1, 1], [2, 17], [101, 15]):
        st = Step([(0, fed[0], portion[0]), (-1, fed[1], portion[1])])        # the second sequence lives in the last row
        cut = lambda j: [data[i][j][fed[i]:fed[i] + n].reshape(n, -1) for i, n in enumerate(portion)]
        qkv = torch.cat([torch.cat([a_, b_, c_], 1) for a_, b_, c_ in zip(cut(0), cut(1), cut(2))])
        wide = torch.zeros((st.N, 3 + H + H * D + 5), dtype=torch.float32, device=DEV)
        wide[:, 3:3 + H] = dev(torch.cat(cut(3)))
        wide[:, 3 + H:3 + H + H * D] = dev(torch.cat(cut(4)))
        out = torch.empty((st.N, H * E), dtype=torch.float32, device=DEV)
        ops.channel_delta_scan(dev(qkv), wide[:, 3:3 + H], wide[:, 3 + H:3 + H + H * D], dev(a_bias.reshape(-1)), dev(a_log),
                               D ** -0.5, 1e-6, state, st.seq_start, st.seq_slot, out, H, K, D, E,
                               single_tokens=all(n == 1 for n in portion))
        for i, n in enumerate(portion):
            got[i].append(out[st.starts[i]:st.starts[i + 1]].cpu().double().view(n, H, E))
            fed[i] += n
    for i in range(2):
        scale = max(1.0, float(want[i].abs().max()))
        assert float((torch.cat(got[i]) - want[i]).abs().max()) < 2e-4 * scale, f"sequence {i}"
    assert float(state[1].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_before_the_norm_and_the_difference_of_two_maps(dtype):
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    N, parts, n = 9, 3, 50
    y, z, gain = randn(g, N, parts * n), randn(g, N, parts * n + 4), randn(g, parts * n)
    want = P.rms_norm((y * P.silu(z[:, 4:])).view(N, parts, n), None, 1e-5).reshape(N, -1) * gain
    out = torch.empty((N, parts * n), dtype=dtype, device=DEV)
    ops.head_norm_gate(dev(y), dev(gain), 1e-5, dev(z)[:, 4:], out, parts, n, silu_first=True)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert float((out.cpu().double() - want).abs().max()) < tol * max(1.0, float(want.abs().max()))
    G, R, E, lam, post = 2, 3, 40, 0.37, 0.6
    a = randn(g, N, G, 2, R, E).to(dtype).double()
    d = a[:, :, 0] - lam * a[:, :, 1]
    want = (P.rms_norm(d, None, 1e-5) * post).reshape(N, -1)
    out = torch.empty((N, G * R * E), dtype=dtype, device=DEV)
    ops.diff_heads(dev(a.reshape(N, -1), dtype), out, lam, 1e-5, post, G, R, E)
    assert float((out.cpu().double() - want).abs().max()) < tol * max(1.0, float(want.abs().max()))


def paged(rows_by_head, dtype, n_pages, order):
    """rows_by_head [T, heads, n] into pages [n_pages, heads, 64, n] at the pages `order` names."""
    T, Hh, n = rows_by_head.shape
    pages = torch.zeros((n_pages, Hh, 64, n), dtype=torch.float64)
    for t in range(T):
        pages[order[t // 64], :, t % 64] = rows_by_head[t]
    return pages.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 1, 2, 37, 63, 64, 65, 130])
def test_two_maps_see_exactly_their_keys_and_share_their_values(window, dtype):
    """Keys are one-hot in their position (modulo the key size) and queries are long, so that a query gives nearly all
    its weight to the visible keys of one residue: a window that is one token off, a key taken from the other map or
    values taken from the wrong value head change the result by its own size.  All queries at once (prompts: in bf16
    the tiles on the matrix cores) and the last ones as single tokens, over pages in a shuffled order."""
    from synaptix_amd.kernels import ops
    H, G, D, E, T = 4, 2, 16, 32, 200
    R = H // G
    g = torch.Generator().manual_seed(window)
    pos = torch.arange(T)
    k = torch.zeros(T, G, 2, D, dtype=F64)
    for t in range(T):
        for gg in range(G):
            k[t, gg, 0, (t + gg) % D] = 1.0
            k[t, gg, 1, (3 * t + gg) % D] = 1.0
    q = torch.zeros(T, H, 2, D, dtype=F64)
    for t in range(T):
        for h in range(H):
            q[t, h, 0, (t - 5 - h) % D] = 9.0           # map 1 looks 5 + h back (and at what shares that residue)
            q[t, h, 1, (3 * (t - 2)) % D] = 9.0
    q = q + 0.1 * randn(g, T, H, 2, D)
    v = randn(g, T, G, E)
    q, k, v = [x.to(dtype).double() for x in (q, k, v)]
    lam, eps, post = 0.45, 1e-6, 0.8
    want = P.two_maps(q, k, v, 1.0, window or None, lam, eps, post).reshape(T, H * E)
    order = [3, 0, 2, 1]
    kp = paged(k.reshape(T, 2 * G, D), dtype, 5, order).to(DEV)
    vp = paged(v, dtype, 5, order).transpose(2, 3).contiguous().to(DEV)
    q_rows = q.view(T, G, R, 2, D).permute(0, 1, 3, 2, 4).reshape(T, 2 * H * D)         # (kv head, map, head of the group)
    qd = dev(q_rows, dtype)
    table = ints(order).view(1, 4)
    tol = 2e-4 if dtype == torch.float32 else 6e-2

    def joined(maps):
        out = torch.empty((maps.shape[0], H * E), dtype=dtype, device=DEV)
        ops.diff_heads(maps, out, lam, eps, post, G, R, E)
        return out.cpu().double()

    st = Step([(0, 0, T)])
    maps = torch.empty((T, 2 * H * E), dtype=dtype, device=DEV)
    ops.window_attention(qd, kp, vp, table, st.tok_seq, st.tok_pos, maps, 1.0, 2 * H, 2 * G, D, E, window=window, v_share=2)
    assert float((joined(maps) - want).abs().max()) < tol, "every query, one wave a (token, head)"
    if dtype == torch.bfloat16:
        maps = torch.empty((T, 2 * H * E), dtype=dtype, device=DEV)
        ops.window_attention_prefill_bf16(qd, kp, vp, table, st.seq_start, st.seq_past, maps, 1.0, 2 * H, 2 * G, D, E,
                                          window=window, v_share=2)
        assert float((joined(maps) - want).abs().max()) < tol, "every query, tiles on the matrix cores"
    for t in (T - 1, 129, 128, 64, 63, 1, 0):
        st = Step([(0, t, 1)])
        maps = torch.empty((1, 2 * H * E), dtype=dtype, device=DEV)
        ops.window_attention(qd[t:t + 1], kp, vp, table, st.tok_seq, st.tok_pos, maps, 1.0, 2 * H, 2 * G, D, E, window=window,
                             v_share=2)
        assert float((joined(maps) - want[t:t + 1]).abs().max()) < tol, f"the single query at {t}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nk,D,E,rot", [(4, 2, 16, 24, 8), (6, 6, 12, 10, 12), (2, 2, 20, 6, 0), (8, 4, 32, 64, 32)])
def test_intake_turns_and_writes_pages_with_shared_value_heads(nq, nk, D, E, rot, dtype):
    from synaptix_amd.kernels import ops
    from synaptix_amd.parts import RotaryScaledHalfSplit
    g = torch.Generator().manual_seed(D)
    nv = nk // 2
    st = Step([(0, 60, 10), (1, 0, 3)])
    rows = randn(g, st.N, (nq + nk) * D + nv * E + 3)
    rotd = {"base": 300.0, "dims": rot, "scaling": {"factor": 3.0, "original": 50, "fast": 8.0, "slow": 1.0}}
    position = RotaryScaledHalfSplit(300.0, rot, 128, factor=3.0, original=50, fast=8.0, slow=1.0)
    pos = torch.tensor([60 + i for i in range(10)] + [0, 1, 2])
    qk = rows[:, :(nq + nk) * D].view(st.N, nq + nk, D)
    turned = P.turn_halves(qk, pos, rotd)
    q = torch.empty((st.N, nq * D), dtype=dtype, device=DEV)
    kp = torch.zeros((4, nk, 64, D), dtype=dtype, device=DEV)
    vp = torch.zeros((4, nv, E, 64), dtype=dtype, device=DEV)
    table = ints([2, 0, 1, 3]).view(2, 2)
    ops.window_intake(dev(rows), None, q, kp, vp, table, st.tok_seq, st.tok_pos, None, None, 0.0, nq, nk, D, E,
                      rotation=position.tables(DEV), v_share=2)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    big = max(1.0, float(rows.abs().max()) * 1.2)
    assert float((q.cpu().double().view(st.N, nq, D) - turned[:, :nq]).abs().max()) < tol * big
    vals = rows[:, (nq + nk) * D:(nq + nk) * D + nv * E].view(st.N, nv, E)
    for n, (page, slot) in enumerate([(2, 60), (2, 61), (2, 62), (2, 63)] + [(0, i) for i in range(6)] + [(1, 0), (1, 1), (1, 2)]):
        assert float((kp[page, :, slot].cpu().double() - turned[n, nq:]).abs().max()) < tol * big, f"key of token {n}"
        assert float((vp[page, :, :, slot].cpu().double() - vals[n]).abs().max()) < tol * big, f"value of token {n}"


@pytest.mark.parametrize("N,E,top,groups,keep", [(50, 8, 3, 4, 2), (3, 5, 5, 1, 1), (200, 16, 4, 4, 2), (7, 15, 4, 3, 1),
                                                 (1, 6, 1, 3, 1), (40, 12, 2, 6, 6)])
def test_router_that_scores_all_experts(N, E, top, groups, keep):
    """On equal inputs the choice is exact: the same experts in the same order, weights that are the scores themselves;
    corrections large enough to move the choice and negative enough that a choice score is below zero."""
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(N + E)
    logits = (2.0 * randn(g, N, E)).float()
    corr = (0.3 * randn(g, E) - 0.2).float()
    w = {"r.router": torch.eye(E, dtype=F64), "r.correction": corr.double()}
    chosen, weights = P.route(logits.double(), w, "r.", {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}})
    ids = torch.empty((N, top), dtype=torch.int32, device=DEV)
    ws = torch.empty((N, top), dtype=torch.float32, device=DEV)
    ops.route_scores(dev(logits), dev(corr), ids, ws, groups, keep)
    assert (ids.cpu().long() == chosen).all()
    assert float((ws.cpu().double() - weights).abs().max()) < 1e-6
    ops.route_scores(dev(logits), dev(corr), ids, ws, groups, keep, renorm=True)
    assert float((ws.cpu().double() - weights / weights.sum(-1, keepdim=True)).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("N,W,F,E,I,top,limit", [(50, 64, 32, 6, 2, 3, 1.4), (3, 40, 24, 5, 0, 5, 0.5), (1, 32, 96, 0, 4, 2, 1.0),
                                                 (200, 96, 64, 16, 1, 4, 7.0), (9, 128, 16, 2, 3, 1, 1.0)])
def test_gated_experts_identity_experts_and_the_shared_expert(N, W, F, E, I, top, limit, dtype):
    """The feed-forward part alone over given rows: some router outputs are the identity (one configuration has no
    other), inputs large enough that both bounds cut, a shared expert with a bound of its own."""
    from synaptix_amd.parts import RoutedExperts, GatedMlp
    g = torch.Generator().manual_seed(N + W)
    w = {"m.router": 2.0 * randn(g, E + I, W) / W ** 0.5, "m.correction": 0.02 * randn(g, E + I)}
    for e in range(E):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"], w[f"m.e{e}.down"] = randn(g, F, W) * 0.3, randn(g, F, W) * 0.3, randn(g, W, F) * 0.2
    w["m.shared.gate"], w["m.shared.up"], w["m.shared.down"] = randn(g, 48, W) * 0.3, randn(g, 48, W) * 0.3, randn(g, W, 48) * 0.2
    w = {n: t.to(dtype).double() for n, t in w.items()}
    h = randn(g, N, W).to(dtype).double()
    c = {"expert": {"ff": F, "limit": limit}, "router": {"experts": E, "identity": I, "top": top}, "shared": {"ff": 48, "limit": 0.8}}
    want = P.routed_experts(h, w, "m.", c)
    shared = GatedMlp("m.shared.", W, 48, ("swiglu_limit", 0.8), names=("gate", "up", "down"))
    part = RoutedExperts("m.", W, F, E, top, ("swiglu_limit", limit), gated=True, router="scores", identity=I, shared=shared)
    part.load(lambda n: dev(w[n], dtype))
    from synaptix_amd.parts import as_delta
    got = as_delta(part.forward(dev(h, dtype), None))
    got = got.sum(0) if got.dim() == 3 else got
    err = float((got.cpu().double() - want).abs().max())
    scale = max(1.0, float(want.abs().max()))
    if dtype == torch.float32:
        assert err < 2e-4 * scale
    else:
        # (a near tie of two choice scores may fall the other way on rounded sums: few rows may differ by an expert)
        bad = ((got.cpu().double() - want).abs().max(-1).values > 0.05 * scale).sum()
        assert int(bad) <= max(1, N // 20), f"{int(bad)} of {N} rows differ"


@pytest.mark.parametrize("force", [0, 1, 2, 3])
@pytest.mark.parametrize("N", [9, 300])
def test_gated_pairs_as_the_epilogue_of_the_experts_product(N, force):
    """Gate and up rows in turns, the bounded activation of each pair of sums stored: in the tiles through LDS (many
    rows an expert), with operands straight from memory (16 and 64 outputs a wave) and in plain FMA; an expert that
    nobody chose; a weight for every row."""
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(N + force)
    E, F, W, top, limit = 5, 48, 64, 2, 0.9
    gate, up = (randn(g, E, F, W) * 0.4).bfloat16(), (randn(g, E, F, W) * 0.4).bfloat16()
    x = randn(g, N, W).bfloat16()
    ids = torch.stack([torch.randperm(E - 1, generator=g)[:top] for _ in range(N)]).int()        # expert 4 stays idle
    weights = torch.rand(N, top, generator=g).float()
    seg, tok_of, pair_of, part_of, weight_of = ops.route_sort(dev(ids, torch.int32), dev(weights), E)
    w = ops.pair_expert_rows(dev(gate, torch.bfloat16), dev(up, torch.bfloat16))
    if force != 1:
        w = ops.pack_expert_weights(w)
    out = torch.zeros((N * top, F), dtype=torch.float32, device=DEV)
    ops.experts_product(dev(x, torch.bfloat16), w, out, seg, tok_of, pair_of, row_weight=weight_of, gated=("swiglu_limit", limit),
                        force_simt=force)
    for n in range(N):
        for t in range(top):
            e = int(ids[n, t])
            gs = torch.clamp(x[n].double() @ gate[e].double().T, max=limit)
            us = torch.clamp(x[n].double() @ up[e].double().T, -limit, limit)
            want = gs * torch.sigmoid(1.702 * gs) * (us + 1.0) * float(weights[n, t])
            assert float((out[n * top + t].cpu().double() - want).abs().max()) < 1e-3, f"token {n} choice {t}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bounded_activation_inside_the_products(dtype):
    """The gated products that apply the activation themselves (few rows over weights in fragment order, many rows in
    tiles) and the activation as a kernel of its own give the plain formula."""
    from synaptix_amd.parts import GatedMlp
    g = torch.Generator().manual_seed(11)
    W, F = 128, 64
    w = {"f.gate": randn(g, F, W) * 0.4, "f.up": randn(g, F, W) * 0.4, "f.down": randn(g, W, F) * 0.2}
    w = {n: t.to(dtype).double() for n, t in w.items()}
    part = GatedMlp("f.", W, F, ("swiglu_limit", 1.2), names=("gate", "up", "down"))
    part.load(lambda n: dev(w[n], dtype))
    from synaptix_amd.parts import as_delta
    for N in (1, 6, 12, 40, 300):
        h = randn(g, N, W).to(dtype).double()
        want = P.clamped_expert(h, w["f.gate"], w["f.up"], w["f.down"], 1.2)
        got = as_delta(part.forward(dev(h, dtype), None))
        got = got.sum(0) if got.dim() == 3 else got
        tol = 2e-4 if dtype == torch.float32 else 3e-2
        assert float((got.cpu().double() - want).abs().max()) < tol * max(1.0, float(want.abs().max())), f"{N} rows"


# ----------------------------------------------------------------------------- whole models

def lengths(name):
    return {"P": [1, 2, 21, 64, 65, 150], "Q": [3, 70, 71, 129, 140], "R": [5, 64, 128, 200], "S": [1, 2, 3, 66, 90]}[name]


@pytest.mark.parametrize("name,dtype", cases(["P", "Q", "R", "S"]))
def test_whole_prompts(name, dtype):
    eng = engine(name, dtype)
    for i, n in enumerate(lengths(name)):
        toks = tokens_for(name, n, 100 + i)
        s = eng.acquire()
        got = eng.step([(s, toks)], want="all")
        assert_logits_close(got, plain_logits(name, toks), dtype, f"{name} {dtype} {n} tokens whole", sharp=True)
        eng.release(s)
    eng.cache.check()


@pytest.mark.parametrize("name", ["P", "Q"])
def test_the_residual_after_every_layer_in_float32(name):
    """The model's layers one after another: the residual rows that each leaves, read from the engine's own pass."""
    from synaptix_amd.parts import as_delta
    toks = tokens_for(name, 70, 3)
    want, _ = plain_model(name).residuals(toks)
    eng = engine(name, "float32")
    got = []
    for block in eng.model.blocks:
        inner = block.forward

        def spy(resid, pending, ctx, cache, owner=True, inner=inner):
            out = inner(resid, pending, ctx, cache, owner)
            got.append(resid.clone() + as_delta(out))
            return out
        block.forward = spy
    eng.step([(eng.acquire(), toks)], want="last")
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert float((a.cpu().double() - b).abs().max()) < 1e-4 * max(1.0, float(b.abs().max())), f"after layer {i}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_portions_of_several_sizes(name, dtype):
    """A prompt in portions of 2, 1, 3, 17, 64 and 2 tokens and the rest: every portion starts from the states and
    pages that the earlier ones left (inside a page, at a page's border, shorter than a filter, inside and beyond the
    first window)."""
    toks = tokens_for(name, 230, 7)
    want = plain_logits(name, toks)
    eng = engine(name, dtype)
    s, at, got = eng.acquire(), 0, []
    for n in [2, 1, 3, 17, 64, 2, 41, 100]:
        got.append(eng.step([(s, toks[at:at + n])], want="all"))
        at += n
    assert at == len(toks)
    assert_logits_close(torch.cat(got), want, dtype, f"{name} {dtype} in portions", sharp=True)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,head,n", [("P", 30, 130), ("Q", 1, 160), ("R", 100, 140), ("S", 3, 90)])
def test_prompt_then_token_by_token(name, head, n, dtype):
    """Decoding long enough that every window passes over decoded tokens and over a page's border."""
    if dtype not in [d for _, d in cases([name])]:
        pytest.skip("this configuration runs in 32-bit only")
    toks = tokens_for(name, n, 21)
    want = plain_logits(name, toks)
    eng = engine(name, dtype)
    s = eng.acquire()
    got = [eng.step([(s, toks[:head])], want="all")]
    for t in toks[head:]:
        got.append(eng.step([(s, [t])], want="last"))
    assert_logits_close(torch.cat(got), want, dtype, f"{name} {dtype} token by token", sharp=True)
    eng.release(s)
    eng.cache.check()


@pytest.mark.parametrize("name,dtype", cases(["P", "Q", "R", "S"]))
def test_unequal_batches_and_slots_used_again(name, dtype):
    """Requests of unequal lengths start together and are decoded together, the shorter ones ending earlier; then
    other requests take the slots, state rows and pages that came free (the cache has room for little more than one
    batch), in another order: each request's logits equal the plain model's for that request alone."""
    reqs = {f"r{i}": tokens_for(name, n + 9, 300 + i) for i, n in enumerate(lengths(name))}
    ids = list(reqs)
    eng = engine(name, dtype, max_tokens=64 * 9, max_slots=3)
    for batch in (ids[:3], (ids[3:] + ids[:1])[:3], list(reversed(ids))[:3]):
        slots = {r: eng.acquire() for r in batch}
        head = {r: max(1, len(reqs[r]) - 9 - 3 * i) for i, r in enumerate(batch)}
        got = {r: [] for r in batch}
        out = eng.step([(slots[r], reqs[r][:head[r]]) for r in batch], want="all")
        at = 0
        for r in batch:
            got[r].append(out[at:at + head[r]])
            at += head[r]
        fed, live = dict(head), list(batch)
        while live:
            out = eng.step([(slots[r], [reqs[r][fed[r]]]) for r in live], want="last")
            for i, r in enumerate(live):
                got[r].append(out[i:i + 1])
                fed[r] += 1
            for r in [r for r in live if fed[r] == len(reqs[r])]:
                eng.release(slots[r])
                live.remove(r)
        for r in batch:
            assert_logits_close(torch.cat(got[r]), plain_logits(name, reqs[r]), dtype, f"{name} {dtype} {r} in a batch",
                                sharp=True)
        eng.cache.check()
    assert eng.cache.free_slots == 3


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens(dtype):
    """Sequences of one and two tokens, and every position up to the window and a little more, one by one."""
    for name in ("P", "S"):
        if name == "S" and dtype != "float32":
            continue
        eng = engine(name, dtype)
        toks = tokens_for(name, 30, 77)
        want = plain_logits(name, toks)
        for n in (1, 2):
            s = eng.acquire()
            assert_logits_close(eng.step([(s, toks[:n])], want="all"), plain_logits(name, toks[:n]), dtype,
                                f"{name} {dtype} first {n}", sharp=True)
            eng.release(s)
        s = eng.acquire()
        got = [eng.step([(s, [t])], want="last") for t in toks]
        assert_logits_close(torch.cat(got), want, dtype, f"{name} {dtype} from the first token one by one", sharp=True)


def test_long_decoding_in_float32():
    """500 tokens one by one through the layers that carry a state and the one that keeps a window of keys."""
    toks = tokens_for("P", 500, 5)
    want = plain_logits("P", toks)
    eng = engine("P", "float32", max_tokens=64 * 10)
    s = eng.acquire()
    got = [eng.step([(s, toks[:2])], want="all")]
    for t in toks[2:]:
        got.append(eng.step([(s, [t])], want="last"))
    assert_logits_close(torch.cat(got), want, "float32", "500 tokens one by one", sharp=True)


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_pipeline(dtype):
    """Pipeline.generate_batch (the scheduler, slots, captured decode steps, the sampler) against greedy decoding with
    the plain model; in bfloat16 a token may differ where the two best logits are close, then the plain model's logits
    for the generated sequence must say so."""
    import synaptix_amd
    name = "R"
    pipe = synaptix_amd.load(model_folder(name), dtype="f32" if dtype == "float32" else "bf16", max_seq=512)
    prompts = [tokens_for(name, n, 900 + n) for n in (3, 70, 20)]
    outs, stats = pipe.generate_batch(prompts, synaptix_amd.GenerationConfig(max_new_tokens=12, temperature=0.0))
    assert stats.new_tokens == 36
    for prompt, out in zip(prompts, outs):
        assert len(out.tokens) == 12 and out.finish_reason == "length"
        logits = plain_logits(name, prompt + out.tokens)
        for i, tok in enumerate(out.tokens):
            row = logits[len(prompt) - 1 + i]
            best = int(row.argmax())
            if dtype == "float32":
                assert tok == best or float(row[best] - row[tok]) < 1e-4
            else:
                assert tok == best or float(row[best] - row[tok]) < 0.05 * float(row.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "R"])
def test_decode_steps_replayed_from_a_graph(name, dtype):
    """Captured decode steps (three rows wide in a graph of four: one row is padding, its states live in the spare row)
    with eager work of another sequence between the replays; every replay against the plain model."""
    eng = engine(name, dtype, max_tokens=64 * 12)
    assert eng.graph_ok
    reqs = [tokens_for(name, n, 40 + n) for n in (90, 20, 140)]
    other = tokens_for(name, 60, 4)
    want = [plain_logits(name, r) for r in reqs]
    heads = [len(r) - 12 for r in reqs]
    slots = [eng.acquire() for _ in reqs]
    eng.step([(s, r[:h]) for s, r, h in zip(slots, reqs, heads)], want=None)
    runner = eng.decode_runner(3, 256)
    assert runner.rows == 4
    extra = eng.acquire()
    for i in range(12):
        _, lg = runner.step(slots, [r[h + i] for r, h in zip(reqs, heads)])
        for j in range(3):
            assert_logits_close(lg[j:j + 1].clone(), want[j][heads[j] + i:heads[j] + i + 1], dtype,
                                f"{name} {dtype} replay {i} row {j}", sharp=True)
        got = eng.step([(extra, other[5 * i:5 * i + 5])], want="last")        # an eager prompt portion in between
        assert_logits_close(got, plain_logits(name, other)[5 * i + 4:5 * i + 5], dtype, f"{name} {dtype} eager between replays",
                            sharp=True)
    eng.cache.check()


def test_short_prompt_steps_replayed_from_a_graph():
    """bfloat16 prompt steps of a few tokens go through captured graphs with padding rows (an extra sequence on the
    spare page and in the spare state row); portions of a prompt one after another, each from what the last one left."""
    name = "R"
    eng = engine(name, "bfloat16")
    assert eng.graph_ok and eng.prompt_graphs
    toks = tokens_for(name, 120, 8)
    want = plain_logits(name, toks)
    s, at = eng.acquire(), 0
    for n in (10, 10, 30, 10, 40, 20):
        got = eng.step([(s, toks[at:at + n])], want="last")
        at += n
        assert_logits_close(got, want[at - 1:at], "bfloat16", f"prompt portion ending at {at} through a graph", sharp=True)
    assert any(k[0] == "prompt" for k in eng._runners), "no prompt step was replayed from a graph"


def test_command_line_and_trace_replay_as_a_user_starts_them(tmp_path):
    """`random` writes a model folder from a configuration file, `run` generates from it, and bin/trace_run replays
    steps over it (prompts of unequal lengths together, then single tokens, a request that ends early, its slot used
    again by a later request) in both types; the logits against the plain model."""
    import json
    import os
    import subprocess
    import sys
    from helpers import ROOT, run_trace
    from plain_repolix import PlainRepolix

    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(CONFIGS["P"]))
    folder = str(tmp_path / "model")
    env = dict(os.environ, PYTHONPATH=ROOT)
    subprocess.run([sys.executable, "-m", "synaptix_amd", "random", str(cfg_file), folder, "--seed", "3"], check=True,
                   env=env, cwd=ROOT, timeout=300)
    plain = PlainRepolix.from_folder(folder)
    prompt = tokens_for("P", 9, 1)
    run = subprocess.run([sys.executable, "-m", "synaptix_amd", "run", folder, "--prompt-ids", ",".join(map(str, prompt)),
                          "--max-tokens", "4", "--temperature", "0", "--compute-dtype", "f32"], check=True, env=env, cwd=ROOT,
                         timeout=300, capture_output=True, text=True)
    assert run.stdout.strip() or run.stderr.strip()
    a, b, c = tokens_for("P", 70, 2), tokens_for("P", 5, 3), tokens_for("P", 30, 4)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]}, {"id": "b", "tokens": b[:3], "want": [2]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[66:67], "want": [0]}, {"id": "b", "tokens": b[3:4], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[67:68], "want": []}, {"id": "b", "tokens": b[4:5], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[68:69], "want": [0]}], "end": []},
             {"step": 4, "entries": [{"id": "c", "tokens": c, "want": [0, 29]}], "end": ["c"]},
             {"step": 5, "entries": [{"id": "a", "tokens": a[69:70], "want": [0]}], "end": ["a"]}]
    la, lb, lc = plain.logits(a), plain.logits(b), plain.logits(c)
    want = {0: torch.stack([la[0], la[65], lb[2]]), 1: torch.stack([la[66], lb[3]]), 2: lb[4:5], 3: la[68:69],
            4: torch.stack([lc[0], lc[29]]), 5: la[69:70]}
    for dtype in DTYPES:
        out = run_trace(folder, dtype, steps, 256, str(tmp_path / f"out_{dtype}"))
        assert sorted(out) == sorted(want)
        for k, w in want.items():
            assert_logits_close(out[k], w, dtype, f"trace step {k} in {dtype}", sharp=True)
