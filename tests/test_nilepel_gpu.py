"""Nilepel on the GPU against the plain implementation (tests/plain_nilepel.py): each new mechanism's kernels alone, with
inputs made so that a window or a run that is one token off, a sink left out, a gate on the wrong head or a wrong pairing
shows; then whole models of four small configurations in 32-bit and in bfloat16: whole prompts, portions, token by token,
unequal batches, slots and pages used again, long decoding, the first tokens, and greedy generation through the pipeline."""
import math

import pytest
import torch

import plain_nilepel as P
from nilepel_cases import CONFIGS, cases, model_folder, plain_logits, plain_model, tokens_for
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
        self.seq_start, self.seq_past = ints(starts), ints(self.past)
        self.tok_seq = ints(b for b, n in enumerate(self.new) for _ in range(n))
        self.tok_pos = ints(p + i for p, n in zip(self.past, self.new) for i in range(n))
        self.N = starts[-1]


def paged(rows_by_head, dtype, n_pages, order):
    """rows_by_head [T, heads, n] into pages [n_pages, heads, 64, n] at the pages `order` names."""
    T, Hh, n = rows_by_head.shape
    pages = torch.zeros((n_pages, Hh, 64, n), dtype=torch.float64)
    for t in range(T):
        pages[order[t // 64], :, t % 64] = rows_by_head[t]
    return pages.to(dtype)


# ----------------------------------------------------------------------------- mechanisms alone
MASKS = [("chunk", 1), ("chunk", 2), ("chunk", 37), ("chunk", 63), ("chunk", 64), ("chunk", 65), ("chunk", 130), ("chunk", 500),
         ("window", 1), ("window", 64), ("window", 65), ("window", 0), ("both", (50, 64))]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind,size", MASKS)
def test_runs_windows_sinks_and_a_gate_a_head(kind, size, dtype):
    """Keys are one-hot in their position (modulo the key size) and queries are long, so that a query gives nearly all
    its weight to the visible keys of one residue: a run or a window that is one token off changes the result by its own
    size.  Half of the heads have a sink that holds about half of the softmax's sum, one head a sink that counts for
    nothing; every head has a gate of its own.  All queries at once (prompts: in bf16 the tiles on the matrix cores),
    a second piece that starts inside a page, and single queries at the borders of pages and runs, over pages in a
    shuffled order."""
    from synaptix_amd.kernels import ops
    H, G, D, E, T = 4, 2, 16, 32, 200
    g = torch.Generator().manual_seed(3)
    k = torch.zeros(T, G, D, dtype=F64)
    q = torch.zeros(T, H, D, dtype=F64)
    for t in range(T):
        for gg in range(G):
            k[t, gg, (t + gg) % D] = 1.0
        for h in range(H):
            q[t, h, (t - 1 - 3 * h) % D] = 9.0           # head h looks 1 + 3 h back (and at what shares that residue)
    q = q + 0.1 * randn(g, T, H, D)
    v = randn(g, T, G, E)
    sinks = torch.tensor([9.0, -30.0, 8.5, 2.0], dtype=F64)
    gates = randn(g, T, H + 3) * 2.0                       # (columns of longer rows)
    q, k, v = [x.to(dtype).double() for x in (q, k, v)]
    window, chunk = {"chunk": (None, size), "window": (size or None, None), "both": size}[kind] if kind != "both" else size
    mask = P.window_mask(T, window)
    if chunk is not None:
        mask = mask & P.chunk_mask(T, chunk)
    want = P.attend(q, k, v, 1.0, mask, sinks) * torch.sigmoid(gates[:, :H])[:, :, None]
    want = want.reshape(T, H * E)
    order = [3, 0, 2, 1]
    kp = paged(k, dtype, 5, order).to(DEV)
    vp = paged(v, dtype, 5, order).transpose(2, 3).contiguous().to(DEV)
    qd, gd = dev(q.reshape(T, H * D), dtype), dev(gates)
    table = ints(order).view(1, 4)
    how = dict(window=window or 0, chunk=chunk or 0, sinks=dev(sinks), gate_per_head=True)
    tol = 2e-4 if dtype == torch.float32 else 6e-2

    def run(first, n, tiles=False):
        st = Step([(0, first, n)])
        out = torch.empty((n, H * E), dtype=dtype, device=DEV)
        if tiles:
            ops.window_attention_prefill_bf16(qd[first:first + n], kp, vp, table, st.seq_start, st.seq_past, out, 1.0, H, G, D, E,
                                              gate=gd[first:first + n, :H], **how)
        else:
            ops.window_attention(qd[first:first + n], kp, vp, table, st.tok_seq, st.tok_pos, out, 1.0, H, G, D, E,
                                 gate=gd[first:first + n, :H], **how)
        return float((out.cpu().double() - want[first:first + n]).abs().max())

    assert run(0, T) < tol, "every query, one wave a (token, head)"
    if dtype == torch.bfloat16:
        assert run(0, T, tiles=True) < tol, "every query, tiles on the matrix cores"
        assert run(70, T - 70, tiles=True) < tol, "a second piece that starts inside a page, in tiles"
        assert run(0, 3, tiles=True) < tol, "the first three tokens, in tiles"
    assert run(70, T - 70) < tol, "a second piece that starts inside a page"
    edges = {T - 1, 130, 129, 128, 65, 64, 63, 1, 0}
    if chunk:
        edges |= {c for c in (chunk - 1, chunk, chunk + 1, 2 * chunk - 1, 2 * chunk, 3 * chunk) if 0 <= c < T}
    for t in sorted(edges):
        assert run(t, 1) < tol, f"the single query at {t}"
    # the sink is not nothing: without it the result differs by its own size
    no_sink = P.attend(q, k, v, 1.0, mask) * torch.sigmoid(gates[:, :H])[:, :, None]
    assert float((no_sink.reshape(T, H * E) - want).abs().max()) > 0.3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_far_key_among_hundreds_and_the_first_keys_of_a_run(dtype):
    """One query and one key are scaled so that this key's score stands out among 700: the result is that key's value
    where the query's run (or window) holds it and another where it does not; the key is the first of its run, the last
    of the run before, and the first one that a window still holds."""
    from synaptix_amd.kernels import ops
    H, G, D, E, T = 2, 1, 32, 16, 700
    g = torch.Generator().manual_seed(5)
    q, k, v = 0.3 * randn(g, T, H, D), 0.3 * randn(g, T, G, D), randn(g, T, G, E)
    order = list(range(11))
    for far, at, window, chunk, seen in [(320, 699, None, 380, False), (380, 699, None, 380, True), (379, 699, None, 380, False),
                                         (3, 699, None, None, True), (100, 699, 600, None, True), (99, 699, 600, None, False),
                                         (640, 640, 1, None, True), (0, 319, None, 320, True)]:
        qq, kk = q.clone(), k.clone()
        kk[far] = 0.0
        kk[far, 0, 5] = 4.0
        qq[at, :, 5] = 8.0
        qq, kk, vv = [x.to(dtype).double() for x in (qq, kk, v)]
        mask = P.window_mask(T, window)
        if chunk:
            mask = mask & P.chunk_mask(T, chunk)
        want = P.attend(qq, kk, vv, 1.0, mask, torch.zeros(H, dtype=F64))[at].reshape(1, H * E)
        near = float((want.view(H, E) - vv[far, 0]).abs().max())
        assert (near < 1e-3) == seen, (far, at, window, chunk)
        kp, vp = paged(kk, dtype, 11, order).to(DEV), paged(vv, dtype, 11, order).transpose(2, 3).contiguous().to(DEV)
        st = Step([(0, at, 1)])
        out = torch.empty((1, H * E), dtype=dtype, device=DEV)
        ops.window_attention(dev(qq[at].reshape(1, H * D), dtype), kp, vp, ints(order).view(1, 11), st.tok_seq, st.tok_pos, out,
                             1.0, H, G, D, E, window=window or 0, chunk=chunk or 0, sinks=torch.zeros(H, device=DEV))
        tol = 2e-4 if dtype == torch.float32 else 4e-2
        assert float((out.cpu().double() - want).abs().max()) < tol, (far, at, window, chunk)
        # the same query among all queries of a prompt (in bf16 also in tiles on the matrix cores)
        st = Step([(0, 0, at + 1)])
        qd = dev(qq[:at + 1].reshape(at + 1, H * D), dtype)
        how = dict(window=window or 0, chunk=chunk or 0, sinks=torch.zeros(H, device=DEV))
        out = torch.empty((at + 1, H * E), dtype=dtype, device=DEV)
        ops.window_attention(qd, kp, vp, ints(order).view(1, 11), st.tok_seq, st.tok_pos, out, 1.0, H, G, D, E, **how)
        assert float((out[at:].cpu().double() - want).abs().max()) < tol, ("prompt", far, at, window, chunk)
        if dtype == torch.bfloat16:
            out = torch.empty((at + 1, H * E), dtype=dtype, device=DEV)
            ops.window_attention_prefill_bf16(qd, kp, vp, ints(order).view(1, 11), st.seq_start, st.seq_past, out, 1.0, H, G, D, E, **how)
            assert float((out[at:].cpu().double() - want).abs().max()) < tol, ("prompt in tiles", far, at, window, chunk)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pairing", ["pairs", "halves"])
@pytest.mark.parametrize("nq,nk,D,E,rot,norm", [(4, 2, 16, 24, 8, True), (6, 6, 12, 10, 12, False), (2, 1, 20, 6, 2, True),
                                                (8, 4, 32, 64, 32, True), (3, 1, 10, 4, 0, False)])
def test_intake_turns_pairs_or_halves_and_leaves_another_layers_pages_alone(nq, nk, D, E, rot, norm, pairing, dtype):
    from synaptix_amd.kernels import ops
    from synaptix_amd.parts import RotaryByWavelength
    g = torch.Generator().manual_seed(D + rot)
    st = Step([(0, 60, 10), (1, 0, 3)])
    width = (nq + nk) * D + nk * E
    rows, bias = randn(g, st.N, width + 3), 0.5 * randn(g, width)
    qg, kg = 1.0 + 0.3 * randn(g, D), 1.0 + 0.3 * randn(g, D)
    position = RotaryByWavelength(300.0, rot, 128, factor=3.0, low=1.0, high=4.0, original=40, pairing=pairing)
    f = P.stretched_rates(P.rates(300.0, rot), 3.0, 1.0, 4.0, 40) if rot else torch.zeros(0, dtype=F64)
    x = rows[:, :width] + bias
    qk = x[:, :(nq + nk) * D].view(st.N, nq + nk, D)
    if norm:
        qk = torch.cat([P.rms_norm(qk[:, :nq], qg, 1e-5), P.rms_norm(qk[:, nq:], kg, 1e-5)], 1)
    turned = torch.cat([P.rotate(qk[:10], f, pairing, first=60), P.rotate(qk[10:], f, pairing, first=0)], 0)
    q = torch.empty((st.N, nq * D), dtype=dtype, device=DEV)
    kp = torch.zeros((4, nk, 64, D), dtype=dtype, device=DEV)
    vp = torch.zeros((4, nk, E, 64), dtype=dtype, device=DEV)
    table = ints([2, 0, 1, 3]).view(2, 2)
    gains = (dev(qg), dev(kg), 1e-5) if norm else (None, None, 0.0)
    ops.window_intake(dev(rows), dev(bias), q, kp, vp, table, st.tok_seq, st.tok_pos, *gains, nq, nk, D, E,
                      rotation=position.tables(DEV), pairs=pairing == "pairs")
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    big = max(1.0, float(turned.abs().max()) * 1.2)
    assert float((q.cpu().double().view(st.N, nq, D) - turned[:, :nq]).abs().max()) < tol * big
    vals = x[:, (nq + nk) * D:].view(st.N, nk, E)
    for n, (page, slot) in enumerate([(2, 60), (2, 61), (2, 62), (2, 63)] + [(0, i) for i in range(6)] + [(1, 0), (1, 1), (1, 2)]):
        assert float((kp[page, :, slot].cpu().double() - turned[n, nq:]).abs().max()) < tol * big, f"key of token {n}"
        assert float((vp[page, :, :, slot].cpu().double() - vals[n]).abs().max()) < tol * big, f"value of token {n}"
    # a layer that reads another layer's keys: rows that hold queries (and a gate) only, pages untouched
    k0, v0 = kp.clone(), vp.clone()
    q2 = torch.empty_like(q)
    narrow = torch.cat([rows[:, :nq * D], rows[:, -3:]], 1)
    ops.window_intake(dev(narrow), dev(bias[:nq * D]), q2, kp, vp, table, st.tok_seq, st.tok_pos, gains[0], gains[0], gains[2],
                      nq, nk, D, E, write_kv=False, rotation=position.tables(DEV), pairs=pairing == "pairs")
    assert torch.equal(q2, q) and torch.equal(kp, k0) and torch.equal(vp, v0)


@pytest.mark.parametrize("N,E,top,groups,keep,scale", [(50, 8, 3, 4, 2, 1.5), (3, 5, 5, 1, 1, 1.0), (200, 16, 4, 4, 2, 0.25),
                                                       (7, 15, 4, 3, 1, 2.0), (1, 6, 1, 3, 1, 3.0), (40, 12, 2, 6, 6, 1.0)])
def test_router_with_a_factor_on_rows_of_a_longer_product(N, E, top, groups, keep, scale):
    """On equal inputs the choice is exact: the same experts in the same order, weights that are the scores times the
    factor; the logits are the first columns of rows that hold one more number (the shared expert's gate)."""
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(N + E)
    z = (2.0 * torch.randn(N, E + 1, generator=g)).float()
    ids_want, w_want = P.route(z[:, :E].double(), top, groups, keep, scale)
    zd = z.to(DEV)
    ids = torch.empty((N, top), dtype=torch.int32, device=DEV)
    w = torch.empty((N, top), dtype=torch.float32, device=DEV)
    ops.route_scores(zd[:, :E], None, ids, w, groups, keep, False, scale)
    assert torch.equal(ids.cpu().long(), ids_want)
    assert float((w.cpu().double() - w_want).abs().max()) < 1e-6 * max(1.0, scale)


@pytest.mark.parametrize("parts", [1, 3])
def test_a_gate_for_every_row_in_the_residual_sum(parts):
    from synaptix_amd.kernels import ops
    g = torch.Generator().manual_seed(parts)
    N, Hd = 37, 72
    x, a, b = randn(g, N, Hd), randn(g, parts, N, Hd), randn(g, N, Hd)
    z = 2.0 * randn(g, N, 5)
    gain, scale = 1.0 + 0.2 * randn(g, Hd), randn(g, Hd)
    summed = x + a.sum(0) + torch.sigmoid(z[:, 4:5]) * scale * b
    rows = torch.tensor([5, 0, 36, 5])
    zd = dev(z)
    for pick in (None, rows):
        resid = dev(x)
        n = N if pick is None else len(pick)
        out = torch.empty((n, Hd), dtype=torch.float32, device=DEV)
        ops.add_scaled_rmsnorm(resid, [(dev(a), None, None), (dev(b), dev(scale), zd[:, 4:])], dev(gain), 1e-6, out,
                               None if pick is None else ints(pick.tolist()))
        want = P.rms_norm(summed, gain, 1e-6)
        want = want if pick is None else want[pick]
        assert float((out.cpu().double() - want).abs().max()) < 1e-5
        assert float((resid.cpu().double() - (summed if pick is None else x)).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_experts_with_a_factor_and_a_shared_expert_behind_its_gate(dtype):
    """parts.RoutedExperts as this design uses it against the plain mixture: silu experts, groups, the factor on the
    weights, and the shared expert times the sigmoid of one number a token."""
    from synaptix_amd.parts import RoutedExperts, GatedMlp, as_delta
    W, F, E, top, S = 64, 32, 8, 3, 48
    g = torch.Generator().manual_seed(8)
    w = {"router": 0.5 * randn(g, E, W), "shared.sg": 0.4 * randn(g, 1, W)}
    for e in range(E):
        w.update({f"e{e}.gate": 0.2 * randn(g, F, W), f"e{e}.up": 0.2 * randn(g, F, W), f"e{e}.down": 0.2 * randn(g, W, F)})
    w.update({"shared.gate": 0.2 * randn(g, S, W), "shared.up": 0.2 * randn(g, S, W), "shared.down": 0.2 * randn(g, W, S)})
    w = {n: t.to(torch.bfloat16).double() for n, t in w.items()}
    names = ("gate", "up", "down")
    ff = RoutedExperts("", W, F, E, top, "silu", router_bias=False, gated=True, router="scores", n_groups=4, keep_groups=2,
                       shared=GatedMlp("shared.", W, S, "silu", names=names), route_scale=1.7, shared_gate="shared.sg")
    assert set(ff.tensor_specs()) == set(w)
    ff.load(lambda n: dev(w[n], dtype))
    c = {"router": {"experts": E, "top": top, "groups": {"count": 4, "keep": 2}, "scale": 1.7}, "shared": {"ff": S}}
    for N in (1, 5, 70):
        h = randn(g, N, W).to(dtype).double()
        want = P.experts(h, w, "", c)
        got = as_delta(ff.forward(dev(h, dtype), None))
        got = got.sum(0) if got.dim() == 3 else got
        tol = 1e-4 if dtype == torch.float32 else 3e-2
        assert float((got.cpu().double() - want).abs().max()) < tol * max(1.0, float(want.abs().max())), f"{N} rows"


# ----------------------------------------------------------------------------- whole models

def lengths(name):
    return {"P": [1, 2, 21, 64, 65, 150], "Q": [3, 70, 71, 129, 140], "R": [5, 64, 128, 200], "S": [1, 2, 3, 66, 90],
            "T": [2, 41, 100, 130]}[name]


@pytest.mark.parametrize("name,dtype", cases(["P", "Q", "R", "S", "T"]))
def test_whole_prompts(name, dtype):
    eng = engine(name, dtype)
    for i, n in enumerate(lengths(name)):
        toks = tokens_for(name, n, 100 + i)
        s = eng.acquire()
        got = eng.step([(s, toks)], want="all")
        assert_logits_close(got, plain_logits(name, toks), dtype, f"{name} {dtype} {n} tokens whole", sharp=True)
        eng.release(s)
    eng.cache.check()


@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_the_residual_after_every_layer_in_float32(name):
    """The model's layers one after another: the residual rows that each leaves, read from the engine's own pass."""
    from synaptix_amd.parts import as_delta
    toks = tokens_for(name, 70, 3)
    want = plain_model(name).residuals(toks)
    eng = engine(name, "float32")
    got = []
    for block in eng.model.blocks:
        inner = block.forward

        def spy(resid, pending, ctx, cache, owner=True, inner=inner):
            out = inner(resid, pending, ctx, cache, owner)
            delta = as_delta(out)
            got.append(resid.clone() + (delta.sum(0) if delta.dim() == 3 else delta))      # (partial sums not yet added)
            return out
        block.forward = spy
    eng.step([(eng.acquire(), toks)], want="last")
    assert len(got) == len(want)
    for i, (a, b) in enumerate(zip(got, want)):
        assert float((a.cpu().double() - b).abs().max()) < 1e-4 * max(1.0, float(b.abs().max())), f"after layer {i}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_portions_of_several_sizes(name, dtype):
    """A prompt in portions of 2, 1, 3, 17, 64 and 2 tokens and the rest: every portion starts from the pages that the
    earlier ones left (inside a page, at a page's border, inside and beyond the first window and run)."""
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
@pytest.mark.parametrize("name,head,n", [("P", 30, 130), ("Q", 1, 160), ("R", 100, 290), ("S", 3, 90), ("T", 35, 100)])
def test_prompt_then_token_by_token(name, head, n, dtype):
    """Decoding long enough that every window and run passes over decoded tokens and over a page's border."""
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


@pytest.mark.parametrize("name,dtype", cases(["P", "Q", "R", "S", "T"]))
def test_unequal_batches_and_slots_used_again(name, dtype):
    """Requests of unequal lengths start together and are decoded together, the shorter ones ending earlier; then
    other requests take the slots and pages that came free (the cache has room for little more than one batch), in
    another order: each request's logits equal the plain model's for that request alone."""
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


@pytest.mark.parametrize("seed", list(range(7000, 7016)))
def test_configurations_drawn_from_a_seed_in_float32(seed):
    """Layer kinds, orders, head counts, sizes, masks, readers of other layers' keys and routers drawn from a seed (the
    cases above are chosen; these are not): a prompt whole, then requests of unequal lengths cut at unequal places
    and decoded together, 3 to 20 of them, against the plain model for each alone."""
    import random
    from nilepel_cases import random_model
    from synaptix_amd import Engine
    cfg, folder, plain = random_model(seed)
    rng = random.Random(seed + 1)
    g = torch.Generator().manual_seed(seed)
    T = rng.choice([70, 150, 330])
    lens = [T, 9, T // 2] + [rng.randint(2, T) for _ in range(rng.choice([0, 6, 10, 17]))]
    toks = [torch.randint(0, cfg.vocab, (n,), generator=g).tolist() for n in lens]
    want = [plain.logits(t) for t in toks]
    eng = Engine.load(folder, dtype="float32", max_tokens=8192, max_slots=32)
    s = eng.acquire()
    assert_logits_close(eng.step([(s, toks[0])], want="all"), want[0], "float32", f"seed {seed} whole", sharp=True)
    eng.release(s)
    slots = [eng.acquire() for _ in toks]
    cut = [min(max(1, len(t) - 12 - 3 * (i % 5)), len(t)) for i, t in enumerate(toks)]
    out = eng.step([(s, t[:k]) for s, t, k in zip(slots, toks, cut)], want="all")
    got, at = [[] for _ in toks], 0
    for i, k in enumerate(cut):
        got[i].append(out[at:at + k])
        at += k
    fed, live = list(cut), [i for i in range(len(toks)) if cut[i] < len(toks[i])]
    while live:
        out = eng.step([(slots[i], [toks[i][fed[i]]]) for i in live], want="last")
        for j, i in enumerate(live):
            got[i].append(out[j:j + 1])
            fed[i] += 1
        live = [i for i in live if fed[i] < len(toks[i])]
    for i in range(len(toks)):
        assert_logits_close(torch.cat(got[i]), want[i], "float32", f"seed {seed} request {i} of {len(toks)}", sharp=True)
    eng.cache.check()


def test_a_window_gives_its_pages_back():
    """A long sequence in a cache that holds far fewer tokens than it has: the groups that keep a window or a run give
    the pages behind it back as the sequence grows (the configuration has no layer that sees every key)."""
    toks = tokens_for("P", 700, 12)
    want = plain_logits("P", toks)
    eng = engine("P", "float32", max_tokens=64 * 5, max_slots=1)
    s = eng.acquire()
    got = [eng.step([(s, toks[:40])], want="all")]
    for at in range(40, 700, 60):
        got.append(eng.step([(s, toks[at:at + 60])], want="all"))
    assert_logits_close(torch.cat(got), want, "float32", "700 tokens through 5 pages", sharp=True)
    eng.release(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens(dtype):
    """Sequences of one and two tokens, and every position up to the windows and runs and a little more, one by one."""
    for name in ("P", "S"):
        if name == "S" and dtype != "float32":
            continue
        eng = engine(name, dtype)
        toks = tokens_for(name, 45, 77)
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
    """500 tokens one by one: every window and run passes many times, pages come back and are used again."""
    toks = tokens_for("P", 500, 5)
    want = plain_logits("P", toks)
    eng = engine("P", "float32", max_tokens=64 * 4, max_slots=1)
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
    """Captured decode steps (three rows wide in a graph of four: one row is padding) with eager work of another
    sequence between the replays; every replay against the plain model."""
    eng = engine(name, dtype, max_tokens=64 * 12)
    assert eng.graph_ok
    # (tokens at none of whose decoded positions the plain model's two best groups of experts nearly tie: where they do,
    # the rounding of bfloat16 activations picks the other group, in eager steps and replays alike)
    reqs = [tokens_for(name, n, 60 + n) for n in (90, 20, 140)]
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
    spare page); portions of a prompt one after another, each from what the last one left."""
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
    from plain_nilepel import PlainNilepel

    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(CONFIGS["P"]))
    folder = str(tmp_path / "model")
    env = dict(os.environ, PYTHONPATH=ROOT)
    subprocess.run([sys.executable, "-m", "synaptix_amd", "random", str(cfg_file), folder, "--seed", "3"], check=True,
                   env=env, cwd=ROOT, timeout=300)
    plain = PlainNilepel.from_folder(folder)
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
