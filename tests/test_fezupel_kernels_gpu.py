"""Each new mechanism's kernels alone against the plain functions of ``plain_fezupel``, in
32-bit and in bfloat16: norms that store or add, embedding plus position row, the router, the
experts, and the attention whose values are its keys (keys spread over shuffled pages; windows
of one token, less than a page, a page, more; with and without the silent soft-max term and
the gate; a key that would dominate planted just inside and just outside the window)."""
import math

import pytest
import torch

import plain_fezupel as P
from gpu_util import DEV, rel_err, tol
from zinfer_amd import ops

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _rand(shape, seed, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


# ------------------------------------------------------------------------------ norms
@pytest.mark.parametrize("T, W", [(1, 48), (5, 77), (33, 336), (3, 4096), (2, 9000)])
@pytest.mark.parametrize("centred, bias", [(True, True), (True, False), (False, True)])
def test_norm_rows_store_and_add(T, W, centred, bias):
    x = _rand((T, W), 1, 3.0) + 1.5
    w = 1 + _rand((W,), 2, 0.2)
    b = _rand((W,), 3, 0.5) if bias else None
    eps = 1e-5
    if centred:
        ref = P.layer_norm(x, w, b if bias else torch.zeros(W), eps)
    else:
        x64 = x.double()
        ref = x64 / torch.sqrt((x64 * x64).mean(-1, keepdim=True) + eps) * w.double() \
            + (b.double() if bias else 0.0)
    xd, wd = x.to(DEV), w.to(DEV)
    bd = b.to(DEV) if bias else None
    for dt in DTYPES:
        out = torch.empty((T, W), dtype=dt, device=DEV)
        ops.norm_rows(xd, wd, bd, eps, out, centred)
        assert rel_err(out, ref) < tol(dt)
    base = _rand((T, W), 4)
    acc = base.to(DEV)
    ops.norm_rows(xd, wd, bd, eps, acc, centred, add=True)
    assert rel_err(acc, base.double() + ref) < tol(torch.float32)


@pytest.mark.parametrize("T, W", [(1, 48), (7, 336), (3, 4096), (2, 8192)])
@pytest.mark.parametrize("dt", DTYPES)
def test_norm_add_norm_is_the_two_norms_one_after_the_other(T, W, dt):
    y, x = _rand((T, W), 81, 2.0) + 0.5, _rand((T, W), 82)
    wa, ba = 1 + _rand((W,), 83, 0.2), _rand((W,), 84, 0.5)
    wb, bb = 1 + _rand((W,), 85, 0.2), _rand((W,), 86, 0.5)
    dev = lambda t: t.to(DEV)
    x1, out1 = dev(x), torch.empty((T, W), dtype=dt, device=DEV)
    ops.norm_add_norm(dev(y), dev(wa), dev(ba), 1e-5, True, x1, dev(wb), dev(bb), 1e-6, True, out1)
    x2, out2 = dev(x), torch.empty((T, W), dtype=dt, device=DEV)
    ops.norm_rows(dev(y), dev(wa), dev(ba), 1e-5, x2, True, add=True)
    ops.norm_rows(x2, dev(wb), dev(bb), 1e-6, out2, True)
    assert rel_err(x1, x2) < 1e-6 and rel_err(out1, out2.double()) < (1e-6 if dt == torch.float32 else 2.0 ** -8)
    ref_x = x.double() + P.layer_norm(y, wa, ba, 1e-5)
    assert rel_err(x1, ref_x) < 2e-5
    assert rel_err(out1, P.layer_norm(ref_x, wb, bb, 1e-6)) < tol(dt)


def test_layer_norm_of_a_row_with_a_large_mean():
    """The variance comes from the deviations: a mean a thousand times the spread leaves it."""
    x = 1000.0 + _rand((4, 256), 5, 1.0)
    ref = P.layer_norm(x, torch.ones(256), torch.zeros(256), 1e-6)
    out = torch.empty((4, 256), dtype=torch.float32, device=DEV)
    ops.norm_rows(x.to(DEV), torch.ones(256, device=DEV), None, 1e-6, out, True)
    assert float((out.cpu().double() - ref).abs().max()) < 1e-3


@pytest.mark.parametrize("dt", DTYPES)
def test_embed_position(dt):
    E, Pt = _rand((50, 72), 6, dtype=dt), _rand((40, 72), 7, dtype=dt)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    pos = torch.tensor([0, 39, 17, 1], dtype=torch.int32)
    out = torch.empty((4, 72), dtype=torch.float32, device=DEV)
    ops.embed_position(E.to(DEV), ids.to(DEV), Pt.to(DEV), pos.to(DEV), out)
    ref = E.double()[ids.long()] + Pt.double()[pos.long()]
    assert rel_err(out, ref) < 1e-6


# ------------------------------------------------------------------------------ experts
@pytest.mark.parametrize("T, W, E, top", [(7, 48, 6, 2), (3, 50, 1, 1), (5, 72, 9, 9),
                                           (4, 64, 130, 70), (2, 384, 12, 5)])
@pytest.mark.parametrize("dt", DTYPES)
def test_router(T, W, E, top, dt):
    h = _rand((T, W), 8, dtype=dt)
    R = _rand((E, W), 9, 0.5).to(torch.bfloat16).float()
    b = _rand((E,), 10, 0.5)
    ids = torch.empty((T, top), dtype=torch.int32, device=DEV)
    wts = torch.empty((T, top), dtype=torch.float32, device=DEV)
    ops.moe_route(h.to(DEV), R.to(DEV), b.to(DEV), ids, wts)
    ref_ids, ref_w = P.route(h, R, b, top)
    assert torch.equal(ids.cpu().long(), ref_ids)       # in the order of their logits
    assert rel_err(wts, ref_w) < 1e-5
    assert torch.allclose(wts.sum(-1).cpu(), torch.ones(T), atol=1e-5)


def test_router_bias_decides():
    h = torch.zeros((1, 16))
    b = torch.tensor([0.0, 3.0, -1.0, 2.0])
    ids = torch.empty((1, 2), dtype=torch.int32, device=DEV)
    wts = torch.empty((1, 2), dtype=torch.float32, device=DEV)
    ops.moe_route(h.to(DEV), torch.zeros((4, 16), device=DEV), b.to(DEV), ids, wts)
    assert ids.cpu().tolist() == [[1, 3]]
    e = math.exp(-1.0)
    assert torch.allclose(wts.cpu(), torch.tensor([[1 / (1 + e), e / (1 + e)]]), atol=1e-6)


@pytest.mark.parametrize("T, W, ff, E, top", [(6, 48, 20, 6, 2), (3, 50, 30, 1, 1),
                                               (9, 72, 17, 5, 5), (4, 128, 64, 8, 3)])
@pytest.mark.parametrize("dt", DTYPES)
def test_experts(T, W, ff, E, top, dt):
    limit, alpha, shift = 0.5, 1.702, 1.0
    h = _rand((T, W), 11, dtype=dt)
    w = {}
    for e in range(E):
        w[f"e{e}.gate"] = _rand((ff, W), 20 + e, 2 / W ** 0.5, dt)
        w[f"e{e}.up"] = _rand((ff, W), 40 + e, 2 / W ** 0.5, dt)
        w[f"e{e}.down"] = _rand((W, ff), 60 + e, 2 / ff ** 0.5, dt)
    g = torch.Generator().manual_seed(12)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    share = torch.rand((T, top), generator=g)
    gate_up = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)]).to(DEV)
    down = torch.stack([w[f"e{e}.down"] for e in range(E)]).to(DEV)
    y = torch.empty((T, top, ff), dtype=dt, device=DEV)
    ops.moe_gate_up(h.to(DEV), gate_up, ids.to(DEV), y, limit, alpha, shift)
    base = _rand((T, W), 13)
    for add in (False, True):
        out = base.to(DEV)
        ops.moe_down(y, down, ids.to(DEV), share.to(DEV), out, add=add)
        ref = base.double() if add else torch.zeros((T, W), dtype=torch.float64)
        for t in range(T):
            for s in range(top):
                ref[t] += share[t, s].double() * P.clamped_expert(h[t:t + 1], w, f"e{int(ids[t, s])}.", limit)[0]
        assert rel_err(out, ref) < (2e-5 if dt == torch.float32 else 2e-2)
    # the limits bite: some products lie beyond them
    gates = h.double() @ w["e0.gate"].double().T
    assert float(gates.max()) > limit


@pytest.mark.parametrize("T, W, ff, E, top", [(40, 64, 24, 6, 2), (300, 128, 64, 8, 3),
                                               (17, 72, 136, 1, 1), (150, 352, 104, 40, 4),
                                               (260, 64, 8, 3, 3)])
def test_experts_of_many_tokens_sorted_by_expert(T, W, ff, E, top):
    """bfloat16, more tokens than stream their experts one by one: the tokens sorted by expert
    through MFMA tiles against the plain expert, and against the streaming kernels."""
    dt = torch.bfloat16
    limit, alpha, shift = 0.6, 1.702, 1.0
    h = _rand((T, W), 14, dtype=dt)
    w = {}
    for e in range(E):
        w[f"e{e}.gate"] = _rand((ff, W), 120 + e, 2 / W ** 0.5, dt)
        w[f"e{e}.up"] = _rand((ff, W), 220 + e, 2 / W ** 0.5, dt)
        w[f"e{e}.down"] = _rand((W, ff), 320 + e, 2 / ff ** 0.5, dt)
    g = torch.Generator().manual_seed(15)
    # an expert nobody uses where there are experts to spare; a token names an expert once
    allowed = [e for e in range(E) if e != 1 or E <= top + 1]
    ids = torch.stack([torch.tensor(allowed)[torch.randperm(len(allowed), generator=g)[:top]]
                       for _ in range(T)]).to(torch.int32)
    share = torch.rand((T, top), generator=g)
    gate_up = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)]).to(DEV)
    down = torch.stack([w[f"e{e}.down"] for e in range(E)]).to(DEV)
    assert ops.moe_grouped_covers(h.to(DEV), gate_up) and T > ops.MOE_STREAM_MAX_TOKENS
    base = _rand((T, W), 16)
    for add in (False, True):
        y = torch.empty((T, top, ff), dtype=dt, device=DEV)
        out = base.to(DEV)
        ops.moe_experts(h.to(DEV), gate_up, down, ids.to(DEV), share.to(DEV), y, out, limit, alpha,
                        shift, add=add)
        y2 = torch.empty((T, top, ff), dtype=dt, device=DEV)
        out2 = base.to(DEV)
        ops.moe_gate_up(h.to(DEV), gate_up, ids.to(DEV), y2, limit, alpha, shift)
        ops.moe_down(y2, down, ids.to(DEV), share.to(DEV), out2, add=add)
        assert rel_err(out, out2) < 2e-2
        if T <= 150:
            ref = base.double() if add else torch.zeros((T, W), dtype=torch.float64)
            for t in range(T):
                for s_ in range(top):
                    ref[t] += share[t, s_].double() * P.clamped_expert(
                        h[t:t + 1], w, f"e{int(ids[t, s_])}.", limit)[0]
            assert rel_err(out, ref) < 2e-2
    # a token's result does not depend on the tokens beside it: the first 20 alone, the same bits
    if T >= 20:
        y3 = torch.empty((20, top, ff), dtype=dt, device=DEV)
        out3 = torch.empty((20, W), dtype=torch.float32, device=DEV)
        ops.moe_experts(h[:20].to(DEV), gate_up, down, ids[:20].contiguous().to(DEV),
                        share[:20].contiguous().to(DEV), y3, out3, limit, alpha, shift)
        out4 = torch.empty((T, W), dtype=torch.float32, device=DEV)
        ops.moe_experts(h.to(DEV), gate_up, down, ids.to(DEV), share.to(DEV), y, out4, limit,
                        alpha, shift)
        assert torch.equal(out3, out4[:20])


@pytest.mark.parametrize("dt", DTYPES)
def test_gated_act(dt):
    gu = _rand((7, 2 * 24), 17, 2.0, dtype=dt)
    out = torch.empty((7, 24), dtype=dt, device=DEV)
    ops.gated_act(gu.to(DEV), out, 1.5, 1.702, 1.0)
    g = gu[:, :24].double().clamp(max=1.5)
    u = gu[:, 24:].double().clamp(-1.5, 1.5)
    assert rel_err(out, g * torch.sigmoid(1.702 * g) * (u + 1)) < tol(dt)


# ------------------------------------------------------------------------------ attention
def _paged(k, n_kv, hd, page_size, seed):
    """Keys [n, n_kv * hd] of one sequence put into a pool through shuffled pages; returns the
    pool, the sequence's block table and the slots."""
    n = k.shape[0]
    pages = (n + page_size - 1) // page_size
    total = pages + 5
    g = torch.Generator().manual_seed(seed)
    table = torch.randperm(total, generator=g)[:pages].to(torch.int32)
    pool = torch.full((total, n_kv * page_size * hd), float("nan"), dtype=k.dtype, device=DEV)
    slots = torch.tensor([int(table[p // page_size]) * page_size + p % page_size for p in range(n)],
                         dtype=torch.int32)
    ops.kv_rows_write(k.to(DEV), slots.to(DEV), pool, n_kv, hd, page_size)
    return pool, table, slots


def _attend(q, gate, pool, table, n_ctx, n_q, nH, nKV, hd, page_size, scale, window, sink,
            mfma=False, n_splits=None, shared_tiles=None):
    """The last ``n_q`` positions of a sequence of ``n_ctx`` keys."""
    dev = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
    out = torch.empty((n_q, nH * hd), dtype=q.dtype, device=DEV)
    if mfma:
        ops.tied_attention_mfma(q.to(DEV), None if gate is None else gate.to(DEV), pool,
                                table.view(1, -1).to(DEV), dev([0, n_q]), dev([n_ctx]), out, scale,
                                window, sink, nH, nKV, hd, page_size, n_q, n_ctx, n_splits=n_splits,
                                shared_tiles=shared_tiles)
        return out
    ops.shared_kv_attention(q.to(DEV), None if gate is None else gate.to(DEV), pool,
                            table.view(1, -1).to(DEV), dev([0, n_q]), dev([n_ctx]),
                            dev([0] * n_q), out, scale, window, sink, nH, nKV, hd, page_size,
                            n_ctx)
    return out


@pytest.mark.parametrize("nH, nKV, hd, page", [(4, 2, 32, 16), (9, 3, 96, 16), (5, 1, 64, 8),
                                               (2, 2, 128, 16), (3, 1, 192, 4), (2, 1, 256, 16),
                                               (40, 2, 32, 16)])
@pytest.mark.parametrize("window", [0, 1, 5, 32, 33, 100])
def test_mfma_attention_against_plain(nH, nKV, hd, page, window):
    """The bfloat16 MFMA kernel: a whole prompt of several tiles, a portion behind a context,
    single tokens with the context unsplit and split over 2 and 5 workgroups."""
    dt = torch.bfloat16
    n = 171
    q = _rand((n, nH * hd), 130, dtype=dt)
    k = _rand((n, nKV * hd), 131, dtype=dt)
    gate = _rand((n, nH * hd), 132, 2.0, dtype=dt)
    pool, table, _ = _paged(k, nKV, hd, page, 133)
    scale = 0.7 / hd ** 0.5
    ref = P.sink_window_attention(q, k, nH, nKV, hd, scale, window if window else 10 ** 6)
    gated = ref * torch.sigmoid(gate.double())
    tolerance = 2.0 ** -7
    for tiles in (None, True):          # waves on their own where the shape allows; shared tiles
        out = _attend(q, gate, pool, table, n, n, nH, nKV, hd, page, scale, window, True, mfma=True,
                      shared_tiles=tiles)
        assert rel_err(out, gated) < tolerance
        tail = _attend(q[-50:], gate[-50:], pool, table, n, 50, nH, nKV, hd, page, scale, window,
                       True, mfma=True, shared_tiles=tiles)
        assert rel_err(tail, gated[-50:]) < tolerance
        one = _attend(q[-1:], gate[-1:], pool, table, n, 1, nH, nKV, hd, page, scale, window, True,
                      mfma=True, n_splits=2, shared_tiles=tiles)
        assert rel_err(one, gated[-1:]) < tolerance
    for splits in (1, 2, 5):
        last = _attend(q[-1:], None, pool, table, n, 1, nH, nKV, hd, page, scale, window, True,
                       mfma=True, n_splits=splits)
        assert rel_err(last, ref[-1:]) < tolerance
    nosink = _attend(q[-1:], gate[-1:], pool, table, n, 1, nH, nKV, hd, page, scale, window, False,
                     mfma=True, n_splits=3)
    exact = _attend(q[-1:], gate[-1:], pool, table, n, 1, nH, nKV, hd, page, scale, window, False)
    assert rel_err(nosink, exact.double()) < tolerance


@pytest.mark.parametrize("nH, nKV, hd, page", [(4, 2, 12, 16), (6, 2, 96, 16), (20, 1, 10, 4),
                                               (3, 3, 200, 8), (2, 1, 64, 16), (34, 2, 8, 16)])
@pytest.mark.parametrize("window", [0, 1, 5, 16, 17, 40])
@pytest.mark.parametrize("dt", DTYPES)
def test_attention_against_plain(nH, nKV, hd, page, window, dt):
    n = 45
    q = _rand((n, nH * hd), 30, dtype=dt)
    k = _rand((n, nKV * hd), 31, dtype=dt)
    gate = _rand((n, nH * hd), 32, 2.0, dtype=dt)
    pool, table, _ = _paged(k, nKV, hd, page, 33)
    scale = 0.7 / hd ** 0.5
    w = window if window else 10 ** 6
    ref = P.sink_window_attention(q, k, nH, nKV, hd, scale, w)
    tolerance = 2e-5 if dt == torch.float32 else 2.0 ** -7
    # the whole sequence as one portion, with the silent term and the gate
    out = _attend(q, gate, pool, table, n, n, nH, nKV, hd, page, scale, window, True)
    assert rel_err(out, ref * torch.sigmoid(gate.double())) < tolerance
    # its last 3 tokens as a portion, and its last token alone: the same rows, bit for bit
    tail = _attend(q[-3:], gate[-3:], pool, table, n, 3, nH, nKV, hd, page, scale, window, True)
    assert torch.equal(tail, out[-3:])
    last = _attend(q[-1:], gate[-1:], pool, table, n, 1, nH, nKV, hd, page, scale, window, True)
    assert torch.equal(last, out[-1:])
    # without the gate
    plain_out = _attend(q, None, pool, table, n, n, nH, nKV, hd, page, scale, window, True)
    assert rel_err(plain_out, ref) < tolerance


def test_attention_without_the_silent_term_is_a_plain_softmax():
    nH, nKV, hd, page, n = 2, 1, 16, 8, 20
    q, k = _rand((n, nH * hd), 34), _rand((n, nKV * hd), 35)
    pool, table, _ = _paged(k, nKV, hd, page, 36)
    out = _attend(q, None, pool, table, n, n, nH, nKV, hd, page, 0.25, 6, False)
    ref = torch.zeros((n, nH, hd), dtype=torch.float64)
    for i in range(n):
        lo = max(0, i - 5)
        for h in range(nH):
            a = torch.softmax((k[lo:i + 1].double() @ q[i].view(nH, hd)[h].double()) * 0.25, 0)
            ref[i, h] = a @ k[lo:i + 1].double()
    assert rel_err(out, ref.view(n, -1)) < 2e-5
    with_sink = _attend(q, None, pool, table, n, n, nH, nKV, hd, page, 0.25, 6, True)
    assert rel_err(with_sink, ref.view(n, -1)) > 1e-2       # the term is not nothing


@pytest.mark.parametrize("window, page", [(7, 16), (16, 16), (33, 8), (64, 16), (65, 16)])
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("mfma", [False, True])
def test_a_loud_key_just_inside_and_just_outside_the_window(window, page, decode, mfma):
    """Among hundreds of quiet keys one key answers the last query loudly.  Planted at the
    oldest position the window still holds it takes the output; one position earlier it
    must not be seen at all."""
    nH, nKV, hd, n = 2, 1, 32, 300
    for planted, seen in ((n - window, True), (n - window - 1, False)):
        dt = torch.bfloat16 if mfma else torch.float32
        k = _rand((n, nKV * hd), 37, 0.05, dt)
        q = _rand((n, nH * hd), 38, 0.05, dt)
        loud = torch.zeros(hd, dtype=dt)
        loud[3] = 6.0
        k[planted] = loud
        q[n - 1] = torch.cat([loud, loud]) * 2.0
        pool, table, _ = _paged(k, nKV, hd, page, 39)
        n_q = 1 if decode else 9
        out = _attend(q[-n_q:], None, pool, table, n, n_q, nH, nKV, hd, page, 1.0, window, True,
                      mfma=mfma)
        got = out[-1].view(nH, hd).float().cpu()
        if seen:
            assert float(got[0, 3]) > 5.9 and float(got[1, 3]) > 5.9
        else:
            assert float(got.abs().max()) < 0.5
        ref = P.sink_window_attention(q, k, nH, nKV, hd, 1.0, window)[-1]
        assert rel_err(out[-1], ref) < (2.0 ** -7 if mfma else 2e-5)


@pytest.mark.parametrize("mfma", [False, True])
def test_pages_before_the_window_are_not_touched(mfma):
    """The block-table entries of pages that lie wholly before the window are -1 (the pages
    have gone back): no kernel may look them up."""
    dt = torch.bfloat16 if mfma else torch.float32
    nH, nKV, hd, page, n, window = 4, 2, 32, 4, 200, 21
    q, k = _rand((n, nH * hd), 70, dtype=dt), _rand((n, nKV * hd), 71, dtype=dt)
    pool, table, _ = _paged(k, nKV, hd, page, 72)
    ref = P.sink_window_attention(q, k, nH, nKV, hd, 0.2, window)
    for n_q in (1, 7):
        gone = table.clone()
        gone[:(n - n_q + 1 - window) // page] = -1         # wholly before the first query's window
        out = _attend(q[-n_q:], None, pool, gone, n, n_q, nH, nKV, hd, page, 0.2, window, True,
                      mfma=mfma)
        assert rel_err(out, ref[-n_q:]) < (2.0 ** -7 if mfma else 2e-5)


def test_first_tokens_and_a_far_key_without_a_window():
    """Position 0 sees itself and the silent term only; with no window the first key of a long
    context still counts."""
    nH, nKV, hd, n, page = 2, 2, 16, 700, 16
    k = _rand((n, nKV * hd), 40, 0.05)
    q = _rand((n, nH * hd), 41, 0.05)
    k[0, :hd] = 0.0
    k[0, 5] = 5.0
    q[n - 1, :hd] = 0.0
    q[n - 1, 5] = 4.0
    pool, table, _ = _paged(k, nKV, hd, page, 42)
    out = _attend(q[-1:], None, pool, table, n, 1, nH, nKV, hd, page, 1.0, 0, True)
    assert float(out[0, 5]) > 4.9
    first = _attend(q[:1], None, pool, table, 1, 1, nH, nKV, hd, page, 1.0, 0, True)
    s = (q[0].view(nH, hd).double() * k[0].view(nKV, hd).double()).sum(-1)
    ref = (torch.exp(s) / (1 + torch.exp(s))).unsqueeze(-1) * k[0].view(nKV, hd).double()
    assert rel_err(first, ref.view(1, -1)) < 2e-5


def test_sequences_of_a_batch_read_their_own_pages():
    """Three sequences in one launch (a portion, a single token, a whole prompt) against each
    alone: the same bits."""
    nH, nKV, hd, page = 4, 2, 24, 8
    lens, q_lens = (50, 31, 12), (6, 1, 12)
    total_pages = sum((n + page - 1) // page for n in lens) + 3
    g = torch.Generator().manual_seed(43)
    perm = torch.randperm(total_pages, generator=g).tolist()
    pool = torch.zeros((total_pages, nKV * page * hd), dtype=torch.float32, device=DEV)
    tables, qs, alone = [], [], []
    max_pages = max((n + page - 1) // page for n in lens)
    for i, (n, nq) in enumerate(zip(lens, q_lens)):
        k = _rand((n, nKV * hd), 50 + i)
        pages = [perm.pop() for _ in range((n + page - 1) // page)]
        slots = torch.tensor([pages[p // page] * page + p % page for p in range(n)], dtype=torch.int32)
        ops.kv_rows_write(k.to(DEV), slots.to(DEV), pool, nKV, hd, page)
        tables.append(pages + [-1] * (max_pages - len(pages)))
        qs.append(_rand((nq, nH * hd), 60 + i))
    dev = lambda a: torch.tensor(a, dtype=torch.int32, device=DEV)
    table = dev(tables)
    for i, (n, nq) in enumerate(zip(lens, q_lens)):
        out = torch.empty((nq, nH * hd), dtype=torch.float32, device=DEV)
        ops.shared_kv_attention(qs[i].to(DEV), None, pool, table[i:i + 1].contiguous(), dev([0, nq]),
                                dev([n]), dev([0] * nq), out, 0.2, 9, True, nH, nKV, hd, page, n)
        alone.append(out)
    T = sum(q_lens)
    out = torch.empty((T, nH * hd), dtype=torch.float32, device=DEV)
    starts = [0, 6, 7, 19]
    seq_index = [0] * 6 + [1] + [2] * 12
    ops.shared_kv_attention(torch.cat(qs).to(DEV), None, pool, table, dev(starts), dev(list(lens)),
                            dev(seq_index), out, 0.2, 9, True, nH, nKV, hd, page, max(lens))
    assert torch.equal(out, torch.cat(alone))
