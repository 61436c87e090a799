"""Each new mechanism's kernels alone against the plain functions of ``plain_lodenex``, in
32-bit and in bfloat16: the activation, the norm that adds and leaves the sum, the rows of a
projection normed over whole segments and rotated in part on their way into rows and pages, a
matrix a head, and the attention with a score cap, a learned sink, chunks or a window and a
gate (keys spread over shuffled pages; chunks and windows of one token, less than a page, a
page, more; a key that would dominate planted just inside and just outside the edge, far back,
and at the first position; a token alone and in a batch)."""
import math

import pytest
import torch

import plain_lodenex as P
from gpu_util import DEV, rel_err, tol
from zinfer_amd import ops

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _rand(shape, seed, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _i32(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------------------ small kernels
@pytest.mark.parametrize("dt", DTYPES)
def test_activation(dt):
    x = _rand((7, 333), 1, 2.5, dt)
    z = x.double()
    want = {"gelu": P.gelu_erf(z),
            "gelu_tanh": 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3))),
            "silu": z * torch.sigmoid(z)}
    for kind, ref in want.items():
        out = torch.empty_like(x, device=DEV)
        ops.activation(x.to(DEV), out, kind)
        assert rel_err(out, ref) < tol(dt), kind
    inplace = x.to(DEV)
    ops.activation(inplace, inplace, "gelu")
    assert rel_err(inplace, want["gelu"]) < tol(dt)
    # the two gelu forms differ by more than the 32-bit tolerance: that run can tell them apart
    assert rel_err(want["gelu_tanh"], want["gelu"]) > 2 * tol(torch.float32)


@pytest.mark.parametrize("T, W", [(1, 48), (7, 336), (3, 4096), (2, 8192)])
@pytest.mark.parametrize("dt", DTYPES)
def test_norm_add_store(T, W, dt):
    y, x = _rand((T, W), 81, 2.0) + 0.5, _rand((T, W), 82)
    w = 1 + _rand((W,), 83, 0.2)
    xd, out = x.to(DEV), torch.empty((T, W), dtype=dt, device=DEV)
    ops.norm_add_store(y.to(DEV), w.to(DEV), None, 1e-5, False, xd, out)
    ref = x.double() + P.rms_norm(y, w, 1e-5)
    assert rel_err(xd, ref) < 2e-6
    assert rel_err(out, ref) < (1e-6 if dt == torch.float32 else 2.0 ** -8)
    # the same numbers as the norm that adds, then a cast
    x2 = x.to(DEV)
    ops.norm_rows(y.to(DEV), w.to(DEV), None, 1e-5, x2, False, add=True)
    assert torch.equal(x2, xd)
    if dt == torch.bfloat16:
        assert torch.equal(out, x2.to(torch.bfloat16))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("T, H, N, K", [(1, 3, 24, 8), (5, 1, 10, 70), (37, 6, 128, 64), (130, 2, 65, 129)])
def test_head_products(dt, T, H, N, K):
    """out[t, h] = W_h a[t, h], with a's heads inside wider rows, into wider rows, with and
    without a gate; a row alone gives the same bits as among the others."""
    a_hd, out_hd, a_off, out_off = K + 5, N + 3, 2, 1
    a = _rand((T, a_off + H * a_hd + 4), 1, 1.0, dt)
    w = _rand((H, N, K), 2, 1.0 / math.sqrt(K), dt)
    gate = _rand((T, H * N), 3, 1.5, dt)
    a64 = torch.stack([a[:, a_off + h * a_hd: a_off + h * a_hd + K] for h in range(H)], 1).double()
    ref = torch.einsum("thk,hnk->thn", a64, w.double())
    for g in (None, gate):
        out = torch.zeros((T, out_off + H * out_hd + 2), dtype=dt, device=DEV)
        ops.head_products(a.to(DEV), a_off, a_hd, w.to(DEV), None if g is None else g.to(DEV),
                          out, out_off, out_hd)
        got = torch.stack([out[:, out_off + h * out_hd: out_off + h * out_hd + N]
                           for h in range(H)], 1)
        want = ref if g is None else ref * torch.sigmoid(g.double()).view(T, H, N)
        assert rel_err(got, want) < tol(dt)
        assert float(out[:, :out_off].abs().max()) == 0.0          # nothing beside the heads
        one = torch.zeros((1, out.shape[1]), dtype=dt, device=DEV)
        ops.head_products(a[T // 2: T // 2 + 1].to(DEV), a_off, a_hd, w.to(DEV),
                          None if g is None else g[T // 2: T // 2 + 1].to(DEV), one, out_off, out_hd)
        assert torch.equal(one[0], out[T // 2])


@pytest.mark.parametrize("T, H, N, K", [(1, 3, 24, 16), (8, 32, 128, 128), (77, 6, 100, 48),
                                        (300, 2, 192, 160)])
def test_head_products_in_mfma_tiles(T, H, N, K):
    """bfloat16 with k a multiple of 16 and rows aligned to 16 bytes: the MFMA form; outputs
    that are no multiple of 32, tokens that are no multiple of 32, a gate, a row alone."""
    dt = torch.bfloat16
    a_hd, out_hd, a_off, out_off = K + 8, N + 3, 8, 1
    a = _rand((T, a_off + H * a_hd + 8), 1, 1.0, dt)
    w = _rand((H, N, K), 2, 1.0 / math.sqrt(K), dt)
    gate = _rand((T, H * N), 3, 1.5, dt)
    a64 = torch.stack([a[:, a_off + h * a_hd: a_off + h * a_hd + K] for h in range(H)], 1).double()
    ref = torch.einsum("thk,hnk->thn", a64, w.double())
    for g in (None, gate):
        out = torch.zeros((T, out_off + H * out_hd + 2), dtype=dt, device=DEV)
        ops.head_products(a.to(DEV), a_off, a_hd, w.to(DEV), None if g is None else g.to(DEV),
                          out, out_off, out_hd)
        got = torch.stack([out[:, out_off + h * out_hd: out_off + h * out_hd + N]
                           for h in range(H)], 1)
        want = ref if g is None else ref * torch.sigmoid(g.double()).view(T, H, N)
        assert rel_err(got, want) < tol(dt)
        assert float(out[:, :out_off].abs().max()) == 0.0
        assert float(out[:, out_off + H * out_hd:].abs().max()) == 0.0
        one = torch.zeros((1, out.shape[1]), dtype=dt, device=DEV)
        ops.head_products(a[T // 2: T // 2 + 1].to(DEV), a_off, a_hd, w.to(DEV),
                          None if g is None else g[T // 2: T // 2 + 1].to(DEV), one, out_off, out_hd)
        assert torch.equal(one[0], out[T // 2])


# ------------------------------------------------------------------------------ rows of a projection
# plain rows; pools in groups of 8; everything in groups of 8 (the kernel that moves 16 bytes)
@pytest.mark.parametrize("d, dv, dims", [(10, 7, 6), (16, 8, 8), (32, 16, 16)])
@pytest.mark.parametrize("dt", DTYPES)
def test_project_rows_norms_rotates_and_stores(dt, d, dv, dims):
    """Three segments of one product: queries (normed over all heads at once, the first 6 of
    10 elements of a head rotated) into rows, keys the same into pages, values as they are into
    pages of their own width; positions up to a few thousand."""
    T, H, G, ps = 9, 3, 2, 4
    src = _rand((T, H * d + G * d + G * dv + (8 if d == 32 else 5)), 1, 1.5, dt)
    gq, gk = 1 + _rand((H * d,), 2, 0.3), 1 + _rand((G * d,), 3, 0.3)
    freqs = P.wavelength_scaled_frequencies(50.0, dims, {"factor": 4.0, "low": 1.0, "high": 3.0,
                                                        "original": 20})
    pos = torch.tensor([0, 1, 2, 3, 50, 51, 4000, 9, 10])
    slots = torch.tensor([17, 3, 0, 5, 6, 30, 12, 9, 22])
    n_pages = 8
    q = torch.zeros((T, H * d), dtype=dt, device=DEV)
    kp = torch.zeros((n_pages, G * ps * d), dtype=dt, device=DEV)
    vp = torch.zeros((n_pages, G * ps * dv), dtype=dt, device=DEV)
    f32 = freqs.to(torch.float32).to(DEV)
    segs = [ops.RowSegment(0, H * d, q, gain=gq.to(DEV), eps=1e-5, hd=d, rot_dims=dims, freq=f32),
            ops.RowSegment(H * d, G * d, kp, gain=gk.to(DEV), eps=1e-5, hd=d, rot_dims=dims,
                           freq=f32, pool_heads=G),
            ops.RowSegment(H * d + G * d, G * dv, vp, hd=dv, pool_heads=G)]
    ops.project_rows(src.to(DEV), _i32(pos.tolist()), _i32(slots.tolist()), ps, segs)
    # the angle is a 32-bit product: at position 4000 it is right to 4000 * 2^-24 (2.4e-4)
    lim = max(tol(dt), 1e-3)
    want_q = P.rotate_leading(P.rms_norm(src[:, :H * d], gq, 1e-5).view(T, H, d), pos, freqs, dims)
    assert rel_err(q.view(T, H, d), want_q) < lim
    want_k = P.rotate_leading(P.rms_norm(src[:, H * d:H * d + G * d], gk, 1e-5).view(T, G, d),
                              pos, freqs, dims)
    got_k = ops.masked_pool_rows(kp, G, ps, d)[slots // ps, :, slots % ps]
    assert rel_err(got_k, want_k) < lim
    got_v = ops.masked_pool_rows(vp, G, ps, dv)[slots // ps, :, slots % ps]
    assert torch.equal(got_v.cpu(), src[:, H * d + G * d:H * d + G * d + G * dv].view(T, G, dv))
    # the elements behind the rotated ones pass through the norm alone
    assert rel_err(q.view(T, H, d)[..., dims:], want_q[..., dims:]) < tol(dt)
    # pages no token was written to stay as they were
    used = set((slots // ps).tolist())
    for p in range(n_pages):
        if p not in used:
            assert float(kp[p].abs().max()) == 0.0


# a pool row of 15: plain rows; of 16: groups of 8; everything in groups of 8
@pytest.mark.parametrize("rank_q, rank, dr, d, extra", [(9, 11, 4, 5, 3), (9, 12, 4, 5, 3),
                                                        (16, 24, 16, 8, 8)])
@pytest.mark.parametrize("dt", DTYPES)
def test_project_rows_latent_layout(dt, rank_q, rank, dr, d, extra):
    """A latent mixer's segments: the normed query latent into rows; the normed key latent and
    behind it the rotated shared part into one pool row; and of a query's heads the rotated
    part alone (``skip``), times a magnitude, behind the columns another kernel fills."""
    T, ps, H = 6, 4, 3
    src = _rand((T, rank_q + rank + dr + extra), 5, 1.2, dt)
    gq, gc = 1 + _rand((rank_q,), 6, 0.3), 1 + _rand((rank,), 7, 0.3)
    freqs, mag = P.yarn_frequencies(11.0, dr, {"factor": 2.0, "original": 8, "fast": 3.0, "slow": 0.5})
    f32 = freqs.to(torch.float32).to(DEV)
    pos = torch.tensor([0, 1, 2, 3, 4, 5])
    slots = torch.tensor([4, 5, 6, 7, 0, 1])
    cq = torch.zeros((T, rank_q), dtype=dt, device=DEV)
    pool = torch.zeros((3, ps * (rank + dr)), dtype=dt, device=DEV)
    ops.project_rows(src.to(DEV), _i32(pos.tolist()), _i32(slots.tolist()), ps, [
        ops.RowSegment(0, rank_q, cq, gain=gq.to(DEV), eps=1e-3),
        ops.RowSegment(rank_q, rank, pool, gain=gc.to(DEV), eps=1e-3, dst_hd=rank + dr, pool_heads=1),
        ops.RowSegment(rank_q + rank, dr, pool, rot_dims=dr, freq=f32, mag=mag, dst_off=rank,
                       dst_hd=rank + dr, pool_heads=1)])
    assert rel_err(cq, P.rms_norm(src[:, :rank_q], gq, 1e-3)) < tol(dt)
    rows = ops.masked_pool_rows(pool, 1, ps, rank + dr)[slots // ps, 0, slots % ps]
    assert rel_err(rows[:, :rank], P.rms_norm(src[:, rank_q:rank_q + rank], gc, 1e-3)) < tol(dt)
    want_r = P.rotate_leading(src[:, rank_q + rank:rank_q + rank + dr].view(T, 1, dr), pos, freqs, dr, mag)
    assert rel_err(rows[:, rank:], want_r.view(T, dr)) < tol(dt)
    q = _rand((T, H * (d + dr)), 8, 1.0, dt)
    qa = torch.full((T, H * (rank + dr)), 7.0, dtype=dt, device=DEV)
    ops.project_rows(q.to(DEV), _i32(pos.tolist()), None, ps, [
        ops.RowSegment(0, H * (d + dr), qa, hd=d + dr, rot_off=d, rot_dims=dr, freq=f32, mag=mag,
                       skip=d, dst_off=rank, dst_hd=rank + dr)])
    got = qa.view(T, H, rank + dr)
    want = P.rotate_leading(q.view(T, H, d + dr)[..., d:], pos, freqs, dr, mag)
    assert rel_err(got[..., rank:], want) < tol(dt)
    assert float((got[..., :rank] - 7.0).abs().max()) == 0.0


# ------------------------------------------------------------------------------ attention
class Paged:
    """Sequences of keys (and values) spread over shuffled pages of a pool."""

    def __init__(self, lens, G, KW, VW, ps, dt, seed, k=None, v=None):
        self.lens, self.G, self.KW, self.VW, self.ps = lens, G, KW, VW, ps
        g = torch.Generator().manual_seed(seed)
        n_pages = sum((n + ps - 1) // ps for n in lens) + 3
        order = torch.randperm(n_pages, generator=g).tolist()
        self.k = k if k is not None else [_rand((n, G, KW), seed + 10 + i, 1.0, dt) for i, n in enumerate(lens)]
        self.v = v if v is not None else ([_rand((n, G, VW), seed + 50 + i, 1.0, dt) for i, n in enumerate(lens)]
                                          if VW else None)
        kp = torch.full((n_pages, G, ps, KW), float("nan"), dtype=dt)
        vp = torch.full((n_pages, G, ps, max(VW, 1)), float("nan"), dtype=dt)
        width = max((n + ps - 1) // ps for n in lens)
        table = torch.full((len(lens), width), -1, dtype=torch.int32)
        for s, n in enumerate(lens):
            for i in range((n + ps - 1) // ps):
                page = order.pop()
                table[s, i] = page
                m = min(ps, n - i * ps)
                kp[page, :, :m] = self.k[s][i * ps:i * ps + m].transpose(0, 1)
                if VW:
                    vp[page, :, :m] = self.v[s][i * ps:i * ps + m].transpose(0, 1)
        # (the kernels' own layout inside a block)
        self.k_pool = ops.masked_pool_from_rows(kp).to(DEV)
        self.v_pool = ops.masked_pool_from_rows(vp).to(DEV) if VW else None
        self.table = table.to(DEV)


def _plain_attention(q, k, v, H, G, scale, cap, window, chunk, sink):
    """q [T, H, KW] the last T positions of a sequence of k [n, G, KW], v [n, G, VW]."""
    n, T = k.shape[0], q.shape[0]
    per = H // G
    mask = torch.ones((n, n), dtype=torch.bool).tril()
    if window:
        mask &= P.window_mask(n, window)
    if chunk:
        mask &= P.chunk_mask(n, chunk)
    kk = k.double().repeat_interleave(per, 1).permute(1, 0, 2)
    vv = v.double().repeat_interleave(per, 1).permute(1, 0, 2)
    qq = torch.zeros((H, n, q.shape[2]), dtype=torch.float64)
    qq[:, n - T:] = q.double().permute(1, 0, 2)
    s = P.tanh_cap(qq @ kk.transpose(1, 2) * scale, cap or None)
    return P.masked_softmax_values(s, mask, vv, sink)[:, n - T:].permute(1, 0, 2)    # [T, H, VW]


def _run(pg, qs, q_lens, dt, H, scale, cap=0.0, window=0, chunk=0, sink=None, gate=None,
         gate_mode=None, tied=None):
    T = sum(q_lens)
    q = torch.cat(qs).reshape(T, -1).to(DEV)
    VW = tied if tied else pg.VW
    out = torch.zeros((T, H * VW), dtype=dt, device=DEV)
    q_start = [0]
    for n in q_lens:
        q_start.append(q_start[-1] + n)
    seq_index = [s for s, n in enumerate(q_lens) for _ in range(n)]
    ops.masked_attention(q, None if gate is None else gate.to(DEV), gate_mode, pg.k_pool,
                         None if tied else pg.v_pool, None if sink is None else sink.to(DEV),
                         pg.table, _i32(q_start), _i32(pg.lens), _i32(seq_index), out, scale, cap,
                         window, chunk, H, pg.G, pg.KW, VW, pg.ps, max(pg.lens))
    return out


CASES = [  # H, G, KW, VW, page, lens, q_lens, cap, window, chunk
    (4, 2, 12, 20, 4, [23, 9, 1], [23, 9, 1], 4.0, 0, 7),
    (3, 3, 16, 16, 8, [70, 41], [13, 1], 0.0, 9, 0),
    (20, 1, 10, 6, 4, [17, 30], [17, 2], 8.0, 0, 1),
    (6, 2, 8, 12, 16, [150], [150], 2.5, 0, 1000),
    (2, 1, 40, 24, 16, [100, 65, 33], [1, 1, 1], 30.0, 0, 32),
    (5, 5, 96, 96, 16, [200], [60], 18.0, 37, 0),
    (2, 2, 7, 3, 2, [11], [11], 1.5, 3, 4),
]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
def test_attention_against_plain(dt, case):
    H, G, KW, VW, ps, lens, q_lens, cap, window, chunk = case
    pg = Paged(lens, G, KW, VW, ps, dt, 3)
    scale = 1.3 / math.sqrt(KW)
    sink = _rand((H,), 5, 1.5)
    T = sum(q_lens)
    qs = [_rand((n, H, KW), 20 + i, 1.0, dt) for i, n in enumerate(q_lens)]
    gate_h = _rand((T, H), 6, 1.5, dt)
    out = _run(pg, qs, q_lens, dt, H, scale, cap, window, chunk, sink, gate_h, "head")
    want = torch.cat([_plain_attention(q, pg.k[s], pg.v[s], H, G, scale, cap, window, chunk, sink)
                      for s, q in enumerate(qs)])
    want_g = want * torch.sigmoid(gate_h.double())[:, :, None]
    assert rel_err(out.view(T, H, VW), want_g) < 2 * tol(dt)
    # no sink, a gate an element
    gate_e = _rand((T, H * VW), 7, 1.5, dt)
    out = _run(pg, qs, q_lens, dt, H, scale, cap, window, chunk, None, gate_e, "element")
    want = torch.cat([_plain_attention(q, pg.k[s], pg.v[s], H, G, scale, cap, window, chunk, None)
                      for s, q in enumerate(qs)])
    assert rel_err(out.view(T, H, VW), want * torch.sigmoid(gate_e.double()).view(T, H, VW)) < 2 * tol(dt)
    # every sequence alone: the same bits as in the batch
    both = _run(pg, qs, q_lens, dt, H, scale, cap, window, chunk, sink)
    at = 0
    for s, n in enumerate(q_lens):
        one = Paged([lens[s]], G, KW, VW, ps, dt, 77 + s, k=[pg.k[s]], v=[pg.v[s]])
        alone = _run(one, [qs[s]], [n], dt, H, scale, cap, window, chunk, sink)
        assert torch.equal(alone, both[at:at + n])
        at += n


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H, KW, VW, ps, n, window", [(3, 28, 24, 4, 50, 5), (7, 13, 11, 16, 40, 1),
                                                       (4, 160, 128, 16, 90, 40), (2, 96, 48, 8, 300, 0),
                                                       (32, 576, 512, 16, 70, 0), (20, 1200, 8, 16, 40, 7)])
def test_values_that_are_the_keys_leading_columns(dt, H, KW, VW, ps, n, window):
    """No value pool: one kv head whose value is the first VW columns of its key row."""
    pg = Paged([n, 7], 1, KW, 0, ps, dt, 9)
    scale = 1.0 / math.sqrt(KW)
    qs = [_rand((n, H, KW), 30, 1.0, dt), _rand((1, H, KW), 31, 1.0, dt)]
    out = _run(pg, qs, [n, 1], dt, H, scale, 0.0, window, 0, tied=VW)
    want = torch.cat([_plain_attention(q, pg.k[s], pg.k[s][..., :VW], H, 1, scale, 0.0, window, 0, None)
                      for s, q in enumerate(qs)])
    assert rel_err(out.view(n + 1, H, VW), want) < 2 * tol(dt)


def _planted(n, G, KW, VW, at, dt, seed):
    """Keys and values of one sequence in which the key at ``at`` is 30 times louder than the
    rest along the query's direction, and its value stands out."""
    k = _rand((n, G, KW), seed, 0.3, dt)
    v = _rand((n, G, VW), seed + 1, 0.3, dt)
    k[at] = 0.0
    k[at, :, 0] = 30.0
    v[at] = 5.0
    return k, v


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("decode", [False, True])
def test_a_loud_key_at_the_edges(dt, decode):
    """A key that takes nearly all the weight when it is seen: far back without a mask; the
    oldest position a window holds and the one before it; the first position of the query's
    chunk and the last of the chunk before; position 0.  In a prompt's portion and for a token
    alone.  With a cap the loud score is bounded, and the sink takes the weight a shut-out key
    leaves."""
    H, G, KW, VW, ps, n = 2, 1, 16, 8, 8, 333
    qv = torch.zeros((H, KW))
    qv[:, 0] = 1.0
    T = 1 if decode else 37
    scale = 1.0
    for name, at, window, chunk, seen in (("far", 3, 0, 0, True), ("first", 0, 0, 0, True),
                                          ("window_in", n - 50, 50, 0, True),
                                          ("window_out", n - 51, 50, 0, False),
                                          ("chunk_in", 320, 0, 64, True),
                                          ("chunk_out", 319, 0, 64, False),
                                          ("page_border", 328, 5, 0, True)):
        k, v = _planted(n, G, KW, VW, at, dt, 40)
        pg = Paged([n], G, KW, VW, ps, dt, 11, k=[k], v=[v])
        q = qv.to(dt).expand(T, H, KW).contiguous()
        out = _run(pg, [q], [T], dt, H, scale, 0.0, window, chunk)
        last = out.view(T, H, VW)[-1].float().cpu()
        if seen:
            assert float((last - 5.0).abs().max()) < 0.05, name
        else:
            assert float(last.abs().max()) < 1.5, name
        want = _plain_attention(q, k, v, H, G, scale, 0.0, window, chunk, None)
        assert rel_err(out.view(T, H, VW), want) < 2 * tol(dt), name
    # capped at 2, the loud key's weight is e^2 against 332 keys of about e^0: not dominant;
    # and a sink of 12 takes nearly everything
    k, v = _planted(n, G, KW, VW, 100, dt, 41)
    pg = Paged([n], G, KW, VW, ps, dt, 12, k=[k], v=[v])
    q = qv.to(dt).expand(T, H, KW).contiguous()
    capped = _run(pg, [q], [T], dt, H, scale, 2.0).view(T, H, VW)[-1].float().cpu()
    assert float(capped.abs().max()) < 1.0
    assert rel_err(_run(pg, [q], [T], dt, H, scale, 2.0).view(T, H, VW),
                   _plain_attention(q, k, v, H, G, scale, 2.0, 0, 0, None)) < 2 * tol(dt)
    sunk = _run(pg, [q], [T], dt, H, 0.2, 0.0, sink=torch.tensor([12.0, -12.0]))
    sunk = sunk.view(T, H, VW)[-1].float().cpu()
    assert float(sunk[0].abs().max()) < 0.1 and float(sunk[1].abs().max()) > 0.5


def test_pages_before_the_mask_are_not_touched():
    """Table entries before a window or a chunk are -1 (the cache manager has taken the pages
    back): the kernel never looks them up."""
    H, G, KW, VW, ps, n = 2, 2, 8, 8, 4, 61
    for window, chunk in ((9, 0), (0, 16)):
        pg = Paged([n], G, KW, VW, ps, torch.float32, 13)
        q = _rand((5, H, KW), 1)
        full = _run(pg, [q], [5], torch.float32, H, 0.4, 0.0, window, chunk)
        first = (n - 5 - window + 1 if window else (n - 5) // chunk * chunk) // ps
        assert first > 2
        pg.table[0, :first] = -1
        assert torch.equal(_run(pg, [q], [5], torch.float32, H, 0.4, 0.0, window, chunk), full)


# ------------------------------------------------------------------------------ the MFMA form
def _run_mfma(pg, qs, q_lens, H, scale, cap=0.0, window=0, chunk=0, sink=None, gate=None,
              gate_mode=None, tied=None, n_splits=None):
    dt = torch.bfloat16
    T = sum(q_lens)
    q = torch.cat(qs).reshape(T, -1).to(DEV)
    VW = tied if tied else pg.VW
    out = torch.zeros((T, H * VW), dtype=dt, device=DEV)
    q_start = [0]
    for n in q_lens:
        q_start.append(q_start[-1] + n)
    ops.masked_attention_mfma(q, None if gate is None else gate.to(DEV), gate_mode, pg.k_pool,
                              None if tied else pg.v_pool, None if sink is None else sink.to(DEV),
                              pg.table, _i32(q_start), _i32(pg.lens), out, scale, cap, window,
                              chunk, H, pg.G, pg.KW, VW, pg.ps, max(q_lens), max(pg.lens),
                              n_splits=n_splits)
    return out


MFMA_CASES = [  # H, G, KW, VW, tied, page, lens, q_lens, cap, window, chunk
    (6, 3, 96, 96, False, 16, [230, 90, 33], [230, 90, 33], 12.0, 0, 100),
    (8, 8, 64, 64, False, 16, [300, 41], [77, 2], 0.0, 100, 0),
    (32, 1, 128, 128, False, 16, [150], [150], 5.0, 0, 1000),
    (5, 1, 160, 128, True, 16, [200, 64], [200, 10], 0.0, 50, 0),
    (3, 1, 96, 64, True, 8, [333], [333], 0.0, 0, 0),
    (16, 1, 192, 128, True, 16, [500], [100], 0.0, 256, 0),
    (12, 4, 128, 128, False, 32, [700], [700], 30.0, 0, 0),
]


@pytest.mark.parametrize("case", MFMA_CASES)
def test_mfma_attention_against_plain(case):
    H, G, KW, VW, tied, ps, lens, q_lens, cap, window, chunk = case
    dt = torch.bfloat16
    pg = Paged(lens, G, KW, 0 if tied else VW, ps, dt, 3)
    scale = 1.3 / math.sqrt(KW)
    sink = None if tied else _rand((H,), 5, 1.5)
    T = sum(q_lens)
    qs = [_rand((n, H, KW), 20 + i, 1.0, dt) for i, n in enumerate(q_lens)]
    gate = _rand((T, H * VW), 7, 1.5, dt) if tied else _rand((T, H), 6, 1.5, dt)
    mode = "element" if tied else "head"
    vals = [k[..., :VW] for k in pg.k] if tied else pg.v
    want = torch.cat([_plain_attention(q, pg.k[s], vals[s], H, G, scale, cap, window, chunk, sink)
                      for s, q in enumerate(qs)])
    g64 = torch.sigmoid(gate.double())
    want_g = want * (g64.view(T, H, VW) if tied else g64[:, :, None])
    assert ops.masked_attention_mfma_covers(dt, H, G, KW, VW, tied)
    for parts in (None, 1, 2, 4):
        out = _run_mfma(pg, qs, q_lens, H, scale, cap, window, chunk, sink, gate, mode,
                        tied=VW if tied else None, n_splits=parts)
        assert rel_err(out.view(T, H, VW), want_g) < 2 * tol(dt), parts
    # the 32-bit kernel on the same operands agrees
    ref = _run(pg, qs, q_lens, dt, H, scale, cap, window, chunk, sink, gate, mode,
               tied=VW if tied else None)
    assert rel_err(out, ref.double()) < 2 * tol(dt)


@pytest.mark.parametrize("case", MFMA_CASES)
def test_mfma_decode_steps_against_plain(case):
    """One token a sequence, the contexts split over 1, 2 and 5 workgroups of four waves."""
    H, G, KW, VW, tied, ps, lens, _, cap, window, chunk = case
    dt = torch.bfloat16
    lens = lens + [1, 31, 32, 33]
    pg = Paged(lens, G, KW, 0 if tied else VW, ps, dt, 4)
    scale = 1.1 / math.sqrt(KW)
    sink = None if tied else _rand((H,), 5, 1.5)
    n = len(lens)
    qs = [_rand((1, H, KW), 60 + i, 1.0, dt) for i in range(n)]
    gate = _rand((n, H * VW), 7, 1.5, dt) if tied else _rand((n, H), 6, 1.5, dt)
    mode = "element" if tied else "head"
    vals = [k[..., :VW] for k in pg.k] if tied else pg.v
    want = torch.cat([_plain_attention(q, pg.k[s], vals[s], H, G, scale, cap, window, chunk, sink)
                      for s, q in enumerate(qs)])
    g64 = torch.sigmoid(gate.double())
    want_g = want * (g64.view(n, H, VW) if tied else g64[:, :, None])
    for blocks in (None, 1, 2, 5):
        out = _run_mfma(pg, qs, [1] * n, H, scale, cap, window, chunk, sink, gate, mode,
                        tied=VW if tied else None, n_splits=blocks)
        assert rel_err(out.view(n, H, VW), want_g) < 2 * tol(dt), blocks


@pytest.mark.parametrize("decode", [False, True])
def test_mfma_a_loud_key_at_the_edges(decode):
    dt = torch.bfloat16
    H, G, KW, VW, ps, n = 2, 1, 64, 64, 16, 333
    qv = torch.zeros((H, KW))
    qv[:, 0] = 1.0
    T = 1 if decode else 37
    for name, at, window, chunk, seen in (("far", 3, 0, 0, True), ("first", 0, 0, 0, True),
                                          ("window_in", n - 50, 50, 0, True),
                                          ("window_out", n - 51, 50, 0, False),
                                          ("chunk_in", 320, 0, 64, True),
                                          ("chunk_out", 319, 0, 64, False),
                                          ("page_border", 320, 13, 0, True),
                                          ("split_border", 256, 0, 0, True)):
        k, v = _planted(n, G, KW, VW, at, dt, 40)
        pg = Paged([n], G, KW, VW, ps, dt, 11, k=[k], v=[v])
        q = qv.to(dt).expand(T, H, KW).contiguous()
        for splits in (None, 3):
            out = _run_mfma(pg, [q], [T], H, 1.0, 0.0, window, chunk, n_splits=splits)
            last = out.view(T, H, VW)[-1].float().cpu()
            if seen:
                assert float((last - 5.0).abs().max()) < 0.05, name
            else:
                assert float(last.abs().max()) < 1.5, name
            want = _plain_attention(q, k, v, H, G, 1.0, 0.0, window, chunk, None)
            assert rel_err(out.view(T, H, VW), want) < 2 * tol(dt), name


def test_mfma_pages_before_the_mask_are_not_touched():
    H, G, KW, VW, ps, n = 4, 2, 64, 64, 16, 301
    dt = torch.bfloat16
    for window, chunk in ((40, 0), (0, 64)):
        for T in (1, 45):
            pg = Paged([n], G, KW, VW, ps, dt, 13)
            q = _rand((T, H, KW), 1, 1.0, dt)
            full = _run_mfma(pg, [q], [T], H, 0.2, 0.0, window, chunk)
            first = (n - T - window + 1 if window else (n - T) // chunk * chunk) // ps
            assert first > 2
            pg.table[0, :first] = -1
            assert torch.equal(_run_mfma(pg, [q], [T], H, 0.2, 0.0, window, chunk), full)
