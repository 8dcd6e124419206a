"""Gosuvik's mechanisms one by one, each kernel against a slow float64 function written from the equations (here or in
`plain_gosuvik.py`): the norm in groups, the PolyNorm activation, the weighted sum of two branches, the gate; the step
after the q|k|v product with norms per head, a partial rotation and rotated values; attention with a sink, a window,
values of another size and the result turned back (one key made to stand out just inside and just outside the window, at
page borders, far back; a sink that outweighs every key); attention over the compressed cache with a window (plain and
on the matrix cores, portions and single tokens); the delta rule with a decay per key channel (row by row and in
chunks, carried over steps and slots); the matrix memory with exponential gates."""
import math

import numpy as np
import pytest
import torch

import plain_gosuvik as pg

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F = torch.float64


def rnd(shape, seed, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def step_rows(lengths, slots):
    from inferx_amd import ops
    q_start = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    seq = np.repeat(np.arange(len(lengths)), lengths).astype(np.int32)
    return ops.StepRows(torch.from_numpy(seq).to(DEV), torch.from_numpy(q_start).to(DEV),
                        torch.tensor(slots, dtype=torch.int32, device=DEV))


# ---- small kernels ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("width,groups", [(96, 2), (72, 3), (40, 1), (128, 4), (30, 5), (256, 256)])
def test_norm_in_groups(width, groups, dtype, tol):
    """h += delta and the norm of every run of the width by its own root mean square; with picked rows h stays."""
    from inferx_amd import ops
    T = 9
    h, delta, w = rnd((T, width), 1, 3.0), rnd((T, width), 2, 1.0, dtype), rnd((width,), 3, 1.0, dtype) + 1.0
    hd, out = h.to(DEV), torch.empty(T, width, dtype=dtype, device=DEV)
    ops.add_rmsnorm(hd, delta.to(DEV), w.to(DEV), out, 1e-5, None, groups)
    total = h.double() + delta.double()
    want = pg.group_norm(total, w.double(), 1e-5, groups)
    assert float((hd.cpu().double() - total).abs().max()) <= 1e-6 * float(total.abs().max())
    assert float((out.cpu().double() - want).abs().max()) <= tol * float(want.abs().max())
    rows = torch.tensor([4, 0, 4], dtype=torch.int32, device=DEV)
    picked = torch.empty(3, width, dtype=dtype, device=DEV)
    before = hd.clone()
    ops.add_rmsnorm(hd, None, w.to(DEV), picked, 1e-5, rows, groups)
    assert torch.equal(hd, before)
    assert float((picked.cpu().double() - want[[4, 0, 4]]).abs().max()) <= tol * float(want.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,groups", [(96, 2), (72, 3), (128, 4), (30, 5)])
def test_experts_sum_rides_on_the_norm_in_groups(width, groups, dtype):
    """The experts' weighted sum, the residual add and the norm in groups in one launch against the three one by one."""
    from inferx_amd import ops
    T, k = 7, 3
    y, w = rnd((T * k + 2, width), 11, 1.0, dtype).to(DEV), (rnd((width,), 12, 0.3, dtype) + 1.0).to(DEV)
    dest = torch.randperm(T * k + 2, generator=torch.Generator().manual_seed(3))[:T * k].to(torch.int32).to(DEV)
    topk_w = torch.rand(T, k, generator=torch.Generator().manual_seed(4)).to(DEV)
    for rows in (None, torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)):
        h1, h2 = rnd((T, width), 13, 2.0).to(DEV), rnd((T, width), 13, 2.0).to(DEV)
        n = T if rows is None else 3
        one, three = torch.empty(n, width, dtype=dtype, device=DEV), torch.empty(n, width, dtype=dtype, device=DEV)
        ops.moe_combine_add_rmsnorm(h1, y, dest, topk_w, None, None, w, one, 1e-5, rows, groups=groups)
        total = torch.zeros(T, width, dtype=torch.float32, device=DEV)
        for s in range(k):
            total += topk_w[:, s:s + 1] * y[dest.view(T, k)[:, s].long()].float()
        ops.add_rmsnorm(h2, total, w, three, 1e-5, rows, groups)
        assert float((h1 - h2).abs().max()) <= 1e-5 * float(h2.abs().max())
        tol = 1e-5 if dtype == torch.float32 else 1e-2
        assert float((one.float() - three.float()).abs().max()) <= tol * float(three.float().abs().max())


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("width", [24, 320, 4100])
def test_polynorm_sum_and_gate(width, dtype, tol):
    from inferx_amd import ops
    z, coef = rnd((5, width), 4, 1.5, dtype), torch.tensor([0.7, -0.4, 0.2, 0.1])
    out = torch.empty(5, width, dtype=dtype, device=DEV)
    ops.polynorm(z.to(DEV), coef.to(DEV), out, 1e-5)
    zd = z.double()
    want = 0.7 * pg.rms_unit(zd, 1e-5) - 0.4 * pg.rms_unit(zd ** 2, 1e-5) + 0.2 * pg.rms_unit(zd ** 3, 1e-5) + 0.1
    assert float((out.cpu().double() - want).abs().max()) <= tol * float(want.abs().max())
    a, b = rnd((5, width), 5, 1.0, dtype), rnd((5, width), 6, 1.0, dtype)
    total = torch.empty(5, width, dtype=torch.float32, device=DEV)
    ops.weighted_sum(a.to(DEV), 0.6, b.to(DEV), -1.3, total)
    assert float((total.cpu().double() - (0.6 * a.double() - 1.3 * b.double())).abs().max()) <= 1e-6 * 5
    ops.weighted_sum(a.to(DEV), 0.25, None, 0.0, total)
    assert float((total.cpu().double() - 0.25 * a.double()).abs().max()) <= 1e-6
    wide = rnd((5, width + 8), 7, 2.0, dtype).to(DEV)  # the gate's rows are a view into a wider product
    y = a.to(DEV).clone()
    ops.sigmoid_gate(y, wide[:, 8:])
    want = a.double() * torch.sigmoid(wide[:, 8:].cpu().double())
    assert float((y.cpu().double() - want).abs().max()) <= tol * float(want.abs().max())


# ---- attention with a sink, a window and rotated values ----------------------------------------------------------------------
class PagedKV:
    """Requests with contexts in paged key and value caches whose pages are dealt out of order; pages that a window
    has passed may be taken away (their table entries become -1 and their contents not-a-number)."""

    def __init__(self, contexts, kv_heads, dim, vdim, page_size, dtype, seed):
        self.page_size = page_size
        pages_of = [-(-n // page_size) for n in contexts]
        total = sum(pages_of) + 3
        order = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
        self.k = torch.full((total, kv_heads, page_size, dim), float("nan"), dtype=dtype)
        self.v = torch.full((total, kv_heads, vdim, page_size), float("nan"), dtype=dtype)
        self.table = torch.full((len(contexts), max(pages_of)), -1, dtype=torch.int32)
        self.keys, self.values = [], []
        for i, n in enumerate(contexts):
            keys, values = rnd((n, kv_heads, dim), seed + 10 + i, 1.0, dtype), rnd((n, kv_heads, vdim), seed + 50 + i, 1.0, dtype)
            self.keys.append(keys)
            self.values.append(values)
            for p in range(pages_of[i]):
                page = order.pop()
                self.table[i, p] = page
                part = slice(p * page_size, min((p + 1) * page_size, n))
                self.k[page, :, :part.stop - part.start] = keys[part].transpose(0, 1)
                self.v[page, :, :, :part.stop - part.start] = values[part].permute(1, 2, 0)

    def give_back(self, request, before):
        """The pages that hold only keys before position `before` are gone."""
        for p in range(before // self.page_size):
            page = int(self.table[request, p])
            self.k[page], self.v[page] = float("nan"), float("nan")
            self.table[request, p] = -1


def plain_sink_attention(q, keys, values, pos, scale, window, sink, angles):
    """q [H, d] at position pos over keys [n, G, d], values [n, G, vd]: softmax with exp(sink) in the denominator
    over the keys pos - window < j <= pos; the result turned back by `angles` [vd / 2] (halves paired)."""
    H, G = q.shape[0], keys.shape[1]
    lo = max(0, pos + 1 - window) if window else 0
    out = torch.zeros(H, values.shape[2], dtype=F)
    for h in range(H):
        g = h // (H // G)
        s = keys[lo:pos + 1, g] @ q[h] * scale
        top = max(float(s.max()), float(sink[h])) if sink is not None else float(s.max())
        e = torch.exp(s - top)
        below = e.sum() + (math.exp(float(sink[h]) - top) if sink is not None else 0.0)
        out[h] = (e / below) @ values[lo:pos + 1, g]
    if angles is not None:
        out = pg.rotate_halves(out[None], -angles[None])[0]
    return out


def run_sink_attention(paged, lengths, contexts, H, scale, window, sink, turn, dtype, standout=None, q_scale=1.0,
                       mfma=False, splits=1, grouped=False):
    """The last lengths[i] positions of request i as one step's rows through `ops.attention_plain` (or, `mfma`, the
    wavefront-level matrix-core kernel in tiles of 16 queries, the keys in `splits` slices); the kernel's result and
    the float64 one.  standout = (request, key): the request's queries are made to match that key."""
    from inferx_amd import ops
    G, d, vd = paged.keys[0].shape[1], paged.keys[0].shape[2], paged.values[0].shape[2]
    T = sum(lengths)
    seq = np.repeat(np.arange(len(lengths)), lengths).astype(np.int32)
    pos = np.concatenate([np.arange(c - n, c) for c, n in zip(contexts, lengths)]).astype(np.int32)
    q = rnd((T, H, d), 91, q_scale, dtype)
    if standout is not None:
        i, key = standout
        for t in np.nonzero(seq == i)[0]:
            for h in range(H):
                direction = paged.keys[i][key, h // (H // G)].float()
                q[t, h] += (14.0 / scale * direction / direction.norm() ** 2).to(dtype)
    angles = None
    if turn:
        freq = 100.0 ** (-2.0 * torch.arange(vd // 2, dtype=F) / vd)
        angles = torch.from_numpy(pos).double()[:, None] * freq[None, :]
        table = torch.stack([torch.cos(angles), torch.sin(angles)], dim=-1).float().contiguous().to(DEV)
    out = torch.empty(T, H, vd, dtype=dtype, device=DEV)
    if mfma:
        tiles, at = [], 0
        for i, n in enumerate(lengths):
            tiles += [(i, at + first, min(1 if grouped else 16, n - first)) for first in range(0, n, 1 if grouped else 16)]
            at += n
        tiles = torch.tensor(tiles, dtype=torch.int32).t().contiguous().to(DEV)
        work = torch.empty(T * H * splits * (d + 2), dtype=torch.float32, device=DEV) if splits > 1 else None
        ops.attention_mfma(q.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), tiles,
                           torch.from_numpy(pos).to(DEV), out, splits, work, scale, window, 16, prefetch=splits > 1,
                           grouped=grouped, sink=None if sink is None else sink.to(DEV), turn_back=table if turn else None)
    else:
        ops.attention_plain(q.to(DEV), paged.k.to(DEV), paged.v.to(DEV), paged.table.to(DEV), torch.from_numpy(seq).to(DEV),
                            torch.from_numpy(pos).to(DEV), out, scale, window, None if sink is None else sink.to(DEV),
                            table if turn else None)
    want = torch.zeros(T, H, vd, dtype=F)
    for t in range(T):
        i = int(seq[t])
        want[t] = plain_sink_attention(q[t].double(), paged.keys[i].double(), paged.values[i].double(), int(pos[t]), scale,
                                       window, None if sink is None else sink.double(), None if angles is None else angles[t])
    return out.cpu().double(), want


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,G,d,vd,page,window", [(4, 2, 16, 24, 16, 9), (3, 3, 10, 6, 8, 0), (6, 1, 64, 64, 16, 80),
                                                   (2, 1, 32, 48, 48, 33), (1, 1, 8, 8, 16, 1)])
def test_attention_with_sink_window_and_values_turned_back(H, G, d, vd, page, window, dtype, tol):
    """Unequal requests in one step: portions (one from position 0), a single token between them; then single tokens.
    Pages that the windows have passed are gone (their contents not-a-number)."""
    contexts = [70, 33, 1, 150, 48]
    sink = rnd((H,), 12, 1.5)
    for lengths in ([70, 20, 1, 9, 16], [1, 1, 1, 1, 1]):
        paged = PagedKV(contexts, G, d, vd, page, dtype, seed=3)
        if window:
            for i, (c, n) in enumerate(zip(contexts, lengths)):
                paged.give_back(i, max(0, c - n + 1 - window))
        for use_sink, turn in ((True, vd % 2 == 0), (False, False)):
            got, want = run_sink_attention(paged, lengths, contexts, H, d ** -0.5, window, sink if use_sink else None,
                                           turn, dtype)
            assert torch.isfinite(got).all()
            assert float((got - want).abs().max()) <= tol * float(want.abs().max()), f"{lengths} sink {use_sink}"


@pytest.mark.parametrize("H,G,d,page,window", [(4, 2, 32, 16, 9), (8, 2, 64, 16, 72), (16, 1, 128, 32, 40), (3, 3, 96, 16, 0),
                                                (2, 1, 48, 48, 33)])
def test_attention_with_sink_on_the_matrix_cores(H, G, d, page, window):
    """The wavefront-level matrix-core kernel with a sink and the result turned back (heads of a multiple of 32; of 48:
    the sink alone): portions in tiles of sixteen queries, single tokens with their keys in slices, single tokens with
    the query heads of a key/value head side by side."""
    contexts = [70, 33, 1, 150, 48]
    sink = rnd((H,), 12, 1.5)
    turn = d % 32 == 0
    for lengths, splits, grouped in (([70, 20, 1, 9, 16], 1, False), ([1, 1, 1, 1, 1], 4, False), ([1, 1, 1, 1, 1], 2, H // G > 1),
                                     ([3, 1, 1, 2, 1], 1, False)):
        paged = PagedKV(contexts, G, d, d, page, torch.bfloat16, seed=3)
        if window:
            for i, (c, n) in enumerate(zip(contexts, lengths)):
                paged.give_back(i, max(0, c - n + 1 - window))
        for use_sink in (True, False):
            got, want = run_sink_attention(paged, lengths, contexts, H, d ** -0.5, window, sink if use_sink else None,
                                           turn, torch.bfloat16, mfma=True, splits=splits, grouped=grouped)
            assert torch.isfinite(got).all()
            assert float((got - want).abs().max()) <= 2e-2 * float(want.abs().max()), f"{lengths} {splits} sink {use_sink}"


@pytest.mark.parametrize("mfma", [False, True])
@pytest.mark.parametrize("window", [40, 72])
@pytest.mark.parametrize("back", [0, 1, 15, 16, 17, "in", "out", "far"])
def test_one_key_that_stands_out_at_the_windows_edge(window, back, mfma):
    """600 keys; the queries match ONE key strongly.  The key lies `back` places behind the last query: the query's own
    place, the one before, around a page's border, the last place inside the window ("in"), the first outside ("out") and
    far outside.  Inside, the result is that key's value (turned by the distance); outside, the key must not count."""
    n, H, G, d, vd = 600, 4, 2, 32, (32 if mfma else 16)
    distance = {"in": window - 1, "out": window, "far": 400}.get(back, back)
    key = n - 1 - distance
    paged = PagedKV([n], G, d, vd, 16, torch.bfloat16, seed=21)
    sink = torch.full((H,), -2.0)
    for lengths in ([1], [24]):
        got, want = run_sink_attention(paged, lengths, [n], H, 0.25, window, sink, True, torch.bfloat16,
                                       standout=(0, key), q_scale=0.2, mfma=mfma, splits=4 if mfma and lengths == [1] else 1)
        last_got, last_want = got[-1], want[-1]
        peak = float(paged.values[0][key].double().abs().max())
        if distance < window:  # nearly all the weight is on the key: the result has its value's size
            assert float(last_want.abs().max()) > 0.5 * peak, "the test's key does not stand out"
        assert float((got - want).abs().max()) <= 2e-2 * float(want.abs().max()), f"key {distance} back, window {window}"
        assert float((last_got - last_want).abs().max()) <= 2e-2 * float(last_want.abs().max())


def test_a_sink_that_outweighs_every_key():
    """With a large sink the weights of all keys together are small: the result shrinks by the sink's share exactly."""
    paged = PagedKV([50], 1, 16, 16, 16, torch.float32, seed=31)
    for value in (8.0, 30.0):
        got, want = run_sink_attention(paged, [5], [50], 2, 0.25, 0, torch.full((2,), value), False, torch.float32)
        without, _ = run_sink_attention(paged, [5], [50], 2, 0.25, 0, None, False, torch.float32)
        assert float(want.abs().max()) < 0.5 * float(without.abs().max())
        assert float((got - want).abs().max()) <= 2e-5 * float(want.abs().max())


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("H,G,d,vd,begin,half", [(4, 2, 16, 24, 0, 4), (3, 3, 10, 6, 0, 5), (8, 1, 64, 64, 0, 8), (2, 1, 12, 8, 4, 2)])
def test_step_after_the_product_norms_rotation_and_rotated_values(H, G, d, vd, begin, half, dtype, tol):
    """q and k normed per head and rotated over a part of the head, v rotated over all of it, k and v in their pages."""
    from inferx_amd import ops
    T, page, pages = 13, 8, 6
    width = (H + G) * d + G * vd
    qkv = rnd((T, width + 8), 41, 1.0, dtype)[:, :width + 8]
    wq, wk = rnd((d,), 42, 0.3, dtype) + 1.0, rnd((d,), 43, 0.3, dtype) + 1.0
    pos = torch.arange(T) + 3
    ang = pos.double()[:, None] * (50.0 ** (-2.0 * torch.arange(half, dtype=F) / (2 * half)))[None, :]
    vang = pos.double()[:, None] * (50.0 ** (-2.0 * torch.arange(vd // 2, dtype=F) / vd))[None, :]
    table = lambda a: torch.stack([torch.cos(a), torch.sin(a)], dim=-1).float().contiguous().to(DEV)
    slots = torch.randperm(page * pages, generator=torch.Generator().manual_seed(5))[:T].to(torch.int32)
    q_out = torch.empty(T, H, d, dtype=dtype, device=DEV)
    k_cache = torch.zeros(pages, G, page, d, dtype=dtype, device=DEV)
    v_cache = torch.zeros(pages, G, vd, page, dtype=dtype, device=DEV)
    ops.qkv_norm_rope_append(qkv.to(DEV)[:, :width], wq.to(DEV), wk.to(DEV), 1e-5, table(ang), begin, table(vang),
                             slots.to(DEV), q_out, k_cache, v_cache, H, G, d, vd)
    x = qkv.double()
    q = pg.rms_unit(x[:, :H * d].view(T, H, d), 1e-5) * wq.double()
    k = pg.rms_unit(x[:, H * d:(H + G) * d].view(T, G, d), 1e-5) * wk.double()
    v = x[:, (H + G) * d:width].view(T, G, vd)
    turn = lambda t: torch.cat([t[..., :begin], pg.rotate_halves(t[..., begin:begin + 2 * half], ang), t[..., begin + 2 * half:]], dim=-1)
    q, k, v = turn(q), turn(k), pg.rotate_halves(v, vang)
    assert float((q_out.cpu().double() - q).abs().max()) <= tol * float(q.abs().max())
    for t in range(T):
        p, o = int(slots[t]) // page, int(slots[t]) % page
        assert float((k_cache[p, :, o].cpu().double() - k[t]).abs().max()) <= tol * float(k.abs().max())
        assert float((v_cache[p, :, :, o].cpu().double() - v[t]).abs().max()) <= tol * float(v.abs().max())


# ---- attention over the compressed cache, with a window ----------------------------------------------------------------------
def plain_latent(q_lat, q_rot, rows, pos, scale, window):
    rank = q_lat.shape[1]
    lo = max(0, pos + 1 - window) if window else 0
    s = (q_lat @ rows[lo:pos + 1, :rank].T + q_rot @ rows[lo:pos + 1, rank:].T) * scale
    return torch.softmax(s, dim=1) @ rows[lo:pos + 1, :rank]


def run_latent(contexts, lengths, H, rank, rot, page, window, dtype, mfma, standout=None):
    from inferx_amd import ops
    width = rank + rot
    pages_of = [-(-n // page) for n in contexts]
    total = sum(pages_of) + 2
    order = torch.randperm(total, generator=torch.Generator().manual_seed(7)).tolist()
    cache = torch.full((total, 1, page, width), float("nan"), dtype=dtype)
    table = torch.full((len(contexts), max(pages_of)), -1, dtype=torch.int32)
    rows = [rnd((n, width), 60 + i, 1.0, dtype) for i, n in enumerate(contexts)]
    for i, (n, length) in enumerate(zip(contexts, lengths)):
        gone = max(0, n - length + 1 - window) // page if window else 0  # pages that the window has passed are gone
        for p in range(gone, pages_of[i]):
            table[i, p] = order.pop()
            part = rows[i][p * page:(p + 1) * page]
            cache[table[i, p], 0, :part.shape[0]] = part
    T = sum(lengths)
    seq = np.repeat(np.arange(len(lengths)), lengths).astype(np.int32)
    pos = np.concatenate([np.arange(c - n, c) for c, n in zip(contexts, lengths)]).astype(np.int32)
    q_lat, q_rot = rnd((T, H, rank), 77, 0.3, dtype), rnd((T, H, rot), 78, 0.3, dtype)
    if standout is not None:
        i, key = standout
        direction = rows[i][key, :rank].float()
        for t in np.nonzero(seq == i)[0]:
            q_lat[t] += (12.0 / 0.1 * direction / direction.norm() ** 2).to(dtype)
    one_each = all(n == 1 for n in lengths)
    out = torch.empty(T, H, rank, dtype=dtype, device=DEV)
    args = (q_lat.to(DEV), q_rot.to(DEV), cache.to(DEV), table.to(DEV), torch.from_numpy(seq).to(DEV), torch.from_numpy(pos).to(DEV))
    if mfma:
        assert ops.latent_mfma_fits(args[0], args[1], out, rank, rot)
        splits, work = 1, None
        if one_each:
            splits = ops.latent_mfma_splits(T, H)
            work = (torch.empty(T * H * splits, rank, dtype=torch.float32, device=DEV),
                    torch.empty(T * H * splits, 2, dtype=torch.float32, device=DEV))
        ops.latent_attention_mfma(*args, out, rank, rot, 0.1, one_each, splits, work, window)
    else:
        ops.latent_attention_plain(*args, out, rank, rot, 0.1, window)
    want = torch.stack([plain_latent(q_lat[t].double(), q_rot[t].double(), rows[int(seq[t])].double(), int(pos[t]), 0.1, window)
                        for t in range(T)])
    return out.cpu().double(), want, rows


@pytest.mark.parametrize("mfma", [False, True])
@pytest.mark.parametrize("window", [0, 1, 20, 33, 80])
def test_latent_attention_with_a_window(mfma, window):
    contexts = [70, 33, 1, 150, 48]
    dtype = torch.bfloat16 if mfma else torch.float32
    for H, rank, rot, page in [(3, 64, 32, 16), (16, 96, 64, 16)] if mfma else [(3, 40, 8, 16), (2, 24, 10, 8)]:
        for lengths in ([70, 20, 1, 9, 16], [1, 1, 1, 1, 1], [3, 1, 1, 2, 1]):
            got, want, _ = run_latent(contexts, lengths, H, rank, rot, page, window, dtype, mfma)
            assert torch.isfinite(got).all()
            err = float((got - want).abs().max()) / float(want.abs().max())
            assert err <= (2e-2 if mfma else 1e-5), f"window {window} {lengths}: {err:.2e}"


@pytest.mark.parametrize("mfma", [False, True])
@pytest.mark.parametrize("distance", [0, 1, 31, 32, 63, 64, 79, 80, 81, 500])
def test_latent_key_that_stands_out_at_the_windows_edge(mfma, distance):
    """A window of 80 over 1,000 rows; one row takes nearly all the weight if it is visible: the query's own, a round's
    and a page's borders, the last inside the window (79), the first outside (80)."""
    n, window = 1000, 80
    for lengths in ([1], [40]):
        got, want, rows = run_latent([n], lengths, 4, 64, 32, 16, window, torch.bfloat16, mfma, standout=(0, n - 1 - distance))
        if distance < window:
            c = rows[0][n - 1 - distance, :64].double()
            assert float((want[-1] - c).abs().max()) < 0.2 * float(c.abs().max()), "the test's key does not stand out"
        assert float((got - want).abs().max()) <= 2e-2 * float(want.abs().max())


# ---- the delta rule with a decay per key channel ------------------------------------------------------------------------------
def plain_channel_delta(q, k, v, b, a, a_log, dt_bias, state, G):
    """q, k [T, G, d] as the convolution leaves them, v [T, H, vd], b [T, H], a [T, H, d]; state [H, d, vd] in place."""
    T, H, vd = v.shape
    d = q.shape[2]
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    out = torch.zeros(T, H, vd, dtype=F)
    for t in range(T):
        for h in range(H):
            g = torch.exp(-math.exp(float(a_log[h])) * pg.softplus(a[t, h] + dt_bias[h]))
            S = g[:, None] * state[h]
            u = torch.sigmoid(b[t, h]) * (v[t, h] - S.T @ k[t, h // (H // G)])
            S = S + torch.outer(k[t, h // (H // G)], u)
            state[h] = S
            out[t, h] = S.T @ q[t, h // (H // G)]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,vd", [(4, 2, 16, 12), (1, 1, 20, 9), (2, 1, 64, 40), (1, 1, 128, 32), (4, 4, 32, 16), (3, 1, 192, 8)])
def test_channel_delta_over_steps_and_slots(H, G, d, vd, dtype):
    """Three requests in slots that are not in order: a step of unequal portions (several chunks, a chunk's edge, one
    row), steps of one row each, a portion of two rows, then portions around a chunk's length: outputs and the state
    that is left against the float64 loop over the rows."""
    from inferx_amd import ops
    steps = [(33, 16, 1), (1, 1, 1), (1, 1, 1), (2, 17, 5), (70, 32, 31)]
    slots = [4, 0, 2]
    state = torch.zeros(6, H * d * vd + 5, dtype=torch.float32, device=DEV)
    state[1] = float("nan")  # a slot nobody owns
    own = [torch.zeros(H, d, vd, dtype=F) for _ in slots]
    a_log, dt_bias = rnd((H,), 81, 0.5), rnd((H * d,), 82, 0.5)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for n, lengths in enumerate(steps):
        T = sum(lengths)
        q, k = rnd((T, G * d), 100 + n, 1.0, dtype), rnd((T, G * d), 200 + n, 1.0, dtype)
        v, b, a = rnd((T, H * vd), 300 + n, 1.0, dtype), rnd((T, H), 400 + n, 1.0), rnd((T, H * d), 500 + n, 1.5)
        out = torch.empty(T, H, vd, dtype=torch.float32, device=DEV)
        decays = a.to(DEV)
        ops.channel_decays(decays, a_log.to(DEV), dt_bias.to(DEV), H, d)
        ops.delta_rule(q.to(DEV), k.to(DEV), v.to(DEV), b.to(DEV), a_log.to(DEV), dt_bias.to(DEV),
                       state[:, :H * d * vd], step_rows(lengths, slots), out, H, G, d, vd, decays)
        at = 0
        for i, length in enumerate(lengths):
            r = slice(at, at + length)
            want = plain_channel_delta(q[r].double().view(-1, G, d), k[r].double().view(-1, G, d), v[r].double().view(-1, H, vd),
                                       b[r].double(), a[r].double().view(-1, H, d), a_log.double(), dt_bias.double().view(H, d), own[i], G)
            err = float((out[r].cpu().double() - want).abs().max()) / max(float(want.abs().max()), 1e-3)
            assert err <= tol, f"step {n} request {i}: {err:.2e}"
            at += length
    for i, slot in enumerate(slots):  # the state lies [head][column][row]
        left = state[slot, :H * d * vd].view(H, vd, d).transpose(1, 2).cpu().double()
        assert float((left - own[i]).abs().max()) <= tol * max(float(own[i].abs().max()), 1e-3)
    assert torch.isnan(state[1]).all() and float(state[3].abs().max()) == 0.0


def test_a_key_written_once_is_read_back_much_later():
    """Decays of nearly one, a key and value written at the first token with a step size of nearly one, 300 tokens of
    other keys (orthogonal to it) one by one: a query for that key at the end reads its value back."""
    from inferx_amd import ops
    H, d, vd, n = 1, 32, 16, 300
    state = torch.zeros(1, d * vd, dtype=torch.float32, device=DEV)
    a_log, dt_bias = torch.zeros(1), torch.full((d,), -12.0)  # softplus(-12) = 6e-6: the decay is 1 - 6e-6
    decays = torch.zeros(1, d, device=DEV)
    ops.channel_decays(decays, a_log.to(DEV), dt_bias.to(DEV), 1, d)
    first = torch.zeros(d)
    first[0] = 1.0
    value = rnd((vd,), 5)
    for t in range(n):
        key = first if t in (0, n - 1) else torch.cat([torch.zeros(1), rnd((d - 1,), 600 + t)])
        v = value if t == 0 else (torch.zeros(vd) if t == n - 1 else rnd((vd,), 900 + t))
        b = torch.tensor([[20.0 if t == 0 else (-20.0 if t == n - 1 else 0.0)]])  # the last token writes nothing
        out = torch.empty(1, 1, vd, dtype=torch.float32, device=DEV)
        ops.delta_rule(key[None].to(DEV), key[None].to(DEV), v[None].to(DEV), b.to(DEV), a_log.to(DEV), dt_bias.to(DEV),
                       state, step_rows([1], [0]), out, H, 1, d, vd, decays)
    want = value.double() * d ** -0.5
    assert float((out.cpu().double().flatten() - want).abs().max()) <= 5e-3 * float(want.abs().max())


# ---- the matrix memory -----------------------------------------------------------------------------------------------------------
def plain_memory(q, k, v, gates, bias, cap, S, nvec, top):
    """q, k [T, H, d], v [T, H, vd], gates [T, 2H]; S [H, d, vd], nvec [H, d], top [H] in place."""
    T, H, d = q.shape
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for t in range(T):
        for h in range(H):
            gi = cap * math.tanh((float(gates[t, h]) + float(bias[h])) / cap)
            y = cap * math.tanh((float(gates[t, H + h]) + float(bias[H + h])) / cap)
            gf = min(y, 0.0) - math.log1p(math.exp(-abs(y)))
            new = max(gf + float(top[h]), gi)
            keep, take = math.exp(gf + float(top[h]) - new), math.exp(gi - new)
            S[h] = keep * S[h] + take * torch.outer(k[t, h], v[t, h])
            nvec[h] = keep * nvec[h] + take * k[t, h]
            top[h] = new
            qs = q[t, h] * d ** -0.5
            out[t, h] = S[h].T @ qs / (max(abs(float(nvec[h] @ qs)), math.exp(-new)) + 1e-6)
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,vd,cap", [(2, 12, 20, 8.0), (1, 20, 7, 3.0), (2, 64, 40, 10.0), (1, 128, 16, 30.0), (3, 32, 33, 1.0),
                                        (2, 128, 128, 15.0)])
def test_matrix_memory_over_steps_and_slots(H, d, vd, cap, dtype):
    """Three requests in slots that are not in order: unequal portions (several chunks of the recurrence, more than
    one round of the gates' scan, a chunk's edge, one row), single rows, two rows: read-outs and the state that is left
    against the float64 loop over the rows.  The division rides on the norm's kernel and is checked through it."""
    from inferx_amd import ops
    steps = [(33, 16, 1), (1, 1, 1), (1, 1, 1), (2, 17, 5), (70, 1, 31), (130, 64, 65)]
    slots = [4, 0, 2]
    floats = ops.matrix_memory_state_floats(H, d, vd)
    assert floats == H * d * (vd + 1) + H
    state = torch.zeros(6, floats + 3, dtype=torch.float32, device=DEV)
    state[1] = float("nan")
    own = [(torch.zeros(H, d, vd, dtype=F), torch.zeros(H, d, dtype=F), torch.zeros(H, dtype=F)) for _ in slots]
    bias = torch.cat([rnd((H,), 71, 1.0), rnd((H,), 72, 1.0) + 2.0])
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for n, lengths in enumerate(steps):
        T = sum(lengths)
        q, k, v = rnd((T, H * d), 100 + n, 1.0, dtype), rnd((T, H * d), 200 + n, 1.0, dtype), rnd((T, H * vd), 300 + n, 1.0, dtype)
        gates = rnd((T, 2 * H), 400 + n, 3.0)
        out, nq = torch.empty(T, H, vd, dtype=torch.float32, device=DEV), torch.empty(T, H, dtype=torch.float32, device=DEV)
        work = torch.empty(T, H, 3, dtype=torch.float32, device=DEV)
        ops.matrix_memory(q.to(DEV), k.to(DEV), v.to(DEV), gates.to(DEV), bias.to(DEV), cap, state[:, :floats],
                          step_rows(lengths, slots), out, nq, work, H, d, vd)
        read = out / (torch.maximum(nq.abs(), work[:, :, 2]) + 1e-6)[:, :, None]
        normed = torch.empty(T, H * vd, dtype=dtype, device=DEV)
        ops.head_norm_gate(out, normed, 1e-5, den_a=nq, den_b=work[:, :, 2])
        at = 0
        for i, length in enumerate(lengths):
            r = slice(at, at + length)
            want = plain_memory(q[r].double().view(-1, H, d), k[r].double().view(-1, H, d), v[r].double().view(-1, H, vd),
                                gates[r].double(), bias.double(), cap, *own[i])
            err = float((read[r].cpu().double() - want).abs().max()) / max(float(want.abs().max()), 1e-3)
            assert err <= tol, f"step {n} request {i}: {err:.2e}"
            unit = pg.rms_unit(want, 1e-5)
            err = float((normed[r].cpu().double().view(-1, H, vd) - unit).abs().max()) / float(unit.abs().max())
            assert err <= max(tol, 1e-2 if dtype == torch.bfloat16 else 0), f"step {n} request {i} normed: {err:.2e}"
            at += length
    for i, slot in enumerate(slots):  # per head [column][row] with n as the last column, then the maxima
        matrices = state[slot, :H * d * (vd + 1)].view(H, vd + 1, d).cpu().double()
        S, nvec = matrices[:, :vd].transpose(1, 2), matrices[:, vd]
        top = state[slot, H * d * (vd + 1):floats].cpu().double()
        assert float((S - own[i][0]).abs().max()) <= tol * max(float(own[i][0].abs().max()), 1e-3)
        assert float((nvec - own[i][1]).abs().max()) <= tol * max(float(own[i][1].abs().max()), 1e-3)
        assert float((top - own[i][2]).abs().max()) <= 1e-4 * max(float(own[i][2].abs().max()), 1.0)
    assert torch.isnan(state[1]).all() and float(state[3].abs().max()) == 0.0
