"""Bibevik's mechanisms one by one, each kernel against a slow float64 function written from the equations (here
or in `plain_bibevik.py`): the recurrence with a matrix of state (per token and in chunks, with and without the
correction, carried over steps and slots), attention over the compressed cache (plain and on the matrix cores, for
prompt portions, mixed steps and single tokens whose keys are cut into slices; one key made to stand out far back, at a
page border and at the last visible place), the router with groups scored by their two best, the clamped gated unit,
the norm with one number."""
import math

import numpy as np
import pytest
import torch

import plain_bibevik as pb

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(shape, seed, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


# ---- the recurrence ---------------------------------------------------------------------------------------------------
def plain_recurrence(r, k, v, w, a, b, state):
    """S <- diag(w_t) S - a_t (b_t^T S) + k_t v_t^T; o_t = S^T r_t, float64.  r, k, w, a, b [T, H, D]; v [T, H, V];
    state [H, D, V] (changed in place)."""
    T, H, _ = r.shape
    out = torch.zeros(T, H, v.shape[2], dtype=torch.float64)
    for t in range(T):
        for h in range(H):
            S = state[h]
            read = b[t, h] @ S
            S = w[t, h][:, None] * S - torch.outer(a[t, h], read) + torch.outer(k[t, h], v[t, h])
            state[h] = S
            out[t, h] = S.T @ r[t, h]
    return out


def step_rows(lengths, slots):
    from inferx_amd import ops
    q_start = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    seq = np.repeat(np.arange(len(lengths)), lengths).astype(np.int32)
    return ops.StepRows(torch.from_numpy(seq).to(DEV), torch.from_numpy(q_start).to(DEV),
                        torch.tensor(slots, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("corrected", [True, False])
@pytest.mark.parametrize("H,D,V", [(2, 16, 24), (3, 20, 12), (1, 32, 40), (2, 64, 64), (2, 128, 80), (1, 192, 16), (32, 128, 128)])
def test_recurrence_over_steps_and_slots(H, D, V, corrected, dtype):
    """Three requests in slots that are not in order: a step of unequal portions (several chunks, a chunk's edge, one
    row), then steps of one row each, then a portion of two rows, then portions around the longest chunk's length:
    outputs and the state that is left against the float64 loop over the rows."""
    from inferx_amd import ops
    silu = not corrected
    steps = [(33, 16, 1), (1, 1, 1), (1, 1, 1), (2, 17, 5)]
    if H <= 3:  # portions longer than the longest chunk: two whole chunks and two rows, a whole chunk, a chunk and a row
        steps.append((130, 64, 65))
    slots = [4, 0, 2]
    state = torch.zeros(6, H * D * V + 8, dtype=torch.float32, device=DEV)
    state[1] = float("nan")  # a slot that nobody owns
    plain_state = [torch.zeros(H, D, V, dtype=torch.float64) for _ in slots]
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    for n, lengths in enumerate(steps):
        T = sum(lengths)
        r, k = rnd((T, H * D), 10 * n + 1, 0.7, dtype), rnd((T, H * D), 10 * n + 2, 0.7, dtype)
        v = rnd((T, H * V), 10 * n + 3, 1.0, dtype)
        if corrected:
            w = torch.exp(-0.6 * torch.sigmoid(rnd((T, H * D), 10 * n + 4)))
            u = rnd((T, H, D), 10 * n + 5)
            u = (u / u.norm(dim=2, keepdim=True)).reshape(T, H * D).contiguous()
            a = (u * torch.sigmoid(rnd((T, H * D), 10 * n + 6))).contiguous()
            w_head = None
        else:
            w_head = torch.tensor(([0.97, 0.6, 1.0] * H)[:H], dtype=torch.float32)
        out = torch.empty(T, H, V, dtype=torch.float32, device=DEV)
        ops.linear_state(r.to(DEV), k.to(DEV), v.to(DEV), state, step_rows(lengths, slots), out, H, D, V,
                         w_rows=w.to(DEV) if corrected else None, w_head=None if corrected else w_head.to(DEV),
                         a_rows=a.to(DEV) if corrected else None, b_rows=u.to(DEV) if corrected else None, silu=silu)
        act = (lambda x: x * torch.sigmoid(x)) if silu else (lambda x: x)
        r64, k64, v64 = (act(x.double()) for x in (r, k, v))
        at = 0
        for i, L in enumerate(lengths):
            rows = slice(at, at + L)
            if corrected:
                w64, a64, b64 = (x.double()[rows].view(L, H, D) for x in (w, a, u))
            else:
                w64 = w_head.double()[None, :, None].expand(L, H, D)
                a64 = b64 = torch.zeros(L, H, D, dtype=torch.float64)
            want = plain_recurrence(r64[rows].view(L, H, D), k64[rows].view(L, H, D), v64[rows].view(L, H, V), w64, a64,
                                    b64, plain_state[i])
            got = out[rows].cpu().double()
            scale = float(want.abs().max()) + 1e-9
            assert float((got - want).abs().max()) <= tol * scale, f"step {n} request {i}"
            at += L
    for i, slot in enumerate(slots):  # the state is kept [head][column][row]
        got = state[slot, :H * D * V].cpu().double().view(H, V, D).transpose(1, 2)
        scale = float(plain_state[i].abs().max())
        assert float((got - plain_state[i]).abs().max()) <= tol * scale
    assert bool(torch.isnan(state[1]).all()), "a slot of no request was written"


def test_delta_operands_and_the_plain_mixer_agree():
    """decay, removal and unit key as the kernel makes them against the plain mixer's formulas."""
    from inferx_amd import ops
    T, H, D = 7, 3, 20
    wl, al, k = rnd((T, H * D), 1, 2.0), rnd((T, H * D), 2, 2.0), rnd((T, H * D), 3)
    w0, ab = rnd((H * D,), 4), rnd((H * D,), 5)
    w, a, u = (torch.empty(T, H * D, dtype=torch.float32, device=DEV) for _ in range(3))
    ops.delta_operands(wl.to(DEV), w0.to(DEV), al.to(DEV), ab.to(DEV), k.to(DEV), w, a, u, H, D, math.exp(-0.5), 1e-6)
    k3 = k.double().view(T, H, D)
    unit = (k3 / torch.sqrt((k3 * k3).sum(dim=2, keepdim=True) + 1e-6)).view(T, H * D)
    assert torch.allclose(w.cpu().double(), torch.exp(-math.exp(-0.5) * torch.sigmoid(wl.double() + w0.double())), atol=1e-6)
    assert torch.allclose(u.cpu().double(), unit, atol=1e-6)
    assert torch.allclose(a.cpu().double(), unit * torch.sigmoid(al.double() + ab.double()), atol=1e-6)


# ---- attention over the compressed cache ------------------------------------------------------------------------------
def plain_latent_scores(q_lat, q_rot, rows, positions, scale):
    """out[t, h] = softmax over j <= pos(t) of (q_lat[t, h] . c[j] + q_rot[t, h] . kr[j]) * scale, times c; float64.
    rows [n, rank + rot] are the request's cached rows."""
    rank = q_lat.shape[2]
    c, kr = rows[:, :rank], rows[:, rank:]
    out = torch.zeros_like(q_lat)
    for t, p in enumerate(positions):
        s = (q_lat[t] @ c[:p + 1].T + q_rot[t] @ kr[:p + 1].T) * scale
        out[t] = torch.softmax(s, dim=1) @ c[:p + 1]
    return out


class Paged:
    """Requests with contexts in a paged cache whose pages are dealt out of order."""

    def __init__(self, contexts, width, page_size, dtype, seed):
        self.page_size, self.width = page_size, width
        pages_of = [-(-n // page_size) for n in contexts]
        total = sum(pages_of) + 3
        order = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
        self.cache = torch.full((total, 1, page_size, width), float("nan"), dtype=dtype)
        self.table = torch.zeros(len(contexts), max(pages_of), dtype=torch.int32)
        self.rows = []
        for i, n in enumerate(contexts):
            rows = rnd((n, width), seed + 10 + i, 1.0, dtype)
            self.rows.append(rows)
            for p in range(pages_of[i]):
                page = order.pop()
                self.table[i, p] = page
                part = rows[p * page_size:(p + 1) * page_size]
                self.cache[page, 0, :part.shape[0]] = part


def run_latent(paged, lengths, contexts, H, rank, rot, scale, dtype, mfma, q_scale=1.0, standout=None):
    """The last `lengths[i]` positions of request i (its context is contexts[i]) as one step's rows; returns the
    kernel's result and the float64 one, [T, H, rank] each.  standout = (request, key): that key's row and every
    query of the request are made to match, so that this key takes nearly all the weight."""
    from inferx_amd import ops
    T = sum(lengths)
    seq = np.repeat(np.arange(len(lengths)), lengths).astype(np.int32)
    pos = np.concatenate([np.arange(c - n, c) for c, n in zip(contexts, lengths)]).astype(np.int32)
    q_lat, q_rot = rnd((T, H, rank), 77, q_scale, dtype), rnd((T, H, max(rot, 8)), 78, q_scale, dtype)[:, :, :rot]
    if standout is not None:
        i, key = standout
        direction = paged.rows[i][key].float()
        direction = direction / direction.norm()
        for t in np.nonzero(seq == i)[0]:
            q_lat[t] += (12.0 / scale * direction[:rank] / direction.norm()).to(dtype)
    full = torch.zeros(T, H, rank + 64, dtype=dtype)  # queries as views with strides, as the mixer hands them over
    full[:, :, :rank] = q_lat
    dq = full.to(DEV)
    qr = q_rot.contiguous().to(DEV)
    out = torch.empty(H, T, rank, dtype=dtype, device=DEV).transpose(0, 1)
    one_each = all(n == 1 for n in lengths)
    args = (dq[:, :, :rank], qr, paged.cache.to(DEV), paged.table.to(DEV), torch.from_numpy(seq).to(DEV),
            torch.from_numpy(pos).to(DEV))
    if mfma:
        assert ops.latent_mfma_fits(dq[:, :, :rank], qr, out, rank, rot)
        splits, work = 1, None
        if one_each:
            out = torch.empty(T, H, rank, dtype=dtype, device=DEV)
            splits = ops.latent_mfma_splits(T, H)
            work = (torch.empty(T * H * splits, rank, dtype=torch.float32, device=DEV),
                    torch.empty(T * H * splits, 2, dtype=torch.float32, device=DEV))
        ops.latent_attention_mfma(*args, out, rank, rot, scale, one_each, splits, work)
    else:
        ops.latent_attention_plain(*args, out, rank, rot, scale)
    want = torch.zeros(T, H, rank, dtype=torch.float64)
    at = 0
    for i, n in enumerate(lengths):
        rows = slice(at, at + n)
        want[rows] = plain_latent_scores(q_lat[rows].double(), q_rot[rows].double(), paged.rows[i].double(),
                                         pos[rows].tolist(), scale)
        at += n
    return out.cpu().double(), want


SIZES = [(2, 64, 32, 16), (5, 96, 64, 8), (16, 128, 64, 16), (3, 256, 64, 48), (4, 512, 64, 16), (70, 32, 32, 16)]


@pytest.mark.parametrize("H,rank,rot,page", SIZES)
def test_latent_attention_on_the_matrix_cores(H, rank, rot, page):
    """Prompt portions of unequal requests in one step (one of them from position 0, one row alone between two
    portions, a portion that ends on a tile's edge), then one token per request with the keys cut into slices."""
    contexts = [70, 33, 1, 150, 48]
    paged = Paged(contexts, rank + rot, page, torch.bfloat16, seed=3)
    scale = (rank + rot) ** -0.5
    for lengths in ([70, 20, 1, 9, 16], [1, 1, 1, 1, 1], [3, 1, 1, 2, 1]):
        got, want = run_latent(paged, lengths, contexts, H, rank, rot, scale, torch.bfloat16, True)
        err = float((got - want).abs().max()) / float(want.abs().max())
        assert err <= 2e-2, f"{lengths}: {err:.2e}"


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_latent_attention_plain_kernel(dtype, tol):
    contexts = [40, 300, 7]
    for H, rank, rot, page in [(3, 40, 8, 16), (2, 24, 0, 8), (1, 64, 32, 48)]:
        paged = Paged(contexts, rank + rot, page, dtype, seed=5)
        for lengths in ([40, 5, 1], [1, 1, 1]):
            got, want = run_latent(paged, lengths, contexts, H, rank, rot, 0.2, dtype, False)
            assert float((got - want).abs().max()) <= tol * float(want.abs().max())


@pytest.mark.parametrize("mfma", [False, True])
@pytest.mark.parametrize("key", [0, 15, 16, 255, 256, 600, 1021, 1022])
def test_one_key_that_stands_out(mfma, key):
    """1,023 keys of which one takes nearly all the weight: the first, the last two, both sides of a page's and of a
    slice's border, one far back.  The queries: a portion of 40 rows, then the last token alone (slices of its keys)."""
    H, rank, rot, page = 4, 64, 32, 16
    n = 1023
    paged = Paged([n], rank + rot, page, torch.bfloat16, seed=9)
    for lengths in ([40], [1]):
        got, want = run_latent(paged, lengths, [n], H, rank, rot, 0.1, torch.bfloat16, mfma, q_scale=0.2, standout=(0, key))
        visible = [t for t in range(lengths[0]) if n - lengths[0] + t >= key]
        assert visible
        c = paged.rows[0][key, :rank].double()
        for t in visible:  # the result is that key's latent, nearly
            assert float((want[t] - c).abs().max()) < 0.2 * float(c.abs().max()), "the test's key does not stand out"
        assert float((got - want).abs().max()) <= 2e-2 * float(want.abs().max())


# ---- router, gated unit, norm -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("E,top,groups,keep", [(8, 2, 2, 1), (6, 2, 3, 2), (16, 4, 8, 3), (5, 1, 1, 1), (12, 3, 4, 4), (6, 2, 6, 3)])
def test_router_with_groups_scored_by_their_two_best(E, top, groups, keep):
    from inferx_amd import ops
    T, W = 37, 48
    x, w = rnd((T, W), 1), rnd((E, W), 2, 0.5)
    topk_w = torch.empty(T, top, dtype=torch.float32, device=DEV)
    topk_e = torch.empty(T, top, dtype=torch.int32, device=DEV)
    ops.moe_route(x.to(DEV), w.to(DEV), None, topk_w, topk_e, None, False, 2.5, 0, groups, keep, True, True)
    scores = torch.sigmoid(x.double() @ w.double().T)
    want = pb.choose_experts(scores, top, groups, keep)
    for t in range(T):
        assert set(topk_e[t].tolist()) == set(want[t].tolist()), f"token {t}"
        for e, wt in zip(topk_e[t].tolist(), topk_w[t].tolist()):
            assert abs(wt - 2.5 * float(scores[t, e])) < 1e-5


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("limit", [0.7, 7.0])
def test_clamped_gated_unit_with_biases(dtype, tol, limit):
    from inferx_amd import ops
    T, n = 9, 40
    gate_up, bias = rnd((T, 2 * n), 1, 3.0, dtype), rnd((2 * n,), 2, 1.0, dtype)
    act = torch.empty(T, n, dtype=dtype, device=DEV)
    ops.glu_bias(gate_up.to(DEV), bias.to(DEV), act, limit)
    z = gate_up.double() + bias.double()
    g, u = z[:, :n].clamp(max=limit), z[:, n:].clamp(-limit, limit)
    want = g * torch.sigmoid(1.702 * g) * (u + 1)
    assert float((act.cpu().double() - want).abs().max()) <= tol * float(want.abs().max())


def test_norm_with_one_number():
    x = rnd((5, 24), 1).double()
    g = torch.tensor(1.3, dtype=torch.float64)
    want = x / torch.sqrt((x * x).mean(dim=1, keepdim=True) + 1e-5) * g
    assert torch.allclose(pb.scalar_norm(x, g, 1e-5), want)
    from inferx_amd import ops
    out = torch.empty(5, 24, dtype=torch.float32, device=DEV)
    h = x.float().to(DEV)
    ops.add_rmsnorm(h, None, torch.full((24,), 1.3, dtype=torch.float32, device=DEV), out, 1e-5, None)
    assert torch.allclose(out.cpu().double(), want, atol=1e-5)
