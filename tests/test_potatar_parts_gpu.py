"""Each mechanism of the Potatar layers alone: the kernel against the plain implementation's function of the same
mechanism (or a few lines of 64-bit torch), in float32 and bfloat16, with its rows cut into steps, its requests in
scattered slots and pages, and inputs made so that a wrong key or a lost state shows."""
import math

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import potatar_plain as N

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    from qwen_engine_amd.kernels import ops as o
    return o


def rel(got, want):
    return float((got.double().cpu() - want.double()).abs().max()) / max(float(want.abs().max()), 1e-30)


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


# ---- the norm after the sum ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,W,alpha", [(1, 80, 1.7), (9, 200, 2.25), (70, 1024, 1.0), (3, 4100, 0.3)])
@pytest.mark.parametrize("ddtype", [torch.float32, torch.bfloat16])
def test_norm_after_the_sum(T, W, alpha, ddtype):
    g = torch.Generator().manual_seed(T + W)
    x, d = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g).to(ddtype)
    w = 1.0 + 0.3 * torch.randn(W, generator=g)
    want = N.rms_norm(alpha * x.double() + d.double(), w.double(), 1e-5)
    xs = x.to(DEV)
    act = ops().postnorm(xs, d.to(DEV), alpha, w.to(DEV), 1e-5, act_dtype=torch.bfloat16)
    assert rel(xs, want) < 3e-6
    assert torch.equal(act.cpu(), xs.cpu().to(torch.bfloat16))


# ---- activations, the soft cap, the weighted sum -------------------------------------------------------------------
def test_activations_between_products_and_the_soft_cap():
    z = torch.linspace(-9, 9, 1001)
    o = ops()
    assert rel(o.unary(z.to(DEV), o.UNARY_GELU), N.gelu_erf(z.double())) < 2e-6
    assert rel(o.unary(z.to(DEV), o.UNARY_TANH), torch.tanh(z.double())) < 2e-6
    for cap in (1.0, 12.0, 40.0):
        assert rel(o.unary((5 * z).to(DEV), o.UNARY_SOFTCAP, cap=cap), cap * torch.tanh(5 * z.double() / cap)) < 2e-6
    zb = z.to(torch.bfloat16)
    got = o.unary(zb.to(DEV), o.UNARY_GELU)
    assert got.dtype == torch.bfloat16 and rel(got, N.gelu_erf(zb.double())) < 5e-3
    a, b = torch.randn(5, 33), torch.randn(5, 33)
    assert rel(o.scaled_sum(a.to(DEV), 1.2, b.to(DEV), -0.7), 1.2 * a.double() - 0.7 * b.double()) < 1e-6


# ---- q, k, v: norms, values from keys, blended values, rotation, cache write -----------------------------------------
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 5e-5), (torch.bfloat16, 6e-3)])      # (angles are 32-bit)
@pytest.mark.parametrize("hq,hkv,dk,dv,dims,norm,from_keys,blend", [
    (4, 2, 12, 20, 4, "whole", False, "source"), (6, 2, 8, 20, 8, "whole", False, "blend"),
    (3, 3, 10, 6, 0, "whole", False, None), (6, 3, 8, 8, 0, "head", True, None),
    (8, 2, 64, 64, 32, "whole", False, "blend"), (16, 1, 16, 16, 8, "head", True, None),
    (2, 2, 128, 32, 128, "whole", False, "source"), (1, 1, 6, 6, 6, None, False, None)])
def test_norms_values_rotation_and_cache_write(dtype, tol, hq, hkv, dk, dv, dims, norm, from_keys, blend):
    o = ops()
    g = torch.Generator().manual_seed(hq * 10 + dk)
    T, P, pages, eps, base = 23, 8, 9, 1e-5, 500.0
    dc = (max(dk, dv) + 3) // 4 * 4
    n_in = hq * dk + hkv * dk + (0 if from_keys else hkv * dv)
    qkv = (torch.randn(T, n_in, generator=g) * 1.5).to(dtype)
    pos = torch.randint(0, 900, (T,), generator=g)
    slots = torch.randperm(pages * P, generator=g)[:T]
    slots[5] = -1                                             # (a row that is written nowhere)
    nq, nk = (hq * dk, hkv * dk) if norm == "whole" else (dk, dk)
    qw, kw = 1 + 0.3 * torch.randn(nq, generator=g), 1 + 0.3 * torch.randn(nk, generator=g)
    lam = torch.tensor([0.37])
    vf = torch.randn(T, hkv * dv, generator=g)
    x = qkv.double()
    q, k = x[:, :hq * dk], x[:, hq * dk:(hq + hkv) * dk]
    v = k.reshape(T, hkv, dk) if from_keys else x[:, (hq + hkv) * dk:].reshape(T, hkv, dv)
    if norm == "whole":
        q, k = N.rms_norm(q, qw.double(), eps), N.rms_norm(k, kw.double(), eps)
    q, k = q.reshape(T, hq, dk), k.reshape(T, hkv, dk)
    if norm == "head":
        q, k = N.rms_norm(q, qw.double(), eps), N.rms_norm(k, kw.double(), eps)
    if dims:
        q, k = N.rotate_half_split(q, pos, base, dims), N.rotate_half_split(k, pos, base, dims)
    if not from_keys:
        v = N.rms(v, eps)
    want_first = v.reshape(T, hkv * dv)
    if blend == "blend":
        v = (1 - lam.double()) * v + lam.double() * vf.double().reshape(T, hkv, dv)
    inv = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64).float().to(DEV) if dims else None
    for value_rows in (True, False):
        if not value_rows and P % 8:
            continue
        cache = torch.full((pages, 2, hkv, P, dc), float("nan"), dtype=dtype, device=DEV)
        v_first = None
        if blend == "source":
            v_first = torch.full((T, hkv * dv), float("nan"), device=DEV)
        elif blend == "blend":
            v_first = vf.to(DEV)
        got_q = o.qkv_norm_store(qkv.to(DEV), hq, hkv, dk, dv, cache, slots.to(torch.int32).to(DEV),
                                 qk_norm={None: o.QK_NORM_NONE, "head": o.QK_NORM_HEAD, "whole": o.QK_NORM_WHOLE}[norm],
                                 q_weight=qw.to(DEV) if norm else None, k_weight=kw.to(DEV) if norm else None, qk_eps=eps,
                                 values_from_keys=from_keys, value_norm_eps=None if from_keys else eps, v_first=v_first,
                                 v_blend=lam.to(DEV) if blend == "blend" else None, positions=pos.to(torch.int32).to(DEV),
                                 inv_freq=inv, value_rows=value_rows)
        assert rel(got_q[:, :, :dk], q) < tol
        if blend == "source":
            assert rel(v_first, want_first) < 3e-6              # (left in 32-bit for the later layers)
        c = cache.cpu().double()
        for t in range(T):
            s = int(slots[t])
            if s < 0:
                continue
            pg, off = s // P, s % P
            assert rel(c[pg, 0, :, off, :dk], k[t]) < tol
            vt = c[pg, 1, :, off, :dv] if value_rows else c[pg, 1].reshape(hkv, dc, P)[:, :dv, off]
            assert rel(vt, v[t]) < tol
        written = {int(s) for s in slots if s >= 0}
        for s in range(pages * P):
            if s not in written:
                assert torch.isnan(c[s // P, 0, :, s % P]).all()


# ---- the bias by distance as one row per distance --------------------------------------------------------------------
@pytest.mark.parametrize("rows,far", [(2, 2), (10, 30), (14, 100.5), (32, 1024), (33, 1000), (9, 64)])
def test_bias_rows_by_distance(rows, far):
    from qwen_engine_amd.parts.attention import distance_bias_rows
    table = torch.arange(rows * 3, dtype=torch.float32).reshape(rows, 3)
    got = distance_bias_rows(table, far)
    for n in range(got.shape[0]):
        assert torch.equal(got[n], table[N.distance_bucket(n, rows, far)]), n
    assert torch.equal(got[-1], table[-1])
    for n in (got.shape[0], 3 * got.shape[0], 100000):           # (beyond the last row: the table's last)
        assert N.distance_bucket(n, rows, far) == rows - 1
    short = distance_bias_rows(table, far, max_distance=3)        # (a chunk of four positions: distances 0 to 3)
    assert torch.equal(short, got[:4]) if got.shape[0] > 4 else torch.equal(short, got)
    assert torch.equal(distance_bias_rows(table, 1e9, max_distance=50)[50], table[N.distance_bucket(50, rows, 1e9)])


# ---- attention whose heads talk, inside chunks, over pages ---------------------------------------------------------
def _paged(k, v, P, pages, g, dtype, dc, start=0):
    """Keys and values of one request [n, G, *] into scattered pages of a cache with rows for both; the table."""
    n, G = k.shape[0], k.shape[1]
    nb = (start + n + P - 1) // P
    table = torch.randperm(pages, generator=g)[:nb].tolist()
    cache = torch.full((pages, 2, G, P, dc), float("nan"), dtype=dtype)
    for j in range(n):
        pg, off = table[(start + j) // P], (start + j) % P
        cache[pg, 0, :, off, :] = 0
        cache[pg, 1, :, off, :] = 0
        cache[pg, 0, :, off, :k.shape[2]] = k[j].to(dtype)
        cache[pg, 1, :, off, :v.shape[2]] = v[j].to(dtype)
    return cache, table


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1.5e-2)])
@pytest.mark.parametrize("hq,hkv,dk,dv,chunk,P,n,bias,talk", [
    (6, 3, 8, 8, 21, 8, 75, True, True), (4, 4, 64, 64, 40, 16, 130, True, True), (10, 2, 44, 44, 110, 16, 300, True, True),
    (1, 1, 16, 16, 1, 4, 9, True, True), (16, 1, 8, 8, 1000, 4, 413, True, True), (3, 1, 64, 64, 70, 16, 150, False, True),
    (5, 5, 12, 20, 64, 8, 129, True, False), (16, 4, 64, 64, 256, 16, 600, True, True), (2, 1, 128, 128, 33, 16, 100, True, True),
    (40, 5, 8, 8, 30, 8, 70, True, True), (2, 1, 256, 256, 50, 16, 120, True, True), (12, 12, 36, 36, 90, 16, 200, True, True),
    (8, 8, 128, 128, 100, 16, 150, True, True), (24, 4, 32, 200, 50, 16, 90, True, True), (32, 8, 64, 160, 70, 16, 100, True, True)])
def test_talking_heads_attention_with_a_bias_by_distance(dtype, tol, hq, hkv, dk, dv, chunk, P, n, bias, talk):
    """Every position of a sequence at once (a prompt), then positions alone (decoded tokens) and in a batch beside
    another request whose pages lie between this one's."""
    o = ops()
    g = torch.Generator().manual_seed(hq * 100 + chunk)
    dc = (max(dk, dv) + 3) // 4 * 4
    q = (torch.randn(n, hq, dk, generator=g)).to(dtype)
    k = (torch.randn(n, hkv, dk, generator=g)).to(dtype)
    v = (torch.randn(n, hkv, dv, generator=g)).to(dtype)
    rows = 10
    table = (torch.randn(rows, hq, generator=g) * 0.8) if bias else None
    far = min(3.0 * chunk, 200.0) + 5.5
    tk = (torch.eye(hq) + 0.4 * torch.randn(hq, hq, generator=g)) if talk else None
    scale = 1.3 / math.sqrt(dk)
    pos = torch.arange(n)
    want = N.chunk_attention(q.double(), k.double(), v.double(), pos, scale, chunk, bias=table.double() if bias else None,
                             far=far, talk=tk.double() if talk else None)
    from qwen_engine_amd.parts.attention import distance_bias_rows
    pages = (n + P - 1) // P + 7
    cache, tab = _paged(k, v, P, pages, g, dtype, dc)
    other = [p for p in range(pages) if p not in tab][:3]
    for pg in other:
        cache[pg] = torch.randn(cache[pg].shape, generator=g).to(dtype)
    width = max(len(tab), len(other))
    bt = torch.full((2, width), -1, dtype=torch.int32)
    bt[1, :len(tab)] = torch.tensor(tab, dtype=torch.int32)
    bt[0, :len(other)] = torch.tensor(other, dtype=torch.int32)
    qp = torch.zeros(n, hq, dc, dtype=dtype)
    qp[:, :, :dk] = q
    kw = dict(chunk=chunk, bias=distance_bias_rows(table, far).to(DEV) if bias else None, talk=tk.to(DEV) if talk else None)
    cd, btd = cache.to(DEV), bt.to(DEV)
    got = o.attention_talk(qp.to(DEV), cd, i32(list(range(n))), i32([1] * n), btd, scale, dk, dv, **kw)
    assert rel(got.view(n, hq, dv), want) < tol
    # single rows: chunk edges, the last positions, beside a row of the other request
    picks = sorted({0, min(chunk - 1, n - 1), min(chunk, n - 1), (n - 1) // chunk * chunk, n - 1, n // 2})
    for p in picks:
        rows_q = torch.stack([torch.zeros(hq, dc, dtype=dtype), qp[p]])
        rows_q[0, :, :dk] = q[0]
        got = o.attention_talk(rows_q.to(DEV), cd, i32([min(P * len(other), 5) - 1, p]), i32([0, 1]), btd, scale, dk, dv, **kw)
        assert rel(got[1].view(hq, dv), want[p]) < tol, p
        assert not torch.isnan(got).any()
    # a portion that starts and ends inside chunks, as rows of a larger output
    a, b = n // 3, n - 2
    wide = torch.zeros(b - a, hq * dv + 5, dtype=dtype, device=DEV)
    o.attention_talk(qp[a:b].to(DEV), cd, i32(list(range(a, b))), i32([1] * (b - a)), btd, scale, dk, dv,
                     out=wide[:, :hq * dv], out_scale=0.5, **kw)
    assert rel(wide[:, :hq * dv].view(b - a, hq, dv), 0.5 * want[a:b]) < tol
    assert float(wide[:, hq * dv:].abs().max()) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk,P,n", [(64, 16, 64), (100, 16, 390), (512, 16, 500), (7, 4, 30)])
def test_one_key_that_stands_out_is_found_or_not_seen(dtype, chunk, P, n):
    """The last query and one key are made so large that their score stands out among hundreds: the output is that
    key's value when the key is the chunk's first, its last but one, or far back inside the chunk, and is not when the
    key is the last of the chunk before."""
    o = ops()
    hq, hkv, d = 4, 2, 16
    g = torch.Generator().manual_seed(chunk)
    first = (n - 1) // chunk * chunk
    for j, seen in ((first, True), (n - 2, n - 2 >= first), (first + (n - 1 - first) // 2, True), (first - 1, False), (0, first == 0)):
        if j < 0:
            continue
        q = torch.randn(n, hq, d, generator=g) * 0.3
        k = torch.randn(n, hkv, d, generator=g) * 0.3
        v = torch.randn(n, hkv, d, generator=g)
        q[n - 1] = 0
        q[n - 1, :, 3] = 6.0
        k[j, :, 3] = 6.0
        cache, tab = _paged(k, v, P, (n + P - 1) // P + 3, g, dtype, d)
        bt = torch.tensor([tab], dtype=torch.int32)
        talk = torch.eye(hq) + 0.05
        bias = torch.zeros(2, hq)
        for rows_q, pos in ((q, list(range(n))), (q[n - 1:], [n - 1])):
            got = o.attention_talk(rows_q.to(dtype).to(DEV), cache.to(DEV), i32(pos), i32([0] * len(pos)), bt.to(DEV), 1.0, d, d,
                                   chunk=chunk, bias=bias.to(DEV), talk=talk.to(DEV))[-1].view(hq, d).float().cpu()
            want = v[j].to(dtype).float().repeat_interleave(hq // hkv, dim=0)
            err = float((got - want).abs().max())
            assert (err < 2e-2) == seen, (j, seen, err)


# ---- attention inside chunks with the framework's attention kernels ------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1.5e-2)])
@pytest.mark.parametrize("hq,hkv,d,chunk,P,n", [(4, 2, 20, 13, 8, 60), (8, 2, 64, 40, 16, 170), (2, 2, 128, 100, 16, 250),
                                                (16, 1, 16, 1, 4, 11), (6, 2, 128, 112, 16, 400), (4, 4, 64, 64, 16, 257)])
def test_attention_inside_chunks(dtype, tol, hq, hkv, d, chunk, P, n):
    o = ops()
    g = torch.Generator().manual_seed(chunk + n)
    q = torch.randn(n, hq, d, generator=g).to(dtype)
    k = torch.randn(n, hkv, d, generator=g).to(dtype)
    v = torch.randn(n, hkv, d, generator=g).to(dtype)
    scale = 1.5 / math.sqrt(d)
    want = N.chunk_attention(q.double(), k.double(), v.double(), torch.arange(n), scale, chunk)
    pages = (n + P - 1) // P + 3
    tab = torch.randperm(pages, generator=g)[:(n + P - 1) // P].tolist()
    cache = torch.full((pages, 2, hkv, P, d), float("nan"), dtype=dtype)
    for j in range(n):
        pg, off = tab[j // P], j % P
        cache[pg, 0, :, off] = k[j]
        cache[pg, 1].view(hkv, d, P)[:, :, off] = v[j]
    for pg in tab[-1:]:                                        # (columns of keys that do not exist yet: never read as numbers)
        cache[pg, 1].view(hkv, d, P)[:, :, (n - 1) % P + 1:] = 0
    bt = torch.tensor([tab], dtype=torch.int32).to(DEV)
    cd = cache.to(DEV)
    got = o.attention(q.to(DEV), cd, i32(list(range(n))), i32([0] * n), bt, scale, chunk=chunk)
    assert rel(got, want) < tol
    for p in sorted({0, min(chunk - 1, n - 1), min(chunk, n - 1), (n - 1) // chunk * chunk, n - 1}):
        got = o.attention(q[p:p + 1].to(DEV), cd, i32([p]), i32([0]), bt, scale, chunk=chunk)
        assert rel(got[0], want[p]) < tol, p


# ---- blends with the token before -------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 8e-3)])
@pytest.mark.parametrize("W", [80, 208, 1030])
def test_blends_with_the_token_before_across_cuts_and_slots(dtype, tol, W):
    o = ops()
    g = torch.Generator().manual_seed(W)
    lengths = {0: 40, 1: 7, 2: 23}
    slot = {0: 3, 1: 0, 2: 2}
    x = {s: torch.randn(n, W, generator=g).to(dtype) for s, n in lengths.items()}
    mu = torch.rand(5, W, generator=g)
    state = torch.full((4, W + 11), 7.0, device=DEV)          # (a row wider than the blends' part, as in the engine)
    for s in slot.values():
        state[s, :W] = 0
    want = {}
    for s in lengths:
        h = x[s].double()
        before = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
        want[s] = torch.stack([h + (before - h) * mu[i].double() for i in range(5)])
    steps = [[(0, 5), (1, 1), (2, 2)], [(1, 1), (0, 1)], [(2, 1)], [(2, 20), (0, 2), (1, 5)], [(0, 32)]]
    done = {s: 0 for s in lengths}
    for step in steps:
        rows, seq = [], []
        for s, n in step:
            rows.append(x[s][done[s]:done[s] + n])
            seq += [slot[s]] * n
        single = all(n == 1 for _, n in step)
        y = o.token_shift(torch.cat(rows).to(DEV), mu.to(DEV), state, i32(seq), single_rows=single)
        at = 0
        for s, n in step:
            assert rel(y[:, at:at + n], want[s][:, done[s]:done[s] + n]) < tol, (s, done[s])
            at += n
            done[s] += n
            assert torch.equal(state[slot[s], :W].cpu(), x[s][done[s] - 1].float())
    assert float(state[:, W:].min()) == 7.0 and float(state[1].min()) == 7.0


# ---- the recurrences --------------------------------------------------------------------------------------------------
REC_STEPS = [[(0, 5), (1, 1), (2, 2)], [(1, 1), (0, 1)], [(2, 1)], [(2, 37), (0, 2), (1, 5)], [(0, 150)], [(0, 1), (2, 1)],
             [(0, 17), (2, 70)]]
REC_LENGTHS = {0: 176, 1: 7, 2: 111}


def _chunks_of(portions, head_dim, chunked):
    """The chunk lists of a step's portions for the chunked path (the kernels then take the rows chunk by chunk, the
    chunks in parallel), or None for the path that walks row by row."""
    if not chunked:
        return None
    ch, po = ops().recurrence_chunks(portions, ops().recurrence_chunk_len(head_dim))
    return ch.to(DEV), po.to(DEV)


def _run_recurrence(call, inputs, widths, slot, out_cols):
    """Feeds the requests' rows through ``call`` in REC_STEPS; returns each request's outputs in order."""
    done = {s: 0 for s in REC_LENGTHS}
    got = {s: [] for s in REC_LENGTHS}
    for step in REC_STEPS:
        seq = []
        rows = [[] for _ in inputs]
        for s, n in step:
            for i, t in enumerate(inputs):
                rows[i].append(t[s][done[s]:done[s] + n])
            seq += [slot[s]] * n
        starts, at = [], 0
        for _, n in step:
            starts.append((at, n))
            at += n
        out = call([torch.cat(r).to(DEV) for r in rows], i32(seq), starts)
        at = 0
        for s, n in step:
            got[s].append(out[at:at + n].cpu())
            at += n
            done[s] += n
    assert done == REC_LENGTHS
    return {s: torch.cat(v) for s, v in got.items()}


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-5)])
@pytest.mark.parametrize("H,D,Dv,decay", [(2, 12, 8, (0.5, 0.93)), (4, 24, 48, (0.55, 0.8, 0.95, 0.995)), (2, 64, 128, (0.8, 0.99)),
                                          (3, 4, 20, (1.0, 0.5, 0.25)), (1, 16, 16, (1.0,)), (2, 128, 128, (0.0, 0.9)),
                                          (1, 24, 200, (0.95,))])
@pytest.mark.parametrize("chunked", [False, True])
def test_recurrence_with_a_decay_per_head_across_cuts_and_slots(dtype, tol, H, D, Dv, decay, chunked):
    """(the inputs are rounded to the activation type first, the recurrence itself is 32-bit in both: one tolerance)"""
    o = ops()
    g = torch.Generator().manual_seed(H * D)
    slot = {0: 2, 1: 0, 2: 3}
    nk, nv = H * D, H * Dv
    y = {s: (torch.randn(n, 2 * nk + nv + 3, generator=g)).to(dtype) for s, n in REC_LENGTHS.items()}
    state = torch.full((4, nk * Dv + 6), float("nan"), device=DEV)
    for s in slot.values():
        state[s, :nk * Dv] = 0
    dec = torch.tensor(decay, dtype=torch.float64)

    def call(rows, seq, portions):
        r = rows[0]
        return o.linear_recurrence(r[:, :nk], r[:, nk:2 * nk], r[:, 2 * nk:2 * nk + nv], state, seq, H,
                                   decay=dec.float().to(DEV), silu=True, chunks=_chunks_of(portions, D, chunked))

    got = _run_recurrence(call, [y], None, slot, nv)
    for s, n in REC_LENGTHS.items():
        z = N.silu(y[s].double())
        want = N.decayed_sum_state(z[:, :nk].reshape(n, H, D), z[:, nk:2 * nk].reshape(n, H, D),
                                   z[:, 2 * nk:2 * nk + nv].reshape(n, H, Dv), dec)
        assert rel(got[s], want) < tol, s
    assert torch.isnan(state[1]).all() and torch.isnan(state[:, nk * Dv:]).all()


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-5)])
@pytest.mark.parametrize("H,D", [(3, 8), (2, 36), (2, 64), (1, 16), (5, 64), (1, 128), (2, 20)])
@pytest.mark.parametrize("chunked", [False, True])
def test_recurrence_with_a_decay_per_channel_and_a_bonus_across_cuts_and_slots(dtype, tol, H, D, chunked):
    o = ops()
    g = torch.Generator().manual_seed(H * D + 1)
    slot = {0: 1, 1: 3, 2: 0}
    n_ = H * D
    r = {s: torch.randn(n, n_, generator=g).to(dtype) for s, n in REC_LENGTHS.items()}
    k = {s: torch.randn(n, n_, generator=g).to(dtype) for s, n in REC_LENGTHS.items()}
    v = {s: torch.randn(n, n_, generator=g).to(dtype) for s, n in REC_LENGTHS.items()}
    wx = {s: torch.randn(n, n_, generator=g) * 1.5 for s, n in REC_LENGTHS.items()}      # decays from nearly 0 to nearly 1
    wx[0][40:44] = 95.0                                           # (and decays of exactly 0: exp(95) is beyond 32-bit)
    w0 = torch.randn(n_, generator=g) * 0.8 - 1.0
    u = torch.randn(n_, generator=g) * 0.5
    W = 9                                                         # (the state's first numbers belong to the blends)
    state = torch.full((4, W + n_ * D), float("nan"), device=DEV)
    for s in slot.values():
        state[s, W:] = 0

    def call(rows, seq, portions):
        return o.linear_recurrence(rows[0], rows[1], rows[2], state[:, W:], seq, H, decay_x=rows[3], decay_bias=w0.to(DEV),
                                   bonus=u.to(DEV), chunks=_chunks_of(portions, D, chunked))

    got = _run_recurrence(call, [r, k, v, wx], None, slot, n_)
    for s, n in REC_LENGTHS.items():
        wdec = torch.exp(-torch.exp(wx[s].double() + w0.double())).reshape(n, H, D)
        want = N.bonus_state(r[s].double().reshape(n, H, D), k[s].double().reshape(n, H, D), v[s].double().reshape(n, H, D),
                             wdec, u.double().reshape(H, D))
        assert rel(got[s], want) < tol, s
    assert torch.isnan(state[2]).all() and torch.isnan(state[:, :W]).all()


@pytest.mark.parametrize("chunked", [False, True])
def test_a_state_far_back_is_kept_or_forgotten(chunked):
    """One early token writes a large k v^T; hundreds of tokens later a query along that key reads it back: whole with a
    decay of 1, scaled by decay^n otherwise.  Random inputs alone would bury a lost state under the recent tokens."""
    o = ops()
    H, D, Dv, n = 2, 16, 16, 400
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(n, H * D, generator=g) * 0.01 for _ in range(3))
    k[2] = 0; k[2, 5] = 10.0; k[2, D + 5] = 10.0
    v[2] = torch.arange(H * Dv).float()
    q[n - 1] = 0; q[n - 1, 5] = 1.0; q[n - 1, D + 5] = 1.0
    dec = torch.tensor([1.0, 0.99])
    want = N.decayed_sum_state(q.double().reshape(n, H, D), k.double().reshape(n, H, D), v.double().reshape(n, H, Dv), dec.double())
    assert float(want[-1, 0].abs().max()) > 100 and float(want[-1, 1].abs().max()) > 1
    for cut in ((n,), (3, 200, 197), (1,) * 20 + (n - 20,)):
        state = torch.zeros(1, H * D * Dv, device=DEV)
        outs, at = [], 0
        for m in cut:
            outs.append(o.linear_recurrence(q[at:at + m].to(DEV), k[at:at + m].to(DEV), v[at:at + m].to(DEV), state, i32([0] * m), H,
                                            decay=dec.to(DEV), chunks=_chunks_of([(0, m)], D, chunked)))
            at += m
        assert rel(torch.cat(outs), want) < 2e-5, cut


# ---- norm and gate after a recurrence -----------------------------------------------------------------------------------
@pytest.mark.parametrize("T,N_,groups", [(5, 24, 3), (9, 256, 1), (3, 640, 5), (2, 2048, 16), (1, 20, 1), (4, 1024, 1), (2, 1200, 2)])
@pytest.mark.parametrize("act", ["silu", "sigmoid", None])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 6e-3)])
def test_norm_and_gate(T, N_, groups, act, dtype, tol):
    o = ops()
    g = torch.Generator().manual_seed(T * N_)
    x, w = torch.randn(T, N_, generator=g) * 3, 1 + 0.3 * torch.randn(N_, generator=g)
    gate = torch.randn(T, N_ + 4, generator=g).to(dtype)
    want = N.rms(x.double().reshape(T, groups, -1), 1e-5).reshape(T, N_) * w.double()
    if act:
        want = want * (N.silu if act == "silu" else N.sigmoid)(gate[:, 4:].double())
    got = o.gated_norm(x.to(DEV), w.to(DEV), 1e-5, groups, dtype, gate=gate.to(DEV)[:, 4:] if act else None,
                       gate_act={"silu": o.GATE_SILU, "sigmoid": o.GATE_SIGMOID, None: o.GATE_NONE}[act])
    assert got.dtype == dtype and rel(got, want) < tol
