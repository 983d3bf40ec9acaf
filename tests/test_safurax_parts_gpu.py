"""Each mechanism of the Safurax layers alone: the kernel against the plain implementation's function of the same
mechanism (or a few lines of 64-bit torch), in float32 and bfloat16."""
import math

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import safurax_plain as S

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    from qwen_engine_amd.kernels import ops as o
    return o


def rel(got, want):
    return float((got.double().cpu() - want.double()).abs().max()) / max(float(want.abs().max()), 1e-30)


# ---- the layer norm, with the residual sum in front of it --------------------------------------------------------
@pytest.mark.parametrize("T,H,parts", [(1, 96, 0), (5, 202, 1), (33, 2048, 3), (700, 256, 2), (3, 8200, 2)])
def test_layer_norm_with_the_residual_sum(T, H, parts):
    g = torch.Generator().manual_seed(T + H)
    x = torch.randn(T, H, generator=g) * 3.0 + 5.0             # (a mean far from zero: a norm that forgot it shows)
    w = 1.0 + 0.3 * torch.randn(H, generator=g)
    delta = torch.randn(parts, T, H, generator=g) if parts else None
    z = x.double() + (delta.double().sum(0) if parts else 0)
    want = S.layer_norm(z, w.double(), 1e-5)
    xs = x.to(DEV)
    got = ops().rmsnorm(xs, w.to(DEV), 1e-5, torch.float32, delta=None if delta is None else delta.to(DEV), center=True)
    assert rel(got, want) < 3e-6
    assert rel(xs, z) < 1e-6                                    # the sum went back into the stream
    rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
    xs = x.to(DEV)
    got = ops().rmsnorm(xs, w.to(DEV), 1e-5, torch.bfloat16, delta=None if delta is None else delta.to(DEV), rows=rows,
                        center=True)
    assert rel(got, want[[T - 1, 0]]) < 6e-3
    assert torch.equal(xs.cpu(), x)                             # only some rows normed: the stream stays


# ---- the token's cache row and the queries' rotated part -----------------------------------------------------------
@pytest.mark.parametrize("R,Dr,dims,H,Dn", [(24, 12, 12, 5, 8), (64, 32, 32, 16, 16), (40, 0, 0, 3, 16), (16, 10, 6, 2, 0)])
def test_latent_row_norm_and_half_split_rotation(R, Dr, dims, H, Dn):
    g = torch.Generator().manual_seed(R + Dr)
    T, P = 9, 4
    kv = torch.randn(T, R + Dr, generator=g) * 2.0
    w = 1.0 + 0.3 * torch.randn(R, generator=g)
    q = torch.randn(T, H, Dn + Dr, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 100, 101, 7, 5000, 31], dtype=torch.int32)
    slots = torch.tensor([5, 0, 9, -1, 17, 2, 3, 11, 30], dtype=torch.int32)
    inv = (100.0 ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / max(dims, 1))).float()
    cache = torch.zeros(8, 1, 1, P, R + Dr, device=DEV)
    qp = torch.zeros(T, H, R + Dr, device=DEV)
    ops().latent_kv_store(kv.to(DEV), w.to(DEV), 1e-5, pos.to(DEV), inv.to(DEV), slots.to(DEV), cache, q.to(DEV), qp, Dn,
                          half_split=True)
    c = S.rms_norm(kv[:, :R].double(), w.double(), 1e-5)
    kr = S.rotate_half_split(kv[:, R:].double(), pos, 100.0, dims) if Dr else kv[:, R:].double()
    flat = cache.view(-1, R + Dr).cpu()
    for t in range(T):
        if slots[t] >= 0:
            assert rel(flat[slots[t], :R], c[t]) < 2e-6 and (Dr == 0 or rel(flat[slots[t], R:], kr[t]) < 2e-4)
    assert float(flat[4].abs().max()) == 0.0                    # a row that no token's slot named
    if Dr:
        qr = S.rotate_half_split(q[..., Dn:].double(), pos, 100.0, dims)
        assert rel(qp[..., R:], qr) < 2e-4                      # (a 32-bit angle of thousands of radians)
        qp2 = torch.zeros(T, H, R + Dr, device=DEV)
        ops().latent_q_rotate(q.to(DEV), pos.to(DEV), inv.to(DEV), qp2, Dn, half_split=True)
        assert torch.equal(qp2[..., R:].cpu(), qp[..., R:].cpu())


# ---- attention over the cached latents with a window and a sink ---------------------------------------------------
def _latent_case(dtype, R, Dr, P, lengths, seed):
    """Requests of the given lengths in scattered pages."""
    g = torch.Generator().manual_seed(seed)
    D = R + Dr
    pages_per = [(n + P - 1) // P for n in lengths]
    order = torch.randperm(sum(pages_per) + 3, generator=g).tolist()
    cache = torch.full((len(order), 1, 1, P, D), float("nan"))
    table = torch.full((len(lengths), max(pages_per)), -1, dtype=torch.int32)
    rows = []
    for b, n in enumerate(lengths):
        rows.append((torch.randn(n, D, generator=g)).to(dtype))
        for i in range(pages_per[b]):
            page = order.pop()
            table[b, i] = page
            chunk = rows[b][i * P:(i + 1) * P]
            cache[page, 0, 0, :len(chunk)] = chunk.float()
    return cache.to(dtype), table, rows


def _latent_reference(q, rows, R, pos, scale, window, sink):
    """q [H, D] at position pos of a request whose cache rows are ``rows``: [H, R] in 64-bit."""
    lo = max(0, pos - window + 1) if window else 0
    keys = rows[lo:pos + 1].double()
    s = (q.double() @ keys.T) * scale
    if sink is not None:
        s = torch.cat([s, sink.double()[:, None]], dim=1)
    p = torch.softmax(s, dim=-1)
    return p[:, :keys.shape[0]] @ keys[:, :R]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 1.2e-2)])
@pytest.mark.parametrize("R,Dr,H,P,window,with_sink", [(24, 12, 5, 8, 37, True), (64, 32, 16, 16, 64, True),
                                                       (64, 32, 16, 16, 0, True), (64, 32, 16, 16, 33, False),
                                                       (40, 0, 3, 4, 9, True), (32, 8, 1, 16, 1, True),
                                                       (128, 32, 20, 16, 200, True)])
def test_latent_attention_with_window_and_sink(dtype, tol, R, Dr, H, P, window, with_sink):
    """Portions of prompts beside single new tokens, scattered pages; pages behind every query's window are taken away
    (their table entries become -1 and their rows NaN), as the cache manager does once a window has passed them."""
    lengths = [3 * P + 1, 1, 150, 65, 300]
    new = [2 * P + 1, 1, 1, 40, 70]                              # the last so many tokens of each request are queries
    cache, table, rows = _latent_case(dtype, R, Dr, P, lengths, seed=R + H + window)
    if window:
        for b, n in enumerate(lengths):
            first_seen = max(0, (n - new[b]) - window + 1)
            for i in range(first_seen // P):
                cache[table[b, i]] = float("nan")
                table[b, i] = -1
    g = torch.Generator().manual_seed(1)
    sink = (1.5 * torch.randn(H, generator=g)) if with_sink else None
    scale = 1.0 / math.sqrt(R + Dr) * 2.0
    qs, poss, seqs = [], [], []
    for b, n in enumerate(lengths):
        for p in range(n - new[b], n):
            qs.append(torch.randn(H, R + Dr, generator=g))
            poss.append(p)
            seqs.append(b)
    q = torch.stack(qs).to(dtype)
    args = (q.to(DEV), cache.to(DEV), torch.tensor(poss, dtype=torch.int32, device=DEV),
            torch.tensor(seqs, dtype=torch.int32, device=DEV), table.to(DEV), R, scale)
    kw = dict(window=window, sink=None if sink is None else sink.to(DEV))
    got = ops().latent_attention(*args, **kw)
    assert not torch.isnan(got.float()).any()
    for t in range(len(poss)):
        want = _latent_reference(q[t], rows[seqs[t]], R, poss[t], scale, window, sink)
        assert rel(got[t], want) < tol, f"row {t}: request {seqs[t]} at position {poss[t]}"
    if dtype == torch.bfloat16:                                   # the kernel on the vector units against the one above
        slow = ops().latent_attention(*args, algo=ops().ALGO_GENERIC, **kw)
        assert rel(slow, got.double().cpu()) < 1.5e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_key_at_the_windows_edge_is_seen_and_the_one_behind_it_is_not(dtype):
    """One key's score stands far out.  A query whose window still holds it returns that key's latent; the query one
    position later, whose window has just passed it, returns something else; a large sink takes the weight away."""
    R, Dr, H, P, W = 64, 32, 16, 16, 48
    n = 200
    cache, table, rows = _latent_case(dtype, R, Dr, P, [n], seed=5)
    target = 77
    q = torch.zeros(2, H, R + Dr)
    q[:] = rows[0][target].float() * 3.0                          # every head's query points at the target's row
    want_in = rows[0][target, :R].double()
    for window, first in ((W, target + W - 1), (1, target), (130 - target + 1, 130)):
        # a portion of two rows: the first still sees the target, the second has just passed it
        pos = torch.tensor([first, first + 1], dtype=torch.int32)
        got = ops().latent_attention(q.to(dtype).to(DEV), cache.to(DEV), pos.to(DEV), torch.zeros(2, dtype=torch.int32, device=DEV),
                                     table.to(DEV), R, 1.0, window=window)
        assert rel(got[0, 3], want_in) < 2e-2, f"window {window}: the key at its edge"
        assert rel(got[1, 3], want_in) > 0.5, f"window {window}: the key behind its edge"
        # the same two queries as single rows of a batch (each the only row of its launch's request)
        for row, inside in ((0, True), (1, False)):
            one = ops().latent_attention(q[row:row + 1].to(dtype).to(DEV), cache.to(DEV), pos[row:row + 1].to(DEV),
                                         torch.zeros(1, dtype=torch.int32, device=DEV), table.to(DEV), R, 1.0, window=window)
            assert (rel(one[0, 3], want_in) < 2e-2) == inside
    big = torch.full((H,), 1000.0)
    got = ops().latent_attention(q.to(dtype).to(DEV), cache.to(DEV), torch.tensor([target, target + 1], dtype=torch.int32, device=DEV),
                                 torch.zeros(2, dtype=torch.int32, device=DEV), table.to(DEV), R, 1.0, window=W, sink=big.to(DEV))
    assert float(got.float().abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_far_key_among_many_decides_the_output(dtype):
    R, Dr, H, P = 64, 32, 16, 16
    n = 700
    cache, table, rows = _latent_case(dtype, R, Dr, P, [n], seed=6)
    for target in (0, 15, 16, 333):
        q = (rows[0][target].float() * 3.0).expand(1, H, R + Dr).contiguous()
        got = ops().latent_attention(q.to(dtype).to(DEV), cache.to(DEV), torch.tensor([n - 1], dtype=torch.int32, device=DEV),
                                     torch.zeros(1, dtype=torch.int32, device=DEV), table.to(DEV), R, 1.0)
        assert rel(got[0, 0], rows[0][target, :R].double()) < 2e-2, f"key {target}"


# ---- products per head with one gate a head ----------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 8e-3)])
@pytest.mark.parametrize("T,H,K,N", [(37, 3, 24, 20), (5, 16, 64, 16), (130, 1, 32, 48)])
def test_products_per_head_with_one_gate_a_head(dtype, tol, T, H, K, N):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, H, K, generator=g).to(dtype)
    w = (torch.randn(H, N, K, generator=g) / math.sqrt(K)).to(dtype)
    wide = torch.randn(T, H + 5, generator=g).to(dtype).to(DEV)    # the gates as the last columns of wider rows
    gate = wide[:, 5:]
    out = torch.empty(T, H, N, dtype=dtype, device=DEV)
    ops().gemm_heads(x.to(DEV), w.to(DEV), out, gate)
    want = torch.einsum("thk,hnk->thn", x.double(), w.double()) * torch.sigmoid(gate.double().cpu())[:, :, None]
    assert rel(out, want) < tol


# ---- the two maps of differential attention joined ---------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("T,H,G,Dv,Dc", [(7, 4, 2, 24, 64), (33, 8, 1, 64, 64), (2, 3, 3, 16, 64), (5, 6, 2, 100, 112)])
def test_maps_joined_normed_scaled_and_gated(dtype, tol, T, H, G, Dv, Dc):
    g = torch.Generator().manual_seed(T + H)
    a = torch.randn(T, 2 * H, Dc, generator=g).to(dtype)
    wide = torch.randn(T, 11 + H, generator=g).to(dtype).to(DEV)
    gate = wide[:, 11:]
    lam, eps, diff = 0.37, 1e-5, 0.3
    got = ops().diff_heads(a.to(DEV), H, G, Dv, lam, eps, 1.0 - diff, gate=gate)
    per = H // G
    for h in range(H):
        grp, j = h // per, h % per
        a1 = a[:, grp * 2 * per + j, :Dv].double()
        a2 = a[:, grp * 2 * per + per + j, :Dv].double()
        want = S.rms_unit(a1 - lam * a2, eps) * (1.0 - diff) * torch.sigmoid(gate[:, h].double().cpu())[:, None]
        assert rel(got[:, h], want) < tol, f"head {h}"


# ---- the router: the largest biased logits, weighed among themselves ----------------------------------------------
@pytest.mark.parametrize("T,E,top,extra,transposed", [(9, 6, 2, 1, False), (70, 16, 4, 1, True), (5, 3, 3, 0, False),
                                                       (40, 4, 1, 0, False), (3, 70, 5, 2, False)])
def test_router_picks_the_largest_biased_logits(T, E, top, extra, transposed):
    g = torch.Generator().manual_seed(T + E)
    z = torch.randn(T, E + extra, generator=g) * 2.0
    z[:, E:] += 50.0                                              # (columns behind the router's must never be chosen)
    b = torch.randn(E, generator=g)
    z[0, :E] -= 200.0 * torch.arange(E)                           # one token whose logits lie far apart
    dev = z.t().contiguous().to(DEV) if transposed else z.to(DEV)
    ids, w = ops().moe_route_biased(dev, None, top, 1.0, transposed=transposed, logit_bias=b.to(DEV), experts=E)
    want_ids, want_w = S.route(z[:, :E].double() + b.double(), top)
    assert torch.equal(ids.cpu().long(), want_ids)
    assert rel(w, want_w) < 2e-6
    assert abs(float(w[0].sum()) - 1.0) < 1e-6


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 1.5e-2)])
@pytest.mark.parametrize("T,E,top,Fd,shared", [(5, 6, 2, 40, 56), (300, 8, 3, 160, 64), (600, 4, 2, 64, 32), (1, 3, 3, 32, 0)])
def test_mixture_with_a_shared_expert(dtype, tol, T, E, top, Fd, shared):
    """The part itself: router with its bias, experts, shared expert behind its gate, summed."""
    from qwen_engine_amd.config.spec import TopSoftmaxMoESpec
    from qwen_engine_amd.parts import Runtime, build_part
    W = 128
    g = torch.Generator().manual_seed(T + E)
    r = lambda *s: torch.randn(*s, generator=g)
    w = {"router": (r(E, W) * 3.0 / math.sqrt(W)).bfloat16(), "router.b": (0.7 * r(E)).bfloat16()}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = [(m * 1.6 / math.sqrt(m.shape[-1])).bfloat16()
                                                          for m in (r(Fd, W), r(Fd, W), r(W, Fd))]
    if shared:
        for n, m in (("gate", r(shared, W)), ("up", r(shared, W)), ("down", r(W, shared)), ("sg", r(1, W))):
            w["shared." + n] = (m * 1.6 / math.sqrt(m.shape[-1])).bfloat16()
    spec = TopSoftmaxMoESpec(num_experts=E, top=top, intermediate_size=Fd, router_bias=True,
                             shared_intermediate_size=shared or None, shared_gate=bool(shared))
    part = build_part(spec, W)
    rt = Runtime(torch.device(DEV), dtype)
    part.load(w, rt)
    x = r(T, W).to(dtype)

    class Ctx:
        pass
    ctx = Ctx()
    ctx.rt = rt
    got = part.forward(x.to(DEV), ctx).sum(0)
    mlp = {"router": {"top": top}, "shared": {"ff": shared} if shared else None}
    want = S.mixture(x.double(), w, "", mlp)
    if dtype == torch.float32:
        assert rel(got, want) < tol
    else:
        # (a router's close call may fall the other way in bfloat16: nearly every row agrees)
        err = (got.double().cpu() - want).abs().amax(dim=1) / float(want.abs().max())
        assert float((err > tol).float().mean()) <= 0.03, f"{int((err > tol).sum())} of {T} rows differ"
