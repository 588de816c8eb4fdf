"""Each kernel alone against a plain float32 formula, at sizes other than the engine's."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _ops():
    from sharpinference_amd import ops

    return ops


def _rand(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


@pytest.mark.parametrize("M", [1, 5, 16, 17, 40, 64])
@pytest.mark.parametrize("N,K", [(132, 128), (1000, 256), (5120, 1024), (20, 384), (48, 640), (208, 1152)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_gemm_skinny(M, N, K, out_dtype):
    ops = _ops()
    x = _rand(M, K, dtype=torch.bfloat16, seed=M)
    w = _rand(N, K, dtype=torch.bfloat16, scale=0.1, seed=N)
    ref = x.float() @ w.float().T
    forms = [w]
    if ops.can_pack(w):                       # the same matrix stored tile by tile
        forms.append(ops.pack_weight(w, keep_rows=False))
        assert torch.equal(ops.unpack_weight(forms[1]), w)
    for form in forms:
        for R in (1, 2, 4):
            for NW in (4, 8, 16):
                if NW == 16 and R > 1:
                    continue   # refused: 1,024-thread blocks only take one weight tile
                got = ops.gemm_skinny(x, form, out_dtype, R=R, NW=NW).float()
                tol = 2e-2 if out_dtype == torch.bfloat16 else 1e-3
                assert float((got - ref).abs().max()) <= tol * float(ref.abs().max()), (M, N, K, R, NW, form is w)


@pytest.mark.parametrize("M", [16, 17, 24, 32, 33])
def test_linear_against_a_very_tall_matrix(M):
    """The head's shape class (more than 65,536 rows): the few-rows kernel up to 32 rows, the
    library beyond; both sides of 16/17 and 32/33 through the dispatcher the model calls, over the
    packed form and the row form, into float32 (logits) and bfloat16."""
    ops = _ops()
    N, K = 65536 + 1024, 256
    x = _rand(M, K, dtype=torch.bfloat16, seed=M)
    w = _rand(N, K, dtype=torch.bfloat16, scale=0.1, seed=7)
    ref = x.float() @ w.float().T
    assert ops.skinny_ok(M, N, K) == (M <= 32) and ops.skinny_ok(M, 4096, K) == (M <= 32)
    for form in (w, ops.pack_weight(w)):
        for out_dtype, tol in ((torch.float32, 1e-3), (torch.bfloat16, 2e-2)):
            got = ops.linear(x, form, out_dtype)
            assert got.dtype == out_dtype and got.shape == (M, N)
            assert float((got.float() - ref).abs().max()) <= tol * float(ref.abs().max()), (M, form is w, out_dtype)
    # a row's result does not depend on how many rows ride along (within the kernel's reach)
    if M <= 32:
        one = ops.linear(x[:1].contiguous(), w, torch.float32)
        assert torch.equal(one[0], ops.linear(x, w, torch.float32)[0])


def test_gemm_skinny_rows_do_not_depend_on_the_batch():
    ops = _ops()
    x = _rand(64, 512, dtype=torch.bfloat16, seed=3)
    for w in (_rand(516, 512, dtype=torch.bfloat16, scale=0.1, seed=4),
              ops.pack_weight(_rand(528, 512, dtype=torch.bfloat16, scale=0.1, seed=5), keep_rows=False)):
        full = ops.gemm_skinny(x, w, torch.float32)
        for m in (1, 7, 16, 33):
            part = ops.gemm_skinny(x[:m].contiguous(), w, torch.float32)
            assert torch.equal(part, full[:m]), m


@pytest.mark.parametrize("rows,E", [(8, 4), (64, 16), (33, 5), (1, 3), (100, 3), (150, 2)])
@pytest.mark.parametrize("N", [264, 272])
def test_gemm_skinny_grouped(rows, E, N):
    ops = _ops()
    K, T = 256, 40
    g = torch.Generator().manual_seed(rows)
    x = _rand(T, K, dtype=torch.bfloat16, seed=1)
    w = _rand(E, N, K, dtype=torch.bfloat16, scale=0.1, seed=2)
    expert = torch.sort(torch.randint(0, E, (rows,), generator=g)).values
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    for e in range(E):
        offsets[e + 1] = offsets[e] + int((expert == e).sum())
    a_rows = torch.randint(0, T, (rows,), generator=g, dtype=torch.int32)
    ref = torch.stack([x[int(a_rows[i])].float() @ w[int(expert[i])].float().T for i in range(rows)])
    for form in ([w, ops.pack_weight(w, keep_rows=False)] if ops.can_pack(w) else [w]):
        for R, NW in ((1, 16), (2, 8), (4, 4)):
            # the bound on an expert's rows chooses how many 16-row blocks are multiplied at a time;
            # a bound that is too small (or none) only costs more passes over the weights
            for bound in (None, int((offsets[1:] - offsets[:-1]).max()), 20):
                got = ops.gemm_skinny(x, form, torch.float32, a_rows=a_rows.to(DEV), offsets=offsets.to(DEV), n_rows=rows,
                                      R=R, NW=NW, group_rows=bound)
                assert float((got - ref).abs().max()) <= 1e-3 * float(ref.abs().max()), (R, NW, form is w, bound)


# ---------------------------------------------------------------------------
# attention over a paged cache
# ---------------------------------------------------------------------------
def _paged_case(lens, nh, nkv, hd, ps, dtype, seed, strong_key=None):
    """Random q/k/v for requests of the given context lengths, scattered over shuffled pages.
    Returns what the kernels need plus dense per-request k, v for the reference."""
    g = torch.Generator().manual_seed(seed)
    n = len(lens)
    blocks = [(L + ps - 1) // ps for L in lens]
    n_pages = sum(blocks) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    maxb = max(blocks)
    bt = torch.full((n, maxb), -1, dtype=torch.int32)
    kc = torch.zeros(n_pages, nkv, ps, hd)
    vc = torch.zeros(n_pages, nkv, hd, ps)
    ks, vs = [], []
    it = iter(perm)
    for i, L in enumerate(lens):
        k = torch.randn(L, nkv, hd, generator=g)
        v = torch.randn(L, nkv, hd, generator=g)
        if strong_key is not None and L > strong_key:
            k[strong_key] *= 6.0                       # one far key that must not be missed
        ks.append(k.to(dtype).float())
        vs.append(v.to(dtype).float())
        for b in range(blocks[i]):
            page = next(it)
            bt[i, b] = page
            seg = slice(b * ps, min(L, (b + 1) * ps))
            m = seg.stop - seg.start
            kc[page, :, :m, :] = ks[i][seg].permute(1, 0, 2)
            vc[page, :, :, :m] = vs[i][seg].permute(1, 2, 0)
    return bt, kc.to(dtype), vc.to(dtype), ks, vs


def _pages_from(ks, vs, ps, dtype, seed):
    """Given dense per-request k, v [L, nkv, hd]: the same scattered over shuffled pages."""
    g = torch.Generator().manual_seed(seed)
    nkv, hd = ks[0].shape[1], ks[0].shape[2]
    blocks = [(k.shape[0] + ps - 1) // ps for k in ks]
    n_pages = sum(blocks) + 3
    it = iter(torch.randperm(n_pages, generator=g).tolist())
    bt = torch.full((len(ks), max(blocks)), -1, dtype=torch.int32)
    kc = torch.zeros(n_pages, nkv, ps, hd)
    vc = torch.zeros(n_pages, nkv, hd, ps)
    for i, (k, v) in enumerate(zip(ks, vs)):
        for b in range(blocks[i]):
            page = next(it)
            bt[i, b] = page
            seg = slice(b * ps, min(k.shape[0], (b + 1) * ps))
            m = seg.stop - seg.start
            kc[page, :, :m, :] = k[seg].permute(1, 0, 2)
            vc[page, :, :, :m] = v[seg].permute(1, 2, 0)
    return bt, kc.to(dtype), vc.to(dtype)


def _ref_attention(q, k, v, p, start, scale):
    """q [nh, hd]; k, v [L, nkv, hd]: softmax over keys start..p."""
    nh, hd = q.shape
    nkv = k.shape[1]
    out = torch.empty(nh, hd)
    for h in range(nh):
        kh, vh = k[start:p + 1, h // (nh // nkv)], v[start:p + 1, h // (nh // nkv)]
        w = torch.softmax((kh @ q[h]) * scale, dim=0)
        out[h] = w @ vh
    return out


def _start(p, kind, window):
    return (p // window) * window if kind == 1 else max(0, p - window + 1) if kind == 2 else 0


_DECODE_CASES = [(nh, nkv, hd, kind, window, ps)
                 for nh, nkv, hd in [(8, 2, 64), (5, 5, 32), (40, 8, 128), (3, 1, 96), (34, 2, 32)]
                 for kind, window in [(0, 0), (1, 24), (1, 300), (2, 50)] for ps in (16, 64)]
# every other head size the kernel is compiled for, each with one kind of window
_DECODE_CASES += [(2, 1, 160, 1, 300, 16), (6, 2, 192, 0, 0, 64), (3, 3, 224, 2, 50, 16), (4, 2, 256, 1, 24, 16),
                  (4, 2, 256, 0, 0, 64)]


@pytest.mark.parametrize("nh,nkv,hd,kind,window,ps", _DECODE_CASES)
def test_attention_decode_kernel(nh, nkv, hd, kind, window, ps):
    ops = _ops()
    assert ops.decode_attention_ok(torch.bfloat16, hd)
    lens = [1, 17, 300, 1000, 257, 512]
    bt, kc, vc, ks, vs = _paged_case(lens, nh, nkv, hd, ps, torch.bfloat16, seed=nh * 7 + hd, strong_key=3)
    n = len(lens)
    g = torch.Generator().manual_seed(5)
    q = torch.randn(n, nh, hd, generator=g).to(torch.bfloat16)
    positions = torch.tensor([L - 1 for L in lens], dtype=torch.int32)
    scale = 1.0 / math.sqrt(hd)
    ref = torch.stack([_ref_attention(q[i].float(), ks[i], vs[i], lens[i] - 1, _start(lens[i] - 1, kind, window), scale)
                       for i in range(n)])
    args = (q.reshape(n, nh * hd).to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), torch.arange(n, dtype=torch.int32, device=DEV),
            positions.to(DEV))
    got = ops.attention_decode(*args, None, max(lens), kind, window, scale, nh, nkv, hd).float().cpu().view(n, nh, hd)
    assert float((got - ref).abs().max()) <= 2e-2, float((got - ref).abs().max())
    gen = ops.attention_generic(*args, kind, window, scale, nh, nkv, hd).float().cpu().view(n, nh, hd)
    assert float((gen - ref).abs().max()) <= 1e-2
    # a subset through the token list leaves the other rows alone
    sel = torch.tensor([4, 1, 3], dtype=torch.int32, device=DEV)
    out = torch.zeros(n, nh * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention_decode(*args, sel, max(lens), kind, window, scale, nh, nkv, hd, out=out)
    out = out.float().cpu().view(n, nh, hd)
    assert torch.equal(out[[4, 1, 3]], got[[4, 1, 3]]) and float(out[[0, 2, 5]].abs().max()) == 0.0


@pytest.mark.parametrize("kind,window", [(0, 0), (1, 256), (2, 89)])
@pytest.mark.parametrize("ps", [16, 32])
def test_attention_sees_one_key_at_every_edge(kind, window, ps):
    """Random keys would average a missed key away.  Here one key at a time is made to carry all
    the weight (it points along the query), at the first and last position, at both sides of a
    page's edge, of the decode kernel's 256-key runs and of the window's first key: the output
    must be that key's value when the key is visible and must not be when it is not."""
    ops = _ops()
    nh, nkv, hd, L = 4, 2, 64, 600
    scale = 1.0 / math.sqrt(hd)
    g = torch.Generator().manual_seed(3)
    u = torch.randn(hd, generator=g)
    u = (u / u.norm() * math.sqrt(hd)).to(torch.bfloat16).float()
    q1 = (2.0 * u).expand(nh, hd)                                   # every head asks the same question
    portion = 100                                                   # prefill: the last 100 positions are queries
    p_last = L - 1
    start = _start(p_last, kind, window)
    edges = {0, 1, ps - 1, ps, ps + 1, 255, 256, 257, 511, 512, 513, L - portion - 1, L - portion, L - 2, L - 1,
             max(start - 1, 0), start, start + 1}
    for j in sorted(edges):
        k = (0.05 * torch.randn(L, nkv, hd, generator=g)).to(torch.bfloat16).float()
        v = torch.randn(L, nkv, hd, generator=g).to(torch.bfloat16).float()
        k[j] = 2.0 * u                                              # score 4 * hd * scale = 32 above the rest
        bt, kc, vc = _pages_from([k], [v], ps, torch.bfloat16, seed=j)
        dev = [t.to(DEV) for t in (kc, vc, bt)]
        # decode: one query at the last position
        qd = q1.reshape(1, nh * hd).to(torch.bfloat16).to(DEV)
        one = torch.zeros(1, dtype=torch.int32, device=DEV)
        pos = torch.tensor([p_last], dtype=torch.int32, device=DEV)
        ref = _ref_attention(q1, k, v, p_last, start, scale)
        for name, got in (("decode", ops.attention_decode(qd, *dev, one, pos, None, L, kind, window, scale, nh, nkv, hd)),
                          ("generic", ops.attention_generic(qd, *dev, one, pos, kind, window, scale, nh, nkv, hd))):
            got = got.float().cpu().view(nh, hd)
            assert float((got - ref).abs().max()) <= 2e-2, (name, j)
            near = float((got - v[j].repeat_interleave(nh // nkv, 0)).abs().max())
            assert (near <= 2e-2) == (j >= start), (name, j, near)
        # prefill: the last `portion` positions in one step, every query the same question
        T = portion
        qp = q1.reshape(1, nh * hd).expand(T, nh * hd).to(torch.bfloat16).contiguous().to(DEV)
        positions = torch.arange(L - T, L, dtype=torch.int32)
        tiles = torch.tensor([(0, o, min(ops.PREFILL_TILE_TOKENS, T - o)) for o in range(0, T, ops.PREFILL_TILE_TOKENS)],
                             dtype=torch.int32, device=DEV)
        got = ops.attention_prefill(qp, *dev, positions.to(DEV), tiles, kind, window, scale, nh, nkv, hd)
        got = got.float().cpu().view(T, nh, hd)
        for i in (0, 1, T // 2, T - 2, T - 1):
            p = int(positions[i])
            st = _start(p, kind, window)
            ref = _ref_attention(q1, k, v, p, st, scale)
            assert float((got[i] - ref).abs().max()) <= 2e-2, ("prefill", j, p)
            near = float((got[i] - v[j].repeat_interleave(nh // nkv, 0)).abs().max())
            assert (near <= 2e-2) == (st <= j <= p), ("prefill", j, p, near)


@pytest.mark.parametrize("kind,window", [(0, 0), (1, 2048), (2, 3000)])
@pytest.mark.parametrize("ps", [16, 64])
def test_attention_over_thousands_of_keys(kind, window, ps):
    """Contexts of thousands of keys: the prefill kernel holds 128 entries of the block table in
    registers and moves on by 64 as it walks (several times here), the decode kernel splits the keys
    into many runs and the merge kernel adds them.  One key at a time carries all the weight: the
    first, one just before and after each place where the held pages run out, one in the middle
    of nowhere, the last.  Whichever is visible must come back as the value; a key outside the
    window must not."""
    ops = _ops()
    nh, nkv, hd, L = 4, 2, 64, 4300
    scale = 1.0 / math.sqrt(hd)
    g = torch.Generator().manual_seed(ps + kind)
    u = torch.randn(hd, generator=g)
    u = (u / u.norm() * math.sqrt(hd)).to(torch.bfloat16).float()
    q1 = (2.0 * u).expand(nh, hd)
    portion = 130                                   # prefill: a full tile and a partial one at the end
    p_last = L - 1
    edges = [0, 1, 64 * ps - 1, 64 * ps, 128 * ps - 1, 128 * ps, 128 * ps + 1, 192 * ps, 3001, p_last - 2048, p_last - 2999,
             p_last - 3000, L - portion - 1, L - portion, p_last]
    edges = sorted({e for e in edges if 0 <= e < L})
    k0 = torch.randn(L, nkv, hd, generator=g) * 0.05
    v0 = torch.randn(L, nkv, hd, generator=g)
    n = len(edges)
    ks, vs = [], []
    for j in edges:
        k = k0.clone()
        k[j] = 4.0 * u                              # score 8 * hd * scale against ~0: all the weight
        ks.append(k.to(torch.bfloat16).float())
        vs.append(v0.to(torch.bfloat16).float())
    bt, kc, vc = _pages_from(ks, vs, ps, torch.bfloat16, 7)
    bt, kc, vc = bt.to(DEV), kc.to(DEV), vc.to(DEV)
    # decode: one query per request at the last position
    q = q1.to(torch.bfloat16).reshape(1, nh * hd).expand(n, nh * hd).contiguous().to(DEV)
    pos = torch.full((n,), p_last, dtype=torch.int32, device=DEV)
    ent = torch.arange(n, dtype=torch.int32, device=DEV)
    dec = ops.attention_decode(q, kc, vc, bt, ent, pos, None, L, kind, window, scale, nh, nkv, hd).float().cpu().view(n, nh, hd)
    st = _start(p_last, kind, window)
    for i, j in enumerate(edges):
        ref = _ref_attention(q1, ks[i], vs[i], p_last, st, scale)
        assert float((dec[i] - ref).abs().max()) <= 2e-2, ("decode", j)
        near = float((dec[i] - vs[i][j].repeat_interleave(nh // nkv, 0)).abs().max())
        assert (near <= 2e-2) == (st <= j <= p_last), ("decode", j, near)
    # prefill: the last `portion` positions of every request are queries (first and last row checked)
    T = n * portion
    qp = q1.to(torch.bfloat16).reshape(1, nh * hd).expand(T, nh * hd).contiguous().to(DEV)
    ppos = torch.cat([torch.arange(L - portion, L, dtype=torch.int32) for _ in range(n)]).to(DEV)
    tiles = []
    for i in range(n):
        for o in range(0, portion, ops.PREFILL_TILE_TOKENS):
            tiles.append((i, i * portion + o, min(ops.PREFILL_TILE_TOKENS, portion - o)))
    pre = ops.attention_prefill(qp, kc, vc, bt, ppos, torch.tensor(tiles, dtype=torch.int32, device=DEV), kind, window,
                                scale, nh, nkv, hd).float().cpu().view(n, portion, nh, hd)
    for i, j in enumerate(edges):
        for row in (0, 77, portion - 1):
            p = L - portion + row
            stp = _start(p, kind, window)
            ref = _ref_attention(q1, ks[i], vs[i], p, stp, scale)
            assert float((pre[i, row] - ref).abs().max()) <= 2e-2, ("prefill", j, p)
            near = float((pre[i, row] - vs[i][j].repeat_interleave(nh // nkv, 0)).abs().max())
            assert (near <= 2e-2) == (stp <= j <= p), ("prefill", j, p, near)


# ---------------------------------------------------------------------------
# routing and the grouped product for many rows
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("T,E,k,H", [(300, 16, 1, 256), (70, 5, 2, 136), (1, 3, 3, 64), (513, 128, 1, 128), (400, 600, 2, 64)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_router_and_permute(T, E, k, H, dtype):
    ops = _ops()
    x = _rand(T, H, dtype=dtype, seed=T)
    wr = _rand(E, H, dtype=dtype, scale=0.3, seed=E)
    ids, wts, gates = ops.router_topk(x, wr, k, want_gates=True)
    sig = torch.sigmoid(x.float() @ wr.float().T)
    assert float((gates - sig).abs().max()) <= 2e-5
    # picks: descending by the kernel's own gate values, lowest index on ties
    order = torch.sort(gates, dim=1, descending=True, stable=True)
    assert torch.equal(ids.long(), order.indices[:, :k])
    assert torch.equal(wts, order.values[:, :k])
    rt = ops.moe_permute(ids, wts, E)
    off = rt.offsets.cpu().tolist()
    flat = ids.flatten().cpu()
    assert off[0] == 0 and off[-1] == T * k
    counts = torch.bincount(flat.long(), minlength=E).tolist()
    assert [off[e + 1] - off[e] for e in range(E)] == counts
    st, inv, sw = rt.sorted_token.cpu(), rt.inv_pos.cpu().long(), rt.sorted_w.cpu()
    assert sorted(inv.tolist()) == list(range(T * k))
    for e in range(E):
        assert all(int(flat[i]) == e for i in (inv >= off[e]).logical_and(inv < off[e + 1]).nonzero().flatten().tolist())
    assert torch.equal(st[inv].long(), torch.arange(T * k) // k)
    assert torch.equal(sw[inv], wts.flatten().cpu())
    _check_plan(ops, rt, counts)


def _check_plan(ops, rt, counts):
    """The plan of the grouped product for many rows: every group with rows is cut into sibling
    row tiles (as few of the library's tile height as hold its rows) and its column blocks into
    parts (2, 4, 8 or 16: more the more siblings); every (group, part) unit appears once, on one of
    the 8 XCDs, the heaviest units dealt first so that the XCDs' loads stay level.  Behind the
    units lie the ticket counters of the product's blocks, zero when the plan is made."""
    G = len(counts)
    tile = ops._lib.grouped_tile_rows()
    plan = rt.plan.cpu().tolist()
    per_xcd = (16 * G + 7) // 8 + 1
    stride = 1 + 4 * per_xcd
    assert len(plan) == 8 * stride + 16 and plan[8 * stride:] == [0] * 16

    def parts_of(sibs):
        return 2 if sibs <= 2 else 4 if sibs <= 4 else 8 if sibs <= 8 else 16

    seen, loads = [], []
    for x in range(8):
        px = plan[x * stride:(x + 1) * stride]
        units = [tuple(px[1 + 4 * j:5 + 4 * j]) for j in range(px[0])]
        weights = []
        for g, part, parts, sibs in units:
            assert counts[g] > 0 and sibs == -(-counts[g] // tile) and parts == parts_of(sibs) and 0 <= part < parts
            weights.append(sibs * (16 // parts))
        assert weights == sorted(weights, reverse=True)
        seen += [(g, part) for g, part, _, _ in units]
        loads.append(sum(weights))
    want = [(g, part) for g in range(G) if counts[g] > 0 for part in range(parts_of(-(-counts[g] // tile)))]
    assert sorted(seen) == sorted(want)
    heaviest = max([-(-c // tile) * (16 // parts_of(-(-c // tile))) for c in counts if c > 0] + [0])
    assert max(loads) - min(loads) <= heaviest


@pytest.mark.parametrize("counts", [[500, 0, 193, 192, 1, 64, 0, 700], [128] * 16, [3], [0, 0, 5000]])
def test_plan_of_the_grouped_product(counts):
    ops = _ops()
    E = len(counts)
    ids = torch.cat([torch.full((c,), e, dtype=torch.int32) for e, c in enumerate(counts)])
    ids = ids[torch.randperm(len(ids), generator=torch.Generator().manual_seed(1))].view(-1, 1).to(DEV)
    rt = ops.moe_permute(ids, torch.ones(ids.shape, device=DEV), E)
    assert [b - a for a, b in zip(rt.offsets.cpu().tolist(), rt.offsets.cpu().tolist()[1:])] == counts
    _check_plan(ops, rt, counts)
    # with an always-on group behind the experts: one more group, of as many rows as there are tokens
    rt = ops.moe_permute(ids, torch.ones(ids.shape, device=DEV), E, shared_group=True)
    _check_plan(ops, rt, counts + [len(ids)])


@pytest.mark.parametrize("T,H,E,k", [(1, 5120, 16, 1), (8, 5120, 16, 1), (16, 256, 5, 2), (3, 8192, 128, 4), (5, 136, 3, 3)])
@pytest.mark.parametrize("w_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("with_delta", [True, False])
def test_norm_and_router_in_one_launch_equal_the_two_kernels(T, H, E, k, w_dtype, with_delta):
    """Residual add + RMSNorm + router for a few tokens in one launch: the residual stream, the
    normalised rows, the picks and their weights are the bits of the two kernels in a row."""
    ops = _ops()
    h0 = _rand(T, H, seed=T + H)
    delta = _rand(T, H, dtype=torch.bfloat16, scale=0.5, seed=H) if with_delta else None
    wn = (torch.rand(H, generator=torch.Generator().manual_seed(E)) + 0.5).to(w_dtype).to(DEV)
    wr = _rand(E, H, dtype=w_dtype, scale=0.3, seed=E + 1)
    for gate, renorm in ((ops.GATE_SIGMOID, False), (ops.GATE_SOFTMAX, True)):
        ha, hb = h0.clone(), h0.clone()
        xa = ops.add_rmsnorm(ha, delta, wn, 1e-5, torch.bfloat16)
        ia, wa = ops.router_topk(xa, wr, k, gate, renorm)
        xb, ib, wb = ops.add_rmsnorm_router(hb, delta, wn, 1e-5, wr, k, gate, renorm)
        assert torch.equal(ha, hb) and torch.equal(xa, xb) and torch.equal(ia, ib) and torch.equal(wa, wb)
    if with_delta:
        assert not torch.equal(ha, h0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [5120, 136, 75])
def test_router_rows_do_not_depend_on_the_batch(dtype, H):
    """Many tokens share a block of the router kernel (and its fetches of the router's rows); a
    token's gate values are the same bits as when it is routed alone."""
    ops = _ops()
    x = _rand(70, H, dtype=dtype, seed=H)
    wr = _rand(16, H, dtype=dtype, scale=0.3, seed=H + 1)
    ids, wts, gates = ops.router_topk(x, wr, 2, want_gates=True)
    for i in (0, 3, 37, 68, 69):
        ids1, wts1, gates1 = ops.router_topk(x[i:i + 1].contiguous(), wr, 2, want_gates=True)
        assert torch.equal(gates1[0], gates[i]) and torch.equal(ids1[0], ids[i]) and torch.equal(wts1[0], wts[i]), i


def test_router_ties_pick_the_lowest_index():
    ops = _ops()
    x = _rand(4, 64)
    wr = torch.zeros(6, 64, device=DEV)
    ids, wts = ops.router_topk(x, wr, 2)
    assert ids.cpu().tolist() == [[0, 1]] * 4 and float((wts - 0.5).abs().max()) == 0.0


@pytest.mark.parametrize("M,E,I,K", [(8, 4, 40, 128), (64, 16, 264, 256), (33, 5, 8192, 384), (1, 3, 20, 640),
                                     (16, 3, 48, 256), (70, 2, 48, 256)])
def test_gemm_skinny_swiglu_equals_product_then_activation(M, E, I, K):
    """The product with the activation in its epilogue gives the bits of the two kernels in a row."""
    ops = _ops()
    x = _rand(M, K, dtype=torch.bfloat16, seed=M)
    w = _rand(E, 2 * I, K, dtype=torch.bfloat16, scale=0.1, seed=I)
    g = torch.Generator().manual_seed(M + E)
    ex = torch.sort(torch.randint(0, E, (M,), generator=g)).values
    offsets = torch.zeros(E + 1, dtype=torch.int32)
    for e in range(E):
        offsets[e + 1] = offsets[e] + int((ex == e).sum())
    a_rows = torch.randperm(M, generator=g).to(torch.int32).to(DEV)
    scale = (torch.rand(M, generator=g) + 0.25).to(DEV)
    for sc in (scale, None):
        for R, NW in ((2, 4), (2, 8), (4, 4), (4, 8)):
            gu = ops.gemm_skinny(x, w, torch.bfloat16, a_rows=a_rows, offsets=offsets.to(DEV), n_rows=M, R=R, NW=NW)
            want = ops.silu_mul(gu, sc)
            for bound in (None, 32, M):
                got = ops.gemm_skinny_swiglu(x, w, offsets.to(DEV), a_rows, M, sc, R=R, NW=NW, group_rows=bound)
                assert torch.equal(got, want), (R, NW, sc is None, bound)
    # and against the formula
    xs = x[a_rows.long()].float().cpu()
    ref = torch.zeros(M, I)
    off = offsets.tolist()
    for e in range(E):
        rows = slice(off[e], off[e + 1])
        gu = (xs[rows] @ w[e].float().cpu().T).to(torch.bfloat16).float() * scale.cpu()[rows, None]
        ref[rows] = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
    got = ops.gemm_skinny_swiglu(x, w, offsets.to(DEV), a_rows, M, scale).float().cpu()
    assert float((got - ref).abs().max()) <= 2e-2 * float(ref.abs().max())
    if ops.can_pack(w) and (2 * I) % 32 == 0:      # the same from weights stored tile by tile
        pw = ops.pack_weight(w, keep_rows=False)
        for R, NW in ((2, 4), (2, 8), (4, 4), (4, 8)):
            gu = ops.gemm_skinny(x, pw, torch.bfloat16, a_rows=a_rows, offsets=offsets.to(DEV), n_rows=M, R=R, NW=NW)
            got = ops.gemm_skinny_swiglu(x, pw, offsets.to(DEV), a_rows, M, scale, R=R, NW=NW)
            assert torch.equal(got, ops.silu_mul(gu, scale)), (R, NW)
            assert float((got.float().cpu() - ref).abs().max()) <= 2e-2 * float(ref.abs().max())


# (260, ...) are deep enough in K for the kernel's steady loop (and its tail of 4 and of 1 stages); the last two
# make 512 blocks and more, from which on a block takes 256 columns instead of 128 (the others run the narrow form)
@pytest.mark.parametrize("T,E,k,N,K", [(300, 4, 1, 264, 256), (700, 16, 2, 512, 128), (65, 3, 1, 20, 384),
                                       (500, 5, 1, 200, 640), (260, 2, 2, 136, 1216), (500, 5, 1, 208, 640),
                                       (260, 2, 2, 144, 1280), (70, 3, 1, 16, 128), (1700, 2, 1, 264, 256),
                                       (600, 40, 1, 3344, 256), (2500, 16, 2, 3088, 128)])
def test_gemm_grouped(T, E, k, N, K):
    ops = _ops()
    x = _rand(T, K, dtype=torch.bfloat16, seed=1)
    w = _rand(E, N, K, dtype=torch.bfloat16, scale=0.1, seed=2)
    g = torch.Generator().manual_seed(T)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    if E == 4:
        ids[:] = 2                                     # one expert takes everything, the others nothing
    wts = torch.rand(T, k, generator=g).to(DEV)
    rt = ops.moe_permute(ids, wts, E)
    got = ops.gemm_grouped(x, w, rt, True, torch.float32).cpu()
    st = rt.sorted_token.cpu().long()
    off = rt.offsets.cpu().tolist()
    xf, wf = x.float().cpu(), w.float().cpu()
    for e in range(E):
        rows = slice(off[e], off[e + 1])
        ref = xf[st[rows]] @ wf[e].T
        if ref.numel():
            assert float((got[rows] - ref).abs().max()) <= 1e-3 * float(ref.abs().max() + 1e-6), e
    # second product: rows already sorted, bfloat16 out
    y = ops.gemm_grouped(x[st.to(DEV)].contiguous(), w, rt, False, torch.bfloat16).float().cpu()
    assert float((y - got).abs().max()) <= 2e-2 * float(got.abs().max())
    if ops.can_pack(w):                       # the same from weights stored tile by tile: the same sums, the same bits
        pw = ops.pack_weight(w, keep_rows=False)
        assert torch.equal(ops.gemm_grouped(x, pw, rt, True, torch.float32).cpu(), got)


@pytest.mark.parametrize("T,E,k,I,K", [(1, 16, 1, 256, 256), (8, 16, 1, 8192, 640), (16, 4, 4, 128, 384), (5, 3, 2, 128, 128),
                                       (16, 2, 1, 384, 256), (48, 2, 1, 128, 128), (64, 16, 1, 256, 256), (27, 5, 1, 128, 256)])
@pytest.mark.parametrize("packed", [False, True])
def test_picked_products_equal_the_sorted_ones(T, E, k, I, K, packed):
    """The few-rows products that find their rows from the router's picks give, pair by pair, the
    bits of the products over the sorted row list (an expert with every pair, experts with none,
    the always-on expert's rows at the end)."""
    ops = _ops()
    H = K
    x = _rand(T, H, dtype=torch.bfloat16, seed=T)
    wgu = _rand(E + 1, 2 * I, H, dtype=torch.bfloat16, scale=0.1, seed=I)
    wdn = _rand(E + 1, H, I, dtype=torch.bfloat16, scale=0.1, seed=I + 1)
    if packed:
        if not (ops.can_pack(wgu) and ops.can_pack(wdn) and (2 * I) % 32 == 0):
            pytest.skip("sizes that are not stored tile by tile")
        wgu_f, wdn_f = ops.pack_weight(wgu, keep_rows=False), ops.pack_weight(wdn, keep_rows=False)
    else:
        wgu_f, wdn_f = wgu, wdn
    g = torch.Generator().manual_seed(T + E)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    if E == 2:
        ids[:] = 1                                         # one expert takes every pair
    ids = ids.to(DEV)
    wts = torch.rand(T, k, generator=g).to(DEV)
    rt = ops.moe_permute(ids, wts, E, True)
    act_s = ops.gemm_skinny_swiglu(x, wgu_f, rt.offsets, rt.sorted_token, rt.n_rows, rt.sorted_w, group_rows=T)
    y_s = ops.gemm_skinny(act_s, wdn_f, torch.bfloat16, offsets=rt.offsets, n_rows=rt.n_rows, group_rows=T)
    act_p = ops.gemm_skinny_picked(x, wgu_f, ids, wts, True, True, True, torch.bfloat16)
    y_p = ops.gemm_skinny_picked(act_p, wdn_f, ids, None, True, False, False, torch.bfloat16)
    inv = rt.inv_pos.long()
    assert torch.equal(act_p[:T * k], act_s[inv]) and torch.equal(act_p[T * k:], act_s[T * k:])
    assert torch.equal(y_p[:T * k], y_s[inv]) and torch.equal(y_p[T * k:], y_s[T * k:])
    # and the sums the next norm forms from either are the same
    a = ops.ExpertSum(y_p, ops.counting(T * k, y_p.device), y_p[T * k:], T, k).tensor()
    b = ops.ExpertSum(y_s, rt.inv_pos, y_s[T * k:], T, k).tensor()
    assert torch.equal(a, b)
    # without the always-on expert
    y1 = ops.gemm_skinny_picked(x, ops.PackedWeight(wgu_f.packed[:E], None) if packed else wgu[:E], ids, None, False, True, False,
                                torch.float32)
    ref = torch.stack([x[i // k].float() @ wgu[int(ids.flatten()[i])].float().T for i in range(T * k)])
    assert float((y1 - ref).abs().max()) <= 1e-3 * float(ref.abs().max())


@pytest.mark.parametrize("T,E,k,I,K", [(300, 4, 1, 128, 256), (700, 16, 2, 272, 128), (65, 3, 1, 16, 384),
                                       (500, 5, 1, 112, 640), (260, 2, 2, 80, 1216), (430, 3, 1, 8192, 128)])
def test_gemm_grouped_swiglu_equals_product_then_activation(T, E, k, I, K):
    """The many-rows product with the activation in its epilogue gives the bits of the two kernels
    in a row, from weights stored row by row and tile by tile (column blocks that end inside a
    block of the kernel, experts with no row, with one tile and with several)."""
    ops = _ops()
    x = _rand(T, K, dtype=torch.bfloat16, seed=3)
    w = _rand(E, 2 * I, K, dtype=torch.bfloat16, scale=0.1, seed=4)
    g = torch.Generator().manual_seed(T)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    if E == 4:
        ids[:] = 2
    wts = torch.rand(T, k, generator=g).to(DEV)
    rt = ops.moe_permute(ids, wts, E)
    for scale in (rt.sorted_w, None):
        want = ops.silu_mul(ops.gemm_grouped(x, w, rt, True, torch.bfloat16), scale)
        got = ops.gemm_grouped_swiglu(x, w, rt, scale)
        assert got.shape == (T * k, I) and torch.equal(got, want)
        if ops.can_pack(w):
            assert torch.equal(ops.gemm_grouped_swiglu(x, ops.pack_weight(w, keep_rows=False), rt, scale), want)
    # the same numbers as the float product followed by the activation, to bfloat16's rounding
    gu = ops.gemm_grouped(x, w, rt, True, torch.float32).cpu()
    s = rt.sorted_w.cpu()[:, None]
    ga, up = (gu[:, :I] * s), (gu[:, I:] * s)
    ref = ga / (1 + torch.exp(-ga)) * up
    assert float((ops.gemm_grouped_swiglu(x, w, rt, rt.sorted_w).float().cpu() - ref).abs().max()) <= 3e-2 * float(ref.abs().max() + 1e-6)


@pytest.mark.parametrize("T,E,N,K", [(900, 6, 1024, 256), (2100, 16, 2560, 128), (70, 3, 48, 128)])
def test_gemm_grouped_gives_the_same_bits_however_many_blocks_take_the_work(T, E, N, K):
    """The many-rows product's blocks stay and take slots from ticket counters that lie behind the
    plan; the slots of a last, partly filled round are cut by columns.  Every output is one chain
    over k whoever computes it: any bound on the number of blocks gives the same bits (a single
    block walks every XCD's slots alone, cut otherwise than 256 blocks cut them), the counters are
    back at zero after every launch, and the loads are very uneven on purpose."""
    ops = _ops()
    x = _rand(T, K, dtype=torch.bfloat16, seed=5)
    w = _rand(E, N, K, dtype=torch.bfloat16, scale=0.1, seed=6)
    g = torch.Generator().manual_seed(T)
    p = torch.tensor([float(2 ** (e % 5)) for e in range(E)])
    ids = torch.multinomial(p / p.sum(), T, replacement=True, generator=g).to(torch.int32).view(T, 1).to(DEV)
    rt = ops.moe_permute(ids, torch.ones(T, 1, device=DEV), E)
    counters = rt.plan[-16:]
    want = None
    for form in (w, ops.pack_weight(w, keep_rows=False)):
        for blocks in (0, 1, 3, 8, 37, 100):
            got = ops.gemm_grouped(x, form, rt, True, torch.bfloat16, max_blocks=blocks)
            assert not bool(counters.any()), "the ticket counters were not set back"
            if want is None:
                want = got
                off = rt.offsets.cpu().tolist()
                st = rt.sorted_token.cpu().long()
                for e in range(E):
                    rows = st[off[e]:off[e + 1]]
                    ref = x.cpu().float()[rows] @ w[e].cpu().float().T
                    assert float((got[off[e]:off[e + 1]].cpu().float() - ref).abs().max()) <= 2e-2 * float(ref.abs().max() + 1e-6), e
            assert torch.equal(got, want), blocks
    if N % 32 == 0:
        want = ops.gemm_grouped_swiglu(x, w, rt, rt.sorted_w)
        for blocks in (1, 5, 64):
            assert torch.equal(ops.gemm_grouped_swiglu(x, w, rt, rt.sorted_w, max_blocks=blocks), want), blocks
        assert not bool(counters.any())


_PREFILL_CASES = [(nh, nkv, hd, kind, window, ps)
                  for nh, nkv, hd in [(8, 2, 64), (5, 5, 32), (40, 8, 128), (3, 1, 96)]
                  for kind, window in [(0, 0), (1, 24), (1, 100), (2, 50)] for ps in (16, 32)]
_PREFILL_CASES += [(2, 1, 160, 1, 100, 16), (3, 3, 160, 0, 0, 32), (6, 2, 192, 2, 50, 16), (2, 2, 192, 1, 24, 32)]


@pytest.mark.parametrize("nh,nkv,hd,kind,window,ps", _PREFILL_CASES)
def test_attention_prefill_kernel(nh, nkv, hd, kind, window, ps):
    """Portions of several requests at different starting positions, against dense softmax."""
    ops = _ops()
    assert ops.prefill_attention_ok(torch.bfloat16, hd)
    ctx_lens = [70, 300, 33, 129]          # context after the portion
    portion = [70, 45, 2, 100]             # the last `portion` tokens are this step's queries
    bt, kc, vc, ks, vs = _paged_case(ctx_lens, nh, nkv, hd, ps, torch.bfloat16, seed=nh + hd + ps, strong_key=5)
    g = torch.Generator().manual_seed(9)
    T = sum(portion)
    q = torch.randn(T, nh, hd, generator=g).to(torch.bfloat16)
    positions, tiles, ref = [], [], []
    scale = 1.0 / math.sqrt(hd)
    tok = 0
    for e, (L, n) in enumerate(zip(ctx_lens, portion)):
        for o in range(0, n, ops.PREFILL_TILE_TOKENS):
            tiles.append((e, tok + o, min(ops.PREFILL_TILE_TOKENS, n - o)))
        for i in range(n):
            p = L - n + i
            positions.append(p)
            ref.append(_ref_attention(q[tok + i].float(), ks[e], vs[e], p, _start(p, kind, window), scale))
        tok += n
    ref = torch.stack(ref)
    got = ops.attention_prefill(q.reshape(T, nh * hd).to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV),
                                torch.tensor(positions, dtype=torch.int32, device=DEV),
                                torch.tensor(tiles, dtype=torch.int32, device=DEV), kind, window, scale, nh, nkv, hd)
    # tiles of half the rows (what a step with few prompt tokens is cut into): every row keeps its bits
    half = ops.PREFILL_TILE_TOKENS // 2
    tiles64 = [(e, t0 + o, min(half, n - o)) for e, t0, n in tiles for o in range(0, n, half)]
    got64 = ops.attention_prefill(q.reshape(T, nh * hd).to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV),
                                  torch.tensor(positions, dtype=torch.int32, device=DEV),
                                  torch.tensor(tiles64, dtype=torch.int32, device=DEV), kind, window, scale, nh, nkv, hd,
                                  tile_tokens=half)
    assert torch.equal(got64, got)
    with pytest.raises(Exception):    # a tile size the kernel has no form for is refused
        ops.attention_prefill(q.reshape(T, nh * hd).to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV),
                              torch.tensor(positions, dtype=torch.int32, device=DEV),
                              torch.tensor(tiles64, dtype=torch.int32, device=DEV), kind, window, scale, nh, nkv, hd,
                              tile_tokens=32)
    got = got.float().cpu().view(T, nh, hd)
    err = (got - ref).abs().max(dim=-1).values.max(dim=-1).values
    assert float(err.max()) <= 2e-2, (float(err.max()), int(err.argmax()))


# ---------------------------------------------------------------------------
# row kernels, at widths with and without 16-byte runs
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("H", [80, 203, 1000, 5120, 9000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm_kernel(H, dtype):
    ops = _ops()
    T = 7
    h = _rand(T, H, seed=1)
    delta = _rand(T, H, dtype=dtype, seed=2)
    w = (torch.rand(H) + 0.5).to(DEV)
    want_sum = h + delta.float()
    want = want_sum * torch.rsqrt(want_sum.pow(2).mean(-1, keepdim=True) + 1e-5) * w
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for wt in (w, w.to(torch.bfloat16)):
        hh = h.clone()
        out = ops.add_rmsnorm(hh, delta, wt, 1e-5, dtype)
        ref = want if wt.dtype == torch.float32 else want / w * wt.float()
        assert float((out.float() - ref).abs().max()) <= tol * float(ref.abs().max())
        assert torch.allclose(hh, want_sum, atol=1e-6)               # the sum went back into the stream
    hh = h.clone()
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    out = ops.add_rmsnorm(hh, delta, None, 1e-5, dtype, rows=rows)
    assert torch.equal(hh, h)                                        # gathered rows leave the stream alone
    assert float((out.float() - (want / w)[[5, 0, 5]]).abs().max()) <= tol * float(want.abs().max())
    plain = ops.add_rmsnorm(h.clone(), None, w, 1e-5, torch.float32)
    assert torch.allclose(plain, h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + 1e-5) * w, atol=1e-5)


@pytest.mark.parametrize("I", [48, 77, 8192])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_silu_mul_and_combine_and_embed(I, dtype):
    ops = _ops()
    M = 9
    gu = _rand(M, 2 * I, dtype=dtype, seed=3)
    scale = torch.rand(M).to(DEV) + 0.2
    g, u = gu.float()[:, :I], gu.float()[:, I:]
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    got = ops.silu_mul(gu).float()
    assert float((got - torch.nn.functional.silu(g) * u).abs().max()) <= tol * 4
    got = ops.silu_mul(gu, scale).float()
    gs, us = g * scale[:, None], u * scale[:, None]
    assert float((got - torch.nn.functional.silu(gs) * us).abs().max()) <= tol * 4
    # combine: 3 tokens, 2 picks each, plus a shared row
    y = _rand(6, I, dtype=dtype, seed=4)
    sh = _rand(3, I, dtype=dtype, seed=5)
    inv = torch.tensor([4, 1, 0, 5, 2, 3], dtype=torch.int32, device=DEV)
    got = ops.moe_combine(y, inv, sh, 3, 2).float()
    want = y.float()[inv.long()].view(3, 2, I).sum(1) + sh.float()
    assert float((got - want).abs().max()) <= tol * 4
    assert float((ops.moe_combine(y, inv, None, 3, 2).float() - (want - sh.float())).abs().max()) <= tol * 4
    table = _rand(50, I, dtype=dtype, seed=6)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.embed_gather(ids, table), table.float()[ids.long()])
    assert torch.equal(ops.embed_gather(ids, table, scale=2.5), table.float()[ids.long()] * 2.5)
    lg = _rand(3, 77, scale=9.0, seed=7)
    assert float((ops.scale_softcap(lg.clone(), 0.5, 3.0) - 3.0 * torch.tanh(lg * 0.5 / 3.0)).abs().max()) <= 1e-5
    assert torch.equal(ops.scale_softcap(lg.clone(), 2.0), lg * 2.0)


@pytest.mark.parametrize("nh,nkv,hd", [(4, 2, 16), (6, 3, 32), (5, 5, 48), (40, 8, 128)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode", ["rope+norm", "rope", "temperature", "bare"])
def test_rope_kv_kernel(nh, nkv, hd, dtype, mode):
    ops = _ops()
    import plain_llama4 as P

    T, ps, pages = 11, 16, 6
    qkv = _rand(T, (nh + 2 * nkv) * hd, dtype=dtype, seed=hd)
    positions = torch.tensor([0, 1, 2, 17, 31, 32, 100, 1000, 4095, 70000, 5], dtype=torch.int32)
    slots = torch.tensor([0, 1, 2, 33, 47, 64, 20, 21, 95, 50, -1], dtype=torch.int32)   # the last one stores nothing
    inv = P.rope_inv_freq(hd, 500000.0, None) if mode.startswith("rope") else None
    kc = torch.zeros(pages, nkv, ps, hd, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, nkv, hd, ps, dtype=dtype, device=DEV)
    q = ops.rope_kv(qkv, kc, vc, slots.to(DEV), positions.to(DEV), inv.to(DEV) if inv is not None else None,
                    mode == "rope+norm", 1e-5, (32.0, 0.2) if mode == "temperature" else None, nh, nkv, hd)
    x = qkv.float().cpu().view(T, nh + 2 * nkv, hd)
    qr, kr, vr = x[:, :nh], x[:, nh:nh + nkv], x[:, nh + nkv:]
    if inv is not None:
        qr, kr = P.apply_rope_interleaved(qr, positions, inv), P.apply_rope_interleaved(kr, positions, inv)
    if mode == "rope+norm":
        qr, kr = P.l2_head_norm(qr, 1e-5), P.l2_head_norm(kr, 1e-5)
    if mode == "temperature":
        qr = qr * P.query_temperature(positions, 32.0, 0.2)[:, None, None]
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    scale = max(1.0, float(qr.abs().max()))
    assert float((q.float().cpu().view(T, nh, hd) - qr).abs().max()) <= tol * scale
    kcc, vcc = kc.float().cpu(), vc.float().cpu()
    for t in range(T - 1):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        assert float((kcc[page, :, off, :] - kr[t]).abs().max()) <= tol * scale, t
        assert float((vcc[page, :, :, off] - vr[t]).abs().max()) <= tol * scale, t
    written = torch.zeros(pages * ps, dtype=torch.bool)
    written[slots[:-1].long()] = True
    assert float(kcc.permute(0, 2, 1, 3).reshape(pages * ps, -1)[~written].abs().max()) == 0.0


def _rotate_plain(x, positions, inv_freq, layout):
    """x [T, heads, hd]: the first 2 * len(inv_freq) elements of every head rotated by
    pos * freq_i, on pairs (2i, 2i+1) ("interleaved") or (i, i + r/2) ("half"); the rest as it is."""
    r = 2 * inv_freq.shape[0]
    ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if layout == "interleaved":
        a, b = x[..., 0:r:2], x[..., 1:r:2]
        out[..., 0:r:2], out[..., 1:r:2] = a * cos - b * sin, a * sin + b * cos
    else:
        a, b = x[..., :r // 2], x[..., r // 2:r]
        out[..., :r // 2], out[..., r // 2:r] = a * cos - b * sin, a * sin + b * cos
    return out


@pytest.mark.parametrize("hd,rotary_dim", [(16, 16), (32, 16), (48, 20), (64, 64), (128, 64), (128, 24)])
@pytest.mark.parametrize("layout", ["interleaved", "half"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_kv_kernel_pair_layouts_and_partial_width(hd, rotary_dim, layout, dtype):
    """The pairing and the rotated width are arguments of the kernel: half-split pairs, and heads
    of which only the first elements rotate (the norm still runs over the whole head)."""
    ops = _ops()
    import plain_llama4 as P
    from sharpinference_amd.parts.position import Rotary

    nh, nkv, T, ps, pages = 3, 1, 9, 16, 4
    rot = Rotary(hd, 10000.0, None, pair_layout=layout, rotary_dim=rotary_dim)
    inv = rot.frequencies()
    assert inv.shape == (rotary_dim // 2,)
    assert torch.allclose(inv, P.rope_inv_freq(rotary_dim, 10000.0, None))
    qkv = _rand(T, (nh + 2 * nkv) * hd, dtype=dtype, seed=hd + rotary_dim)
    positions = torch.tensor([0, 1, 2, 17, 31, 100, 1000, 4095, 5], dtype=torch.int32)
    slots = torch.arange(T, dtype=torch.int32) + 3
    kc = torch.zeros(pages, nkv, ps, hd, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, nkv, hd, ps, dtype=dtype, device=DEV)
    q = ops.rope_kv(qkv, kc, vc, slots.to(DEV), positions.to(DEV), inv.to(DEV), True, 1e-5, None, nh, nkv, hd,
                    ops.PAIRS_HALF_SPLIT if layout == "half" else ops.PAIRS_INTERLEAVED)
    x = qkv.float().cpu().view(T, nh + 2 * nkv, hd)
    qr = P.l2_head_norm(_rotate_plain(x[:, :nh], positions, inv, layout), 1e-5)
    kr = P.l2_head_norm(_rotate_plain(x[:, nh:nh + nkv], positions, inv, layout), 1e-5)
    if layout == "interleaved" and rotary_dim == hd:      # the plain model's own rotation is this case
        assert torch.allclose(_rotate_plain(x[:, :nh], positions, inv, layout), P.apply_rope_interleaved(x[:, :nh], positions, inv))
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    assert float((q.float().cpu().view(T, nh, hd) - qr).abs().max()) <= tol * max(1.0, float(qr.abs().max()))
    kcc = kc.float().cpu()
    for t in range(T):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        assert float((kcc[page, :, off, :] - kr[t]).abs().max()) <= tol * max(1.0, float(kr.abs().max())), t
    # the two pairings differ (a kernel that ignored the argument would pass one of them only)
    if rotary_dim > 2:
        other = _rotate_plain(x[:, :nh], positions, inv, "half" if layout == "interleaved" else "interleaved")
        assert float((other - _rotate_plain(x[:, :nh], positions, inv, layout)).abs().max()) > 0.1


@pytest.mark.parametrize("nh,nkv,hd", [(3, 1, 48), (6, 3, 32), (5, 5, 128)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_kv_kernel_adds_the_projections_biases_first(nh, nkv, hd, dtype):
    """A bias on q, k and v is added to each token's row before anything else (in float): the result
    is what the kernel gives for rows that already hold the sum, to the rounding of one more store."""
    ops = _ops()
    import plain_llama4 as P

    T, ps, pages = 7, 16, 3
    qkv = _rand(T, (nh + 2 * nkv) * hd, dtype=dtype, seed=hd)
    bias = _rand((nh + 2 * nkv) * hd, seed=hd + 1)
    positions = torch.tensor([0, 1, 5, 17, 31, 100, 4095], dtype=torch.int32)
    slots = torch.tensor([0, 1, 2, 33, 47, 20, 21], dtype=torch.int32)
    inv = P.rope_inv_freq(hd, 10000.0, None)
    kc = torch.zeros(pages, nkv, ps, hd, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, nkv, hd, ps, dtype=dtype, device=DEV)
    q = ops.rope_kv(qkv, kc, vc, slots.to(DEV), positions.to(DEV), inv.to(DEV), True, 1e-5, None, nh, nkv, hd, bias=bias)
    x = (qkv.float().cpu() + bias.cpu()).view(T, nh + 2 * nkv, hd)
    qr = P.l2_head_norm(P.apply_rope_interleaved(x[:, :nh], positions, inv), 1e-5)
    kr = P.l2_head_norm(P.apply_rope_interleaved(x[:, nh:nh + nkv], positions, inv), 1e-5)
    vr = x[:, nh + nkv:]
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    assert float((q.float().cpu().view(T, nh, hd) - qr).abs().max()) <= tol * max(1.0, float(qr.abs().max()))
    kcc, vcc = kc.float().cpu(), vc.float().cpu()
    for t in range(T):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        assert float((kcc[page, :, off, :] - kr[t]).abs().max()) <= tol * max(1.0, float(kr.abs().max())), t
        assert float((vcc[page, :, :, off] - vr[t]).abs().max()) <= tol * max(1.0, float(vr.abs().max())), t
    # without the bias the queries differ (a kernel that ignored the argument fails)
    q0 = ops.rope_kv(qkv, kc.clone(), vc.clone(), slots.to(DEV), positions.to(DEV), inv.to(DEV), True, 1e-5, None, nh, nkv, hd)
    assert float((q0.float() - q.float()).abs().max()) > 0.05


@pytest.mark.parametrize("T,N", [(1, 5), (9, 76), (130, 512)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_bias_rows(T, N, dtype):
    ops = _ops()
    x = _rand(T, N, dtype=dtype, seed=T)
    b = _rand(N, seed=N)
    want = (x.float() + b).to(dtype)
    got = ops.add_bias(x.clone(), b)
    assert torch.equal(got, want)


@pytest.mark.parametrize("M,N,K", [(1, 5, 3), (70, 130, 50), (64, 64, 16), (129, 203, 96)])
def test_gemm_tiled_is_a_true_float_product_and_batch_invariant(M, N, K):
    ops = _ops()
    x, w = _rand(M, K, seed=1), _rand(N, K, seed=2)
    got = ops.gemm_tiled(x, w)
    want = (x.double() @ w.double().T).float()
    assert float((got - want).abs().max()) <= 2e-6 * K * float(want.abs().max() + 1)
    # values that bfloat16 or tf32 products would lose
    a = torch.tensor([[1.0, 2.0 ** -20]], device=DEV)
    b = torch.tensor([[1.0, 1.0]], device=DEV)
    assert float(ops.gemm_tiled(a, b)[0, 0]) == 1.0 + 2.0 ** -20
    if M > 1:
        assert torch.equal(ops.gemm_tiled(x[:1].contiguous(), w), got[:1])
        assert torch.equal(ops.gemm_tiled(x[M // 2:].contiguous(), w), got[M // 2:])


def test_the_library_says_which_head_sizes_its_attention_kernels_take():
    """The choice between the matrix-core kernels and the generic one asks the library: a head size is
    either compiled or goes to the generic kernel, which takes every size up to 256."""
    ops = _ops()
    assert [hd for hd in range(16, 273, 16) if ops.decode_attention_ok(torch.bfloat16, hd)] == [32, 64, 96, 128, 160, 192, 224, 256]
    assert [hd for hd in range(16, 273, 16) if ops.prefill_attention_ok(torch.bfloat16, hd)] == [32, 64, 96, 128, 160, 192]
    assert not ops.decode_attention_ok(torch.float32, 128) and not ops.prefill_attention_ok(torch.float32, 128)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_random_fill_on_the_device_equals_the_host(dtype):
    """Seeded random weights are a function of (seed, name, element): the device's fill kernel and
    the host give the same bits, so a model made in device memory is the model a file written on
    the host from the same seed holds."""
    ops = _ops()
    from sharpinference_amd.weights import random_fill as rf

    for name, shape, kind, std in (("a.weight", (3, 1001), rf.FILL_NORMAL, 0.02), ("b", (70001,), rf.FILL_NORMAL, 1.0),
                                   ("norm.weight", (5120,), rf.FILL_UNIFORM, 0.0)):
        key = rf.name_key(7, name)
        dev = ops.random_fill(torch.empty(shape, dtype=dtype, device=DEV), key, kind, std).cpu()
        host = rf.host_tensor(shape, key, kind, dtype, std)
        assert torch.equal(dev, host), name
    ints = ops.random_fill(torch.empty(999, dtype=torch.int32, device=DEV), rf.name_key(7, "i"), rf.FILL_INT).cpu()
    assert torch.equal(ints, rf.host_tensor((999,), rf.name_key(7, "i"), rf.FILL_INT, torch.int32))
    x = rf.host_tensor((200000,), rf.name_key(1, "x"), rf.FILL_NORMAL, torch.float32, 0.5)
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 0.5) < 0.01
    u = rf.host_tensor((50000,), rf.name_key(1, "u"), rf.FILL_UNIFORM, torch.float32)
    assert 0.9 <= float(u.min()) and float(u.max()) < 1.1 and abs(float(u.mean()) - 1.0) < 0.005


def test_a_model_made_on_the_device_is_the_model_written_on_the_host(tmp_path):
    from sharpinference_amd import load_config
    from sharpinference_amd.engine import Engine, StepEntry
    from sharpinference_amd.weights.loader import write_random_model
    from tiny_configs import CONFIGS

    cfg = load_config(CONFIGS["D"])
    d = write_random_model(cfg, str(tmp_path / "m"), 4, std=0.06)
    toks = [5, 17, 3, 99, 200, 41, 8, 8]
    out = []
    for eng in (Engine(d, dtype="bfloat16", kv_tokens=64, max_num_seqs=1),
                Engine(config=cfg, weight_seed=4, weight_std=0.06, dtype="bfloat16", kv_tokens=64, max_num_seqs=1)):
        eng.add_request("r")
        out.append(eng.step([StepEntry("r", toks, list(range(len(toks))))]))
    assert torch.equal(out[0], out[1])


@pytest.mark.parametrize("M,N,K", [(70, 272, 256), (200, 528, 640), (200, 512, 256), (384, 5120, 256), (500, 5120, 1280)])
def test_plain_products_of_many_rows_through_the_grouped_kernel(M, N, K):
    """A matrix kept only in the packed order is multiplied by many rows in the grouped kernel,
    the whole matrix as its one group (rows in their own order); with SwiGLU in the epilogue it
    gives the bits of the product followed by the activation kernel."""
    ops = _ops()
    x = _rand(M, K, dtype=torch.bfloat16, seed=M)
    w = _rand(N, K, dtype=torch.bfloat16, scale=0.1, seed=N)
    pw = ops.pack_weight(w, keep_rows=False)
    assert pw.rows is None
    ref = x.float() @ w.float().T
    for out_dtype, tol in ((torch.float32, 1e-3), (torch.bfloat16, 2e-2)):
        got = ops.linear(x, pw, out_dtype)          # no row-major copy: this library's kernels, whatever the row count
        assert got.dtype == out_dtype and float((got.float() - ref).abs().max()) <= tol * float(ref.abs().max())
    few = ops.linear(x[:40].contiguous(), pw, torch.float32)       # 17 to 64 rows: the few-rows kernel
    assert float((few - ref[:40]).abs().max()) <= 1e-3 * float(ref.abs().max())
    if N % 32 == 0:
        act = ops.swiglu_many_rows(x, pw)
        assert torch.equal(act, ops.silu_mul(ops.linear_many_rows(x, pw, torch.bfloat16)))


def test_an_engine_that_keeps_only_packed_weights_gives_the_same_logits(tmp_path):
    from sharpinference_amd.engine import Engine, StepEntry
    from tiny_configs import make_model_dir

    d = make_model_dir(tmp_path, "D", std=0.06)
    toks = [int(t) for t in torch.randint(0, 500, (450,), generator=torch.Generator().manual_seed(3))]
    out = []
    for copies in (True, False):
        eng = Engine(d, dtype="bfloat16", kv_tokens=512, max_num_seqs=1, row_major_copies=copies)
        assert (eng.model.blocks[0].mixer.w_qkv.rows is not None) == copies
        eng.add_request("r")
        # 420 rows: three row tiles side by side in the grouped kernel
        out.append(eng.step([StepEntry("r", toks[:420], list(range(420)))]).float().cpu())
        out.append(eng.step([StepEntry("r", toks[420:421], [0])]).float().cpu())      # a decode step: the same kernel either way
    rms = out[0].pow(2).mean().sqrt()
    assert float((out[0] - out[2]).abs().max()) <= 0.1 * float(rms)        # other kernels at prompt size: roundings apart
    assert float((out[1] - out[3]).abs().max()) <= 0.1 * float(rms)
