"""Each mechanism of the Nufavik layers alone: the kernel against the plain implementation's function of the same
mechanism (or a few lines of 64-bit torch), in float32 and bfloat16."""
import math

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import nufavik_plain as N

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    from qwen_engine_amd.kernels import ops as o
    return o


def rel(got, want):
    return float((got.double().cpu() - want.double()).abs().max()) / max(float(want.abs().max()), 1e-30)


def test_stream_scale():
    x = torch.randn(7, 100)
    xs = x.to(DEV)
    ops().scale_(xs, 0.37)
    assert torch.equal(xs.cpu(), x * torch.tensor(0.37))


# ---- convolution of q | k | v, rotation, cache write, state -----------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 6e-3)])
@pytest.mark.parametrize("taps,hq,hkv,dk,dv,dc,dims,page", [(3, 4, 2, 16, 24, 64, 8, 8), (1, 2, 2, 32, 8, 64, 32, 4),
                                                            (5, 3, 1, 8, 80, 128, 0, 16), (2, 8, 2, 64, 64, 64, 62, 16),
                                                            (4, 1, 1, 128, 96, 128, 128, 16)])
@pytest.mark.parametrize("with_transposed", [False, True])
def test_convolution_rotation_and_cache_write_across_cuts_and_between_requests(dtype, tol, taps, hq, hkv, dk, dv, dc, dims, page, with_transposed):
    """Three requests whose rows are cut into steps of unequal portions (down to one row, with other requests' rows
    between them), each with a state slot and scattered cache slots of its own: q, the cache's key rows and value
    columns (zeros beyond a head's own numbers) and the state are what the whole sequences give."""
    g = torch.Generator().manual_seed(taps * 100 + hq)
    C = hq * dk + hkv * (dk + dv)
    lengths = {0: 23 + 40, 1: 9, 2: 14 + 19}
    u = {s: (torch.randn(n, C, generator=g)).to(dtype) for s, n in lengths.items()}
    w = torch.randn(C, taps, generator=g) * 0.6
    base = 100.0
    inv_freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64).float() if dims else None
    start = {0: 0, 1: 5, 2: 130}          # request 1 and 2 as if they began earlier (their states given below)
    pages = 40
    cache = torch.full((pages, 2, hkv, page, dc), float("nan"), dtype=dtype, device=DEV)
    state = torch.zeros(4, max(taps - 1, 1), C, device=DEV) if taps > 1 else None
    hist = {s: (torch.randn(taps - 1, C, generator=g)).to(dtype) if (taps > 1 and start[s] > 0) else torch.zeros(max(taps - 1, 0), C).to(dtype)
            for s in lengths}
    slot_row = {0: 2, 1: 0, 2: 3}
    if taps > 1:
        for s in lengths:
            state[slot_row[s]] = hist[s].float().to(DEV)
    # what the whole sequences give
    want_q, want_k, want_v = {}, {}, {}
    for s, n in lengths.items():
        full = torch.cat([hist[s].double(), u[s].double()])
        y = N.causal_conv(full, w.double())[len(hist[s]):] if taps > 1 else u[s].double() * w.double()[:, 0]
        pos = torch.arange(start[s], start[s] + n)
        q = y[:, :hq * dk].reshape(n, hq, dk)
        k = y[:, hq * dk:(hq + hkv) * dk].reshape(n, hkv, dk)
        want_q[s] = N.rotate_half_split(q, pos, base, dims)
        want_k[s] = N.rotate_half_split(k, pos, base, dims)
        want_v[s] = y[:, (hq + hkv) * dk:].reshape(n, hkv, dv)
    perm = torch.randperm(pages * page, generator=g).tolist()
    slot_of = {}
    # (steps of more than 16 rows go to the kernel for many rows, with a request's rows crossing its tiles of 16)
    steps = [[(0, 5), (1, 1), (2, 2)], [(1, 1), (0, 1)], [(2, 12), (0, 2), (1, 7)], [(0, 15)], [(2, 19), (0, 40)]]
    done = {s: 0 for s in lengths}
    got_q = {s: [] for s in lengths}
    for step in steps:
        rows, seq, pos, slots, owner = [], [], [], [], []
        for s, n in step:
            rows.append(u[s][done[s]:done[s] + n])
            for i in range(n):
                p = done[s] + i
                seq.append(slot_row[s])
                pos.append(start[s] + p)
                slot_of[(s, p)] = perm.pop()
                slots.append(slot_of[(s, p)])
                owner.append(s)
            done[s] += n
        single = all(n == 1 for _, n in step)
        q = ops().qkv_conv_rope_store(torch.cat(rows).to(DEV), w.to(DEV), state, torch.tensor(seq, dtype=torch.int32, device=DEV),
                                      torch.tensor(pos, dtype=torch.int32, device=DEV),
                                      inv_freq.to(DEV) if inv_freq is not None else None,
                                      torch.tensor(slots, dtype=torch.int32, device=DEV), cache, hq, hkv, dk, dv, single_rows=single,
                                      conv_w_t=w.t().contiguous().to(DEV) if with_transposed else None)
        for i, s in enumerate(owner):
            got_q[s].append(q[i].cpu())
    vt = cache[:, 1].reshape(pages, hkv, dc, page).cpu()
    kt = cache[:, 0].cpu()
    for s, n in lengths.items():
        gq = torch.stack(got_q[s])
        assert rel(gq[:, :, :dk], want_q[s]) < tol
        assert dc == dk or float(gq[:, :, dk:].abs().max()) == 0.0
        for p in range(n):
            pg, off = divmod(slot_of[(s, p)], page)
            assert rel(kt[pg, :, off, :dk], want_k[s][p]) < tol, (s, p)
            assert rel(vt[pg, :, :dv, off], want_v[s][p]) < tol, (s, p)
            assert dc == dk or float(kt[pg, :, off, dk:].abs().max()) == 0.0
            assert dc == dv or float(vt[pg, :, dv:, off].abs().max()) == 0.0
        if taps > 1:
            last = torch.cat([hist[s].float(), u[s].float()])[-(taps - 1):]
            assert torch.equal(state[slot_row[s]].cpu(), last), s


# ---- attention: window, kept first keys, sink ---------------------------------------------------------------------------
def _paged(k, v, page, seed, dtype, extra=3):
    """k, v [L, Hkv, D] -> (cache [pages, 2, Hkv, P, D] with shuffled pages, block table row)."""
    L, hkv, d = k.shape
    n = (L + page - 1) // page
    g = torch.Generator().manual_seed(seed)
    ids = torch.randperm(n + extra, generator=g)[:n]
    cache = torch.full((n + extra, 2, hkv, page, d), float("nan")).to(dtype)
    vt = cache[:, 1].view(-1, hkv, d, page)
    for pos in range(L):
        cache[ids[pos // page], 0, :, pos % page] = k[pos]
        vt[ids[pos // page], :, :, pos % page] = v[pos]
    return cache, ids.to(torch.int32)


def _plain_attention(q, k, v, pos, scale, size, keep, sink):
    """q [n, Hq, D] at positions pos; k, v [L, Hkv, D] (64-bit)."""
    n, hq, d = q.shape
    G = hq // k.shape[1]
    out = torch.zeros(n, hq, d, dtype=torch.float64)
    for i in range(n):
        js = [j for j in range(k.shape[0]) if N.sees(int(pos[i]), j, size if size else 1 << 30, keep)]
        for h in range(hq):
            s = (k[js, h // G] @ q[i, h]) * scale
            p = N.softmax_with_sink(s) if sink else torch.softmax(s, 0)
            out[i, h] = p @ v[js, h // G]
    return out


CASES = [  # window, kept first keys, sink
    (41, 5, True), (41, 0, True), (0, 0, True), (16, 16, False), (17, 33, True), (150, 140, True), (1, 1, True),
    (300, 7, False), (64, 130, True), (5, 40, True),
]


@pytest.mark.parametrize("window,keep,sink", CASES)
@pytest.mark.parametrize("kind", ["float32", "float32 vector units", "bfloat16", "bfloat16 vector units"])
def test_attention_with_a_window_kept_first_keys_and_a_sink(kind, window, keep, sink):
    """Three requests in one batch over scattered pages: a portion of 150 rows that starts inside the first page
    (its rows pass the kept keys' end and the window's first full turn), a portion of 37 rows after 500 cached keys,
    and single new tokens at position 699 and at position 3.  One key far back among the kept ones, and the keys just
    inside and just outside the window of the last row, are made to stand out: a row that sees one key too many or
    too few is wrong by much more than rounding."""
    o = ops()
    dtype = torch.float32 if kind.startswith("float32") else torch.bfloat16
    hq, hkv, d, page = 8, 2, 64, 16
    scale = 0.3
    lens = [(3, 150), (500, 37), (699, 1), (3, 1)]
    qs, pos, seq, tables, caches, want = [], [], [], [], [], []
    base_page = 0
    for b, (before, n) in enumerate(lens):
        L = before + n
        g = torch.Generator().manual_seed(50 + b)
        k, v = torch.randn(L, hkv, d, generator=g).to(dtype), torch.randn(L, hkv, d, generator=g).to(dtype)
        q = torch.randn(n, hq, d, generator=g).to(dtype)
        # keys that stand out for the last row: one among the kept first keys, the window's oldest, the one before it
        last = L - 1
        for j, gain in ((min(2, L - 1), 0.6), (max(0, last - window + 1), 0.5), (max(0, last - window), 0.7)) if window else ((min(2, L - 1), 0.6),):
            k[j, :] = (k[j, :].float() + gain * q[-1, ::hq // hkv].float()).to(dtype)
        p = torch.arange(before, L)
        want.append(_plain_attention(q.double(), k.double(), v.double(), p, scale, window, keep, sink))
        cache, ids = _paged(k, v, page, 60 + b, dtype)
        caches.append(cache)
        tables.append(ids + base_page)
        base_page += cache.shape[0]
        qs.append(q)
        pos += p.tolist()
        seq += [b] * n
    width = max(len(t) for t in tables)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        table[b, :len(t)] = t
    q = torch.cat(qs).to(DEV)
    cache = torch.cat(caches).to(DEV)
    positions = torch.tensor(pos, dtype=torch.int32, device=DEV)
    tok_seq = torch.tensor(seq, dtype=torch.int32, device=DEV)
    want = torch.cat(want)
    T = q.shape[0]
    dec = torch.tensor([T - 2, T - 1], dtype=torch.int32, device=DEV)
    other = torch.arange(T - 2, dtype=torch.int32, device=DEV)
    from qwen_engine_amd.parts.attention import prefill_tiles
    rows = o.prefill_tile_rows(hq, hkv)
    tiles = torch.tensor(prefill_tiles([(0, 150), (150, 37)], rows), dtype=torch.int32).view(-1, 2).to(DEV) if rows > 0 else None
    vector = kind.endswith("vector units")
    if vector and dtype == torch.float32:
        o.use_matrix_f32(False)
    try:
        got = o.attention(q, cache, positions, tok_seq, table.to(DEV), scale, window, dec_tokens=dec, max_dec_position=699,
                          other_tokens=other, other_tiles=tiles, max_other_keys=537, keep_first=keep, sink=sink,
                          algo=o.ALGO_GENERIC if vector else o.ALGO_AUTO)
    finally:
        o.use_matrix_f32(True)
    assert not torch.isnan(got).any()
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    err = (got.double().cpu() - want).abs().amax(dim=(1, 2)) / float(want.abs().max())
    bad = (err > tol).nonzero().flatten().tolist()
    assert not bad, f"rows {bad[:8]} (positions {[pos[i] for i in bad[:8]]}): {float(err.max())}"


def test_attention_takes_what_the_decode_and_prefill_kernels_take():
    """(the test above runs the matrix-unit kernels in its bfloat16 case only if they take its sizes)"""
    o = ops()
    q = torch.zeros(1, 8, 64, dtype=torch.bfloat16, device=DEV)
    cache = torch.zeros(1, 2, 2, 16, 64, dtype=torch.bfloat16, device=DEV)
    assert o.attention_decode_supported(q, cache) and o.attention_prefill_supported(q, cache) and o.prefill_tile_rows(8, 2) > 0


# ---- the router -------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("E,top,scale", [(6, 2, 1.5), (20, 4, 1.0), (2, 2, 0.5), (73, 5, 2.0), (1, 1, 1.0), (130, 130, 3.0)])
def test_router_chooses_by_corrected_scores_and_weighs_by_the_scores(E, top, scale):
    g = torch.Generator().manual_seed(E)
    z = torch.randn(40, E, generator=g) * 2.0
    corr = torch.randn(E, generator=g) * 0.2
    ids, w = ops().moe_route_biased(z.to(DEV), corr.to(DEV), top, scale)
    for t in range(z.shape[0]):
        wi, ww = N.route(z[t].double(), corr.double(), top, scale)
        assert ids[t].tolist() == wi, t
        assert rel(w[t], ww) < 1e-5
    ids_t, w_t = ops().moe_route_biased(z.t().contiguous().to(DEV), corr.to(DEV), top, scale, transposed=True)
    assert torch.equal(ids_t, ids) and torch.equal(w_t, w)            # (the logits the other way round: the same bits)
    ids, w = ops().moe_route_biased(torch.zeros(2, E, device=DEV), torch.zeros(E, device=DEV), top, scale)
    assert ids[1].tolist() == list(range(top))            # ties: the lower index
    assert rel(w[1], torch.full((top,), scale / top, dtype=torch.float64)) < 1e-5


# ---- the experts ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol,T,H,Fd,E,ident,top", [
    (torch.float32, 2e-5, 37, 96, 40, 6, 2, 3), (torch.float32, 2e-5, 1, 64, 24, 3, 1, 4), (torch.bfloat16, 2e-2, 9, 128, 64, 8, 3, 2),
    (torch.bfloat16, 2e-2, 1, 256, 64, 4, 0, 1), (torch.bfloat16, 2e-2, 600, 128, 64, 5, 2, 3), (torch.bfloat16, 2e-2, 50, 100, 20, 4, 1, 2),
    (torch.bfloat16, 2e-2, 300, 64, 128, 1, 1, 2)])
def test_squared_relu_experts_and_identity_experts_over_rows_grouped_on_the_device(dtype, tol, T, H, Fd, E, ident, top):
    """Few pairs (rows read in place), many pairs (gathered rows through the tiled product) and sizes that only the
    kernel on the vector units takes: every token's weighted sum over its chosen experts, identity experts among them."""
    g = torch.Generator().manual_seed(T + H)
    x = torch.randn(T, H, generator=g).to(dtype)
    up = (torch.randn(E, Fd, H, generator=g) / math.sqrt(H)).to(dtype)
    down = (torch.randn(E, H, Fd, generator=g) / math.sqrt(Fd)).to(dtype)
    ids = torch.stack([torch.randperm(E + ident, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, top, generator=g) + 0.1
    want = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            y = x[t].double() if e >= E else N.expert(x[t].double(), up[e].double(), down[e].double())
            want[t] += float(w[t, j]) * y
    for rows_dtype in {torch.float32, dtype}:             # (the element type of an expert's output rows where the pairs are many)
        parts = ops().moe_experts(x.to(DEV), ids.to(DEV), w.to(DEV), up.to(DEV), down.to(DEV), act="relu_sq", identity=ident,
                                  rows_dtype=rows_dtype)
        assert parts.dtype == torch.float32 and parts.shape[1:] == (T, H)
        assert rel(parts.sum(0), want) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,Fd,E,ident,top", [(1, 128, 64, 8, 3, 2), (8, 256, 32, 32, 4, 4), (37, 96, 40, 6, 2, 3), (64, 64, 16, 70, 3, 5),
                                                (5, 128, 64, 1, 1, 2), (3, 64, 8, 4, 0, 1)])
def test_few_tokens_route_sort_and_identity_rows_in_one_launch(dtype, T, H, Fd, E, ident, top):
    """A step of few tokens routes, sorts and writes the identity experts' rows in one launch: the same parts, bit for
    bit, as the router's kernel, the sort's and the identity rows' one after the other."""
    o = ops()
    g = torch.Generator().manual_seed(T * 7 + E)
    x = torch.randn(T, H, generator=g).to(dtype).to(DEV)
    up = (torch.randn(E, Fd, H, generator=g) / math.sqrt(H)).to(dtype).to(DEV)
    down = (torch.randn(E, H, Fd, generator=g) / math.sqrt(Fd)).to(dtype).to(DEV)
    z = (torch.randn(T, E + ident, generator=g) * 2.0).to(DEV)
    corr = (torch.randn(E + ident, generator=g) * 0.2).to(DEV)
    ids, w = o.moe_route_biased(z, corr, top, 1.7)
    want = o.moe_experts(x, ids, w, up, down, act="relu_sq", identity=ident)
    got = o.moe_experts(x, None, None, up, down, act="relu_sq", identity=ident, biased_route=(z, corr, top, 1.7))
    assert torch.equal(got, want)
