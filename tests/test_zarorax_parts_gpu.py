"""Each mechanism of the Zarorax layers alone: the kernel against the plain implementation's function
of the same mechanism (or a few lines of 64-bit torch), in float32 and bfloat16."""
import math

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import zarorax_plain as Z

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    from qwen_engine_amd.kernels import ops as o
    return o


def rel(got, want):
    return float((got.double().cpu() - want.double()).abs().max()) / max(float(want.abs().max()), 1e-30)


# ---- the norm after the sum ---------------------------------------------------------------------------
@pytest.mark.parametrize("T,H,parts", [(1, 96, 0), (5, 200, 1), (33, 2048, 3), (3, 4100, -1)])
def test_norm_after_the_sum(T, H, parts):
    g = torch.Generator().manual_seed(T + H)
    x = torch.randn(T, H, generator=g)
    gain = torch.tensor([1.3])
    if parts == 0:
        delta = None
    elif parts < 0:
        delta = torch.randn(T, H, generator=g).bfloat16()
    else:
        delta = torch.randn(parts, T, H, generator=g)
    z = 2.5 * x.double() + (0 if delta is None else (delta.double() if delta.dim() == 2 else delta.double().sum(0)))
    want = Z.scalar_norm(z, gain.double(), 1e-5)
    xs = x.to(DEV)
    act = ops().postnorm(xs, None if delta is None else delta.to(DEV), 2.5, gain.to(DEV), 1e-5, torch.bfloat16)
    assert rel(xs, want) < 2e-6
    assert torch.equal(act.cpu(), xs.cpu().bfloat16())
    if parts >= 0:                                      # (a bfloat16 branch output only comes with bfloat16 activations)
        xs = x.to(DEV)
        assert ops().postnorm(xs, None if delta is None else delta.to(DEV), 2.5, gain.to(DEV), 1e-5, torch.float32) is None
        assert rel(xs, want) < 2e-6


def test_polynomial_activation_norms_every_power_by_itself():
    g = torch.Generator().manual_seed(4)
    z = torch.randn(7, 160, generator=g) * 1.7
    coef = torch.tensor([0.9, 0.5, -0.4, 0.1])
    zd = z.double()
    want = coef[0] * Z.unit_rms(zd, 1e-5) + coef[1] * Z.unit_rms(zd ** 2, 1e-5) + coef[2] * Z.unit_rms(zd ** 3, 1e-5) + coef[3]
    got = ops().polynorm(z.to(DEV), coef.to(DEV), 1e-5, torch.float32)
    assert rel(got, want) < 2e-6
    got = ops().polynorm(z.to(DEV), coef.to(DEV), 1e-5, torch.bfloat16)
    assert rel(got, want) < 6e-3


# ---- the short convolution and its state -----------------------------------------------------------------
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_short_convolution_continues_across_cuts_and_between_requests(taps):
    H = 70
    g = torch.Generator().manual_seed(taps)
    w = torch.randn(H, taps, generator=g)
    seqs = {0: torch.randn(23, H, generator=g), 2: torch.randn(9, H, generator=g), 1: torch.randn(14, H, generator=g)}
    want = {s: Z.short_conv(x.double(), w.double()) for s, x in seqs.items()}
    state = torch.full((4, max(taps - 1, 1), H), 7.0, device=DEV)[:, :taps - 1].contiguous() if taps > 1 else None
    if state is not None:
        state[[0, 1, 2]] = 0.0                         # what the step function does for a new request
    done = {s: 0 for s in seqs}
    got = {s: [] for s in seqs}
    # steps of unequal portions, down to single tokens; slot 1 joins late; slot 2 ends early
    plan = [{0: 1, 2: 2}, {0: 1, 2: 1}, {0: 2, 1: 5, 2: 6}, {1: 1, 0: 7}, {0: 1, 1: 1}, {0: 11, 1: 7}]
    for step in plan:
        rows, tok_seq = [], []
        for s, n in step.items():
            rows.append(seqs[s][done[s]:done[s] + n])
            tok_seq += [s] * n
        x = torch.cat(rows).to(DEV)
        out = ops().short_conv(x, w.to(DEV), state, torch.tensor(tok_seq, dtype=torch.int32, device=DEV), torch.float32)
        at = 0
        for s, n in step.items():
            got[s].append(out[at:at + n].cpu())
            at += n
            done[s] += n
    for s in seqs:
        assert done[s] == len(seqs[s])
        assert rel(torch.cat(got[s]), want[s]) < 1e-6, f"request in slot {s}"
    if state is not None:
        assert torch.equal(state[0].cpu(), seqs[0][-(taps - 1):])
        assert float(state[3].min()) == 7.0            # a slot that no row named stays as it was


# ---- the products per head --------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 8e-3)])
@pytest.mark.parametrize("T,H,K,N", [(37, 3, 20, 45), (5, 2, 24, 70), (130, 3, 64, 33), (64, 1, 128, 64)])
def test_products_per_head_read_and_write_parts_of_wider_heads(dtype, tol, T, H, K, N):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, H, K + 8, generator=g).to(dtype)
    w = (torch.randn(H, N, K, generator=g) / math.sqrt(K)).to(dtype)
    out = torch.full((T, H, N + 4), 9.0).to(dtype).to(DEV)
    ops().gemm_heads(x.to(DEV), w.to(DEV), out)
    want = torch.einsum("thk,hnk->thn", x[..., :K].double(), w.double())
    assert rel(out[..., :N], want) < tol
    assert float(out[..., N:].float().min()) == 9.0
    gate = torch.randn(T, H * N, generator=g).to(dtype)
    out2 = torch.empty(T, H, N, dtype=dtype, device=DEV)
    ops().gemm_heads(x.to(DEV), w.to(DEV), out2, gate.to(DEV))
    assert rel(out2, want * torch.sigmoid(gate.double()).view(T, H, N)) < tol


# ---- attention over the cached latents -----------------------------------------------------------------------
def _latent_case(dtype, R, Dr, H, P, lengths, seed, stand_out=None):
    """Requests of the given lengths in scattered pages; every request's last ``new`` tokens are queries."""
    g = torch.Generator().manual_seed(seed)
    D = R + Dr
    pages_per = [(n + P - 1) // P for n in lengths]
    order = torch.randperm(sum(pages_per) + 3, generator=g).tolist()
    cache = torch.full((len(order), 1, 1, P, D), float("nan"))
    table = torch.full((len(lengths), max(pages_per)), -1, dtype=torch.int32)
    rows = []
    for b, n in enumerate(lengths):
        r = torch.randn(n, D, generator=g)
        if stand_out is not None and b == 0:
            r[stand_out] *= 6.0
        rows.append(r.to(dtype))
        for i in range(pages_per[b]):
            page = order.pop()
            table[b, i] = page
            chunk = rows[b][i * P:(i + 1) * P]
            cache[page, 0, 0, :len(chunk)] = chunk.float()
    return cache.to(dtype), table, rows


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("R,Dr,H,P", [(40, 8, 3, 8), (64, 64, 1, 16), (96, 32, 16, 4)])
def test_latent_attention_over_pages(dtype, tol, R, Dr, H, P):
    lengths = [3 * P + 1, 1, 64, 65, 5 * P]
    cache, table, rows = _latent_case(dtype, R, Dr, H, P, lengths, seed=R + H)
    g = torch.Generator().manual_seed(1)
    # queries: the last min(n, 3) positions of every request (page borders and first tokens among them)
    qs, pos, seq = [], [], []
    for b, n in enumerate(lengths):
        for p in range(max(0, n - 3), n):
            qs.append(torch.randn(H, R + Dr, generator=g))
            pos.append(p)
            seq.append(b)
    qp = torch.stack(qs).to(dtype)
    scale = 0.7 / math.sqrt(R + Dr)
    out = ops().latent_attention(qp.to(DEV), cache.to(DEV), torch.tensor(pos, dtype=torch.int32, device=DEV),
                                 torch.tensor(seq, dtype=torch.int32, device=DEV), table.to(DEV), R, scale)
    for i, (p, b) in enumerate(zip(pos, seq)):
        keys = rows[b][:p + 1].double()
        w = torch.softmax(qp[i].double() @ keys.t() * scale, dim=-1)
        assert rel(out[i], w @ keys[:, :R]) < tol, f"query {i} at position {p} of request {b}"
    assert not torch.isnan(out.float()).any()


def test_latent_attention_finds_one_far_key_among_hundreds():
    R, Dr, H, P = 48, 16, 2, 16
    n, far = 700, 37
    cache, table, rows = _latent_case(torch.float32, R, Dr, H, P, [n], seed=9)
    q = rows[0][far].clone()[None].repeat(H, 1)[None] * 3.0       # points at the row of position 37
    out = ops().latent_attention(q.to(DEV), cache.to(DEV), torch.tensor([n - 1], dtype=torch.int32, device=DEV),
                                 torch.zeros(1, dtype=torch.int32, device=DEV), table.to(DEV), R, 1.0)
    assert rel(out[0, 0], rows[0][far, :R]) < 1e-4                # the softmax is that one key


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 8e-3)])
def test_cache_rows_are_the_normed_latent_and_the_rotated_key_part(dtype, tol):
    g = torch.Generator().manual_seed(6)
    T, R, Dr, dims, P = 9, 40, 12, 8, 4
    kv = torch.randn(T, R + Dr, generator=g)
    weight = 1 + 0.3 * torch.randn(R, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 500, 501, 70000, 5, 6], dtype=torch.int32)
    slots = torch.tensor([8, 9, 10, 11, 0, 1, 2, -1, 30], dtype=torch.int32)
    inv = torch.pow(torch.tensor(777.0, dtype=torch.float64), -torch.arange(0, dims, 2).double() / dims).float()
    cache = torch.full((8, 1, 1, P, R + Dr), 5.0).to(dtype).to(DEV)
    ops().latent_kv_store(kv.to(DEV), weight.to(DEV), 1e-5, pos.to(DEV), inv.to(DEV), slots.to(DEV), cache)
    flat = cache.view(-1, R + Dr).float().cpu()
    c = Z.vector_norm(kv[:, :R].double(), weight.double(), 1e-5)
    kr = Z.rotate_interleaved(kv[:, R:].double(), pos, 777.0, dims)
    for t in range(T):
        if slots[t] < 0:
            continue
        assert rel(flat[slots[t], :R], c[t]) < tol
        # (at position 70000 a 32-bit angle is exact to 0.004: the plain rotation is 64-bit)
        assert rel(flat[slots[t], R:], kr[t]) < (max(tol, 2e-5) if pos[t] < 1000 else 1e-2)
    untouched = [s for s in range(32) if s not in slots.tolist()]
    assert float(flat[untouched].min()) == 5.0 and float(flat[untouched].max()) == 5.0
    # the queries' rotated parts
    H, dn = 3, 7
    q = torch.randn(T, H, dn + Dr, generator=g).to(dtype)
    qp = torch.zeros(T, H, R + Dr, dtype=dtype, device=DEV)
    ops().latent_q_rotate(q.to(DEV), pos.to(DEV), inv.to(DEV), qp, dn)
    want = Z.rotate_interleaved(q[..., dn:].double(), pos, 777.0, dims)
    keep = pos < 1000
    assert rel(qp[keep][..., R:], want[keep]) < max(tol, 2e-5) and float(qp[..., :R].float().abs().max()) == 0.0


# ---- the mixture of experts -----------------------------------------------------------------------------------
@pytest.mark.parametrize("E,G,keep,top", [(6, 3, 2, 2), (4, 1, 1, 1), (8, 4, 4, 3), (64, 8, 3, 6), (130, 1, 1, 8)])
def test_router_choices_and_weights(E, G, keep, top):
    g = torch.Generator().manual_seed(E)
    T, H = 50, 24
    h = torch.randn(T, H, generator=g)
    router = torch.randn(E, H, generator=g)
    logits = (h.double() @ router.double().t()).float()
    ids, weights = ops().moe_route(logits.to(DEV), G, keep, top)
    want = Z.route(h, router, {"experts": E, "top": top, "groups": {"count": G, "keep": keep}})
    for t in range(T):
        assert ids[t].tolist() == [e for e, _ in want[t]], f"token {t}"
        assert rel(weights[t], torch.tensor([w for _, w in want[t]])) < 1e-5


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 1.5e-2)])
@pytest.mark.parametrize("T,H,Fd", [(1, 72, 40), (7, 72, 40), (150, 72, 40), (400, 72, 40), (9, 64, 96), (300, 64, 96),
                                    (700, 128, 64)])
def test_experts_over_rows_grouped_on_the_device(dtype, tol, T, H, Fd):
    g = torch.Generator().manual_seed(T)
    E, top, limit = 6, 2, 0.8
    x = torch.randn(T, H, generator=g).to(dtype)
    w = {"m.router": torch.randn(E, H, generator=g) * 0.5}
    for e in range(E):
        w[f"m.e{e}.gate"] = (torch.randn(Fd, H, generator=g) / math.sqrt(H) * 1.5).to(dtype)
        w[f"m.e{e}.up"] = (torch.randn(Fd, H, generator=g) / math.sqrt(H) * 1.5).to(dtype)
        w[f"m.e{e}.down"] = (torch.randn(H, Fd, generator=g) / math.sqrt(Fd)).to(dtype)
    mlp = {"expert": {"ff": Fd, "limit": limit}, "router": {"experts": E, "top": top, "groups": {"count": 3, "keep": 2}}}
    want = Z.moe_ffn(x.double(), {k: v.double() for k, v in w.items()}, "m", mlp)
    logits = (x.double() @ w["m.router"].double().t()).float().to(DEV)
    ids, weights = ops().moe_route(logits, 3, 2, top)
    il = Fd % 32 == 0                                  # gate and up rows in alternating blocks of 32 where the width allows
    stack = (lambda a, b: ops().interleave_gate_up(a, b)) if il else (lambda a, b: torch.cat([a, b]))
    wgu = torch.stack([stack(w[f"m.e{e}.gate"], w[f"m.e{e}.up"]) for e in range(E)]).to(DEV)
    wd = torch.stack([w[f"m.e{e}.down"] for e in range(E)]).to(DEV)
    parts = ops().moe_experts(x.to(DEV), ids, weights, wgu, wd, limit, 1.702, interleaved=il)
    assert parts.shape in ((top, T, H), (1, T, H)) and parts.dtype == torch.float32
    assert rel(parts.sum(0), want) < tol
    plain = ops().moe_experts(x.to(DEV), ids, weights, wgu, wd, limit, 1.702, interleaved=il, algo=ops().ALGO_GENERIC)
    assert plain.shape == (top, T, H) and rel(plain.sum(0), want) < tol
    # a token's result does not depend on the batch around it (while the same kernel serves it)
    if parts.shape[0] == top:
        alone = ops().moe_experts(x[:1].to(DEV), ids[:1].contiguous(), weights[:1].contiguous(), wgu, wd, limit, 1.702,
                                  interleaved=il)
        assert rel(alone[:, 0], parts[:, 0].double().cpu()) < (1e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("R,Dr,H,P,lengths,new", [
    (512, 64, 16, 16, [300, 1, 77], [300, 1, 77]),        # whole prompts side by side, many rows: tokens share a block
    (512, 64, 16, 16, [700, 33, 64, 65, 129], [1, 1, 1, 1, 1]),   # single new tokens: the keys are cut into splits
    (256, 32, 128, 8, [90, 200], [3, 70]),                # many heads: several head groups per token
    (160, 32, 5, 16, [40, 41, 260], [40, 2, 100]),        # fewer heads than a wave has columns; mixed step
    (64, 0, 24, 4, [130, 19], [130, 1]),                  # no rotated part; heads that fill one group and half of the next
    (200, 24, 8, 32, [150], [150]),                       # sizes that are no multiple of 16 or 32
])
def test_latent_attention_on_the_matrix_units(R, Dr, H, P, lengths, new):
    """The kernel on the matrix units against 64-bit torch, with the requests' last ``new`` tokens as the
    step's rows: portions beside single tokens, borders between requests inside a block of rows."""
    cache, table, rows = _latent_case(torch.bfloat16, R, Dr, H, P, lengths, seed=R + H + len(lengths))
    g = torch.Generator().manual_seed(2)
    qs, pos, seq = [], [], []
    for b, (n, k) in enumerate(zip(lengths, new)):
        for p in range(n - k, n):
            qs.append(torch.randn(H, R + Dr, generator=g))
            pos.append(p)
            seq.append(b)
    qp = torch.stack(qs).bfloat16()
    scale = 1.5 / math.sqrt(R + Dr)
    args = (qp.to(DEV), cache.to(DEV), torch.tensor(pos, dtype=torch.int32, device=DEV),
            torch.tensor(seq, dtype=torch.int32, device=DEV), table.to(DEV), R, scale)
    out = ops().latent_attention(*args)
    plain = ops().latent_attention(*args, algo=ops().ALGO_GENERIC)
    assert not torch.isnan(out.float()).any()
    worst = 0.0
    for i in range(0, len(pos), max(1, len(pos) // 40)):       # a sample of the rows against 64-bit arithmetic
        keys = rows[seq[i]][:pos[i] + 1].double()
        w = torch.softmax(qp[i].double() @ keys.t() * scale, dim=-1)
        worst = max(worst, rel(out[i], w @ keys[:, :R]))
    assert worst < 1.5e-2, worst
    assert rel(out, plain.double().cpu()) < 2e-2               # every row against the kernel on the vector units


@pytest.mark.parametrize("taps", [2, 4])
def test_short_convolution_of_single_rows_in_one_launch(taps):
    """Steps in which every request brings one token: convolution and the state's shift in one launch give what
    the two launches give, state included."""
    H, B = 96, 5
    g = torch.Generator().manual_seed(taps)
    w = torch.randn(H, taps, generator=g).to(DEV)
    xs = [torch.randn(B, H, generator=g).to(DEV) for _ in range(6)]
    seq = torch.tensor([3, 0, 4, 1, 2], dtype=torch.int32, device=DEV)
    a = torch.randn(6, taps - 1, H, generator=g).to(DEV)
    b = a.clone()
    for x in xs:
        one = ops().short_conv(x, w, a, seq, torch.float32, single_rows=True)
        two = ops().short_conv(x, w, b, seq, torch.float32)
        assert torch.equal(one, two) and torch.equal(a, b)
    assert torch.equal(a[3, -1], xs[-1][0]) and torch.equal(a[5], b[5])
