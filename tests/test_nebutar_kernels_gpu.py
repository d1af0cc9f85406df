"""Each kernel of the Nebutar design's mechanisms alone, against the plain functions of ``plain_nebutar.py`` in 64-bit, at sizes
that are no multiples of the kernels' tiles: the embedding with its position table, the norm over copies of the residual, the
cache write and the attention with cap, chunks and window (keys at every edge, pages in scrambled order, a key far back that
carries the weight), the convolutions from their tails, the gated delta rule (portions against single steps to the bit, slots
used again), the gated head norm, the router over all scores with a correction, gated experts and identity experts."""
import math

import pytest
import torch

import plain_nebutar as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype, loose=1.0):
    return dict(atol=2e-5 * loose, rtol=2e-5 * loose) if dtype == torch.float32 else dict(atol=2e-2 * loose, rtol=2e-2 * loose)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("copies", [0, 1, 3])
def test_embedding_with_position_rows(dtype, copies):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    V, H, T, P = 50, 70, 9, 40
    table, pos = torch.randn(V, H, generator=g).to(dtype), torch.randn(P, H, generator=g).to(dtype)
    ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    at = torch.randint(0, P, (T,), generator=g, dtype=torch.int32)
    out = torch.full((copies, T, H) if copies else (T, H), float("nan"), device="cuda")
    ops.embedding(ids.cuda(), table.cuda(), out, 3.0, at.cuda(), pos.cuda())
    want = table.double()[ids.long()] * 3.0 + pos.double()[at.long()]
    torch.testing.assert_close(out.cpu().double(), want.expand(out.shape) if copies else want, atol=1e-6, rtol=1e-6)
    plain_out = torch.empty(T, H, device="cuda")
    ops.embedding(ids.cuda(), table.cuda(), plain_out, 0.5)
    torch.testing.assert_close(plain_out.cpu().double(), table.double()[ids.long()] * 0.5, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["layernorm", "rmsnorm"])
@pytest.mark.parametrize("S, parts", [(1, 0), (3, 0), (4, 2), (8, 0)])
def test_norm_over_copies_of_the_residual(dtype, kind, S, parts):
    """The pending output enters the copies through (mix, out), the norm reads through ``in``: updated copies and normed rows; then the
    final form (no read vector: the sum of the copies) on chosen rows, which writes nothing back; then a first norm with nothing pending."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    T, H, eps = 6, 150, 1e-5
    x = torch.randn(S, T, H, generator=g) * 3 + 5.0                 # a mean well away from zero: the deviations are taken from the mean
    pen = torch.randn(parts, T, H, generator=g) if parts else torch.randn(T, H, generator=g).to(dtype)
    p = pen.double().sum(0) if parts else pen.double()
    mix, gate, read = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    w, b = 1 + 0.1 * torch.randn(H, generator=g), 0.1 * torch.randn(H, generator=g)
    norm = (lambda u: plain.layer_norm(u, w.double(), b.double(), eps)) if kind == "layernorm" else \
        (lambda u: u / torch.sqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w.double())
    bias = b.cuda() if kind == "layernorm" else None
    new = torch.einsum("st,snw->tnw", mix.double(), x.double()) + gate.double()[:, None, None] * p[None]
    xs = x.cuda()
    out = torch.empty(T, H, dtype=dtype, device="cuda")
    ops.streams_norm(xs, pen.cuda(), (mix.cuda(), gate.cuda()), read.cuda(), kind, w.cuda(), bias, eps, out)
    torch.testing.assert_close(xs.cpu().double(), new, atol=2e-5, rtol=1e-5)            # the copies stay 32-bit in both engines
    torch.testing.assert_close(out.cpu().double(), norm(torch.einsum("s,snw->nw", read.double(), new)), **_tol(dtype, 3))
    rows = torch.tensor([4, 0, 4], dtype=torch.int32)
    xs = x.cuda()
    few = torch.empty(3, H, dtype=dtype, device="cuda")
    ops.streams_norm(xs, pen.cuda(), (mix.cuda(), gate.cuda()), None, kind, w.cuda(), bias, eps, few, rows.cuda(), gain=2.0)
    assert torch.equal(xs.cpu(), x)
    torch.testing.assert_close(few.cpu().double(), 2.0 * norm(new.sum(0))[rows.long()], **_tol(dtype, 3))
    ops.streams_norm(xs, None, None, read.cuda(), kind, w.cuda(), bias, eps, out)
    assert torch.equal(xs.cpu(), x)
    torch.testing.assert_close(out.cpu().double(), norm(torch.einsum("s,snw->nw", read.double(), x.double())), **_tol(dtype, 3))


# ------------------------------------------------------------------ attention

def _paged(G, dim, vdim, page, lengths, dtype, g, scramble=True):
    """Keys and values of requests of the given lengths in pages handed out in scrambled order; every place that holds no key is NaN."""
    blocks = [-(-n // page) for n in lengths]
    pages = sum(blocks) + 1
    order = (torch.randperm(pages - 1, generator=g) + 1).tolist() if scramble else list(range(1, pages))
    table = torch.zeros(len(lengths), max(blocks), dtype=torch.int32)
    k_plane = torch.full((pages, G, page, dim), float("nan")).to(dtype)
    v_plane = torch.full((pages, G, vdim, page), float("nan")).to(dtype)            # the values of a page lie transposed
    keys = [torch.randn(n, G, dim, generator=g).to(dtype) for n in lengths]
    values = [torch.randn(n, G, vdim, generator=g).to(dtype) for n in lengths]
    for r, n in enumerate(lengths):
        for b in range(blocks[r]):
            table[r, b] = order.pop()
    return table, k_plane, v_plane, keys, values


def _tiles(new, lengths, tq=16):
    """What a step context hands the matrix-core kernel: tiles of up to ``tq`` tokens of one request."""
    tile_req = [r for r, n in enumerate(new) for _ in range(-(-n // tq))]
    tile_tok0 = [i * tq for n in new for i in range(-(-n // tq))]
    indptr = [0]
    for n in new:
        indptr.append(indptr[-1] + n)
    as_int = lambda v: torch.tensor(v, dtype=torch.int32).cuda()
    return as_int(indptr), as_int([L - n for L, n in zip(lengths, new)]), as_int(tile_req), as_int(tile_tok0), len(tile_req)


def _attend(q, keys, values, p, H, G, scale, cap, chunk, window):
    """One query at position p of a request against its keys, in 64-bit."""
    ok = plain.visible(p + 1, chunk=chunk or None, window=window or None)[p]
    of = torch.arange(H) // (H // G)
    s = torch.einsum("hd,jhd->hj", q.double(), keys[: p + 1, of].double()) * scale
    if cap:
        s = cap * torch.tanh(s / cap)
    w = torch.softmax(s.masked_fill(~ok, float("-inf")), dim=-1)
    return torch.einsum("hj,jhd->hd", w, values[: p + 1, of].double()).reshape(-1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, dim, vdim, page, chunk, window, cap", [
    (4, 2, 6, 10, 4, 7, 0, 5.0),          # odd sizes, a chunk that is no multiple of the page
    (4, 1, 64, 128, 16, 80, 0, 12.0),     # one key/value head for all, values twice as wide as keys
    (6, 3, 40, 24, 8, 0, 0, 0.0),         # no chunk, no window, no cap: plain causal attention
    (2, 2, 16, 16, 2, 0, 9, 3.0),         # a window alone
    (3, 1, 20, 36, 4, 30, 11, 0.0),       # a chunk and a window: whichever starts later
    (16, 4, 128, 128, 16, 200, 0, 50.0),  # more keys than one pass of the waves takes
])
def test_attention_with_cap_chunks_and_window(dtype, H, G, dim, vdim, page, chunk, window, cap):
    """Queries of three requests in one step: a whole prompt, a portion that starts and ends in the middle of chunks and pages, a
    single token; written to scrambled pages by the cache-write kernel, read back through the block table.  Every position is a
    query, so every edge (first and last key of a chunk, of a window, of a page) is met."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    lengths, new = [50, 431, 230], [50, 67, 1]
    table, k_plane, v_plane, keys, values = _paged(G, dim, vdim, page, lengths, dtype, g)
    q = [torch.randn(n, H, dim, generator=g).to(dtype) for n in new]
    scale, gain = 0.7 / math.sqrt(dim), 0.6
    token_req = torch.cat([torch.full((n,), r, dtype=torch.int32) for r, n in enumerate(new)])
    positions = torch.cat([torch.arange(L - n, L, dtype=torch.int32) for L, n in zip(lengths, new)])
    kd, vd, tab = k_plane.cuda(), v_plane.cuda(), table.cuda()
    # what lies before the step's tokens is in the pages already; the step's own keys and values go there through the kernel
    for r, (L, n) in enumerate(zip(lengths, new)):
        for j in range(L - n):
            kd[table[r, j // page], :, j % page] = keys[r][j].cuda()
            vd[table[r, j // page], :, :, j % page] = values[r][j].cuda()
    k_new = torch.cat([keys[r][L - n:].reshape(n, -1) for r, (L, n) in enumerate(zip(lengths, new))])
    v_new = torch.cat([values[r][L - n:].reshape(n, -1) for r, (L, n) in enumerate(zip(lengths, new))])
    wide = torch.cat((k_new, v_new), dim=1).cuda()                  # row-strided views, as a mixer hands them over
    ops.kv_cache_write(wide[:, : G * dim], wide[:, G * dim:], token_req.cuda(), positions.cuda(), tab, kd, vd, page)
    for r, L in enumerate(lengths):
        j = L - 1
        assert torch.equal(kd[table[r, j // page], :, j % page].cpu(), keys[r][j]) and torch.equal(vd[table[r, j // page], :, :, j % page].cpu(), values[r][j])
    assert bool(torch.isnan(kd[0].float()).all())                   # the sentinel page stays unwritten
    qs = torch.cat([x.reshape(x.shape[0], -1) for x in q]).cuda()
    out = torch.full((qs.shape[0], H * vdim + 5), float("nan"), dtype=dtype, device="cuda")
    ops.local_attention(qs, out[:, 3: 3 + H * vdim], kd, vd, tab, token_req.cuda(), positions.cuda(), H, G, dim, vdim, page, scale, cap, chunk, window, gain)
    want = torch.stack([gain * _attend(q[r][i], keys[r], values[r], lengths[r] - new[r] + i, H, G, scale, cap, chunk, window)
                        for r in range(3) for i in range(new[r])])
    torch.testing.assert_close(out[:, 3: 3 + H * vdim].cpu().double(), want, **_tol(dtype, 2))
    assert bool(torch.isnan(out[:, :3].float()).all() and torch.isnan(out[:, 3 + H * vdim:].float()).all())
    assert ops.local_attention_mfma_fits(dtype, dim, vdim, page) == (dtype == torch.bfloat16 and dim in (64, 128) and page == 16)
    if ops.local_attention_mfma_fits(dtype, dim, vdim, page):       # the matrix-core kernel on the same operands, in tiles of 16 tokens
        tiled = torch.full((qs.shape[0], H * vdim + 8), float("nan"), dtype=dtype, device="cuda")
        ops.local_attention(qs, tiled[:, 8:], kd, vd, tab, token_req.cuda(), positions.cuda(), H, G, dim, vdim, page, scale, cap, chunk, window, gain,
                            tiles=_tiles(new, lengths))
        torch.testing.assert_close(tiled[:, 8:].cpu().double(), want, **_tol(dtype, 2))
        assert bool(torch.isnan(tiled[:, :8].float()).all())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("new", [1, 40])
def test_one_key_at_the_edge_of_a_chunk_carries_the_weight(dtype, new):
    """The first key of the query's chunk is scaled up so that it takes nearly all the weight, and its value is unlike the others: the
    output shows whether it was read.  The key just before the chunk is scaled up as much in another run: it must not show."""
    from torchlet_amd.kernels import ops
    H, G, dim, vdim, page, chunk = 2, 1, 32, 64, 16, 112
    L = chunk * 3 + 57
    for edge, seen in ((chunk * 3, True), (chunk * 3 - 1, False)):
        g = torch.Generator().manual_seed(4)
        table, k_plane, v_plane, keys, values = _paged(G, dim, vdim, page, [L], dtype, g)
        q = torch.randn(new, H, dim, generator=g).to(dtype)
        keys[0][edge] = (q[-1, 0].float() * 4.0).to(dtype)          # the last query's first head leans on this key
        values[0][edge] = 100.0
        kd, vd = k_plane.cuda(), v_plane.cuda()
        for j in range(L):
            kd[table[0, j // page], :, j % page] = keys[0][j].cuda()
            vd[table[0, j // page], :, :, j % page] = values[0][j].cuda()
        # pages before the query's chunk may have gone back to the pool: their table entries point at the sentinel page, which holds NaN here
        tab = table.clone()
        tab[0, : (chunk * 3 - 1) // page] = 0
        token_req = torch.zeros(new, dtype=torch.int32).cuda()
        positions = torch.arange(L - new, L, dtype=torch.int32).cuda()
        want = _attend(q[-1], keys[0], values[0], L - 1, H, G, 1.0, 0.0, chunk, 0)
        for tiles in (None, _tiles([new], [L])) if dtype == torch.bfloat16 and new > 1 else (None,):
            out = torch.empty((new, H * vdim), dtype=dtype, device="cuda")
            ops.local_attention(q.reshape(new, -1).cuda(), out, kd, vd, tab.cuda(), token_req, positions, H, G, dim, vdim, page, 1.0, 0.0, chunk, 0, 1.0, tiles=tiles)
            torch.testing.assert_close(out[-1].cpu().double(), want, **_tol(dtype, 50))
            assert (float(out[-1, :vdim].float().mean()) > 90.0) == seen


# ------------------------------------------------------------------ the gated delta rule

def _delta_inputs(g, T, H, G, dim, vdim, taps, dtype):
    C = 2 * G * dim + H * vdim
    proj = torch.randn(T, C + 7, generator=g).to(dtype)             # rows longer than the convolved channels
    conv_w = torch.randn(C, taps, generator=g) * 0.5
    gates = torch.randn(T, 2 * H, generator=g) * 2
    a_log, dt_bias = torch.log(torch.rand(H, generator=g) * 2 + 0.05), torch.randn(H, generator=g)
    return C, proj, conv_w, gates, a_log, dt_bias


def _plain_prepare(proj, conv_w, gates, a_log, dt_bias, H, G, dim, vdim, qscale, eps):
    T, C = proj.shape[0], conv_w.shape[0]
    y = plain.silu(plain.short_convolution(proj[:, :C].double(), conv_w.double()))
    q = plain.unit(y[:, : G * dim].view(T, G, dim), eps) * qscale
    k = plain.unit(y[:, G * dim: 2 * G * dim].view(T, G, dim), eps)
    beta = torch.sigmoid(gates[:, :H].double())
    decay = torch.exp(-torch.exp(a_log.double()) * plain.softplus(gates[:, H:].double() + dt_bias.double()))
    return q, k, y[:, 2 * G * dim:].view(T, H, vdim), beta, decay


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, dim, vdim, taps", [(4, 2, 5, 7, 4), (8, 4, 64, 96, 2), (2, 1, 130, 20, 1), (3, 3, 16, 200, 8)])
def test_convolutions_from_their_tails_units_and_gates(dtype, H, G, dim, vdim, taps):
    """A request's tokens in portions of 1, 2, 1, 5 and the rest (portions shorter than the taps reach into the tail that earlier
    portions left), beside another request that is whole, in slots 2 and 0 of a state whose other numbers must stay as they are."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    T, qscale, eps = 23, dim ** -0.5, 1e-6
    C, proj, conv_w, gates, a_log, dt_bias = _delta_inputs(g, T, H, G, dim, vdim, taps, dtype)
    other = torch.randn(9, C + 7, generator=g).to(dtype)
    other_gates = torch.randn(9, 2 * H, generator=g)
    tail_off = 11
    state = torch.full((4, tail_off + (taps - 1) * C + 3), 7.0, device="cuda")
    state[:, tail_off: tail_off + (taps - 1) * C] = 0.0
    q, k, v, beta, decay = _plain_prepare(proj, conv_w, gates, a_log, dt_bias, H, G, dim, vdim, qscale, eps)
    oq, ok_, ov, _, _ = _plain_prepare(other, conv_w, other_gates, a_log, dt_bias, H, G, dim, vdim, qscale, eps)
    slots = torch.tensor([2, 0], dtype=torch.int32).cuda()
    at = 0
    for i, n in enumerate((1, 2, 1, 5, T - 9)):
        with_other = i == 3
        rows = torch.cat((proj[at: at + n], other)) if with_other else proj[at: at + n]
        graw = (torch.cat((gates[at: at + n], other_gates)) if with_other else gates[at: at + n]).cuda().contiguous()
        indptr = torch.tensor([0, n, n + 9] if with_other else [0, n], dtype=torch.int32).cuda()
        token_req = torch.tensor([0] * n + [1] * (9 if with_other else 0), dtype=torch.int32).cuda()
        qkv = torch.empty((rows.shape[0], C), device="cuda")
        ops.delta_prepare(rows.cuda()[:, :C], conv_w.cuda(), graw, a_log.cuda(), dt_bias.cuda(), state, tail_off, slots, indptr, token_req, qkv,
                          H, G, dim, vdim, taps, qscale, eps)
        want = torch.cat((q[at: at + n].reshape(n, -1), k[at: at + n].reshape(n, -1), v[at: at + n].reshape(n, -1)), dim=1)
        torch.testing.assert_close(qkv[:n].cpu().double(), want, atol=1e-5, rtol=1e-4)
        torch.testing.assert_close(graw[:n].cpu().double(), torch.cat((beta[at: at + n], decay[at: at + n]), dim=1), atol=1e-6, rtol=1e-5)
        if with_other:
            torch.testing.assert_close(qkv[n:].cpu().double(), torch.cat((oq.reshape(9, -1), ok_.reshape(9, -1), ov.reshape(9, -1)), dim=1), atol=1e-5, rtol=1e-4)
        at += n
        if taps > 1:        # the tail holds the last inputs, oldest first, zeros before the sequence's start
            held = torch.cat((torch.zeros(taps - 1, C), proj[:at, :C].float()))[-(taps - 1):]
            assert torch.equal(state[2, tail_off: tail_off + (taps - 1) * C].cpu().view(taps - 1, C), held)
    assert bool((state[:, :tail_off] == 7.0).all() and (state[:, tail_off + (taps - 1) * C:] == 7.0).all() and (state[1] [tail_off: -3] == 0).all())


@pytest.mark.parametrize("H, G, dim, vdim", [(4, 2, 5, 7), (6, 3, 64, 96), (2, 1, 130, 20), (3, 3, 16, 200), (8, 2, 128, 128), (1, 1, 256, 40)])
def test_delta_rule_against_plain_and_portions_to_the_bit(H, G, dim, vdim):
    """Two requests from given states: whole against the plain recurrence; then the first request again token by token and in portions
    of 2, 17, 1 and the rest beside the other request, in other slots: the same numbers bit for bit, and the states left behind too."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(6)
    T1, T2 = 45, 19
    C = 2 * G * dim + H * vdim

    def inputs(T):
        q = plain.unit(torch.randn(T, G, dim, generator=g)) * dim ** -0.5
        k = plain.unit(torch.randn(T, G, dim, generator=g))
        v = torch.randn(T, H, vdim, generator=g)
        gates = torch.cat((torch.rand(T, H, generator=g), 0.6 + 0.4 * torch.rand(T, H, generator=g)), dim=1)
        return torch.cat((q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)), dim=1).contiguous(), gates.contiguous()

    (x1, g1), (x2, g2) = inputs(T1), inputs(T2)
    extra = 8 if dim % 8 == 0 else 5            # rows of the state that are, and are not, aligned for 16-byte pieces
    start = torch.randn(3, H * dim * vdim + extra, generator=g) * 0.3

    def want(x, gates, S0):
        T = x.shape[0]
        of = torch.arange(H) // (H // G)
        q, k = x[:, : G * dim].view(T, G, dim)[:, of].double(), x[:, G * dim: 2 * G * dim].view(T, G, dim)[:, of].double()
        v = x[:, 2 * G * dim:].view(T, H, vdim).double()
        S = S0.double().view(H, vdim, dim).transpose(1, 2).clone()          # a head's state lies column by column
        out = []
        for t in range(T):
            S = S * gates[t, H:, None, None].double()
            u = gates[t, :H, None].double() * (v[t] - torch.einsum("hde,hd->he", S, k[t]))
            S = S + k[t][:, :, None] * u[:, None, :]
            out.append(torch.einsum("hde,hd->he", S, q[t]).reshape(-1))
        return torch.stack(out), S.transpose(1, 2).reshape(-1)

    def run(portions, slot_of):
        """``portions``: a list of steps, each a list of (request, tokens of it).  Returns the outputs per request and the state tensor."""
        state = start.clone().cuda()
        data = {0: (x1, g1), 1: (x2, g2)}
        at, got = {0: 0, 1: 0}, {0: [], 1: []}
        for step in portions:
            xs = torch.cat([data[r][0][at[r]: at[r] + n] for r, n in step]).cuda()
            gs = torch.cat([data[r][1][at[r]: at[r] + n] for r, n in step]).cuda()
            indptr = torch.tensor([0] + list(torch.tensor([n for _, n in step]).cumsum(0)), dtype=torch.int32).cuda()
            slots = torch.tensor([slot_of[r] for r, _ in step], dtype=torch.int32).cuda()
            out = torch.empty((xs.shape[0], H * vdim), device="cuda")
            ops.delta_scan(xs, gs, state, slots, indptr, out, H, G, dim, vdim, max_new_tokens=max(n for _, n in step))
            o = 0
            for r, n in step:
                got[r].append(out[o: o + n].cpu())
                o += n
                at[r] += n
        return {r: torch.cat(v) for r, v in got.items() if v}, state.cpu()

    whole, state = run([[(0, T1), (1, T2)]], {0: 2, 1: 0})
    for r, (x, gates, slot) in enumerate(((x1, g1, 2), (x2, g2, 0))):
        o, S = want(x, gates, start[slot, : H * dim * vdim])
        torch.testing.assert_close(whole[r].double(), o, atol=2e-5, rtol=1e-4)
        torch.testing.assert_close(state[slot, : H * dim * vdim].double(), S, atol=2e-5, rtol=1e-4)
    assert torch.equal(state[1], start[1]) and torch.equal(state[:, H * dim * vdim:], start[:, H * dim * vdim:])
    singles, s_state = run([[(0, 1)] for _ in range(T1)], {0: 2})
    assert torch.equal(singles[0], whole[0]) and torch.equal(s_state[2], state[2])
    cut, c_state = run([[(0, 2)], [(1, 3), (0, 17)], [(0, 1), (1, T2 - 3)], [(0, T1 - 20)]], {0: 2, 1: 0})
    assert torch.equal(cut[0], whole[0]) and torch.equal(cut[1], whole[1]) and torch.equal(c_state, state)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_head_norm_with_silu_and_one_weight_for_all_heads(dtype):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(7)
    T, H, vdim, eps, gain = 5, 3, 70, 1e-5, 0.9
    o = torch.randn(T, H * vdim, generator=g) * 4
    gate = torch.randn(T, H * vdim + 9, generator=g).to(dtype)
    w = 1 + 0.2 * torch.randn(vdim, generator=g)
    out = torch.full((T, H * vdim + 4), float("nan"), dtype=dtype, device="cuda")
    ops.gated_head_norm(o.cuda(), gate.cuda()[:, 9:], w.cuda(), eps, out[:, : H * vdim], H, vdim, gate="silu", gain=gain)
    x = o.double().view(T, H, vdim)
    want = (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.double()).reshape(T, -1) * plain.silu(gate[:, 9:].double()) * gain
    torch.testing.assert_close(out[:, : H * vdim].cpu().double(), want, **_tol(dtype, 3))
    assert bool(torch.isnan(out[:, H * vdim:].float()).all())
    # the earlier form: a weight per head and a sigmoid
    per_head = 1 + 0.2 * torch.randn(H * vdim, generator=g)
    dense = torch.empty((T, H * vdim), dtype=dtype, device="cuda")
    ops.gated_head_norm(o.cuda(), gate.cuda()[:, 9:], per_head.cuda(), eps, dense, H, vdim)
    want = (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, -1) * per_head.double() * torch.sigmoid(gate[:, 9:].double())
    torch.testing.assert_close(dense.cpu().double(), want, **_tol(dtype, 3))


# ------------------------------------------------------------------ the routed feed-forward

@pytest.mark.parametrize("E, top", [(20, 4), (7, 7), (130, 5), (3, 1)])
def test_router_over_all_scores_with_a_correction(E, top):
    """The scores are the softmax over all logits; the correction moves the choice (it is made large for a few experts that the scores
    alone would not pick) and stays out of the weights, which are not renormalised."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(8)
    T = 37
    logits = torch.randn(T, E, generator=g) * 2
    corr = torch.randn(E, generator=g) * 0.01
    corr[:: max(2, E // 3)] += 0.5
    s = torch.softmax(logits.double(), dim=-1)
    picked = torch.topk(s + corr.double(), top, dim=-1).indices
    assert not torch.equal(torch.sort(picked).values, torch.sort(torch.topk(s, top, dim=-1).indices).values) or top == E
    weights, offsets, slot_token, pair_slot = ops.route(logits.cuda(), top, "all", corr.cuda())
    weights, offsets, slot_token, pair_slot = weights.cpu(), offsets.cpu(), slot_token.cpu(), pair_slot.cpu()
    torch.testing.assert_close(weights.double(), s.gather(1, picked), atol=1e-6, rtol=1e-5)          # best first, as topk gives them
    assert int(offsets[0]) == 0 and int(offsets[-1]) == T * top
    for t in range(T):
        for j in range(top):
            slot = int(pair_slot[t * top + j])
            e = int(picked[t, j])
            assert int(offsets[e]) <= slot < int(offsets[e + 1]) and int(slot_token[slot]) == t
    plain_w, _, _, _ = ops.route(logits.cuda(), top, "all", None)
    torch.testing.assert_close(plain_w.cpu().double(), torch.topk(s, top, dim=-1).values, atol=1e-6, rtol=1e-5)
    chosen_w, _, _, _ = ops.route(logits.cuda(), top)                                           # the earlier form: softmax over the chosen
    torch.testing.assert_close(chosen_w.cpu().double(), torch.softmax(torch.topk(logits.double(), top, dim=-1).values, dim=-1), atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, ff, E, ident, top", [(40, 12, 5, 2, 3), (192, 64, 12, 3, 2), (64, 70, 3, 0, 1), (72, 32, 2, 3, 4)])
def test_gated_experts_and_identity_experts(dtype, H, ff, E, ident, top):
    """Route, the two grouped products (the first with the gate applied to pairs of columns) and the weighted sum, against the plain
    feed-forward; every row of the scratch buffers that belongs to an identity expert is NaN before and after."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(9)
    T = 45
    h = torch.randn(T, H, generator=g).to(dtype)
    w = {f"e{e}.{n}": (torch.randn(*shape, generator=g) / math.sqrt(shape[1])).to(dtype)
         for e in range(E) for n, shape in (("gate", (ff, H)), ("up", (ff, H)), ("down", (H, ff)))}
    w["router"] = torch.randn(E + ident, H, generator=g).to(dtype) * 0.3
    w["correction"] = torch.randn(E + ident, generator=g) * 0.02
    mlp = dict(router=dict(experts=E, identity=ident, top=top))
    want = plain.routed_gated_experts(h.double(), {k: v.double() for k, v in w.items()}, mlp)
    logits = (h.double() @ w["router"].double().T).float().cuda()
    weights, offsets, slot_token, pair_slot = ops.route(logits, top, "all", w["correction"].cuda())
    up = torch.stack([torch.stack((w[f"e{e}.gate"], w[f"e{e}.up"]), dim=1).reshape(2 * ff, H) for e in range(E)]).cuda()
    down = torch.stack([w[f"e{e}.down"] for e in range(E)]).cuda()
    z = torch.full((T * top, ff), float("nan"), dtype=dtype, device="cuda")
    y = torch.full((T * top, H), float("nan"), dtype=dtype, device="cuda")
    for general in ((False, True) if dtype == torch.bfloat16 else (False,)):
        ops.experts_linear(h.cuda(), slot_token, up, offsets, z, "silu_pairs", general=general)
        ops.experts_linear(z, None, down, offsets, y, general=general)
        out = torch.empty((T, H), dtype=dtype, device="cuda")
        ops.combine(y, pair_slot, weights, out, identity=(h.cuda(), offsets, E) if ident else None)
        torch.testing.assert_close(out.cpu().double(), want, **_tol(dtype, 4))
        real = int(offsets[E])
        assert not bool(torch.isnan(y[:real].float()).any()) and bool(torch.isnan(y[real:].float()).all()) and bool(torch.isnan(z[real:].float()).all())
