"""Each kernel of the recurrent mixer, the latent attention and the routed feed-forward alone, against plain 32/64-bit
formulas written here, at sizes that are no multiples of the kernels' tiles."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype, loose=1.0):
    return dict(atol=2e-5 * loose, rtol=2e-5 * loose) if dtype == torch.float32 else dict(atol=2e-2 * loose, rtol=2e-2 * loose)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("parts", [0, 1, 3])
def test_norm_after_the_sum(dtype, parts):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    T, H, alpha, eps = 7, 200, 1.7, 1e-5
    res = torch.randn(T, H, generator=g)
    w = (1 + 0.1 * torch.randn(H, generator=g)).to(dtype)
    if parts == 0:
        pen = torch.randn(T, H, generator=g).to(dtype)
        add = pen.float()
    else:
        pen = torch.randn(parts, T, H, generator=g)
        add = pen.sum(0)
    r = alpha * res.double() + add.double()
    want = r / torch.sqrt(r.pow(2).mean(-1, keepdim=True) + eps) * w.double()
    residual = res.cuda()
    out = torch.empty(T, H, dtype=dtype, device="cuda") if dtype == torch.bfloat16 else None
    ops.scaled_add_rmsnorm(residual, pen.cuda(), alpha, w.cuda(), eps, out)
    torch.testing.assert_close(residual.cpu().double(), want, atol=1e-5, rtol=1e-5)       # the stream stays 32-bit in both engines
    if out is not None:
        torch.testing.assert_close(out.cpu().double(), want, atol=2e-2, rtol=1e-2)
    plain = res.cuda()
    ops.scaled_add_rmsnorm(plain, None, 1.0, w.cuda(), eps, None if dtype == torch.float32 else out)
    r = res.double()
    torch.testing.assert_close(plain.cpu().double(), r / torch.sqrt(r.pow(2).mean(-1, keepdim=True) + eps) * w.double(), atol=1e-5, rtol=1e-5)


def _plain_mlstm(q, k, v, gi, gf, cap, state):
    S, n, m = state
    out = []
    for t in range(q.shape[0]):
        i = cap * torch.tanh(gi[t] / cap) if cap else gi[t]
        f = torch.nn.functional.logsigmoid(cap * torch.tanh(gf[t] / cap) if cap else gf[t])
        m_new = torch.maximum(f + m, i)
        keep, take = torch.exp(f + m - m_new), torch.exp(i - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out.append(torch.einsum("hdv,hd->hv", S, q[t]) / den[:, None])
    return torch.stack(out), (S, n, m)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim,cap", [(2, 40, 56, 12.0), (3, 20, 70, None), (1, 130, 96, 4.0), (2, 300, 130, 9.0), (1, 700, 40, 5.0)])
def test_mlstm_scan_portions_and_slots(dtype, heads, dim, vdim, cap):
    """Three requests in slots out of order, one of them continuing from a state that an earlier call left; a request's
    tokens in one call and the same tokens over two calls give the same outputs and the same state, bit for bit."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(heads * 1000 + dim)
    lens = [11, 1, 19]
    T = sum(lens)
    W = 2 * heads * dim + heads * vdim + 5            # a row longer than what the kernel reads
    qkv = torch.randn(T, W, generator=g).to(dtype)
    gates = torch.randn(T, 2 * heads, generator=g) * 3
    gates[:, heads:] += 2.0
    width = dim * vdim + dim + 1
    slots = torch.tensor([2, 0, 3], dtype=torch.int32)
    state = torch.zeros(5, heads, width)
    indptr = torch.tensor([0, 11, 12, 31], dtype=torch.int32)
    qscale = dim ** -0.5
    dev_state = state.cuda()
    out = torch.empty(T, heads * vdim, device="cuda")
    ops.mlstm_scan(qkv.cuda(), heads * dim, 2 * heads * dim, gates.cuda(), dev_state, slots.cuda(), indptr.cuda(), out, heads, dim, vdim,
                   cap, qscale, 1e-6)
    x = qkv.double()
    start = 0
    for r, n in enumerate(lens):
        rows = slice(start, start + n)
        q = x[rows, : heads * dim].view(n, heads, dim) * qscale
        k = x[rows, heads * dim: 2 * heads * dim].view(n, heads, dim)
        v = x[rows, 2 * heads * dim: 2 * heads * dim + heads * vdim].view(n, heads, vdim)
        zero = (torch.zeros(heads, dim, vdim, dtype=torch.float64), torch.zeros(heads, dim, dtype=torch.float64), torch.zeros(heads, dtype=torch.float64))
        want, (S, nn, m) = _plain_mlstm(q, k, v, gates[rows, :heads].double(), gates[rows, heads:].double(), cap, zero)
        torch.testing.assert_close(out[rows].cpu().double().view(n, heads, vdim), want, atol=2e-4, rtol=2e-4)
        st = dev_state[int(slots[r])].cpu().double()
        torch.testing.assert_close(st[:, : dim * vdim].view(heads, dim, vdim), S, atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(st[:, dim * vdim: dim * vdim + dim], nn, atol=1e-4, rtol=1e-4)
        torch.testing.assert_close(st[:, -1], m, atol=1e-5, rtol=1e-5)
        start += n
    assert float(dev_state[1].abs().max()) == 0 and float(dev_state[4].abs().max()) == 0        # slots of no request: untouched
    # the third request again, cut after 7 and after 8 tokens (one token alone), in another slot
    again = torch.zeros(5, heads, width).cuda()
    out2 = torch.empty(19, heads * vdim, device="cuda")
    for lo, hi in ((0, 7), (7, 8), (8, 19)):
        ops.mlstm_scan(qkv[12 + lo: 12 + hi].cuda(), heads * dim, 2 * heads * dim, gates[12 + lo: 12 + hi].cuda().contiguous(), again,
                       torch.tensor([1], dtype=torch.int32).cuda(), torch.tensor([0, hi - lo], dtype=torch.int32).cuda(), out2[lo:hi],
                       heads, dim, vdim, cap, qscale, 1e-6)
    assert torch.equal(out2, out[12:]) and torch.equal(again[1], dev_state[3])


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_head_norm(dtype):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    T, heads, vdim, eps = 5, 3, 70, 1e-5
    o = torch.randn(T, heads * vdim, generator=g) * 3
    gate_full = torch.randn(T, 2 * heads * vdim, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(heads * vdim, generator=g)).to(dtype)
    out = torch.empty(T, heads * vdim, dtype=dtype, device="cuda")
    ops.gated_head_norm(o.cuda(), gate_full.cuda()[:, heads * vdim:], w.cuda(), eps, out, heads, vdim)
    x = o.double().view(T, heads, vdim)
    want = (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, -1) * w.double() * torch.sigmoid(gate_full[:, heads * vdim:].double())
    torch.testing.assert_close(out.cpu().double(), want, **_tol(dtype))


def _turn(x, positions, inv_freq):
    d = 2 * inv_freq.numel()
    ang = positions.double()[:, None] * inv_freq.double()[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [d // 2]
    c, s = ang.cos().view(shape), ang.sin().view(shape)
    y = x.clone()
    y[..., 0:d:2] = x[..., 0:d:2] * c - x[..., 1:d:2] * s
    y[..., 1:d:2] = x[..., 1:d:2] * c + x[..., 0:d:2] * s
    return y


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rot,rot_dims", [(32, 32), (24, 16)])
def test_latent_prepare_and_rotate(dtype, rot, rot_dims):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    T, q_rank, rank, page, eps = 9, 40, 72, 4, 1e-5
    down = torch.randn(T, q_rank + rank + rot, generator=g).to(dtype)
    wq = (1 + 0.1 * torch.randn(q_rank, generator=g)).to(dtype)
    wkv = (1 + 0.1 * torch.randn(rank, generator=g)).to(dtype)
    inv_freq = (500.0 ** (-2.0 * torch.arange(rot_dims // 2, dtype=torch.float64) / rot_dims)).float()
    positions = torch.tensor([5, 6, 7, 0, 1, 2, 3, 4, 33], dtype=torch.int32)
    token_req = torch.tensor([0, 0, 0, 1, 1, 1, 1, 1, 2], dtype=torch.int32)
    table = torch.tensor([[0, 3, 0, 0, 0, 0, 0, 0, 0], [5, 2, 0, 0, 0, 0, 0, 0, 0], [0, 0, 0, 0, 0, 0, 0, 0, 0]], dtype=torch.int32)   # request 2: the sentinel
    plane = torch.full((7, 1, page, rank + rot), float("nan"), dtype=dtype, device="cuda")
    cq = torch.empty(T, q_rank, dtype=dtype, device="cuda")
    ops.latent_prepare(down.cuda(), q_rank, rank, rot, rot_dims, wq.cuda(), wkv.cuda(), eps, positions.cuda(), inv_freq.cuda(), cq,
                       token_req.cuda(), table.cuda(), plane, page)
    x = down.double()
    norm = lambda t, w: t / torch.sqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w.double()
    torch.testing.assert_close(cq.cpu().double(), norm(x[:, :q_rank], wq), **_tol(dtype))
    rows = torch.cat((norm(x[:, q_rank: q_rank + rank], wkv), _turn(x[:, q_rank + rank:], positions, inv_freq)), dim=-1)
    written = torch.zeros(7, page, dtype=torch.bool)
    for t in range(T - 1):
        p = int(positions[t]); pg = int(table[int(token_req[t]), p // page])
        torch.testing.assert_close(plane[pg, 0, p % page].cpu().double(), rows[t], **_tol(dtype, 2))
        written[pg, p % page] = True
    assert bool(torch.isnan(plane.cpu().float()[:, 0][~written]).all())        # nothing else was written, the sentinel page least of all
    heads, dim = 3, 10
    q = torch.randn(T, heads * (dim + rot), generator=g).to(dtype)
    dst = torch.zeros(T, heads * (rank + rot), dtype=dtype, device="cuda")
    ops.rotate_pairs(q.cuda(), dim + rot, dim, dst, rank + rot, rank, positions.cuda(), inv_freq.cuda(), heads, rot)
    want = _turn(q.double().view(T, heads, dim + rot)[..., dim:], positions, inv_freq)
    got = dst.cpu().double().view(T, heads, rank + rot)
    torch.testing.assert_close(got[..., rank:], want, **_tol(dtype, 2))
    assert float(got[..., :rank].abs().max()) == 0


def _plain_latent_attention(q, rows_of, ctx_lens, new_lens, heads, rank, rot, scale, sink):
    """q [T, heads, D] float64; rows_of[r]: [total, D] cached rows of request r."""
    out, t = [], 0
    for r, n in enumerate(new_lens):
        for i in range(n):
            keys = rows_of[r][: ctx_lens[r] + i + 1]
            s = (q[t] @ keys.T) * scale
            top = s.max(-1, keepdim=True).values
            if sink is not None:
                top = torch.maximum(top, sink[:, None])
            e = torch.exp(s - top)
            den = e.sum(-1, keepdim=True) + (torch.exp(sink[:, None] - top) if sink is not None else 0)
            out.append((e / den) @ keys[:, :rank])
            t += 1
    return torch.stack(out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tile_rows", [16, 64])
@pytest.mark.parametrize("heads,rank,rot,page,splits,with_sink", [(7, 64, 32, 16, 1, True), (3, 40, 8, 4, 3, True), (20, 72, 16, 8, 2, False),
                                                                   (1, 130, 0, 16, 1, True), (16, 128, 32, 16, 2, True), (5, 192, 64, 8, 1, False),
                                                                   (2, 64, 0, 4, 3, True), (9, 512, 64, 16, 1, True)])
def test_latent_attention_against_formula(dtype, heads, rank, rot, page, splits, with_sink, tile_rows):
    """Portions and single tokens in one call, over pages handed out in a scrambled order; one request's last query leans
    on its first key, far back, and its sink is large enough to show when it is left out."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(heads * 100 + rank)
    D = rank + rot
    ctx_lens, new_lens = [0, 70, 133, 5], [37, 1, 9, 1]
    totals = [c + n for c, n in zip(ctx_lens, new_lens)]
    blocks = [-(-t // page) for t in totals]
    pages = sum(blocks) + 1
    order = (torch.randperm(pages - 1, generator=g) + 1).tolist()
    table = torch.zeros(len(totals), max(blocks), dtype=torch.int32)
    plane = torch.full((pages, 1, page, D), float("nan"), dtype=dtype)
    rows_of = []
    for r, total in enumerate(totals):
        rows = torch.randn(total, D, generator=g).to(dtype)
        rows[0] *= 3.0
        rows_of.append(rows.double())
        for b in range(blocks[r]):
            table[r, b] = order.pop()
            chunk = rows[b * page: (b + 1) * page]
            plane[int(table[r, b]), 0, : chunk.shape[0]] = chunk
    plane = torch.nan_to_num(plane, nan=1e4)          # unwritten places: large numbers that a mask must hide
    T = sum(new_lens)
    q = (torch.randn(T, heads, D, generator=g) * 0.5).to(dtype)
    q[37 + 1 + 8] = (rows_of[2][0] * 0.8).to(dtype)    # the last token of request 2 looks for its first key
    sink = (torch.randn(heads, generator=g) * 2 + 3) if with_sink else None
    scale = 0.3
    on_matrix_cores = ops.latent_attention_mfma_fits(dtype, heads, rank, rot)
    assert on_matrix_cores == (dtype == torch.bfloat16 and (rank + rot) % 32 == 0 and rank % 64 == 0)
    if tile_rows > 16 and not on_matrix_cores:
        pytest.skip("tiles of more than 16 rows are the matrix-core kernel's")
    tq = ops.latent_tile_tokens(heads, tile_rows)
    tile_req, tile_tok0 = [], []
    for r, n in enumerate(new_lens):
        for t0 in range(0, n, tq):
            tile_req.append(r); tile_tok0.append(t0)
    indptr = torch.tensor([0, 37, 38, 47, 48], dtype=torch.int32)
    out = torch.empty(T, heads * rank, dtype=dtype, device="cuda")
    ops.latent_attention(q.view(T, heads * D).cuda(), out, plane.cuda(), table.cuda(), indptr.cuda(), torch.tensor(ctx_lens, dtype=torch.int32).cuda(),
                         torch.tensor(tile_req, dtype=torch.int32).cuda(), torch.tensor(tile_tok0, dtype=torch.int32).cuda(), len(tile_req), tq,
                         heads, rank, rot, page, scale, sink.cuda() if with_sink else None, splits, max_new_tokens=max(new_lens))
    want = _plain_latent_attention(q.double(), rows_of, ctx_lens, new_lens, heads, rank, rot, scale, sink.double() if with_sink else None)
    torch.testing.assert_close(out.cpu().double().view(T, heads, rank), want, **_tol(dtype))
    if on_matrix_cores:        # the general kernel on the same operands
        out2 = torch.empty_like(out)
        if tile_rows == 16:
            ops.latent_attention(q.view(T, heads * D).cuda(), out2, plane.cuda(), table.cuda(), indptr.cuda(), torch.tensor(ctx_lens, dtype=torch.int32).cuda(),
                                 torch.tensor(tile_req, dtype=torch.int32).cuda(), torch.tensor(tile_tok0, dtype=torch.int32).cuda(), len(tile_req), tq,
                                 heads, rank, rot, page, scale, sink.cuda() if with_sink else None, splits, general=True)
            torch.testing.assert_close(out2.cpu().double().view(T, heads, rank), want, **_tol(dtype))
    if with_sink:          # the sink matters here: left out, the result would be off by far more than the tolerance
        without = _plain_latent_attention(q.double(), rows_of, ctx_lens, new_lens, heads, rank, rot, scale, None)
        assert float((without - want).abs().max()) > 0.05


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,rank,rot,page", [(5, 48, 16, 8), (8, 64, 32, 8), (24, 256, 64, 16)])
def test_latent_attention_decode_without_tile_list(dtype, heads, rank, rot, page):
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(9)
    D = rank + rot
    ctx_lens = [300, 0, 17]
    table = torch.zeros(3, 40, dtype=torch.int32)
    plane = torch.full((64, 1, page, D), 1e4, dtype=dtype)
    rows_of, nxt = [], 1
    for r, c in enumerate(ctx_lens):
        rows = torch.randn(c + 1, D, generator=g).to(dtype)
        rows_of.append(rows.double())
        for b in range(-(-(c + 1) // page)):
            table[r, b] = nxt
            chunk = rows[b * page: (b + 1) * page]
            plane[nxt, 0, : chunk.shape[0]] = chunk
            nxt += 1
    q = (torch.randn(3, heads, D, generator=g) * 0.5).to(dtype)
    sink = torch.randn(heads, generator=g)
    for splits in (1, 4):
        out = torch.empty(3, heads * rank, dtype=dtype, device="cuda")
        ops.latent_attention(q.view(3, -1).cuda(), out, plane.cuda(), table.cuda(), None, torch.tensor(ctx_lens, dtype=torch.int32).cuda(), None, None, 3, 1,
                             heads, rank, rot, page, 0.25, sink.cuda(), splits)
        want = _plain_latent_attention(q.double(), rows_of, ctx_lens, [1, 1, 1], heads, rank, rot, 0.25, sink.double())
        torch.testing.assert_close(out.cpu().double().view(3, heads, rank), want, **_tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,G,N,K,gap", [(70, 3, 37, 22, 6), (70, 3, 37, 64, 8), (1, 5, 300, 32, 0), (33, 2, 64, 96, 16), (16, 1, 130, 160, 8)])
def test_heads_linear(dtype, T, G, N, K, gap):
    """Sizes the matrix-core kernel takes (bfloat16, K a multiple of 32, aligned rows) and sizes it leaves to the general one."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, G * (K + gap) + (8 if K % 32 == 0 else 2), generator=g).to(dtype)
    w = torch.randn(G, N, K, generator=g).to(dtype)
    out = torch.zeros(T, G * (N + 3), dtype=dtype, device="cuda")
    ops.heads_linear(x.cuda(), K + gap, w.cuda(), out, N + 3)
    got = out.cpu().double()
    for h in range(G):
        want = x[:, h * (K + gap): h * (K + gap) + K].double() @ w[h].double().T
        torch.testing.assert_close(got[:, h * (N + 3): h * (N + 3) + N], want, **_tol(dtype, 4))
        assert float(got[:, h * (N + 3) + N: (h + 1) * (N + 3)].abs().max()) == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,F", [(24, 19), (64, 96)])
@pytest.mark.parametrize("T,experts,top", [(1, 4, 2), (150, 7, 3), (33, 5, 5), (64, 16, 1)])
def test_routed_products(dtype, T, experts, top, H, F):
    """The choice (ties go to the lower index), the weights, the sort by expert, and both products with the weighted sum."""
    from torchlet_amd.kernels import ops
    g = torch.Generator().manual_seed(T + experts)
    logits = torch.randn(T, experts, generator=g)
    logits[0, :] = 0.5                         # a tie over all experts: the lowest indices win
    weights, offsets, slot_token, pair_slot = ops.route(logits.cuda(), top)
    want_idx = torch.stack([torch.tensor(sorted(range(experts), key=lambda e: (-float(logits[t, e]), e))[:top]) for t in range(T)])
    want_w = torch.softmax(torch.gather(logits, 1, want_idx).double(), dim=-1)
    torch.testing.assert_close(weights.cpu().double(), want_w, atol=1e-6, rtol=1e-6)
    offsets, slot_token, pair_slot = offsets.cpu(), slot_token.cpu(), pair_slot.cpu()
    assert int(offsets[0]) == 0 and int(offsets[-1]) == T * top and sorted(pair_slot.tolist()) == list(range(T * top))
    for t in range(T):
        for j in range(top):
            s = int(pair_slot[t * top + j]); e = int(want_idx[t, j])
            assert int(offsets[e]) <= s < int(offsets[e + 1]) and int(slot_token[s]) == t
    x = torch.randn(T, H, generator=g).to(dtype)
    w_up = torch.randn(experts, F, H, generator=g).to(dtype) * 0.3
    w_down = torch.randn(experts, H, F, generator=g).to(dtype) * 0.3
    z = torch.empty(T * top, F, dtype=dtype, device="cuda")
    ops.experts_linear(x.cuda(), slot_token.cuda(), w_up.cuda(), offsets.cuda(), z, "relu2")
    y = torch.empty(T * top, H, dtype=dtype, device="cuda")
    ops.experts_linear(z, None, w_down.cuda(), offsets.cuda(), y)
    out = torch.empty(T, H, dtype=dtype, device="cuda")
    ops.combine(y, pair_slot.cuda(), weights, out)
    want = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(top):
            e = int(want_idx[t, j])
            want[t] += want_w[t, j] * (torch.clamp(x[t].double() @ w_up[e].double().T, min=0) ** 2 @ w_down[e].double().T)
    torch.testing.assert_close(out.cpu().double(), want, **_tol(dtype, 8))


@pytest.mark.parametrize("dtype", DTYPES)
def test_activation_in_place(dtype):
    from torchlet_amd.kernels import ops
    x = torch.linspace(-3, 3, 1001).to(dtype)
    y = x.cuda()
    ops.activation(y, "relu2")
    torch.testing.assert_close(y.cpu().double(), torch.clamp(x.double(), min=0) ** 2, **_tol(dtype))
