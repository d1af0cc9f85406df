"""A plain, slow evaluation of the Migurax design: whole sequences, no cache, no batching.

One function per mechanism, written out from the design's equations with ``torch`` tensor arithmetic in
whatever floating-point type the weights come in (the tests pass float64).  It shares no code with the
package: the tests compare the engine against it.

Notation: ``T`` tokens, ``W`` the model width; a weight matrix is stored ``[out, in]`` and applied as
``x @ M.T``.  ``w`` maps tensor names (``l<i>.mix.q``, ``l<i>.mlp.e3.up``, ...) to tensors; ``cfg`` is the
content of ``config.json``.  ``stored`` is applied where separate kernels of an engine hand each other
activations through memory in the activation type, so that the tests can measure what such roundings do.
"""
import math

import torch


def _same(t):
    return t


def rms_norm(x, weight, eps):
    """``x / sqrt(mean(x^2) + eps) * weight`` over the last axis (``weight`` may be ``None``)."""
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def relu_squared(z):
    return torch.clamp(z, min=0) ** 2


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


def rotate_pairs(x, positions, base, dims):
    """Rotary encoding in the interleaved layout: of the first ``dims`` entries of the last axis, entry ``2i`` is
    paired with ``2i + 1`` and the pair turned by ``position * base**(-2i / dims)``; the rest passes unchanged.
    ``x [T, ..., n]``, ``positions [T]``.  Angles are taken in 32-bit, as an engine takes them."""
    i = torch.arange(dims // 2, dtype=torch.float32)
    freq = (float(base) ** (-2.0 * i / dims)).to(torch.float32)
    ang = (positions.to(torch.float32)[:, None] * freq[None, :]).to(x.dtype)
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = ang.cos().view(shape), ang.sin().view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    y = x.clone()
    y[..., 0:dims:2] = u * c - v * s
    y[..., 1:dims:2] = v * c + u * s
    return y


# ------------------------------------------------------------------------------------------- mLSTM

def mlstm_gates(h, w, cap):
    """Log input gate and log forget gate per head, ``[T, heads]`` each."""
    i = soft_cap(h @ w["i"].T + w["i.b"], cap)
    f = torch.nn.functional.logsigmoid(soft_cap(h @ w["f"].T + w["f.b"], cap))
    return i, f


def mlstm_recurrence(q, k, v, i, f, state=None):
    """The matrix memory, token by token.  ``q, k [T, heads, dim]`` (q already scaled), ``v [T, heads, vdim]``,
    ``i, f [T, heads]``.  Returns ``o [T, heads, vdim]`` and the state ``(S [heads, dim, vdim], n [heads, dim],
    m [heads])`` after the last token."""
    T, heads, dim = q.shape
    vdim = v.shape[-1]
    if state is None:
        S = torch.zeros(heads, dim, vdim, dtype=q.dtype)
        n = torch.zeros(heads, dim, dtype=q.dtype)
        m = torch.zeros(heads, dtype=q.dtype)
    else:
        S, n, m = (t.clone() for t in state)
    out = []
    for t in range(T):
        m_new = torch.maximum(f[t] + m, i[t])
        keep = torch.exp(f[t] + m - m_new)
        take = torch.exp(i[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out.append(num / den[:, None])
    return torch.stack(out), (S, n, m)


def mlstm_mixer(h, w, spec, eps, stored=_same):
    """``w``: the mixer's tensors by their short names (``q``, ``k``, ``v``, ``g``, ``o``, ``norm``, ``i``, ``i.b``, ...)."""
    T = h.shape[0]
    heads, dim, vdim = spec["heads"], spec["dim"], spec["vdim"]
    q = stored(h @ w["q"].T).view(T, heads, dim) * dim ** -0.5
    k = stored(h @ w["k"].T).view(T, heads, dim)
    v = stored(h @ w["v"].T).view(T, heads, vdim)
    i, f = mlstm_gates(h, w, spec["gate_cap"])
    o, _ = mlstm_recurrence(q, k, v, i, f)
    o = rms_norm(o, None, eps).reshape(T, heads * vdim) * w["norm"]
    o = stored(o * torch.sigmoid(stored(h @ w["g"].T)))
    return stored(o @ w["o"].T)


# -------------------------------------------------------------------------------- latent attention

def sink_softmax_weights(scores, sink):
    """Causal weights of ``scores [heads, T, T]`` whose denominator also holds ``exp(sink[head])``."""
    T = scores.shape[-1]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    scores = scores.masked_fill(~mask, -math.inf)
    top = torch.maximum(scores.max(-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(scores - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink[:, None, None] - top))


def latent_attention_mixer(h, w, spec, eps, positions, stored=_same):
    T = h.shape[0]
    H, dim, rot, vdim, rank = spec["heads"], spec["dim"], spec["rot_dim"], spec["vdim"], spec["kv_rank"]
    cq = stored(rms_norm(stored(h @ w["dq"].T), w["dq.norm"], eps))
    q = stored(cq @ w["uq"].T).view(T, H, dim + rot)
    q_plain, q_rot = q[..., :dim], q[..., dim:]
    down = stored(h @ w["dkv"].T)
    c = stored(rms_norm(down[:, :rank], w["dkv.norm"], eps))
    k_rot = down[:, rank:]
    base, dims = spec["rot"]["base"], spec["rot"]["dims"]
    q_rot = stored(rotate_pairs(q_rot, positions, base, dims))
    k_rot = stored(rotate_pairs(k_rot, positions, base, dims))
    k_plain = (c @ w["uk"].T).view(T, H, dim)
    val = (c @ w["uv"].T).view(T, H, vdim)
    scores = (torch.einsum("thd,shd->hts", q_plain, k_plain) + torch.einsum("thr,sr->hts", q_rot, k_rot)) * spec["scale"]
    p = sink_softmax_weights(scores, w["sink"])
    mixed = stored(torch.einsum("hts,shv->thv", p, val).reshape(T, H * vdim))
    return stored(mixed @ w["o"].T)


# ------------------------------------------------------------------------------------ feed-forward

def dense_ff(h, w, stored=_same):
    z = stored(relu_squared(stored(h @ w["up"].T + w["up.b"])))
    return stored(z @ w["down"].T + w["down.b"])


def route(h, w, top):
    """The chosen experts ``[T, top]`` (largest logit first) and their weights: the softmax over the chosen logits."""
    z = h @ w["router"].T + w["router.b"]
    best = z.topk(top, dim=-1)
    return best.indices, torch.softmax(best.values, dim=-1), z


def moe_ff(h, w, spec, stored=_same, gaps=None):
    top = spec["router"]["top"]
    idx, weight, z = route(h, w, top)
    if gaps is not None and z.shape[-1] > top:
        s = z.sort(dim=-1, descending=True).values
        gaps.append(float((s[:, top - 1] - s[:, top]).min()))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            z_e = stored(relu_squared(stored(h[t] @ w[f"e{e}.up"].T)))
            out[t] += weight[t, j] * stored(z_e @ w[f"e{e}.down"].T)
    return stored(out)


# ------------------------------------------------------------------------------------------- model

def sub(w, prefix):
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def forward(cfg, w, ids, stored=_same, layers_out=None, gaps=None):
    """Logits ``[T, vocab]`` of the token ids.  ``layers_out``: a list that receives the stream after every layer."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = w["embed"][torch.tensor(ids)]
    positions = torch.arange(len(ids))
    for n, layer in enumerate(cfg["layers"]):
        lw = sub(w, f"l{n}.")
        h = stored(x)
        if layer["type"] == "mlstm":
            y = mlstm_mixer(h, sub(lw, "mix."), layer["mixer"], eps, stored)
        elif layer["type"] == "latent_attention":
            y = latent_attention_mixer(h, sub(lw, "mix."), layer["mixer"], eps, positions, stored)
        else:
            raise ValueError(layer["type"])
        x = rms_norm(alpha * x + y, lw["norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = stored(x)
            y = dense_ff(h, sub(lw, "mlp."), stored) if mlp["kind"] == "dense" else moe_ff(h, sub(lw, "mlp."), mlp, stored, gaps)
            x = rms_norm(alpha * x + y, lw["norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return stored(rms_norm(x, w["final.norm"], eps)) @ w["head"].T
