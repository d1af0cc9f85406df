"""A plain, slow evaluation of the Nebutar design: whole sequences, no cache, one function per mechanism, in the
dtype of the tensors it is given (the tests hand it float64).  It shares nothing with the package.

The design: token embedding times a factor plus a learned position row; layers whose residual is ``S`` streams joined by
hyper-connections; a layer norm with weight and bias ahead of every sublayer; a mixer made of two mixers side by side
(attention without positions, scores soft-capped, masked to chunks of the sequence; a gated delta rule behind short causal
convolutions), a feed-forward routed over gated experts, some of which are the identity; a span of layers run several
times in a row; the output head is the embedding table.
"""
import math

import torch


def layer_norm(x, weight, bias, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight + bias


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ------------------------------------------------------------------ the left mixer

def visible(n, chunk=None, window=None):
    """``[n, n]`` booleans: may query i read key j?  Causal; with ``chunk`` only inside its own chunk of the sequence
    (chunks are counted from position 0); with ``window`` only the last ``window`` keys."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    ok = j <= i
    if chunk:
        ok = ok & (i // chunk == j // chunk)
    if window:
        ok = ok & (j > i - window)
    return ok


def capped_attention(h, w, m):
    """Grouped-query attention with ``m['dim']`` query/key and ``m['vdim']`` value dimensions per head, no position encoding,
    ``score <- cap * tanh(score * scale / cap)``, the chunk mask, an ordinary softmax, and the output projection."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(n, H, d)
    k = (h @ w["k"].T).view(n, G, d)
    v = (h @ w["v"].T).view(n, G, dv)
    kv_of = torch.arange(H) // (H // G)
    s = torch.einsum("ihd,jhd->hij", q, k[:, kv_of]) * m["scale"]
    cap = m.get("softcap")
    if cap:
        s = cap * torch.tanh(s / cap)
    mask = m.get("mask") or {}
    s = s.masked_fill(~visible(n, chunk=mask.get("size")), float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhd->ihd", p, v[:, kv_of]).reshape(n, H * dv)
    return o @ w["o"].T


# ------------------------------------------------------------------ the right mixer

def short_convolution(x, taps_weight):
    """Per channel over time: ``y[t, c] = sum_j taps_weight[c, j] * x[t - (taps - 1) + j, c]`` with zeros before the start."""
    n, C = x.shape
    taps = taps_weight.shape[1]
    padded = torch.cat((torch.zeros(taps - 1, C, dtype=x.dtype), x), 0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + padded[j: j + n] * taps_weight[:, j]
    return y


def unit(x, eps=1e-6):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def delta_rule(q, k, v, beta, decay):
    """Per head, token after token: ``S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``.
    ``q, k [n, H, d]``, ``v [n, H, dv]``, ``beta, decay [n, H]``."""
    n, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv, dtype=q.dtype)
    out = torch.zeros(n, H, dv, dtype=q.dtype)
    for t in range(n):
        S = S * decay[t][:, None, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hde,hd->he", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    return out


def gated_delta_mixer(h, w, m, eps):
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_convolution(h @ w["q"].T, w["q.conv"])).view(n, G, d)
    k = silu(short_convolution(h @ w["k"].T, w["k.conv"])).view(n, G, d)
    v = silu(short_convolution(h @ w["v"].T, w["v.conv"])).view(n, H, dv)
    q = unit(q) * d ** -0.5
    k = unit(k)
    qk_of = torch.arange(H) // (H // G)
    beta = torch.sigmoid(h @ w["b"].T)
    decay = torch.exp(-torch.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))
    o = delta_rule(q[:, qk_of], k[:, qk_of], v, beta, decay)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w["norm"]
    o = o.reshape(n, H * dv) * silu(h @ w["g"].T)
    return o @ w["o"].T


def parallel_mixer(h, w, m, eps):
    left = capped_attention(h, sub(w, "left"), m["left"])
    right = gated_delta_mixer(h, sub(w, "right"), m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# ------------------------------------------------------------------ the feed-forward

def routed_gated_experts(h, w, mlp, chosen_out=None, gaps=None):
    """``gaps``: a list that receives, per token, how far the last chosen expert's choice score lies above the best one left out, as a
    share of the two scores' sizes (about the difference of their logits)."""
    r = mlp["router"]
    E, ident, top = r["experts"], r.get("identity", 0), r["top"]
    s = torch.softmax(h @ w["router"].T, dim=-1)                  # over all experts, the identity ones included
    pick = s + w["correction"] if "correction" in w else s
    idx = torch.topk(pick, top, dim=-1).indices
    if chosen_out is not None:
        chosen_out.append(idx)
    if gaps is not None and top < E + ident:
        ranked = torch.sort(pick, dim=-1, descending=True).values
        gaps.extend(((ranked[:, top - 1] - ranked[:, top]) / (ranked[:, top - 1].abs() + ranked[:, top].abs())).tolist())
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in idx[t].tolist():
            if e >= E:
                y = h[t]
            else:
                y = (silu(h[t] @ w[f"e{e}.gate"].T) * (h[t] @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T
            out[t] = out[t] + s[t, e] * y
    assert E + ident == w["router"].shape[0]
    return out


# ------------------------------------------------------------------ the model

def sub(w, prefix):
    return {k[len(prefix) + 1:]: v for k, v in w.items() if k.startswith(prefix + ".")}


def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg, w, ids, layers_out=None, chosen_out=None, gaps=None, stored=lambda t: t):
    """Logits ``[n, vocab]`` of the whole sequence ``ids``.  ``layers_out``: a list that receives the sum of the streams after every
    layer run.  ``stored``: applied to what the sublayers read and hand back (the tests round there, to see what reduced precision
    between the parts does to the logits)."""
    dtype = w["embed"].dtype
    n = len(ids)
    eps = cfg["norm"]["eps"]
    x0 = w["embed"][torch.tensor(ids)] * cfg["embedding"]["scale"] + w["pos"][:n]
    S = cfg.get("streams")
    xs = x0[None].repeat(S or 1, 1, 1)                          # [streams, n, width]
    for li in run_order(cfg):
        layer = cfg["layers"][li]
        lw = sub(w, f"l{li}")
        assert layer["type"] == "parallel"
        for q, fn in ((1, lambda z: parallel_mixer(z, sub(lw, "mix"), layer["mixer"], eps)),
                      (2, (lambda z: routed_gated_experts(z, sub(lw, "mlp"), layer["mlp"], chosen_out, gaps)) if layer.get("mlp") else None)):
            if fn is None:
                continue
            if S:
                u = torch.einsum("s,snw->nw", lw[f"hc{q}.in"], xs)
            else:
                u = xs[0]
            y = stored(fn(stored(layer_norm(u, lw[f"norm{q}"], lw[f"norm{q}.b"], eps))))
            if S:
                xs = torch.einsum("st,snw->tnw", lw[f"hc{q}.mix"], xs) + lw[f"hc{q}.out"][:, None, None] * y[None]
            else:
                xs = xs + y[None]
        if layers_out is not None:
            layers_out.append(xs.sum(0))
    x = stored(layer_norm(xs.sum(0), w["final.norm"], w["final.norm.b"], eps))
    return (x @ w["embed"].T).to(dtype)
