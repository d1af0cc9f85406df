"""Tiny random-weight folders of the Nebutar design for the tests: sizes chosen so that what could coincide does not (query/key
size against value size, heads of the two mixers, key heads against heads), with one stream, several and none, with and without a
span of layers that runs more than once, with convolutions of one tap and of several, with routers that pick one, some or all of
their experts, with and without identity experts, a layer without a feed-forward, attention with and without cap and chunks, at
sizes that the matrix-core kernels take and at sizes they leave to the general ones."""
import json
from pathlib import Path

import torch
from safetensors.torch import save_file


def _left(heads, kv_heads, dim, vdim, scale, softcap=None, chunk=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if softcap is not None:
        m["softcap"] = softcap
    if chunk is not None:
        m["mask"] = dict(size=chunk)
    return m


def _right(heads, kv_heads, dim, vdim, conv):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)


def _layer(left, right, left_scale, right_scale, mlp):
    return dict(type="parallel", mixer=dict(left=left, right=right, left_scale=left_scale, right_scale=right_scale), mlp=mlp)


def _moe(ff, experts, identity, top):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, identity=identity, top=top))


CONFIGS = {
    # nothing coincides; three streams; the middle layer (which has no feed-forward) runs three times
    "A": dict(architecture="Nebutar", vocab=97, width=40, max_positions=256, norm=dict(eps=1e-5), embedding=dict(scale=2.0), streams=3,
              loop=dict(start=1, stop=2, times=3), layers=[
        _layer(_left(4, 2, 6, 10, 0.4, softcap=5.0, chunk=7), _right(4, 2, 5, 7, 4), 0.7, 1.2, _moe(12, 5, 2, 3)),
        _layer(_left(3, 3, 8, 4, 0.3, softcap=2.0, chunk=5), _right(1, 1, 16, 8, 2), 1.0, 0.5, None),
        _layer(_left(2, 1, 4, 12, 0.5, softcap=8.0, chunk=16), _right(2, 2, 3, 5, 1), 1.3, 0.8, _moe(8, 3, 0, 1)),
    ]),
    # sizes of the matrix-core kernels; one stream (with its own connection weights); two layers looped twice; a chunk that is no multiple of the page
    "B": dict(architecture="Nebutar", vocab=80, width=64, max_positions=512, norm=dict(eps=3e-6), embedding=dict(scale=4.0), streams=1,
              loop=dict(start=0, stop=2, times=2), layers=[
        _layer(_left(8, 2, 32, 64, 0.18, softcap=12.0, chunk=24), _right(4, 2, 32, 32, 3), 0.6, 0.9, _moe(32, 4, 1, 2)),
        _layer(_left(4, 4, 64, 32, 0.12, softcap=30.0, chunk=40), _right(2, 1, 64, 80, 4), 1.0, 1.0, _moe(64, 6, 2, 3)),
    ]),
    # no streams (the plain residual), no loop, attention without cap and without chunks, a router that picks all
    "C": dict(architecture="Nebutar", vocab=53, width=36, max_positions=128, norm=dict(eps=2e-5), embedding=dict(scale=1.0), layers=[
        _layer(_left(2, 1, 16, 16, 0.25), _right(3, 1, 20, 6, 3), 1.0, 1.0, _moe(9, 2, 1, 3)),
        _layer(_left(6, 2, 5, 3, 0.45, chunk=3), _right(2, 2, 70, 9, 5), 0.9, 1.1, _moe(7, 4, 0, 2)),
    ]),
    # every token takes the one expert: nothing hangs on a choice; far-away context reaches the logits through the recurrent state
    "S": dict(architecture="Nebutar", vocab=80, width=64, max_positions=512, norm=dict(eps=1e-5), embedding=dict(scale=3.0), streams=2, layers=[
        _layer(_left(4, 1, 16, 32, 0.25, softcap=15.0, chunk=32), _right(2, 2, 16, 24, 3), 0.8, 1.0, _moe(48, 1, 0, 1)),
        _layer(_left(4, 2, 16, 32, 0.25, softcap=25.0, chunk=48), _right(4, 1, 32, 16, 3), 0.8, 1.0, _moe(48, 1, 0, 1)),
    ]),
}
SEEDS = {"A": 13, "B": 14, "C": 16, "S": 18}
PAGE_SIZES = {"A": 4, "B": 16, "C": 8, "S": 16}


def tensors_for(name: str, sharpen: float = 1.0) -> dict[str, torch.Tensor]:
    """bfloat16 tensors of configuration ``name``: the framework's random draw, then matrices scaled up to give activations of order
    one, routers that look along directions the embeddings carry (so that choices of experts are clear), connection weights away
    from the trivial ones, decays between slow and fast.  ``sharpen`` multiplies the attention's query projections."""
    from torchlet_amd.registry import config_class
    from torchlet_amd.weights.random_init import random_tensors
    conf = CONFIGS[name]
    cfg = config_class("Nebutar").from_dict(conf)
    g = torch.Generator().manual_seed(SEEDS[name] + 100)
    width, vocab = conf["width"], conf["vocab"]
    routed = {n: (layer["mlp"]["router"]["experts"] + layer["mlp"]["router"].get("identity", 0), layer["mlp"]["router"]["top"])
              for n, layer in enumerate(conf["layers"]) if layer["mlp"]}
    basis = torch.linalg.qr(torch.randn(width, max(1, sum(o for o, _ in routed.values())), generator=g)).Q.T * width ** 0.5
    directions, code, at = {}, torch.zeros(vocab, width), 0
    for n, (outputs, top) in routed.items():
        directions[n] = basis[at: at + outputs]
        at += outputs
        for t in range(vocab):      # a token's embedding leans towards as many of the layer's experts as the router picks, each less than the one before
            picks = torch.randperm(outputs, generator=g)[:top].tolist()
            for j, e in enumerate(picks):
                code[t] += (1.0 - 0.3 * j) * directions[n][e]
    routed_choices = any(outputs > top for outputs, top in routed.values())
    out = {}
    for k, v in random_tensors(cfg, SEEDS[name], torch.float32).items():
        tail = k.split(".", 1)[-1]
        if v.dim() == 2 and k not in ("embed", "pos") and not k.endswith((".conv", ".mix")) and ".hc" not in k:
            v = v * (50.0 / v.shape[1] ** 0.5)                  # N(0, 1 / fan_in)
        if k.endswith((".o", ".down")):
            v = v * (0.2 if routed_choices else 1.0)            # where no choice of experts hangs on it, the layers write at full strength
        if k.endswith(".A_log") and not routed_choices:
            v = torch.log(0.002 + 0.02 * torch.rand(v.shape, generator=g))      # slow decays: the state remembers hundreds of tokens
        if k == "embed":
            v = v * 15.0 + 1.2 * code
        if k == "pos":
            v = v * 10.0
        if k.endswith(".router"):
            v = v * 0.03 + directions[int(k.split(".")[0][1:])] * (4.0 / width)
        if k.endswith(".correction"):
            v = torch.randn(v.shape, generator=g) * 0.01
        if k.endswith(".left.q"):
            v = v * sharpen
        if k.endswith(".conv"):
            v = v * 2.0 + (torch.arange(v.shape[1]) == v.shape[1] - 1).float() * 0.5
        if k.endswith(".dt_bias"):
            v = torch.randn(v.shape, generator=g) * 0.7
        if k.endswith((".norm1.b", ".norm2.b", "final.norm.b")):
            v = torch.randn(v.shape, generator=g) * 0.1
        if k.endswith((".norm1", ".norm2", "final.norm", ".right.norm")):
            v = 1.0 + (v - 1.0) * 8.0
        if ".hc" in k:
            streams = conf.get("streams", 1)
            if tail.endswith(".in"):
                v = torch.randn(v.shape, generator=g) * 0.25 + 1.0 / streams ** 0.5
            elif tail.endswith(".out"):
                v = torch.randn(v.shape, generator=g) * 0.2 + 0.6
            else:
                v = torch.eye(streams) + torch.randn(v.shape, generator=g) * 0.08
        out[k] = v.to(torch.bfloat16)
    return out


def write(name: str, root: Path, dtype=torch.bfloat16, sharpen: float = 1.0) -> Path:
    folder = Path(root) / f"nebutar_{name}"
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(CONFIGS[name], indent=1))
    save_file({k: v.to(dtype).contiguous() for k, v in tensors_for(name, sharpen).items()}, str(folder / "model.safetensors"))
    return folder


def clear_sequences(name: str, weights, lengths, min_gap: float = 0.03, first_seed: int = 0):
    """Token sequences of the given lengths for which no token's choice of experts hangs on less than ``min_gap`` in a choice score
    (a reduced-precision engine would otherwise be free to choose differently), with the plain logits of each."""
    import plain_nebutar
    cfg = CONFIGS[name]
    best = None
    for seed in range(first_seed, first_seed + 30):
        g = torch.Generator().manual_seed(seed)
        seqs = {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}
        gaps: list[float] = []
        refs = {r: plain_nebutar.forward(cfg, weights, t, gaps=gaps) for r, t in seqs.items()}
        if not gaps or min(gaps) > min_gap:
            return seqs, refs
        best = max(best or 0.0, min(gaps))
    raise AssertionError(f"no seed gives every token a clear choice of experts (best smallest gap {best})")
