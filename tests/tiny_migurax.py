"""Tiny random-weight folders of the Migurax design for the tests: sizes chosen so that what could coincide does not
(query/key size against value size, rotated against unrotated dimensions, the query latent against the cache row),
with one head and with more heads than a tile has rows, at sizes that the matrix-core kernels take (Q, R) and at sizes they leave
to the general ones (P, S), with a router that picks one, some or all of its experts, with
a dense feed-forward, and with a layer that has none."""
import json
from pathlib import Path

import torch
from safetensors.torch import save_file


def _latent(heads, dim, rot, vdim, rank, q_rank, scale, base, dims=None):
    return dict(heads=heads, dim=dim, rot_dim=rot, vdim=vdim, kv_rank=rank, q_rank=q_rank, scale=scale,
                rot=dict(base=base, dims=rot if dims is None else dims))


def _moe(ff, experts, top):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


CONFIGS = {
    "P": dict(architecture="Migurax", vocab=97, width=40, postln_alpha=1.5, norm=dict(eps=1e-5), layers=[
        dict(type="latent_attention", mixer=_latent(3, 8, 4, 12, 24, 16, 0.3, 100.0), mlp=_moe(16, 5, 2)),
        dict(type="mlstm", mixer=dict(heads=2, dim=6, vdim=10, gate_cap=8.0), mlp=dict(kind="dense", ff=56)),
        dict(type="mlstm", mixer=dict(heads=1, dim=16, vdim=8, gate_cap=20.0), mlp=None),
        dict(type="latent_attention", mixer=_latent(1, 16, 8, 8, 16, 32, 0.2, 5000.0, dims=4), mlp=_moe(24, 3, 1)),
    ]),
    "Q": dict(architecture="Migurax", vocab=131, width=72, postln_alpha=1.0, norm=dict(eps=3e-6), layers=[
        dict(type="mlstm", mixer=dict(heads=4, dim=70, vdim=130, gate_cap=14.0), mlp=_moe(24, 4, 4)),
        dict(type="latent_attention", mixer=_latent(20, 16, 64, 16, 64, 40, 0.25, 20000.0), mlp=dict(kind="dense", ff=96)),
    ]),
    "R": dict(architecture="Migurax", vocab=64, width=64, postln_alpha=3.0, norm=dict(eps=1e-6), layers=[
        dict(type="latent_attention", mixer=_latent(4, 16, 32, 32, 128, 48, 0.18, 1000.0), mlp=_moe(32, 8, 3)),
        dict(type="mlstm", mixer=dict(heads=2, dim=32, vdim=64, gate_cap=10.0), mlp=_moe(32, 8, 3)),
        dict(type="latent_attention", mixer=_latent(4, 16, 32, 32, 128, 48, 0.18, 1000.0), mlp=dict(kind="dense", ff=128)),
    ]),
    # odd sizes everywhere: no width, rank or head size is a multiple of what the vectorised and matrix-core kernels want
    "T": dict(architecture="Migurax", vocab=53, width=36, postln_alpha=2.5, norm=dict(eps=2e-5), layers=[
        dict(type="latent_attention", mixer=_latent(2, 6, 2, 5, 10, 7, 0.4, 77.0), mlp=_moe(9, 2, 1)),
        dict(type="mlstm", mixer=dict(heads=3, dim=5, vdim=7, gate_cap=6.0), mlp=dict(kind="dense", ff=11)),
    ]),
    # no routing, outputs at full strength, for tests in which far-away context must show in the logits
    "S": dict(architecture="Migurax", vocab=80, width=64, postln_alpha=1.0, norm=dict(eps=1e-5), layers=[
        dict(type="latent_attention", mixer=_latent(2, 16, 16, 32, 32, 24, 0.25, 300.0), mlp=dict(kind="dense", ff=96)),
        dict(type="mlstm", mixer=dict(heads=2, dim=16, vdim=24, gate_cap=12.0), mlp=None),
        dict(type="latent_attention", mixer=_latent(2, 16, 16, 32, 32, 24, 0.25, 300.0), mlp=dict(kind="dense", ff=96)),
    ]),
}
SEEDS = {"P": 3, "Q": 4, "R": 6, "S": 8, "T": 9}
PAGE_SIZES = {"P": 4, "Q": 16, "R": 8, "S": 16, "T": 2}


def tensors_for(name: str, sharpen: float = 1.0) -> dict[str, torch.Tensor]:
    """bfloat16 tensors of configuration ``name``: the framework's random draw, then matrices scaled up to give activations
    of order one, routers scaled up so that choices are clear, forget gates biased open and sinks of order one.
    ``sharpen`` multiplies the query up-projections of the attention layers (peaked attention weights)."""
    from torchlet_amd.registry import config_class
    from torchlet_amd.weights.random_init import random_tensors
    cfg = config_class("Migurax").from_dict(CONFIGS[name])
    g = torch.Generator().manual_seed(SEEDS[name] + 100)
    # Clear choices of experts: every token's embedding carries three of a few fixed directions of the stream with weights
    # 1, 0.7 and 0.4, and expert e's router row looks along direction e.  (The stream keeps most of the embedding from
    # layer to layer.)  A choice that hung on the last bits of a logit would let a reduced-precision engine choose otherwise.
    width, vocab = CONFIGS[name]["width"], CONFIGS[name]["vocab"]
    routed = {n: layer["mlp"]["router"]["experts"] for n, layer in enumerate(CONFIGS[name]["layers"]) if layer["mlp"] and layer["mlp"]["kind"] == "moe"}
    basis = torch.linalg.qr(torch.randn(width, max(1, sum(routed.values())), generator=g)).Q.T * width ** 0.5   # orthogonal rows, entries of order one
    directions, code, at = {}, torch.zeros(vocab, width), 0
    for n, experts in routed.items():
        directions[n] = basis[at: at + experts]
        at += experts
        for t in range(vocab):
            a = t % experts
            b = (a + 1 + (t // experts) % max(experts - 1, 1)) % experts
            rest = [e for e in range(experts) if e not in (a, b)]
            picks = [a, b] + ([rest[(t // 7) % len(rest)]] if rest else [])
            for weight, e in zip((1.0, 0.7, 0.4), dict.fromkeys(picks)):
                code[t] += weight * directions[n][e]
    out = {}
    for k, v in random_tensors(cfg, SEEDS[name], torch.float32).items():
        if v.dim() == 2 and k not in ("embed",):
            v = v * (50.0 / v.shape[1] ** 0.5)                  # N(0, 1 / fan_in)
        if k.endswith((".mix.o", ".down")) and routed:
            v = v * 0.35                                        # the stream keeps most of what the layer before left
        if k == "embed":
            v = v * 25.0 + 2.5 * code
        if k.endswith(".router"):
            v = v * 0.1 + directions[int(k.split(".")[0][1:])] * (12.0 / width)
        if k.endswith(".uq"):
            v = v * sharpen
        if k.endswith(".sink"):
            v = torch.randn(v.shape, generator=g) + 1.0
        if k.endswith(".f.b"):
            v = v + 2.0
        if k.endswith(".b") and not k.endswith((".i.b", ".f.b")):
            v = torch.randn(v.shape, generator=g) * (0.1 if k.endswith(".router.b") else 0.3)
        out[k] = v.to(torch.bfloat16)
    return out


def write(name: str, root: Path, dtype=torch.bfloat16, sharpen: float = 1.0) -> Path:
    folder = Path(root) / f"migurax_{name}"
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(CONFIGS[name], indent=1))
    save_file({k: v.to(dtype).contiguous() for k, v in tensors_for(name, sharpen).items()}, str(folder / "model.safetensors"))
    return folder


def clear_sequences(name: str, weights, lengths, min_gap: float = 0.15, first_seed: int = 0):
    """Token sequences of the given lengths for which no token's choice of experts hangs on less than ``min_gap`` in a
    router logit (a reduced-precision engine would otherwise be free to choose differently), with the plain logits of each."""
    import plain_migurax
    cfg = CONFIGS[name]
    for seed in range(first_seed, first_seed + 20):
        g = torch.Generator().manual_seed(seed)
        seqs = {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}
        gaps: list[float] = []
        refs = {r: plain_migurax.forward(cfg, weights, t, gaps=gaps) for r, t in seqs.items()}
        if not gaps or min(gaps) > min_gap:
            return seqs, refs
    raise AssertionError("no seed gives every token a clear choice of experts")
