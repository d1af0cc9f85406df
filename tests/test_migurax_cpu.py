"""The Migurax design through the framework's host side on the CPU: configuration, tensor names, cache plan, the step
function under every way of cutting requests, and greedy generation through scheduler and sampler, with the HIP entry points
replaced by the stand-ins of ``emulated_ops.py``.  The kernels are tested on the GPU (``-m gpu``)."""
import json

import pytest
import torch

import plain_migurax
import scenarios
import tiny_migurax
from torchlet_amd.config import ConfigError, MiguraxConfig
from torchlet_amd.engine.batch import StepEntry
from torchlet_amd.engine.engine import Engine
from torchlet_amd.engine.loading import load_model, make_runner
from torchlet_amd.engine.request import Request
from torchlet_amd.registry import load_config

TOL = dict(atol=2e-4, rtol=2e-4)       # 32-bit stand-ins against a 64-bit evaluation, logits of order one to ten


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("migurax")
    return {name: tiny_migurax.write(name, root) for name in tiny_migurax.CONFIGS}


def _weights(name):
    return {k: v.double() for k, v in tiny_migurax.tensors_for(name).items()}


def test_configuration_expands_to_parts_and_names(folders):
    cfg = load_config(folders["P"])
    assert isinstance(cfg, MiguraxConfig)
    spec = cfg.to_spec()
    kinds = [(b.kind, b.mixer.kind, b.ffn.kind if b.ffn is not None else None) for b in spec.layers]
    assert kinds == [("postnorm_residual", "latent_attention", "routed_experts"), ("postnorm_residual", "mlstm", "dense_ff"),
                     ("postnorm_residual", "mlstm", None), ("postnorm_residual", "latent_attention", "routed_experts")]
    assert spec.layers[0].alpha == 1.5 and spec.layers[3].mixer.position.dims == 4 and spec.layers[1].mixer.gate_cap == 8.0
    from torchlet_amd.models.decoder import DecoderModel
    names = set(DecoderModel(spec, torch.float32, "cpu").weight_specs())
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.dq.norm", "l0.mix.sink", "l0.mlp.e4.down", "l0.mlp.router.b",
            "l1.mix.i.b", "l1.mix.norm", "l1.mlp.up.b", "l2.norm1", "l3.mlp.e2.up"} <= names
    assert "l2.norm2" not in names and not any(n.startswith("l2.mlp") for n in names)        # the layer without a feed-forward
    assert json.loads(json.dumps(cfg.to_dict()))["architecture"] == "Migurax"
    for bad in (dict(layers=[]), dict(layers=[dict(type="other", mixer={}, mlp=None)]), dict(norm={}),
                dict(layers=[dict(type="mlstm", mixer=dict(heads=1, dim=4, vdim=4), mlp=None)]),
                dict(layers=[dict(type="mlstm", mixer=dict(heads=1, dim=4, vdim=4, gate_cap=1.0), mlp=dict(kind="moe", expert=dict(ff=4), router=dict(experts=2, top=3)))])):
        with pytest.raises(ConfigError):
            MiguraxConfig.from_dict({**tiny_migurax.CONFIGS["P"], **bad})


def test_cache_plan_has_a_state_per_recurrent_layer_and_one_page_group_per_row_shape(cpu_ops, folders):
    _, model = load_model(folders["P"], "float32", device="cpu")
    runner = make_runner(model, page_size=4, num_pages=12, max_requests=3)
    cache = runner.cache
    assert [g.need.plane_shapes for g in cache.groups] == [((1, 28),), ((1, 24),)]
    states = [c.state for c in runner.caches]
    assert states[0] is None and states[3] is None
    assert tuple(states[1].shape) == (4, 2, 6 * 10 + 6 + 1) and tuple(states[2].shape) == (4, 1, 16 * 8 + 16 + 1)
    assert states[1].dtype == torch.float32
    # a slot that is used again starts from zero
    runner.step([StepEntry("a", [1, 2, 3], [])])
    slot = cache.slot("a")
    assert float(states[1][slot].abs().max()) > 0
    runner.release("a")
    runner.step([StepEntry("b", [4], [])])
    assert cache.slot("b") == slot
    fresh = make_runner(model, page_size=4, num_pages=12, max_requests=3)
    fresh.step([StepEntry("b", [4], [])])
    assert torch.equal(states[1][slot], fresh.caches[1].state[fresh.cache.slot("b")])


@pytest.mark.parametrize("name", ["P", "Q", "R", "T"])
@pytest.mark.parametrize("mode", ["whole", "tail_singles", "portions", "mixed"])
def test_step_function_equals_plain_under_every_split(cpu_ops, folders, name, mode):
    lengths = [37, 5, 70, 1, 18, 33] if name not in "QT" else [21, 1, 30]
    seqs, refs = tiny_migurax.clear_sequences(name, _weights(name), lengths)
    steps = scenarios.number(getattr(scenarios, mode)(seqs) if mode != "tail_singles" else scenarios.tail_singles(seqs, tail=9))
    page = tiny_migurax.PAGE_SIZES[name]
    _, model = load_model(folders[name], "float32", device="cpu")
    runner = make_runner(model, page_size=page, num_pages=-(-scenarios.max_tokens_needed(steps) // page) + 1, max_requests=4)
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            out[s["step"]] = logits.numpy()
        for r in s["end"]:
            runner.release(r)
        runner.cache.check()
    scenarios.check(steps, out, refs, TOL, f"{name}/{mode}")
    assert runner.cache.live_requests() == []


def test_layers_one_by_one_against_plain(cpu_ops, folders):
    """The stream after every layer, which the blocks keep in 32-bit."""
    w = _weights("P")
    ids = [5, 17, 3, 60, 2, 2, 41, 9, 30]
    want = []
    plain_migurax.forward(tiny_migurax.CONFIGS["P"], w, ids, layers_out=want)
    _, model = load_model(folders["P"], "float32", device="cpu")
    runner = make_runner(model, page_size=4, num_pages=8, max_requests=1)
    seen = []
    for block in model.blocks:
        inner = block.forward
        block.forward = lambda stream, ctx, cache, inner=inner: (lambda s: (seen.append(s.residual.clone()), s)[1])(inner(stream, ctx, cache))
    runner.step([StepEntry("a", ids, [len(ids) - 1])])
    assert len(seen) == 4
    for got, ref in zip(seen, want):
        torch.testing.assert_close(got.double(), ref, atol=1e-5, rtol=1e-5)


def _greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(plain_migurax.forward(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]


def test_greedy_generation_through_scheduler_and_sampler(cpu_ops, folders):
    """Prompts in portions of at most 12 tokens beside decode tokens, five requests over three slots (slots and pages are
    used again), against the plain loop."""
    w = _weights("R")
    cfg = tiny_migurax.CONFIGS["R"]
    g = torch.Generator().manual_seed(11)
    prompts = [torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for n in (5, 17, 33, 1, 9)]
    _, model = load_model(folders["R"], "float32", device="cpu")
    engine = Engine(make_runner(model, page_size=8, num_pages=20, max_requests=3), max_tokens_per_step=12)
    reqs = [Request(prompt_tokens=p, seed=i, max_new_tokens=6) for i, p in enumerate(prompts)]
    for r in reqs:
        engine.add_request(r)
    engine.run_until_done()
    for r, p in zip(reqs, prompts):
        assert r.output_tokens == _greedy(cfg, w, p, 6)
    assert engine.runner.cache.live_requests() == [] and len({tuple(r.output_tokens) for r in reqs}) > 1


def test_trace_replay_reads_the_architecture_from_the_folder(cpu_ops, folders, tmp_path, monkeypatch):
    from torchlet_amd.engine import loading, trace
    monkeypatch.setattr(loading, "require_gpu", lambda: torch.device("cpu"))
    seqs, refs = tiny_migurax.clear_sequences("P", _weights("P"), [13, 6])
    steps = scenarios.number(scenarios.mixed(seqs, seed=1))
    args = trace.parse_args(["--model", str(folders["P"]), "--dtype", "float32", "--out", str(tmp_path / "out"),
                             "--max-tokens", str(scenarios.max_tokens_needed(steps)), "--page-size", "4"])
    assert args.max_requests == 4
    import io
    said = io.StringIO()
    assert trace.run(args, [json.dumps(s) for s in steps], out=said) == 0
    assert said.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    import numpy as np
    out = {s["step"]: np.fromfile(tmp_path / "out" / f"{s['step']}.f32", dtype="<f4").reshape(-1, 97) for s in steps
           if any(e["want"] for e in s["entries"])}
    scenarios.check(steps, out, refs, TOL, "trace replay")


def test_command_line_writes_a_random_folder_of_the_architecture(tmp_path):
    """``python -m torchlet_amd init`` from a Migurax config.json: the folder it writes declares the same layers, stores
    every tensor the model declares under the design's names, and loads back through the registry."""
    from safetensors import safe_open
    from torchlet_amd.llm import main
    from torchlet_amd.models.decoder import DecoderModel
    src = tmp_path / "config.json"
    src.write_text(json.dumps(tiny_migurax.CONFIGS["T"]))
    assert main(["init", "--config", str(src), "--seed", "3", "--out", str(tmp_path / "out")]) == 0
    cfg = load_config(tmp_path / "out")
    assert isinstance(cfg, MiguraxConfig) and cfg.layers == tiny_migurax.CONFIGS["T"]["layers"] and cfg.postln_alpha == 2.5
    with safe_open(str(tmp_path / "out" / "model.safetensors"), framework="pt") as f:
        stored = set(f.keys())
    assert stored == set(DecoderModel(cfg.to_spec(), torch.float32, "cpu").weight_specs())
    assert {"embed", "head", "final.norm", "l0.mix.sink", "l0.mlp.router.b", "l1.mix.f.b", "l1.mlp.down.b"} <= stored
