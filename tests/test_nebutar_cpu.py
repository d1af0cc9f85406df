"""The Nebutar design through the framework's host side on the CPU: configuration, tensor names, run order, cache plan, pages given
back behind a chunk, the step function under every way of cutting requests, the streams after every layer run, greedy generation
through scheduler and sampler, the trace replay and the command line, with the HIP entry points replaced by the stand-ins of
``emulated_ops.py``.  The kernels are tested on the GPU (``-m gpu``)."""
import json

import numpy as np
import pytest
import torch

import plain_nebutar
import scenarios
import tiny_nebutar
from torchlet_amd.cache.manager import CacheManager
from torchlet_amd.config import ConfigError, NebutarConfig
from torchlet_amd.engine.batch import StepEntry
from torchlet_amd.engine.engine import Engine
from torchlet_amd.engine.loading import load_model, make_runner
from torchlet_amd.engine.request import Request
from torchlet_amd.parts.base import PagedNeed
from torchlet_amd.registry import load_config

TOL = dict(atol=5e-4, rtol=2e-4)       # 32-bit stand-ins against a 64-bit evaluation, logits of order ten


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("nebutar")
    return {name: tiny_nebutar.write(name, root) for name in tiny_nebutar.CONFIGS}


def _weights(name):
    return {k: v.double() for k, v in tiny_nebutar.tensors_for(name).items()}


def test_configuration_expands_to_parts_names_and_run_order(folders):
    cfg = load_config(folders["A"])
    assert isinstance(cfg, NebutarConfig)
    spec = cfg.to_spec()
    assert [e.layer for e in spec.order] == [0, 1, 1, 1, 2] and all(e.cache_of is None for e in spec.order)
    assert [(b.kind, b.mixer.kind, b.ffn.kind if b.ffn is not None else None) for b in spec.layers] == \
        [("hyper_connections", "parallel", "routed_experts"), ("hyper_connections", "parallel", None), ("hyper_connections", "parallel", "routed_experts")]
    left, right = (s for _, s, _ in spec.layers[0].mixer.branches)
    assert (left.kind, left.chunk, left.softcap, left.scale, left.vdim) == ("capped_attention", 7, 5.0, 0.4, 10)
    assert (right.kind, right.conv, right.kv_heads, right.norm_eps) == ("gated_delta", 4, 2, 1e-5)
    assert [s for _, _, s in spec.layers[0].mixer.branches] == [0.7, 1.2]
    ffn = spec.layers[0].ffn
    assert (ffn.experts, ffn.identity, ffn.top, ffn.gated, ffn.scores, ffn.choice_bias, ffn.router_bias) == (5, 2, 3, True, "all", True, False)
    assert spec.streams == 3 and spec.tie_head and spec.embed_scale == 2.0 and spec.position_table_name == "pos"
    from torchlet_amd.models.decoder import DecoderModel
    names = {n for n, s in DecoderModel(spec, torch.float32, "cpu").weight_specs().items() if not s.optional}
    assert names == set(tiny_nebutar.tensors_for("A"))
    assert {"embed", "pos", "final.norm", "final.norm.b", "l0.norm1.b", "l0.hc1.in", "l0.hc2.mix", "l0.mix.left.q", "l0.mix.right.q.conv",
            "l0.mix.right.A_log", "l0.mix.right.dt_bias", "l0.mix.right.norm", "l0.mlp.e4.gate", "l0.mlp.correction", "l0.mlp.router"} <= names
    assert "l1.norm2" not in names and "l1.hc2.in" not in names and "l0.mlp.e5.up" not in names       # no feed-forward; identity experts have no tensors
    assert json.loads(json.dumps(cfg.to_dict()))["loop"] == dict(start=1, stop=2, times=3)
    # no streams: the plain pre-norm block; no loop: every layer once
    plain = load_config(folders["C"]).to_spec()
    assert plain.streams == 0 and [b.kind for b in plain.layers] == ["prenorm_residual"] * 2 and [e.layer for e in plain.order] == [0, 1]
    base = tiny_nebutar.CONFIGS["A"]
    layer = base["layers"][0]
    for bad in (dict(layers=[]), dict(layers=[dict(layer, type="other")]), dict(norm={}), dict(streams=9), dict(loop=dict(start=2, stop=1, times=1)),
                dict(layers=[dict(layer, mixer=dict(layer["mixer"], left=dict(layer["mixer"]["left"], heads=3)))]),
                dict(layers=[dict(layer, mlp=dict(kind="dense", ff=8))]),
                dict(layers=[dict(layer, mlp=dict(kind="moe", expert=dict(ff=4), router=dict(experts=2, identity=1, top=4)))])):
        with pytest.raises(ConfigError):
            NebutarConfig.from_dict({**base, **bad})


def test_cache_plan_a_state_and_pages_per_run_of_a_layer(cpu_ops, folders):
    _, model = load_model(folders["A"], "float32", device="cpu")
    runner = make_runner(model, page_size=4, num_pages=40, max_requests=3)
    cache = runner.cache
    # five runs (the middle layer three times, each pass with its own cache): three kinds of pages, the middle one shared by three runs
    assert [(g.need.plane_shapes, g.need.chunk, len(g.runs)) for g in cache.groups] == \
        [(((2, 6), (2, 10)), 7, 1), (((3, 8), (3, 4)), 5, 3), (((1, 4), (1, 12)), 16, 1)]
    states = [c.state for c in runner.caches]
    assert [tuple(s.shape) for s in states] == [(4, 4 * 5 * 7 + 3 * (20 + 28))] + [(4, 16 * 8 + 1 * (32 + 8))] * 3 + [(4, 2 * 3 * 5)]
    assert states[1].data_ptr() != states[2].data_ptr() and all(s.dtype == torch.float32 for s in states)
    # a slot that is used again starts from zero: states and the convolutions' tails
    runner.step([StepEntry("a", [1, 2, 3], [])])
    slot = cache.slot("a")
    assert all(float(s[slot].abs().max()) > 0 for s in states)
    runner.release("a")
    runner.step([StepEntry("b", [4], [])])
    assert cache.slot("b") == slot
    fresh = make_runner(model, page_size=4, num_pages=40, max_requests=3)
    fresh.step([StepEntry("b", [4], [])])
    for s, f in zip(states, fresh.caches):
        assert torch.equal(s[slot], f.state[fresh.cache.slot("b")])


def test_pages_before_the_chunk_of_the_next_position_go_back():
    need = PagedNeed(num_heads=1, head_dim=4, chunk=10, planes=((1, 4), (1, 6)))
    cache = CacheManager([(need, None, None)], page_size=4, num_pages=20, max_requests=2)
    cache.add_request("a")
    assert cache.reserve("a", 9)
    cache.commit("a", 9)
    assert cache.free_pages() == [19 - 3]                      # positions 0..8: nothing behind the chunk of position 9 yet
    assert cache.reserve("a", 23)                              # a portion over two chunk borders: its queries read back to position 0
    assert [bool(p) for p in cache.groups[0].tables["a"]] == [True] * 6
    cache.commit("a", 23)                                      # the next position lies in the chunk from 20 on: blocks 0..4 are dead
    assert [bool(p) for p in cache.groups[0].tables["a"]] == [False] * 5 + [True] and cache.free_pages() == [18]
    assert cache.pages_missing("a", 24) == [0] and cache.pages_missing("a", 25) == [1]
    for n in range(24, 61):                                    # token by token: never more than a chunk's pages (and one) are held
        assert cache.reserve("a", n)
        cache.commit("a", n)
        cache.check()
        assert 19 - cache.free_pages()[0] <= 4
    # with a window as well, whichever reaches less far back decides
    both = PagedNeed(num_heads=1, head_dim=4, chunk=10, window=3, planes=2)
    assert both.reach == 3 and both.bounded and PagedNeed(num_heads=1, head_dim=4).reach is None
    cache = CacheManager([(both, None, None)], page_size=2, num_pages=20, max_requests=1, max_step_tokens=6)
    assert cache.capacity() == [(3 + 6 - 2) // 2 + 2]
    cache.add_request("b")
    cache.reserve("b", 9)
    cache.commit("b", 9)
    assert [bool(p) for p in cache.groups[0].tables["b"]] == [False, False, False, True, True]      # position 9 reads 7 and 8 (block 3 on)
    cache.release("b")
    cache.check()


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "tail_singles", "portions", "mixed"])
def test_step_function_equals_plain_under_every_split(cpu_ops, folders, name, mode):
    lengths = [37, 5, 50, 1, 18, 33] if name != "B" else [45, 1, 27]
    seqs, refs = tiny_nebutar.clear_sequences(name, _weights(name), lengths)
    steps = scenarios.number(getattr(scenarios, mode)(seqs) if mode != "tail_singles" else scenarios.tail_singles(seqs, tail=9))
    page = tiny_nebutar.PAGE_SIZES[name]
    _, model = load_model(folders[name], "float32", device="cpu")
    runner = make_runner(model, page_size=page, num_pages=-(-scenarios.max_tokens_needed(steps, unit=page) // page) + 1, max_requests=4)
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


def test_streams_after_every_layer_run_against_plain(cpu_ops, folders):
    """The sum of the copies of the residual after every run of a layer (a looped layer counts each time)."""
    w = _weights("A")
    ids = [5, 17, 3, 60, 2, 2, 41, 9, 30, 11, 90]
    want = []
    plain_nebutar.forward(tiny_nebutar.CONFIGS["A"], w, ids, layers_out=want)
    _, model = load_model(folders["A"], "float32", device="cpu")
    runner = make_runner(model, page_size=4, num_pages=8, max_requests=1)
    seen = []
    import emulated_ops

    def settled(stream):            # what the next norm would see: the pending output entered through its connection
        x = stream.residual.clone()
        emulated_ops.streams_norm(x, stream.pending, stream.fold, None, "rmsnorm", torch.ones(x.shape[2]), None, 1e-5, torch.empty(x.shape[1:]))
        return x.sum(0)

    for block in model.blocks:
        inner = block.forward
        block.forward = lambda stream, ctx, cache, inner=inner: (lambda s: (seen.append(settled(s)), s)[1])(inner(stream, ctx, cache))
    runner.step([StepEntry("a", ids, [len(ids) - 1])])
    assert len(seen) == 5
    for got, ref in zip(seen, want):
        torch.testing.assert_close(got.double(), ref, atol=2e-5, rtol=1e-5)


def _greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(plain_nebutar.forward(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]


def test_greedy_generation_through_scheduler_and_sampler(cpu_ops, folders):
    """Prompts in portions of at most 12 tokens beside decode tokens, five requests over three slots (slots and pages are
    used again), against the plain loop."""
    w = _weights("B")
    cfg = tiny_nebutar.CONFIGS["B"]
    g = torch.Generator().manual_seed(11)
    prompts = [torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for n in (5, 17, 33, 1, 9)]
    _, model = load_model(folders["B"], "float32", device="cpu")
    engine = Engine(make_runner(model, page_size=16, num_pages=12, max_requests=3), max_tokens_per_step=12)
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
    seqs, refs = tiny_nebutar.clear_sequences("A", _weights("A"), [13, 6, 22])
    steps = scenarios.number(scenarios.mixed(seqs, seed=1))
    args = trace.parse_args(["--model", str(folders["A"]), "--dtype", "float32", "--out", str(tmp_path / "out"),
                             "--max-tokens", str(scenarios.max_tokens_needed(steps)), "--page-size", "4"])
    import io
    said = io.StringIO()
    assert trace.run(args, [json.dumps(s) for s in steps], out=said) == 0
    assert said.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    out = {s["step"]: np.fromfile(tmp_path / "out" / f"{s['step']}.f32", dtype="<f4").reshape(-1, 97) for s in steps
           if any(e["want"] for e in s["entries"])}
    scenarios.check(steps, out, refs, TOL, "trace replay")


def test_command_line_writes_a_random_folder_of_the_architecture(cpu_ops, tmp_path):
    """``python -m torchlet_amd init`` from a Nebutar config.json: the folder it writes declares the same layers, stores every tensor
    the model declares under the design's names, loads back through the registry, and steps."""
    from safetensors import safe_open
    from torchlet_amd.llm import main
    from torchlet_amd.models.decoder import DecoderModel
    src = tmp_path / "config.json"
    src.write_text(json.dumps(tiny_nebutar.CONFIGS["A"]))
    assert main(["init", "--config", str(src), "--seed", "3", "--out", str(tmp_path / "out")]) == 0
    cfg = load_config(tmp_path / "out")
    assert isinstance(cfg, NebutarConfig) and cfg.layers == tiny_nebutar.CONFIGS["A"]["layers"] and cfg.streams == 3
    with safe_open(str(tmp_path / "out" / "model.safetensors"), framework="pt") as f:
        stored = set(f.keys())
        decay = f.get_tensor("l0.mix.right.A_log")
    assert stored == {n for n, s in DecoderModel(cfg.to_spec(), torch.float32, "cpu").weight_specs().items() if not s.optional}
    assert float(decay.max()) <= 0.0                      # the law of the decay rates' logarithms
    _, model = load_model(tmp_path / "out", "float32", device="cpu")
    logits = make_runner(model, page_size=4, num_pages=8, max_requests=1).step([StepEntry("a", [1, 2, 3, 4, 5], [4])])
    assert logits.shape == (1, 97) and bool(torch.isfinite(logits).all())
