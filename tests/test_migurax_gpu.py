"""The Migurax design on the GPU through the framework's step function, cache manager, scheduler and entry point, against
the plain implementation: every way of cutting requests in both dtypes, long decoding from the first token, slots and
pages used again, decode steps replayed as graphs, context far back, and greedy generation."""
import pytest
import torch

import plain_migurax
import scenarios
import tiny_migurax

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
FP32_TOL = dict(atol=3e-4, rtol=3e-4)        # logits of order one to ten; sums in another order than the 64-bit evaluation


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("migurax")
    return {name: tiny_migurax.write(name, root) for name in tiny_migurax.CONFIGS}


_weights_cache: dict = {}


def _weights(name, sharpen=1.0):
    key = (name, sharpen)
    if key not in _weights_cache:
        _weights_cache[key] = {k: v.double() for k, v in tiny_migurax.tensors_for(name, sharpen).items()}
    return _weights_cache[key]


def _tolerance(dtype, name, seqs, refs, sharpen=1.0):
    """32-bit: a fixed bound.  bfloat16: twice what rounding every tensor that kernels hand each other through memory to
    bfloat16 does to the logits in a 64-bit evaluation (the engine rounds at such places, not necessarily the same ones)."""
    if dtype == "float32":
        return FP32_TOL
    rounded = lambda t: t.to(torch.bfloat16).double()
    moved = max(float((plain_migurax.forward(tiny_migurax.CONFIGS[name], _weights(name, sharpen), t, stored=rounded) - refs[r]).abs().max())
                for r, t in seqs.items())
    return dict(atol=2 * moved, rtol=0.0)


def _runner(folder, name, dtype, pages, slots=4, graphs=False):
    from torchlet_amd.engine.loading import load_model, make_runner
    _, model = load_model(folder, dtype)
    return make_runner(model, page_size=tiny_migurax.PAGE_SIZES[name], num_pages=pages, max_requests=slots, use_graphs=graphs)


def _replay(runner, steps):
    from torchlet_amd.engine.batch import StepEntry
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            out[s["step"]] = logits.cpu().numpy()
        for r in s["end"]:
            runner.release(r)
        runner.cache.check()
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["P", "Q", "R", "T"])
def test_every_way_of_cutting_requests_equals_plain(folders, name, dtype):
    """Whole requests; most of a request and its last tokens one by one; portions of changing size down to two tokens; up to
    four live requests with portions beside single tokens, in a pool that holds no more than the live ones need, so pages and
    slots are used again."""
    lengths = [37, 5, 70, 1, 18, 33] if name not in "QT" else [21, 1, 30]
    seqs, refs = tiny_migurax.clear_sequences(name, _weights(name), lengths, min_gap=0.15)
    tol = _tolerance(dtype, name, seqs, refs)
    page = tiny_migurax.PAGE_SIZES[name]
    for mode in ("whole", "tail_singles", "portions", "mixed"):
        steps = scenarios.number(getattr(scenarios, mode)(seqs) if mode != "tail_singles" else scenarios.tail_singles(seqs, tail=9))
        runner = _runner(folders[name], name, dtype, pages=-(-scenarios.max_tokens_needed(steps) // page) + 1)
        scenarios.check(steps, _replay(runner, steps), refs, tol, f"{name}/{mode}/{dtype}")
        assert runner.cache.live_requests() == []


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_from_the_first_token_and_slots_used_again(folders, dtype):
    """300 tokens one by one from an empty cache equal the plain implementation; the same request once more in the slot and the
    pages that the first one gave back, after another request has used them, gives the same logits bit for bit."""
    from torchlet_amd.engine.batch import StepEntry
    name = "R"
    seqs, refs = tiny_migurax.clear_sequences(name, _weights(name), [300], min_gap=0.15, first_seed=40)
    tol = _tolerance(dtype, name, seqs, refs)
    ids = seqs["r0"]
    runner = _runner(folders[name], name, dtype, pages=-(-300 // 8) + 1, slots=1)

    def one_by_one(req):
        rows = [runner.step([StepEntry(req, [t], [0])]).cpu() for t in ids]
        runner.release(req)
        return torch.cat(rows)

    first = one_by_one("a")
    torch.testing.assert_close(first.double(), refs["r0"], **tol)
    runner.step([StepEntry("other", ids[50:150], [])])          # leaves its own state and rows in the slot and the pages
    runner.release("other")
    assert torch.equal(one_by_one("b"), first)
    whole = runner.step([StepEntry("c", ids, list(range(300)))]).cpu()
    torch.testing.assert_close(whole.double(), refs["r0"], **tol)


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_steps_replayed_as_graphs(folders, dtype):
    """Three requests of unequal lengths decode together from static buffers under a recorded graph (padding rows use the state
    row and the page that belong to no request): replays give what eager steps give."""
    from torchlet_amd.engine.batch import StepEntry
    name = "R"
    seqs, refs = tiny_migurax.clear_sequences(name, _weights(name), [40, 9, 23], min_gap=0.15, first_seed=7)
    got = {}
    for graphs in (False, True):
        runner = _runner(folders[name], name, dtype, pages=20, slots=3, graphs=graphs)
        assert runner.use_graphs == graphs
        rows = {r: [] for r in seqs}
        for r, t in seqs.items():
            rows[r].append(runner.step([StepEntry(r, t[:5], list(range(5)))]).cpu())
        for i in range(5, 40):
            live = [r for r, t in seqs.items() if i < len(t)]
            out = runner.step([StepEntry(r, [seqs[r][i]], [0]) for r in live]).cpu()
            for j, r in enumerate(live):
                rows[r].append(out[j: j + 1])
        got[graphs] = {r: torch.cat(v) for r, v in rows.items()}
        if graphs:
            assert runner.graph_replays > 20
    tol = _tolerance(dtype, name, seqs, refs)
    for r in seqs:
        torch.testing.assert_close(got[True][r].double(), refs[r], **tol)
        torch.testing.assert_close(got[True][r], got[False][r], atol=tol["atol"] / 2, rtol=0.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_context_far_back_shows_in_the_logits(folders, tmp_path, dtype):
    """A model without routing, with sharpened attention and outputs at full strength: changing the first token of a 200-token
    request changes the last logits (through keys far back and through the recurrent state) by several times the bound that the
    engine meets, in a prompt's portion and in a token decoded alone."""
    from torchlet_amd.engine.batch import StepEntry
    name, sharpen = "S", 3.0
    folder = tiny_migurax.write(name, tmp_path, sharpen=sharpen)
    w = _weights(name, sharpen)
    cfg = tiny_migurax.CONFIGS[name]
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, cfg["vocab"], (200,), generator=g).tolist()
    seqs = {"a": ids}
    refs = {"a": plain_migurax.forward(cfg, w, ids)}
    tol = _tolerance(dtype, name, seqs, refs, sharpen)
    other = plain_migurax.forward(cfg, w, [(ids[0] + 1) % cfg["vocab"]] + ids[1:])
    assert float((other[-1] - refs["a"][-1]).abs().max()) > 3 * max(tol["atol"], 1e-3)
    runner = _runner(folder, name, dtype, pages=14, slots=2)
    whole = runner.step([StepEntry("w", ids, [198, 199])]).cpu()
    torch.testing.assert_close(whole.double(), refs["a"][198:], **tol)
    runner.release("w")
    runner.step([StepEntry("d", ids[:150], [])])
    runner.step([StepEntry("d", ids[150:199], [])])
    last = runner.step([StepEntry("d", ids[199:], [0])]).cpu()
    torch.testing.assert_close(last.double(), refs["a"][199:], **tol)


def _greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(plain_migurax.forward(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_entry_point(folders, dtype):
    """``LLM(folder).generate``: the registry picks the architecture from config.json, the scheduler cuts the prompts into
    portions of at most 16 tokens beside decode tokens, four requests share three slots, decode steps run as graphs."""
    from torchlet_amd import LLM
    name = "S"
    cfg, w = tiny_migurax.CONFIGS[name], _weights(name)
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for n in (5, 40, 1, 23)]
    llm = LLM(str(folders[name]), max_decode_slots=3, kv_block_size=16, max_num_blocks=24, dtype=dtype, max_num_batched_tokens=16,
              max_model_len=128)
    outs = llm.generate(prompts, max_new_tokens=7)
    assert [len(o) for o in outs] == [7] * 4 and len({tuple(o) for o in outs}) > 1
    for p, o in zip(prompts, outs):
        if dtype == "float32":
            assert o == _greedy(cfg, w, p, 7)
        else:                                   # a reduced-precision engine may pick another token among near-ties
            ids = list(p)
            for tok in o:
                logits = plain_migurax.forward(cfg, w, ids)[-1]
                assert float(logits.max() - logits[tok]) <= 0.1
                ids.append(tok)
    assert llm.runner.cache.live_requests() == []
