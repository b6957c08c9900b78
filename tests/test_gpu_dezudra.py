"""The Dezudra design through the engine against the plain implementation (`plain_dezudra.py`): whole prompts, last
tokens one by one, portions of changing size, mixed batches with few pages, in float32 and in bfloat16, on tiny
configurations that differ in every size and option; requests alone against in a batch; pages and state slots used
again; windows that pass over decoded tokens and give their pages back; long decoding; greedy generation through
`LLMEngine` and the command lines."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_dezudra as pd
import replay_util as ru
import tiny_dezudra as td

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"A": (5, 9, 27, 70), "B": (7, 23, 40, 75), "C": (1, 2, 33, 70), "D": (3, 50, 66), "E": (4, 19, 45), "F": (6, 31, 52)}
# relative to the largest |logit| of the expected rows; fixed before the first run
TOL = {"float32": ru.FP32_TOL, "bfloat16": ru.BF16_TOL}
NAMES = sorted(td.CONFIGS)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in td.CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            d = tmp_path_factory.mktemp(f"dezudra_{name}_{dtype}")
            td.make_folder(cfg, seed=31, out_dir=str(d), dtype=dtype)
            out[(name, dtype)] = str(d)
    return out


def prompts_for(name):
    return {f"r{i}": td.random_tokens(n, td.CONFIGS[name]["vocab"], seed=400 + i) for i, n in enumerate(LENGTHS[name])}


_cache = {}


def plain_for(folders, name, dtype, prompts=None):
    """Per request: (logits, per routed layer the plain choice of experts), and for bfloat16 how far rounding every
    stored activation to 16 bits moves the logits of these prompts (relative to the largest logit): what 16-bit
    storage alone costs, with the same experts."""
    key = (name, dtype)
    if prompts is None and key in _cache:
        return _cache[key]
    cfg, weights = td.read_folder(folders[key])
    out, gap, scale = {}, 0.0, 0.0
    for rid, toks in (prompts or prompts_for(name)).items():
        scores = []
        logits = pd.forward(cfg, weights, toks, scores_out=scores)
        own = [ids for _, ids in scores]
        out[rid] = (logits, own)
        scale = max(scale, float(np.abs(logits).max()))
        if dtype == "bfloat16":
            stored = pd.forward(cfg, weights, toks, store=pd.bfloat16, experts=own)
            gap = max(gap, float(np.abs(stored - logits).max()))
    result = (out, gap / max(scale, 1e-30))
    if prompts is None:
        _cache[key] = result
    return result


class ChosenExperts:
    """What the engine's router chose, per (request, position) and routed layer: every step's batch is noted when it
    is run, and every routing call of that step (they come in layer order) has its selection read back."""

    def __init__(self, runner, monkeypatch):
        from inferx_amd.parts.moe import MoeFeedForward
        self.by_place = {}
        self._rows, self._calls = None, 0
        real_step, real_route = runner.step, MoeFeedForward.route_and_dispatch
        owner = self

        def step(batch):
            owner._rows = [(batch.request_ids[int(s)], int(p)) for s, p in zip(batch.seq_of_token, batch.positions)]
            owner._calls = 0
            return real_step(batch)

        def route_and_dispatch(part, ctx, x, tile_rows, norm=None, always=0):
            out = real_route(part, ctx, x, tile_rows, norm, always)
            if torch.cuda.is_current_stream_capturing():
                return out
            layer, owner._calls = owner._calls, owner._calls + 1
            for place, chosen in zip(owner._rows, out[1][:, :part.top_k].cpu().tolist()):
                owner.by_place.setdefault(place, {})[layer] = chosen
            return out
        runner.step = step
        monkeypatch.setattr(MoeFeedForward, "route_and_dispatch", route_and_dispatch)

    def of_request(self, rid, length, layers):
        return [np.array([self.by_place[(rid, pos)][l] for pos in range(length)]) for l in range(layers)]


NEAR_TIE_16 = 5e-2  # how far apart (relatively) two scores may lie for a 16-bit run to take either


def near_tie(scores, own, theirs, router):
    """Whether the engine's choice `theirs` for one token differs from the plain choice `own` by no more than a near
    tie: of the experts taken against those left out, or of the groups kept against those dropped."""
    if set(own) == set(theirs):
        return True
    groups = router.get("groups") or {"count": 1, "keep": 1}
    per = len(scores) // groups["count"]
    best = scores.reshape(groups["count"], per).max(axis=1)
    kept = set(np.argsort(-best, kind="stable")[:groups["keep"]].tolist())
    strangers = {e // per for e in theirs} - kept
    if strangers:  # another group was kept: its best score must be close to the worst kept group's
        worst_kept = min(best[g] for g in kept)
        return all((worst_kept - best[g]) / worst_kept < NEAR_TIE_16 for g in strangers)
    lost = max(scores[e] for e in set(own) - set(theirs))
    taken = min(scores[e] for e in set(theirs) - set(own))
    return (lost - taken) / lost < NEAR_TIE_16


def run_and_check(folders, name, dtype, steps, monkeypatch, what, prompts=None, only=None, **runner_kw):
    """Replays `steps` and compares every position with the plain implementation.  float32: as it is.  bfloat16: run
    kernel by kernel with the router's choices read back; where they differ from the plain ones they must be near
    ties, and the plain implementation is run with the engine's choices; the tolerance is twice what 16-bit storage
    alone costs (never below the fixed one)."""
    if dtype == "bfloat16":
        runner_kw.setdefault("use_graphs", False)
    runner = make_runner(folders, name, dtype, **runner_kw)
    chosen = ChosenExperts(runner, monkeypatch) if dtype == "bfloat16" else None
    got = ru.replay(runner, steps)
    plain, gap = plain_for(folders, name, dtype, prompts)
    every = prompts or prompts_for(name)
    expected = {}
    cfg, weights = td.read_folder(folders[(name, dtype)])
    routers = [l["mlp"]["router"] for l in cfg["layers"] if l.get("mlp") is not None]
    for rid in (only or every):
        logits, own = plain[rid]
        if chosen is not None and routers:
            theirs = chosen.of_request(rid, len(every[rid]), len(routers))
            if any(not np.array_equal(np.sort(a, axis=1), np.sort(b, axis=1)) for a, b in zip(own, theirs)):
                scores = []
                logits = pd.forward(cfg, weights, every[rid], experts=theirs, scores_out=scores)
                for l, ((s, ids), t) in enumerate(zip(scores, theirs)):
                    for pos in range(len(every[rid])):
                        assert near_tie(s[pos], ids[pos].tolist(), t[pos].tolist(), routers[l]), \
                            f"{what}: request {rid} position {pos} routed layer {l}: the engine chose {t[pos].tolist()}, " \
                            f"the plain implementation {ids[pos].tolist()}, and that is no near tie"
        expected[rid] = torch.from_numpy(logits)
    tol = TOL[dtype] if dtype == "float32" else max(TOL[dtype], 2 * gap)
    worst = ru.compare(got, expected, tol, what)
    print(f"{what}: worst {worst:.2e} (tolerance {tol:.1e})")
    return runner, got


def make_runner(folders, name, dtype, num_pages=64, page_size=16, max_requests=4, **kw):
    from inferx_amd.engine.runner import ModelRunner
    return ModelRunner.from_directory(folders[(name, dtype)], dtype=dtype, page_size=page_size, num_pages=num_pages,
                                      max_requests=max_requests, max_seq_len=num_pages * page_size, **kw)


WAYS = {"whole": lambda p: ru.whole(p), "tail": lambda p: ru.tail_decoded(p, 32), "portions": lambda p: ru.chunked(p)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("way", ["whole", "tail", "portions"])
def test_each_request_alone(folders, name, dtype, way, monkeypatch):
    run_and_check(folders, name, dtype, WAYS[way](prompts_for(name)), monkeypatch, f"{way} {name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_few_pages(folders, name, dtype, monkeypatch):
    """Up to four live requests, portions of some beside single tokens of others, in a pool with room for about two
    of the longer ones: pages and state slots are given back and used again, and that must happen for the run to
    count."""
    prompts = prompts_for(name)
    for i in range(4):  # more requests than slots
        prompts[f"x{i}"] = td.random_tokens(11 + 7 * i, td.CONFIGS[name]["vocab"], seed=500 + i)
    max_tokens = 192
    steps = ru.mixed(prompts, seed=8, max_tokens=max_tokens)
    assert any(len(s["entries"]) > 1 and {len(e[1]) for e in s["entries"]} & {1} and
               max(len(e[1]) for e in s["entries"]) > 1 for s in steps), "no step mixes a portion with a single token"
    run_and_check(folders, name, dtype, steps, monkeypatch, f"mixed {name} {dtype}", prompts, num_pages=max_tokens // 16)
    # the same steps once more, to see that pages really are used again
    owners = {}
    runner = make_runner(folders, name, dtype, num_pages=max_tokens // 16)
    ru.replay(runner, steps, page_owners=owners)
    if runner.cache.groups:  # (a model of recurrent layers only keeps nothing in pages)
        assert any(len(who) > 1 for who in owners.values()), "no physical page was used by two requests"


@pytest.mark.parametrize("name", ["A", "B"])
def test_a_batch_gives_what_each_request_gives_alone(folders, name):
    """float32: the logits of a request in a batch of unequal requests, cut into unequal portions, equal the logits of
    the same request run alone and whole, to rounding."""
    prompts = prompts_for(name)
    alone = ru.replay(make_runner(folders, name, "float32"), ru.whole(prompts))
    together = ru.replay(make_runner(folders, name, "float32"), ru.mixed(prompts, seed=5))
    scale = max(float(v.abs().max()) for v in alone.values())
    for key, row in alone.items():
        assert float((row - together[key]).abs().max()) <= 1e-5 * scale, f"{key} differs between alone and in a batch"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_slots_and_pages_that_others_left_dirty(folders, name, dtype, monkeypatch):
    """A request that starts in a state slot and on pages that hold another request's leftovers (made not-a-number
    here) gives the same logits: a sequence's first tokens read no state (neither the recurrent matrices nor the
    convolutions' last inputs), and no key beyond its own."""
    from inferx_amd.engine.runner import ModelRunner
    prompts = prompts_for(name)
    made = ModelRunner.from_directory

    def dirty(*a, **kw):  # every page and every state slot starts as not-a-number
        runner = made(*a, **kw)
        for arrays in runner.pages:
            for t in arrays.values():
                t.fill_(float("nan"))
        for state in runner._states:
            state.fill_(float("nan"))
        return runner
    monkeypatch.setattr(ModelRunner, "from_directory", dirty)
    second = {"r3": prompts["r3"], "r2": prompts["r2"], "r1": prompts["r1"]}  # one after the other in the one slot
    run_and_check(folders, name, dtype, ru.chunked(second, sizes=(3, 2, 5)), monkeypatch, f"dirty slots {name} {dtype}",
                  only=second, num_pages=8, max_requests=1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding_past_the_windows(folders, name, dtype, monkeypatch):
    """A short prompt and 150 tokens one by one (replayed from graphs once a shape has come three times), two requests
    side by side that started at different times: every window passes over decoded tokens, its pages go back, and
    the kept first tokens stay readable."""
    vocab = td.CONFIGS[name]["vocab"]
    prompts = {"a": td.random_tokens(156, vocab, 1), "b": td.random_tokens(140, vocab, 2)}
    steps = [{"entries": [("a", prompts["a"][:6], list(range(6)))], "end": []},
             {"entries": [("a", prompts["a"][6:16], list(range(10)))], "end": []},
             {"entries": [("a", prompts["a"][16:17], [0]), ("b", prompts["b"][:1], [0])], "end": []}]
    for i in range(1, 140):
        steps.append({"entries": [("a", prompts["a"][16 + i:17 + i], [0]), ("b", prompts["b"][i:i + 1], [0])],
                      "end": ["a", "b"] if i == 139 else []})
    _, plainly = run_and_check(folders, name, dtype, steps, monkeypatch, f"long decoding {name} {dtype}", prompts,
                               use_graphs=False)
    # the same steps with graphs: the same bits, the windows give pages back, the kept first tokens' page stays
    runner = make_runner(folders, name, dtype)
    held, got = [], {}
    for step in steps:
        got.update(ru.replay(runner, [dict(step, end=[])]))
        held.append(sum(p >= 0 for p in runner.cache.block_row("a", 0)))
        first_page = runner.cache.block_row("a", 0)[0]
        for rid in step["end"]:
            runner.end_request(rid)
    assert runner._graphs, "no step was replayed from a graph"
    assert held[-1] < -(-156 // 16), "the window never gave a page back"
    assert first_page >= 0, "the page of the kept first tokens was given back"
    for key, row in plainly.items():
        assert torch.equal(row, got[key]), f"{key}: replayed from a graph differs from kernel by kernel"


def test_giving_passed_pages_back_changes_no_logit(folders):
    """The same requests with windowed groups that keep every page: bit-equal logits."""
    prompts = prompts_for("A")
    give = ru.replay(make_runner(folders, "A", "float32"), ru.chunked(prompts))
    keep = ru.replay(make_runner(folders, "A", "float32", release_window_pages=False), ru.chunked(prompts))
    for key, row in give.items():
        assert torch.equal(row, keep[key]), f"{key} differs"


@pytest.mark.parametrize("page_size", [8, 48])
def test_other_page_sizes(folders, page_size, monkeypatch):
    for dtype in ("float32", "bfloat16"):
        run_and_check(folders, "A", dtype, ru.chunked(prompts_for("A")), monkeypatch, f"pages of {page_size} {dtype}",
                      num_pages=24, page_size=page_size)


def greedy_agrees(cfg, weights, prompt, out, dtype, what):
    seq = list(prompt)
    for i, token in enumerate(out):
        logits = pd.forward(cfg, weights, seq)[-1]
        want = int(np.argmax(logits))
        if token != want:
            top2 = np.sort(logits)[-2:]
            margin = float(top2[1] - top2[0]) / float(np.abs(logits).max())
            # a bfloat16 run may pick the other of two near-equal logits; anything else is a fault
            assert dtype == "bfloat16" and margin < 2e-2, f"{what}: token {i} is {token}, the plain implementation says {want}"
        seq.append(token)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    cfg, weights = td.read_folder(folders[(name, dtype)])
    prompts = [td.random_tokens(n, cfg["vocab"], seed=n) for n in (5, 9, 17, 30, 3, 12)]
    # a token budget below the longest prompt: prompts come in portions beside decoding requests; four at a time
    engine = LLMEngine(folders[(name, dtype)], dtype, max_num_seqs=4, max_model_len=96, max_num_batched_tokens=16,
                       num_gpu_blocks_override=20)
    outs = engine.generate(prompts, SamplingParams(max_tokens=12))
    for prompt, out in zip(prompts, outs):
        assert len(out) == 12
        if dtype == "float32":
            greedy_agrees(cfg, weights, prompt, out, dtype, f"{name} {dtype}")


def test_command_lines(folders, tmp_path):
    """`bin/inferx-generate` and `bin/trace_run` choose the model class by config.json."""
    folder = folders[("A", "float32")]
    cfg, weights = td.read_folder(folder)
    prompt = td.random_tokens(7, cfg["vocab"], 4)
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "inferx-generate"), "--model", folder, "--dtype",
                        "float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "5", "--max-model-len",
                        "64", "--num-gpu-blocks-override", "8"], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    tokens = json.loads(p.stdout.strip().splitlines()[-1])["output_token_ids"]
    assert len(tokens) == 5
    greedy_agrees(cfg, weights, prompt, list(tokens), "float32", "inferx-generate")

    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompt[:4], "want": [0, 3]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": prompt[4:], "want": [2]},
                                     {"id": "b", "tokens": prompt[:2], "want": []}], "end": ["a"]},
             {"step": 2, "entries": [{"id": "b", "tokens": prompt[2:3], "want": [0]}], "end": ["b"]}]
    out_dir = tmp_path / "logits"
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out",
                        str(out_dir), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = pd.forward(cfg, weights, prompt)
    scale = float(np.abs(want).max())
    for step, rows in ((0, [0, 3]), (1, [6]), (2, [2])):
        got = np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(len(rows), -1)
        assert float(np.abs(got - want[rows]).max()) <= ru.FP32_TOL * scale
