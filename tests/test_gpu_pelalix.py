"""The Pelalix design through the engine against the plain implementation (`plain_pelalix.py`): whole prompts, last
tokens one by one, portions of changing size, mixed batches with few pages, in float32 and in bfloat16, on tiny
configurations that differ in every size and option; requests alone against in a batch; pages and state slots used
again; long decoding; greedy generation through `LLMEngine` and the command lines."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_pelalix as pp
import replay_util as ru
import tiny_pelalix as tp

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"P": (5, 9, 17, 70), "Q": (7, 23, 40, 75), "R": (3, 50, 66), "S": (1, 2, 33, 70), "U": (4, 19, 45)}
# relative to the largest |logit| of the expected rows; fixed before the first run
TOL = {"float32": ru.FP32_TOL, "bfloat16": ru.BF16_TOL}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in tp.CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            d = tmp_path_factory.mktemp(f"pelalix_{name}_{dtype}")
            tp.make_folder(cfg, seed=21, out_dir=str(d), dtype=dtype)
            out[(name, dtype)] = str(d)
    return out


def prompts_for(name):
    return {f"r{i}": tp.random_tokens(n, tp.CONFIGS[name]["vocab"], seed=200 + i) for i, n in enumerate(LENGTHS[name])}


_expected = {}


def expected_for(folders, name, dtype, prompts=None):
    key = (name, dtype)
    if prompts is not None:
        cfg, weights = tp.read_folder(folders[key])
        return {rid: pp.forward(cfg, weights, toks) for rid, toks in prompts.items()}
    if key not in _expected:
        cfg, weights = tp.read_folder(folders[key])
        _expected[key] = {rid: pp.forward(cfg, weights, toks) for rid, toks in prompts_for(name).items()}
    return _expected[key]


def make_runner(folders, name, dtype, num_pages=64, page_size=16, max_requests=4):
    from inferx_amd.engine.runner import ModelRunner
    return ModelRunner.from_directory(folders[(name, dtype)], dtype=dtype, page_size=page_size, num_pages=num_pages,
                                      max_requests=max_requests, max_seq_len=num_pages * page_size)


WAYS = {"whole": lambda p: ru.whole(p), "tail": lambda p: ru.tail_decoded(p, 32), "portions": lambda p: ru.chunked(p)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R", "S", "U"])
@pytest.mark.parametrize("way", ["whole", "tail", "portions"])
def test_each_request_alone(folders, name, dtype, way):
    runner = make_runner(folders, name, dtype)
    got = ru.replay(runner, WAYS[way](prompts_for(name)))
    worst = ru.compare(got, expected_for(folders, name, dtype), TOL[dtype], f"{way} {name} {dtype}")
    print(f"{way} {name} {dtype}: worst {worst:.2e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q", "R", "S", "U"])
def test_mixed_batches_with_few_pages(folders, name, dtype):
    """Up to four live requests, portions of some beside single tokens of others, in a pool with room for about two
    of the longer ones: pages and state slots are given back and used again, and that must happen for the run to
    count."""
    prompts = prompts_for(name)
    for i in range(4):  # more requests than slots
        prompts[f"x{i}"] = tp.random_tokens(11 + 7 * i, tp.CONFIGS[name]["vocab"], seed=300 + i)
    max_tokens = 192
    runner = make_runner(folders, name, dtype, num_pages=max_tokens // 16)
    owners = {}
    steps = ru.mixed(prompts, seed=8, max_tokens=max_tokens)
    assert any(len(s["entries"]) > 1 and {len(e[1]) for e in s["entries"]} & {1} and
               max(len(e[1]) for e in s["entries"]) > 1 for s in steps), "no step mixes a portion with a single token"
    got = ru.replay(runner, steps, page_owners=owners)
    assert any(len(who) > 1 for who in owners.values()), "no physical page was used by two requests"
    ru.compare(got, expected_for(folders, name, dtype, prompts), TOL[dtype], f"mixed {name} {dtype}")


@pytest.mark.parametrize("name", ["P", "Q"])
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
def test_slots_and_pages_that_others_left_dirty(folders, dtype):
    """A request that starts in a state slot and on pages that hold another request's leftovers (made not-a-number
    here) gives the same logits: a sequence's first token reads no state, and no key beyond its own."""
    name = "P"
    prompts = prompts_for(name)
    runner = make_runner(folders, name, dtype, num_pages=8, max_requests=1)
    first = {"r3": prompts["r3"]}
    ru.replay(runner, ru.chunked(first))
    for arrays in runner.pages:
        for t in arrays.values():
            t.fill_(float("nan"))
    for state in runner._states:
        state.fill_(float("nan"))
    second = {"r2": prompts["r2"], "r1": prompts["r1"]}
    got = ru.replay(runner, ru.chunked(second, sizes=(3, 2, 5)))
    exp = expected_for(folders, name, dtype)
    ru.compare(got, {k: exp[k] for k in second}, TOL[dtype], f"dirty slots {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_long_decoding(folders, name, dtype):
    """A short prompt and 150 tokens one by one (replayed from graphs once a shape has come three times), two requests
    side by side that started at different times."""
    vocab = tp.CONFIGS[name]["vocab"]
    prompts = {"a": tp.random_tokens(156, vocab, 1), "b": tp.random_tokens(140, vocab, 2)}
    steps = [{"entries": [("a", prompts["a"][:6], list(range(6)))], "end": []},
             {"entries": [("a", prompts["a"][6:16], list(range(10)))], "end": []},
             {"entries": [("a", prompts["a"][16:17], [0]), ("b", prompts["b"][:1], [0])], "end": []}]
    for i in range(1, 140):
        steps.append({"entries": [("a", prompts["a"][16 + i:17 + i], [0]), ("b", prompts["b"][i:i + 1], [0])],
                      "end": ["a", "b"] if i == 139 else []})
    runner = make_runner(folders, name, dtype)
    got = ru.replay(runner, steps)
    assert runner._graphs, "no step was replayed from a graph"
    ru.compare(got, expected_for(folders, name, dtype, prompts), TOL[dtype], f"long decoding {name} {dtype}")


@pytest.mark.parametrize("page_size", [8, 48])
def test_other_page_sizes(folders, page_size):
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folders, "P", dtype, num_pages=24, page_size=page_size)
        got = ru.replay(runner, ru.chunked(prompts_for("P")))
        ru.compare(got, expected_for(folders, "P", dtype), TOL[dtype], f"pages of {page_size} {dtype}")


def greedy_agrees(cfg, weights, prompt, out, dtype, what):
    seq = list(prompt)
    for i, token in enumerate(out):
        logits = pp.forward(cfg, weights, seq)[-1]
        want = pp.greedy(logits)
        if token != want:
            top2 = torch.topk(logits, 2).values
            margin = float(top2[0] - top2[1]) / float(logits.abs().max())
            # a bfloat16 run may pick the other of two near-equal logits; anything else is a fault
            assert dtype == "bfloat16" and margin < 2e-2, f"{what}: token {i} is {token}, the plain implementation says {want}"
        seq.append(token)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_engine(folders, name, dtype):
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    cfg, weights = tp.read_folder(folders[(name, dtype)])
    prompts = [tp.random_tokens(n, cfg["vocab"], seed=n) for n in (5, 9, 17, 30, 3, 12)]
    # a token budget below the longest prompt: prompts come in portions beside decoding requests; four at a time
    engine = LLMEngine(folders[(name, dtype)], dtype, max_num_seqs=4, max_model_len=96, max_num_batched_tokens=16,
                       num_gpu_blocks_override=20)
    outs = engine.generate(prompts, SamplingParams(max_tokens=12))
    for prompt, out in zip(prompts, outs):
        assert len(out) == 12
        greedy_agrees(cfg, weights, prompt, out, dtype, f"{name} {dtype}")


def test_command_lines(folders, tmp_path):
    """`bin/inferx-generate` and `bin/trace_run` choose the model class by config.json."""
    folder = folders[("P", "float32")]
    cfg, weights = tp.read_folder(folder)
    prompt = tp.random_tokens(7, cfg["vocab"], 4)
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
    import numpy as np
    want = pp.forward(cfg, weights, prompt)
    scale = float(want.abs().max())
    for step, rows in ((0, [0, 3]), (1, [6]), (2, [2])):
        got = torch.from_numpy(np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(len(rows), -1).copy())
        assert float((got.double() - want[rows]).abs().max()) <= ru.FP32_TOL * scale
