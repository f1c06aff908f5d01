"""The Gimozen design through the framework: replayed traces (whole prompts, decoding, portions, mixed batches with pages
and slots used again) against the plain implementation, generation through the entry point and the scheduler, and weights
made so that a far key, a sink or the edge of a page shows in the logits."""

import copy
import json

import numpy as np
import pytest

import plain_gimozen as plain
import plain_gpt2
import replay
from conftest import random_tokens
from gimozen_cases import CASES, attention_layer, latent_layer, model

pytestmark = pytest.mark.gpu


def sharpen(config, weights, factor=4.0):
    """Random projections give nearly uniform softmaxes, under which a wrong key or page hardly moves a logit: the query
    matrices are scaled up so that attention weights differ by orders of magnitude."""
    for index, layer in enumerate(config["layers"]):
        weights[f"l{index}.mix.q"] = plain_gpt2.round_to_bf16(weights[f"l{index}.mix.q"] * factor)
        if layer["type"] == "attention":   # normed heads undo a scaled matrix: scale the gain instead
            weights[f"l{index}.mix.q.norm"] = plain_gpt2.round_to_bf16(weights[f"l{index}.mix.q.norm"] * factor)
    return weights


@pytest.fixture(scope="module")
def gimozen_dirs(tmp_path_factory):
    out = {}
    for seed, (name, config) in enumerate(CASES.items()):
        weights = sharpen(config, plain.random_weights(config, 20 + seed))
        folder = plain.write_model_dir(tmp_path_factory.mktemp(f"gimozen_{name}"), config, weights)
        out[name] = (folder, copy.deepcopy(config), weights)
    return out


def requests_for(config, lengths, seed=300):
    return {f"r{i}": random_tokens(seed + i, n, config["vocab"]) for i, n in enumerate(lengths)}


def plain_logits(config, weights, requests, bf16):
    stored = plain_gpt2.stored_as_bf16 if bf16 else plain._keep
    return {name: plain.forward(config, weights, tokens, stored=stored) for name, tokens in requests.items()}


LENGTHS = {"mixed": [5, 130, 64, 65, 1, 200, 33], "attention": [2, 70, 129, 63, 40], "latent": [3, 300, 64, 17, 128, 66], "odd": [67, 2, 130, 31]}
MODES = {"whole": replay.whole, "tail": replay.prefill_then_decode, "chunked": replay.chunked, "mixed": replay.mixed}
# 32-bit: sums in another order than numpy's
TOLERANCE = {"float32": dict(atol=5e-5, rtol=5e-5)}


def check(got, config, weights, requests, dtype):
    """32-bit: every logit within the tolerance. bfloat16: the engine rounds at other places than the plain implementation
    does when it rounds what a bfloat16 run stores (it keeps folded queries, summed latents and the sublayers' outputs in
    32-bit), so the two are not compared with each other: the engine may lie as far from exact arithmetic as the plain
    bfloat16 run does, twice that at the worst logit of a request and one and a half times in the root mean square. A wrong
    key, page or slot moves logits by tens of times that."""
    exact = plain_logits(config, weights, requests, False)
    if dtype == "float32":
        return replay.compare(got, exact, **TOLERANCE[dtype])
    rounded = plain_logits(config, weights, requests, True)
    for name, rows in exact.items():
        assert set(got[name]) == set(range(len(rows))), name
        noise = np.abs(rounded[name] - rows)
        error = np.abs(np.stack([got[name][p] for p in range(len(rows))]).astype(np.float64) - rows)
        worst = int(error.max(axis=1).argmax())
        assert error.max() <= 2.0 * noise.max() + 2e-3, f"request {name!r} position {worst}: error {error.max():.3e}, rounding noise {noise.max():.3e}"
        assert np.sqrt((error ** 2).mean()) <= 1.5 * np.sqrt((noise ** 2).mean()) + 1e-3, f"request {name!r}: rms error against rms noise"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", list(CASES))
def test_replay_matches_plain(gimozen_dirs, tmp_path, name, mode, dtype):
    folder, config, weights = gimozen_dirs[name]
    requests = requests_for(config, LENGTHS[name])
    collector = MODES[mode](requests)
    for page_size in ((None, 16) if mode == "mixed" and dtype == "float32" else (None,)):
        # exactly the pages that are needed: they and the slots are used again (16: many pages a request, borders everywhere)
        outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / f"out{page_size}", replay.peak_tokens(collector, page_size or 64), page_size=page_size)
        check(collector.gather(outputs), config, weights, requests, dtype)


def test_replay_hands_out_the_stream_after_every_layer(gimozen_dirs, tmp_path):
    folder, config, weights = gimozen_dirs["mixed"]
    requests = requests_for(config, [40, 9])
    collector = replay.chunked(requests, sizes=(7, 2, 16))
    replay.run_trace(folder, "float32", collector.steps, tmp_path / "out", replay.peak_tokens(collector), hidden_out=tmp_path / "hidden")
    layers = {name: [] for name in requests}
    for name, tokens in requests.items():
        plain.forward(config, weights, tokens, layer_outputs=layers[name])
    fed = {}
    for step in collector.steps:
        for e in step["entries"]:   # one request a step
            start, n = fed.get(e["id"], 0), len(e["tokens"])
            for index in range(len(config["layers"])):
                rows = np.fromfile(tmp_path / "hidden" / f"{step['step']}.{index}.f32", dtype="<f4").reshape(n, config["width"])
                np.testing.assert_allclose(rows, layers[e["id"]][index][start : start + n], atol=2e-5, rtol=2e-5, err_msg=f"step {step['step']} layer {index}")
            fed[e["id"]] = start + n


def hot_key_model(kind):
    """One layer whose attention is all that tells a logit from another: the value path carries the token, the query is
    made to look for one cached token, and the feed-forward is left out."""
    layer = attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, ff=None, coef=0.0) if kind == "attention" else latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, ff=None)
    return model([layer], width=32, vocab=50, scale=1.0, alpha=0.05)


@pytest.mark.parametrize("kind", ["attention", "latent"])
def test_a_far_key_at_the_edges_of_pages_is_found_in_prompts_and_in_decoding(tmp_path, kind):
    # Token 7 appears once, far back, at a page's first or last place; every other token is drawn from 10..49. The layer has
    # no feed-forward and a weak residual, and its queries are scaled up, so that what the attention finds is what the logits
    # are made of: the logits behind token 7's place move, by far more than the 32-bit tolerance, when it is taken away, and
    # token-by-token decoding, portions and whole prompts all agree with the plain implementation on them.
    config = hot_key_model(kind)
    weights = sharpen(config, plain.random_weights(config, 77), 6.0)
    rng = np.random.default_rng(3)
    folder = plain.write_model_dir(tmp_path / "model", config, weights)
    requests = {}
    for at in (0, 63, 64, 127, 128, 190):
        tokens = rng.integers(10, 50, size=200).tolist()
        tokens[at] = 7
        requests[f"hot{at}"] = tokens
    for dtype in ("float32", "bfloat16"):
        for mode in ("whole", "tail", "chunked"):
            collector = MODES[mode](requests)
            outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / f"{dtype}{mode}", replay.peak_tokens(collector))
            check(collector.gather(outputs), config, weights, requests, dtype)
    # the key matters: without token 7 the logits behind its place move by far more than any tolerance
    for at in (0, 64):
        without = list(requests[f"hot{at}"])
        without[at] = 11
        moved = np.abs(plain.forward(config, weights, without)[at + 1 :] - plain.forward(config, weights, requests[f"hot{at}"])[at + 1 :]).max()
        assert moved > 100 * TOLERANCE["float32"]["atol"], (kind, at, moved)


def test_the_sink_takes_its_share(tmp_path):
    # with every score far below the sink the heads' outputs vanish; with the sink far below every score it changes nothing
    config = model([latent_layer(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=16, ff=None)], width=32, vocab=40, alpha=0.1)
    base = plain.random_weights(config, 5)
    requests = requests_for(config, [20, 3])
    logits = {}
    for name, sink in (("high", 30.0), ("low", -30.0), ("mid", 0.5)):
        weights = dict(base)
        weights["l0.mix.sink"] = np.full(2, sink, dtype=np.float32)
        folder = plain.write_model_dir(tmp_path / name, config, weights)
        collector = replay.whole(requests)
        got = collector.gather(replay.run_trace(folder, "float32", collector.steps, tmp_path / f"out_{name}", 128))
        check(got, config, weights, requests, "float32")
        logits[name] = got
    assert np.abs(logits["high"]["r0"][19] - logits["low"]["r0"][19]).max() > 1e-2
    assert np.abs(logits["mid"]["r0"][19] - logits["low"]["r0"][19]).max() > 1e-3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_through_the_engine_and_its_scheduler(gimozen_dirs, dtype):
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = gimozen_dirs["mixed"]
    prompts = [random_tokens(9, 5, config["vocab"]), random_tokens(10, 70, config["vocab"]), [3], random_tokens(11, 31, config["vocab"])]
    # few pages: four requests of up to 70 + 24 tokens do not all fit at once, so pages are given back and used again
    with Engine(folder, EngineOptions(dtype=dtype, max_sessions=4, max_length=256, max_tokens=256)) as engine:
        generated = engine.generate(prompts, max_new_tokens=24)
        with engine.open_session() as session:
            first = session.prefill(prompts[1])
    stored = plain_gpt2.stored_as_bf16 if dtype == "bfloat16" else plain._keep
    for prompt, new in zip(prompts, generated):
        assert len(new) == 24
        logits = plain.forward(config, weights, list(prompt) + list(new), stored=stored)
        for k, token in enumerate(new):   # greedy: the plain implementation's own choice, unless the two lie within rounding
            row = logits[len(prompt) - 1 + k]
            assert row[token] >= row.max() - (1e-4 if dtype == "float32" else 0.15), (prompt[:3], k, token, int(row.argmax()))
    want = plain.forward(config, weights, prompts[1])[-1]
    np.testing.assert_allclose(first, want, atol=5e-5 if dtype == "float32" else 0.2, rtol=5e-5 if dtype == "float32" else 0.05)


def test_the_command_line_completes_greedily(gimozen_dirs):
    import subprocess
    import sys

    folder, config, weights = gimozen_dirs["attention"]
    prompt = random_tokens(12, 9, config["vocab"])
    done = subprocess.run([sys.executable, str(replay.ROOT / "bin" / "complete"), "--model", str(folder), "--dtype", "float32", "--temperature", "0",
                           "--max-new-tokens", "12", "--max-length", "128", "--tokens", ",".join(map(str, prompt))], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    new = [int(t) for t in done.stdout.strip().split(",")]
    logits = plain.forward(config, weights, prompt + new)
    assert len(new) == 12
    for k, token in enumerate(new):
        row = logits[len(prompt) - 1 + k]
        assert row[token] >= row.max() - 1e-4, (k, token, int(row.argmax()))


def test_long_decoding_crosses_pages_and_key_runs(gimozen_dirs):
    # 700 decoded tokens, one by one, from captured steps: past ten pages and past the lengths at which the latent
    # attention cuts a row's keys into runs
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = gimozen_dirs["latent"]
    prompt = random_tokens(4, 3, config["vocab"])
    with Engine(folder, EngineOptions(dtype="float32", max_sessions=2, max_length=768, max_tokens=1536)) as engine:
        new = engine.generate([prompt], max_new_tokens=700)[0]
    logits = plain.forward(config, weights, prompt + new)
    wrong = [k for k, token in enumerate(new) if logits[len(prompt) - 1 + k][token] < logits[len(prompt) - 1 + k].max() - 1e-4]
    assert not wrong, wrong[:5]


def test_config_json_round_trip_and_random_weights(tmp_path):
    from mini_llm_amd.config import config_from_dict
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.weights import write_model_dir

    config = config_from_dict(CASES["mixed"])
    folder = write_model_dir(config, 3, tmp_path / "random")
    assert json.loads((folder / "config.json").read_text())["layers"][2]["mixer"]["kv_from"] == 0
    plain_config, weights = plain.load_model_dir(folder)
    with Engine(folder, EngineOptions(dtype="float32", max_sessions=2, max_length=64)) as engine:
        got = engine.forward_last([1, 2, 3, 4, 5])
    np.testing.assert_allclose(got, plain.forward(plain_config, weights, [1, 2, 3, 4, 5])[-1], atol=1e-4, rtol=1e-4)
