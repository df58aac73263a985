"""Models of the Dedelorn design in the engine against the plain implementation: whole prompts, prefill against
token-by-token decoding, portions down to two tokens, batches of unequal requests with pages and state slots
used again, long decoding past every window (replayed as graphs), greedy generation through the serving
engine and its scheduler, and the trace replay tool.  The configurations are the tests' own
(``dedelorn_models``)."""
import os

import numpy as np
import pytest
import torch

import dedelorn_models as models
import traces
from plain import dedelorn_plain as plain
from tolerances import BF16_REL_MEAN, BF16_REL_WORST, F32_TOL

pytestmark = pytest.mark.gpu

LENGTHS = {"all": [70, 41, 3, 55, 1, 26, 64], "latent": [45, 33, 2, 70, 17], "delta": [38, 9, 61, 1, 24]}
PAGE = {"all": 8, "latent": 4, "delta": 16}


def _setup(tmp_path, name, dtype, pages, max_live=4, seed=0):
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine
    folder = models.write_model(str(tmp_path / name), name, seed=seed,
                                dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, w = plain.load_folder(folder, torch.float64)
    engine = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=pages, kv_block_size=PAGE[name],
                                                               max_batch_requests=max_live, max_batch_tokens=4096,
                                                               max_seq_len=4096))
    return folder, cfg, w, engine


def _rows_within(worst_of_rows, mean_of_rows, scale, dtype, what):
    """float32: every row within rounding.  bfloat16: the mean within the bound, and at most one row in fifty beyond
    the bound of a row: with random weights a router's choice between two experts, or a sharp softmax, now and then
    lies within bfloat16 rounding, and such a row then differs by the size of an expert's output; a mechanism that
    is wrong moves every row."""
    worst_of_rows, mean = np.asarray(worst_of_rows), float(np.mean(mean_of_rows))
    if dtype == "float32":
        assert worst_of_rows.max() <= F32_TOL * max(1.0, scale), (what, float(worst_of_rows.max()), scale, int(worst_of_rows.argmax()))
        return
    over = int((worst_of_rows > BF16_REL_WORST * scale).sum())
    assert mean <= BF16_REL_MEAN * scale and over <= max(1, len(worst_of_rows) // 50), \
        (what, mean, scale, over, len(worst_of_rows), float(worst_of_rows.max()))


def _check(steps, out, ref, requests, dtype, what):
    """Every written row against the plain logits at (request, position); returns the rows compared."""
    fed, worst, mean, scale = {}, [], [], 0.0
    for st in steps:
        row = 0
        for e in st["entries"]:
            base = fed.get(e["id"], 0)
            for wpos in e["want"]:
                r = ref[e["id"]][base + wpos].numpy()
                d = np.abs(out[st["step"]][row] - r)
                worst.append(float(d.max()))
                mean.append(float(d.mean()))
                scale = max(scale, float(np.abs(r).max()))
                row += 1
            fed[e["id"]] = base + len(e["tokens"])
        for rid in st["end"]:
            fed.pop(rid, None)
    _rows_within(worst, mean, scale, dtype, what)
    return len(worst)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["all", "latent", "delta"])
def test_every_way_of_cutting_and_batching_gives_the_plain_logits(tmp_path, name, dtype):
    vocab = models.CONFIGS[name]["vocab"]
    requests = {f"r{i}": traces.random_tokens(vocab, n, seed=40 + i) for i, n in enumerate(LENGTHS[name])}
    ps = PAGE[name]
    # so few pages that the batches use them again: four live requests of the longest kind, and one page more
    pages = 4 * -(-max(LENGTHS[name]) // ps) + 1
    folder, cfg, w, engine = _setup(tmp_path, name, dtype, pages)
    ref = {rid: plain.forward(cfg, w, toks).float() for rid, toks in requests.items()}
    total = sum(len(t) for t in requests.values())
    takes = [g.pool.takes for g in engine.cache.groups]
    for what, steps in (("whole", traces.whole(requests)), ("decode", traces.last_decoded(requests, tail=30)),
                        ("portions", traces.portions(requests, seed=1)),
                        ("portions of two", traces.portions(requests, seed=2, sizes=(2, 2, 3, 2, 1, 2))),
                        ("mixed", traces.mixed(requests, max_live=4, seed=3)),
                        ("mixed, three live", traces.mixed(requests, max_live=3, seed=4, decode_tail=20, max_portion=9))):
        out = traces.run_in_process(engine, steps)
        assert _check(steps, out, ref, requests, dtype, what) == total
    for what, steps in (("last rows", traces.few_wanted(traces.mixed(requests, max_live=4, seed=5), seed=5)),
                        ("random rows", traces.random_wanted(traces.mixed(requests, max_live=4, seed=6), seed=6))):
        out = traces.run_in_process(engine, steps)
        _check(steps, out, ref, requests, dtype, what)
    engine.cache.check()
    assert not engine.cache.live
    for g, before in zip(engine.cache.groups, takes):
        assert g.pool.takes - before > g.pool.total              # pages went round
    assert engine.cache.slots.takes > 4 * 7                       # and so did the state slots


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_in_a_slot_that_another_left_starts_from_nothing(tmp_path, dtype):
    """One state slot and few pages: every request runs where the one before it ran, and must not see what it left."""
    name = "all"
    vocab = models.CONFIGS[name]["vocab"]
    requests = {f"s{i}": traces.random_tokens(vocab, n, seed=70 + i) for i, n in enumerate([30, 52, 7, 30])}
    folder, cfg, w, engine = _setup(tmp_path, name, dtype, pages=7, max_live=1)
    ref = {rid: plain.forward(cfg, w, toks).float() for rid, toks in requests.items()}
    for steps in (traces.whole(requests), traces.portions(requests, seed=7, sizes=(5, 1, 9, 2))):
        out = traces.run_in_process(engine, steps)
        _check(steps, out, ref, requests, dtype, "one slot")
    assert engine.cache.slots.total == 1 and engine.cache.slots.takes == 8


@pytest.mark.parametrize("name, dtype", [("all", "float32"), ("all", "bfloat16"), ("delta", "bfloat16"), ("latent", "bfloat16")])
def test_long_decoding_past_every_window_replays_graphs(tmp_path, name, dtype):
    """Two requests decode 150 tokens each, one step a token, far past the windows (9, 20 and 33 keys) and over many
    pages; the decode steps are recorded and replayed, and a state that a replay did not carry would show."""
    from zedinfer_amd.engine import StepEntry
    vocab = models.CONFIGS[name]["vocab"]
    a, b = traces.random_tokens(vocab, 160, seed=81), traces.random_tokens(vocab, 171, seed=82)
    folder, cfg, w, engine = _setup(tmp_path, name, dtype, pages=128)
    ref_a, ref_b = plain.forward(cfg, w, a).float(), plain.forward(cfg, w, b).float()
    sa, sb = engine.open("a"), engine.open("b")
    out = engine.step([StepEntry(sa, a[:10], [9]), StepEntry(sb, b[:21], [20])])
    worst, mean = [], []
    rows = [(out[0].cpu(), ref_a[9]), (out[1].cpu(), ref_b[20])]
    for i in range(150):
        out = engine.step([StepEntry(sa, [a[10 + i]], [0]), StepEntry(sb, [b[21 + i]], [0])]).cpu()
        rows += [(out[0], ref_a[10 + i]), (out[1], ref_b[21 + i])]
    for row, ref in rows:
        d = (row - ref).abs()
        worst.append(float(d.max()))
        mean.append(float(d.mean()))
    engine.close(sa)
    engine.close(sb)
    _rows_within(worst, mean, max(float(ref_a.abs().max()), float(ref_b.abs().max())), dtype, "long decoding")
    assert engine.graph_replays + engine.tape_runs > 100, (engine.graph_replays, engine.tape_runs)
    assert engine.graph_replays > 50


@pytest.mark.parametrize("name", ["all", "latent", "delta"])
def test_greedy_generation_through_the_serving_engine(tmp_path, name):
    """Several requests at once through InferenceEngine (its scheduler cuts the prompts into portions of 16 tokens and
    batches them beside decoding requests): in float32 the tokens are the plain implementation's."""
    from zedinfer_amd import GenerationConfig, InferenceEngine, SchedulerConfig
    folder = models.write_model(str(tmp_path / name), name, seed=9)
    cfg, w = plain.load_folder(folder, torch.float64)
    vocab = cfg["vocab"]
    prompts = [traces.random_tokens(vocab, n, seed=90 + n) for n in (37, 5, 21, 50)]
    want = [plain.greedy_generate(cfg, w, p, 12) for p in prompts]
    ie = InferenceEngine.create(folder, "float32", SchedulerConfig(num_kv_blocks=64, kv_block_size=PAGE[name],
                                                                   max_batch_requests=3, max_prefill_tokens=16))
    got = [r.output_ids for r in ie.generate(prompts, GenerationConfig(max_new_tokens=12, ignore_eos=True))]
    assert got == want
    alone = ie.generate_tokens(prompts[0], GenerationConfig(max_new_tokens=12, ignore_eos=True)).output_ids
    assert alone == want[0]


def test_the_replay_tool_runs_a_model_of_the_design(tmp_path):
    name = "all"
    folder = models.write_model(str(tmp_path / name), name, seed=3, dtype=torch.bfloat16)
    cfg, w = plain.load_folder(folder, torch.float64)
    requests = {f"q{i}": traces.random_tokens(cfg["vocab"], n, seed=20 + i) for i, n in enumerate([66, 19, 130, 4, 40])}
    ref = {rid: plain.forward(cfg, w, toks).float() for rid, toks in requests.items()}
    steps = traces.mixed(requests, max_live=4, seed=8)
    for dtype in ("float32", "bfloat16"):
        out = traces.run_tool(folder, dtype, steps, str(tmp_path / f"out_{dtype}"), traces.max_live_tokens(steps),
                              stderr_to=str(tmp_path / f"err_{dtype}.txt"))
        _check(steps, out, ref, requests, dtype, "tool")
        said = open(str(tmp_path / f"err_{dtype}.txt")).read()
        assert "4 live requests" in said


def test_command_lines_take_a_model_of_the_design(tmp_path):
    """random_model writes a folder from the design's config.json, ping generates from it what the plain implementation
    generates, batch_bench runs its scheduler over it with random weights."""
    import json
    import subprocess
    import sys
    ROOT = traces.ROOT
    env = dict(os.environ, PYTHONPATH=ROOT)
    run = lambda *a: subprocess.run([sys.executable, *a], capture_output=True, text=True, env=env, timeout=300,  # noqa: E731
                                    cwd=str(tmp_path))
    (tmp_path / "cfg").mkdir()
    with open(tmp_path / "cfg" / "config.json", "w") as f:
        json.dump(models.ALL, f)
    folder = str(tmp_path / "made")
    r = run(os.path.join(ROOT, "bin", "random_model"), str(tmp_path / "cfg"), folder, "--seed", "5", "--dtype", "float32",
            "--std", "0.1", "--noisy-norms")
    assert r.returncode == 0 and "Dedelorn" in r.stdout, r.stderr
    with open(os.path.join(folder, "config.json")) as f:
        assert json.load(f) == models.ALL
    cfg, w = plain.load_folder(folder, torch.float64)
    assert set(w) == set(models.tensor_shapes(models.ALL))
    prompt = traces.random_tokens(cfg["vocab"], 27, seed=3)
    r = run(os.path.join(ROOT, "bin", "ping"), folder, "--dtype", "fp32", "--prompt-ids", ",".join(map(str, prompt)),
            "--max-new-tokens", "6", "--ignore-eos", "--num-kv-blocks", "32", "--kv-block-size", "8", "--no-log-to-console")
    assert r.returncode == 0, r.stderr
    want = plain.greedy_generate(cfg, w, prompt, 6)
    assert "output_ids: " + ",".join(map(str, want)) in r.stdout, r.stdout
    r = run(os.path.join(ROOT, "bin", "batch_bench"), str(tmp_path / "cfg"), "-b", "3", "-p", "20", "-d", "6", "--num-kv-blocks",
            "64", "--kv-block-size", "8", "--random-weights", "--seed", "4", "--no-log-to-console")
    assert r.returncode == 0 and "18 tokens generated" in r.stdout, r.stderr + r.stdout


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Twelve models whose sizes, layer order, windows, shared caches and constants are drawn at random, each in both
    engine types, over a batch of unequal requests with pages and slots used again and over whole prompts."""
    import json
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine
    from zedinfer_amd.weights.safetensors_io import write_safetensors
    cfg = models.random_config(seed)
    requests = {f"z{i}": traces.random_tokens(cfg["vocab"], n, seed=seed * 10 + i) for i, n in enumerate([83, 5, 140, 31, 1, 66])}
    for dtype in ("float32", "bfloat16"):
        folder = str(tmp_path / dtype)
        os.makedirs(folder)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(cfg, f)
        write_safetensors(os.path.join(folder, "model.safetensors"),
                          models.make_weights(cfg, seed, torch.float32 if dtype == "float32" else torch.bfloat16), metadata={"format": "pt"})
        pcfg, w = plain.load_folder(folder, torch.float64)
        ref = {rid: plain.forward(pcfg, w, toks).float() for rid, toks in requests.items()}
        ps = [4, 8, 16, 32][seed % 4]
        engine = Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=3 * -(-140 // ps) + 6, kv_block_size=ps,
                                                                   max_batch_requests=3, max_batch_tokens=4096, max_seq_len=4096))
        for what, steps in (("mixed", traces.mixed(requests, max_live=3, seed=seed, decode_tail=25, max_portion=40)),
                            ("whole", traces.whole(requests))):
            out = traces.run_in_process(engine, steps)
            _check(steps, out, ref, requests, dtype, (what, seed, json.dumps(cfg)))
