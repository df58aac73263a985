"""Models of the Tosisun design in the engine against the plain implementation: whole prompts, prefill against
token-by-token decoding, portions down to two tokens (shorter than the convolution's tail), batches of unequal
requests with pages and state slots used again, long decoding (replayed as graphs), a key far back that carries
the weight, sinks that take it, greedy generation through the serving engine and its scheduler, the trace replay
tool and the command lines.  The configurations are the tests' own (``tosisun_models``)."""
import json
import os

import numpy as np
import pytest
import torch

import tosisun_models as models
import traces
from plain import tosisun_plain as plain
from tolerances import BF16_REL_MEAN, BF16_REL_WORST, F32_TOL

pytestmark = pytest.mark.gpu

LENGTHS = {"main": [70, 41, 3, 55, 1, 26, 64], "odd": [45, 33, 2, 70, 17], "wide": [38, 9, 61, 1, 24]}
PAGE = {"main": 8, "odd": 4, "wide": 16}


def _engine(folder, dtype, pages, page, max_live=4):
    from zedinfer_amd.config import SchedulerConfig
    from zedinfer_amd.engine import Engine
    return Engine.from_folder(folder, dtype, SchedulerConfig(num_kv_blocks=pages, kv_block_size=page,
                                                             max_batch_requests=max_live, max_batch_tokens=4096,
                                                             max_seq_len=4096))


def _setup(tmp_path, name, dtype, pages, max_live=4, seed=0):
    folder = models.write_model(str(tmp_path / name), name, seed=seed,
                                dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    cfg, w = plain.load_folder(folder, torch.float64)
    return folder, cfg, w, _engine(folder, dtype, pages, PAGE[name], max_live)


def _rows_within(worst_of_rows, mean_of_rows, scale, dtype, what):
    """float32: every row within rounding.  bfloat16: the mean within the bound, and at most one row in fifty beyond
    the bound of a row: with random weights a router's choice between two experts now and then lies within bfloat16
    rounding, and such a row then differs by the size of an expert's output; a mechanism that is wrong moves every
    row."""
    worst_of_rows, mean = np.asarray(worst_of_rows), float(np.mean(mean_of_rows))
    if dtype == "float32":
        assert worst_of_rows.max() <= F32_TOL * max(1.0, scale), (what, float(worst_of_rows.max()), scale, int(worst_of_rows.argmax()))
        return
    over = int((worst_of_rows > BF16_REL_WORST * scale).sum())
    assert mean <= BF16_REL_MEAN * scale and over <= max(1, len(worst_of_rows) // 50), \
        (what, mean, scale, over, len(worst_of_rows), float(worst_of_rows.max()))


CLOSE_CALL = 0.05      # a router's choice whose margin is below this can turn under bfloat16 rounding


def _reference(cfg, w, requests):
    """The plain logits of every request, and for every position the least margin of its routers' choices."""
    ref, margin = {}, {}
    for rid, toks in requests.items():
        ms = []
        ref[rid] = plain.forward(cfg, w, toks, margins=ms).float()
        margin[rid] = torch.stack(ms).min(0).values.numpy() if ms else np.full(len(toks), np.inf)
    return ref, margin


def _check(steps, out, ref, dtype, what, margin=None):
    """Every written row against the plain logits at (request, position); returns the rows compared.  With
    ``margin``, in bfloat16, the rows of positions where a router's choice is a close call in the plain model are
    left out of the count of rows beyond the bound (the other expert's output is no rounding error, and no fault);
    they must stay few, and they stay in the mean."""
    fed, worst, mean, scale, close = {}, [], [], 0.0, 0
    for st in steps:
        row = 0
        for e in st["entries"]:
            base = fed.get(e["id"], 0)
            for wpos in e["want"]:
                r = ref[e["id"]][base + wpos].numpy()
                d = np.abs(out[st["step"]][row] - r)
                row += 1
                scale = max(scale, float(np.abs(r).max()))
                mean.append(float(d.mean()))
                if margin is not None and dtype != "float32" and margin[e["id"]][base + wpos] < CLOSE_CALL:
                    close += 1
                    continue
                worst.append(float(d.max()))
            fed[e["id"]] = base + len(e["tokens"])
        for rid in st["end"]:
            fed.pop(rid, None)
    assert close <= 0.6 * len(mean), (what, close, len(mean))
    _rows_within(worst, mean, scale, dtype, what)
    return len(mean)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["main", "odd", "wide"])
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
        assert _check(steps, out, ref, dtype, what) == total
    for what, steps in (("last rows", traces.few_wanted(traces.mixed(requests, max_live=4, seed=5), seed=5)),
                        ("random rows", traces.random_wanted(traces.mixed(requests, max_live=4, seed=6), seed=6))):
        out = traces.run_in_process(engine, steps)
        _check(steps, out, ref, dtype, what)
    engine.cache.check()
    assert not engine.cache.live
    for g, before in zip(engine.cache.groups, takes):
        assert g.pool.takes - before > g.pool.total              # pages went round
    assert engine.cache.slots.takes > 4 * 7                       # and so did the state slots


def test_in_float32_every_cut_gives_the_same_bits(tmp_path):
    """The sums of a position do not depend on the cut, the batch or the pages: in float32 the logits of whole
    prompts, of portions and of a mixed batch agree to the last bit."""
    name = "main"
    vocab = models.CONFIGS[name]["vocab"]
    requests = {f"b{i}": traces.random_tokens(vocab, n, seed=140 + i) for i, n in enumerate([33, 150, 6])}
    folder, cfg, w, engine = _setup(tmp_path, name, "float32", pages=64)
    rows = {}
    for what, steps in (("whole", traces.whole(requests)), ("portions", traces.portions(requests, seed=3, sizes=(2, 5, 1, 7))),
                        ("mixed", traces.mixed(requests, max_live=3, seed=9))):
        out = traces.run_in_process(engine, steps)
        fed = {}
        for st in steps:
            row = 0
            for e in st["entries"]:
                base = fed.get(e["id"], 0)
                for wpos in e["want"]:
                    rows.setdefault((e["id"], base + wpos), []).append(out[st["step"]][row].copy())
                    row += 1
                fed[e["id"]] = base + len(e["tokens"])
    assert len(rows) == 33 + 150 + 6
    for key, got in rows.items():
        assert len(got) == 3 and np.array_equal(got[0], got[1]) and np.array_equal(got[0], got[2]), key


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_in_a_slot_that_another_left_starts_from_nothing(tmp_path, dtype):
    """One state slot and few pages: every request runs where the one before it ran, and must not see what it left
    (the convolution's tail of the request before would show in the first tokens)."""
    name = "main"
    vocab = models.CONFIGS[name]["vocab"]
    requests = {f"s{i}": traces.random_tokens(vocab, n, seed=70 + i) for i, n in enumerate([30, 52, 7, 30])}
    folder, cfg, w, engine = _setup(tmp_path, name, dtype, pages=7, max_live=1)
    ref = {rid: plain.forward(cfg, w, toks).float() for rid, toks in requests.items()}
    for steps in (traces.whole(requests), traces.portions(requests, seed=7, sizes=(5, 1, 9, 2))):
        out = traces.run_in_process(engine, steps)
        _check(steps, out, ref, dtype, "one slot")
    assert engine.cache.slots.total == 1 and engine.cache.slots.takes == 8


@pytest.mark.parametrize("name, dtype", [("main", "float32"), ("main", "bfloat16"), ("wide", "bfloat16")])
def test_long_decoding_replays_graphs(tmp_path, name, dtype):
    """Two requests decode 300 tokens each, one step a token, over many pages and past the first chunk of keys of
    the decode kernel; the decode steps are recorded and replayed, and a tail that a replay did not carry would show."""
    from zedinfer_amd.engine import StepEntry
    vocab = models.CONFIGS[name]["vocab"]
    a, b = traces.random_tokens(vocab, 310, seed=81), traces.random_tokens(vocab, 321, seed=82)
    folder, cfg, w, engine = _setup(tmp_path, name, dtype, pages=128)
    ref_a, ref_b = plain.forward(cfg, w, a).float(), plain.forward(cfg, w, b).float()
    sa, sb = engine.open("a"), engine.open("b")
    out = engine.step([StepEntry(sa, a[:10], [9]), StepEntry(sb, b[:21], [20])])
    worst, mean = [], []
    rows = [(out[0].cpu(), ref_a[9]), (out[1].cpu(), ref_b[20])]
    for i in range(300):
        out = engine.step([StepEntry(sa, [a[10 + i]], [0]), StepEntry(sb, [b[21 + i]], [0])]).cpu()
        rows += [(out[0], ref_a[10 + i]), (out[1], ref_b[21 + i])]
    for row, ref in rows:
        d = (row - ref).abs()
        worst.append(float(d.max()))
        mean.append(float(d.mean()))
    engine.close(sa)
    engine.close(sb)
    _rows_within(worst, mean, max(float(ref_a.abs().max()), float(ref_b.abs().max())), dtype, "long decoding")
    assert engine.graph_replays + engine.tape_runs > 200, (engine.graph_replays, engine.tape_runs)
    assert engine.graph_replays > 100


# one attention layer whose softmax is as sharp as the test makes it, and a head that reads the values out
SHARP = dict(
    architecture="Tosisun", width=64, vocab=128, norm=dict(eps=1e-5),
    layers=[dict(type="attention",
                 mixer=dict(heads=2, kv_heads=1, dim=32, vdim=32, conv=1, scale=1.0, rot=dict(base=10000.0, dims=0)),
                 mlp=None)])


def _sharp_weights(sink):
    """Token 5 is the only one whose key points where every query points (a score of 40 against 0), and its value
    is the only one that the output projection lets through on channel 0."""
    cfg = SHARP
    w = {k: torch.zeros_like(v) for k, v in models.make_weights(cfg, 0).items()}
    W, V = cfg["width"], cfg["vocab"]
    g = torch.Generator().manual_seed(3)
    w["embed"] = 0.3 * torch.randn(V, W, generator=g)
    w["embed"][:, 0] = 0.0
    w["embed"][5, 0] = 6.0                                    # the mark of the far token
    for n in ("l0.norm1", "l0.norm2", "final.norm"):
        w[n] = torch.ones(W)
    w["l0.mix.q.conv"], w["l0.mix.k.conv"], w["l0.mix.v.conv"] = torch.ones(64, 1), torch.ones(32, 1), torch.ones(32, 1)
    w["l0.mix.q.norm"], w["l0.mix.k.norm"] = torch.ones(64), torch.ones(32)
    w["l0.mix.q.b"][0], w["l0.mix.q.b"][32] = 1.0, 1.0        # after the norm over 64 channels: sqrt(32) on dim 0 of each head
    w["l0.mix.k"][0, 0] = 1.0                                 # the key's dim 0 is the mark; the norm over 32 channels makes it sqrt(32)
    w["l0.mix.k.b"][1] = 1e-3                                 # other tokens' keys lie on dim 1, which no query has
    w["l0.mix.v"][0, 0] = 1.0
    w["l0.mix.v.b"][1] = 1.0                                  # every value has 1 on dim 1
    w["l0.mix.o"][0, 0], w["l0.mix.o"][1, 1] = 1.0, 1.0       # head 0's dims 0 and 1 go to channels 0 and 1
    w["l0.mix.o"][2, 33] = 1.0                                # head 1 (no sink to speak of) gives the measure: the norm
                                                              # on the mixer's output would hide a common factor
    w["l0.mix.sink"] = torch.tensor([float(sink), 0.0])
    w["head"] = 0.2 * torch.randn(V, W, generator=g)
    return w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sink", [-30.0, 28.0, 36.0])
def test_a_key_far_back_among_hundreds_and_a_sink_that_takes_its_weight(tmp_path, dtype, sink):
    """The marked token stands at position 2 of 700; the last tokens, in the prompt and decoded, must find it (score
    32 against about 0 for 700 others), and a sink of about that size must take its share: the three sinks give
    three different outputs, each the plain one."""
    from zedinfer_amd.engine import StepEntry
    cfg = SHARP
    toks = [t if t != 5 else 6 for t in traces.random_tokens(cfg["vocab"], 700, seed=11)]
    toks[2] = 5
    w = _sharp_weights(sink)
    folder = models.write_config(str(tmp_path / "sharp"), cfg,
                                 {k: v.to(torch.float32 if dtype == "float32" else torch.bfloat16) for k, v in w.items()})
    pcfg, pw = plain.load_folder(folder, torch.float64)
    ref, layers = plain.forward(pcfg, pw, toks, return_layers=True)
    # the plain model does find the token: channel 0 of the mixer's output follows the far value or the sink
    engine = _engine(folder, dtype, pages=64, page=16)
    seq = engine.open("x")
    want_rows = [400, 650, 689]
    out = [engine.step([StepEntry(seq, toks[:690], want_rows)]).cpu()]
    for t in range(690, 700):
        out.append(engine.step([StepEntry(seq, [toks[t]], [0])]).cpu())
    engine.close(seq)
    got = torch.cat(out)
    rows = want_rows + list(range(690, 700))
    err = (got.double() - ref[rows]).abs()
    scale = float(ref.abs().max())
    if dtype == "float32":
        assert float(err.max()) <= F32_TOL * max(1.0, scale)
    else:
        assert float(err.max()) <= BF16_REL_WORST * scale and float(err.mean()) <= BF16_REL_MEAN * scale
    # and the result does depend on the far token and on the sink
    other = list(toks)
    other[2] = 6
    assert float((plain.forward(pcfg, pw, other)[rows] - ref[rows]).abs().max()) > (0.05 if sink > 35 else 0.1) * scale
    if sink > 0:
        no_sink = {k: v.double() for k, v in _sharp_weights(-30.0).items()}
        assert float((plain.forward(pcfg, no_sink, toks)[rows] - ref[rows]).abs().max()) > (0.1 if sink > 35 else 0.002) * scale


@pytest.mark.parametrize("name", ["main", "odd"])
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
    name = "main"
    folder = models.write_model(str(tmp_path / name), name, seed=3, dtype=torch.bfloat16)
    cfg, w = plain.load_folder(folder, torch.float64)
    requests = {f"q{i}": traces.random_tokens(cfg["vocab"], n, seed=20 + i) for i, n in enumerate([66, 19, 130, 4, 40])}
    ref = {rid: plain.forward(cfg, w, toks).float() for rid, toks in requests.items()}
    steps = traces.mixed(requests, max_live=4, seed=8)
    for dtype in ("float32", "bfloat16"):
        out = traces.run_tool(folder, dtype, steps, str(tmp_path / f"out_{dtype}"), traces.max_live_tokens(steps),
                              stderr_to=str(tmp_path / f"err_{dtype}.txt"))
        _check(steps, out, ref, dtype, "tool")
        said = open(str(tmp_path / f"err_{dtype}.txt")).read()
        assert "4 live requests" in said


def test_command_lines_take_a_model_of_the_design(tmp_path):
    """random_model writes a folder from the design's config.json, ping generates from it what the plain implementation
    generates, batch_bench runs its scheduler over it with random weights."""
    import subprocess
    import sys
    ROOT = traces.ROOT
    env = dict(os.environ, PYTHONPATH=ROOT)
    run = lambda *a: subprocess.run([sys.executable, *a], capture_output=True, text=True, env=env, timeout=300,  # noqa: E731
                                    cwd=str(tmp_path))
    (tmp_path / "cfg").mkdir()
    with open(tmp_path / "cfg" / "config.json", "w") as f:
        json.dump(models.MAIN, f)
    folder = str(tmp_path / "made")
    r = run(os.path.join(ROOT, "bin", "random_model"), str(tmp_path / "cfg"), folder, "--seed", "5", "--dtype", "float32",
            "--std", "0.1", "--noisy-norms")
    assert r.returncode == 0 and "Tosisun" in r.stdout, r.stderr
    with open(os.path.join(folder, "config.json")) as f:
        assert json.load(f) == models.MAIN
    cfg, w = plain.load_folder(folder, torch.float64)
    assert set(w) == set(models.tensor_shapes(models.MAIN))
    prompt = traces.random_tokens(cfg["vocab"], 27, seed=3)
    r = run(os.path.join(ROOT, "bin", "ping"), folder, "--dtype", "fp32", "--prompt-ids", ",".join(map(str, prompt)),
            "--max-new-tokens", "6", "--ignore-eos", "--num-kv-blocks", "32", "--kv-block-size", "8", "--no-log-to-console")
    assert r.returncode == 0, r.stderr
    want = plain.greedy_generate(cfg, w, prompt, 6)
    assert "output_ids: " + ",".join(map(str, want)) in r.stdout, r.stdout
    r = run(os.path.join(ROOT, "bin", "batch_bench"), str(tmp_path / "cfg"), "-b", "3", "-p", "20", "-d", "6", "--num-kv-blocks",
            "64", "--kv-block-size", "8", "--random-weights", "--seed", "4", "--no-log-to-console")
    assert r.returncode == 0 and "18 tokens generated" in r.stdout, r.stderr + r.stdout


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Ten models whose sizes, layer order, shared weights and constants are drawn at random, each in both engine
    types, over a batch of unequal requests with pages and slots used again and over whole prompts."""
    cfg = models.random_config(seed)
    requests = {f"z{i}": traces.random_tokens(cfg["vocab"], n, seed=seed * 10 + i) for i, n in enumerate([83, 5, 140, 31, 1, 66])}
    for dtype in ("float32", "bfloat16"):
        folder = models.write_config(str(tmp_path / dtype), cfg,
                                     models.make_weights(cfg, seed, torch.float32 if dtype == "float32" else torch.bfloat16))
        pcfg, w = plain.load_folder(folder, torch.float64)
        ref, margin = _reference(pcfg, w, requests)
        ps = [4, 8, 16, 32][seed % 4]
        engine = _engine(folder, dtype, 3 * -(-140 // ps) + 6, ps, max_live=3)
        for what, steps in (("mixed", traces.mixed(requests, max_live=3, seed=seed, decode_tail=25, max_portion=40)),
                            ("whole", traces.whole(requests))):
            out = traces.run_in_process(engine, steps)
            _check(steps, out, ref, dtype, (what, seed, json.dumps(cfg)), margin)
