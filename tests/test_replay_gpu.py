"""Trace replay against the plain implementation: whole, last 32 decoded, changing portions, mixed with page reuse."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

from helpers import PAGE, check, model_folder, reference_logits

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
LENGTHS = {"a": 100, "b": 180, "c": 150}


def runner(name, dtype, max_tokens):
    from prelude_amd.trace import TraceRunner
    folder, _, _ = model_folder(name)
    return TraceRunner(folder, dtype, max_tokens, page_size=PAGE[name])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_sequence(gpu, name, dtype):
    toks, ref = reference_logits(name, 0, LENGTHS[name])
    r = runner(name, dtype, 256)
    got = r.step([{"id": "x", "tokens": toks, "want": list(range(len(toks)))}], ["x"])
    check(got, ref, dtype, f"{name} whole")
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_last_32_tokens_one_by_one(gpu, name, dtype):
    toks, ref = reference_logits(name, 1, LENGTHS[name])
    n = len(toks) - 32
    r = runner(name, dtype, 256)
    outs = [r.step([{"id": 0, "tokens": toks[:n], "want": list(range(n))}])]
    for i in range(n, len(toks)):
        outs.append(r.step([{"id": 0, "tokens": [toks[i]], "want": [0]}]))
    check(np.concatenate(outs), ref, dtype, f"{name} prefill + 32 decode")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_portions_of_changing_size(gpu, name, dtype):
    toks, ref = reference_logits(name, 2, LENGTHS[name])
    sizes = [7, 2, 13, 2, 1, 31, 2, 9, 16, 3, 8, 2]
    r = runner(name, dtype, 256)
    outs, i, k = [], 0, 0
    while i < len(toks):
        n = min(sizes[k % len(sizes)], len(toks) - i)
        k += 1
        outs.append(r.step([{"id": "p", "tokens": toks[i:i + n], "want": list(range(n))}]))
        i += n
    check(np.concatenate(outs), ref, dtype, f"{name} portions")


def mixed_trace(name, lengths, max_live=4, seed=0):
    """Steps over several requests: up to max_live at a time, portions of some beside single
    tokens of others, some left out of a step; a request ends as soon as it is fed."""
    rng = np.random.default_rng(seed)
    seqs = [reference_logits(name, 10 + i, n) for i, n in enumerate(lengths)]
    fed = [0] * len(seqs)
    waiting = list(range(len(seqs)))
    live, steps = [], []
    mode = {}
    while waiting or live:
        while waiting and len(live) < max_live:
            r = waiting.pop(0)
            live.append(r)
            mode[r] = "portion"
        entries, end = [], []
        for r in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                           # left out of this step
            left = len(seqs[r][0]) - fed[r]
            if mode[r] == "portion":
                n = int(min(left, rng.choice([2, 3, 5, 11, 17, 40])))
                if fed[r] + n >= len(seqs[r][0]) * 0.6:
                    mode[r] = "decode"
            else:
                n = 1
            entries.append({"id": f"r{r}", "tokens": seqs[r][0][fed[r]:fed[r] + n], "want": list(range(n)),
                            "_r": r, "_at": fed[r]})
            fed[r] += n
            if fed[r] == len(seqs[r][0]):
                end.append(f"r{r}")
                live.remove(r)
        if entries:
            steps.append((entries, end))
    return seqs, steps


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_mixed_batches_with_page_reuse(gpu, name, dtype):
    lengths = {"a": [70, 45, 100, 33, 64, 90, 20, 128, 77, 50, 110, 60],
               "b": [130, 60, 200, 31, 90, 150, 64, 256, 100, 40, 180, 75],
               "c": [120, 40, 300, 64, 90, 200, 33, 500, 150, 260, 70, 400]}[name]
    seqs, steps = mixed_trace(name, lengths, seed=3)
    # the pool holds the four largest requests, each rounded up to 64: later requests get used pages
    pool = sum(sorted(-(-n // 64) * 64 for n in lengths)[-4:])
    r = runner(name, dtype, pool)
    pages_seen = set()
    reused = False
    got = [np.zeros((len(s[0]), s[1].shape[1])) for s in seqs]
    for entries, end in steps:
        out = r.step([{k: v for k, v in e.items() if not k.startswith("_")} for e in entries], [])
        row = 0
        for e in entries:
            n = len(e["tokens"])
            got[e["_r"]][e["_at"]:e["_at"] + n] = out[row:row + n]
            row += n
            table = set(p for p in r.engine.tables.table(r._ids[e["id"]], 0) if p >= 0)
            if e["_at"] == 0 and table & pages_seen:
                reused = True
            pages_seen |= table
        r.step([], end)
        assert r.engine.tables.audit() == ""
    assert reused, "the trace never reused a page; make the pool smaller"
    for i, (toks, ref) in enumerate(seqs):
        check(got[i], ref, dtype, f"{name} mixed, request {i}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(gpu, dtype):
    toks, ref = reference_logits("c", 5, 400)
    r = runner("c", dtype, 448)
    outs = [r.step([{"id": 0, "tokens": toks[:6], "want": list(range(6))}])]
    for i in range(6, 400):
        outs.append(r.step([{"id": 0, "tokens": [toks[i]], "want": [0]}]))
    check(np.concatenate(outs), ref, dtype, "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b"])
def test_first_tokens(gpu, name, dtype):
    toks, ref = reference_logits(name, 6, 4)
    r = runner(name, dtype, 64)
    for n in (1, 2, 3, 4):
        got = r.step([{"id": n, "tokens": toks[:n], "want": list(range(n))}], [n])
        check(got, ref[:n], dtype, f"{name} first {n}")
    outs = [r.step([{"id": "d", "tokens": [toks[i]], "want": [0]}]) for i in range(4)]   # from the very first token
    check(np.concatenate(outs), ref, dtype, f"{name} decode from token 0")


def test_wanted_places_only(gpu):
    toks, ref = reference_logits("b", 7, 50)
    r = runner("b", "float32", 128)
    assert r.step([{"id": 0, "tokens": toks[:20], "want": []}]) is None
    got = r.step([{"id": 0, "tokens": toks[20:50], "want": [29, 0, 7]}, {"id": 1, "tokens": toks[:5], "want": [4]}])
    check(got[:3], ref[[49, 20, 27]], "float32", "wanted rows in the order asked")
    check(got[3:], ref[[4]], "float32", "second request")


def test_bfloat16_storage_is_used_as_stored(gpu):
    """A folder stored in bfloat16, run in float32: the engine widens exactly, so it matches the plain
    implementation on the rounded weights to float32 accuracy."""
    from prelude_amd.trace import TraceRunner
    folder, _, _ = model_folder("a", "bfloat16")
    toks, ref = reference_logits("a", 8, 60, "bfloat16")
    r = TraceRunner(folder, "float32", 128, page_size=8)
    got = r.step([{"id": 0, "tokens": toks, "want": list(range(60))}])
    check(got, ref, "float32", "bf16-stored weights in the 32-bit path")


def test_errors_leave_the_cache_intact(gpu):
    from prelude_amd.cache import OutOfPages
    from prelude_amd.engine import StepError
    toks, _ = reference_logits("a", 9, 100)
    r = runner("a", "float32", 64)
    r.step([{"id": 0, "tokens": toks[:40], "want": []}])
    with pytest.raises(OutOfPages):
        r.step([{"id": 1, "tokens": toks[:40], "want": []}])
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 1
    with pytest.raises(StepError, match="vocabulary"):
        r.step([{"id": 0, "tokens": [5, 256], "want": []}])
    with pytest.raises(StepError, match="wanted place"):
        r.step([{"id": 0, "tokens": [5], "want": [1]}])
    with pytest.raises(StepError, match="max_position_embeddings"):
        r.step([{"id": 0, "tokens": toks[:89], "want": []}])
    assert r.engine.length(0) == 40


def _trace_steps(toks, toks2):
    return [
        {"step": 0, "entries": [{"id": "a", "tokens": toks[:50], "want": [0, 49]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks[50:52], "want": []},
                                {"id": "b", "tokens": toks2[:30], "want": [29]}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": toks[52:53], "want": [0]},
                                {"id": "b", "tokens": toks2[30:31], "want": [0]}], "end": ["a"]},
        {"step": 5, "entries": [{"id": "b", "tokens": toks2[31:40], "want": [8]}], "end": ["b"]},
    ]


def _run_program(args, steps, out):
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), *args, "--out", str(out)],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,pool", [("a", ["--page-size", "8", "--num-pages", "13"]), ("b", ["--max-tokens", "128"])])
def test_trace_run_program(gpu, dtype, name, pool, tmp_path):
    """bin/trace_run as a user runs it: JSON lines in, <step>.f32 files and `done <step>` lines out; Tiny A with
    its pages of 8 given as a number of pages, Tiny B with pages of 16 and the pool given in tokens."""
    folder, cfg, _ = model_folder(name)
    n = LENGTHS[name]
    toks, ref = reference_logits(name, 0, n)
    toks2, ref2 = reference_logits(name, 1, n)
    out = tmp_path / "out"
    _run_program(["--model", folder, "--dtype", dtype, *pool], _trace_steps(toks, toks2), out)
    v = cfg["vocab_size"]
    load = lambda s: np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(-1, v)
    check(load(0), ref[[0, 49]], dtype, "step 0")
    check(load(1), ref2[[29]], dtype, "step 1")
    check(load(2), torch.stack([ref[52], ref2[30]]), dtype, "step 2")
    check(load(5), ref2[[39]], dtype, "step 5")
    assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "2.f32", "5.f32"]


def test_trace_run_program_from_a_bare_config(gpu, tmp_path):
    """--random-weights: only a config.json is there; the weights are drawn on the device from the seed, the
    same ones ``random_tensors_on_device`` gives, which the plain implementation is run on here."""
    from prelude_amd.weights import random_tensors_on_device
    import plain_model as pm
    cfg = pm.tiny_config_a()
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    w = {k: v.float().cpu() for k, v in random_tensors_on_device(cfg, 5, gpu, dtype=torch.float32).items()}
    g = torch.Generator().manual_seed(77)
    toks, toks2 = (torch.randint(0, cfg["vocab_size"], (60,), generator=g).tolist() for _ in range(2))
    ref, ref2 = pm.forward(cfg, w, toks), pm.forward(cfg, w, toks2)
    out = tmp_path / "out"
    _run_program(["--random-weights", str(tmp_path / "config.json"), "--weights-seed", "5", "--dtype", "float32",
                  "--page-size", "8", "--num-pages", "13"], _trace_steps(toks, toks2), out)
    load = lambda s: np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(-1, cfg["vocab_size"])
    check(load(0), ref[[0, 49]], "float32", "step 0")
    check(load(2), torch.stack([ref[52], ref2[30]]), "float32", "step 2")
    check(load(5), ref2[[39]], "float32", "step 5")
    # another seed, other weights
    out2 = tmp_path / "out2"
    _run_program(["--random-weights", str(tmp_path), "--weights-seed", "6", "--dtype", "float32", "--max-tokens", "128"],
                 _trace_steps(toks, toks2)[:1], out2)
    assert float(np.abs(np.fromfile(out2 / "0.f32", dtype="<f4").reshape(-1, cfg["vocab_size"]) - load(0)).max()) > 1e-3


def test_a_seed_names_one_model_on_the_cpu_and_on_the_gpu(gpu):
    """The random-weights mode draws the same values wherever it draws: what ``--write-model`` puts into a folder
    from the CPU is what ``--random-weights`` alone draws on the device."""
    from prelude_amd.weights import random_tensors, random_tensors_on_device
    import plain_model as pm
    cfg = pm.tiny_config_c()
    host = random_tensors(cfg, 7, std=0.05, norm_std=0.02, dtype=torch.float32, device="cpu")
    dev = random_tensors_on_device(cfg, 7, gpu, std=0.05, norm_std=0.02, dtype=torch.float32)
    assert set(host) == set(dev)
    for name in host:
        assert torch.equal(host[name], dev[name].cpu()), name
    host16 = random_tensors(cfg, 7, dtype=torch.bfloat16, device="cpu")
    dev16 = random_tensors_on_device(cfg, 7, gpu, dtype=torch.bfloat16)
    assert all(torch.equal(host16[n].float(), dev16[n].cpu().float().to(torch.bfloat16).float()) for n in host16)


def test_graph_replays_equal_eager_steps(gpu):
    """Decode steps replayed from HIP graphs, with eager work (prompt portions, other batch sizes) between the
    replays: every replay gives the logits of the eager step, bit for bit."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    folder, cfg, _ = model_folder("b")
    seqs = [reference_logits("b", 20 + i, n)[0] for i, n in enumerate([150, 40, 90])]

    def play(hip_graph):
        eng = Engine.from_model_dir(folder, EngineConfig(dtype="bfloat16", page_size=16, max_cache_tokens=1024,
                                                         hip_graph=hip_graph))
        outs = []
        at = [0, 0, 0]

        def feed(parts):
            entries = []
            for r, n in parts:
                entries.append(StepEntry(r, seqs[r][at[r]:at[r] + n], [n - 1]))
                at[r] += n
            outs.append(eng.step(entries).cpu())
        feed([(0, 60)])
        for _ in range(5):
            feed([(0, 1)])                       # batch of one: first capture, then replays
        feed([(1, 20), (0, 1)])                  # eager, mixed
        for _ in range(4):
            feed([(0, 1), (1, 1)])               # batch of two
        feed([(2, 70)])
        for _ in range(6):
            feed([(0, 1), (1, 1), (2, 1)])
        for _ in range(3):
            feed([(0, 1)])                       # the first graph again, after the others
        feed([(2, 1), (0, 1)])                   # other order of requests, same graph as batch of two
        return eng, outs

    eager_eng, eager = play(False)
    graph_eng, graphed = play(True)
    assert eager_eng._graphs is None and graph_eng._graphs.captures == 3 and graph_eng._graphs.replays == 19
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert torch.equal(a, b), f"step {i}: the replay differs from the eager step"


def test_graph_replays_equal_eager_steps_where_the_grid_sets_the_wavefronts(gpu):
    """The decode attention runs grids of 769 to 1,536 workgroups with two wavefronts a workgroup, which add a
    split's steps in another order than four.  A replayed step knows its longest context only as a bound (the
    width of its block tables), so a step run directly counts its splits from the same bound: five requests of 8
    KV heads at some 4,200 tokens are 8 x 17 x 5 = 680 workgroups by their lengths and 8 x 20 x 5 = 800 by the
    bound.  Replay and direct run give the same bits there too."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    import plain_model as pm
    cfg = dict(pm.tiny_config_b(), num_attention_heads=8, num_key_value_heads=8, head_dim=64, num_hidden_layers=1,
               max_position_embeddings=4400, vocab_size=200, eos_token_id=199)
    rng = np.random.default_rng(9)
    lens = [4200, 4150, 3000, 4199, 500]
    seqs = [rng.integers(0, cfg["vocab_size"], size=n + 6).tolist() for n in lens]

    def play(hip_graph):
        eng = Engine.from_config(cfg, EngineConfig(dtype="bfloat16", page_size=16, max_cache_tokens=5 * 4416,
                                                   hip_graph=hip_graph), seed=4, std=0.05)
        outs = []
        for r, n in enumerate(lens):
            for lo in range(0, n, 2048):
                hi = min(n, lo + 2048)
                eng.step([StepEntry(r, seqs[r][lo:hi], [])])
        for k in range(6):
            outs.append(eng.step([StepEntry(r, [seqs[r][n + k]], [0]) for r, n in enumerate(lens)]).cpu())
        return eng, outs

    eager_eng, eager = play(False)
    graph_eng, graphed = play(True)
    assert eager_eng._graphs is None and graph_eng._graphs.replays == 6
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert torch.equal(a, b), f"step {i}: the replay differs from the eager step"


def test_graph_replays_of_steps_with_portions_equal_eager_steps(gpu):
    """Small steps that bring prompt portions are captured when their shape (portion lengths, wanted rows, table
    width, whether every portion has its own length behind it) comes a second time, and replayed from then on: whole
    prompts of one length, portions without wanted rows, portions behind a long context, and steps of portions
    beside single tokens, with other requests, other pages and other positions at every replay.  Every step gives
    the eager step's logits bit for bit."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    folder, cfg, _ = model_folder("b")
    rng = np.random.default_rng(12)
    seqs = [rng.integers(0, cfg["vocab_size"], size=200).tolist() for _ in range(8)]

    def play(hip_graph, portion_tokens=1024):
        eng = Engine.from_model_dir(folder, EngineConfig(dtype="bfloat16", page_size=16, max_cache_tokens=8 * 208,
                                                         hip_graph=hip_graph, hip_graph_portion_tokens=portion_tokens))
        outs, at = [], [0] * 8

        def feed(parts):
            entries = []
            for r, n, wanted in parts:
                entries.append(StepEntry(r, seqs[r][at[r]:at[r] + n], [n - 1] if wanted else []))
                at[r] += n
            outs.append(eng.step(entries).cpu())
        for r in range(4):
            feed([(r, 40, True)])                    # a prompt of 40 tokens: met, then captured and replayed
        for r in range(4):
            feed([(r, 30, False)])                   # a portion behind 40 tokens, nothing wanted
        for r in range(4):
            feed([(r, 24, True)])                    # a portion with more than its own length behind it
        for r in range(4, 7):
            feed([(0, 1, True), (r, 33, True), (1, 1, True)])     # a prompt between two decoding requests
        for r in range(4):
            feed([(r, 40, True)])                    # 40 tokens again, behind 94 or 95: a shape of its own
        feed([(7, 37, True)])                        # a shape that comes once
        for _ in range(2):                           # single tokens, one of which wants no logits: no decode step's
            feed([(0, 1, True), (1, 1, False), (2, 1, True)])   # graph fits that; met, then captured as a shape of its own
        for _ in range(3):
            feed([(r, 1, True) for r in range(8)])   # decode steps: captured at once, as ever
        return eng, outs

    eager_eng, eager = play(False)
    graph_eng, graphed = play(True)
    off_eng, off = play(True, portion_tokens=0)
    # shapes: (40,) from the start; (30,) behind 40; (24,) behind 70; (1, 33, 1); (40,) behind 94; (1, 1, 1) with two
    # rows wanted; the decode step
    # a shape of portions runs eagerly the first time and from its graph after that
    assert graph_eng._graphs.captures == 7 and graph_eng._graphs.replays == 3 + 3 + 3 + 2 + 3 + 1 + 3
    assert off_eng._graphs.captures == 1 and off_eng._graphs.replays == 3
    for i, (a, b, c) in enumerate(zip(eager, graphed, off)):
        assert a.shape == b.shape and torch.equal(a, b), f"step {i}: the replay differs from the eager step"
        assert torch.equal(a, c)
    assert graph_eng.tables.audit() == ""


def test_a_step_whose_capture_fails_runs_directly(gpu, monkeypatch):
    """The capture of a step is an extra: if it fails (here: made to), the step runs directly and gives the direct
    run's logits, its shape is not tried again, and other shapes are captured as ever."""
    import contextlib
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    from prelude_amd.engine import graph as graph_module
    folder, cfg, _ = model_folder("b")
    rng = np.random.default_rng(14)
    seqs = [rng.integers(0, cfg["vocab_size"], size=60).tolist() for _ in range(4)]

    def play(hip_graph, break_portions):
        eng = Engine.from_model_dir(folder, EngineConfig(dtype="bfloat16", page_size=16, max_cache_tokens=512,
                                                         hip_graph=hip_graph))
        if break_portions:
            real = torch.cuda.graph

            @contextlib.contextmanager
            def refusing(graph, pool=None):
                if eng._graphs.captures >= 0 and refusing.portions:
                    raise torch.cuda.OutOfMemoryError("no memory for this capture (made up by the test)")
                with real(graph, pool=pool):
                    yield
            refusing.portions = True
            monkeypatch.setattr(graph_module.torch.cuda, "graph", refusing)
        outs = []
        for r in range(4):
            outs.append(eng.step([StepEntry(r, seqs[r][:40], [39])]).cpu())     # the same shape four times
        if break_portions:
            refusing.portions = False
        for k in range(3):
            outs.append(eng.step([StepEntry(r, [seqs[r][40 + k]], [0]) for r in range(4)]).cpu())
        if break_portions:
            refusing.portions = True
        for k in range(2):    # a decode step of another batch size whose capture fails as well: it runs directly too
            outs.append(eng.step([StepEntry(r, [seqs[r][43 + k]], [0]) for r in range(2)]).cpu())
        if break_portions:
            monkeypatch.undo()
        return eng, outs

    eager_eng, eager = play(False, False)
    graph_eng, graphed = play(True, True)
    assert graph_eng._graphs.captures == 1 and graph_eng._graphs.replays == 3       # the decode step of four only
    assert len(graph_eng._graphs._refused) == 2
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert torch.equal(a, b), f"step {i}"
    assert graph_eng.tables.audit() == ""


def test_no_garbage_is_collected_while_a_step_is_captured(gpu):
    """A collection inside a capture would run the destructors of dead cycles there, an earlier engine's graphs among
    them, whose destructor waits for the device: not allowed while a stream is captured.  So the collector is off
    exactly while a step is recorded and on again afterwards, also when the capture fails; and an engine that is let
    go takes its graphs with it at once, with no cycle left for a collection to find."""
    import gc
    import weakref
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    folder, cfg, _ = model_folder("a")
    rng = np.random.default_rng(15)
    seqs = [rng.integers(0, cfg["vocab_size"], size=40).tolist() for _ in range(2)]
    eng = Engine.from_model_dir(folder, EngineConfig(dtype="bfloat16", page_size=16, max_cache_tokens=256, hip_graph=True))
    seen = []
    forward = eng.forward

    def watching(*args):
        seen.append((torch.cuda.is_current_stream_capturing(), gc.isenabled()))
        return forward(*args)
    eng.forward = watching
    assert gc.isenabled()
    for r in range(2):
        eng.step([StepEntry(r, seqs[r][:30], [29])])
    for k in range(3):
        eng.step([StepEntry(r, [seqs[r][30 + k]], [0]) for r in range(2)])
    assert eng._graphs.captures == 2      # the portion's shape at its second sighting, the decode step
    assert (True, False) in seen and (False, True) in seen
    assert all(collecting != capturing for capturing, collecting in seen), seen
    assert gc.isenabled()
    del eng.forward       # the class's own again

    graphs = weakref.ref(eng._graphs)
    captured = [weakref.ref(c.graph) for c in eng._graphs._graphs.values()]
    gc.disable()
    try:
        del eng, forward, watching
        assert graphs() is None and all(c() is None for c in captured)
    finally:
        gc.enable()


def test_graph_replays_with_library_products_equal_eager_steps(gpu):
    """A decode step of more than 48 requests multiplies through the library product, also inside a captured
    graph (with its workspace): every replay, with eager steps of other shapes between them, gives the eager
    step's logits bit for bit."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    folder, cfg, _ = model_folder("b")
    rng = np.random.default_rng(5)
    n = 56
    seqs = [rng.integers(0, cfg["vocab_size"], size=40).tolist() for _ in range(n)]

    def play(hip_graph):
        eng = Engine.from_model_dir(folder, EngineConfig(dtype="bfloat16", page_size=16, max_cache_tokens=n * 48,
                                                         hip_graph=hip_graph))
        outs, at = [], [0] * n

        def feed(parts):
            entries = []
            for r, k in parts:
                entries.append(StepEntry(r, seqs[r][at[r]:at[r] + k], [k - 1]))
                at[r] += k
            outs.append(eng.step(entries).cpu())
        feed([(r, 7 + r % 5) for r in range(n)])
        for i in range(4):
            feed([(r, 1) for r in range(n)])      # the graph of 56 single tokens: capture, then replays
            feed([(i, 2), (n - 1 - i, 3)])        # eager work between the replays
            torch.cuda.synchronize()
        for _ in range(3):
            feed([(r, 1) for r in range(n)])
        return eng, outs

    eager_eng, eager = play(False)
    graph_eng, graphed = play(True)
    assert graph_eng._graphs.captures >= 1 and graph_eng._graphs.replays >= 6
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert torch.equal(a, b), f"step {i}: the replay differs from the eager step"


@pytest.mark.parametrize("dtype,hip_graph", [("float32", False), ("bfloat16", False), ("bfloat16", True)])
def test_tokens_carried_on_the_device(gpu, dtype, hip_graph):
    """A step whose last tokens are taken from a device tensor (the previous step's samples, never read by the
    host) gives the logits of the step fed the same ids from the host, bit for bit: in decode steps, in a
    mixed step, and at the end of a prompt portion."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    from prelude_amd.engine.engine import StepError
    folder, cfg, _ = model_folder("b", dtype)
    seqs = [reference_logits("b", 30 + i, n, dtype)[0] for i, n in enumerate([70, 33, 50])]
    dev = torch.device("cuda:0")

    def play(carry):
        eng = Engine.from_model_dir(folder, EngineConfig(dtype=dtype, page_size=16, max_cache_tokens=1024,
                                                         hip_graph=hip_graph))
        outs, at = [], [0, 0, 0]

        def feed(parts):
            entries, ids = [], []
            for r, n in parts:
                toks = list(seqs[r][at[r]:at[r] + n])
                at[r] += n
                if carry:
                    ids.append(toks[-1])
                    entries.append(StepEntry(r, toks[:-1] + [0], [n - 1], carry=len(ids) - 1))
                else:
                    entries.append(StepEntry(r, toks, [n - 1]))
            # rows in another order than the entries, with a row nobody takes
            carried = torch.tensor([7] + ids[::-1], dtype=torch.int32, device=dev) if carry else None
            for e in entries:
                if carry:
                    e.carry = len(ids) - e.carry
            outs.append(eng.step(entries, carried=carried).cpu())
        feed([(0, 40), (1, 9)])
        for _ in range(4):
            feed([(0, 1), (1, 1)])
        feed([(2, 30), (0, 1)])
        for _ in range(3):
            feed([(1, 1), (2, 1), (0, 1)])
        return eng, outs

    _, plain = play(False)
    eng, carried = play(True)
    for i, (a, b) in enumerate(zip(plain, carried)):
        assert torch.equal(a, b), f"step {i}: carried ids gave other logits"
    with pytest.raises(StepError, match="carried"):
        eng.step([StepEntry(0, [0], [0], carry=0)])
    with pytest.raises(StepError, match="outside"):
        eng.step([StepEntry(0, [0], [0], carry=3)], carried=torch.zeros(3, dtype=torch.int32, device=dev))
    with pytest.raises(StepError, match="int32"):
        eng.step([StepEntry(0, [0], [0], carry=0)], carried=torch.zeros(3, dtype=torch.int64, device=dev))
    assert eng.tables.audit() == ""
