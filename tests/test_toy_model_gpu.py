"""Generality of the parts: a toy mixer with state of its own and a toy architecture, both defined here, are
registered, built, loaded from a folder the random-weights mode writes, and stepped -- without a change to the
framework's files.  The toy model also names a layer twice in its run order and lets a run read another run's cache.
It is no model of anyone's: a decaying sum as mixer, beside the framework's attention in the other layer.
"""
import dataclasses
import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu


def register_toy():
    from prelude_amd.config.registry import Architecture, register_architecture
    from prelude_amd.models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec
    from prelude_amd.ops import kernels as K
    from prelude_amd.parts import MATRIX, Mixer, StateSpec, TensorReq, register_part

    @register_part("mixer", "toy_decay")
    class ToyDecay(Mixer):
        """s_t = decay * s_{t-1} + x_t per request; y_t = W s_t.  The state s lives in a slot of the cache manager."""

        GRAPH_SAFE = False     # it walks the step's host-side lists

        def __init__(self, hidden_size, decay):
            self.hidden_size, self.decay = hidden_size, decay
            self.w = None

        def cache_spec(self):
            return StateSpec((("s", (self.hidden_size,), torch.float32),))

        def tensors(self):
            return {"proj.weight": TensorReq((self.hidden_size, self.hidden_size), MATRIX)}

        def load(self, tensors, dtype, device):
            self.w = tensors["proj.weight"]

        def forward(self, x, step, cache, write_cache=True):
            s_all = cache.tensors["s"]
            out = torch.empty_like(x)
            t = 0
            for i, n in enumerate(step.q_lens):            # a request's portion is processed in order
                slot = step.state_slots_host[i]
                s = s_all[slot].clone()
                for j in range(n):
                    s = self.decay * s + x[t + j].float()
                    out[t + j] = s.to(x.dtype)
                s_all[slot] = s
                t += n
            return K.linear(out, self.w)

    @register_part("mixer", "toy_decay_device")
    class ToyDecayDevice(ToyDecay):
        """The same mixer with its decode step written on the device alone: it finds its slots through
        ``step.state_slots``, so a step of single tokens can be captured once and replayed."""
        GRAPH_SAFE = True

        def forward(self, x, step, cache, write_cache=True):
            if not step.all_decode:
                return super().forward(x, step, cache, write_cache)
            s_all = cache.tensors["s"]
            slots = step.state_slots.to(torch.int64)
            s = self.decay * s_all.index_select(0, slots) + x.float()
            s_all.index_copy_(0, slots, s)
            return K.linear(s.to(x.dtype), self.w)

    @register_part("mixer", "toy_decay_whole")
    class ToyDecayWhole(ToyDecay):
        """The same mixer, declared unable to take a prompt in portions: it refuses any portion of several tokens
        that does not start its request, and the scheduler is to feed it prompts whole."""
        ATOMIC_PREFILL = True
        portions = []          # (tokens, fresh) of every portion it was given, for the test to look at

        def forward(self, x, step, cache, write_cache=True):
            for n, fresh in zip(step.q_lens, step.fresh_host):
                ToyDecayWhole.portions.append((n, bool(fresh)))
                if n > 1 and not fresh:
                    raise RuntimeError(f"a prompt came in portions: {n} tokens behind an earlier portion")
            return super().forward(x, step, cache, write_cache)

    @dataclasses.dataclass
    class ToyConfig:
        vocab_size: int
        hidden_size: int
        inter: int
        heads: int
        head_dim: int
        decay: float
        eps: float
        max_positions: int

    def parse(raw):
        return ToyConfig(**{f.name: raw[f.name] for f in dataclasses.fields(ToyConfig)})

    def spec(c, mixer="toy_decay"):
        norm = lambda name: PartSpec("rms_norm", dict(size=c.hidden_size, eps=c.eps), {"weight": name})
        ffn = lambda p: PartSpec("gated_mlp", dict(hidden_size=c.hidden_size, intermediate_size=c.inter),
                                 {f"{x}_proj.weight": f"{p}.ffn.{x}" for x in ("gate", "up", "down")})
        toy = LayerSpec("prenorm", {"input_norm": norm("l0.n1"), "post_mixer_norm": norm("l0.n2"), "ffn": ffn("l0"),
                                    "mixer": PartSpec(mixer, dict(hidden_size=c.hidden_size, decay=c.decay),
                                                      {"proj.weight": "l0.mix.proj"})})
        attn = LayerSpec("prenorm", {"input_norm": norm("l1.n1"), "post_mixer_norm": norm("l1.n2"), "ffn": ffn("l1"),
                                     "mixer": PartSpec("gqa_attention", dict(
                                         hidden_size=c.hidden_size, num_heads=c.heads, num_kv_heads=1,
                                         head_dim=c.head_dim, norm_eps=c.eps, qk_norm=False, position="rope"),
                                         {f"{x}_proj.weight": f"l1.attn.{x}" for x in "qkvo"})})
        # layer 0 twice (two states per request), and the last run reads the keys and values run 1 wrote
        order = [RunSpec(0), RunSpec(1), RunSpec(0), RunSpec(1, reads_cache_of=1)]
        return ModelSpec("ToyForCausalLM", c.vocab_size, c.hidden_size, c.max_positions, (0,),
                         PartSpec("token_embedding", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size), {"weight": "emb"}),
                         [toy, attn], order, norm("final"),
                         PartSpec("linear_head", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size), {"weight": "emb"}),
                         {"rope": PartSpec("rope", dict(rotary_dim=c.head_dim, max_positions=c.max_positions, theta=100.0))})

    register_architecture(Architecture("toy", ("Toy",), ("toy",), parse, spec))
    register_architecture(Architecture("toydevice", ("ToyDevice",), ("toydevice",), parse,
                                       lambda c: spec(c, "toy_decay_device")))
    register_architecture(Architecture("toywhole", ("ToyWhole",), ("toywhole",), parse,
                                       lambda c: spec(c, "toy_decay_whole")))
    return ToyDecayWhole


RAW = dict(architectures=["ToyForCausalLM"], vocab_size=97, hidden_size=48, inter=80, heads=3, head_dim=16, decay=0.7,
           eps=1e-5, max_positions=128)


def plain_toy(w, toks):
    """The toy model for a whole sequence, in float64, from plain_model's functions."""
    w = {k: v.double() for k, v in w.items()}
    n = len(toks)
    cos, sin = pm.rope_tables(16, 128, 100.0)
    x = w["emb"][toks]

    def toy(x, p):
        h = pm.rms_norm(x, w[p + ".n1"], 1e-5)
        s = torch.zeros(48, dtype=torch.float64)
        ys = []
        for t in range(n):
            s = 0.7 * s + h[t]
            ys.append(s.float().double())     # the state is kept in 32-bit
        x = x + torch.stack(ys) @ w[p + ".mix.proj"].T
        return x + pm.swiglu(pm.rms_norm(x, w[p + ".n2"], 1e-5), w[p + ".ffn.gate"], w[p + ".ffn.up"], w[p + ".ffn.down"])

    def attn(x, p, kv=None):
        h = pm.rms_norm(x, w[p + ".n1"], 1e-5)
        q = pm.apply_rope((h @ w[p + ".attn.q"].T).reshape(n, 3, 16), cos[:n], sin[:n])
        if kv is None:
            k = pm.apply_rope((h @ w[p + ".attn.k"].T).reshape(n, 1, 16), cos[:n], sin[:n])
            kv = (k, (h @ w[p + ".attn.v"].T).reshape(n, 1, 16))
        o = pm.attention(q, kv[0], kv[1], 0.25)
        x = x + o.reshape(n, 48) @ w[p + ".attn.o"].T
        x = x + pm.swiglu(pm.rms_norm(x, w[p + ".n2"], 1e-5), w[p + ".ffn.gate"], w[p + ".ffn.up"], w[p + ".ffn.down"])
        return x, kv

    x = toy(x, "l0")
    x, kv = attn(x, "l1")
    x = toy(x, "l0")
    x, _ = attn(x, "l1", kv)
    return pm.rms_norm(x, w["final"], 1e-5) @ w["emb"].T


def test_toy_model_is_built_and_stepped(gpu, tmp_path):
    register_toy()
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    from prelude_amd.weights import WeightFiles, write_random_model
    folder = write_random_model(RAW, str(tmp_path / "toy"), seed=4, std=0.2, norm_std=0.1, dtype=torch.float32)
    files = WeightFiles(folder)
    w = {n: files.tensor(n).clone() for n in files.names()}
    assert set(w) == {"emb", "final"} | {f"l{i}.n{j}" for i in (0, 1) for j in (1, 2)} | {"l0.mix.proj"} | \
        {f"l{i}.ffn.{x}" for i in (0, 1) for x in ("gate", "up", "down")} | {f"l1.attn.{x}" for x in "qkvo"}
    eng = Engine.from_model_dir(folder, EngineConfig(dtype="float32", page_size=8, max_cache_tokens=128, max_state_slots=2))
    m = eng.model
    assert m.needs_state and len(m.cache_slots) == 3 and m.run_cache == [0, 1, 2, 1]      # two states, one KV cache
    g = torch.Generator().manual_seed(0)
    seqs = [torch.randint(0, 97, (n,), generator=g).tolist() for n in (50, 31, 44)]
    refs = [plain_toy(w, s) for s in seqs]

    def close(got, ref):
        assert float((got.double().cpu() - ref).abs().max()) < 2e-5 * max(1.0, float(ref.abs().max()))

    # whole
    close(eng.step([StepEntry(0, seqs[0], list(range(50)))]), refs[0])
    eng.release(0)
    # two requests in portions, mixed in one batch: state is carried across portions and kept apart per request
    got = {1: [], 2: []}
    cuts = {1: [7, 2, 20, 1, 1], 2: [3, 11, 1, 5, 24]}
    at = {1: 0, 2: 0}
    for k in range(5):
        entries = []
        for rid in (1, 2):
            n = cuts[rid][k]
            entries.append(StepEntry(rid, seqs[rid][at[rid]:at[rid] + n], list(range(n))))
            at[rid] += n
        out = eng.step(entries)
        got[1].append(out[:cuts[1][k]])
        got[2].append(out[cuts[1][k]:])
    close(torch.cat(got[1]), refs[1][:31])
    close(torch.cat(got[2]), refs[2][:44])
    # both slots are taken: a third request cannot open; after a release its slot starts from zero again
    from prelude_amd.cache import CacheError
    with pytest.raises(CacheError, match="state slot"):
        eng.step([StepEntry(3, seqs[0][:4], [3])])
    assert eng.tables.audit() == ""
    eng.release(1)
    close(eng.step([StepEntry(3, seqs[0], list(range(50)))]), refs[0])
    eng.release(2)
    eng.release(3)
    assert eng.tables.audit() == "" and eng.tables.free_state_slots() == 2


def test_toy_model_generates_through_the_entry_point(gpu, tmp_path):
    register_toy()
    from prelude_amd import LLM
    from prelude_amd.weights import WeightFiles, write_random_model
    folder = write_random_model(RAW, str(tmp_path / "toy"), seed=5, std=0.2, norm_std=0.1, dtype=torch.float32)
    files = WeightFiles(folder)
    w = {n: files.tensor(n).clone() for n in files.names()}
    llm = LLM(folder, dtype="float32", page_size=8, max_cache_tokens=256, max_state_slots=2, max_num_batched_tokens=16)
    prompts = [[5, 6, 7, 8, 9] * 5, [11, 12, 13], [20] * 30]           # three requests over two state slots
    outs = llm.generate(prompts, max_tokens=6, temperature=0.0)
    for p, o in zip(prompts, outs):
        seq = list(p)
        for tok in o.token_ids:
            assert tok == int(torch.argmax(plain_toy(w, seq)[-1]))
            seq.append(tok)
        assert o.finish_reason in ("length", "eos")
    assert llm.engine.tables.audit() == "" and llm.engine.tables.free_state_slots() == 2


def test_toy_model_with_state_decodes_from_graphs(gpu, tmp_path):
    """A model whose mixer keeps state per request is captured and replayed like any other once its decode step
    stays on the device: slots come through ``step.state_slots``, and the slot of a request that starts inside a
    captured step (a prompt of one token, in a slot another request has used) is cleared on the device."""
    register_toy()
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    from prelude_amd.weights import WeightFiles, write_random_model
    raw = dict(RAW, architectures=["ToyDeviceForCausalLM"])
    folder = write_random_model(raw, str(tmp_path / "toydev"), seed=6, std=0.2, norm_std=0.1, dtype=torch.bfloat16)
    files = WeightFiles(folder)
    w = {n: files.tensor(n).float() for n in files.names()}
    g = torch.Generator().manual_seed(3)
    seqs = [torch.randint(0, 97, (n,), generator=g).tolist() for n in (40, 33, 25)]
    refs = [plain_toy(w, s) for s in seqs]

    def play(hip_graph):
        eng = Engine.from_model_dir(folder, EngineConfig(dtype="bfloat16", page_size=8, max_cache_tokens=256,
                                                         max_state_slots=2, hip_graph=hip_graph))
        assert eng.model.needs_state and eng.model.graph_safe
        rows = {0: [], 1: [], 2: []}
        eng.step([StepEntry(0, seqs[0][:20], [])])
        eng.step([StepEntry(1, seqs[1][:9], [])])
        for k in range(12):                               # both slots in use, a batch of two, replayed
            out = eng.step([StepEntry(0, [seqs[0][20 + k]], [0]), StepEntry(1, [seqs[1][9 + k]], [0])])
            rows[0].append(out[0:1].cpu()), rows[1].append(out[1:2].cpu())
        eng.release(1)                                    # its slot holds what request 1 left there
        for k in range(8):                                # request 2 starts inside the captured step of two
            out = eng.step([StepEntry(0, [seqs[0][32 + k]], [0]), StepEntry(2, [seqs[2][k]], [0])])
            rows[0].append(out[0:1].cpu()), rows[2].append(out[1:2].cpu())
        return eng, {r: torch.cat(v) for r, v in rows.items()}

    eager_eng, eager = play(False)
    eng, replayed = play(True)
    assert eager_eng._graphs is None and eng._graphs.captures == 1 and eng._graphs.replays == 20
    for r in rows_of(eager):
        assert torch.equal(eager[r], replayed[r])
    from helpers import check
    for r, lo, hi in ((0, 20, 40), (1, 9, 21), (2, 0, 8)):
        check(replayed[r], refs[r][lo:hi], "bfloat16", f"request {r}")


def test_toy_mixer_that_takes_prompts_whole(gpu, tmp_path):
    """A mixer that sets ATOMIC_PREFILL: under a token budget that would cut prompts, the scheduler feeds each
    prompt in one step (later, if it does not fit beside the others), the tokens are the plain model's, and a
    request that could never be fed whole is refused when it is added."""
    whole = register_toy()
    from prelude_amd import LLM
    from prelude_amd.engine.scheduler import SchedulerError
    from prelude_amd.weights import WeightFiles, write_random_model
    raw = dict(RAW, architectures=["ToyWholeForCausalLM"])
    folder = write_random_model(raw, str(tmp_path / "toywhole"), seed=7, std=0.2, norm_std=0.1, dtype=torch.float32)
    files = WeightFiles(folder)
    w = {n: files.tensor(n).clone() for n in files.names()}
    llm = LLM(folder, dtype="float32", page_size=8, max_cache_tokens=256, max_state_slots=3, max_num_batched_tokens=16)
    assert llm.engine.model.atomic_prefill and not llm.engine.model.graph_safe
    whole.portions.clear()
    prompts = [[5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15], [11, 12, 13, 14, 15, 16, 17, 18, 19], [20] * 12, [3, 4]]
    outs = llm.generate(prompts, max_tokens=4, temperature=0.0)
    for p, o in zip(prompts, outs):
        seq = list(p)
        assert o.finish_reason in ("length", "eos") and o.error is None
        for tok in o.token_ids:
            assert tok == int(torch.argmax(plain_toy(w, seq)[-1]))
            seq.append(tok)
    # every prompt arrived whole (11 + 9 would fit a step of 16 only in part: the second waited), none in pieces
    firsts = sorted(n for n, fresh in whole.portions if fresh)
    assert firsts == sorted([len(p) for p in prompts] * 2)        # the mixer runs twice a step (its layer is named twice)
    assert all(n == 1 for n, fresh in whole.portions if not fresh)
    # 14 prompt tokens and up to 4 new ones cannot be fed in one step of 16 after an eviction: refused at once
    session = llm.session()
    with pytest.raises(SchedulerError, match="must be fed whole"):
        session.add(list(range(14)), max_tokens=4)
    assert session.add(list(range(13)), max_tokens=4) == 0
    session.abandon()
    assert llm.engine.tables.audit() == "" and llm.engine.tables.free_state_slots() == 3


def rows_of(d):
    return sorted(d)
