"""Generality of the parts, again from outside the package: a feed-forward that routes every token to one of its
experts, and another position encoding (rotation by scaled positions over half of each head), registered here,
built into a toy architecture beside the framework's attention, loaded from a folder the random-weights mode
writes, and stepped whole, in portions and token by token.  The routed feed-forward looks at its routing on the
host, so it says that its steps cannot be replayed from a captured graph.  No model of anyone's.
"""
import dataclasses

import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu
E, INTER, ROT, FACTOR, THETA = 3, 24, 8, 2.5, 50.0


def register_toy_parts():
    from prelude_amd.config.registry import Architecture, register_architecture
    from prelude_amd.models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec
    from prelude_amd.ops import kernels as K
    from prelude_amd.parts import MATRIX, FeedForward, PositionEncoding, TensorReq, register_part

    @register_part("ffn", "toy_routed")
    class ToyRouted(FeedForward):
        """y_t = p_t[e] * expert_e(x_t) with e = argmax of p_t = softmax(R x_t); experts are gated products."""
        GRAPH_SAFE = False   # which rows go to which expert is read on the host

        def __init__(self, hidden_size, intermediate_size, experts):
            self.h, self.i, self.e = hidden_size, intermediate_size, experts

        def tensors(self):
            t = {"router.weight": TensorReq((self.e, self.h), MATRIX)}
            for e in range(self.e):
                t[f"experts.{e}.gate.weight"] = TensorReq((self.i, self.h), MATRIX)
                t[f"experts.{e}.up.weight"] = TensorReq((self.i, self.h), MATRIX)
                t[f"experts.{e}.down.weight"] = TensorReq((self.h, self.i), MATRIX)
            return t

        def load(self, tensors, dtype, device):
            self.router = tensors["router.weight"]
            self.gate_up, self.down = [], []
            for e in range(self.e):
                g, u = tensors[f"experts.{e}.gate.weight"], tensors[f"experts.{e}.up.weight"]
                self.gate_up.append(K.prepare_weight(torch.stack([g, u], dim=1).reshape(2 * self.i, self.h).contiguous()))
                self.down.append(K.prepare_weight(tensors[f"experts.{e}.down.weight"]))

        def forward(self, x):
            p = torch.softmax(K.linear(x, self.router).float(), dim=-1)      # router in 32-bit
            top = p.argmax(dim=-1)
            out = torch.zeros_like(x)
            for e in range(self.e):
                rows = (top == e).nonzero().flatten()
                if rows.numel():
                    y = K.linear(K.linear_silu_mul(x[rows].contiguous(), self.gate_up[e]), self.down[e])
                    out[rows] = (y.float() * p[rows, e:e + 1]).to(x.dtype)
            return out

    @register_part("position", "toy_scaled_rotation")
    class ToyScaledRotation(PositionEncoding):
        """cos/sin of (position / factor) * theta^(-2j/d): what a mixer that rotates expects of a position part
        is ``rotary_dim`` and the two tables [positions, rotary_dim / 2] in float32."""

        def __init__(self, rotary_dim, max_positions, theta, factor):
            self.rotary_dim, self.max_positions, self.theta, self.factor = rotary_dim, max_positions, theta, factor
            self.cos = self.sin = None

        def prepare(self, device):
            j = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64)
            ang = (torch.arange(self.max_positions, dtype=torch.float64) / self.factor).reshape(-1, 1) \
                * (self.theta ** (-j / self.rotary_dim)).reshape(1, -1)
            self.cos, self.sin = torch.cos(ang).float().to(device), torch.sin(ang).float().to(device)

    @dataclasses.dataclass
    class Cfg:
        vocab_size: int
        hidden_size: int
        heads: int
        kv_heads: int
        head_dim: int
        eps: float
        max_positions: int

    def spec(c):
        norm = lambda name: PartSpec("rms_norm", dict(size=c.hidden_size, eps=c.eps), {"weight": name})

        def layer(i):
            ffn_names = {"router.weight": f"l{i}.router"}
            for e in range(E):
                for x in ("gate", "up", "down"):
                    ffn_names[f"experts.{e}.{x}.weight"] = f"l{i}.e{e}.{x}"
            attn_names = {f"{x}_proj.weight": f"l{i}.attn.{x}" for x in "qkvo"}
            attn_names.update({"q_norm.weight": f"l{i}.attn.qn", "k_norm.weight": f"l{i}.attn.kn"})
            return LayerSpec("prenorm", {
                "input_norm": norm(f"l{i}.n1"), "post_mixer_norm": norm(f"l{i}.n2"),
                "mixer": PartSpec("gqa_attention", dict(hidden_size=c.hidden_size, num_heads=c.heads,
                                                        num_kv_heads=c.kv_heads, head_dim=c.head_dim, norm_eps=c.eps,
                                                        qk_norm=True, position="scaled", rotary_dim=ROT), attn_names),
                "ffn": PartSpec("toy_routed", dict(hidden_size=c.hidden_size, intermediate_size=INTER, experts=E),
                                ffn_names)})

        return ModelSpec("ToyRoutedForCausalLM", c.vocab_size, c.hidden_size, c.max_positions, (0,),
                         PartSpec("token_embedding", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size), {"weight": "emb"}),
                         [layer(0), layer(1)], [RunSpec(0), RunSpec(1)], norm("final"),
                         PartSpec("linear_head", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size), {"weight": "head"}),
                         {"scaled": PartSpec("toy_scaled_rotation", dict(rotary_dim=ROT, max_positions=c.max_positions,
                                                                        theta=THETA, factor=FACTOR))})

    register_architecture(Architecture("toy_routed", ("ToyRouted",), ("toy_routed",),
                                       lambda raw: Cfg(**{f.name: raw[f.name] for f in dataclasses.fields(Cfg)}), spec))


RAW = dict(architectures=["ToyRoutedForCausalLM"], vocab_size=61, hidden_size=40, heads=4, kv_heads=2, head_dim=16,
           eps=1e-5, max_positions=96)


def plain(w, toks):
    """The toy model for a whole sequence in float64; returns (logits, the smallest margin by which a router chose)."""
    w = {k: v.double() for k, v in w.items()}
    n = len(toks)
    j = torch.arange(0, ROT, 2, dtype=torch.float64)
    ang = (torch.arange(n, dtype=torch.float64) / FACTOR).reshape(-1, 1) * (THETA ** (-j / ROT)).reshape(1, -1)
    cos, sin = torch.cos(ang).reshape(n, 1, -1), torch.sin(ang).reshape(n, 1, -1)

    def rotate(x):            # the first ROT of each head's 16 elements, as two halves
        a, b, rest = x[..., :ROT // 2], x[..., ROT // 2:ROT], x[..., ROT:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin, rest], dim=-1)

    x = w["emb"][toks]
    margin = float("inf")
    for i in (0, 1):
        p = f"l{i}."
        h = pm.rms_norm(x, w[p + "n1"], 1e-5)
        q = rotate(pm.rms_norm((h @ w[p + "attn.q"].T).reshape(n, 4, 16), w[p + "attn.qn"], 1e-5))
        k = rotate(pm.rms_norm((h @ w[p + "attn.k"].T).reshape(n, 2, 16), w[p + "attn.kn"], 1e-5))
        v = (h @ w[p + "attn.v"].T).reshape(n, 2, 16)
        x = x + pm.attention(q, k, v, 0.25).reshape(n, 64) @ w[p + "attn.o"].T
        h = pm.rms_norm(x, w[p + "n2"], 1e-5)
        pr = torch.softmax(h @ w[p + "router"].T, dim=-1)
        best = torch.sort(pr, dim=-1, descending=True).values
        margin = min(margin, float((best[:, 0] - best[:, 1]).min()))
        top = pr.argmax(dim=-1)
        y = torch.zeros_like(x)
        for t in range(n):
            e = int(top[t])
            y[t] = pr[t, e] * pm.swiglu(h[t:t + 1], w[p + f"e{e}.gate"], w[p + f"e{e}.up"], w[p + f"e{e}.down"])[0]
        x = x + y
    return pm.rms_norm(x, w["final"], 1e-5) @ w["head"].T, margin


def test_routed_ffn_and_another_position_encoding(gpu, tmp_path):
    register_toy_parts()
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    from prelude_amd.weights import WeightFiles, write_random_model
    folder = write_random_model(RAW, str(tmp_path / "toy"), seed=9, std=0.3, norm_std=0.1, dtype=torch.float32)
    files = WeightFiles(folder)
    w = {n: files.tensor(n).clone() for n in files.names()}
    assert len(w) == 3 + 2 * (2 + 6 + 1 + 3 * E)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, 61, (70,), generator=g).tolist()
    ref, margin = plain(w, toks)
    assert margin > 1e-4, "a router nearly tied; take another seed"   # so that 32-bit rounding picks the same expert

    eng = Engine.from_model_dir(folder, EngineConfig(dtype="float32", page_size=8, max_cache_tokens=256))

    def close(got, want):
        assert float((got.double().cpu() - want).abs().max()) < 2e-5 * max(1.0, float(want.abs().max()))

    close(eng.step([StepEntry(0, toks, list(range(70)))]), ref)
    eng.release(0)
    # portions beside a request that feeds single tokens: the experts see other rows each step
    eng.step([StepEntry(1, toks[:30], [])])
    at, got_a, got_b = 0, [], []
    for k, n in enumerate((9, 2, 17, 1, 5, 30, 6)):
        out = eng.step([StepEntry(2, toks[at:at + n], list(range(n))), StepEntry(1, [toks[30 + k]], [0])])
        got_a.append(out[:n]), got_b.append(out[n:])
        at += n
    close(torch.cat(got_a), ref)
    close(torch.cat(got_b), ref[30:37])
    eng.release(1), eng.release(2)
    assert eng.tables.audit() == ""

    # in the serving type such a model is stepped without captured graphs, and generation runs through the entry point
    from prelude_amd import LLM
    llm = LLM(folder, dtype="bfloat16", page_size=8, max_cache_tokens=256)
    assert not llm.engine.model.graph_safe and llm.engine._graphs is None
    outs = llm.generate([toks[:12], toks[20:25]], max_tokens=8, temperature=0.0)
    assert all(len(o.token_ids) == 8 or o.finish_reason == "eos" for o in outs)
    f32 = LLM(folder, dtype="float32", page_size=8, max_cache_tokens=256).generate([toks[:12]], max_tokens=4, temperature=0.0)[0]
    seq = list(toks[:12])
    for tok in f32.token_ids:
        assert tok == int(torch.argmax(plain(w, seq)[0][-1]))
        seq.append(tok)


# ---------------------------------------------------------------------------------------------------------------
# a mixer whose values are narrower than its keys: the pages of its group are shaped by the mixer's own spec
KD, VD = 16, 8


def register_narrow_values():
    from prelude_amd.config.registry import Architecture, register_architecture
    from prelude_amd.models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec
    from prelude_amd.ops import kernels as K
    from prelude_amd.parts import MATRIX, KVCacheSpec, Mixer, TensorReq, register_part

    @register_part("mixer", "toy_narrow_values")
    class ToyNarrowValues(Mixer):
        """One head, no rotation: keys of KD elements, values of VD, both kept in the framework's pages and found
        through the step's block table and slot numbers (plain tensor indexing; it walks the step's host lists)."""
        GRAPH_SAFE = False

        def __init__(self, hidden_size):
            self.hidden_size = hidden_size

        def cache_spec(self):
            return KVCacheSpec(1, KD, 0, value_dim=VD)

        def tensors(self):
            h = self.hidden_size
            return {"q.weight": TensorReq((KD, h), MATRIX), "k.weight": TensorReq((KD, h), MATRIX),
                    "v.weight": TensorReq((VD, h), MATRIX), "o.weight": TensorReq((h, VD), MATRIX)}

        def load(self, tensors, dtype, device):
            self.w = dict(tensors)

        def forward(self, x, step, cache, write_cache=True):
            q, k, v = (K.linear(x, self.w[n + ".weight"]) for n in "qkv")
            grp = step.kv[cache.group]
            page = step.page_size
            assert cache.k.shape[1:] == (1, page, KD) and cache.v.shape[1:] == (1, VD, page)
            slots = grp.slots.to(torch.int64)
            cache.k[slots // page, 0, slots % page] = k
            cache.v[slots // page, 0, :, slots % page] = v
            out = torch.empty((x.shape[0], VD), dtype=x.dtype, device=x.device)
            t = 0
            for i, n in enumerate(step.q_lens):
                ctx = step.starts[i] + n
                pages = grp.block_table[i, :-(-ctx // page)].to(torch.int64)
                keys = cache.k[pages, 0].reshape(-1, KD)[:ctx].float()
                vals = cache.v[pages, 0].permute(0, 2, 1).reshape(-1, VD)[:ctx].float()
                s = q[t:t + n].float() @ keys.T / 4.0
                pos = torch.arange(step.starts[i], ctx, device=x.device).reshape(-1, 1)
                s = s.masked_fill(torch.arange(ctx, device=x.device).reshape(1, -1) > pos, float("-inf"))
                out[t:t + n] = (torch.softmax(s, dim=-1) @ vals).to(x.dtype)
                t += n
            return K.linear(out, self.w["o.weight"])

    @dataclasses.dataclass
    class Cfg:
        vocab_size: int
        hidden_size: int
        inter: int
        eps: float
        max_positions: int

    def spec(c):
        norm = lambda name: PartSpec("rms_norm", dict(size=c.hidden_size, eps=c.eps), {"weight": name})
        layer = LayerSpec("prenorm", {
            "input_norm": norm("n1"), "post_mixer_norm": norm("n2"),
            "mixer": PartSpec("toy_narrow_values", dict(hidden_size=c.hidden_size), {f"{x}.weight": f"mix.{x}" for x in "qkvo"}),
            "ffn": PartSpec("gated_mlp", dict(hidden_size=c.hidden_size, intermediate_size=c.inter),
                            {f"{x}_proj.weight": f"ffn.{x}" for x in ("gate", "up", "down")})})
        return ModelSpec("ToyNarrowForCausalLM", c.vocab_size, c.hidden_size, c.max_positions, (0,),
                         PartSpec("token_embedding", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size), {"weight": "emb"}),
                         [layer], [RunSpec(0)], norm("final"),
                         PartSpec("linear_head", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size), {"weight": "emb"}), {})

    register_architecture(Architecture("toy_narrow", ("ToyNarrow",), ("toy_narrow",),
                                       lambda raw: Cfg(**{f.name: raw[f.name] for f in dataclasses.fields(Cfg)}), spec))


def test_a_mixer_with_values_narrower_than_its_keys(gpu, tmp_path):
    register_narrow_values()
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    from prelude_amd.weights import WeightFiles, write_random_model
    raw = dict(architectures=["ToyNarrowForCausalLM"], vocab_size=53, hidden_size=24, inter=40, eps=1e-5, max_positions=64)
    folder = write_random_model(raw, str(tmp_path / "narrow"), seed=3, std=0.3, norm_std=0.1, dtype=torch.float32)
    files = WeightFiles(folder)
    w = {n: files.tensor(n).double() for n in files.names()}
    toks = torch.randint(0, 53, (45,), generator=torch.Generator().manual_seed(2)).tolist()
    n = len(toks)
    x = w["emb"][toks]
    h = pm.rms_norm(x, w["n1"], 1e-5)
    q, k, v = (h @ w["mix." + c].T for c in "qkv")
    o = pm.attention(q.reshape(n, 1, KD), k.reshape(n, 1, KD), torch.cat([v, torch.zeros(n, KD - VD, dtype=v.dtype)], -1).reshape(n, 1, KD),
                     0.25).reshape(n, KD)[:, :VD]
    x = x + o @ w["mix.o"].T
    x = x + pm.swiglu(pm.rms_norm(x, w["n2"], 1e-5), w["ffn.gate"], w["ffn.up"], w["ffn.down"])
    ref = pm.rms_norm(x, w["final"], 1e-5) @ w["emb"].T

    eng = Engine.from_model_dir(folder, EngineConfig(dtype="float32", page_size=8, max_cache_tokens=128))
    assert eng.caches[0].k.shape[-1] == KD and eng.caches[0].v.shape[-2] == VD
    assert eng.group_specs[0].v_dim == VD

    def close(got, want):
        assert float((got.double().cpu() - want).abs().max()) < 2e-5 * max(1.0, float(want.abs().max()))

    close(eng.step([StepEntry(0, toks, list(range(n)))]), ref)
    eng.release(0)
    at, got = 0, []
    for size in (7, 2, 13, 1, 1, 9, 12):                  # portions and single tokens, across pages of 8
        got.append(eng.step([StepEntry(1, toks[at:at + size], list(range(size)))]))
        at += size
    close(torch.cat(got), ref)
    eng.release(1)
    assert eng.tables.audit() == ""
