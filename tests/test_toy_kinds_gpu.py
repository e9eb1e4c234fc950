"""Three things another architecture could want of the framework's own parts, asked for from outside the package
without editing a file of it: a gated feed-forward with another activation (GELU in its tanh form: one epilogue
code of the same kernels), attention whose scores are capped (cap * tanh(score / cap) before the softmax: one
scalar through the attention kernels), and a mixer that keeps something else than keys and values per token -- one
latent vector -- in pages of a kind of its own, which the cache manager hands out, counts and frees like any
other.  A toy architecture with all three, against its plain form; no model of anyone's.
"""
import dataclasses
import math

import pytest
import torch
import torch.nn.functional as F

import plain_model as pm

pytestmark = pytest.mark.gpu
CAP, LATENT, HD = 1.5, 24, 64


def capped_attention(q, k, v, scale, cap, window=None):
    """``plain_model.attention`` with the scaled scores bent to cap * tanh(s / cap) before the mask."""
    sq, nh, hd = q.shape
    group = nh // k.shape[1]
    out = torch.empty_like(q)
    qi, ki = torch.arange(sq).reshape(sq, 1), torch.arange(sq).reshape(1, sq)
    allowed = ki <= qi
    if window is not None:
        allowed &= ki > qi - window
    for h in range(nh):
        s = (q[:, h] @ k[:, h // group].T) * scale
        s = (cap * torch.tanh(s / cap)).masked_fill(~allowed, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, h // group]
    return out


def register_toy_kinds():
    from prelude_amd.config.registry import Architecture, register_architecture
    from prelude_amd.models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec
    from prelude_amd.ops import kernels as K
    from prelude_amd.parts import MATRIX, Mixer, PagedCacheSpec, TensorReq, register_part

    @dataclasses.dataclass
    class LatentPages:
        data: torch.Tensor      # [pages, page_size, dim]
        group: int

    @dataclasses.dataclass(frozen=True)
    class LatentSpec(PagedCacheSpec):
        """One vector of ``dim`` elements a token: a cache kind the framework does not have."""
        dim: int
        window: int = 0

        def bytes_per_token(self, element_size):
            return self.dim * element_size

        def allocate(self, pages, page_size, dtype, device, group):
            return LatentPages(torch.zeros((pages, page_size, self.dim), dtype=dtype, device=device), group)

    @register_part("mixer", "toy_latent")
    class ToyLatent(Mixer):
        """out_t = W_o sum_j softmax_j(q_t . c_j / sqrt(dim)) c_j over the latents c_j = W_c x_j of the tokens so far."""
        GRAPH_SAFE = False     # it walks the step's host-side lists

        def __init__(self, hidden_size, dim):
            self.h, self.dim = hidden_size, dim

        def cache_spec(self):
            return LatentSpec(self.dim)

        def tensors(self):
            return {"q.weight": TensorReq((self.dim, self.h), MATRIX), "c.weight": TensorReq((self.dim, self.h), MATRIX),
                    "o.weight": TensorReq((self.h, self.dim), MATRIX)}

        def load(self, tensors, dtype, device):
            self.w = dict(tensors)

        def forward(self, x, step, cache, write_cache=True):
            q, c = K.linear(x, self.w["q.weight"]), K.linear(x, self.w["c.weight"])
            grp, page = step.kv[cache.group], step.page_size
            slots = grp.slots.to(torch.int64)
            cache.data[slots // page, slots % page] = c
            out = torch.empty_like(q)
            t = 0
            for i, n in enumerate(step.q_lens):
                ctx = step.starts[i] + n
                pages = grp.block_table[i, :-(-ctx // page)].to(torch.int64)
                lat = cache.data[pages].reshape(-1, self.dim)[:ctx].float()
                s = q[t:t + n].float() @ lat.T / math.sqrt(self.dim)
                pos = torch.arange(step.starts[i], ctx, device=x.device).reshape(-1, 1)
                s = s.masked_fill(torch.arange(ctx, device=x.device).reshape(1, -1) > pos, float("-inf"))
                out[t:t + n] = (torch.softmax(s, dim=-1) @ lat).to(x.dtype)
                t += n
            return K.linear(out, self.w["o.weight"])

    @dataclasses.dataclass
    class Cfg:
        vocab_size: int
        hidden_size: int
        inter: int
        heads: int
        kv_heads: int
        eps: float
        max_positions: int
        window: int

    def spec(c):
        norm = lambda name: PartSpec("rms_norm", dict(size=c.hidden_size, eps=c.eps), {"weight": name})
        ffn = lambda i: PartSpec("gated_mlp", dict(hidden_size=c.hidden_size, intermediate_size=c.inter,
                                                  activation="gelu_tanh"),
                                 {f"{x}_proj.weight": f"l{i}.ffn.{x}" for x in ("gate", "up", "down")})
        attn_names = {f"{x}_proj.weight": f"l0.attn.{x}" for x in "qkvo"}
        attn_names.update({"q_norm.weight": "l0.attn.qn", "k_norm.weight": "l0.attn.kn"})
        capped = LayerSpec("prenorm", {
            "input_norm": norm("l0.n1"), "post_mixer_norm": norm("l0.n2"),
            "mixer": PartSpec("gqa_attention", dict(hidden_size=c.hidden_size, num_heads=c.heads, num_kv_heads=c.kv_heads,
                                                    head_dim=HD, norm_eps=c.eps, qk_norm=True, position="rope",
                                                    window=c.window, score_cap=CAP), attn_names),
            "ffn": ffn(0)})
        latent = LayerSpec("prenorm", {
            "input_norm": norm("l1.n1"), "post_mixer_norm": norm("l1.n2"),
            "mixer": PartSpec("toy_latent", dict(hidden_size=c.hidden_size, dim=LATENT),
                              {f"{x}.weight": f"l1.lat.{x}" for x in "qco"}),
            "ffn": ffn(1)})
        return ModelSpec("ToyKindsForCausalLM", c.vocab_size, c.hidden_size, c.max_positions, (0,),
                         PartSpec("token_embedding", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size), {"weight": "emb"}),
                         [capped, latent], [RunSpec(0), RunSpec(1)], norm("final"),
                         PartSpec("linear_head", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size), {"weight": "head"}),
                         {"rope": PartSpec("rope", dict(rotary_dim=HD, max_positions=c.max_positions, theta=10000.0))})

    register_architecture(Architecture("toy_kinds", ("ToyKinds",), ("toy_kinds",),
                                       lambda raw: Cfg(**{f.name: raw[f.name] for f in dataclasses.fields(Cfg)}), spec))
    return LatentSpec, LatentPages


RAW = dict(architectures=["ToyKindsForCausalLM"], vocab_size=211, hidden_size=128, inter=320, heads=4, kv_heads=2, eps=1e-5,
           max_positions=320, window=0)


def plain(raw, w, toks, cap=CAP, gelu=lambda x: F.gelu(x, approximate="tanh")):
    w = {k: v.double() for k, v in w.items()}
    n = len(toks)
    cos, sin = pm.rope_tables(HD, n, 10000.0)
    ffn = lambda h, p: (gelu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T
    x = w["emb"][toks]
    h = pm.rms_norm(x, w["l0.n1"], 1e-5)
    q = pm.apply_rope(pm.rms_norm((h @ w["l0.attn.q"].T).reshape(n, 4, HD), w["l0.attn.qn"], 1e-5), cos, sin)
    k = pm.apply_rope(pm.rms_norm((h @ w["l0.attn.k"].T).reshape(n, 2, HD), w["l0.attn.kn"], 1e-5), cos, sin)
    v = (h @ w["l0.attn.v"].T).reshape(n, 2, HD)
    o = capped_attention(q, k, v, 1.0 / math.sqrt(HD), cap, raw["window"] or None)
    x = x + o.reshape(n, 4 * HD) @ w["l0.attn.o"].T
    x = x + ffn(pm.rms_norm(x, w["l0.n2"], 1e-5), "l0.ffn.")
    h = pm.rms_norm(x, w["l1.n1"], 1e-5)
    q, c = h @ w["l1.lat.q"].T, h @ w["l1.lat.c"].T
    s = (q @ c.T / math.sqrt(LATENT)).masked_fill(torch.arange(n).reshape(1, n) > torch.arange(n).reshape(n, 1), float("-inf"))
    x = x + (torch.softmax(s, dim=-1) @ c) @ w["l1.lat.o"].T
    x = x + ffn(pm.rms_norm(x, w["l1.n2"], 1e-5), "l1.ffn.")
    return pm.rms_norm(x, w["final"], 1e-5) @ w["head"].T


@pytest.mark.parametrize("dtype,window", [("float32", 0), ("bfloat16", 0), ("bfloat16", 40), ("float32", 40)])
def test_capped_scores_a_gelu_gate_and_a_cache_kind_of_the_mixers_own(gpu, tmp_path, dtype, window):
    LatentSpec, LatentPages = register_toy_kinds()
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    from prelude_amd.weights import WeightFiles, write_random_model
    raw = dict(RAW, window=window)
    stored = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = write_random_model(raw, str(tmp_path / "kinds"), seed=13, std=0.08, norm_std=0.1, dtype=stored)
    files = WeightFiles(folder)
    w = {n: files.tensor(n).clone().float() for n in files.names()}
    toks = torch.randint(0, raw["vocab_size"], (230,), generator=torch.Generator().manual_seed(4)).tolist()
    n = len(toks)
    ref = plain(raw, w, toks)
    eng = Engine.from_model_dir(folder, EngineConfig(dtype=dtype, page_size=16, max_cache_tokens=3 * 256))
    # two groups of pages: the attention's keys and values, and the latent mixer's own kind
    assert len(eng.group_specs) == 2 and isinstance(eng.group_specs[1], LatentSpec) and isinstance(eng.caches[1], LatentPages)
    assert eng.caches[1].data.shape[1:] == (16, LATENT) and eng.caches[1].group == 1
    el = 4 if dtype == "float32" else 2
    from prelude_amd.cache.manager import bytes_per_token
    assert bytes_per_token([c.spec for c in eng.model.cache_slots], eng.dtype) == (2 * 2 * HD + LATENT) * el

    def close(got, want, what):
        err = float((got.double().cpu() - want).abs().max())
        bound = 2e-5 * max(1.0, float(want.abs().max())) if dtype == "float32" else 0.1 * float(want.std())
        assert err <= bound, f"{what}: {err:.3e} > {bound:.3e}"

    # whole (in bfloat16 its 230 rows take the gated product tiled both ways, its activation in that epilogue)
    close(eng.step([StepEntry(0, toks, list(range(n)))]), ref, "whole")
    eng.release(0)
    # portions (the prefill attention) beside a request that feeds single tokens (the decode attention)
    eng.step([StepEntry(1, toks[:150], [])])
    at, got_a, got_b = 0, [], []
    for k, size in enumerate((70, 2, 40, 1, 9, 64, 17, 27)):
        out = eng.step([StepEntry(2, toks[at:at + size], list(range(size))), StepEntry(1, [toks[150 + k]], [0])])
        got_a.append(out[:size]), got_b.append(out[size:])
        at += size
    close(torch.cat(got_a), ref, "portions")
    close(torch.cat(got_b), ref[150:158], "single tokens beside them")
    # single tokens alone: the decode attention that takes the raw projection
    got = [eng.step([StepEntry(1, [toks[158 + k]], [0])]) for k in range(12)]
    close(torch.cat(got), ref[158:170], "single tokens")
    eng.release(1), eng.release(2)
    assert eng.tables.audit() == "" and all(eng.tables.free_pages(g) == eng.pages_per_group[g] for g in range(2))


def test_the_cap_and_the_activation_matter_here():
    """That the toy's logits depend on its cap and its activation (so the agreement above says something): the plain
    form with the cap far away, and with SiLU for GELU, lands elsewhere."""
    raw = dict(RAW)
    w = pm_random(raw)
    toks = torch.randint(0, raw["vocab_size"], (60,), generator=torch.Generator().manual_seed(4)).tolist()
    ref = plain(raw, w, toks)
    assert float((plain(raw, w, toks, cap=1e6) - ref).abs().max()) > 0.2 * float(ref.std())
    assert float((plain(raw, w, toks, gelu=F.silu) - ref).abs().max()) > 0.2 * float(ref.std())


def pm_random(raw):
    g = torch.Generator().manual_seed(13)
    shapes = {"emb": (raw["vocab_size"], 128), "head": (raw["vocab_size"], 128), "final": (128,)}
    for i in (0, 1):
        shapes.update({f"l{i}.n1": (128,), f"l{i}.n2": (128,), f"l{i}.ffn.gate": (320, 128), f"l{i}.ffn.up": (320, 128),
                       f"l{i}.ffn.down": (128, 320)})
    shapes.update({"l0.attn.q": (4 * HD, 128), "l0.attn.k": (2 * HD, 128), "l0.attn.v": (2 * HD, 128), "l0.attn.o": (128, 4 * HD),
                   "l0.attn.qn": (HD,), "l0.attn.kn": (HD,), "l1.lat.q": (LATENT, 128), "l1.lat.c": (LATENT, 128),
                   "l1.lat.o": (128, LATENT)})
    out = {}
    for name, shape in sorted(shapes.items()):
        t = torch.randn(shape, generator=g)
        out[name] = 1 + 0.1 * t if len(shape) == 1 else 0.08 * t
    return out
