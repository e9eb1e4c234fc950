"""Another arrangement of a layer's parts and another norm, asked for from outside the package without editing a
file of it: a block that runs its mixer and its feed-forward side by side on one normed input (x + mixer(n(x)) +
ffn(n(x))) next to a layer of the framework's own pre-norm arrangement, and a norm that subtracts the mean and has a
bias (in the second layer and as the model's final norm, which norms the wanted rows only); an embedding that scales
its rows by the square root of the width, and a head that bends its logits to cap * tanh(logit / cap).  The mixer
and the feed-forward in both layers are the framework's own; a toy architecture, against its plain form; no model of
anyone's.
"""
import dataclasses
import math

import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu
HD = 64
LOGIT_CAP = 3.0


def register_toy_block():
    from prelude_amd.config.registry import Architecture, register_architecture
    from prelude_amd.models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec
    from prelude_amd.ops import kernels as K
    from prelude_amd.parts import MATRIX, NORM, VECTOR, Block, Norm, Part, TensorReq, register_part

    @register_part("embedding", "toy_scaled_embedding")
    class ScaledEmbedding(Part):
        def __init__(self, vocab_size, hidden_size):
            self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)

        def tensors(self):
            return {"weight": TensorReq((self.vocab_size, self.hidden_size), MATRIX)}

        def load(self, tensors, dtype, device):
            self.weight = tensors["weight"]

        def forward(self, token_ids):
            rows = K.embed_gather(token_ids, self.weight)
            return (rows.float() * math.sqrt(self.hidden_size)).to(rows.dtype)

    @register_part("head", "toy_capped_head")
    class CappedHead(Part):
        def __init__(self, vocab_size, hidden_size, cap):
            self.vocab_size, self.hidden_size, self.cap = int(vocab_size), int(hidden_size), float(cap)

        def tensors(self):
            return {"weight": TensorReq((self.vocab_size, self.hidden_size), MATRIX)}

        def load(self, tensors, dtype, device):
            self.weight = K.prepare_weight(tensors["weight"])

        def forward(self, hidden_rows):
            logits = K.linear(hidden_rows, self.weight, out_dtype=torch.float32)
            return self.cap * torch.tanh(logits / self.cap)

    @register_part("norm", "toy_centered_norm")
    class CenteredNorm(Norm):
        """(x - mean) / sqrt(var + eps) * weight + bias, in 32-bit; with a residual the sum is rounded once for the
        residual and normed unrounded, as the framework's own norm does."""

        def __init__(self, size, eps):
            self.size, self.eps = int(size), float(eps)

        def tensors(self):
            return {"weight": TensorReq((self.size,), NORM), "bias": TensorReq((self.size,), VECTOR)}

        def load(self, tensors, dtype, device):
            self.weight, self.bias = tensors["weight"], tensors["bias"]

        def _norm(self, s, dtype):
            s = s - s.mean(-1, keepdim=True)
            return (s * torch.rsqrt((s * s).mean(-1, keepdim=True) + self.eps) * self.weight + self.bias).to(dtype)

        def forward(self, x):
            return self._norm(x.float(), x.dtype)

        def forward_residual(self, x, residual):
            if residual is None:
                return x, self._norm(x.float(), x.dtype)
            s = x.float() + residual.float()
            residual.copy_(s)
            return residual, self._norm(s, x.dtype)

        def forward_rows(self, x, residual, rows):
            rows = rows.long()
            s = x.float()[rows] if residual is None else x.float()[rows] + residual.float()[rows]
            return self._norm(s, x.dtype)

    @register_part("block", "toy_side_by_side")
    class SideBySide(Block):
        """One norm, then the mixer and the feed-forward on the same normed rows; their sum goes on as the hidden
        state, the residual beside it (the add is the next norm's, as everywhere in the framework)."""
        SLOTS = {"norm": "norm", "mixer": "mixer", "ffn": "ffn"}

        def __init__(self, norm, mixer, ffn):
            self.norm, self.mixer, self.ffn = norm, mixer, ffn

        def forward(self, hidden, residual, step, cache, write_cache=True):
            if not self.norm.TAKES_SLICE_SUMS:
                hidden = K.as_tensor(hidden)
            residual, h = self.norm.forward_residual(hidden, residual)
            a = K.as_tensor(self.mixer.forward(h, step, cache, write_cache))
            f = K.as_tensor(self.ffn.forward(h))
            return a + f, residual

    @dataclasses.dataclass
    class Cfg:
        vocab_size: int
        hidden_size: int
        inter: int
        heads: int
        kv_heads: int
        eps: float
        max_positions: int

    def spec(c):
        rms = lambda name: PartSpec("rms_norm", dict(size=c.hidden_size, eps=c.eps), {"weight": name})
        centered = lambda name: PartSpec("toy_centered_norm", dict(size=c.hidden_size, eps=c.eps),
                                         {"weight": name + ".w", "bias": name + ".b"})
        ffn = lambda i: PartSpec("gated_mlp", dict(hidden_size=c.hidden_size, intermediate_size=c.inter),
                                 {f"{x}_proj.weight": f"l{i}.ffn.{x}" for x in ("gate", "up", "down")})

        def attn(i):
            names = {f"{x}_proj.weight": f"l{i}.attn.{x}" for x in "qkvo"}
            names.update({"q_norm.weight": f"l{i}.attn.qn", "k_norm.weight": f"l{i}.attn.kn"})
            return PartSpec("gqa_attention", dict(hidden_size=c.hidden_size, num_heads=c.heads, num_kv_heads=c.kv_heads,
                                                  head_dim=HD, norm_eps=c.eps, qk_norm=True, position="rope"), names)
        first = LayerSpec("prenorm", {"input_norm": rms("l0.n1"), "post_mixer_norm": rms("l0.n2"), "mixer": attn(0), "ffn": ffn(0)})
        second = LayerSpec("toy_side_by_side", {"norm": centered("l1.n"), "mixer": attn(1), "ffn": ffn(1)})
        return ModelSpec("ToyBlockForCausalLM", c.vocab_size, c.hidden_size, c.max_positions, (0,),
                         PartSpec("toy_scaled_embedding", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size), {"weight": "emb"}),
                         [first, second], [RunSpec(0), RunSpec(1), RunSpec(0)], centered("final"),
                         PartSpec("toy_capped_head", dict(vocab_size=c.vocab_size, hidden_size=c.hidden_size, cap=LOGIT_CAP),
                                  {"weight": "head"}),
                         {"rope": PartSpec("rope", dict(rotary_dim=HD, max_positions=c.max_positions, theta=10000.0))})

    register_architecture(Architecture("toy_block", ("ToyBlock",), ("toy_block",),
                                       lambda raw: Cfg(**{f.name: raw[f.name] for f in dataclasses.fields(Cfg)}), spec))


def centered_norm(x, w, b, eps):
    x = x - x.mean(-1, keepdim=True)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w + b


RAW = dict(architectures=["ToyBlockForCausalLM"], vocab_size=173, hidden_size=96, inter=200, heads=3, kv_heads=1, eps=1e-5,
           max_positions=256)


def plain(raw, w, toks, norm=centered_norm, side_by_side=True):
    """x -> pre-norm layer 0 -> side-by-side layer 1 -> layer 0 again (its weights, a cache of its own) -> centered
    final norm -> head, in float64 from the plain implementation's own functions."""
    w = {k: v.double() for k, v in w.items()}
    n = len(toks)
    cos, sin = pm.rope_tables(HD, n, 10000.0)
    eps, nh, nkv = raw["eps"], raw["heads"], raw["kv_heads"]

    def attn(h, p):
        q = pm.apply_rope(pm.rms_norm((h @ w[p + "q"].T).reshape(n, nh, HD), w[p + "qn"], eps), cos, sin)
        k = pm.apply_rope(pm.rms_norm((h @ w[p + "k"].T).reshape(n, nkv, HD), w[p + "kn"], eps), cos, sin)
        v = (h @ w[p + "v"].T).reshape(n, nkv, HD)
        return pm.attention(q, k, v, 1.0 / math.sqrt(HD)).reshape(n, nh * HD) @ w[p + "o"].T

    ffn = lambda h, p: (pm.silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T

    def prenorm(x):
        x = x + attn(pm.rms_norm(x, w["l0.n1"], eps), "l0.attn.")
        return x + ffn(pm.rms_norm(x, w["l0.n2"], eps), "l0.ffn.")
    x = prenorm(w["emb"][toks] * math.sqrt(raw["hidden_size"]))
    h = norm(x, w["l1.n.w"], w["l1.n.b"], eps)
    if side_by_side:
        x = x + attn(h, "l1.attn.") + ffn(h, "l1.ffn.")
    else:
        x = x + attn(h, "l1.attn.")
        x = x + ffn(norm(x, w["l1.n.w"], w["l1.n.b"], eps), "l1.ffn.")
    x = prenorm(x)
    return LOGIT_CAP * torch.tanh(norm(x, w["final.w"], w["final.b"], eps) @ w["head"].T / LOGIT_CAP)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_block_and_a_norm_from_outside_the_package(gpu, tmp_path, dtype):
    register_toy_block()
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    from prelude_amd.weights import WeightFiles, write_random_model
    stored = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = write_random_model(RAW, str(tmp_path / "block"), seed=5, std=0.08, norm_std=0.1, dtype=stored)
    files = WeightFiles(folder)
    w = {n: files.tensor(n).clone().float() for n in files.names()}
    assert {"l1.n.w", "l1.n.b", "final.b"} <= set(w) and "l1.n2" not in " ".join(w)
    toks = torch.randint(0, RAW["vocab_size"], (150,), generator=torch.Generator().manual_seed(8)).tolist()
    n = len(toks)
    ref = plain(RAW, w, toks)
    eng = Engine.from_model_dir(folder, EngineConfig(dtype=dtype, page_size=16, max_cache_tokens=3 * 192))
    assert len(eng.model.cache_slots) == 3        # three runs, a cache each (layer 0 runs twice)

    def close(got, want, what):
        err = float((got.double().cpu() - want).abs().max())
        bound = 2e-5 * max(1.0, float(want.abs().max())) if dtype == "float32" else 0.1 * float(want.std())
        assert err <= bound, f"{what}: {err:.3e} > {bound:.3e}"

    close(eng.step([StepEntry(0, toks, list(range(n)))]), ref, "whole")
    # only some rows wanted: the final norm norms those alone
    close(eng.step([StepEntry(3, toks[:90], [0, 41, 89])]), ref[[0, 41, 89]], "three rows of a prompt")
    eng.release(0), eng.release(3)
    # portions beside single tokens, then single tokens alone (replayed from a graph in bfloat16 if every part allows it)
    eng.step([StepEntry(1, toks[:100], [])])
    at, got_a, got_b = 0, [], []
    for k, size in enumerate((33, 2, 40, 1, 17, 9)):
        out = eng.step([StepEntry(2, toks[at:at + size], list(range(size))), StepEntry(1, [toks[100 + k]], [0])])
        got_a.append(out[:size]), got_b.append(out[size:])
        at += size
    close(torch.cat(got_a), ref[:at], "portions")
    close(torch.cat(got_b), ref[100:106], "single tokens beside them")
    got = [eng.step([StepEntry(1, [toks[106 + k]], [0])]) for k in range(10)]
    close(torch.cat(got), ref[106:116], "single tokens")
    eng.release(1), eng.release(2)
    assert eng.tables.audit() == "" and eng.tables.num_requests() == 0


def test_the_arrangement_and_the_norm_matter_here():
    """The toy's logits depend on how its second layer is arranged and on its norm's centring (so the agreement
    above says something): the plain form with that layer run as a pre-norm one, and with the mean left in, lands
    elsewhere."""
    g = torch.Generator().manual_seed(5)
    h, i = RAW["hidden_size"], RAW["inter"]
    shapes = {"emb": (RAW["vocab_size"], h), "head": (RAW["vocab_size"], h), "final.w": (h,), "final.b": (h,),
              "l0.n1": (h,), "l0.n2": (h,), "l1.n.w": (h,), "l1.n.b": (h,)}
    for l in (0, 1):
        shapes.update({f"l{l}.ffn.gate": (i, h), f"l{l}.ffn.up": (i, h), f"l{l}.ffn.down": (h, i),
                       f"l{l}.attn.q": (3 * HD, h), f"l{l}.attn.k": (HD, h), f"l{l}.attn.v": (HD, h), f"l{l}.attn.o": (h, 3 * HD),
                       f"l{l}.attn.qn": (HD,), f"l{l}.attn.kn": (HD,)})
    w = {}
    for name, shape in sorted(shapes.items()):
        t = torch.randn(shape, generator=g)
        w[name] = (0.1 * t if name.endswith(".b") else 1 + 0.1 * t) if len(shape) == 1 else 0.08 * t
    toks = torch.randint(0, RAW["vocab_size"], (40,), generator=torch.Generator().manual_seed(8)).tolist()
    ref = plain(RAW, w, toks)
    uncentred = lambda x, w_, b, eps: pm.rms_norm(x, w_, eps) + b
    assert float((plain(RAW, w, toks, norm=uncentred) - ref).abs().max()) > 0.1 * float(ref.std())
    assert float((plain(RAW, w, toks, side_by_side=False) - ref).abs().max()) > 0.1 * float(ref.std())
