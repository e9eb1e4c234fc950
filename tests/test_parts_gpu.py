"""Each part of a layer alone, built through the registry with sizes of its own."""
import math

import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu


def rnd(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def one_sequence_step(gpu, n, page, pages_order, start=0):
    """A StepBatch for one request feeding positions [start, start + n) whose pages are pages_order."""
    from prelude_amd.engine.batch import GroupStep, StepBatch
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    pos = list(range(start, start + n))
    slots = [pages_order[p // page] * page + p % page for p in pos]
    return StepBatch(num_tokens=n, num_seqs=1, token_ids=i32([0] * n), positions=i32(pos), seq_of_token=i32([0] * n),
                     cu_q=i32([0, n]), context_lens=i32([start + n]), state_slots=i32([-1]), fresh=i32([int(start == 0)]),
                     want_rows=i32([n - 1]), kv=[GroupStep(i32([pages_order]), i32(slots))], q_lens=[n], starts=[start],
                     state_slots_host=[-1], fresh_host=[int(start == 0)], max_q_len=n, max_context_len=start + n,
                     page_size=page)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm_part(gpu, dtype):
    from prelude_amd.parts import build_part
    n = build_part("norm", "rms_norm", dict(size=200, eps=2e-5))
    assert n.tensors()["weight"].shape == (200,)
    w = 1 + 0.1 * rnd(200, seed=1)
    n.load({"weight": w.to(gpu)}, dtype, gpu)
    x, r = rnd(7, 200).to(dtype), rnd(7, 200, seed=2).to(dtype)
    tol = 2e-6 if dtype == torch.float32 else 2e-2
    res, h = n.forward_residual(x.to(gpu), None)
    assert torch.equal(res.cpu(), x)                                       # first use: the residual is the input itself
    assert float((h.double().cpu() - pm.rms_norm(x.double(), w.double(), 2e-5)).abs().max()) < tol * 4
    rd = r.to(gpu).clone()
    res, h = n.forward_residual(x.to(gpu), rd)
    s = x.double() + r.double()
    assert res is rd and torch.equal(rd.cpu(), s.to(dtype))
    assert float((h.double().cpu() - pm.rms_norm(s, w.double(), 2e-5)).abs().max()) < tol * 4
    rows = torch.tensor([6, 1], dtype=torch.int32, device=gpu)
    h2 = n.forward_rows(x.to(gpu), r.to(gpu), rows)
    assert float((h2.double().cpu() - pm.rms_norm(s[[6, 1]], w.double(), 2e-5)).abs().max()) < tol * 4


def test_rope_part_tables(gpu):
    from prelude_amd.parts import build_part
    r = build_part("position", "rope", dict(rotary_dim=48, max_positions=300, theta=50000.0))
    r.prepare(gpu)
    cos, sin = pm.rope_tables(48, 300, 50000.0, torch.float32)
    assert r.cos.shape == (300, 24) and r.cos.dtype == torch.float32
    assert float((r.cos.cpu() - cos).abs().max()) < 1e-6 and float((r.sin.cpu() - sin).abs().max()) < 1e-6
    with pytest.raises(Exception, match="even"):
        build_part("position", "rope", dict(rotary_dim=7, max_positions=8, theta=1.0))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_mlp_part(gpu, dtype):
    from prelude_amd.parts import build_part
    m = build_part("ffn", "gated_mlp", dict(hidden_size=72, intermediate_size=200))
    w = {"gate_proj.weight": rnd(200, 72, seed=1, scale=0.1), "up_proj.weight": rnd(200, 72, seed=2, scale=0.1),
         "down_proj.weight": rnd(72, 200, seed=3, scale=0.1)}
    assert {k: v.shape for k, v in m.tensors().items()} == {k: tuple(v.shape) for k, v in w.items()}
    w = {k: v.to(dtype) for k, v in w.items()}
    m.load({k: v.to(gpu) for k, v in w.items()}, dtype, gpu)
    x = rnd(9, 72).to(dtype)
    ref = pm.swiglu(x.double(), *(w[k].double() for k in ("gate_proj.weight", "up_proj.weight", "down_proj.weight")))
    tol = 2e-6 if dtype == torch.float32 else 2e-2
    assert float((m.forward(x.to(gpu)).double().cpu() - ref).abs().max()) < tol * max(1.0, float(ref.abs().max()))
    with pytest.raises(Exception, match="activation"):
        build_part("ffn", "gated_mlp", dict(hidden_size=8, intermediate_size=8, activation="relu"))


@pytest.mark.parametrize("hidden,inter,rows,one_kernel", [(72, 200, 9, False), (2560, 8200, 5, True), (2560, 8200, 17, False)])
def test_gated_mlp_behind_a_norm(gpu, hidden, inter, rows, one_kernel):
    """What a block asks of its feed-forward behind the mixer: (residual + x, forward(norm(residual + x))).  At
    small sizes and at more than 16 rows that is the norm's kernel and then the feed-forward's; a few rows at the
    widths of real models take the add and the norm into the gated product.  Both against the plain functions."""
    from prelude_amd.ops import kernels as K
    from prelude_amd.parts import build_part
    m = build_part("ffn", "gated_mlp", dict(hidden_size=hidden, intermediate_size=inter))
    norm = build_part("norm", "rms_norm", dict(size=hidden, eps=1e-5))
    w = {"gate_proj.weight": rnd(inter, hidden, seed=1, scale=0.03), "up_proj.weight": rnd(inter, hidden, seed=2, scale=0.03),
         "down_proj.weight": rnd(hidden, inter, seed=3, scale=0.03)}
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    gain = 1 + 0.2 * rnd(hidden, seed=4)
    m.load({k: v.to(gpu) for k, v in w.items()}, torch.bfloat16, gpu)
    norm.load({"weight": gain.to(gpu)}, torch.bfloat16, gpu)
    x, res = rnd(rows, hidden, seed=5).to(torch.bfloat16), rnd(rows, hidden, seed=6, scale=4.0).to(torch.bfloat16)
    xd, resd = x.to(gpu), res.to(gpu)
    assert K.gated_after_norm_supported(xd, resd, m.gate_up) == one_kernel
    new_res, y = m.forward_after_norm(xd, resd, norm)
    total = x.double() + res.double()
    ref = pm.swiglu(pm.rms_norm(total, gain.double(), 1e-5), *(w[k].double() for k in ("gate_proj.weight", "up_proj.weight", "down_proj.weight")))
    assert torch.equal(new_res.cpu(), (x.float() + res.float()).to(torch.bfloat16))
    y = K.as_tensor(y)
    assert float((y.double().cpu() - ref).abs().max()) < 2e-2 * max(1.0, float(ref.abs().max()))
    # a norm that is not that formula is never taken in: the plain order, which asks nothing of the norm but its own methods
    class Doubled(type(norm)):
        def as_rms(self):
            return None

        def forward_residual(self, x, residual):
            residual, h = super().forward_residual(x, residual)
            return residual, h * 2
    other = Doubled(hidden, 1e-5)
    other.load({"weight": gain.to(gpu)}, torch.bfloat16, gpu)
    _, y2 = m.forward_after_norm(xd, res.to(gpu), other)
    ref2 = pm.swiglu(2 * pm.rms_norm(total, gain.double(), 1e-5), *(w[k].double() for k in ("gate_proj.weight", "up_proj.weight", "down_proj.weight")))
    assert float((K.as_tensor(y2).double().cpu() - ref2).abs().max()) < 2e-2 * max(1.0, float(ref2.abs().max()))


def test_embedding_and_head_parts(gpu):
    from prelude_amd.parts import build_part
    # crates/prelude-core/tests/modules.rs:245-271: arange(12).reshape(4, 3), ids [2, 0, 3]
    e = build_part("embedding", "token_embedding", dict(vocab_size=4, hidden_size=3))
    table = torch.arange(12, dtype=torch.float32).reshape(4, 3)
    e.load({"weight": table.to(gpu)}, torch.float32, gpu)
    out = e.forward(torch.tensor([2, 0, 3], dtype=torch.int32, device=gpu)).cpu()
    assert out.tolist() == [[6, 7, 8], [0, 1, 2], [9, 10, 11]]
    h = build_part("head", "linear_head", dict(vocab_size=4, hidden_size=3))
    h.load({"weight": table.to(gpu)}, torch.float32, gpu)
    x = rnd(2, 3)
    assert torch.allclose(h.forward(x.to(gpu)).cpu(), x @ table.T, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,bias,window,qk_norm", [(6, 2, 48, True, 0, True), (4, 4, 16, False, 10, True),
                                                            (8, 1, 64, False, 0, False)])
def test_attention_part(gpu, dtype, nh, nkv, hd, bias, window, qk_norm):
    """The mixer alone: projection, QK norm, rotation, cache write, attention, output projection; fed whole
    and fed in two portions through a cache whose pages are out of order."""
    from prelude_amd.cache import KVLayerCache
    from prelude_amd.parts import build_part
    hidden, n, page, eps = 40, 37, 8, 1e-5
    rope = build_part("position", "rope", dict(rotary_dim=hd, max_positions=64, theta=10000.0))
    rope.prepare(gpu)
    a = build_part("mixer", "gqa_attention", dict(hidden_size=hidden, num_heads=nh, num_kv_heads=nkv, head_dim=hd,
                                                  norm_eps=eps, qk_norm=qk_norm, bias=bias, window=window,
                                                  position="rope"))
    a.bind({"rope": rope})
    spec = a.cache_spec()
    assert (spec.num_kv_heads, spec.head_dim, spec.window) == (nkv, hd, window)
    w = {}
    for i, (name, req) in enumerate(a.tensors().items()):
        t = rnd(*req.shape, seed=10 + i, scale=0.15)
        w[name] = (1 + t) if req.kind == "norm" else t
    wd = {k: v.to(dtype if a.tensors()[k].kind == "matrix" else torch.float32) for k, v in w.items()}
    a.load({k: v.to(gpu) for k, v in wd.items()}, dtype, gpu)
    x = rnd(n, hidden).to(dtype)
    # plain: the same formulas through plain_model.attention_block on a one-layer config
    cfg = dict(num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd, attention_bias=bias, rms_norm_eps=eps,
               use_sliding_window=bool(window), sliding_window=window or None, max_window_layers=0)
    pw = {f"model.layers.0.self_attn.{k}": v.double() for k, v in wd.items()}
    if not qk_norm:
        pw["model.layers.0.self_attn.q_norm.weight"] = torch.ones(hd, dtype=torch.float64)
        pw["model.layers.0.self_attn.k_norm.weight"] = torch.ones(hd, dtype=torch.float64)
    cos, sin = pm.rope_tables(hd, 64, 10000.0)
    if qk_norm:
        ref = pm.attention_block(cfg, pw, 0, x.double(), cos[:n], sin[:n])
    else:   # no norm: written out, since plain_model's block always norms
        q = pm.linear(x.double(), pw["model.layers.0.self_attn.q_proj.weight"]).reshape(n, nh, hd)
        k = pm.linear(x.double(), pw["model.layers.0.self_attn.k_proj.weight"]).reshape(n, nkv, hd)
        v = pm.linear(x.double(), pw["model.layers.0.self_attn.v_proj.weight"]).reshape(n, nkv, hd)
        o = pm.attention(pm.apply_rope(q, cos[:n], sin[:n]), pm.apply_rope(k, cos[:n], sin[:n]), v, 1 / math.sqrt(hd))
        ref = pm.linear(o.reshape(n, nh * hd), pw["model.layers.0.self_attn.o_proj.weight"])
    tol = (3e-6 if dtype == torch.float32 else 3e-2) * max(1.0, float(ref.abs().max()))
    pages = [5, 2, 7, 0, 3]
    mk = lambda: KVLayerCache(torch.zeros(8, nkv, page, hd, dtype=dtype, device=gpu),
                              torch.zeros(8, nkv, hd, page, dtype=dtype, device=gpu), 0)
    cache = mk()
    out = a.forward(x.to(gpu), one_sequence_step(gpu, n, page, pages), cache)
    assert float((out.double().cpu() - ref).abs().max()) < tol
    cache2 = mk()
    o1 = a.forward(x[:21].to(gpu), one_sequence_step(gpu, 21, page, pages), cache2)
    o2 = a.forward(x[21:].to(gpu), one_sequence_step(gpu, n - 21, page, pages, start=21), cache2)
    assert float((torch.cat([o1, o2]).double().cpu() - ref).abs().max()) < tol
    if dtype == torch.float32:   # one product kernel whatever the number of rows: the same bits
        assert torch.equal(cache.k, cache2.k) and torch.equal(cache.v, cache2.v)
    else:                        # few rows and many rows take different product kernels: equal to rounding
        assert float((cache.k.float() - cache2.k.float()).abs().max()) < 0.05
        assert float((cache.v.float() - cache2.v.float()).abs().max()) < 0.05
    # reading a cache another run wrote: queries only
    o3 = a.forward(x[21:].to(gpu), one_sequence_step(gpu, n - 21, page, pages, start=21), cache, write_cache=False)
    assert float((o3.double().cpu() - ref[21:]).abs().max()) < tol


def test_prenorm_block(gpu):
    """The arrangement alone, with stand-in parts that make the order of operations visible."""
    from prelude_amd.parts import build_part
    from prelude_amd.parts.base import FeedForward, Mixer, Norm

    class N(Norm):
        def __init__(self, tag):
            self.tag = tag

        def forward_residual(self, x, residual):
            residual = x if residual is None else residual + x
            return residual, residual * self.tag

    class M(Mixer):
        def forward(self, x, step, cache, write_cache=True):
            return x + 1.0

    class Fd(FeedForward):
        def forward(self, x):
            return x * 10.0

    b = build_part("block", "prenorm", {}, input_norm=N(2.0), mixer=M(), post_mixer_norm=N(3.0), ffn=Fd())
    x = torch.ones(2, 4, device=gpu)
    h, r = b.forward(x, None, None, None)
    # residual = x; mixer(2x) = 3; residual = 1 + 3 = 4; ffn(3 * 4) = 120
    assert torch.all(r == 4.0) and torch.all(h == 120.0)
    h2, r2 = b.forward(h, r, None, None)
    # residual = 124; mixer(248) = 249; residual = 373; ffn(1119) = 11190
    assert torch.all(r2 == 373.0) and torch.all(h2 == 11190.0)
