"""Pins of the plain implementation: what fixes each formula beside the reference's text.

Vectors the reference's own tests hold, special cases that reduce to a library
routine, and invariants, each chosen so that a plausible mistake fails it.
"""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_model as pm

torch.manual_seed(0)
D = torch.float64


# ---- RMSNorm ---------------------------------------------------------------
def test_rmsnorm_reference_vectors():
    # crates/prelude-core/tests/modules.rs:344-365: x=[3,4], w=1 -> x / sqrt(12.5 + eps)
    x = torch.tensor([[3.0, 4.0]], dtype=D)
    y = pm.rms_norm(x, torch.ones(2, dtype=D), 1e-6)
    assert torch.allclose(y, x / math.sqrt(12.5 + 1e-6), atol=1e-12)
    # crates/prelude-core/tests/modules.rs:154: x=[1,2,3,4], mean square 7.5
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]], dtype=D)
    w = torch.tensor([0.5, 1.0, 1.5, 2.0], dtype=D)
    assert torch.allclose(pm.rms_norm(x, w, 1e-5), x / math.sqrt(7.5 + 1e-5) * w, atol=1e-12)


def test_rmsnorm_is_the_library_routine():
    x = torch.randn(5, 96, dtype=D)
    w = torch.randn(96, dtype=D)
    assert torch.allclose(pm.rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5), atol=1e-12)


def test_rmsnorm_invariants():
    x = torch.randn(3, 64, dtype=D)
    one = torch.ones(64, dtype=D)
    y = pm.rms_norm(x, one, 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(3, dtype=D), atol=1e-9)       # unit RMS
    assert torch.allclose(pm.rms_norm(7.0 * x, one, 1e-12), y, atol=1e-9)            # scale of x drops out
    # a mean over the wrong axis or a subtraction of the mean would fail this one
    x = torch.tensor([[2.0, 2.0, 2.0, 2.0]], dtype=D)
    assert torch.allclose(pm.rms_norm(x, torch.ones(4, dtype=D), 0.0), torch.ones(1, 4, dtype=D))


# ---- RoPE ----------------------------------------------------------------------
def _rotate_half(x):
    h = x.shape[-1] // 2
    return torch.cat([-x[..., h:], x[..., :h]], dim=-1)


def test_rope_reference_vector():
    # crates/prelude-core/tests/tensor_ops.rs:1669-1706: l=2, h=2, d=4, x = 0.1 i, cos/sin(0.3 i),
    # expected x * cat(cos, cos) + rotate_half(x) * cat(sin, sin)
    x = (0.1 * torch.arange(16, dtype=D)).reshape(2, 2, 4)
    ang = (0.3 * torch.arange(4, dtype=D)).reshape(2, 2)
    cos, sin = torch.cos(ang), torch.sin(ang)
    want = x * torch.cat([cos, cos], -1)[:, None, :] + _rotate_half(x) * torch.cat([sin, sin], -1)[:, None, :]
    assert torch.allclose(pm.apply_rope(x, cos, sin), want, atol=1e-12)
    # hand value: token 1, head 0: x=[0.8,0.9,1.0,1.1], angles [0.6, 0.9]
    o = pm.apply_rope(x, cos, sin)[1, 0]
    assert abs(o[0] - (0.8 * math.cos(0.6) - 1.0 * math.sin(0.6))) < 1e-12
    assert abs(o[3] - (1.1 * math.cos(0.9) + 0.9 * math.sin(0.9))) < 1e-12


def test_rope_tables_and_invariants():
    cos, sin = pm.rope_tables(8, 64, 10000.0, D)
    assert cos.shape == (64, 4)
    assert torch.allclose(cos[0], torch.ones(4, dtype=D)) and torch.allclose(sin[0], torch.zeros(4, dtype=D))
    # inv_freq_j = theta^(-2j/d): entry [p, j] = cos(p * 10000^(-j/4)) up to the float32 rounding of the angle
    assert abs(float(cos[3, 1]) - math.cos(3 * 10000 ** (-0.25))) < 1e-6
    assert abs(float(sin[5, 0]) - math.sin(5.0)) < 1e-6
    x = torch.randn(64, 3, 8, dtype=D)
    y = pm.apply_rope(x, cos, sin)
    assert torch.allclose(y[0], x[0])                                                  # position 0 is the identity
    # each (j, j + d/2) pair keeps its length: pairing (2j, 2j+1) instead would fail for random x
    assert torch.allclose(y[..., :4] ** 2 + y[..., 4:] ** 2, x[..., :4] ** 2 + x[..., 4:] ** 2, atol=1e-9)


def test_rope_scores_depend_on_distance_only():
    cos, sin = pm.rope_tables(16, 128, 10000.0, D)
    q = torch.randn(1, 1, 16, dtype=D)
    k = torch.randn(1, 1, 16, dtype=D)

    def score(pq, pk):
        qq = pm.apply_rope(q, cos[pq:pq + 1], sin[pq:pq + 1])
        kk = pm.apply_rope(k, cos[pk:pk + 1], sin[pk:pk + 1])
        return float((qq * kk).sum())

    # float32 angles: equal up to the rounding of the table's angles, far below a wrong sign's effect
    assert abs(score(17, 5) - score(57, 45)) < 1e-4
    assert abs(score(17, 5) - score(5, 17)) > 1e-3       # the sign of the rotation matters


# ---- attention -----------------------------------------------------------------
def _sdpa(q, k, v, scale, mask):
    nh, nkv = q.shape[1], k.shape[1]
    kk = k.repeat_interleave(nh // nkv, dim=1).transpose(0, 1)
    vv = v.repeat_interleave(nh // nkv, dim=1).transpose(0, 1)
    o = F.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, attn_mask=mask, scale=scale)
    return o.transpose(0, 1)


@pytest.mark.parametrize("nh,nkv", [(4, 2), (6, 1), (3, 3)])
def test_attention_is_sdpa_with_causal_mask(nh, nkv):
    # crates/prelude-core/tests/tensor_ops.rs:2283-2299: mask c > (sk - sq) + r -> -inf, KV repeat_interleave
    s, hd = 13, 8
    q, k, v = torch.randn(s, nh, hd, dtype=D), torch.randn(s, nkv, hd, dtype=D), torch.randn(s, nkv, hd, dtype=D)
    mask = torch.tril(torch.ones(s, s, dtype=torch.bool))
    got = pm.attention(q, k, v, 0.3)
    assert torch.allclose(got, _sdpa(q, k, v, 0.3, mask), atol=1e-10)


def test_attention_continuation_and_window():
    # the reference's mixed case: q rows are the last rows of a longer context (tests/tensor_ops.rs:2425-2439)
    sk, sq, hd = 20, 5, 8
    q, k, v = torch.randn(sq, 2, hd, dtype=D), torch.randn(sk, 2, hd, dtype=D), torch.randn(sk, 2, hd, dtype=D)
    r = torch.arange(sq).reshape(sq, 1)
    c = torch.arange(sk).reshape(1, sk)
    mask = c <= (sk - sq) + r
    assert torch.allclose(pm.attention(q, k, v, 0.5, q_offset=sk - sq), _sdpa(q, k, v, 0.5, mask), atol=1e-10)
    # window of 4 keys, own included (SlidingWindow{left: 3}, crates/prelude-core/src/models/gemma3.rs:298-301)
    maskw = mask & (c > (sk - sq) + r - 4)
    assert torch.allclose(pm.attention(q, k, v, 0.5, window=4, q_offset=sk - sq), _sdpa(q, k, v, 0.5, maskw), atol=1e-10)
    assert int(maskw.sum(-1).min()) == 4 and int(maskw.sum(-1).max()) == 4


def test_attention_lone_token_and_far_key():
    v = torch.randn(1, 1, 8, dtype=D)
    o = pm.attention(torch.randn(1, 2, 8, dtype=D), torch.randn(1, 1, 8, dtype=D), v, 1.0)
    assert torch.allclose(o[0, 0], v[0, 0]) and torch.allclose(o[0, 1], v[0, 0])       # sees only itself
    # one key made to stand out takes all the weight: the output is its value
    s = 40
    q, k, v = torch.zeros(s, 1, 8, dtype=D), torch.zeros(s, 1, 8, dtype=D), torch.randn(s, 1, 8, dtype=D)
    q[:, 0, 0] = 30.0
    k[3, 0, 0] = 30.0
    o = pm.attention(q, k, v, 1.0)
    assert torch.allclose(o[39, 0], v[3, 0], atol=1e-9) and torch.allclose(o[3, 0], v[3, 0], atol=1e-9)
    assert not torch.allclose(o[2, 0], v[3, 0], atol=1e-3)                             # causal: row 2 cannot see key 3


# ---- feed-forward, linear, embedding ------------------------------------------------
def test_swiglu_reference_vector_and_library():
    # crates/prelude-core/tests/modules.rs:318-327
    g = torch.tensor([0.0, 1.0, -1.0, 2.0, -2.0, 0.5], dtype=D)
    u = torch.tensor([1.0, 2.0, 3.0, 0.5, 1.0, 4.0], dtype=D)
    assert torch.allclose(pm.silu(g) * u, F.silu(g) * u, atol=1e-12)
    assert float(pm.silu(torch.tensor(0.0, dtype=D))) == 0.0
    x = torch.randn(4, 6, dtype=D)
    wg, wu, wd = torch.randn(10, 6, dtype=D), torch.randn(10, 6, dtype=D), torch.randn(6, 10, dtype=D)
    assert torch.allclose(pm.swiglu(x, wg, wu, wd), F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd), atol=1e-10)
    # gate and up swapped would fail:
    assert not torch.allclose(pm.swiglu(x, wg, wu, wd), pm.swiglu(x, wu, wg, wd), atol=1e-3)


def test_linear_is_x_wT():
    x, w, b = torch.randn(3, 5, dtype=D), torch.randn(7, 5, dtype=D), torch.randn(7, dtype=D)
    assert torch.allclose(pm.linear(x, w, b), F.linear(x, w, b), atol=1e-12)


# ---- the whole model ----------------------------------------------------------------
@pytest.fixture(scope="module", params=["a", "b", "c"])
def tiny(request):
    cfg = {"a": pm.tiny_config_a, "b": pm.tiny_config_b, "c": pm.tiny_config_c}[request.param]()
    return cfg, pm.random_weights(cfg, seed=1, std=0.05, norm_std=0.05)


def test_model_is_causal_and_deterministic(tiny):
    cfg, w = tiny
    toks = torch.randint(0, cfg["vocab_size"], (30,)).tolist()
    full = pm.forward(cfg, w, toks)
    assert full.shape == (30, cfg["vocab_size"])
    head = pm.forward(cfg, w, toks[:11])
    assert torch.allclose(full[:11], head, atol=1e-10)          # later tokens do not reach back
    changed = list(toks)
    changed[20] = (changed[20] + 1) % cfg["vocab_size"]
    assert torch.allclose(pm.forward(cfg, w, changed)[:20], full[:20], atol=1e-10)
    assert not torch.allclose(pm.forward(cfg, w, changed)[20:], full[20:], atol=1e-6)


def test_model_shift_of_all_positions(tiny):
    cfg, w = tiny
    toks = torch.randint(0, cfg["vocab_size"], (24,)).tolist()
    a = pm.forward(cfg, w, toks)
    b = pm.forward(cfg, w, toks, position_offset=37)
    # only distances count; the float32 angle table limits how exactly
    assert (a - b).abs().max() < 2e-4 * max(1.0, float(a.abs().max()))


def test_zero_weights_give_zero_logits():
    # the reference's own fixture (crates/prelude-core/src/models/qwen3.rs:915-919)
    cfg = pm.tiny_config_a()
    w = {k: torch.zeros(s) for k, s in pm.tensor_shapes(cfg).items()}
    assert float(pm.forward(cfg, w, [1, 2, 3]).abs().max()) == 0.0


def test_one_layer_by_hand():
    """One layer, one head, written out again without the helper functions: a norm in the
    wrong place (after the rotation, or on V) or a missing residual would differ."""
    cfg = dict(pm.tiny_config_a(), num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1, head_dim=16,
               hidden_size=16, intermediate_size=24, vocab_size=50, tie_word_embeddings=False, eos_token_id=1)
    w = {k: v.double() for k, v in pm.random_weights(cfg, seed=5, std=0.3, norm_std=0.3).items()}
    toks = [3, 9, 27]
    eps = cfg["rms_norm_eps"]
    p = "model.layers.0."

    def norm(x, name):
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w[name]

    x = w["model.embed_tokens.weight"][toks]
    h = norm(x, p + "input_layernorm.weight")
    q = norm(h @ w[p + "self_attn.q_proj.weight"].T, p + "self_attn.q_norm.weight")
    k = norm(h @ w[p + "self_attn.k_proj.weight"].T, p + "self_attn.k_norm.weight")
    v = h @ w[p + "self_attn.v_proj.weight"].T
    inv = torch.tensor([10000.0 ** (-2 * j / 16) for j in range(8)], dtype=D)
    out = torch.zeros(3, 16, dtype=D)

    def rot(vec, pos):
        a = pos * inv
        x1, x2 = vec[:8], vec[8:]
        return torch.cat([x1 * torch.cos(a) - x2 * torch.sin(a), x2 * torch.cos(a) + x1 * torch.sin(a)])

    qr = torch.stack([rot(q[i], i) for i in range(3)])
    kr = torch.stack([rot(k[i], i) for i in range(3)])
    for i in range(3):
        s = torch.stack([qr[i] @ kr[j] / 4.0 for j in range(i + 1)])
        pr = torch.exp(s - s.max())
        pr = pr / pr.sum()
        out[i] = sum(pr[j] * v[j] for j in range(i + 1))
    x = x + out @ w[p + "self_attn.o_proj.weight"].T
    h = norm(x, p + "post_attention_layernorm.weight")
    g = h @ w[p + "mlp.gate_proj.weight"].T
    x = x + ((g / (1 + torch.exp(-g))) * (h @ w[p + "mlp.up_proj.weight"].T)) @ w[p + "mlp.down_proj.weight"].T
    want = norm(x, "model.norm.weight") @ w["lm_head.weight"].T
    got = pm.forward(cfg, w, toks)
    assert torch.allclose(got, want, atol=1e-5)     # the angle goes through float32 in the plain implementation


def _library_model(cfg, w, toks):
    """The whole decoder put together from library routines only (``F.embedding``, ``F.linear``, ``F.rms_norm``,
    ``F.silu``, ``F.scaled_dot_product_attention`` with its own default scale and its own causal mask,
    ``repeat_interleave`` for the grouped heads) and the rotation in the form the reference's test fixes,
    x * cat(cos, cos) + rotate_half(x) * cat(sin, sin) (crates/prelude-core/tests/tensor_ops.rs:1684-1691).  It
    shares no function with the plain implementation: what it pins is the wiring -- which norm goes where, that
    values are not normed, the scale 1 / sqrt(head_dim), both residual sums, the final norm, the head."""
    w = {k: v.double() for k, v in w.items()}
    nh, nkv, hd, hid = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["hidden_size"]
    eps, bias = cfg["rms_norm_eps"], cfg["attention_bias"]
    toks = torch.as_tensor(toks)
    s = toks.shape[0]
    # the angle in 32-bit, as the reference forms it (crates/prelude-core/src/models/commons/attn_utils.rs:39-49)
    inv_freq = (1.0 / torch.tensor(cfg["rope_theta"], dtype=D).pow(torch.arange(0, hd, 2, dtype=D) / hd).float()).float()
    ang = torch.outer(torch.arange(s, dtype=torch.float32), inv_freq).double()
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1)[:, None, :], torch.cat([ang.sin(), ang.sin()], -1)[:, None, :]
    x = F.embedding(toks, w["model.embed_tokens.weight"])
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = p + "self_attn."
        b = (lambda n: w[a + n + ".bias"]) if bias else (lambda n: None)
        h = F.rms_norm(x, (hid,), w[p + "input_layernorm.weight"], eps)
        q = F.linear(h, w[a + "q_proj.weight"], b("q_proj")).view(s, nh, hd)
        k = F.linear(h, w[a + "k_proj.weight"], b("k_proj")).view(s, nkv, hd)
        v = F.linear(h, w[a + "v_proj.weight"], b("v_proj")).view(s, nkv, hd)
        q = F.rms_norm(q, (hd,), w[a + "q_norm.weight"], eps)
        k = F.rms_norm(k, (hd,), w[a + "k_norm.weight"], eps)
        q = q * cos + _rotate_half(q) * sin
        k = k * cos + _rotate_half(k) * sin
        k, v = k.repeat_interleave(nh // nkv, dim=1), v.repeat_interleave(nh // nkv, dim=1)
        window = pm.layer_window(cfg, i)
        if window is None:
            o = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
        else:
            r, c = torch.arange(s)[:, None], torch.arange(s)[None, :]
            o = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                               attn_mask=(c <= r) & (c > r - window))
        x = x + F.linear(o.transpose(0, 1).reshape(s, nh * hd), w[a + "o_proj.weight"], b("o_proj"))
        h = F.rms_norm(x, (hid,), w[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]),
                         w[p + "mlp.down_proj.weight"])
    x = F.rms_norm(x, (hid,), w["model.norm.weight"], eps)
    return F.linear(x, w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"])


def test_model_is_the_library_routines_wired_together(tiny):
    cfg, w = tiny
    toks = torch.randint(0, cfg["vocab_size"], (60,)).tolist()
    got, want = pm.forward(cfg, w, toks), _library_model(cfg, w, toks)
    assert float((got - want).abs().max()) < 1e-9 * max(1.0, float(want.abs().max()))
    # each of these plausible mistakes moves the library model's logits by far more than that bound, so the
    # agreement above is not one that any wiring would reach
    p = "model.layers.0.self_attn."
    swapped = dict(w)
    swapped[p + "q_norm.weight"], swapped[p + "k_norm.weight"] = w[p + "k_norm.weight"], w[p + "q_norm.weight"]
    assert float((_library_model(cfg, swapped, toks) - want).abs().max()) > 1e-5


def _attention_block_inputs(cfg, seed):
    w = {k: v.double() for k, v in pm.random_weights(cfg, seed=seed, std=0.3, norm_std=0.3).items()}
    h = torch.randn(9, cfg["hidden_size"], dtype=D)
    cos_t, sin_t = pm.rope_tables(cfg["head_dim"], 16, cfg["rope_theta"], D)
    return w, h, cos_t[:9], sin_t[:9]


def test_values_are_not_normed():
    """Scaling W_v by c scales the block's output by c (o_proj is linear): a norm on V would undo the scale."""
    cfg = dict(pm.tiny_config_b(), num_hidden_layers=1)
    w, h, cos, sin = _attention_block_inputs(cfg, 3)
    base = pm.attention_block(cfg, w, 0, h, cos, sin)
    w2 = dict(w)
    w2["model.layers.0.self_attn.v_proj.weight"] = 3.0 * w["model.layers.0.self_attn.v_proj.weight"]
    assert torch.allclose(pm.attention_block(cfg, w2, 0, h, cos, sin), 3.0 * base, atol=1e-10)
    # ... while queries and keys are: scaling W_q or W_k changes nothing (up to eps)
    for name in ("q_proj", "k_proj"):
        w3 = dict(w)
        w3[f"model.layers.0.self_attn.{name}.weight"] = 5.0 * w[f"model.layers.0.self_attn.{name}.weight"]
        assert torch.allclose(pm.attention_block(cfg, w3, 0, h, cos, sin), base, rtol=1e-4, atol=1e-4)


def test_heads_are_independent_and_keep_their_kv_head():
    """With o_proj the identity the block's output is the heads side by side.  Exchanging two query heads of one
    KV head exchanges their outputs and touches no other head; exchanging the two KV heads exchanges the outputs of
    their groups only if the query heads go with them."""
    cfg = dict(pm.tiny_config_a(), num_hidden_layers=1)              # 4 heads over 2 KV heads, 4 * 16 = hidden
    w, h, cos, sin = _attention_block_inputs(cfg, 4)
    p = "model.layers.0.self_attn."
    w[p + "o_proj.weight"] = torch.eye(64, dtype=D)
    base = pm.attention_block(cfg, w, 0, h, cos, sin).reshape(9, 4, 16)
    w2 = dict(w)
    wq = w[p + "q_proj.weight"].reshape(4, 16, 64)
    w2[p + "q_proj.weight"] = wq[[1, 0, 2, 3]].reshape(64, 64)       # heads 0 and 1 share KV head 0
    out = pm.attention_block(cfg, w2, 0, h, cos, sin).reshape(9, 4, 16)
    assert torch.allclose(out, base[:, [1, 0, 2, 3]], atol=1e-12)
    w3 = dict(w)
    w3[p + "q_proj.weight"] = wq[[2, 3, 0, 1]].reshape(64, 64)       # the groups exchanged, KV heads with them
    for name in ("k_proj", "v_proj"):
        w3[p + name + ".weight"] = w[p + name + ".weight"].reshape(2, 16, 64)[[1, 0]].reshape(32, 64)
    out = pm.attention_block(cfg, w3, 0, h, cos, sin).reshape(9, 4, 16)
    assert torch.allclose(out, base[:, [2, 3, 0, 1]], atol=1e-12)
    w4 = dict(w3)
    w4[p + "q_proj.weight"] = w[p + "q_proj.weight"]                 # KV heads exchanged alone: other results
    assert not torch.allclose(pm.attention_block(cfg, w4, 0, h, cos, sin).reshape(9, 4, 16), base, atol=1e-3)


def test_tied_head_uses_the_embedding():
    cfg = pm.tiny_config_a()
    w = pm.random_weights(cfg, seed=2)
    assert "lm_head.weight" not in w
    a = pm.forward(cfg, w, [1, 2, 3])
    cfg2 = dict(cfg, tie_word_embeddings=False)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    assert torch.allclose(a, pm.forward(cfg2, w2, [1, 2, 3]))


def test_greedy_prefers_the_lowest_index_on_ties():
    # crates/prelude-core/src/engine/sampling/logits_processor.rs:144-149
    assert int(torch.argmax(torch.tensor([0.1, 0.2, 0.9, 0.3]))) == 2
    assert int(torch.argmax(torch.tensor([0.9, 0.2, 0.9, 0.3]))) == 0


# ---- sampling -----------------------------------------------------------------------
def test_sampling_distribution_rules():
    logits = torch.tensor([2.0, 1.0, 0.5, -1.0, 0.0])
    p = pm.sampling_probs(logits, 0.8)
    assert abs(float(p.sum()) - 1.0) < 1e-12 and torch.allclose(p, torch.softmax(logits.double() / 0.8, -1))
    p2 = pm.sampling_probs(logits, 1.0, top_k=2)
    assert (p2 > 0).tolist() == [True, True, False, False, False]
    full = torch.softmax(logits.double(), -1)
    p3 = pm.sampling_probs(logits, 1.0, top_p=float(full[0]) + 1e-9)    # the first alone is just short of p
    assert (p3 > 0).tolist() == [True, True, False, False, False]
    p4 = pm.sampling_probs(logits, 1.0, top_p=float(full[0]) - 1e-9)
    assert (p4 > 0).tolist() == [True, False, False, False, False]
    # low temperature approaches the argmax
    assert int(torch.argmax(pm.sampling_probs(logits, 1e-3))) == 0 and float(pm.sampling_probs(logits, 1e-3)[0]) > 0.999
    assert pm.draw(torch.tensor([0.25, 0.25, 0.5]), 0.1) == 0
    assert pm.draw(torch.tensor([0.25, 0.25, 0.5]), 0.3) == 1
    assert pm.draw(torch.tensor([0.25, 0.25, 0.5]), 0.99) == 2
    assert pm.draw(torch.tensor([0.0, 1.0, 0.0]), 0.0) == 1
