"""Pins for the plain implementation: what fixes each formula besides the reference's
text.  Each check is chosen so that a plausible mistake fails it."""
import math

import numpy as np
import pytest

from tests.helpers import CONFIGS, random_tokens
from tests.plain import qwen3 as plain

rng = np.random.default_rng(0)


def test_rms_norm_closed_form_and_weight():
    # constant vector c with unit weight -> c / sqrt(c^2 + eps); a mean subtraction would give 0
    c, eps = 3.0, 1e-6
    out = plain.rms_norm(np.full((2, 8), c), np.ones(8), eps)
    assert np.allclose(out, c / math.sqrt(c * c + eps), rtol=0, atol=1e-12)
    # the weight multiplies as it is (a "1 + w" convention would double this)
    x = rng.normal(size=(3, 16))
    w = rng.normal(size=16)
    want = x / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-5) * w
    assert np.allclose(plain.rms_norm(x, w, 1e-5), want, atol=1e-12)
    # eps sits inside the square root, added to the mean (not to the root)
    tiny = np.full((1, 4), 1e-4)
    assert np.allclose(plain.rms_norm(tiny, np.ones(4), 1e-6), 1e-4 / math.sqrt(1e-8 + 1e-6))


def test_rope_position_zero_is_identity_and_pairs_keep_their_norm():
    x = rng.normal(size=(2, 5, 16))
    cos, sin = plain.rope_tables([0, 1, 2, 3, 4], 16, 10000.0)
    out = plain.apply_rope(x, cos, sin)
    assert np.allclose(out[:, 0], x[:, 0], atol=1e-12)
    # each (i, i + d/2) pair is rotated: its norm stays
    before = x[..., :8] ** 2 + x[..., 8:] ** 2
    after = out[..., :8] ** 2 + out[..., 8:] ** 2
    assert np.allclose(before, after, atol=1e-9)
    assert not np.allclose(out[:, 3], x[:, 3])


def test_rope_pairs_element_i_with_i_plus_half():
    # A one-hot at element 0 rotates into elements 0 and d/2, not 0 and 1 (interleaved pairing).
    d = 8
    x = np.zeros((1, 1, d))
    x[0, 0, 0] = 1.0
    cos, sin = plain.rope_tables([1], d, 100.0)
    out = plain.apply_rope(x, cos, sin)[0, 0]
    assert np.isclose(out[0], math.cos(1.0)) and np.isclose(out[d // 2], math.sin(1.0))
    assert np.allclose(np.delete(out, [0, d // 2]), 0.0)
    # frequency of pair i is theta^(-2i/d): pair 1 at position 1 turns by 100^(-2/8)
    x[:] = 0
    x[0, 0, 1] = 1.0
    out = plain.apply_rope(x, cos, sin)[0, 0]
    angle = np.float32(100.0) ** np.float32(-2 / 8)
    assert np.isclose(out[1], math.cos(angle), atol=1e-6) and np.isclose(out[1 + d // 2], math.sin(angle), atol=1e-6)


def test_rope_scores_depend_only_on_distance():
    d = 16
    q = rng.normal(size=(1, 1, d))
    k = rng.normal(size=(1, 1, d))

    def score(pq, pk):
        cq, sq = plain.rope_tables([pq], d, 10000.0)
        ck, sk = plain.rope_tables([pk], d, 10000.0)
        return float((plain.apply_rope(q, cq, sq) * plain.apply_rope(k, ck, sk)).sum())

    assert np.isclose(score(7, 3), score(27, 23), atol=1e-5)
    assert not np.isclose(score(7, 3), score(7, 4), atol=1e-3)
    # the sign of the rotation: q later than k by 4 differs from k later than q by 4
    assert not np.isclose(score(7, 3), score(3, 7), atol=1e-3)


def test_attention_reduces_to_library_softmax_without_mask_effects():
    # the last query sees every key: it must equal plain softmax(q k^T * scale) v
    h, t, d = 3, 6, 8
    q, k, v = (rng.normal(size=(h, t, d)) for _ in range(3))
    out = plain.causal_attention(q, k, v, 1 / math.sqrt(d))
    s = (q[:, -1:] @ k.transpose(0, 2, 1)) / math.sqrt(d)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    assert np.allclose(out[:, -1:], p @ v, atol=1e-12)
    # the first query sees only itself: output = v[0] exactly (a mask off by one fails here)
    assert np.allclose(out[:, 0], v[:, 0], atol=1e-12)
    # identical keys -> plain mean of the visible values
    same_k = np.repeat(k[:, :1], t, axis=1)
    out = plain.causal_attention(q, same_k, v, 1 / math.sqrt(d))
    assert np.allclose(out[:, 3], v[:, :4].mean(1), atol=1e-12)


def test_attention_causality_and_window():
    h, t, d = 2, 9, 8
    q, k, v = (rng.normal(size=(h, t, d)) for _ in range(3))
    base = plain.causal_attention(q, k, v, 0.3)
    k2, v2 = k.copy(), v.copy()
    k2[:, 5] += 1.0
    v2[:, 5] -= 2.0
    changed = plain.causal_attention(q, k2, v2, 0.3)
    assert np.allclose(base[:, :5], changed[:, :5], atol=0) and not np.allclose(base[:, 5:], changed[:, 5:])
    # window w: query i sees keys i-w+1 .. i
    win = plain.causal_attention(q, k, v, 0.3, window=3)
    assert np.allclose(win[:, :3], base[:, :3], atol=1e-12)
    s6 = (q[:, 6:7] @ k[:, 4:7].transpose(0, 2, 1)) * 0.3  # query 6 over keys 4, 5, 6 only
    p6 = np.exp(s6 - s6.max(-1, keepdims=True))
    p6 /= p6.sum(-1, keepdims=True)
    assert np.allclose(win[:, 6:7], p6 @ v[:, 4:7], atol=1e-12)


def test_grouped_heads_read_kv_head_h_div_group():
    # per-KV-head distinct constant values: query head h must return the constant of h // group
    heads, kv, t, d = 6, 2, 4, 8
    q = rng.normal(size=(heads, t, d))
    k = rng.normal(size=(kv, t, d))
    v = np.stack([np.full((t, d), 10.0 * (j + 1)) for j in range(kv)])
    out = plain.causal_attention(q, k, v, 0.25)
    for h in range(heads):
        assert np.allclose(out[h], 10.0 * (h // 3 + 1))
    # as many KV heads as query heads is ordinary multi-head attention
    k6, v6 = rng.normal(size=(heads, t, d)), rng.normal(size=(heads, t, d))
    full = plain.causal_attention(q, k6, v6, 0.25)
    for h in range(heads):
        assert np.allclose(full[h], plain.causal_attention(q[h:h + 1], k6[h:h + 1], v6[h:h + 1], 0.25)[0])


def test_gated_feed_forward():
    x = rng.normal(size=(3, 8))
    gate, up, down = rng.normal(size=(12, 8)), rng.normal(size=(12, 8)), rng.normal(size=(8, 12))
    assert np.allclose(plain.gated_feed_forward(x, gate * 0, up, down), 0.0)  # silu(0) = 0
    g = x @ gate.T
    want = ((g / (1 + np.exp(-g))) * (x @ up.T)) @ down.T
    assert np.allclose(plain.gated_feed_forward(x, gate, up, down), want, atol=1e-12)
    # the activation is on the gate, not on up: swapping them changes the result
    assert not np.allclose(plain.gated_feed_forward(x, up, gate, down), want)


def _weights(cfg, seed):
    r = np.random.default_rng(seed)
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    w = {"model.embed_tokens.weight": r.normal(size=(V, H)) * 0.05,
         "model.norm.weight": 1 + 0.2 * r.normal(size=H)}
    if not cfg["tie_word_embeddings"]:
        w["lm_head.weight"] = r.normal(size=(V, H)) * 0.05
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        w[f"{p}.self_attn.q_proj.weight"] = r.normal(size=(nh * hd, H)) * 0.1
        w[f"{p}.self_attn.k_proj.weight"] = r.normal(size=(nkv * hd, H)) * 0.1
        w[f"{p}.self_attn.v_proj.weight"] = r.normal(size=(nkv * hd, H)) * 0.1
        w[f"{p}.self_attn.o_proj.weight"] = r.normal(size=(H, nh * hd)) * 0.1
        w[f"{p}.self_attn.q_norm.weight"] = 1 + 0.2 * r.normal(size=hd)
        w[f"{p}.self_attn.k_norm.weight"] = 1 + 0.2 * r.normal(size=hd)
        w[f"{p}.input_layernorm.weight"] = 1 + 0.2 * r.normal(size=H)
        w[f"{p}.post_attention_layernorm.weight"] = 1 + 0.2 * r.normal(size=H)
        w[f"{p}.mlp.gate_proj.weight"] = r.normal(size=(I, H)) * 0.1
        w[f"{p}.mlp.up_proj.weight"] = r.normal(size=(I, H)) * 0.1
        w[f"{p}.mlp.down_proj.weight"] = r.normal(size=(H, I)) * 0.1
    return w


@pytest.mark.parametrize("name", ["A", "B"])
def test_model_is_causal_and_shift_invariant(name):
    cfg = CONFIGS[name]
    w = _weights(cfg, 1)
    toks = random_tokens(cfg["vocab_size"], 12, 2)
    base = plain.forward(w, cfg, toks)
    assert base.shape == (12, cfg["vocab_size"])
    other = list(toks)
    other[8] = (other[8] + 1) % cfg["vocab_size"]
    changed = plain.forward(w, cfg, other)
    assert np.array_equal(base[:8], changed[:8]) and not np.allclose(base[8:], changed[8:])
    # only distances count: shifting every position by the same amount changes nothing
    shifted = plain.forward(w, cfg, toks, start_position=40)
    assert np.allclose(base, shifted, atol=2e-4 * np.abs(base).max())
    # a prefix of the sequence gives the prefix of the logits
    assert np.allclose(plain.forward(w, cfg, toks[:5]), base[:5], atol=1e-12)


def test_norm_placement_and_head():
    cfg = CONFIGS["B"]
    w = _weights(cfg, 3)
    toks = random_tokens(cfg["vocab_size"], 6, 4)
    base = plain.forward(w, cfg, toks)
    # q/k norms act (a model that skipped them would not notice this change)
    w2 = dict(w)
    w2["model.layers.0.self_attn.k_norm.weight"] = w["model.layers.0.self_attn.k_norm.weight"] * 1.5
    assert not np.allclose(plain.forward(w2, cfg, toks), base)
    # v is not normed: scaling v_proj scales... not invariant (a norm on v would hide the scale)
    w3 = dict(w)
    w3["model.layers.0.self_attn.v_proj.weight"] = w["model.layers.0.self_attn.v_proj.weight"] * 2.0
    assert not np.allclose(plain.forward(w3, cfg, toks), base)
    # q is normed before the rotation: scaling q_proj changes nothing
    w4 = dict(w)
    w4["model.layers.1.self_attn.q_proj.weight"] = w["model.layers.1.self_attn.q_proj.weight"] * 3.0
    assert np.allclose(plain.forward(w4, cfg, toks), base, atol=1e-5)
    # untied: the head is lm_head, not the embedding
    w5 = dict(w)
    w5["lm_head.weight"] = w["lm_head.weight"] * 2.0
    assert np.allclose(plain.forward(w5, cfg, toks), 2.0 * base, atol=1e-12)
    # tied: the embedding is the head
    cfg_a = CONFIGS["A"]
    wa = _weights(cfg_a, 5)
    xa = plain.forward(wa, cfg_a, [1, 2, 3])
    wa2 = dict(wa)
    wa2["lm_head.weight"] = rng.normal(size=wa["model.embed_tokens.weight"].shape)
    assert np.array_equal(plain.forward(wa2, cfg_a, [1, 2, 3]), xa)


def _one_head_attention(cfg, q1, keys, values):
    """``plain.attention_half`` of two tokens at position 0 (no rotation) with projections
    that copy slices of the input: head 0's query is ``q1`` for the second token, the one
    key/value head's keys and values are ``keys`` and ``values``, and the output is head
    0's context.  Unit norm weights.  Returns the second token's context."""
    nh, nkv, hd, H = (cfg[k] for k in ("num_attention_heads", "num_key_value_heads", "head_dim", "hidden_size"))
    assert nkv == 1 and H >= 3 * hd
    eye = np.eye(hd)
    p = "model.layers.0"
    w = {f"{p}.self_attn.q_proj.weight": np.zeros((nh * hd, H)), f"{p}.self_attn.k_proj.weight": np.zeros((hd, H)),
         f"{p}.self_attn.v_proj.weight": np.zeros((hd, H)), f"{p}.self_attn.o_proj.weight": np.zeros((H, nh * hd)),
         f"{p}.self_attn.q_norm.weight": np.ones(hd), f"{p}.self_attn.k_norm.weight": np.ones(hd)}
    w[f"{p}.self_attn.q_proj.weight"][:hd, :hd] = eye          # head 0 of q = h[:, 0:hd]
    w[f"{p}.self_attn.k_proj.weight"][:, hd:2 * hd] = eye       # k = h[:, hd:2hd]
    w[f"{p}.self_attn.v_proj.weight"][:, 2 * hd:3 * hd] = eye   # v = h[:, 2hd:3hd]
    w[f"{p}.self_attn.o_proj.weight"][:hd, :hd] = eye           # out[:, 0:hd] = context of head 0
    h = np.zeros((2, H))
    h[1, :hd] = q1
    h[:, hd:2 * hd] = keys
    h[:, 2 * hd:3 * hd] = values
    out, _ = plain.attention_half(h, w, p, cfg, positions=[0, 0])
    return out[1, :hd]


def test_attention_scale_is_one_over_root_head_dim():
    """B's head size (32) is not hidden / heads (16): a scale taken from the wrong one of the
    two moves the softmax weight of the closed form below from 0.804 to 0.881."""
    cfg = CONFIGS["B"]
    hd, eps = cfg["head_dim"], cfg["rms_norm_eps"]
    assert hd != cfg["hidden_size"] // cfg["num_attention_heads"]
    a = np.ones(hd)
    b = np.ones(hd)
    b[:4] = -1.0  # a . b = hd - 8, both of unit mean square
    values = rng.normal(size=(2, hd))
    got = _one_head_attention(cfg, a, np.stack([b, a]), values)
    # normed vectors are a, b / sqrt(1 + eps); scores differ by (a.a - a.b) / (1 + eps) * scale
    delta = 8.0 / (1.0 + eps) / math.sqrt(hd)
    weight = 1.0 / (1.0 + math.exp(-delta))
    assert np.allclose(got, weight * values[1] + (1 - weight) * values[0], atol=1e-12)
    wrong = 1.0 / (1.0 + math.exp(-8.0 / (1.0 + eps) / math.sqrt(cfg["hidden_size"] // cfg["num_attention_heads"])))
    assert abs(weight - wrong) > 0.05


def test_head_norms_use_the_configurations_eps():
    """A query so small that eps decides its normed length: with B's 1e-5 the softmax weight
    below is 0.605, with a fixed 1e-6 it would be 0.731."""
    cfg = CONFIGS["B"]
    hd, eps = cfg["head_dim"], cfg["rms_norm_eps"]
    assert eps == 1e-5
    t = 1e-3
    a = np.ones(hd)
    b = np.ones(hd)
    b[:4] = -1.0
    values = rng.normal(size=(2, hd))
    got = _one_head_attention(cfg, t * a, np.stack([b, a]), values)
    shrink = t / math.sqrt(t * t + eps)  # the normed query is shrink * a
    delta = shrink * 8.0 / math.sqrt(1.0 + eps) / math.sqrt(hd)
    weight = 1.0 / (1.0 + math.exp(-delta))
    assert np.allclose(got, weight * values[1] + (1 - weight) * values[0], atol=1e-12)
    other = 1.0 / (1.0 + math.exp(-(t / math.sqrt(t * t + 1e-6)) * 8.0 / math.sqrt(1.0 + eps) / math.sqrt(hd)))
    assert abs(weight - other) > 0.05


def test_schedule_names_a_layer_twice_and_borrows_a_cache():
    cfg = CONFIGS["A"]
    w = _weights(cfg, 7)
    toks = random_tokens(cfg["vocab_size"], 7, 8)
    plainly = plain.forward(w, cfg, toks)
    same = plain.forward(w, cfg, toks, schedule=[(0, None), (1, None)])
    assert np.array_equal(plainly, same)
    twice = plain.forward(w, cfg, toks, schedule=[(0, None), (1, None), (0, None)])
    borrow = plain.forward(w, cfg, toks, schedule=[(0, None), (1, 0)])
    assert not np.allclose(twice, plainly) and not np.allclose(borrow, plainly)


def test_top_p_rule_and_sampling():
    logits = np.log(np.array([0.5, 0.3, 0.15, 0.05]))
    # cumulative before each: 0, .5, .8, .95 -> with top_p .8 the third is still kept (.8 > .8 is false)
    p = plain.sampling_distribution(logits, 1.0, 0.8)
    assert np.allclose(p, np.array([0.5, 0.3, 0.15, 0]) / 0.95)
    p = plain.sampling_distribution(logits, 1.0, 0.79)
    assert np.allclose(p, np.array([0.5, 0.3, 0, 0]) / 0.8)
    # the first token is always kept
    p = plain.sampling_distribution(logits, 1.0, 0.01)
    assert np.allclose(p, [1, 0, 0, 0])
    assert np.allclose(plain.sampling_distribution(logits, 1.0, 1.0), [0.5, 0.3, 0.15, 0.05])
    # temperature divides the logits
    assert np.allclose(plain.sampling_distribution(logits, 0.5, 1.0),
                       np.array([0.25, 0.09, 0.0225, 0.0025]) / 0.365)
    assert plain.sample_with_uniform(logits, 0.0, 1.0, 0.99) == 0
    assert plain.sample_with_uniform(logits, 1.0, 1.0, 0.49) == 0
    assert plain.sample_with_uniform(logits, 1.0, 1.0, 0.51) == 1
    assert plain.sample_with_uniform(logits, 1.0, 1.0, 0.96) == 3
    order = np.array([2, 0, 3, 1])  # vocabulary order differs from probability order
    assert plain.sample_with_uniform(logits[order], 1.0, 0.79, 0.1) == 1  # p = [0, .625, 0, .375]
    assert plain.sample_with_uniform(logits[order], 1.0, 0.79, 0.7) == 3
