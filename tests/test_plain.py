"""Pins of the plain implementation: what fixes each formula beside the reference's text.

Each test is chosen so that one plausible misreading (a wrong sign or pairing in the rotation, eps
outside the root, the norm in the wrong place, a wrong head mapping) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from tests.conftest import TINY, plain_random_weights, write_plain_model
from tests.plain import qwen2_plain as P

torch.manual_seed(0)


def plain_cfg(cfg):
    H, nh = cfg["hidden_size"], cfg["num_attention_heads"]
    return {
        "vocab_size": cfg["vocab_size"], "hidden_size": H, "intermediate_size": cfg["intermediate_size"],
        "num_layers": cfg["num_hidden_layers"], "num_heads": nh, "num_kv_heads": cfg["num_key_value_heads"],
        "rms_norm_eps": cfg["rms_norm_eps"], "rope_theta": cfg["rope_theta"],
        "tie_word_embeddings": cfg["tie_word_embeddings"], "head_dim": cfg.get("head_dim") or H // nh,
    }


# ------------------------------------------------------------------ RMSNorm
def test_rms_norm_equals_library_routine():
    x = torch.randn(5, 48, dtype=torch.float64)
    w = torch.randn(48, dtype=torch.float64)
    assert torch.allclose(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5), atol=1e-12)


def test_rms_norm_eps_is_inside_the_root_and_added_to_the_mean():
    # a row far below eps: output = x / sqrt(eps) (eps outside the root or added to the sum gives another value)
    x = torch.full((1, 16), 1e-6, dtype=torch.float64)
    y = P.rms_norm(x, torch.ones(16, dtype=torch.float64), 1e-2)
    assert torch.allclose(y, x / math.sqrt(1e-12 + 1e-2), rtol=1e-9)


def test_rms_norm_scale_invariance_and_no_mean_subtraction():
    x = torch.randn(3, 32, dtype=torch.float64) + 5.0  # a mean that LayerNorm would remove
    w = torch.ones(32, dtype=torch.float64)
    y = P.rms_norm(x, w, 0.0)
    assert torch.allclose(P.rms_norm(7.0 * x, w, 0.0), y, atol=1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(3, dtype=torch.float64), atol=1e-12)
    assert (y.mean(-1) > 0.5).all()


# ------------------------------------------------------------------ rotation
def test_rope_position_zero_is_identity_and_norms_are_kept():
    x = torch.randn(2, 4, 32, dtype=torch.float64)
    cos, sin = P.rope_cos_sin(torch.tensor([0, 3, 100, 8191]), 32, 1e6)
    y = P.apply_rope(x, cos, sin)
    assert torch.allclose(y[:, 0], x[:, 0], atol=1e-15)
    pair = lambda t: t[..., :16] ** 2 + t[..., 16:] ** 2  # pairs (j, j + d/2) keep their length
    assert torch.allclose(pair(y), pair(x), atol=1e-12)


def test_rope_pairs_halves_and_pair_zero_turns_by_the_position():
    d = 16
    e0 = torch.zeros(1, 1, d, dtype=torch.float64)
    e0[..., 0] = 1.0
    cos, sin = P.rope_cos_sin(torch.tensor([1]), d, 10000.0)
    y = P.apply_rope(e0, cos, sin)[0, 0]
    want = torch.zeros(d, dtype=torch.float64)
    want[0], want[d // 2] = math.cos(1.0), math.sin(1.0)  # inv_freq[0] = 1; interleaved pairing would hit index 1
    assert torch.allclose(y, want, atol=1e-15)
    # the sign: a unit vector on the second half turns the other way round into the first half
    e8 = torch.zeros(1, 1, d, dtype=torch.float64)
    e8[..., d // 2] = 1.0
    y = P.apply_rope(e8, cos, sin)[0, 0]
    assert math.isclose(y[0].item(), -math.sin(1.0), abs_tol=1e-15) and math.isclose(y[d // 2].item(), math.cos(1.0), abs_tol=1e-15)


def test_rope_inverse_frequencies():
    f = P.rope_inv_freq(8, 10000.0)
    assert torch.allclose(f, torch.tensor([1.0, 0.1, 0.01, 0.001], dtype=torch.float64), rtol=1e-12)


def test_rope_scores_depend_only_on_distance():
    q = torch.randn(1, 1, 32, dtype=torch.float64)
    k = torch.randn(1, 1, 32, dtype=torch.float64)

    def score(m, n):
        cq, sq = P.rope_cos_sin(torch.tensor([m]), 32, 1e4)
        ck, sk = P.rope_cos_sin(torch.tensor([n]), 32, 1e4)
        return (P.apply_rope(q, cq, sq) * P.apply_rope(k, ck, sk)).sum()

    assert torch.allclose(score(5, 2), score(105, 102), atol=1e-10)
    assert not torch.allclose(score(5, 2), score(5, 3), atol=1e-6)


# ------------------------------------------------------------------ attention
def test_attention_equals_library_routine_without_groups():
    q, k, v = (torch.randn(4, 9, 16, dtype=torch.float64) for _ in range(3))
    want = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    assert torch.allclose(P.causal_attention(q, k, v), want, atol=1e-12)


def test_grouped_heads_use_kv_head_h_div_rep():
    q = torch.randn(6, 7, 16, dtype=torch.float64)
    k, v = (torch.randn(2, 7, 16, dtype=torch.float64) for _ in range(2))
    want = F.scaled_dot_product_attention(
        q[None], k.repeat_interleave(3, 0)[None], v.repeat_interleave(3, 0)[None], is_causal=True)[0]
    assert torch.allclose(P.causal_attention(q, k, v), want, atol=1e-12)
    # a tiled mapping (h % nkv) would differ
    wrong = F.scaled_dot_product_attention(q[None], k.repeat(3, 1, 1)[None], v.repeat(3, 1, 1)[None], is_causal=True)[0]
    assert not torch.allclose(P.causal_attention(q, k, v), wrong, atol=1e-6)


def test_attention_first_token_returns_its_value_and_zero_query_averages_the_visible_rows():
    k, v = (torch.randn(1, 6, 16, dtype=torch.float64) for _ in range(2))
    out = P.causal_attention(torch.zeros(1, 6, 16, dtype=torch.float64), k, v)
    for i in range(6):
        assert torch.allclose(out[0, i], v[0, : i + 1].mean(0), atol=1e-12)
    out = P.causal_attention(torch.randn(1, 6, 16, dtype=torch.float64), k, v)
    assert torch.allclose(out[0, 0], v[0, 0], atol=1e-12)


def test_attention_scale_is_one_over_root_d():
    q, k, v = (torch.randn(1, 3, 64, dtype=torch.float64) for _ in range(3))
    s = (q[0] @ k[0].T) / 8.0
    s = s.masked_fill(torch.triu(torch.ones(3, 3, dtype=torch.bool), 1), float("-inf"))
    assert torch.allclose(P.causal_attention(q, k, v)[0], s.softmax(-1) @ v[0], atol=1e-12)


def test_window_keeps_the_last_w_keys():
    k, v = (torch.randn(1, 8, 16, dtype=torch.float64) for _ in range(2))
    out = P.causal_attention(torch.zeros(1, 8, 16, dtype=torch.float64), k, v, window=3)
    assert torch.allclose(out[0, 7], v[0, 5:8].mean(0), atol=1e-12)
    assert torch.allclose(out[0, 1], v[0, 0:2].mean(0), atol=1e-12)


# ------------------------------------------------------------------ feed-forward, bias, layer order
def test_swiglu_uses_library_silu_on_the_gate_only():
    w = {"gate_proj.weight": torch.randn(12, 8, dtype=torch.float64), "up_proj.weight": torch.randn(12, 8, dtype=torch.float64),
         "down_proj.weight": torch.randn(8, 12, dtype=torch.float64)}
    x = torch.randn(3, 8, dtype=torch.float64)
    want = (F.silu(x @ w["gate_proj.weight"].T) * (x @ w["up_proj.weight"].T)) @ w["down_proj.weight"].T
    assert torch.allclose(P.swiglu_mlp(x, w, ""), want, atol=1e-12)
    swapped = {"gate_proj.weight": w["up_proj.weight"], "up_proj.weight": w["gate_proj.weight"], "down_proj.weight": w["down_proj.weight"]}
    assert not torch.allclose(P.swiglu_mlp(x, swapped, ""), want, atol=1e-6)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_zero_output_projections_leave_embedding_norm_head(name):
    cfg = TINY[name]
    w = plain_random_weights(cfg, 3, dtype=torch.float64)
    for k in w:
        if k.endswith("o_proj.weight") or k.endswith("down_proj.weight"):
            w[k].zero_()
    pc = plain_cfg(cfg)
    ids = [1, 5, 9, 2]
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    want = P.rms_norm(w["model.embed_tokens.weight"][ids], w["model.norm.weight"], cfg["rms_norm_eps"]) @ head.T
    assert torch.allclose(P.forward(w, pc, ids), want, atol=1e-12)


def test_bias_is_added_to_q_k_v_and_not_to_o():
    cfg = dict(TINY["A"])
    pc = plain_cfg(cfg)
    w = plain_random_weights(cfg, 4, dtype=torch.float64)
    p = "model.layers.0.self_attn."
    x = torch.zeros(3, cfg["hidden_size"], dtype=torch.float64)
    cos, sin = P.rope_cos_sin(torch.arange(3), pc["head_dim"], pc["rope_theta"])
    # zero input: q, k are pure (rotated) biases, v is its bias; softmax-weighted mean of equal rows is that row
    out = P.attention_block(x, w, p, pc, cos, sin)
    vb = w[p + "v_proj.bias"].view(pc["num_kv_heads"], pc["head_dim"]).repeat_interleave(2, 0).reshape(-1)
    assert torch.allclose(out, (vb @ w[p + "o_proj.weight"].T).expand(3, -1), atol=1e-12)
    w[p + "v_proj.bias"].zero_()
    assert torch.allclose(P.attention_block(x, w, p, pc, cos, sin), torch.zeros_like(x), atol=1e-15)


def _one_layer(cfg_name="B", seed=6):
    cfg = dict(TINY[cfg_name])
    cfg["num_hidden_layers"] = 1
    return cfg, plain_cfg(cfg), plain_random_weights(cfg, seed, std=0.2, dtype=torch.float64)


def test_each_norm_feeds_its_own_branch_known_answers():
    """One layer, sequences of one token (attention over one key returns its value): with the feed-forward's
    norm scale zeroed the feed-forward adds silu(0) * 0 = 0 and the logits are the attention branch's over
    ``input_layernorm``; with the attention's norm scale zeroed the attention adds o(v's bias) and the
    feed-forward sees ``post_attention_layernorm`` of that sum.  Both answers are written with library routines.
    Dropping a norm, using one scale for both branches or swapping the two fails one of them."""
    cfg, pc, w = _one_layer()
    eps, p = cfg["rms_norm_eps"], "model.layers.0."
    H, nh, nkv, d = cfg["hidden_size"], pc["num_heads"], pc["num_kv_heads"], pc["head_dim"]
    head = w["lm_head.weight"]

    def finish(x):
        return F.linear(F.rms_norm(x, (H,), w["model.norm.weight"], eps), head)

    def value_of(h, wts):   # one key: every query head returns the value of its key/value head
        v = F.linear(h, wts[p + "self_attn.v_proj.weight"], wts[p + "self_attn.v_proj.bias"])
        return F.linear(v.view(nkv, d).repeat_interleave(nh // nkv, 0).reshape(-1), wts[p + "self_attn.o_proj.weight"])

    def mlp(h, wts):
        return F.linear(F.silu(F.linear(h, wts[p + "mlp.gate_proj.weight"])) * F.linear(h, wts[p + "mlp.up_proj.weight"]),
                        wts[p + "mlp.down_proj.weight"])

    for tok in (3, 77):
        x = w["model.embed_tokens.weight"][tok]
        a = {k: v.clone() for k, v in w.items()}
        a[p + "post_attention_layernorm.weight"].zero_()
        want = finish(x + value_of(F.rms_norm(x, (H,), a[p + "input_layernorm.weight"], eps), a))
        assert torch.allclose(P.forward(a, pc, [tok])[0], want, atol=1e-10)
        b = {k: v.clone() for k, v in w.items()}
        b[p + "input_layernorm.weight"].zero_()
        x1 = x + value_of(torch.zeros(H, dtype=torch.float64), b)
        want = finish(x1 + mlp(F.rms_norm(x1, (H,), b[p + "post_attention_layernorm.weight"], eps), b))
        assert torch.allclose(P.forward(b, pc, [tok])[0], want, atol=1e-10)
        assert not torch.allclose(want, finish(x1), atol=1e-4)      # the feed-forward branch is really there
    swapped = dict(w)
    swapped[p + "input_layernorm.weight"], swapped[p + "post_attention_layernorm.weight"] = \
        w[p + "post_attention_layernorm.weight"], w[p + "input_layernorm.weight"]
    ids = [3, 77, 5, 190]
    assert (P.forward(swapped, pc, ids) - P.forward(w, pc, ids)).abs().max() > 1e-3


def test_bias_is_added_before_the_rotation_closed_form():
    """Zero q and k matrices, biases s * e_0 on both: pair 0 (inverse frequency 1) turns by the position, so the
    score of query i against key j is s^2 cos(i - j) / sqrt(d) if and only if the bias is rotated too (added
    after the rotation it would give equal scores and uniform weights).  Values are one-hot rows, so the
    output rows are the softmax weights themselves."""
    d = T = 8
    s = 3.0
    pc = {"num_heads": 1, "num_kv_heads": 1, "head_dim": d}
    e0 = torch.zeros(d, dtype=torch.float64)
    e0[0] = s
    z, eye = torch.zeros(d, d, dtype=torch.float64), torch.eye(d, dtype=torch.float64)
    w = {"q_proj.weight": z, "q_proj.bias": e0, "k_proj.weight": z, "k_proj.bias": e0.clone(),
         "v_proj.weight": eye, "v_proj.bias": torch.zeros(d, dtype=torch.float64), "o_proj.weight": eye}
    cos, sin = P.rope_cos_sin(torch.arange(T), d, 10000.0)
    out = P.attention_block(eye[:T], w, "", pc, cos, sin)
    for i in range(T):
        scores = torch.tensor([s * s * math.cos(i - j) / math.sqrt(d) for j in range(i + 1)], dtype=torch.float64)
        assert torch.allclose(out[i, :i + 1], torch.softmax(scores, 0), atol=1e-12), i
        assert torch.allclose(out[i, i + 1:], torch.zeros(T - i - 1, dtype=torch.float64), atol=1e-15)
    assert not torch.allclose(out[5, :6], torch.full((6,), 1 / 6, dtype=torch.float64), atol=1e-2)


def test_bias_then_rotation_on_non_zero_input_against_complex_arithmetic():
    """The attention block on random input and weights against an independent formulation: biased projections
    from the library's linear, the rotation as a multiplication of the complex numbers (x_j + i x_{j+d/2}) by
    exp(i pos / theta^(2j/d)), the library's causal attention with repeated key/value heads.  Rotating first and
    adding the bias afterwards gives another result."""
    cfg, pc, w = _one_layer("C", seed=8)
    p = "model.layers.0.self_attn."
    T, nh, nkv, d, theta = 9, pc["num_heads"], pc["num_kv_heads"], pc["head_dim"], pc["rope_theta"]
    x = torch.randn(T, cfg["hidden_size"], dtype=torch.float64)
    turn = torch.polar(torch.ones(T, d // 2, dtype=torch.float64),
                       torch.arange(T, dtype=torch.float64)[:, None] * theta ** (-torch.arange(0, d, 2, dtype=torch.float64) / d))

    def rotate(t):      # [T, heads, d]
        c = torch.complex(t[..., :d // 2], t[..., d // 2:]) * turn[:, None, :]
        return torch.cat((c.real, c.imag), dim=-1)

    def block(bias_first):
        q = F.linear(x, w[p + "q_proj.weight"], w[p + "q_proj.bias"] if bias_first else None).view(T, nh, d)
        k = F.linear(x, w[p + "k_proj.weight"], w[p + "k_proj.bias"] if bias_first else None).view(T, nkv, d)
        v = F.linear(x, w[p + "v_proj.weight"], w[p + "v_proj.bias"]).view(T, nkv, d)
        q, k = rotate(q), rotate(k)
        if not bias_first:
            q, k = q + w[p + "q_proj.bias"].view(nh, d), k + w[p + "k_proj.bias"].view(nkv, d)
        k, v = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)
        o = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
        return F.linear(o.transpose(0, 1).reshape(T, nh * d), w[p + "o_proj.weight"])

    cos, sin = P.rope_cos_sin(torch.arange(T), d, theta)
    got = P.attention_block(x, w, p, pc, cos, sin)
    assert torch.allclose(got, block(True), atol=1e-10)
    assert (got - block(False)).abs().max() > 1e-3



# ------------------------------------------------------------------ whole model
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_causality_and_shift_of_all_positions(name):
    cfg = TINY[name]
    pc = plain_cfg(cfg)
    w = plain_random_weights(cfg, 5, std=0.2, dtype=torch.float64)
    ids = torch.randint(0, cfg["vocab_size"], (12,)).tolist()
    full = P.forward(w, pc, ids)
    assert torch.allclose(P.forward(w, pc, ids[:7]), full[:7], atol=1e-10)  # later tokens do not change earlier logits
    assert torch.allclose(P.forward(w, pc, ids, position_offset=37), full, atol=1e-8)  # only distances count
    other = list(ids)
    other[0] = (other[0] + 1) % cfg["vocab_size"]
    assert not torch.allclose(P.forward(w, pc, other)[-1], full[-1], atol=1e-6)  # the far token is seen


def test_reads_a_model_folder(tmp_path):
    cfg = TINY["B"]
    w = plain_random_weights(cfg, 1)
    write_plain_model(tmp_path / "m", cfg, w)
    c = P.read_config(tmp_path / "m")
    assert c["head_dim"] == 32 and c["num_layers"] == 3 and c["tie_word_embeddings"] is False
    w2 = P.read_weights(tmp_path / "m")
    assert set(w2) == set(w)
    assert P.forward(w2, c, [1, 2, 3]).shape == (3, 384)
    c2 = dict(cfg)
    del c2["rope_theta"]
    write_plain_model(tmp_path / "m2", c2, w)
    assert P.read_config(tmp_path / "m2")["rope_theta"] == 10000.0  # the reference's default


def test_greedy_generation_stops_before_the_stop_id():
    cfg = TINY["A"]
    pc = plain_cfg(cfg)
    w = plain_random_weights(cfg, 0, std=0.2, dtype=torch.float64)
    out = P.greedy_generate(w, pc, [3, 4, 5], 8)
    assert len(out) == 8
    stop = out[3]
    assert P.greedy_generate(w, pc, [3, 4, 5], 8, eos_ids=(stop,)) == out[: out.index(stop)]


# ------------------------------------------------------------------ sampler (vectors of the reference's tests/test_sampler.py)
def test_sampler_vectors():
    lg = torch.tensor([[0.1, 2.0, 0.5], [3.0, 0.0, 0.0]])
    assert P.logits_to_probs(lg, 0.0).argmax(-1).tolist() == [1, 0]
    assert P.logits_to_probs(lg, 0.0).sum(-1).tolist() == [1.0, 1.0]
    assert torch.allclose(P.logits_to_probs(lg, 1.0), lg.double().softmax(-1))
    p = P.logits_to_probs(torch.tensor([[0.1, 2.0, 0.5]]), 1.0, top_k=1)
    assert p.tolist() == [[0.0, 1.0, 0.0]]
    p = P.logits_to_probs(torch.tensor([[2.0, 1.0, 0.0, -1.0]]), 1.0, top_p=0.7)
    assert (p > 0).tolist() == [[True, True, False, False]]
    p = P.logits_to_probs(torch.tensor([[10.0, 0.0, 0.0]]), 1.0, top_p=1e-4)
    assert p.tolist() == [[1.0, 0.0, 0.0]]
    p = P.logits_to_probs(torch.randn(1, 50), 1.0, top_k=2)
    assert (p > 0).sum() == 2 and math.isclose(p.sum().item(), 1.0, abs_tol=1e-12)
    p = P.logits_to_probs(torch.tensor([[1.0, 2.0, 3.0]]), 0.5)
    assert torch.allclose(p, torch.tensor([[2.0, 4.0, 6.0]], dtype=torch.float64).softmax(-1))
