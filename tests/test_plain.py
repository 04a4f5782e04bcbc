"""What fixes the plain implementation beside the reference's text: vectors that the reference's own
tests hold, special cases that reduce to a library routine, and invariants - each chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place, a wrong head mapping) fails."""
import math

import pytest
import torch
import torch.nn.functional as F

from conftest import TINY_A, TINY_B, token_ids
from plain import qwen3_plain as P

DT = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=DT)


# ------------------------------------------------------------------ attention
def test_attention_reference_vector_single_head():
    """reference: tests/ops/test_mha.cpp:118-156"""
    q = torch.tensor([[[1.0, 0, 0, 0]]], dtype=DT)
    k = torch.tensor([[[1.0, 0, 0, 0]]], dtype=DT)
    v = torch.tensor([[[2.0, 3, 4, 5]]], dtype=DT)
    assert torch.allclose(P.causal_attention(q, k, v, 0.5), v)


def test_attention_reference_vector_gqa_head_mapping():
    """reference: tests/ops/test_mha.cpp:196-240 - heads 0,1 read kv head 0, heads 2,3 read kv head 1."""
    q = torch.tensor([[[1.0, 0], [0, 1], [1, 1], [-1, 1]]], dtype=DT)
    k = torch.tensor([[[1.0, 0], [0, 1]]], dtype=DT)
    v = torch.tensor([[[10.0, 20], [30, 40]]], dtype=DT)
    out = P.causal_attention(q, k, v, 2 ** -0.5)
    assert torch.allclose(out[0], torch.tensor([[10.0, 20], [10, 20], [30, 40], [30, 40]], dtype=DT))


def test_attention_reference_case_two_heads_position_one():
    """reference: tests/ops/test_mha.cpp:158-194, against a softmax written out here."""
    q = torch.tensor([[[0.0, 0], [0, 0]], [[1.0, 0], [0, 1]]], dtype=DT)      # only position 1 is checked
    k = torch.tensor([[[1.0, 0], [0, 1]], [[0.0, 1], [1, 0]]], dtype=DT)
    v = torch.tensor([[[2.0, 3], [4, 5]], [[6.0, 7], [8, 9]]], dtype=DT)
    out = P.causal_attention(q, k, v, 2 ** -0.5)[1]
    for h in range(2):
        s = torch.tensor([float(q[1, h] @ k[j, h]) * 2 ** -0.5 for j in range(2)], dtype=DT)
        w = torch.exp(s - s.max())
        w = w / w.sum()
        assert torch.allclose(out[h], w[0] * v[0, h] + w[1] * v[1, h])


def test_attention_equals_library_sdpa_without_rotation():
    t, nq, nkv, d = 9, 6, 2, 8
    q, k, v = rnd(t, nq, d, seed=1), rnd(t, nkv, d, seed=2), rnd(t, nkv, d, seed=3)
    kk = k.repeat_interleave(nq // nkv, dim=1)       # consecutive query heads share a kv head
    vv = v.repeat_interleave(nq // nkv, dim=1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True,
                                          scale=0.3).transpose(0, 1)
    assert torch.allclose(P.causal_attention(q, k, v, 0.3), want, atol=1e-12)


def test_attention_window_equals_masked_sdpa_and_full_when_wide():
    t, nq, nkv, d, w = 12, 2, 1, 4, 5
    q, k, v = rnd(t, nq, d, seed=4), rnd(t, nkv, d, seed=5), rnd(t, nkv, d, seed=6)
    i = torch.arange(t)
    mask = (i[None, :] <= i[:, None]) & (i[None, :] > i[:, None] - w)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(2, 1).transpose(0, 1),
                                          v.repeat_interleave(2, 1).transpose(0, 1), attn_mask=mask,
                                          scale=0.5).transpose(0, 1)
    assert torch.allclose(P.causal_attention(q, k, v, 0.5, window=w), want, atol=1e-12)
    assert torch.allclose(P.causal_attention(q, k, v, 0.5, window=t), P.causal_attention(q, k, v, 0.5))
    # a window of one sees only the token's own value
    assert torch.allclose(P.causal_attention(q, k, v, 0.5, window=1), v.repeat_interleave(2, 1))


def test_attention_far_key_dominates_when_its_score_stands_out():
    t, d = 300, 8
    q, k, v = rnd(t, 1, d, seed=7) * 0.1, rnd(t, 1, d, seed=8) * 0.1, rnd(t, 1, d, seed=9)
    k[3, 0] = 0.0
    k[3, 0, 0] = 40.0
    q[-1, 0, 0] = 40.0
    out = P.causal_attention(q, k, v, 1.0)
    assert torch.allclose(out[-1, 0], v[3, 0], atol=1e-9)


# ----------------------------------------------------------------------- rope
def test_rope_is_complex_multiplication_of_adjacent_pairs():
    """Adjacent pairing (2i, 2i+1): x viewed as complex numbers times e^{i angle}.  The half-split pairing
    (i, i + d/2) is a different function and must differ."""
    t, h, d, theta = 5, 3, 8, 1e4
    x = rnd(t, h, d, seed=10)
    pos = [0, 1, 7, 100, 4095]
    angle = torch.tensor(pos, dtype=DT)[:, None] / theta ** (torch.arange(0, d, 2, dtype=DT) / d)
    want = torch.view_as_real(torch.view_as_complex(x.reshape(t, h, d // 2, 2).contiguous())
                              * torch.polar(torch.ones_like(angle), angle)[:, None, :]).reshape(t, h, d)
    got = P.rope(x, pos, theta)
    assert torch.allclose(got, want, atol=1e-12)
    assert not torch.allclose(P.rope(x, pos, theta, pairing="half"), want, atol=1e-3)
    assert torch.allclose(got[0], x[0])                                  # position 0 is the identity
    assert torch.allclose(got.norm(dim=-1), x.norm(dim=-1))              # rotations keep lengths


def test_rope_sign_of_the_rotation():
    """(1, 0) at angle a becomes (cos a, sin a): reference src/ops/rope.cpp:63-66."""
    x = torch.tensor([[[1.0, 0.0]]], dtype=DT)
    out = P.rope(x, [1], 10.0)          # d = 2: exponent 0, angle = 1
    assert torch.allclose(out[0, 0], torch.tensor([math.cos(1.0), math.sin(1.0)], dtype=DT))


def test_rope_scores_depend_only_on_distance():
    d, theta = 16, 1e6
    q, k = rnd(1, 1, d, seed=11), rnd(1, 1, d, seed=12)
    def score(m, n):
        return float((P.rope(q, [m], theta) * P.rope(k, [n], theta)).sum())
    assert abs(score(9, 4) - score(105, 100)) < 1e-9
    assert abs(score(9, 4) - score(4, 9)) > 1e-3                          # direction matters


def test_rope_partial_dimension_leaves_the_tail():
    """reference: tests/ops/test_rope.cpp:224-240"""
    x = rnd(2, 4, 8, seed=13)
    out = P.rope(x, [2, 3], 5000.0, rotary_dim=4)
    assert torch.equal(out[..., 4:], x[..., 4:]) and not torch.allclose(out[..., :4], x[..., :4])
    assert torch.allclose(out[..., :4], P.rope(x[..., :4].contiguous(), [2, 3], 5000.0))


# ------------------------------------------------------------- norms and mlp
def test_rms_norm_special_cases():
    x = rnd(4, 33, seed=14)
    one = torch.ones(33, dtype=DT)
    y = P.rms_norm(x, one, 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(4, dtype=DT))      # unit root-mean-square
    assert torch.allclose(P.rms_norm(3.0 * x, one, 0.0), y)               # scale invariance without eps
    w = rnd(33, seed=15)
    assert torch.allclose(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (33,), w, 1e-5), atol=1e-12)
    # the weight multiplies after the normalisation: norm(x) * w, not norm(x * w)
    assert not torch.allclose(P.rms_norm(x, w, 1e-5), P.rms_norm(x * w, one, 1e-5), atol=1e-3)
    # eps sits inside the root
    tiny = torch.full((1, 4), 1e-4, dtype=DT)
    assert torch.allclose(P.rms_norm(tiny, torch.ones(4, dtype=DT), 1e-6), tiny / math.sqrt(1e-8 + 1e-6))


def test_silu_and_gated_mlp():
    x = rnd(3, 7, seed=16)
    assert torch.allclose(P.silu(x), F.silu(x), atol=1e-12) and P.silu(torch.zeros(1, dtype=DT)).item() == 0.0
    assert abs(P.silu(torch.tensor([30.0], dtype=DT)).item() - 30.0) < 1e-9
    assert abs(P.silu(torch.tensor([-30.0], dtype=DT)).item()) < 1e-9
    wg, wu, wd = rnd(5, 7, seed=17), rnd(5, 7, seed=18), rnd(7, 5, seed=19)
    want = (F.silu(x @ wg.T) * (x @ wu.T)) @ wd.T                         # the activation is on the gate, not on up
    assert torch.allclose(P.gated_mlp(x, wg, wu, wd), want, atol=1e-12)


def test_linear_and_embedding():
    x, w = rnd(4, 6, seed=20), rnd(3, 6, seed=21)
    assert torch.allclose(P.linear(x, w), F.linear(x, w))                 # weight stored [out, in]
    table = rnd(10, 6, seed=22)
    assert torch.equal(P.embedding(table, [3, 0, 3]), table[[3, 0, 3]])


# ------------------------------------------------------------------ the model
def test_whole_model_is_causal_and_ties_the_head(plain_models):
    a = plain_models["A"]
    ids = token_ids(TINY_A["vocab_size"], 20, 5)
    full = a.logits(ids)
    assert torch.allclose(full[:12], a.logits(ids[:12]), atol=1e-10)      # later tokens change nothing earlier
    assert "lm_head.weight" not in a.w
    untied = P.PlainQwen3(dict(a.c, tie_word_embeddings=False),
                          dict(a.w, **{"lm_head.weight": a.w["model.embed_tokens.weight"].clone()}))
    assert torch.allclose(untied.logits(ids), full)
    with pytest.raises(KeyError):
        P.PlainQwen3(dict(a.c, tie_word_embeddings=False), a.w).logits(ids)


def test_one_layer_by_hand(plain_models):
    """The order of operations of a layer, spelled out with library routines."""
    b = plain_models["B"]
    c, w = b.c, b.w
    ids = token_ids(c["vocab_size"], 6, 6)
    h = w["model.embed_tokens.weight"][ids]
    p = "model.layers.0."
    nq, nkv, d, eps = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"], c["rms_norm_eps"]
    a = F.rms_norm(h, (h.shape[1],), w[p + "input_layernorm.weight"], eps)
    q = F.rms_norm((a @ w[p + "self_attn.q_proj.weight"].T).view(6, nq, d), (d,), w[p + "self_attn.q_norm.weight"], eps)
    k = F.rms_norm((a @ w[p + "self_attn.k_proj.weight"].T).view(6, nkv, d), (d,), w[p + "self_attn.k_norm.weight"], eps)
    v = (a @ w[p + "self_attn.v_proj.weight"].T).view(6, nkv, d)
    pos = list(range(6))
    q, k = P.rope(q, pos, c["rope_theta"]), P.rope(k, pos, c["rope_theta"])
    o = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(nq // nkv, 1).transpose(0, 1),
                                       v.repeat_interleave(nq // nkv, 1).transpose(0, 1), is_causal=True).transpose(0, 1)
    h = h + o.reshape(6, nq * d) @ w[p + "self_attn.o_proj.weight"].T
    m = F.rms_norm(h, (h.shape[1],), w[p + "post_attention_layernorm.weight"], eps)
    h = h + (F.silu(m @ w[p + "mlp.gate_proj.weight"].T) * (m @ w[p + "mlp.up_proj.weight"].T)) @ w[p + "mlp.down_proj.weight"].T
    got = b.layer(w["model.embed_tokens.weight"][ids], 0, pos)
    assert torch.allclose(got, h, atol=1e-10)


def test_shifting_all_positions_changes_nothing(plain_models):
    """Only distances count: a layer run at positions p + 1000 gives the same output."""
    b = plain_models["B"]
    ids = token_ids(b.c["vocab_size"], 7, 8)
    h = b.w["model.embed_tokens.weight"][ids]
    assert torch.allclose(b.layer(h, 1, list(range(7))), b.layer(h, 1, list(range(1000, 1007))), atol=1e-9)


def test_greedy_takes_the_lowest_index_among_equals(plain_models):
    a = plain_models["A"]
    ids = token_ids(TINY_A["vocab_size"], 5, 9)
    out = a.greedy(ids, 3)
    assert len(out) == 3 and out[0] == int(torch.argmax(a.logits(ids)[-1]))
    assert int(torch.argmax(torch.tensor([1.0, 3.0, 3.0]))) == 1


def test_logits_of_chosen_rows_are_those_of_the_whole(plain_models):
    """``logits(ids, rows)`` computes the last layer's queries for the rows only; nothing else may change, with and
    without windows."""
    for name in ("B", "W"):
        model = plain_models[name]
        ids = token_ids(model.c["vocab_size"], 70, seed=5)
        rows = [0, 69, 31, 32]
        assert torch.allclose(model.logits(ids, rows), model.logits(ids)[rows], rtol=0, atol=1e-12)
