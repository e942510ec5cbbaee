"""What pins the plain implementation beside the reference's text: special cases that
reduce to a library routine, and invariants, each chosen so that a plausible mistake
(a wrong sign or pairing, a norm in the wrong place, a wrong head mapping) fails."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain

torch.manual_seed(0)
F64 = torch.float64


def test_embedding_is_index_select():
    table = torch.randn(11, 6, dtype=F64)
    ids = [3, 0, 10, 3]
    assert torch.equal(plain.embedding(table, ids), table[torch.tensor(ids)])


def test_rms_norm_library_formula_and_eps():
    x = torch.randn(5, 12, dtype=F64) * 1e-2
    w = torch.randn(12, dtype=F64)
    for eps in (1e-5, 1e-6):
        want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w
        got = plain.rms_norm(x, w, eps)
        assert torch.allclose(got, want, rtol=1e-12, atol=0)
    # eps matters at this scale: the two differ visibly
    a = plain.rms_norm(x, w, 1e-5)
    b = plain.rms_norm(x, w, 1e-6)
    assert (a - b).abs().max() > 1e-3 * a.abs().max()


def test_rms_norm_unit_mean_square_and_scale_invariance():
    x = torch.randn(4, 24, dtype=F64)
    y = plain.rms_norm(x, torch.ones(24, dtype=F64), 0.0)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(4, dtype=F64), atol=1e-12)
    assert torch.allclose(plain.rms_norm(7.5 * x, torch.ones(24, dtype=F64), 0.0), y, atol=1e-12)
    # the weight multiplies directly: w = 0 gives 0 (a "1 + w" form would not)
    assert plain.rms_norm(x, torch.zeros(24, dtype=F64), 1e-5).abs().max() == 0


def test_rope_table_values():
    sin, cos = plain.rope_tables(50, 16, 10000.0)
    assert sin.shape == (50, 8)
    for pos, i in ((0, 0), (1, 0), (7, 3), (49, 7)):
        ang = pos * 10000.0 ** (-2 * i / 16)
        assert abs(float(sin[pos, i]) - math.sin(ang)) < 1e-5
        assert abs(float(cos[pos, i]) - math.cos(ang)) < 1e-5


def test_rope_adjacent_is_complex_multiplication():
    n, h, dh = 6, 3, 8
    x = torch.randn(n, h, dh, dtype=F64)
    pos = [0, 1, 5, 9, 2, 30]
    sin, cos = plain.rope_tables(64, dh, 10000.0)
    got = plain.rope(x, pos, sin, cos, "adjacent")
    xc = torch.view_as_complex(x.reshape(n, h, dh // 2, 2).contiguous())
    rot = torch.polar(torch.ones(n, dh // 2, dtype=F64),
                      torch.atan2(sin[pos], cos[pos]))
    want = torch.view_as_real(xc * rot[:, None, :]).reshape(n, h, dh)
    assert torch.allclose(got, want, atol=1e-12)


def test_rope_half_is_rotate_half_form():
    n, h, dh = 5, 2, 16
    x = torch.randn(n, h, dh, dtype=F64)
    pos = [3, 0, 11, 7, 1]
    sin, cos = plain.rope_tables(16, dh, 500000.0)
    got = plain.rope(x, pos, sin, cos, "half")
    c = torch.cat([cos[pos], cos[pos]], -1)[:, None, :]
    s = torch.cat([sin[pos], sin[pos]], -1)[:, None, :]
    rot_half = torch.cat([-x[..., dh // 2:], x[..., :dh // 2]], -1)
    assert torch.allclose(got, x * c + rot_half * s, atol=1e-12)
    # the two pairings are different functions
    assert not torch.allclose(got, plain.rope(x, pos, sin, cos, "adjacent"), atol=1e-3)


@pytest.mark.parametrize("pairing", ["half", "adjacent"])
def test_rope_identity_norm_and_relative_positions(pairing):
    dh = 16
    sin, cos = plain.rope_tables(128, dh, 10000.0)
    q = torch.randn(1, 1, dh, dtype=F64)
    k = torch.randn(1, 1, dh, dtype=F64)
    assert torch.allclose(plain.rope(q, [0], sin, cos, pairing), q, atol=1e-15)
    assert torch.allclose(plain.rope(q, [37], sin, cos, pairing).norm(), q.norm(), atol=1e-12)

    def dot(m, n):
        return float((plain.rope(q, [m], sin, cos, pairing) * plain.rope(k, [n], sin, cos, pairing)).sum())
    # only the distance counts (angles are 32-bit products, hence the tolerance);
    # a wrong sign in the rotation breaks this
    assert abs(dot(9, 4) - dot(25, 20)) < 1e-4
    assert abs(dot(9, 4) - dot(105, 100)) < 1e-4
    assert abs(dot(9, 4) - dot(4, 9)) > 1e-3


def _sdpa(q, k, v, causal):
    # [n, h, dh] -> [h, n, dh]
    return F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                          is_causal=causal).transpose(0, 1)


def test_attention_whole_sequence_is_library_causal_attention():
    n, nh, nkvh, dh = 9, 4, 2, 8
    q = torch.randn(n, nh, dh, dtype=F64)
    k = torch.randn(n, nkvh, dh, dtype=F64)
    v = torch.randn(n, nkvh, dh, dtype=F64)
    got = plain.attention(q, k, v, dh ** -0.5)
    want = _sdpa(q, k.repeat_interleave(nh // nkvh, 1), v.repeat_interleave(nh // nkvh, 1), True)
    assert torch.allclose(got, want, atol=1e-12)
    # a wrong head mapping (h % nkvh) differs
    wrong = _sdpa(q, k.repeat(1, nh // nkvh, 1), v.repeat(1, nh // nkvh, 1), True)
    assert not torch.allclose(got, wrong, atol=1e-3)


def test_attention_last_query_is_unmasked_library_attention_one_head():
    n, dh = 7, 16
    q = torch.randn(1, 1, dh, dtype=F64)
    k = torch.randn(n, 1, dh, dtype=F64)
    v = torch.randn(n, 1, dh, dtype=F64)
    got = plain.attention(q, k, v, dh ** -0.5, first_pos=n - 1)
    assert torch.allclose(got, _sdpa(q, k, v, False), atol=1e-12)


def test_attention_special_cases():
    dh = 8
    k = torch.randn(5, 2, dh, dtype=F64)
    v = torch.randn(5, 2, dh, dtype=F64)
    # one key: the output is its value
    q = torch.randn(1, 2, dh, dtype=F64)
    assert torch.allclose(plain.attention(q, k[:1], v[:1], 1.0), v[:1], atol=1e-15)
    # zero queries: the mean of the visible values
    o = plain.attention(torch.zeros(5, 2, dh, dtype=F64), k, v, 1.0)
    for t in range(5):
        assert torch.allclose(o[t], v[:t + 1].mean(0), atol=1e-12)
    # a window of w keys is the attention over the last w keys
    q = torch.randn(5, 2, dh, dtype=F64)
    o = plain.attention(q, k, v, 0.3, window=2)
    t = 4
    assert torch.allclose(o[t:t + 1], plain.attention(q[t:t + 1], k[3:5], v[3:5], 0.3, first_pos=1), atol=1e-12)


def test_swiglu_is_library_silu_times_up():
    g = torch.randn(4, 10, dtype=F64) * 3
    u = torch.randn(4, 10, dtype=F64)
    assert torch.allclose(plain.swiglu(g, u), F.silu(g) * u, atol=1e-12)
    assert plain.swiglu(torch.zeros(3), torch.ones(3)).abs().max() == 0
    assert plain.swiglu(torch.full((3,), -50.0), torch.ones(3)).abs().max() < 1e-15


def _cfg(**kw):
    base = dict(num_hidden_layers=2, hidden_size=32, num_attention_heads=4, num_key_value_heads=2,
                head_dim=8, intermediate_size=44, vocab_size=50, max_position_embeddings=64,
                rope_theta=10000.0, rms_norm_eps=1e-5)
    base.update(kw)
    return plain.PlainConfig(**base)


def test_block_is_prenorm_zero_branches_reduce_to_head_of_normed_embedding():
    """With zero output and down projections every block adds nothing, so the logits
    are ``head(norm(embedding))``: true for norms before the branches, false for a norm
    on the residual stream after them."""
    cfg = _cfg()
    w = plain.random_weights(cfg, 1)
    for i in range(cfg.num_hidden_layers):
        w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{i}.mlp.down_proj.weight"].zero_()
    toks = [3, 9, 9, 41]
    x = w["model.embed_tokens.weight"][toks].to(F64)
    want = F.linear(x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg.rms_norm_eps)
                    * w["model.norm.weight"].to(F64), w["lm_head.weight"].to(F64))
    assert torch.allclose(plain.forward(cfg, w, toks), want, atol=1e-12)


def test_single_token_closed_form():
    """One token: softmax over one key is 1, the rotation at position 0 is the identity,
    so the attention branch is ``Wo (repeat(Wv x1))``."""
    cfg = _cfg(num_hidden_layers=1)
    w = plain.random_weights(cfg, 2, std=0.2)
    p = "model.layers.0."
    x = w["model.embed_tokens.weight"][[7]].to(F64)
    n1 = lambda t, name: t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + cfg.rms_norm_eps) * w[name].to(F64)
    x1 = n1(x, p + "input_layernorm.weight")
    v = F.linear(x1, w[p + "self_attn.v_proj.weight"].to(F64)).view(1, 2, 8).repeat_interleave(2, 1)
    x = x + F.linear(v.reshape(1, 32), w[p + "self_attn.o_proj.weight"].to(F64))
    x2 = n1(x, p + "post_attention_layernorm.weight")
    h = F.silu(F.linear(x2, w[p + "mlp.gate_proj.weight"].to(F64))) * F.linear(x2, w[p + "mlp.up_proj.weight"].to(F64))
    x = x + F.linear(h, w[p + "mlp.down_proj.weight"].to(F64))
    want = F.linear(n1(x, "model.norm.weight"), w["lm_head.weight"].to(F64))
    assert torch.allclose(plain.forward(cfg, w, [7]), want, atol=1e-12)


def test_tied_output_uses_the_embedding_table():
    cfg = _cfg(tie_word_embeddings=True)
    w = plain.random_weights(cfg, 3)
    assert "lm_head.weight" not in w
    a = plain.forward(cfg, w, [1, 2, 3])
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    cfg2 = _cfg(tie_word_embeddings=False)
    assert torch.allclose(a, plain.forward(cfg2, w2, [1, 2, 3]), atol=1e-12)


def test_causality_a_later_token_changes_no_earlier_logits():
    cfg = _cfg()
    w = plain.random_weights(cfg, 4, std=0.2)
    a = plain.forward(cfg, w, [5, 6, 7, 8, 9])
    b = plain.forward(cfg, w, [5, 6, 7, 1, 2])
    assert torch.allclose(a[:3], b[:3], atol=1e-12)
    assert not torch.allclose(a[3:], b[3:], atol=1e-6)


def test_shift_of_all_positions_leaves_the_attention_branch_unchanged():
    cfg = _cfg(num_hidden_layers=1)
    w = plain.random_weights(cfg, 5, std=0.2)
    x1 = torch.randn(6, 32, dtype=F64)
    sin, cos = plain.rope_tables(64, cfg.head_dim, cfg.rope_theta)
    a = plain.attention_block(cfg, w, "model.layers.0.", x1, list(range(6)), sin, cos)
    b = plain.attention_block(cfg, w, "model.layers.0.", x1, list(range(20, 26)), sin, cos)
    assert torch.allclose(a, b, atol=1e-4)
    c = plain.attention_block(cfg, w, "model.layers.0.", x1, [0, 1, 2, 3, 4, 9], sin, cos)
    assert not torch.allclose(a, c, atol=1e-4)


def test_sampling_greedy_and_limits():
    l = torch.tensor([0.1, 2.0, -1.0, 2.0, 0.5], dtype=F64)
    assert plain.sample(l, 0.0, 1.0, 10**9, 0.7) == 1            # lowest index among equals
    assert plain.sample(l, 0.8, 1.0, 1, 0.7) == 1                # top_k = 1 is greedy
    assert plain.sample(l, 0.8, 1.0, 10**9, 0.0) == 1            # u = 0: the first of the sorted
    assert plain.sample(l, 1.0, 1.0, 2, 0.999) == 3              # top_k = 2: only the two 2.0s
    # tiny top_p: always the largest
    assert plain.sample(l, 1.0, 1e-6, 10**9, 0.999) == 1


def test_sampling_frequencies_follow_softmax():
    l = torch.tensor([1.0, 0.0, -1.0, 0.5], dtype=F64)
    T = 0.7
    rng = np.random.default_rng(0)
    n = 20000
    cnt = np.zeros(4)
    for u in rng.random(n):
        cnt[plain.sample(l, T, 1.0, 10**9, float(u))] += 1
    p = torch.softmax(l / T, 0).numpy()
    assert np.abs(cnt / n - p).max() < 0.015
    # top_k = 2 keeps the two largest, renormalised
    cnt = np.zeros(4)
    for u in rng.random(n):
        cnt[plain.sample(l, T, 1.0, 2, float(u))] += 1
    q = p.copy(); q[[1, 2]] = 0; q /= q.sum()
    assert np.abs(cnt / n - q).max() < 0.015


def test_rounding_model_rounds_what_is_stored_and_nothing_else():
    """``forward(..., rounding="bfloat16")``: with weights and activations that bfloat16 holds exactly all the way (a
    model of zeros and ones: the embedding rows are unit vectors scaled by powers of two, the projections pick
    coordinates) the rounding changes nothing; with ordinary weights it moves the logits by about 2^-8 of their
    size, not by 2^-16 (nothing rounded) and not by 2^-4 (something rounded that must not be: the sums of a
    product, the residual stream)."""
    cfg = plain.PlainConfig(num_hidden_layers=2, hidden_size=32, num_attention_heads=2, num_key_value_heads=1, head_dim=16,
                            intermediate_size=48, vocab_size=64, max_position_embeddings=64)
    w = plain.random_weights(cfg, 3, std=0.2)
    w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    toks = [3, 9, 27, 1, 60, 33, 7]
    a = plain.forward(cfg, w, toks)
    b = plain.forward(cfg, w, toks, rounding="bfloat16")
    rel = float((a - b).abs().max() / a.abs().max())
    assert 2.0 ** -12 < rel < 2.0 ** -5, rel
    # the residual stream is not rounded: a stream that bfloat16 cannot hold (1 + 2^-12) survives a layer whose
    # branches give zero
    for k in w:
        if "o_proj" in k or "down_proj" in k:
            w[k] = torch.zeros_like(w[k])
    w["model.embed_tokens.weight"] = torch.full_like(w["model.embed_tokens.weight"], 1.0 + 2.0 ** -12)
    w["model.embed_tokens.weight"][:, 0] = 3.0
    st = []
    plain.forward(cfg, w, toks, rounding="bfloat16", states=st)
    assert len(st) == cfg.num_hidden_layers + 1
    assert all(torch.equal(s, st[0]) for s in st) and float(st[-1][0, 1]) == 1.0 + 2.0 ** -12
    assert float(plain.rounded(st[-1], "bfloat16")[0, 1]) == 1.0
