"""What fixes the plain implementation beside the reference's text: special cases that reduce to a library
routine, invariants, and the reference's own stated facts, each chosen so that a plausible mistake fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

from helpers import TINY_A, TINY_B, make_model_dir, random_tokens, read_model_dir
from plain import qwen3_plain as P


def test_rms_norm_is_the_library_routine_and_scale_invariant():
    torch.manual_seed(0)
    x, w = torch.randn(7, 96, dtype=torch.float64), 1 + 0.1 * torch.randn(96, dtype=torch.float64)
    assert torch.allclose(P.rms_norm(x, w, 1e-6), F.rms_norm(x, (96,), w, 1e-6), atol=1e-12)
    ones = torch.ones(96, dtype=torch.float64)
    y = P.rms_norm(x, ones, 1e-12)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(7, dtype=torch.float64), atol=1e-9)     # unit RMS
    assert torch.allclose(P.rms_norm(3.7 * x, w, 1e-12), P.rms_norm(x, w, 1e-12), atol=1e-9)    # f(cx) = f(x)
    # the weight multiplies (it is not 1 + w): a zero weight gives zero
    assert not P.rms_norm(x, torch.zeros(96, dtype=torch.float64), 1e-6).any()
    # eps sits inside the square root, added to the mean square (not to the sum, not outside)
    z = torch.zeros(1, 4, dtype=torch.float64)
    z[0, 0] = 2.0
    assert torch.allclose(P.rms_norm(z, torch.ones(4, dtype=torch.float64), 3.0)[0, 0],
                          torch.tensor(2.0 / math.sqrt(1.0 + 3.0), dtype=torch.float64))


def test_rope_tables_match_the_formula():
    cos, sin = P.rope_tables(8, 10000.0, 5)
    assert cos.shape == (5, 8) and torch.equal(cos[:, :4], cos[:, 4:])                # cat(freqs, freqs)
    assert torch.equal(cos[0], torch.ones(8)) and torch.equal(sin[0], torch.zeros(8))  # position 0: identity
    for i in range(4):
        assert math.isclose(float(cos[3, i]), math.cos(3 / 10000 ** (2 * i / 8)), rel_tol=1e-6)
        assert math.isclose(float(sin[3, i]), math.sin(3 / 10000 ** (2 * i / 8)), rel_tol=1e-6, abs_tol=1e-9)


def test_rope_is_a_rotation_of_pairs_j_and_j_plus_half():
    torch.manual_seed(1)
    d, T = 16, 9
    x = torch.randn(T, 3, d, dtype=torch.float64)
    cos, sin = P.rope_tables(d, 1e4, T, torch.float64)
    y = P.apply_rope(x, cos, sin)
    # the pair (j, j + d/2) as a complex number, multiplied by exp(i * angle): the library's polar form
    z = torch.complex(x[..., : d // 2], x[..., d // 2:])
    inv = 1.0 / (1e4 ** (torch.arange(0, d, 2).float() / d))
    ang = (torch.arange(T).float()[:, None] * inv[None]).double()
    zr = z * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    assert torch.allclose(y, torch.cat((zr.real, zr.imag), -1), atol=1e-6)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-9)                  # a rotation keeps lengths
    assert torch.equal(y[0], x[0])                                                    # position 0
    assert torch.equal(P.rotate_half(torch.arange(4.0)), torch.tensor([-2.0, -3.0, 0.0, 1.0]))


def test_rope_scores_depend_on_distance_only():
    torch.manual_seed(2)
    d = 32
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)
    cos, sin = P.rope_tables(d, 1e4, 64, torch.float64)

    def score(m, n):
        return float((P.apply_rope(q, cos[m:m + 1], sin[m:m + 1]) * P.apply_rope(k, cos[n:n + 1], sin[n:n + 1])).sum())

    assert math.isclose(score(5, 2), score(40, 37), rel_tol=1e-4, abs_tol=1e-4)      # float32 angles
    assert not math.isclose(score(5, 2), score(5, 3), rel_tol=1e-3)
    assert not math.isclose(score(5, 2), score(2, 5), rel_tol=1e-3)                  # the sign of the distance counts


def test_attention_reduces_to_the_library_routine():
    torch.manual_seed(3)
    T, n_heads, n_kv, d = 11, 6, 2, 8
    q = torch.randn(T, n_heads, d, dtype=torch.float64)
    k, v = torch.randn(T, n_kv, d, dtype=torch.float64), torch.randn(T, n_kv, d, dtype=torch.float64)
    scale = 0.37
    got = P.causal_gqa_attention(q, k, v, scale)
    # grouped heads: query head h reads kv head h // group  ==  repeat_interleave + plain causal attention
    kk, vv = k.repeat_interleave(3, 1), v.repeat_interleave(3, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kk.transpose(0, 1)[None], vv.transpose(0, 1)[None],
                                          is_causal=True, scale=scale)[0].transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-10)
    # a wrong grouping (h % n_kv) would differ
    wrong = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat(1, 3, 1).transpose(0, 1)[None],
                                           v.repeat(1, 3, 1).transpose(0, 1)[None], is_causal=True, scale=scale)
    assert not torch.allclose(got, wrong[0].transpose(0, 1), atol=1e-3)
    # one head, one group: plain multi-head attention
    one = P.causal_gqa_attention(q[:, :1], k[:, :1], v[:, :1], scale)
    lib = F.scaled_dot_product_attention(q[:, :1].transpose(0, 1)[None], k[:, :1].transpose(0, 1)[None],
                                         v[:, :1].transpose(0, 1)[None], is_causal=True, scale=scale)
    assert torch.allclose(one, lib[0].transpose(0, 1), atol=1e-10)


def test_attention_special_cases():
    torch.manual_seed(4)
    T, d = 6, 4
    q = torch.randn(T, 2, d, dtype=torch.float64)
    k, v = torch.randn(T, 1, d, dtype=torch.float64), torch.randn(T, 1, d, dtype=torch.float64)
    out = P.causal_gqa_attention(q, k, v, 1.0)
    assert torch.allclose(out[0], v[0].expand(2, d))                      # the first row sees one key: its value
    same = P.causal_gqa_attention(q, k[:1].expand(T, 1, d), v, 1.0)       # equal keys: the mean of the values seen
    for i in range(T):
        assert torch.allclose(same[i, 0], v[: i + 1, 0].mean(0), atol=1e-12)
    # keys after a row have no influence on it
    v2 = v.clone()
    v2[4:] += 100.0
    k2 = k.clone()
    k2[4:] -= 50.0
    assert torch.allclose(P.causal_gqa_attention(q, k2, v2, 1.0)[:4], out[:4], atol=1e-12)
    # a window of w keeps keys i-w+1..i
    win = P.causal_gqa_attention(q, k, v, 1.0, window=2)
    assert torch.allclose(win[:2], out[:2], atol=1e-12)
    assert torch.allclose(win[5], P.causal_gqa_attention(q[4:], k[4:], v[4:], 1.0)[1], atol=1e-12)


def test_swiglu_is_silu_gate_times_up():
    torch.manual_seed(5)
    h = torch.randn(3, 8, dtype=torch.float64)
    w = {"mlp.gate_proj.weight": torch.randn(12, 8, dtype=torch.float64),
         "mlp.up_proj.weight": torch.randn(12, 8, dtype=torch.float64),
         "mlp.down_proj.weight": torch.randn(8, 12, dtype=torch.float64)}
    g, u = h @ w["mlp.gate_proj.weight"].T, h @ w["mlp.up_proj.weight"].T
    want = ((g / (1 + torch.exp(-g))) * u) @ w["mlp.down_proj.weight"].T          # silu(g) = g / (1 + exp(-g))
    assert torch.allclose(P.swiglu(h, w, ""), want, atol=1e-12)
    swapped = dict(w, **{"mlp.gate_proj.weight": w["mlp.up_proj.weight"], "mlp.up_proj.weight": w["mlp.gate_proj.weight"]})
    assert not torch.allclose(P.swiglu(h, swapped, ""), want, atol=1e-3)           # gate and up are not interchangeable
    zero_up = dict(w, **{"mlp.up_proj.weight": torch.zeros(12, 8, dtype=torch.float64)})
    assert not P.swiglu(h, zero_up, "").any()


@pytest.fixture(scope="module")
def tiny_b(tmp_path_factory):
    path = make_model_dir(str(tmp_path_factory.mktemp("plain") / "b"), TINY_B, seed=22, norm_std=0.1)
    return read_model_dir(path)


def test_q_and_k_are_normed_before_the_rotation(tiny_b):
    """With a non-constant norm weight the order matters (a typical mistake, AGENTS.md:393-395)."""
    raw, w = tiny_b
    torch.manual_seed(6)
    h = torch.randn(5, raw["hidden_size"], dtype=torch.float64)
    w64 = {k: v.double() for k, v in w.items()}
    d = raw["head_dim"]
    cos, sin = P.rope_tables(d, raw["rope_theta"], 5, torch.float64)
    got = P.attention_block(h, w64, "model.layers.0.", raw, cos, sin)
    # the other order, written out here
    p = "model.layers.0.self_attn."
    q = (h @ w64[p + "q_proj.weight"].T).view(5, 8, d)
    k = (h @ w64[p + "k_proj.weight"].T).view(5, 2, d)
    v = (h @ w64[p + "v_proj.weight"].T).view(5, 2, d)
    q2 = P.rms_norm(P.apply_rope(q, cos, sin), w64[p + "q_norm.weight"], raw["rms_norm_eps"])
    k2 = P.rms_norm(P.apply_rope(k, cos, sin), w64[p + "k_norm.weight"], raw["rms_norm_eps"])
    other = P.causal_gqa_attention(q2, k2, v, 1 / math.sqrt(d)).reshape(5, -1) @ w64[p + "o_proj.weight"].T
    assert not torch.allclose(got, other, atol=1e-4)
    # v is neither normed nor rotated: scaling v scales the output
    w_scaled = dict(w64, **{p + "v_proj.weight": 2 * w64[p + "v_proj.weight"]})
    assert torch.allclose(P.attention_block(h, w_scaled, "model.layers.0.", raw, cos, sin), 2 * got, atol=1e-10)


def test_layer_is_the_textbook_pre_norm_block(tiny_b):
    raw, w = tiny_b
    torch.manual_seed(7)
    w64 = {k: v.double() for k, v in w.items()}
    x = torch.randn(4, raw["hidden_size"], dtype=torch.float64)
    cos, sin = P.rope_tables(raw["head_dim"], raw["rope_theta"], 4, torch.float64)
    p = "model.layers.1."
    a = x + P.attention_block(P.rms_norm(x, w64[p + "input_layernorm.weight"], raw["rms_norm_eps"]), w64, p, raw, cos, sin)
    want = a + P.swiglu(P.rms_norm(a, w64[p + "post_attention_layernorm.weight"], raw["rms_norm_eps"]), w64, p)
    assert torch.allclose(P.decoder_layer(x, w64, 1, raw, cos, sin), want, atol=1e-12)


def test_whole_model_properties(tiny_b, tmp_path):
    raw, w = tiny_b
    toks = random_tokens(20, raw["vocab_size"], seed=1)
    logits = P.forward(raw, w, toks, torch.float64)
    assert logits.shape == (20, raw["vocab_size"])
    # causal: logits at a position do not depend on later tokens
    changed = toks[:12] + random_tokens(8, raw["vocab_size"], seed=2)
    assert torch.allclose(P.forward(raw, w, changed, torch.float64)[:12], logits[:12], atol=1e-12)
    # float32 and float64 runs agree to float32 rounding
    assert float((P.forward(raw, w, toks).double() - logits).abs().max()) < 1e-4 * float(logits.abs().max())
    # a tied head is the embedding: tiny A's logits at the one position of a one-token prompt
    raw_a, w_a = read_model_dir(make_model_dir(str(tmp_path / "a"), TINY_A, seed=11))
    assert "lm_head.weight" not in w_a
    la = P.forward(raw_a, w_a, [3], torch.float64)
    untied = dict(raw_a, tie_word_embeddings=False)
    w_a2 = dict(w_a, **{"lm_head.weight": w_a["model.embed_tokens.weight"]})
    assert torch.equal(P.forward(untied, w_a2, [3], torch.float64), la)


def test_greedy_takes_the_lowest_index_among_equals_and_sampling_follows_the_cdf():
    assert P.greedy(torch.tensor([0.5, 2.0, 2.0, -1.0])) == 1
    logits = torch.log(torch.tensor([0.1, 0.2, 0.3, 0.4]))
    picks = [P.sample_with_temperature(logits, 1.0, u) for u in (0.0, 0.05, 0.1001, 0.29, 0.31, 0.61, 0.999)]
    assert picks == [0, 0, 1, 1, 2, 3, 3]
    # a low temperature sharpens towards the largest logit
    assert P.sample_with_temperature(logits, 0.01, 0.5) == 3
    assert P.cdf_margin(logits, 1.0, 0.31) == pytest.approx(0.01, abs=1e-6)


def test_generate_rule(tiny_b):
    raw, w = tiny_b
    prompt = random_tokens(6, raw["vocab_size"], seed=9)
    toks, logits = P.generate(raw, w, prompt, 4)
    assert len(toks) == 4
    full = P.forward(raw, w, prompt + toks[:-1])
    for t in range(4):
        assert toks[t] == int(torch.argmax(full[len(prompt) - 1 + t]))   # teacher-forcing our tokens reproduces them
    stopped, _ = P.generate(raw, w, prompt, 4, stop_token_ids=[toks[1]])
    assert stopped == toks[:2]
