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


# The reference states four of its formulas a second time, element by element, in the docstrings and bodies of
# its kernels. The tests below write those second statements out as scalar arithmetic and hold the plain
# implementation (written from the first statements, model.py) against them; in each, the plausible other
# reading is shown to give another number.

def test_rotation_pairs_element_by_element():
    """kernels/rope_qknorm.py:15-20, 39-47: with x1, x2 the two halves of a head and c, s the first half of a table
    row, o1 = x1 c - x2 s and o2 = x2 c + x1 s: element j is paired with element j + d/2 (not with j + 1)."""
    d, pos, theta = 8, 3, 100.0
    x = torch.tensor([0.5, -1.0, 2.0, 0.25, 1.5, 3.0, -0.75, 1.0], dtype=torch.float64)
    cos, sin = P.rope_tables(d, theta, pos + 1, torch.float64)
    got = P.apply_rope(x.view(1, 1, d), cos[pos:pos + 1], sin[pos:pos + 1]).view(d)
    want = torch.empty(d, dtype=torch.float64)
    interleaved = torch.empty(d, dtype=torch.float64)
    for j in range(d // 2):
        angle = float(torch.tensor(pos, dtype=torch.float32) * (1.0 / torch.tensor(theta, dtype=torch.float32) ** (2 * j / d)))
        c, sn = math.cos(angle), math.sin(angle)
        x1, x2 = float(x[j]), float(x[j + d // 2])
        want[j], want[j + d // 2] = x1 * c - x2 * sn, x2 * c + x1 * sn
        a, b = float(x[2 * j]), float(x[2 * j + 1])                     # the other convention: neighbours
        interleaved[2 * j], interleaved[2 * j + 1] = a * c - b * sn, b * c + a * sn
    assert torch.allclose(got, want, atol=1e-6)
    assert not torch.allclose(got, interleaved, atol=1e-2)
    # the sign: a quarter turn takes (1, 0) to (0, 1), i.e. x1 goes to the second half with a plus
    quarter = P.apply_rope(torch.tensor([1.0, 0.0]).view(1, 1, 2), torch.zeros(1, 2), torch.ones(1, 2)).view(2)
    assert quarter.tolist() == [0.0, 1.0]


def test_norm_then_rotation_element_by_element(tiny_b):
    """kernels/rope_qknorm.py:15-18 and 39-47 (`_norm_rope`): n = x * rsqrt(mean(x^2) + eps) * w first, then the
    rotation of n. `attention_block` applied to one head must give keys that are exactly that."""
    raw, w = tiny_b
    d, eps = raw["head_dim"], raw["rms_norm_eps"]
    w64 = {k: v.double() for k, v in w.items()}
    torch.manual_seed(8)
    h = torch.randn(3, raw["hidden_size"], dtype=torch.float64)
    p = "model.layers.0.self_attn."
    cos, sin = P.rope_tables(d, raw["rope_theta"], 3, torch.float64)
    k = (h @ w64[p + "k_proj.weight"].T).view(3, raw["num_key_value_heads"], d)
    kn = P.apply_rope(P.rms_norm(k, w64[p + "k_norm.weight"], eps), cos, sin)
    pos, head = 2, 1
    x, wt = k[pos, head], w64[p + "k_norm.weight"]
    inv = 1.0 / math.sqrt(float((x * x).sum()) / d + eps)
    for j in range(d // 2):
        n1, n2 = float(x[j]) * inv * float(wt[j]), float(x[j + d // 2]) * inv * float(wt[j + d // 2])
        c, sn = float(cos[pos, j]), float(sin[pos, j])
        assert math.isclose(float(kn[pos, head, j]), n1 * c - n2 * sn, rel_tol=1e-9, abs_tol=1e-12)
        assert math.isclose(float(kn[pos, head, j + d // 2]), n2 * c + n1 * sn, rel_tol=1e-9, abs_tol=1e-12)


def test_gate_columns_come_first_and_carry_the_silu():
    """kernels/silu_mul.py:3-5, 29-32: of the fused product's [M, 2I] columns the first I are the gate, the next I
    the up projection (weights.py:98-100 stacks gate above up), and y = silu(g) * u with silu(x) = x / (1 + exp(-x)).
    A gate far below zero closes the unit whatever `up` says; an `up` far below zero does not."""
    w = {"mlp.gate_proj.weight": torch.tensor([[1.0, 0.0], [0.0, 1.0]], dtype=torch.float64),
         "mlp.up_proj.weight": torch.tensor([[0.0, 1.0], [1.0, 0.0]], dtype=torch.float64),
         "mlp.down_proj.weight": torch.eye(2, dtype=torch.float64)}
    h = torch.tensor([[-40.0, 3.0]], dtype=torch.float64)              # g = (-40, 3), u = (3, -40)
    y = P.swiglu(h, w, "")[0]
    assert abs(float(y[0])) < 1e-12                                    # silu(-40) * 3: closed
    silu3 = 3.0 / (1.0 + math.exp(-3.0))
    assert math.isclose(float(y[1]), silu3 * -40.0, rel_tol=1e-12)     # silu(3) * (-40): open, and large
    # were the silu on `up`, the first unit would give -40 * silu(3) and the second one nothing


def test_scores_are_scaled_by_one_over_root_head_dim():
    """model.py:65 (`self.scale = 1.0 / math.sqrt(cfg.head_dim)`) and kernels/attn_decode.py:180-196: with head
    size 4, a query and a key that are both (1, -1, 1, -1) after the norm score 4 * 1/2 = 2 against 0 for an
    orthogonal key, so the second position's probabilities are (1, e^2) / (1 + e^2) and its output
    p0 * h0 + p1 * h1, whose second element is 1 - 2 p1 = -tanh(1)."""
    cfg = {"num_attention_heads": 1, "num_key_value_heads": 1, "head_dim": 4, "hidden_size": 4, "rms_norm_eps": 1e-12}
    eye = torch.eye(4, dtype=torch.float64)
    p = "l."
    w = {p + f"self_attn.{n}_proj.weight": eye for n in "qkvo"}
    w[p + "self_attn.q_norm.weight"] = w[p + "self_attn.k_norm.weight"] = torch.ones(4, dtype=torch.float64)
    h = torch.tensor([[1.0, 1.0, 1.0, 1.0], [1.0, -1.0, 1.0, -1.0]], dtype=torch.float64)
    no_turn = (torch.ones(2, 4, dtype=torch.float64), torch.zeros(2, 4, dtype=torch.float64))
    out = P.attention_block(h, w, p, cfg, *no_turn)
    assert torch.allclose(out[0], h[0], atol=1e-9)
    assert math.isclose(float(out[1, 0]), 1.0, rel_tol=1e-9)
    assert math.isclose(float(out[1, 1]), -math.tanh(1.0), rel_tol=1e-9)            # scale 1/2
    assert not math.isclose(float(out[1, 1]), -math.tanh(0.5), rel_tol=1e-3)        # scale 1/4 (1 / head_dim)
    assert not math.isclose(float(out[1, 1]), -math.tanh(2.0), rel_tol=1e-3)        # no scale


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
