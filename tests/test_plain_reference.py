"""Pins the plain implementation by what fixes it beside the reference's text.

Vectors: the operator goldens that the reference tracks in data/golden/operators.json (atol
1e-6, operators.json:3).  Special cases: attention without rotation or mask against a library
softmax-matmul; one head; a one-token sequence.  Invariants: a shift of all positions; causality.
Each is chosen so that a plausible mistake fails it (named in the test).
"""
import math

import pytest
import torch

from plain_llama import (plain_attention, plain_forward, plain_greedy, plain_linear, plain_rms_norm,
                         plain_rope, plain_silu_mul, plain_softmax, plain_top_p_distribution)

ATOL = 1e-6


def test_rms_norm_golden():
    # data/golden/operators.json:4-24.  eps outside the root, or a (1 + w) weight, fails it.
    out = plain_rms_norm(torch.tensor([1.0, -2.0, 3.0, -4.0]), torch.tensor([0.5, 1.0, 1.5, 2.0]), 1e-5)
    want = [0.182574063539505, -0.73029625415802, 1.6431666612625122, -2.92118501663208]
    assert torch.allclose(out, torch.tensor(want, dtype=torch.float64), atol=ATOL, rtol=0)


def test_rms_norm_invariants():
    x = torch.randn(5, 24, dtype=torch.float64)
    w = torch.ones(24)
    y = plain_rms_norm(x, w, 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-9)
    assert torch.allclose(plain_rms_norm(1e4 * x, w, 1e-6), plain_rms_norm(x, w, 1e-14), atol=1e-9)
    assert torch.equal(plain_rms_norm(torch.zeros(3, 8), torch.ones(8), 1e-5), torch.zeros(3, 8, dtype=torch.float64))
    # no mean is subtracted: a constant row keeps its sign and size
    assert torch.allclose(plain_rms_norm(torch.full((1, 4), 3.0), torch.ones(4), 1e-12),
                          torch.ones(1, 4, dtype=torch.float64), atol=1e-9)


def test_rope_golden():
    # data/golden/operators.json:25-63: 2 query heads, 1 kv head, d = 4, position 7, theta 1e4.
    # An interleaved (2i, 2i+1) pairing or a flipped sine sign fails it.
    q = torch.tensor([0.1, 0.2, 0.3, 0.4, -0.5, 0.6, -0.7, 0.8], dtype=torch.float32).view(1, 2, 4)
    k = torch.tensor([0.9, -1.0, 1.1, -1.2], dtype=torch.float32).view(1, 1, 4)
    pos = torch.tensor([7])
    want_q = [-0.12170576304197311, 0.17153306305408478, 0.2918693423271179, 0.41300898790359497,
              0.08293947577476501, 0.5425763726234436, -0.8562248945236206, 0.8400065302848816]
    want_k = [-0.044173240661621094, -0.9136196374893188, 1.4205803871154785, -1.267004132270813]
    assert torch.allclose(plain_rope(q, pos, 10000.0).flatten(), torch.tensor(want_q, dtype=torch.float64), atol=ATOL, rtol=0)
    assert torch.allclose(plain_rope(k, pos, 10000.0).flatten(), torch.tensor(want_k, dtype=torch.float64), atol=ATOL, rtol=0)


def test_rope_invariants():
    torch.manual_seed(1)
    q = torch.randn(6, 3, 8, dtype=torch.float64)
    k = torch.randn(6, 3, 8, dtype=torch.float64)
    zero = torch.zeros(6, dtype=torch.long)
    assert torch.allclose(plain_rope(q, zero, 500000.0), q)             # position 0 is the identity
    pos = torch.arange(6)
    rq = plain_rope(q, pos, 10000.0)
    half = 4
    assert torch.allclose(rq[..., :half] ** 2 + rq[..., half:] ** 2, q[..., :half] ** 2 + q[..., half:] ** 2)
    # only distances count: <R(p)q, R(p')k> is unchanged when both positions move by 16
    a = torch.einsum("thd,shd->hts", plain_rope(q, pos, 10000.0), plain_rope(k, pos, 10000.0))
    b = torch.einsum("thd,shd->hts", plain_rope(q, pos + 16, 10000.0), plain_rope(k, pos + 16, 10000.0))
    assert torch.allclose(a, b, atol=1e-5)


def test_softmax_golden():
    # data/golden/operators.json:64-77: the maximum is subtracted, so +-1000 stays finite.
    out = plain_softmax(torch.tensor([1000.0, 1001.0, 999.0, -1000.0]))
    want = [0.2447284758090973, 0.6652409434318542, 0.09003057330846786, 0.0]
    assert torch.allclose(out, torch.tensor(want, dtype=torch.float64), atol=ATOL, rtol=0)
    assert abs(out.sum().item() - 1.0) < 1e-12


def test_attention_golden():
    # data/golden/operators.json:78-131: 3 keys, 2 query heads on 1 kv head, d = 4; the query is
    # the last position, so it sees all three keys.
    q = torch.tensor([0.2, -0.1, 0.4, 0.3, -0.5, 0.7, 0.1, -0.2]).view(1, 2, 4)
    keys = torch.tensor([0.1, 0.2, 0.3, 0.4, -0.4, 0.3, -0.2, 0.1, 0.5, -0.6, 0.7, -0.8]).view(3, 1, 4)
    values = torch.tensor([1.0, 0.0, -1.0, 0.5, 0.2, 0.4, 0.6, 0.8, -0.3, 0.7, 0.9, -0.1]).view(3, 1, 4)
    full_q = torch.zeros(3, 2, 4)
    full_q[2] = q[0]
    out = plain_attention(full_q, keys, values)[2].flatten()
    want = [0.31072109937667847, 0.3621496558189392, 0.13341431319713593, 0.3776317536830902,
            0.3371150493621826, 0.3447031080722809, 0.14012068510055542, 0.46016252040863037]
    assert torch.allclose(out, torch.tensor(want, dtype=torch.float64), atol=ATOL, rtol=0)


def test_attention_reduces_to_library_softmax_matmul():
    # nkv == nq, last query row sees every key: plain softmax(q K^T / sqrt(d)) V of a library.
    torch.manual_seed(2)
    T, h, d = 7, 3, 8
    q, k, v = (torch.randn(T, h, d, dtype=torch.float64) for _ in range(3))
    out = plain_attention(q, k, v)
    for head in range(h):
        scores = (q[:, head] @ k[:, head].T) / math.sqrt(d)
        scores = scores.masked_fill(torch.ones(T, T).triu(1).bool(), float("-inf"))
        want = torch.softmax(scores, dim=-1) @ v[:, head]
        assert torch.allclose(out[:, head], want, atol=1e-12)


def test_attention_grouping_and_special_cases():
    torch.manual_seed(3)
    T, d = 5, 4
    q = torch.randn(T, 6, d, dtype=torch.float64)
    k = torch.randn(T, 2, d, dtype=torch.float64)
    v = torch.randn(T, 2, d, dtype=torch.float64)
    out = plain_attention(q, k, v)
    # consecutive query heads share a kv head: heads 0..2 -> kv 0, heads 3..5 -> kv 1
    repeated = plain_attention(q, k.repeat_interleave(3, dim=1), v.repeat_interleave(3, dim=1))
    assert torch.allclose(out, repeated, atol=1e-12)
    wrong = plain_attention(q, k.repeat(1, 3, 1), v.repeat(1, 3, 1))      # interleaved sharing
    assert not torch.allclose(out, wrong, atol=1e-6)
    # the first token of a sequence returns its own value exactly
    assert torch.allclose(out[0], v[0].repeat_interleave(3, dim=0), atol=1e-12)
    # causal: editing a later token leaves earlier rows unchanged
    k2, v2 = k.clone(), v.clone()
    k2[4] += 1.0
    v2[4] -= 2.0
    assert torch.allclose(plain_attention(q, k2, v2)[:4], out[:4], atol=1e-12)
    # a window of T or more is no window; a window of 1 returns each token's own value
    assert torch.allclose(plain_attention(q, k, v, window=T), out, atol=1e-12)
    assert torch.allclose(plain_attention(q, k, v, window=1), v.repeat_interleave(3, dim=1), atol=1e-12)


def test_silu_mul_golden():
    # data/golden/operators.json:132-151.  SiLU on `up` instead of `gate` fails it.
    out = plain_silu_mul(torch.tensor([-2.0, -0.5, 0.0, 1.5]), torch.tensor([0.5, -1.0, 2.0, 3.0]))
    want = [-0.11920291930437088, 0.1887703388929367, 0.0, 3.6790847778320312]
    assert torch.allclose(out, torch.tensor(want, dtype=torch.float64), atol=ATOL, rtol=0)
    big = plain_silu_mul(torch.tensor([50.0, -800.0]), torch.tensor([2.0, 2.0]))
    assert abs(big[0].item() - 100.0) < 1e-9 and big[1].item() == 0.0 or abs(big[1].item()) < 1e-300


def test_linear_case():
    # the 3x4, batch 2 case has the layout of tests/cuda/kernel_tests.cu:309-319: W is [out, in].
    w = torch.arange(12, dtype=torch.float64).view(3, 4) / 10
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [-1.0, 0.5, 0.0, 2.0]])
    want = torch.tensor([[sum(w[o, i] * x[b, i] for i in range(4)) for o in range(3)] for b in range(2)])
    assert torch.allclose(plain_linear(x, w), want.double(), atol=1e-12)
    assert torch.allclose(plain_linear(x, w, torch.tensor([1.0, 2.0, 3.0])), want.double() + torch.tensor([1.0, 2.0, 3.0]), atol=1e-12)


def test_greedy_ties_take_the_lowest_index():
    # tests/unit_tests.cpp:198-207: [1, 3, 3, 2] -> 1
    assert plain_greedy(torch.tensor([1.0, 3.0, 3.0, 2.0])) == 1


def test_top_p_distribution():
    logits = torch.tensor([2.0, 1.0, 0.0, -1.0])
    full = plain_top_p_distribution(logits, 1.0, 1.0)
    assert torch.allclose(full, torch.softmax(logits.double(), 0), atol=1e-12)
    # p0 = 0.6439, p1 = 0.2369: top_p 0.7 keeps two (the one that crosses is kept)
    kept = plain_top_p_distribution(logits, 1.0, 0.7)
    assert (kept > 0).tolist() == [True, True, False, False]
    assert abs(kept.sum().item() - 1.0) < 1e-12
    assert (plain_top_p_distribution(logits, 1.0, 1e-9) > 0).tolist() == [True, False, False, False]
    cold = plain_top_p_distribution(logits, 0.01, 1.0)
    assert cold[0] > 1 - 1e-12


def _tiny(seed=0, tie=False, bias=False):
    torch.manual_seed(seed)
    cfg = dict(hidden_size=24, intermediate_size=40, num_hidden_layers=2, num_attention_heads=3,
               num_key_value_heads=1, head_dim=8, vocab_size=50, rms_norm_eps=1e-5, rope_theta=10000.0,
               tie_word_embeddings=tie)
    H, I, qd, kvd = 24, 40, 24, 8
    w = {"model.embed_tokens.weight": torch.randn(50, H) * 0.5, "model.norm.weight": 1 + 0.1 * torch.randn(H)}
    if not tie:
        w["lm_head.weight"] = torch.randn(50, H) * 0.5
    for l in range(2):
        p = f"model.layers.{l}."
        w[p + "input_layernorm.weight"] = 1 + 0.1 * torch.randn(H)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(H)
        for name, shape in (("self_attn.q_proj", (qd, H)), ("self_attn.k_proj", (kvd, H)), ("self_attn.v_proj", (kvd, H)),
                            ("self_attn.o_proj", (H, qd)), ("mlp.gate_proj", (I, H)), ("mlp.up_proj", (I, H)),
                            ("mlp.down_proj", (H, I))):
            w[p + name + ".weight"] = torch.randn(*shape) * 0.3
            if bias and name.startswith("self_attn"):
                w[p + name + ".bias"] = torch.randn(shape[0]) * 0.3
    return cfg, w


def test_model_identity_blocks_reduce_to_head_of_normed_embedding():
    # with o_proj and down_proj zero every block is the identity (pre-norm, two residual adds):
    # logits = head(norm(E[token])).  A norm applied to the residual in place fails it.
    cfg, w = _tiny()
    for l in range(2):
        w[f"model.layers.{l}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{l}.mlp.down_proj.weight"].zero_()
    tokens = [3, 7, 7, 1]
    want = plain_linear(plain_rms_norm(w["model.embed_tokens.weight"][tokens], w["model.norm.weight"], 1e-5), w["lm_head.weight"])
    assert torch.allclose(plain_forward(cfg, w, tokens), want, atol=1e-12)


def test_model_causal_and_shift_invariant_and_tied():
    cfg, w = _tiny(seed=4, bias=True)
    tokens = [5, 9, 2, 2, 41, 17]
    full = plain_forward(cfg, w, tokens)
    assert torch.allclose(plain_forward(cfg, w, tokens[:4]), full[:4], atol=1e-10)
    # rotary positions enter through distances only
    assert torch.allclose(plain_forward(cfg, w, tokens, first_position=9), full, atol=1e-4)
    cfg_t, w_t = _tiny(seed=4, tie=True)
    w_u = dict(w_t)
    w_u["lm_head.weight"] = w_t["model.embed_tokens.weight"]
    cfg_u = dict(cfg_t, tie_word_embeddings=False)
    assert torch.allclose(plain_forward(cfg_t, w_t, tokens), plain_forward(cfg_u, w_u, tokens), atol=1e-12)


def test_model_bias_is_applied_before_rotation():
    # with zero weights in q/k/v the projections are the biases alone; the keys of two positions
    # then differ only by rotation, so position 1's attention is not uniform unless the bias
    # were added after the rotation.
    cfg, w = _tiny(seed=5, bias=True)
    cfg = dict(cfg, num_hidden_layers=1)
    assert not torch.allclose(plain_forward(cfg, w, [1, 2, 3])[2], plain_forward(cfg, {**w, "model.layers.0.self_attn.k_proj.bias": torch.zeros(8)}, [1, 2, 3])[2], atol=1e-6)


def test_model_trace_names_and_the_residual_sums():
    """The named tensors of the reference's ModelTrace (src/model.cpp:98-231): 5 a layer + 3 (113
    for its 22 layers, scripts/export_golden.py:73-107), and what ties them together: a layer's
    output is its input plus its two projected outputs."""
    cfg, w = _tiny(seed=2)
    tokens = [4, 8, 15, 16, 23, 42]
    trace = {}
    logits = plain_forward(cfg, w, tokens, trace=trace)
    assert len(trace) == 5 * 2 + 3 and torch.equal(trace["logits"], logits)
    assert torch.equal(trace["embedding"], w["model.embed_tokens.weight"].double()[tokens])
    before = trace["embedding"]
    for layer in range(2):
        p = f"layer{layer}."
        assert torch.allclose(trace[p + "output"], before + trace[p + "attention_output"] + trace[p + "mlp_output"], atol=1e-12)
        assert torch.allclose(trace[p + "input_norm"], plain_rms_norm(before, w[f"model.layers.{layer}.input_layernorm.weight"], 1e-5))
        before = trace[p + "output"]
    assert torch.allclose(trace["final_norm"], plain_rms_norm(before, w["model.norm.weight"], 1e-5))


def test_rows_of_a_one_layer_model_are_the_whole_forward_at_those_rows():
    """`plain_forward_rows` (for sequences too long to compute whole) against `plain_forward`."""
    from plain_llama import plain_forward, plain_forward_rows
    torch.manual_seed(3)
    cfg = dict(hidden_size=48, intermediate_size=80, num_hidden_layers=1, num_attention_heads=6, num_key_value_heads=2, head_dim=8,
               vocab_size=40, rms_norm_eps=1e-5, rope_theta=777.0, tie_word_embeddings=False)
    p = "model.layers.0."
    shapes = {"model.embed_tokens.weight": (40, 48), "lm_head.weight": (40, 48), "model.norm.weight": (48,),
              p + "input_layernorm.weight": (48,), p + "post_attention_layernorm.weight": (48,),
              p + "self_attn.q_proj.weight": (48, 48), p + "self_attn.k_proj.weight": (16, 48), p + "self_attn.v_proj.weight": (16, 48),
              p + "self_attn.o_proj.weight": (48, 48), p + "self_attn.q_proj.bias": (48,), p + "self_attn.k_proj.bias": (16,),
              p + "self_attn.v_proj.bias": (16,), p + "self_attn.o_proj.bias": (48,),
              p + "mlp.gate_proj.weight": (80, 48), p + "mlp.up_proj.weight": (80, 48), p + "mlp.down_proj.weight": (48, 80)}
    w = {name: torch.randn(shape, dtype=torch.float64) * 0.3 for name, shape in shapes.items()}
    tokens = [(7 * i * i + 3) % 40 for i in range(33)]
    whole = plain_forward(cfg, w, tokens)
    rows = [0, 1, 16, 31, 32]
    assert torch.allclose(plain_forward_rows(cfg, w, tokens, rows), whole[rows], rtol=1e-12, atol=1e-12)
