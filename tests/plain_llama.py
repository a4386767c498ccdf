"""A plain, slow implementation of the Llama dense decoder, used only as the tests' oracle.

Every function works on whole sequences, keeps no cache, and shares no code with the engine.
Each is written from the formula at the cited place of the reference
(BetterThanAny/tinyllama-inference-engine); paths are relative to that repository.

Arithmetic is float64 by default, so that an engine running in true 32-bit is compared with
something more exact than itself.  The one exception is the rotary angle, which the reference
forms in 32-bit (`pow`, then `position * frequency`, src/operators.cpp:63-65): the angle is what
the formula *means*, so the oracle forms it the same way and only then widens it.
"""
from __future__ import annotations

import math

import torch


def plain_rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w, eps added to the mean inside the root.

    src/operators.cpp:31-40 (sum of squares, mean, `1/sqrt(mean + eps)`, then `x * scale * w`).
    """
    x = x.double()
    mean_square = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    scale = 1.0 / torch.sqrt(mean_square + eps)
    return x * scale * weight.double()


def plain_rope_angles(positions: torch.Tensor, head_dim: int, theta: float) -> torch.Tensor:
    """angle[t, i] = float(pos[t]) * theta^(-2i/d), formed in 32-bit as the reference does.

    src/operators.cpp:63-65.
    """
    half = head_dim // 2
    index = torch.arange(half, dtype=torch.float32)
    exponent = (-2.0 * index) / float(head_dim)
    frequency = torch.pow(torch.tensor(theta, dtype=torch.float32), exponent)
    return positions.to(torch.float32)[:, None] * frequency[None, :]


def plain_rope(x: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Half-split rotation of x[T, heads, d]: the pair is (i, i + d/2).

    src/operators.cpp:58-73: first' = first*cos - second*sin, second' = second*cos + first*sin.
    """
    tokens, heads, head_dim = x.shape
    assert head_dim % 2 == 0
    half = head_dim // 2
    angle = plain_rope_angles(positions, head_dim, theta).double()
    cosine = torch.cos(angle)[:, None, :]
    sine = torch.sin(angle)[:, None, :]
    x = x.double()
    first, second = x[..., :half], x[..., half:]
    return torch.cat([first * cosine - second * sine, second * cosine + first * sine], dim=-1)


def plain_softmax(values: torch.Tensor) -> torch.Tensor:
    """Stable softmax over the last axis: exp(v - max) / sum.  src/operators.cpp:87-98."""
    values = values.double()
    shifted = torch.exp(values - values.max(dim=-1, keepdim=True).values)
    return shifted / shifted.sum(dim=-1, keepdim=True)


def plain_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                    window: int | None = None) -> torch.Tensor:
    """Causal grouped-query attention over one whole sequence.

    q[T, nq, d], k and v[T, nkv, d] -> [T, nq, d].  Query head h reads key/value head
    h // (nq / nkv) (src/operators.cpp:117,123); score = dot * (1/sqrt(d)), scaled after the
    product (:119,131); softmax over the keys; output = sum of p * v (:138-143).  The query at
    position t sees keys 0..t only, because the reference passes `position + 1` keys
    (src/model.cpp:159-169).  `window` is not in the reference: when given, the query at t sees
    keys j with t - window < j <= t.
    """
    tokens, query_heads, head_dim = q.shape
    kv_heads = k.shape[1]
    assert query_heads % kv_heads == 0
    groups = query_heads // kv_heads
    scale = 1.0 / math.sqrt(float(head_dim))
    q, k, v = q.double(), k.double(), v.double()
    out = torch.zeros_like(q)
    for head in range(query_heads):
        kv_head = head // groups
        for t in range(tokens):
            first = 0 if window is None else max(0, t - window + 1)
            keys = k[first:t + 1, kv_head]
            scores = (keys @ q[t, head]) * scale
            probabilities = plain_softmax(scores)
            out[t, head] = probabilities @ v[first:t + 1, kv_head]
    return out


def plain_silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """(g / (1 + exp(-g))) * u.  src/operators.cpp:157-159."""
    gate, up = gate.double(), up.double()
    return (gate / (1.0 + torch.exp(-gate))) * up


def plain_linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """y[t, o] = sum_i x[t, i] * W[o, i] (+ b[o]); W is [out, in].  src/model.cpp:65-72."""
    y = x.double() @ weight.double().T
    if bias is not None:
        y = y + bias.double()
    return y


def plain_greedy(logits: torch.Tensor) -> int:
    """First index of the maximum (`std::max_element`).  src/operators.cpp:173-174."""
    logits = logits.double()
    best, best_index = None, -1
    for index, value in enumerate(logits.tolist()):
        if best is None or value > best:
            best, best_index = value, index
    return best_index


def plain_top_p_distribution(logits: torch.Tensor, temperature: float, top_p: float) -> torch.Tensor:
    """The distribution that the reference's sampler draws from.

    app/server.cpp:242-266: w_i = exp((l_i - max) / T); sort descending; keep the shortest
    prefix whose normalised cumulative mass reaches top_p (the element that crosses it is
    kept, at least one is kept); draw in proportion to w over the kept ones.
    Returns probabilities over the vocabulary, zero outside the kept set.
    """
    logits = logits.double()
    weights = torch.exp((logits - logits.max()) / temperature)
    total = weights.sum()
    order = sorted(range(weights.numel()), key=lambda i: -weights[i].item())
    cumulative, kept = 0.0, 0
    for kept in range(len(order)):
        cumulative += weights[order[kept]].item() / total.item()
        if cumulative >= top_p:
            kept += 1
            break
    else:
        kept = len(order)
    kept = max(kept, 1)
    out = torch.zeros_like(weights)
    for index in order[:kept]:
        out[index] = weights[index]
    return out / out.sum()


def stored_as(dtype: torch.dtype):
    """A function that rounds a tensor to `dtype` and widens it again: what storing an
    activation in that type between two kernels does to it."""
    return lambda tensor: tensor.to(dtype).double()


def plain_block(x: torch.Tensor, positions: torch.Tensor, w: dict, prefix: str, cfg: dict, trace: dict | None = None,
                trace_prefix: str = "", stored=None) -> torch.Tensor:
    """One pre-norm block: x + attn(norm(x)), then x + mlp(norm(x)).  src/model.cpp:132-203.
    `trace` receives the five tensors the reference's ModelTrace keeps per layer
    (src/model.cpp:136-138,176-177,184-185,200-201,204-205).

    `stored` (default: nothing) is applied to every activation that a 16-bit device path keeps in
    memory between two operators, as the reference's FP16 path keeps them
    (src/cuda/model.cu:412-447: normed input, q, k, v, attention output, both projections' results,
    the gated activation); the residual stays as it is.  With `stored_as(torch.bfloat16)` this is
    a model of what 16-bit storage alone costs in precision, every sum still being float64: the
    yardstick for a 16-bit engine's error over many layers, not a second implementation of it."""
    def keep(name, tensor):
        if trace is not None:
            trace[trace_prefix + name] = tensor
    if stored is None:
        stored = lambda tensor: tensor

    heads = cfg["num_attention_heads"]
    kv_heads = cfg.get("num_key_value_heads", heads)
    head_dim = cfg.get("head_dim", cfg["hidden_size"] // heads)
    eps, theta = cfg["rms_norm_eps"], cfg.get("rope_theta", 10000.0)
    tokens = x.shape[0]

    def bias(name):
        return w.get(prefix + name)

    normed = stored(plain_rms_norm(x, w[prefix + "input_layernorm.weight"], eps))
    keep("input_norm", normed)
    q = stored(plain_linear(normed, w[prefix + "self_attn.q_proj.weight"], bias("self_attn.q_proj.bias")))
    k = stored(plain_linear(normed, w[prefix + "self_attn.k_proj.weight"], bias("self_attn.k_proj.bias")))
    v = stored(plain_linear(normed, w[prefix + "self_attn.v_proj.weight"], bias("self_attn.v_proj.bias")))
    q = stored(plain_rope(q.view(tokens, heads, head_dim), positions, theta))
    k = stored(plain_rope(k.view(tokens, kv_heads, head_dim), positions, theta))
    attended = stored(plain_attention(q, k, v.view(tokens, kv_heads, head_dim)))
    projected = stored(plain_linear(attended.reshape(tokens, heads * head_dim),
                                    w[prefix + "self_attn.o_proj.weight"], bias("self_attn.o_proj.bias")))
    keep("attention_output", projected)
    x = x + projected
    normed = stored(plain_rms_norm(x, w[prefix + "post_attention_layernorm.weight"], eps))
    keep("post_attention_norm", normed)
    gate = stored(plain_linear(normed, w[prefix + "mlp.gate_proj.weight"]))
    up = stored(plain_linear(normed, w[prefix + "mlp.up_proj.weight"]))
    projected = stored(plain_linear(stored(plain_silu_mul(gate, up)), w[prefix + "mlp.down_proj.weight"]))
    keep("mlp_output", projected)
    keep("output", x + projected)
    return x + projected


def plain_forward(cfg: dict, w: dict, tokens: list[int], first_position: int = 0, trace: dict | None = None,
                  stored=None) -> torch.Tensor:
    """Logits [T, V] of one whole sequence.  src/model.cpp:80-234.

    Embedding row copy (:94-97), the blocks in order (:112-207), final norm (:217) and the
    output projection (:224-225); with tied embeddings the output projection is the
    embedding table.  `first_position` shifts every position; it is for the tests' invariants.
    `trace` receives the named tensors of the reference's ModelTrace ("embedding", "layerN.*",
    "final_norm", "logits": src/model.cpp:98-99,221-222,229-230).  `stored`: see `plain_block`.
    """
    ids = torch.tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens)) + first_position
    x = w["model.embed_tokens.weight"].double()[ids]
    if trace is not None:
        trace["embedding"] = x
    for layer in range(cfg["num_hidden_layers"]):
        x = plain_block(x, positions, w, f"model.layers.{layer}.", cfg, trace, f"layer{layer}.", stored)
    normed = plain_rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    if stored is not None:
        normed = stored(normed)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    logits = plain_linear(normed, head)
    if trace is not None:
        trace["final_norm"], trace["logits"] = normed, logits
    return logits


def plain_generate_greedy(cfg: dict, w: dict, prompt: list[int], max_tokens: int) -> list[int]:
    """Greedy continuation, recomputing the whole sequence for every token.

    app/reference_cli.cpp:88-110: sample from the last prompt position, feed the sample back.
    """
    sequence = list(prompt)
    generated = []
    for _ in range(max_tokens):
        token = plain_greedy(plain_forward(cfg, w, sequence)[-1])
        generated.append(token)
        sequence.append(token)
    return generated


def plain_forward_rows(cfg: dict, w: dict, tokens: list[int], rows: list[int]) -> torch.Tensor:
    """Logits [len(rows), V] of a ONE-layer model at the chosen positions only: what `plain_forward`
    gives at those rows, for sequences too long to compute whole.  Keys and values are made for
    every position (they need only the embedding and the first norm), queries, attention, the
    feed-forward and the head at the chosen rows; the same formulas as above, at the same places
    of the reference (src/model.cpp:132-225)."""
    assert cfg["num_hidden_layers"] == 1
    heads = cfg["num_attention_heads"]
    kv_heads = cfg.get("num_key_value_heads", heads)
    head_dim = cfg.get("head_dim", cfg["hidden_size"] // heads)
    eps, theta = cfg["rms_norm_eps"], cfg.get("rope_theta", 10000.0)
    prefix = "model.layers.0."
    count = len(tokens)
    positions = torch.arange(count)
    picked = torch.tensor(rows, dtype=torch.long)
    x = w["model.embed_tokens.weight"].double()[torch.tensor(tokens, dtype=torch.long)]
    normed = plain_rms_norm(x, w[prefix + "input_layernorm.weight"], eps)
    k = plain_linear(normed, w[prefix + "self_attn.k_proj.weight"], w.get(prefix + "self_attn.k_proj.bias"))
    v = plain_linear(normed, w[prefix + "self_attn.v_proj.weight"], w.get(prefix + "self_attn.v_proj.bias")).view(count, kv_heads, head_dim)
    k = plain_rope(k.view(count, kv_heads, head_dim), positions, theta)
    q = plain_linear(normed[picked], w[prefix + "self_attn.q_proj.weight"], w.get(prefix + "self_attn.q_proj.bias"))
    q = plain_rope(q.view(len(rows), heads, head_dim), positions[picked], theta)
    groups = heads // kv_heads
    scale = 1.0 / math.sqrt(float(head_dim))
    attended = torch.zeros(len(rows), heads, head_dim, dtype=torch.float64)
    for index, t in enumerate(rows):
        for head in range(heads):
            scores = (k[:t + 1, head // groups] @ q[index, head]) * scale          # src/operators.cpp:119,131
            attended[index, head] = plain_softmax(scores) @ v[:t + 1, head // groups]
    x = x[picked] + plain_linear(attended.reshape(len(rows), heads * head_dim), w[prefix + "self_attn.o_proj.weight"],
                                 w.get(prefix + "self_attn.o_proj.bias"))
    normed = plain_rms_norm(x, w[prefix + "post_attention_layernorm.weight"], eps)
    x = x + plain_linear(plain_silu_mul(plain_linear(normed, w[prefix + "mlp.gate_proj.weight"]),
                                        plain_linear(normed, w[prefix + "mlp.up_proj.weight"])), w[prefix + "mlp.down_proj.weight"])
    head_matrix = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return plain_linear(plain_rms_norm(x, w["model.norm.weight"], eps), head_matrix)
