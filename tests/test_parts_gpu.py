"""Each part alone against its plain reference, and the generality of the parts: a mixer with state
of its own, a feed-forward with routing, a position encoding that is no rotation, and an architecture of its own, all defined
here and registered without a change to the engine's files; a layer order that names a layer twice
and lets a run read another run's cache; a windowed attention whose pages come back."""
import json
import math
import os
from dataclasses import dataclass

import pytest
import torch

from plain_llama import plain_attention, plain_linear, plain_rms_norm, plain_rope, plain_silu_mul
from gpu_helpers import assert_close, load_plain
from tlie_amd import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


def part_weights(part_class, spec, prefix, dtype, seed):
    from tlie_amd.weights import random_tensors
    tensors = random_tensors(part_class.tensor_specs(spec, prefix), seed, std=0.2, norm_std=0.2, dtype=dtype)
    return tensors, {name: tensor.to(DEV) for name, tensor in tensors.items()}


class MixerHarness:
    """A cache manager and step contexts around one mixer, nothing else of a model."""

    def __init__(self, mixer, dtype, num_pages=40, page_size=8):
        from tlie_amd.cache import CacheManager, RunNeed
        self.mixer = mixer
        self.cache = CacheManager([RunNeed(0, mixer.cache_need(), mixer.state_need())], page_size, num_pages, 4, dtype, DEV)

    def run(self, items):
        """items: [(request, x [n, hidden])]; returns the mixer's output rows per request."""
        from tlie_amd.engine.step import StepEntry, build_context
        from tlie_amd.ops import as_product
        entries = []
        for request, x in items:
            if not self.cache.is_live(request):
                self.cache.admit(request)
            self.cache.reserve(request, x.shape[0])
            entries.append(StepEntry(request, [0] * x.shape[0], []))
        ctx = build_context(self.cache, entries, DEV)
        out = as_product(self.mixer.forward(torch.cat([x for _, x in items]).contiguous(), ctx, self.cache.bindings[0])).dense()
        for request, x in items:
            self.cache.commit(request, x.shape[0])
        self.cache.check()
        return torch.split(out, [x.shape[0] for _, x in items])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rms_norm_part(dtype):
    from tlie_amd.config import PartSpec
    from tlie_amd.parts.norm import RMSNorm
    spec = PartSpec("rms_norm", {"size": 200, "eps": 3e-4})
    host, device = part_weights(RMSNorm, spec, "n.", DT[dtype], 1)
    part = RMSNorm(spec, DT[dtype], DEV)
    part.load(device, "n.")
    x = torch.randn(5, 200)
    assert_close(part.forward(x.to(DEV)), plain_rms_norm(x, host["n.weight"].double(), 3e-4), TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_mlp_part(dtype):
    from tlie_amd.config import PartSpec
    from tlie_amd.ops import as_product
    from tlie_amd.parts.mlp import GatedMLP
    spec = PartSpec("gated_mlp", {"hidden_size": 72, "intermediate_size": 200, "activation": "silu"})
    host, device = part_weights(GatedMLP, spec, "m.", DT[dtype], 2)
    part = GatedMLP(spec, DT[dtype], DEV)
    part.load(device, "m.")
    x = torch.randn(11, 72).to(DT[dtype])
    got = as_product(part.forward(x.to(DEV), None)).dense()
    hidden = plain_silu_mul(plain_linear(x.double(), host["m.gate_proj.weight"]), plain_linear(x.double(), host["m.up_proj.weight"]))
    if dtype == "bfloat16":
        hidden = hidden.to(torch.bfloat16).double()          # the activation between the two products is stored in bfloat16
    assert_close(got, plain_linear(hidden, host["m.down_proj.weight"]), TOL[dtype])


def plain_attention_part(x, host, prefix, nq, nkv, d, theta, window, bias, rot_dim=None):
    tokens = x.shape[0]
    def lin(name):
        return plain_linear(x.double(), host[f"{prefix}{name}_proj.weight"], host.get(f"{prefix}{name}_proj.bias") if bias else None)
    positions = torch.arange(tokens)
    q, k, v = lin("q").view(tokens, nq, d), lin("k").view(tokens, nkv, d), lin("v").view(tokens, nkv, d)
    if theta is not None:
        rot = rot_dim or d
        q = torch.cat([plain_rope(q[..., :rot], positions, theta), q[..., rot:]], dim=-1)
        k = torch.cat([plain_rope(k[..., :rot], positions, theta), k[..., rot:]], dim=-1)
    attended = plain_attention(q, k, v, window=window).reshape(tokens, nq * d)
    return plain_linear(attended, host[prefix + "o_proj.weight"], host.get(prefix + "o_proj.bias") if bias else None)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", [
    dict(hidden=40, nq=5, nkv=5, d=16, bias=False, window=None, theta=10000.0),        # plain multi-head
    dict(hidden=72, nq=6, nkv=2, d=48, bias=True, window=None, theta=500000.0),
    dict(hidden=64, nq=4, nkv=1, d=32, bias=False, window=11, theta=10000.0),          # a window; pages come back
    dict(hidden=64, nq=2, nkv=2, d=64, bias=True, window=None, theta=None),            # no position encoding
    dict(hidden=48, nq=3, nkv=1, d=32, bias=False, window=None, theta=10000.0, rot_dim=16),   # part of the head turns
])
def test_attention_part_whole_and_in_portions(dtype, case):
    from tlie_amd.config import PartSpec
    from tlie_amd.parts.attention import Attention
    position = PartSpec("none") if case["theta"] is None else PartSpec("rotary", {
        "head_dim": case["d"], "theta": case["theta"], **({"rot_dim": case["rot_dim"]} if "rot_dim" in case else {})})
    spec = PartSpec("attention", {"hidden_size": case["hidden"], "num_heads": case["nq"], "num_kv_heads": case["nkv"],
                                  "head_dim": case["d"], "bias": case["bias"], "window": case["window"], "position": position})
    host, device = part_weights(Attention, spec, "a.", DT[dtype], 3)
    part = Attention(spec, DT[dtype], DEV)
    part.load(device, "a.")
    tokens = 61
    x = torch.randn(tokens, case["hidden"]).to(DT[dtype])
    want = plain_attention_part(x, host, "a.", case["nq"], case["nkv"], case["d"], case["theta"], case["window"], case["bias"],
                                case.get("rot_dim"))
    harness = MixerHarness(part, DT[dtype])
    (whole,) = harness.run([("w", x.to(DEV))])
    assert_close(whole, want, TOL[dtype], "whole")
    pieces, cursor = [], 0
    for size in (9, 2, 1, 17, 1, 1, 8, 22):
        other = torch.randn(3, case["hidden"]).to(DT[dtype]).to(DEV)            # another request beside it in the batch
        out = harness.run([("other", other), ("p", x[cursor:cursor + size].to(DEV))])
        pieces.append(out[1])
        cursor += size
    assert cursor == tokens
    assert_close(torch.cat(pieces), want, TOL[dtype], "in portions")
    if case["window"] is not None:
        held = [page for page in harness.cache.page_list("p", 0) if page >= 0]
        assert len(held) <= (case["window"] + 7) // 8 + 1, "pages a window has passed were not given back"


def test_rotary_part_table_and_refusals():
    """The position encoding alone: its table is the plain angles at position 1, for the part of
    the head that turns; sizes that cannot be paired are refused."""
    from tlie_amd import EngineError
    from tlie_amd.config import PartSpec
    from tlie_amd.parts.rotary import NoPositions, Rotary
    from plain_llama import plain_rope_angles
    for head_dim, rot_dim, theta in ((64, 64, 10000.0), (48, 16, 500000.0), (16, 2, 3.5)):
        part = Rotary(PartSpec("rotary", {"head_dim": head_dim, "theta": theta, "rot_dim": rot_dim}), torch.bfloat16, DEV)
        inv_freq, turned = part.rotary_table()
        assert turned == rot_dim and inv_freq.dtype == torch.float32 and inv_freq.shape == (rot_dim // 2,)
        assert torch.equal(inv_freq.cpu(), plain_rope_angles(torch.tensor([1]), rot_dim, theta)[0])
    assert Rotary(PartSpec("rotary", {"head_dim": 32, "theta": 1e4}), torch.float32, DEV).rotary_table()[1] == 32
    assert NoPositions(PartSpec("none"), torch.float32, DEV).rotary_table() is None
    for bad in ({"head_dim": 32, "theta": 1e4, "rot_dim": 7}, {"head_dim": 32, "theta": 1e4, "rot_dim": 34},
                {"head_dim": 32, "theta": 0.0}):
        with pytest.raises(EngineError):
            Rotary(PartSpec("rotary", bad), torch.float32, DEV)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("tied", [False, True])
def test_embedding_and_head_parts(dtype, tied):
    """The two ends alone: rows of the table, unscaled, as a 32-bit residual; logits in 32-bit from
    the head's own matrix or, tied, from the table."""
    from tlie_amd.config import PartSpec
    from tlie_amd.parts.embedding import LMHead, TokenEmbedding
    spec = PartSpec("token_embedding", {"vocab_size": 301, "hidden_size": 72})
    head_spec = PartSpec("lm_head", {"vocab_size": 301, "hidden_size": 72, "tied": tied})
    host, device = part_weights(TokenEmbedding, spec, "", DT[dtype], 4)
    head_host, head_device = part_weights(LMHead, head_spec, "", DT[dtype], 5)
    assert [t.optional for t in LMHead.tensor_specs(head_spec)] == [tied]
    embedding, head = TokenEmbedding(spec, DT[dtype], DEV), LMHead(head_spec, DT[dtype], DEV)
    embedding.load(device)
    head.load({**device, **({} if tied else head_device)})
    tokens = torch.tensor([0, 300, 17, 17, 5, 299], dtype=torch.int32, device=DEV)
    residual = embedding.forward(tokens)
    assert residual.dtype == torch.float32
    assert torch.equal(residual.cpu(), host[TokenEmbedding.NAME].float()[tokens.long().cpu()])
    x = torch.randn(6, 72).to(DT[dtype])
    logits = head.forward(x.to(DEV))
    matrix = host[TokenEmbedding.NAME] if tied else head_host[LMHead.NAME]
    assert logits.dtype == torch.float32 and logits.shape == (6, 301)
    assert_close(logits, plain_linear(x.double(), matrix.double()), TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows", [40, 7])
def test_pre_norm_block_part(dtype, rows):
    """The arrangement alone: one block of norm, attention, norm, feed-forward around a 32-bit
    residual, against the plain block; the block's last product is handed on, not added.  With 7
    rows a bfloat16 step takes the route on which the products fold the norms and the adds in."""
    from tlie_amd.cache import CacheManager, RunNeed
    from tlie_amd.config import LlamaConfig
    from tlie_amd.engine.step import StepEntry, build_context
    from tlie_amd.ops import ResidualUpdated, as_product
    from tlie_amd.parts.block import PreNormBlock
    from tlie_amd.weights import random_tensors
    from plain_llama import plain_block
    raw = dict(model_type="llama", hidden_size=72, intermediate_size=200, num_hidden_layers=1, num_attention_heads=6,
               num_key_value_heads=2, head_dim=16, max_position_embeddings=64, vocab_size=50, rms_norm_eps=2e-5,
               rope_theta=777.0, attention_bias=True)
    layer = LlamaConfig.from_dict(raw).to_spec().layers[0]
    host = random_tensors(PreNormBlock.tensor_specs(layer), 6, std=0.2, norm_std=0.2, dtype=DT[dtype])
    block = PreNormBlock(layer, DT[dtype], DEV)
    block.load({name: tensor.to(DEV) for name, tensor in host.items()})
    cache = CacheManager([RunNeed(0, block.mixer.cache_need(), block.mixer.state_need())], 16, 8, 2, DT[dtype], DEV)
    cache.admit("r")
    cache.reserve("r", rows)
    ctx = build_context(cache, [StepEntry("r", [0] * rows, [])], DEV)
    assert ops.few_rows_route(rows, DT[dtype]) == (rows <= 16 and dtype == "bfloat16")
    x = torch.randn(rows, 72)
    residual = x.clone().to(DEV)
    pending = block.forward(residual, None, ctx, cache.bindings[0])
    if isinstance(pending, ResidualUpdated):
        got = residual                                       # the feed-forward added its result itself
    else:
        got = residual + as_product(pending).dense(torch.float32)
    want = plain_block(x.double(), torch.arange(rows), {name: tensor.double() for name, tensor in host.items()},
                       layer.prefix, raw)
    assert_close(got, want, TOL[dtype])


# ---------------------------------------------------------------------------------------------------
# Parts and an architecture defined by the test.

def register_toys():
    from tlie_amd import ops
    from tlie_amd.config import LayerSpec, ModelSpec, PartSpec, Run, TensorSpec
    from tlie_amd.parts import FeedForward, Mixer, PositionEncoding, StateNeed
    from tlie_amd.parts.linear import Linear
    from tlie_amd.registry import register

    @register("mixer", "toy_running_mean")
    class RunningMean(Mixer):
        """out[t] = W . mean(x[0..t]): the only thing carried from step to step is the running sum,
        a state of fixed size per request."""

        @classmethod
        def tensor_specs(cls, spec, prefix):
            return [TensorSpec(prefix + "mix.weight", (spec["hidden_size"], spec["hidden_size"]))]

        def load(self, weights, prefix):
            self.mix = Linear(weights[prefix + "mix.weight"], None, self.dtype)

        def state_need(self):
            return StateNeed((self.spec["hidden_size"],), torch.float32)

        def forward(self, x, ctx, binding):
            means = torch.empty_like(x, dtype=torch.float32)
            starts = ctx.host["seq_start"]
            for index in range(ctx.num_seqs):
                begin, end, slot = int(starts[index]), int(starts[index + 1]), int(ctx.host["seq_slot"][index])
                sums = torch.cumsum(x[begin:end].float(), dim=0) + binding.state[slot]
                binding.state[slot] = sums[-1]
                means[begin:end] = sums / (ctx.positions[begin:end].float() + 1.0)[:, None]
            return self.mix(means.to(self.dtype).contiguous())

    @register("feed_forward", "toy_routed")
    class Routed(FeedForward):
        """A feed-forward with routing: the router's logits (32-bit) choose one of `experts` small
        two-matrix networks per token; its result is weighted by the router's softmax probability."""

        @classmethod
        def tensor_specs(cls, spec, prefix):
            hidden, inter, experts = spec["hidden_size"], spec["intermediate_size"], spec["experts"]
            specs = [TensorSpec(prefix + "router.weight", (experts, hidden))]
            for e in range(experts):
                specs += [TensorSpec(f"{prefix}experts.{e}.up.weight", (inter, hidden)),
                          TensorSpec(f"{prefix}experts.{e}.down.weight", (hidden, inter))]
            return specs

        def load(self, weights, prefix):
            self.router = Linear(weights[prefix + "router.weight"], None, self.dtype)
            self.experts = [(Linear(weights[f"{prefix}experts.{e}.up.weight"], None, self.dtype),
                             Linear(weights[f"{prefix}experts.{e}.down.weight"], None, self.dtype))
                            for e in range(self.spec["experts"])]

        def forward(self, x, ctx):
            logits = ops.as_product(self.router(x, out_dtype=torch.float32)).dense(torch.float32)
            probability, choice = torch.softmax(logits, dim=-1).max(dim=-1)
            out = torch.zeros((x.shape[0], self.spec["hidden_size"]), dtype=torch.float32, device=x.device)
            for e, (up, down) in enumerate(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                hidden = torch.relu(ops.as_product(up(x[rows].contiguous())).dense(torch.float32)).to(self.dtype)
                out[rows] = ops.as_product(down(hidden)).dense(torch.float32) * probability[rows, None]
            return out.to(self.dtype)

    @register("position_encoding", "toy_scale_by_position")
    class ScaleByPosition(PositionEncoding):
        """Not a rotation: keys are scaled by 1 / (1 + position / 64)."""

        def apply_qk(self, q, k, positions):
            scale = (1.0 / (1.0 + positions.float() / 64.0))[:, None, None]
            return q, (k.float() * scale).to(k.dtype)

    @register("architecture", "ToyForCausalLM")
    @dataclass(frozen=True)
    class ToyConfig:
        hidden_size: int
        vocab_size: int
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["hidden_size"], raw["vocab_size"], raw["eps"])

        def to_dict(self):
            return {"architectures": ["ToyForCausalLM"], "hidden_size": self.hidden_size, "vocab_size": self.vocab_size, "eps": self.eps}

        def to_spec(self):
            norm = PartSpec("rms_norm", {"size": self.hidden_size, "eps": self.eps})
            attention = PartSpec("attention", {"hidden_size": self.hidden_size, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16,
                                               "bias": False, "window": None, "position": PartSpec("toy_scale_by_position")})
            mean = PartSpec("toy_running_mean", {"hidden_size": self.hidden_size})
            mlp = PartSpec("gated_mlp", {"hidden_size": self.hidden_size, "intermediate_size": 40, "activation": "silu"})
            routed = PartSpec("toy_routed", {"hidden_size": self.hidden_size, "intermediate_size": 24, "experts": 3})
            layers = (LayerSpec("model.layers.0.", "pre_norm", attention, mlp, norm, norm),
                      LayerSpec("model.layers.1.", "pre_norm", mean, routed, norm, norm))
            # layer 0 runs three times: with a cache of its own, again with another cache of its own,
            # and once more reading the first run's cache; the toy mixer's layer runs in between
            runs = (Run(0, 0), Run(1, 1), Run(0, 2), Run(0, 0))
            return ModelSpec("ToyForCausalLM", self.hidden_size, self.vocab_size, 128,
                             PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size}),
                             layers, runs, norm,
                             PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "tied": False}))
    return ToyConfig


def plain_toy_forward(raw, w, tokens):
    """The toy architecture, whole sequence, from the plain functions."""
    hidden, eps = raw["hidden_size"], raw["eps"]
    count = len(tokens)
    positions = torch.arange(count)
    x = w["model.embed_tokens.weight"][tokens]
    kept = {}

    def attention_run(x, own_cache, read=None):
        p = "model.layers.0."
        normed = plain_rms_norm(x, w[p + "input_layernorm.weight"], eps)
        q = plain_linear(normed, w[p + "self_attn.q_proj.weight"]).view(count, 2, 16)
        k = plain_linear(normed, w[p + "self_attn.k_proj.weight"]).view(count, 1, 16) / (1.0 + positions.double() / 64.0)[:, None, None]
        v = plain_linear(normed, w[p + "self_attn.v_proj.weight"]).view(count, 1, 16)
        if own_cache is not None:
            kept[own_cache] = (k, v)
        else:
            k, v = kept[read]
        x = x + plain_linear(plain_attention(q, k, v).reshape(count, 32), w[p + "self_attn.o_proj.weight"])
        return x + mlp(x, p)

    def mlp(x, p):
        normed = plain_rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        return plain_linear(plain_silu_mul(plain_linear(normed, w[p + "mlp.gate_proj.weight"]),
                                           plain_linear(normed, w[p + "mlp.up_proj.weight"])), w[p + "mlp.down_proj.weight"])

    x = attention_run(x, own_cache=0)
    p = "model.layers.1."
    normed = plain_rms_norm(x, w[p + "input_layernorm.weight"], eps)
    means = torch.cumsum(normed, dim=0) / (positions.double() + 1.0)[:, None]
    x = x + plain_linear(means, w[p + "self_attn.mix.weight"])
    normed = plain_rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
    probability, choice = torch.softmax(plain_linear(normed, w[p + "mlp.router.weight"]), dim=-1).max(dim=-1)
    assert len(set(choice.tolist())) > 1, "the routing test wants tokens on more than one expert"
    routed = torch.stack([plain_linear(torch.relu(plain_linear(normed[t], w[f"{p}mlp.experts.{int(choice[t])}.up.weight"])),
                                       w[f"{p}mlp.experts.{int(choice[t])}.down.weight"]) * probability[t] for t in range(count)])
    x = x + routed
    x = attention_run(x, own_cache=2)
    x = attention_run(x, own_cache=None, read=0)
    return plain_linear(plain_rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])


def test_toy_parts_register_build_and_step(tmp_path):
    from tlie_amd import Engine, write_random_model
    from gpu_helpers import Replayer
    toy = register_toys()
    config = toy(hidden_size=32, vocab_size=90, eps=1e-5)
    write_random_model(str(tmp_path), config, seed=5, std=0.15, norm_std=0.1, dtype=torch.float32)
    raw, weights = load_plain(str(tmp_path))
    engine = Engine(str(tmp_path), dtype="float32", max_tokens=256, page_size=8, max_requests=3)
    assert [binding.group for binding in engine.cache.bindings] == [0, None, 0, 0]
    assert engine.cache.bindings[3].cache is engine.cache.bindings[0].cache and not engine.cache.bindings[3].writes
    assert engine.cache.bindings[2].cache is not engine.cache.bindings[0].cache
    assert engine.cache.bindings[1].state.shape == (3, 32)
    tokens = [(7 * i * i + 3) % 90 for i in range(50)]
    other = [(5 * i + 1) % 90 for i in range(23)]
    want, want_other = plain_toy_forward(raw, weights, tokens), plain_toy_forward(raw, weights, other)
    replay = Replayer(engine)
    replay.step([("whole", tokens, list(range(50)))], end=["whole"])
    assert_close(replay.logits_of("whole", range(50)), want, 2e-5, "whole")
    # in portions, with another request beside it that ends and whose slot (and state row) is used again
    replay.step([("a", tokens[:13], list(range(13))), ("b", other, list(range(23)))], end=["b"])
    replay.step([("a", tokens[13:15], [0, 1]), ("c", other[:9], list(range(9)))])
    replay.step([("c", other[9:], list(range(14))), ("a", tokens[15:16], [0])], end=["c"])
    replay.step([("a", tokens[16:], list(range(34)))], end=["a"])
    assert_close(replay.logits_of("a", range(50)), want, 2e-5, "in portions")
    assert_close(replay.logits_of("b", range(23)), want_other, 2e-5, "beside it")
    assert_close(replay.logits_of("c", range(23)), want_other, 2e-5, "in a slot that was used before")
    assert engine.cache.free_slots == 3


def register_recorded_state_toy():
    """A mixer with state of its own that may be recorded: every operation is a launch on the
    current stream whose sizes depend on the token and sequence counts alone.  It reads the
    request slots from the device (`token_slot`, `seq_slot`) and moves the state of live rows
    only: a recorded step's padding has slot -1."""
    from tlie_amd.config import LayerSpec, ModelSpec, PartSpec, Run, TensorSpec
    from tlie_amd.parts import Mixer, PositionEncoding, StateNeed
    from tlie_amd.parts.linear import Linear
    from tlie_amd.registry import register

    @register("position_encoding", "toy_recorded_scale_by_position")
    class RecordedScaleByPosition(PositionEncoding):
        """Not a rotation: keys are scaled by 1 / (1 + position / 64), with tensor operations whose
        sizes depend on the token count alone, so it says that it may be recorded (and the attention
        around it then may be too)."""
        graph_safe = True

        def apply_qk(self, q, k, positions):
            scale = (1.0 / (1.0 + positions.float() / 64.0))[:, None, None]
            return q, (k.float() * scale).to(k.dtype)

    @register("mixer", "toy_recorded_running_mean")
    class RecordedRunningMean(Mixer):
        """out[t] = W . mean(x[0..t]) with the running sum as the request's state."""
        graph_safe = True

        @classmethod
        def tensor_specs(cls, spec, prefix):
            return [TensorSpec(prefix + "mix.weight", (spec["hidden_size"], spec["hidden_size"]))]

        def load(self, weights, prefix):
            self.mix = Linear(weights[prefix + "mix.weight"], None, self.dtype)

        def state_need(self):
            return StateNeed((self.spec["hidden_size"],), torch.float32)

        def forward(self, x, ctx, binding):
            count = x.shape[0]
            live = ctx.token_slot >= 0
            rows = ctx.token_slot.long().clamp(min=0)
            # padding tokens count for nothing (their rows of x may hold anything, not even finite values:
            # no attention tile serves them, so they are taken out, not multiplied by zero)
            values = torch.where(live[:, None], x.float(), torch.zeros((), device=x.device))
            index = torch.arange(count, device=x.device)
            before = (ctx.token_seq[:, None] == ctx.token_seq[None, :]) & (index[None, :] <= index[:, None]) & live[None, :]
            sums = (before[:, :, None] * values[None, :, :]).sum(dim=1) + binding.state[rows]
            # the state moves for sequences that ran, once each; a padding sequence adds zeros
            sequence = torch.arange(ctx.num_seqs, device=x.device)
            member = (ctx.token_seq[None, :] == sequence[:, None]) & live[None, :]
            totals = (member[:, :, None] * values[None, :, :]).sum(dim=1) * (ctx.seq_slot >= 0)[:, None]
            binding.state.index_add_(0, ctx.seq_slot.long().clamp(min=0), totals)
            means = sums / (ctx.positions.float() + 1.0)[:, None]
            return self.mix(means.to(self.dtype).contiguous())

    @register("architecture", "ToyRecordedStateForCausalLM")
    @dataclass(frozen=True)
    class RecordedStateConfig:
        hidden_size: int
        vocab_size: int
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["hidden_size"], raw["vocab_size"], raw["eps"])

        def to_dict(self):
            return {"architectures": ["ToyRecordedStateForCausalLM"], "hidden_size": self.hidden_size,
                    "vocab_size": self.vocab_size, "eps": self.eps}

        def to_spec(self):
            norm = PartSpec("rms_norm", {"size": self.hidden_size, "eps": self.eps})
            attention = PartSpec("attention", {"hidden_size": self.hidden_size, "num_heads": 2, "num_kv_heads": 1, "head_dim": 16,
                                               "bias": False, "window": None,
                                               "position": PartSpec("toy_recorded_scale_by_position")})
            mean = PartSpec("toy_recorded_running_mean", {"hidden_size": self.hidden_size})
            mlp = PartSpec("gated_mlp", {"hidden_size": self.hidden_size, "intermediate_size": 40, "activation": "silu"})
            layers = (LayerSpec("model.layers.0.", "pre_norm", attention, mlp, norm, norm),
                      LayerSpec("model.layers.1.", "pre_norm", mean, mlp, norm, norm))
            return ModelSpec("ToyRecordedStateForCausalLM", self.hidden_size, self.vocab_size, 128,
                             PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size}),
                             layers, (Run(0, 0), Run(1, 1)), norm,
                             PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "tied": False}))
    return RecordedStateConfig


def plain_recorded_state_forward(raw, w, tokens):
    count, eps = len(tokens), raw["eps"]
    x = w["model.embed_tokens.weight"][tokens]

    def mlp(x, p):
        normed = plain_rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        return plain_linear(plain_silu_mul(plain_linear(normed, w[p + "mlp.gate_proj.weight"]),
                                           plain_linear(normed, w[p + "mlp.up_proj.weight"])), w[p + "mlp.down_proj.weight"])
    p = "model.layers.0."
    normed = plain_rms_norm(x, w[p + "input_layernorm.weight"], eps)
    q = plain_linear(normed, w[p + "self_attn.q_proj.weight"]).view(count, 2, 16)
    k = plain_linear(normed, w[p + "self_attn.k_proj.weight"]).view(count, 1, 16) / (1.0 + torch.arange(count).double() / 64.0)[:, None, None]
    v = plain_linear(normed, w[p + "self_attn.v_proj.weight"]).view(count, 1, 16)
    x = x + plain_linear(plain_attention(q, k, v).reshape(count, 32), w[p + "self_attn.o_proj.weight"])
    x = x + mlp(x, p)
    p = "model.layers.1."
    normed = plain_rms_norm(x, w[p + "input_layernorm.weight"], eps)
    means = torch.cumsum(normed, dim=0) / (torch.arange(count).double() + 1.0)[:, None]
    x = x + plain_linear(means, w[p + "self_attn.mix.weight"])
    x = x + mlp(x, p)
    return plain_linear(plain_rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_state_of_fixed_size_in_recorded_steps(tmp_path, dtype):
    """A request's state row moves only for rows that ran (reference: `next_positions` moves for
    the step's own slots only, src/cuda/model.cu:550-554,721-723).  A recorded step pads its
    sequences and tokens; the request in slot 0 runs beside that padding, in recorded steps of
    portions and of single tokens, several replays each, and its logits stay the plain ones:
    they would not if padding rows carried slot 0, as any live row may."""
    from tlie_amd import Engine, write_random_model
    from gpu_helpers import Replayer
    config = register_recorded_state_toy()(hidden_size=32, vocab_size=80, eps=1e-5)
    write_random_model(str(tmp_path), config, seed=21, std=0.15, norm_std=0.1,
                       dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    raw, weights = load_plain(str(tmp_path))
    tolerance = 2e-5 if dtype == "float32" else 3e-2
    engine = Engine(str(tmp_path), dtype=dtype, max_tokens=512, page_size=16, max_requests=4)
    assert engine.runner.use_graphs and engine.cache.bindings[1].state.shape == (4, 32)
    streams = {"a": [(7 * i * i + 3) % 80 for i in range(60)], "b": [(5 * i + 1) % 80 for i in range(45)],
               "c": [(11 * i + 2 * (i % 3)) % 80 for i in range(33)]}
    want = {request: plain_recorded_state_forward(raw, weights, tokens) for request, tokens in streams.items()}
    replay = Replayer(engine)
    engine.admit("a")
    assert engine.cache.slot("a") == 0
    # portions: 5 + 3 tokens in a recording of 16 tokens and 8 sequences, replayed with other cuts
    replay.step([("a", streams["a"][:5], [4]), ("b", streams["b"][:3], [2])])
    replay.step([("a", streams["a"][5:12], [6]), ("b", streams["b"][3:9], [5])])
    replay.step([("b", streams["b"][9:20], [10]), ("c", streams["c"][:2], [1]), ("a", streams["a"][12:13], [0])])
    recording = next(iter(engine.runner._portion_graphs.values()))
    assert recording.graph is not None, "the steps of portions were not replayed from a recording"
    assert (recording.host["seq_slot"][3:] == -1).all() and (recording.host["token_slot"][14:] == -1).all()
    assert sorted(recording.host["seq_slot"][:3].tolist()) == [0, 1, 2]
    done = {"a": 13, "b": 20, "c": 2}
    # single tokens: three requests in a recording of four rows (one row of padding), many replays
    for _ in range(12):
        replay.step([(request, streams[request][done[request]:done[request] + 1], [0]) for request in ("c", "a", "b")])
        for request in done:
            done[request] += 1
    decode = next(iter(engine.runner._graphs.values()))
    assert decode.bucket == 4 and decode.graph is not None and decode.host["seq_slot"][3] == -1 and decode.host["token_slot"][3] == -1
    # "c" ends; its slot and state row are taken by "d", which starts from zero beside the others
    engine.finish("c")
    streams["d"], want["d"] = streams["c"], want["c"]
    done["d"] = 0
    replay.step([("a", streams["a"][done["a"]:done["a"] + 1], [0]), ("d", streams["d"][:9], [8])])
    done["a"], done["d"] = done["a"] + 1, 9
    for _ in range(10):
        replay.step([(request, streams[request][done[request]:done[request] + 1], [0]) for request in ("a", "b", "d")])
        for request in ("a", "b", "d"):
            done[request] += 1
    keys = sorted(replay.rows, key=str)
    for request in ("a", "b", "c", "d"):
        places = [place for name, place in keys if name == request]
        assert len(places) >= 11
        assert_close(replay.logits_of(request, places), want[request][places], tolerance, f"request {request}")
    # the state rows hold the running sums of exactly the tokens that ran
    for request in ("a", "b", "d"):
        engine.finish(request)
    assert engine.cache.free_slots == 4


def register_latent_cache_toy():
    """A mixer that keeps one vector per position in pages of its own shape and type, and an
    architecture that runs it beside an attention layer: the two runs share page numbers (one
    group), their pools have nothing else in common."""
    from tlie_amd.config import LayerSpec, ModelSpec, PartSpec, Run, TensorSpec
    from tlie_amd.parts import CacheNeed, Mixer
    from tlie_amd.parts.linear import Linear
    from tlie_amd.registry import register

    @register("mixer", "toy_latent_mean")
    class LatentMean(Mixer):
        """Caches latent[t] = P . x[t] (float32, `latent` values per position, one plane) and
        gives out[t] = W . mean(latent[0..t]), read back from the pages through the block table."""

        @classmethod
        def tensor_specs(cls, spec, prefix):
            return [TensorSpec(prefix + "down.weight", (spec["latent"], spec["hidden_size"])),
                    TensorSpec(prefix + "up.weight", (spec["hidden_size"], spec["latent"]))]

        def load(self, weights, prefix):
            self.down = Linear(weights[prefix + "down.weight"], None, self.dtype)
            self.up = Linear(weights[prefix + "up.weight"], None, self.dtype)

        def cache_need(self):
            return CacheNeed((), int(self.spec["latent"]), None, torch.float32)

        def forward(self, x, ctx, binding):
            width = int(self.spec["latent"])
            latent = ops.as_product(self.down(x, out_dtype=torch.float32)).dense(torch.float32)
            rows = binding.cache.view(-1, width)                       # [pages * page_size, latent]
            page_size = binding.cache.shape[1] // width
            group = binding.group
            rows[ctx.groups[group].slot_map.long()] = latent
            table, starts = ctx.host[f"block_table{group}"], ctx.host["seq_start"]
            means = torch.empty_like(latent)
            for index in range(ctx.num_seqs):
                begin, end, length = int(starts[index]), int(starts[index + 1]), int(ctx.host["seq_len"][index])
                where = torch.tensor([int(table[index, p // page_size]) * page_size + p % page_size for p in range(length)],
                                     device=x.device)
                running = torch.cumsum(rows[where], dim=0) / torch.arange(1, length + 1, device=x.device)[:, None]
                means[begin:end] = running[length - (end - begin):]
            return self.up(means.to(self.dtype).contiguous())

    @register("architecture", "ToyLatentForCausalLM")
    @dataclass(frozen=True)
    class LatentConfig:
        hidden_size: int
        vocab_size: int
        latent: int

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["hidden_size"], raw["vocab_size"], raw["latent"])

        def to_dict(self):
            return {"architectures": ["ToyLatentForCausalLM"], "hidden_size": self.hidden_size, "vocab_size": self.vocab_size,
                    "latent": self.latent}

        def to_spec(self):
            norm = PartSpec("rms_norm", {"size": self.hidden_size, "eps": 1e-5})
            attention = PartSpec("attention", {"hidden_size": self.hidden_size, "num_heads": 2, "num_kv_heads": 2, "head_dim": 16,
                                               "bias": False, "window": None,
                                               "position": PartSpec("rotary", {"head_dim": 16, "theta": 50.0})})
            latent = PartSpec("toy_latent_mean", {"hidden_size": self.hidden_size, "latent": self.latent})
            mlp = PartSpec("gated_mlp", {"hidden_size": self.hidden_size, "intermediate_size": 48, "activation": "silu"})
            layers = (LayerSpec("model.layers.0.", "pre_norm", latent, mlp, norm, norm),
                      LayerSpec("model.layers.1.", "pre_norm", attention, mlp, norm, norm))
            return ModelSpec("ToyLatentForCausalLM", self.hidden_size, self.vocab_size, 128,
                             PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size}),
                             layers, (Run(0, 0), Run(1, 1)), norm,
                             PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "tied": False}))
    return LatentConfig


def test_a_mixer_whose_pages_hold_one_vector_per_position(tmp_path):
    """The cache manager allocates what a mixer's need says and knows nothing of keys or values:
    a toy mixer with pages [page_size * latent] of float32 beside an attention layer's
    [2, heads, page_size * d], on the same page numbers; whole, in portions beside another request,
    and with pages that an ended request gave back."""
    from tlie_amd import Engine, write_random_model
    from gpu_helpers import Replayer
    config = register_latent_cache_toy()(hidden_size=32, vocab_size=70, latent=5)
    write_random_model(str(tmp_path), config, seed=4, std=0.15, norm_std=0.1, dtype=torch.float32)
    raw, w = load_plain(str(tmp_path))

    def plain(tokens):
        count = len(tokens)
        x = w["model.embed_tokens.weight"][tokens]

        def mlp(x, p):
            normed = plain_rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5)
            return plain_linear(plain_silu_mul(plain_linear(normed, w[p + "mlp.gate_proj.weight"]),
                                               plain_linear(normed, w[p + "mlp.up_proj.weight"])), w[p + "mlp.down_proj.weight"])
        p = "model.layers.0."
        latent = plain_linear(plain_rms_norm(x, w[p + "input_layernorm.weight"], 1e-5), w[p + "self_attn.down.weight"])
        means = torch.cumsum(latent, dim=0) / (torch.arange(count).double() + 1.0)[:, None]
        x = x + plain_linear(means, w[p + "self_attn.up.weight"])
        x = x + mlp(x, p)
        p = "model.layers.1."
        x = x + plain_attention_part(plain_rms_norm(x, w[p + "input_layernorm.weight"], 1e-5), w, p + "self_attn.", 2, 2, 16, 50.0, None, False)
        x = x + mlp(x, p)
        return plain_linear(plain_rms_norm(x, w["model.norm.weight"], 1e-5), w["lm_head.weight"])

    engine = Engine(str(tmp_path), dtype="float32", max_tokens=96, page_size=8, max_requests=3)
    assert len(engine.cache.groups) == 1
    assert engine.cache.bindings[0].cache.shape == (12, 8 * 5) and engine.cache.bindings[0].cache.dtype == torch.float32
    assert engine.cache.bindings[1].cache.shape == (12, 2, 2, 8 * 16)
    tokens = [(13 * i * i + 5) % 70 for i in range(50)]
    other = [(3 * i + 1) % 70 for i in range(30)]
    want, want_other = plain(tokens), plain(other)
    replay = Replayer(engine)
    replay.step([("whole", tokens, list(range(50)))], end=["whole"])
    assert_close(replay.logits_of("whole", range(50)), want, 2e-5, "whole")
    replay.step([("a", tokens[:11], list(range(11))), ("b", other, list(range(30)))], end=["b"])
    replay.step([("a", tokens[11:13], [0, 1]), ("c", other[:17], list(range(17)))])       # "c" on pages that "b" gave back
    replay.step([("c", other[17:], list(range(13))), ("a", tokens[13:14], [0])], end=["c"])
    replay.step([("a", tokens[14:], list(range(36)))], end=["a"])
    assert_close(replay.logits_of("a", range(50)), want, 2e-5, "in portions")
    assert_close(replay.logits_of("b", range(30)), want_other, 2e-5, "beside it")
    assert_close(replay.logits_of("c", range(30)), want_other, 2e-5, "on pages that were used before")
    assert engine.cache.free_pages() == [12]


def register_windowed_toy():
    """A second architecture of the test's own, out of the framework's parts only: a layer whose
    attention sees a window of 11 positions (its pages come back while a request runs) and turns
    half of each head, then a layer whose attention sees everything.  Two page groups; every part
    may be recorded."""
    from tlie_amd.config import LayerSpec, ModelSpec, PartSpec, Run
    from tlie_amd.registry import register

    @register("architecture", "ToyWindowedForCausalLM")
    @dataclass(frozen=True)
    class WindowedConfig:
        hidden_size: int
        vocab_size: int
        eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["hidden_size"], raw["vocab_size"], raw["eps"])

        def to_dict(self):
            return {"architectures": ["ToyWindowedForCausalLM"], "hidden_size": self.hidden_size, "vocab_size": self.vocab_size,
                    "eps": self.eps}

        def to_spec(self):
            norm = PartSpec("rms_norm", {"size": self.hidden_size, "eps": self.eps})

            def attention(window, rot_dim):
                position = PartSpec("rotary", {"head_dim": 32, "theta": 300.0, "rot_dim": rot_dim})
                return PartSpec("attention", {"hidden_size": self.hidden_size, "num_heads": 3, "num_kv_heads": 1, "head_dim": 32,
                                              "bias": False, "window": window, "position": position})
            mlp = PartSpec("gated_mlp", {"hidden_size": self.hidden_size, "intermediate_size": 56, "activation": "silu"})
            layers = (LayerSpec("model.layers.0.", "pre_norm", attention(11, 16), mlp, norm, norm),
                      LayerSpec("model.layers.1.", "pre_norm", attention(None, 32), mlp, norm, norm))
            return ModelSpec("ToyWindowedForCausalLM", self.hidden_size, self.vocab_size, 256,
                             PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size}),
                             layers, (Run(0, 0), Run(1, 1)), norm,
                             PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "tied": False}))
    return WindowedConfig


def plain_windowed_forward(raw, w, tokens):
    count, eps = len(tokens), raw["eps"]
    x = w["model.embed_tokens.weight"][tokens]
    for layer, (window, rot_dim) in enumerate(((11, 16), (None, 32))):
        p = f"model.layers.{layer}."
        normed = plain_rms_norm(x, w[p + "input_layernorm.weight"], eps)
        x = x + plain_attention_part(normed, w, p + "self_attn.", 3, 1, 32, 300.0, window, False, rot_dim=rot_dim)
        normed = plain_rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + plain_linear(plain_silu_mul(plain_linear(normed, w[p + "mlp.gate_proj.weight"]),
                                            plain_linear(normed, w[p + "mlp.up_proj.weight"])), w[p + "mlp.down_proj.weight"])
    return plain_linear(plain_rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_windowed_architecture_through_recorded_steps(tmp_path, dtype):
    """Two page groups, one of them windowed, through steps of portions and of single tokens that
    are replayed from recordings (a block table's entries of pages that the window has given back
    stay what they were), against the plain implementation; an engine without recordings runs the
    same steps kernel by kernel."""
    from tlie_amd import Engine, write_random_model
    from gpu_helpers import Replayer
    config = register_windowed_toy()(hidden_size=48, vocab_size=70, eps=1e-5)
    write_random_model(str(tmp_path), config, seed=9, std=0.15, norm_std=0.1, dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    raw, weights = load_plain(str(tmp_path))
    tolerance = 2e-5 if dtype == "float32" else 3e-2
    recorded = Engine(str(tmp_path), dtype=dtype, max_tokens=448, page_size=16, max_requests=3)
    eager = Engine(str(tmp_path), dtype=dtype, max_tokens=448, page_size=16, max_requests=3, use_graphs=False)
    assert len(recorded.cache.groups) == 2 and recorded.runner.use_graphs
    streams = {"u": [(11 * i * i + 5) % 70 for i in range(200)], "v": [(3 * i + 7 * (i % 5)) % 70 for i in range(150)]}
    want = {request: plain_windowed_forward(raw, weights, tokens) for request, tokens in streams.items()}
    a, b = Replayer(recorded), Replayer(eager)
    done = {"u": 0, "v": 0}
    sizes = [20, 3, 1, 1, 17, 1, 1, 1, 40, 2, 1, 1, 1, 1, 9]
    turn = 0
    while any(done[request] < len(streams[request]) for request in streams):
        items = []
        for index, request in enumerate(streams):
            left = len(streams[request]) - done[request]
            if left == 0:
                continue
            count = min(left, sizes[(turn + 4 * index) % len(sizes)])
            items.append((request, streams[request][done[request]:done[request] + count], [count - 1]))
            done[request] += count
        for replay in (a, b):
            replay.step(items)
        turn += 1
    # the windowed group holds two or three pages a request, the other all 13 of the 200 positions
    held = recorded.cache.held("u").pages
    assert sum(page >= 0 for page in held[0]) <= 3 and sum(page >= 0 for page in held[1]) == 13
    assert recorded.runner._graphs and recorded.runner._portion_graphs and not eager.runner._graphs
    keys = sorted(a.rows, key=str)
    assert keys == sorted(b.rows, key=str) and len(keys) >= 40
    for request, tokens in streams.items():
        places = [place for name, place in keys if name == request]
        assert_close(a.logits_of(request, places), want[request][places], tolerance, f"{request} recorded")
        assert_close(b.logits_of(request, places), want[request][places], tolerance, f"{request} eager")


def test_an_embedding_with_learned_positions(tmp_path):
    """A position encoding of another kind, defined here: a table of learned rows, one per place,
    added to the token's row by an embedding part of the test's own; the attention then runs with
    no position encoding of its own.  Whole, in portions and token by token, against the plain
    functions."""
    from tlie_amd import Engine, write_random_model
    from tlie_amd.config import LayerSpec, ModelSpec, PartSpec, Run, TensorSpec
    from tlie_amd.parts.base import Part
    from tlie_amd.registry import register
    from gpu_helpers import Replayer

    @register("embedding", "toy_token_and_place")
    class TokenAndPlace(Part):
        @classmethod
        def tensor_specs(cls, spec, prefix=""):
            return [TensorSpec("model.embed_tokens.weight", (spec["vocab_size"], spec["hidden_size"])),
                    TensorSpec("model.embed_places.weight", (spec["places"], spec["hidden_size"]))]

        def load(self, weights, prefix=""):
            self.tokens, self.places = weights["model.embed_tokens.weight"], weights["model.embed_places.weight"]

        def forward(self, tokens, ctx):
            return (self.tokens[tokens.long()].float() + self.places[ctx.positions.long()].float()).contiguous()

    @register("architecture", "ToyPlacesForCausalLM")
    @dataclass(frozen=True)
    class PlacesConfig:
        hidden_size: int
        vocab_size: int
        places: int

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["hidden_size"], raw["vocab_size"], raw["places"])

        def to_dict(self):
            return {"architectures": ["ToyPlacesForCausalLM"], "hidden_size": self.hidden_size, "vocab_size": self.vocab_size,
                    "places": self.places}

        def to_spec(self):
            norm = PartSpec("rms_norm", {"size": self.hidden_size, "eps": 1e-5})
            attention = PartSpec("attention", {"hidden_size": self.hidden_size, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                               "bias": False, "window": None, "position": PartSpec("none")})
            mlp = PartSpec("gated_mlp", {"hidden_size": self.hidden_size, "intermediate_size": 48, "activation": "silu"})
            return ModelSpec("ToyPlacesForCausalLM", self.hidden_size, self.vocab_size, self.places,
                             PartSpec("toy_token_and_place", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                                                              "places": self.places}),
                             (LayerSpec("model.layers.0.", "pre_norm", attention, mlp, norm, norm),), (Run(0, 0),), norm,
                             PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size, "tied": False}))

    write_random_model(str(tmp_path), PlacesConfig(hidden_size=40, vocab_size=60, places=96), seed=3, std=0.2, norm_std=0.1,
                       dtype=torch.float32)
    raw, w = load_plain(str(tmp_path))
    tokens = [(13 * i * i + 7) % 60 for i in range(70)]
    x = w["model.embed_tokens.weight"][tokens] + w["model.embed_places.weight"][:70]
    p = "model.layers.0."
    x = x + plain_attention_part(plain_rms_norm(x, w[p + "input_layernorm.weight"], 1e-5), w, p + "self_attn.", 4, 2, 16, None, None, False)
    normed = plain_rms_norm(x, w[p + "post_attention_layernorm.weight"], 1e-5)
    x = x + plain_linear(plain_silu_mul(plain_linear(normed, w[p + "mlp.gate_proj.weight"]),
                                        plain_linear(normed, w[p + "mlp.up_proj.weight"])), w[p + "mlp.down_proj.weight"])
    want = plain_linear(plain_rms_norm(x, w["model.norm.weight"], 1e-5), w["lm_head.weight"])
    engine = Engine(str(tmp_path), dtype="float32", max_tokens=256, page_size=16, max_requests=2)
    replay = Replayer(engine)
    replay.step([("whole", tokens, list(range(70)))], end=["whole"])
    assert_close(replay.logits_of("whole", range(70)), want, 2e-5, "whole")
    replay.step([("cut", tokens[:33], list(range(33)))])
    replay.step([("cut", tokens[33:35], [0, 1])])
    for place in range(35, 70):
        replay.step([("cut", tokens[place:place + 1], [0])])
    engine.finish("cut")
    assert_close(replay.logits_of("cut", range(70)), want, 2e-5, "in portions and token by token")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_architecture_whose_checkpoint_names_every_place_otherwise(tmp_path, dtype):
    """The seven places a checkpoint's names come from (the embedding's table, the final norm, the
    head, and per layer the two norms, the mixer and the feed-forward) are the specification's: an
    architecture registered here, whose files call all of them otherwise, is written, loaded and
    stepped with no file of the package changed, and gives the logits of the plain implementation on
    the same values under the reference's names."""
    import dataclasses
    from tlie_amd import Engine, LlamaConfig, write_random_model
    from tlie_amd.registry import register
    from plain_llama import plain_forward
    from gpu_helpers import CONFIG_B, TOLERANCE, Replayer

    @register("architecture", "RenamedForCausalLM")
    class RenamedConfig(LlamaConfig):
        @classmethod
        def from_dict(cls, raw):
            return super().from_dict({**raw, "architectures": ["LlamaForCausalLM"]})

        def to_dict(self):
            return {**super().to_dict(), "architectures": ["RenamedForCausalLM"]}

        def to_spec(self):
            spec = super().to_spec()
            layers = tuple(dataclasses.replace(layer, prefix=f"h.{index}.", mixer_norm_place="ln_1.", mixer_place="attn.",
                                               feed_forward_norm_place="ln_2.", feed_forward_place="ffn.")
                           for index, layer in enumerate(spec.layers))
            head = dataclasses.replace(spec.head, params={**spec.head.params, "tied_to": "wte.weight"})
            return dataclasses.replace(spec, layers=layers, head=head, embedding_name="wte.weight", final_norm_prefix="ln_f.",
                                       head_name="out.weight")

    for tied in (True, False):
        folder = tmp_path / f"tied{tied}"
        raw = {**CONFIG_B, "tie_word_embeddings": tied}
        write_random_model(str(folder), RenamedConfig.from_dict(raw), seed=11, std=0.08, norm_std=0.1,
                           dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
        stored, weights = load_plain(str(folder))
        assert stored["architectures"] == ["RenamedForCausalLM"]
        assert "wte.weight" in weights and "ln_f.weight" in weights and "h.0.attn.q_proj.weight" in weights
        assert ("out.weight" in weights) != tied and not any(name.startswith("model.") for name in weights)

        def reference_name(name):
            for old, new in (("wte.", "model.embed_tokens."), ("ln_f.", "model.norm."), ("out.", "lm_head."), ("h.", "model.layers."),
                             (".ln_1.", ".input_layernorm."), (".ln_2.", ".post_attention_layernorm."), (".attn.", ".self_attn."),
                             (".ffn.", ".mlp.")):
                name = name.replace(old, new) if old.startswith(".") or name.startswith(old) else name
            return name
        tokens = [(29 * i * i + 5) % raw["vocab_size"] for i in range(40)]
        want = plain_forward(raw, {reference_name(name): tensor for name, tensor in weights.items()}, tokens)
        engine = Engine(str(folder), dtype=dtype, max_tokens=128, page_size=16, max_requests=2)
        replay = Replayer(engine)
        replay.step([("r", tokens[:30], list(range(30)))])
        for place in range(30, 40):
            replay.step([("r", tokens[place:place + 1], [0])])
        assert_close(replay.logits_of("r", range(40)), want, TOLERANCE[dtype], f"renamed checkpoint, tied {tied}")
