"""Each HIP kernel alone against its plain reference, at sizes other than the engine's tiny
configurations (no power of two, odd head counts), in float32 and bfloat16, and with inputs built
so that a fault at a special place shows: a far key among hundreds, a page's edge, a window's edge,
pages in shuffled physical order."""
import math
import random

import pytest
import torch

from plain_llama import (plain_attention, plain_greedy, plain_linear, plain_rms_norm, plain_rope, plain_silu_mul,
                         plain_top_p_distribution)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-6, "bfloat16": 1.2e-2}      # relative to the largest expected value; bf16 = 2^-8 output rounding + input rounding


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).abs().max() / want.abs().max().clamp_min(1e-30)).item()


def rounded(tensor, dtype):
    """The values a kernel sees: rounded to the storage type, as float64 for the plain reference."""
    return tensor.to(dtype).double()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed_gather(dtype):
    from tlie_amd import ops
    table = torch.randn(301, 72).to(DT[dtype]).to(DEV)
    tokens = torch.tensor([0, 300, 17, 17, 5], dtype=torch.int32, device=DEV)
    out = ops.embed_gather(tokens, table)
    assert out.dtype == torch.float32 and torch.equal(out.cpu(), table.float().cpu()[tokens.long().cpu()])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden", [72, 1000, 2048, 5000])
def test_add_rmsnorm(dtype, hidden):
    from tlie_amd import ops
    torch.manual_seed(hidden)
    tokens = 7
    residual = torch.randn(tokens, hidden) * 3
    delta = (torch.randn(3, tokens, hidden)).float()
    weight = (1 + 0.2 * torch.randn(hidden)).to(DT[dtype])
    eps = 1e-6
    res_dev = residual.to(DEV)
    out = ops.add_rmsnorm(res_dev, ops.Product(delta.to(DEV), 3), weight.to(DEV), eps, DT[dtype])
    summed = residual.double() + delta.double().sum(0)
    assert rel_err(res_dev, summed) < 2e-6                                  # the residual sum is 32-bit in both modes
    assert rel_err(out, plain_rms_norm(summed, weight.double(), eps)) < TOL[dtype]
    # norm only, golden vector of the reference (data/golden/operators.json:4-24)
    x = torch.tensor([[1.0, -2.0, 3.0, -4.0]], device=DEV)
    w = torch.tensor([0.5, 1.0, 1.5, 2.0], device=DEV)
    got = ops.add_rmsnorm(x, None, w, 1e-5, torch.float32)
    want = torch.tensor([[0.182574063539505, -0.73029625415802, 1.6431666612625122, -2.92118501663208]])
    assert torch.allclose(got.cpu(), want, atol=1e-6, rtol=0)
    # picked rows: the residual is left alone, the output is norm(residual + delta) of those rows
    res_dev = residual.to(DEV)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    one = ops.Product(delta[0].to(DT[dtype]).to(DEV).contiguous(), 1)
    picked = ops.add_rmsnorm(res_dev, one, weight.to(DEV), eps, DT[dtype], rows=rows)
    assert torch.equal(res_dev.cpu(), residual)
    want = plain_rms_norm(residual.double()[[5, 0, 5]] + rounded(delta[0], DT[dtype])[[5, 0, 5]], weight.double(), eps)
    assert rel_err(picked, want) < TOL[dtype]
    # a zero row gives zero, not NaN (eps is inside the root)
    zero = ops.add_rmsnorm(torch.zeros(1, hidden, device=DEV), None, weight.to(DEV), eps, DT[dtype])
    assert float(zero.float().abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_silu_mul(dtype):
    from tlie_amd import ops
    gate_up = torch.tensor([[-2.0, -0.5, 0.0, 1.5, 0.5, -1.0, 2.0, 3.0]], device=DEV)      # operators.json:132-151
    got = ops.silu_mul(ops.Product(gate_up, 1), torch.float32)
    want = torch.tensor([[-0.11920291930437088, 0.1887703388929367, 0.0, 3.6790847778320312]])
    assert torch.allclose(got.cpu(), want, atol=1e-6, rtol=0)
    torch.manual_seed(0)
    parts = torch.randn(2, 9, 2 * 177) * 2
    got = ops.silu_mul(ops.Product(parts.to(DEV), 2), DT[dtype])
    total = parts.double().sum(0)
    assert rel_err(got, plain_silu_mul(total[:, :177], total[:, 177:])) < TOL[dtype]
    # a width that takes the kernel with eight results a thread, three summands, both layouts
    parts = torch.randn(3, 9, 2 * 176) * 2
    total = parts.double().sum(0)
    got = ops.silu_mul(ops.Product(parts.to(DEV), 3), DT[dtype])
    assert rel_err(got, plain_silu_mul(total[:, :176], total[:, 176:])) < TOL[dtype]
    got = ops.silu_mul(ops.Product(parts.to(DEV), 3), DT[dtype], interleaved=True)
    assert rel_err(got, plain_silu_mul(total[:, 0::2], total[:, 1::2])) < TOL[dtype]
    extreme = torch.tensor([[80.0, -90.0, 2.0, 2.0]], device=DEV)
    got = ops.silu_mul(ops.Product(extreme, 1), torch.float32).cpu()
    assert got[0, 0] == 160.0 and abs(got[0, 1]) < 1e-30 and torch.isfinite(got).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(1, 40, 24), (5, 72, 100), (70, 129, 333), (130, 64, 2048)])
def test_gemm_generic(dtype, shape):
    from tlie_amd import ops
    m, n, k = shape
    torch.manual_seed(m)
    x = torch.randn(m, k).to(DT[dtype])
    w = (torch.randn(n, k) / math.sqrt(k)).to(DT[dtype])
    b = torch.randn(n).to(DT[dtype])
    got = ops.gemm_generic(x.to(DEV), w.to(DEV), b.to(DEV), torch.float32).dense()
    assert rel_err(got, plain_linear(x.double(), w.double(), b.double())) < 5e-6
    got = ops.gemm_generic(x.to(DEV), w.to(DEV), None, DT[dtype]).dense()
    assert rel_err(got, plain_linear(x.double(), w.double())) < TOL[dtype]


@pytest.mark.parametrize("shape", [(3, 50, 37), (16, 129, 640), (17, 33, 131), (64, 200, 2052), (9, 2048, 5632)])
def test_gemm_generic_gives_few_rows_the_same_bits_as_many(shape):
    """Few rows take a kernel of their own; a row's sums must not depend on which one ran: the
    first rows of a batch of 100 against the same rows alone, bit for bit."""
    from tlie_amd import ops
    m, n, k = shape
    torch.manual_seed(k)
    x = torch.randn(100, k, device=DEV)
    w = torch.randn(n, k, device=DEV) / math.sqrt(k)
    b = torch.randn(n, device=DEV)
    many = ops.gemm_generic(x, w, b, torch.float32).dense()
    few = ops.gemm_generic(x[:m].contiguous(), w, b, torch.float32).dense()
    assert torch.equal(few, many[:m])
    assert rel_err(few, plain_linear(x[:m].double().cpu(), w.double().cpu(), b.double().cpu())) < 5e-6


@pytest.mark.parametrize("shape", [(65, 96, 64), (200, 2560, 2048), (333, 177, 200), (70, 129, 333), (1024, 2048, 5632)])
def test_library_product_of_many_rows(shape):
    """The vendor library's product, called directly where it offers an algorithm (and through
    torch where it does not: odd inner sizes), against the plain product of the rounded inputs."""
    from tlie_amd import ops
    m, n, k = shape
    torch.manual_seed(n)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    got = ops.library_mm(x.to(DEV), w.to(DEV))
    assert got.dtype == torch.bfloat16 and got.shape == (m, n)
    assert rel_err(got, plain_linear(x.double(), w.double())) < TOL["bfloat16"]
    again = ops.library_mm(x.to(DEV), w.to(DEV))              # the kept plan
    assert torch.equal(got, again)
    # float32 out (the output head's logits): the sums are not rounded to bfloat16
    wide = ops.library_mm(x.to(DEV), w.to(DEV), torch.float32)
    assert wide.dtype == torch.float32 and rel_err(wide, plain_linear(x.double(), w.double())) < 1e-5
    # recorded: the library's product where it has an algorithm, else the plain kernel (never torch's)
    xd, wd = x.to(DEV), w.to(DEV)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = ops.library_mm(xd, wd)
    for _ in range(3):
        xd.copy_(torch.randn(m, k).bfloat16())
        graph.replay()
        torch.cuda.synchronize()
        assert rel_err(recorded, plain_linear(xd.double().cpu(), w.double())) < TOL["bfloat16"]


def test_gemm_is_true_32_bit():
    """(1 + 2^-12)^2 accumulated onto -(1 + 2^-11) leaves 2^-24: it needs all 24 bits of both
    factors and a fused multiply-add; a product whose inputs were cut to fewer bits leaves -2^-11
    or 0.  (The sum runs in index order, so the negative term is accumulated first.)"""
    from tlie_amd import ops
    a = 1.0 + 2.0 ** -12
    x = torch.tensor([[1.0, a] + [0.0] * 30], device=DEV)
    w = torch.tensor([[-(1.0 + 2.0 ** -11), a] + [0.0] * 30], device=DEV)
    got = ops.gemm_generic(x, w, None, torch.float32).dense().item()
    assert got == 2.0 ** -24


def build_cache(k, v, page_size, dtype, shuffle_seed=0, extra_pages=3):
    """Puts one sequence's keys and values [T, nkv, d] on pages in shuffled physical order.
    Returns (cache [pages, 2, nkv, page_size * d], block table row).  Per page and kv head the keys
    lie as [row][dim], the values transposed as [dim][row].  Rows that hold no token of the sequence
    hold NaN: a kernel that lets them reach a result shows it."""
    tokens, nkv, d = k.shape
    blocks = (tokens + page_size - 1) // page_size
    order = list(range(blocks + extra_pages))
    random.Random(shuffle_seed).shuffle(order)
    keys = torch.full((blocks + extra_pages, nkv, page_size, d), float("nan"))
    values = torch.full((blocks + extra_pages, nkv, d, page_size), float("nan"))
    for position in range(tokens):
        page, row = order[position // page_size], position % page_size
        keys[page, :, row, :] = k[position]
        values[page, :, :, row] = v[position]
    cache = torch.stack([keys.reshape(-1, nkv, page_size * d), values.reshape(-1, nkv, page_size * d)], dim=1).to(dtype)
    return cache.contiguous(), order[:blocks]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", [
    dict(tokens=3, nq=2, nkv=1, d=4, page=16, golden=True),
    dict(tokens=77, nq=6, nkv=3, d=48, page=16),
    dict(tokens=300, nq=5, nkv=5, d=80, page=32),
    dict(tokens=700, nq=8, nkv=1, d=128, page=16, window=None),
    dict(tokens=333, nq=4, nkv=2, d=16, page=8, window=37),
    dict(tokens=130, nq=3, nkv=1, d=256, page=64),
])
def test_attention_generic(dtype, case):
    from tlie_amd import ops
    tokens, nq, nkv, d, page = case["tokens"], case["nq"], case["nkv"], case["d"], case["page"]
    window = case.get("window")
    torch.manual_seed(tokens)
    if case.get("golden"):                                               # data/golden/operators.json:78-131
        q = torch.zeros(3, 2, 4)
        q[2] = torch.tensor([0.2, -0.1, 0.4, 0.3, -0.5, 0.7, 0.1, -0.2]).view(2, 4)
        k = torch.tensor([0.1, 0.2, 0.3, 0.4, -0.4, 0.3, -0.2, 0.1, 0.5, -0.6, 0.7, -0.8]).view(3, 1, 4)
        v = torch.tensor([1.0, 0.0, -1.0, 0.5, 0.2, 0.4, 0.6, 0.8, -0.3, 0.7, 0.9, -0.1]).view(3, 1, 4)
    else:
        q, k, v = torch.randn(tokens, nq, d), torch.randn(tokens, nkv, d), torch.randn(tokens, nkv, d)
    cache, pages = build_cache(k, v, page, DT[dtype], shuffle_seed=tokens)
    table = torch.tensor([[0] * len(pages), pages], dtype=torch.int32, device=DEV)      # row 1 is the sequence
    token_seq = torch.ones(tokens, dtype=torch.int32, device=DEV)
    positions = torch.arange(tokens, dtype=torch.int32, device=DEV)
    got = ops.attention_generic(q.to(DT[dtype]).view(tokens, nq * d).to(DEV), cache.to(DEV), table, token_seq, positions,
                                nq, nkv, d, window, 1.0 / math.sqrt(d)).view(tokens, nq, d)
    want = plain_attention(rounded(q, DT[dtype]), rounded(k, DT[dtype]), rounded(v, DT[dtype]), window=window)
    assert rel_err(got, want) < TOL[dtype]
    if case.get("golden"):
        golden = torch.tensor([0.31072109937667847, 0.3621496558189392, 0.13341431319713593, 0.3776317536830902,
                               0.3371150493621826, 0.3447031080722809, 0.14012068510055542, 0.46016252040863037])
        if dtype == "float32":
            assert torch.allclose(got[2].flatten().cpu().double(), golden.double(), atol=1e-6, rtol=0)
    # a step that brings only some of the tokens (a portion, or one decoded token) gives the same rows
    some = [tokens - 1] if tokens < 5 else [0, 1, page - 1, page, page + 1, tokens // 2, tokens - 2, tokens - 1]
    sub = ops.attention_generic(q[some].to(DT[dtype]).reshape(len(some), nq * d).to(DEV).contiguous(), cache.to(DEV), table,
                                torch.ones(len(some), dtype=torch.int32, device=DEV),
                                torch.tensor(some, dtype=torch.int32, device=DEV), nq, nkv, d, window, 1.0 / math.sqrt(d))
    assert torch.equal(sub.view(len(some), nq, d).cpu(), got[some].cpu())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", [
    dict(nq=8, nkv=2, d=64, page=16, window=None), dict(nq=6, nkv=3, d=48, page=16, window=70),
    dict(nq=5, nkv=5, d=7, page=8, window=None), dict(nq=40, nkv=1, d=16, page=16, window=300),   # 40 heads a group: two blocks of heads
])
def test_attention_that_shares_keys_among_neighbouring_tokens_gives_the_same_bits(dtype, case):
    """The plain attention kernel has a form for steps whose sequences bring several tokens: a
    workgroup serves up to 32 (token, head) columns and reads each chunk of keys once for all of
    them.  A column's arithmetic is the same operation for operation, so the two forms must agree in
    every bit, whatever the step: here portions of three sequences of different lengths (one of
    them a single token, one starting mid-way), tokens of different sequences falling into one
    workgroup; and both agree with the plain implementation."""
    from tlie_amd import ops
    nq, nkv, d, page, window = case["nq"], case["nkv"], case["d"], case["page"], case["window"]
    torch.manual_seed(nq * 100 + d)
    lengths, firsts = [613, 1, 290], [0, 0, 201]                  # the step brings positions firsts[i] .. lengths[i] - 1
    padding = 5                                                   # tokens of the first sequence again, at position 0, at the step's end (a recording's padding)
    caches, tables, offset = [], [], 0
    qs, wants, token_seq, positions = [], [], [], []
    for index, (length, first) in enumerate(zip(lengths, firsts)):
        q, k, v = torch.randn(length, nq, d), torch.randn(length, nkv, d), torch.randn(length, nkv, d)
        cache, pages = build_cache(k, v, page, DT[dtype], shuffle_seed=index)
        caches.append(cache)
        tables.append([page_index + offset for page_index in pages])
        offset += cache.shape[0]
        qs.append(q[first:])
        wants.append(plain_attention(rounded(q, DT[dtype]), rounded(k, DT[dtype]), rounded(v, DT[dtype]), window=window)[first:])
        token_seq += [index] * (length - first)
        positions += list(range(first, length))
    qs.append(torch.randn(padding, nq, d))
    token_seq += [0] * padding
    positions += [0] * padding
    width = max(len(row) for row in tables)
    table = torch.tensor([row + [0] * (width - len(row)) for row in tables], dtype=torch.int32, device=DEV)
    cache = torch.cat(caches).to(DEV)
    q = torch.cat(qs).to(DT[dtype]).reshape(-1, nq * d).to(DEV).contiguous()
    arguments = (q, cache, table, torch.tensor(token_seq, dtype=torch.int32, device=DEV),
                 torch.tensor(positions, dtype=torch.int32, device=DEV), nq, nkv, d, window, 1.0 / math.sqrt(d))
    alone = ops.attention_generic(*arguments, tiled=False)
    shared = ops.attention_generic(*arguments, tiled=True)
    assert torch.isfinite(shared.float()).all()
    assert torch.equal(alone, shared)
    # a mixed step launches both forms, and each sequence's token count decides which one serves it: the
    # single token goes to the first form (and, with a higher bar, the portion of 89 tokens too)
    seq_start = torch.tensor([0, 613, 614, 703], dtype=torch.int32, device=DEV)
    for bar in (4, 100, 1000):
        split = ops.attention_generic(*arguments, tiled=2, seq_start=seq_start, min_tokens=bar)
        assert torch.equal(alone, split), f"served by both forms, sequences of {bar} tokens and more by the second"
    assert rel_err(shared.view(-1, nq, d)[:-padding], torch.cat(wants)) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_finds_one_key_among_hundreds(dtype):
    """One key is made to stand out (its score is far above the rest), at places where an index
    mistake would miss it: the first key, a page's last row and the next page's first, the last
    key but one, the window's first key and the key just outside the window."""
    from tlie_amd import ops
    tokens, nq, nkv, d, page = 600, 4, 2, 32, 16
    torch.manual_seed(1)
    base_k, v = torch.randn(tokens, nkv, d) * 0.1, torch.randn(tokens, nkv, d)
    q = torch.randn(1, nq, d) * 0.1
    direction = torch.zeros(d)
    direction[3] = 1.0
    q = q + 12.0 * direction
    position = tokens - 1
    for window, needle, inside in [(None, 0, True), (None, 15, True), (None, 16, True), (None, 511, True), (None, 598, True),
                                   (100, 500, True), (100, 499, False), (100, 599, True), (16, 584, True), (16, 583, False)]:
        k = base_k.clone()
        k[needle] += 12.0 * direction                   # score about 144 / sqrt(32) = 25 above the others
        cache, pages = build_cache(k, v, page, DT[dtype], shuffle_seed=needle)
        got = ops.attention_generic(q.to(DT[dtype]).view(1, nq * d).to(DEV), cache.to(DEV),
                                    torch.tensor([pages], dtype=torch.int32, device=DEV),
                                    torch.zeros(1, dtype=torch.int32, device=DEV),
                                    torch.tensor([position], dtype=torch.int32, device=DEV), nq, nkv, d, window,
                                    1.0 / math.sqrt(d)).view(nq, d).float().cpu()
        wanted_rows = rounded(v[needle], DT[dtype]).float().repeat_interleave(nq // nkv, dim=0)
        hit = (got - wanted_rows).abs().max().item() < 0.05
        assert hit == inside, f"window {window}, needle at {needle}: {'missed' if inside else 'seen'}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rope_cache(dtype):
    from tlie_amd import ops
    # the reference's golden vector (data/golden/operators.json:25-63): 2 q heads, 1 kv head, d = 4, position 7
    qkv = torch.tensor([[0.1, 0.2, 0.3, 0.4, -0.5, 0.6, -0.7, 0.8, 0.9, -1.0, 1.1, -1.2, 5.0, 6.0, 7.0, 8.0]], device=DEV)
    inv_freq = torch.pow(torch.tensor(10000.0), -2.0 * torch.arange(2, dtype=torch.float32) / 4.0).to(DEV)
    cache = torch.zeros(3, 2, 1, 4 * 4, device=DEV)
    q = ops.rope_cache(ops.Product(qkv, 1), torch.tensor([7], dtype=torch.int32, device=DEV),
                       torch.tensor([2 * 4 + 1], dtype=torch.int32, device=DEV), inv_freq, 4, cache, 2, 1, 4, torch.float32)
    want_q = torch.tensor([-0.12170576304197311, 0.17153306305408478, 0.2918693423271179, 0.41300898790359497,
                           0.08293947577476501, 0.5425763726234436, -0.8562248945236206, 0.8400065302848816])
    want_k = torch.tensor([-0.044173240661621094, -0.9136196374893188, 1.4205803871154785, -1.267004132270813])
    assert torch.allclose(q.cpu().flatten(), want_q, atol=1e-6, rtol=0)
    assert torch.allclose(cache[2, 0, 0].view(4, 4)[1].cpu(), want_k, atol=1e-6, rtol=0)   # keys: [row][dim]
    assert torch.equal(cache[2, 1, 0].view(4, 4)[:, 1].cpu(), torch.tensor([5.0, 6.0, 7.0, 8.0]))   # values: [dim][row], unrotated
    assert float(cache.abs().sum()) == pytest.approx(float(want_k.abs().sum()) + 26.0, rel=1e-5)   # nothing else was written

    # other sizes, split partial sums, far positions (the reference tests position 4095: tests/cuda/kernel_tests.cu:144-146)
    tokens, nq, nkv, d, page = 9, 5, 3, 48, 8
    torch.manual_seed(3)
    parts = torch.randn(2, tokens, (nq + 2 * nkv) * d)
    positions = torch.tensor([0, 1, 2, 4095, 77, 1000, 8, 9, 31], dtype=torch.int32)
    slots = torch.tensor([3, 12, -1, 40, 41, 7, 0, 63, 20], dtype=torch.int32)
    theta = 500000.0
    inv_freq = torch.pow(torch.tensor(theta), -2.0 * torch.arange(d // 2, dtype=torch.float32) / d).to(DEV)
    cache = torch.full((8, 2, nkv, page * d), -3.0).to(DT[dtype]).to(DEV)
    q = ops.rope_cache(ops.Product(parts.to(DEV), 2), positions.to(DEV), slots.to(DEV), inv_freq, d, cache, nq, nkv, d, DT[dtype])
    total = parts.double().sum(0)
    want_q = plain_rope(total[:, :nq * d].view(tokens, nq, d), positions, theta)
    want_k = plain_rope(total[:, nq * d:(nq + nkv) * d].view(tokens, nkv, d), positions, theta)
    want_v = total[:, (nq + nkv) * d:].view(tokens, nkv, d)
    assert rel_err(q.view(tokens, nq, d), want_q) < TOL[dtype]
    cache = cache.cpu()
    keys, values = cache[:, 0].view(8, nkv, page, d), cache[:, 1].view(8, nkv, d, page)
    written = torch.zeros(8, page, dtype=torch.bool)
    for t in range(tokens):
        if slots[t] < 0:
            continue
        page_index, row = int(slots[t]) // page, int(slots[t]) % page
        written[page_index, row] = True
        assert rel_err(keys[page_index, :, row, :], want_k[t]) < TOL[dtype]
        assert rel_err(values[page_index, :, :, row], want_v[t]) < TOL[dtype]
    for page_index in range(8):
        for row in range(page):
            if not written[page_index, row]:
                assert float((keys[page_index, :, row, :].float() + 3.0).abs().max()) == 0.0
                assert float((values[page_index, :, :, row].float() + 3.0).abs().max()) == 0.0
    # no rotation table: q and k pass through
    plain_q = ops.rope_cache(ops.Product(parts[0].to(DEV).contiguous(), 1), positions.to(DEV), slots.to(DEV), None, 0,
                             torch.zeros(8, 2, nkv, page * d, dtype=DT[dtype], device=DEV), nq, nkv, d, DT[dtype])
    assert rel_err(plain_q, parts[0][:, :nq * d]) < TOL[dtype]


def test_kernels_refuse_what_they_do_not_take():
    from tlie_amd import EngineError, ops
    x = torch.randn(4, 8, device=DEV)
    with pytest.raises(EngineError):
        ops.gemm_generic(x, torch.randn(5, 9, device=DEV), None, torch.float32)                  # inner sizes differ
    with pytest.raises(EngineError):
        ops.gemm_generic(x.cpu(), torch.randn(5, 8), None, torch.float32)                        # not on the GPU
    with pytest.raises(EngineError):
        ops.add_rmsnorm(x, None, torch.ones(9, device=DEV), 1e-5, torch.float32)
    with pytest.raises(EngineError):
        ops.add_rmsnorm(x, None, torch.ones(8, device=DEV), 0.0, torch.float32)                  # src/operators.cpp:27
    with pytest.raises(EngineError):
        ops.gemm_generic(x.half(), torch.randn(5, 8, device=DEV).half(), None, torch.float16)    # float16 is not a storage type here
    with pytest.raises(EngineError):
        ops.attention_generic(torch.randn(2, 2 * 300, device=DEV), torch.zeros(1, 2, 1, 16 * 300, device=DEV),
                              torch.zeros(1, 1, dtype=torch.int32, device=DEV), torch.zeros(2, dtype=torch.int32, device=DEV),
                              torch.zeros(2, dtype=torch.int32, device=DEV), 2, 1, 300, None, 1.0)   # head size above 256


# ---- the bfloat16 kernels on the matrix cores ---------------------------------------------------------

@pytest.mark.parametrize("shape", [(1, 40, 64), (3, 177, 176), (16, 2560, 2048), (17, 100, 520), (33, 64, 5632),
                                   (64, 515, 1000), (8, 32000, 2048), (5, 16, 8)])
def test_gemm_skinny(shape):
    from tlie_amd import ops
    m, n, k = shape
    torch.manual_seed(n)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    b = torch.randn(n).bfloat16()
    want = plain_linear(x.double(), w.double(), b.double())
    product = ops.gemm_skinny(x.to(DEV), w.to(DEV), b.to(DEV))
    assert product.data.shape == (product.nsplit, m, n) and product.data.dtype == torch.float32
    assert rel_err(product.dense(), want) < 5e-6                          # bfloat16 products are exact in float32; only the sums round
    for split_len in (64, 128, 512, 8192):
        product = ops.gemm_skinny(x.to(DEV), w.to(DEV), None, split_len=split_len)
        assert product.nsplit == (k + split_len - 1) // split_len
        assert rel_err(product.dense(), plain_linear(x.double(), w.double())) < 5e-6
    # a row's result does not depend on how many other rows come with it
    if m > 1:
        alone = ops.gemm_skinny(x[:1].to(DEV).contiguous(), w.to(DEV), b.to(DEV), split_len=128).data
        together = ops.gemm_skinny(x.to(DEV), w.to(DEV), b.to(DEV), split_len=128).data
        assert torch.equal(alone[:, 0], together[:, 0])                      # every partial sum, bit for bit


@pytest.mark.parametrize("rows", [5, 23, 40, 64])
def test_gemm_skinny_launch_shapes(rows):
    """Every number of waves a workgroup and both numbers of strips a wave give the same partial
    sums, bit for bit (the shape decides who computes an output, not how), at sizes where the last
    workgroup and the last split are ragged; and the shape that the policy picks is one of them."""
    from tlie_amd import ops
    n, k = 1000, 840                                          # 1000 = 62.5 strips; 840 = 3 splits of 320, the last of 200
    torch.manual_seed(rows)
    x = torch.randn(rows, k).bfloat16().to(DEV)
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16().to(DEV)
    b = torch.randn(n).bfloat16().to(DEV)
    first = ops.gemm_skinny(x, w, b, split_len=320, waves=4, strips=1)
    assert first.nsplit == 3
    assert rel_err(first.dense().cpu(), plain_linear(x.cpu().double(), w.cpu().double(), b.cpu().double())) < 5e-6
    for waves in range(3, 17):
        for strips in (1, 2):
            if strips == 2 and (rows <= 32 or waves > 8):
                with pytest.raises(ops.EngineError):
                    ops.gemm_skinny(x, w, b, split_len=320, waves=waves, strips=strips)
                continue
            other = ops.gemm_skinny(x, w, b, split_len=320, waves=waves, strips=strips)
            assert torch.equal(other.data, first.data), (waves, strips)
    split_len, waves, strips = ops.skinny_plan(rows, n, k, 256)
    planned = ops.gemm_skinny(x, w, b)
    assert planned.nsplit == (k + split_len - 1) // split_len and 4 <= waves <= 16 and strips in (1, 2)
    assert rel_err(planned.dense().cpu(), plain_linear(x.cpu().double(), w.cpu().double(), b.cpu().double())) < 5e-6
    for bad in (dict(waves=2), dict(waves=17), dict(strips=3)):
        with pytest.raises(ops.EngineError):
            ops.gemm_skinny(x, w, b, split_len=320, **{"waves": 4, "strips": 1, **bad})
    # the gated form: all of K in a workgroup, silu(gate) * up stored by the product itself, for every launch shape
    # (W's rows alternate gate and up), against the plain activation of the plain product
    y = plain_linear(x.cpu().double(), w.cpu().double(), b.cpu().double())
    want = plain_silu_mul(y[:, 0::2], y[:, 1::2])
    for waves, strips in ((3, 1), (4, 1), (7, 1), (16, 1), (5, 2), (8, 2), (None, None)):
        if strips == 2 and rows <= 32:
            continue
        got = ops.gemm_skinny(x, w, b, waves=waves, strips=strips, gated=True)
        assert got.dtype == torch.bfloat16 and got.shape == (rows, n // 2)
        assert rel_err(got.cpu(), want) < 6e-3, (waves, strips)                  # one rounding to bfloat16
    with pytest.raises(ops.EngineError):
        ops.gemm_skinny(x, w, b, split_len=320, gated=True)                      # the gated product does not split K
    with pytest.raises(ops.EngineError):
        ops.gemm_skinny(x, w[:999].contiguous(), b[:999].contiguous(), gated=True)   # an odd number of rows: a gate without its up


@pytest.mark.parametrize("shape", [(15832, 2560, 2048), (40000, 2048, 5632), (70000, 704, 512), (65, 96, 64), (300, 32000, 256)])
def test_library_mm_takes_the_library_for_many_rows(shape):
    """Steps of very many rows (all prompts of a batch in one step) still go through the vendor's
    library: its first choice for some of these shapes wants more workspace than is there, and the
    product then takes the first candidate that fits, not the plain kernel (ten times slower)."""
    from tlie_amd import ops
    m, n, k = shape
    torch.manual_seed(m)
    x = torch.randn(m, k, device=DEV).bfloat16()
    w = (torch.randn(n, k, device=DEV) / math.sqrt(k)).bfloat16()
    before = ops.library_fallbacks()
    got = ops.library_mm(x, w)
    got32 = ops.library_mm(x[:70], w, torch.float32)
    assert ops.library_fallbacks() == before
    rows = torch.tensor([0, 1, m // 2, m - 1], device=DEV)
    want = x[rows].double() @ w.double().t()
    assert rel_err(got[rows].cpu(), want.cpu()) < 6e-3                       # one rounding to bfloat16
    assert rel_err(got32[:2].cpu(), want[:2].cpu()) < 5e-5


@pytest.mark.parametrize("shape", [(1, 4, 64), (65, 260, 128), (130, 2560, 2048), (300, 96, 5632), (257, 1000, 192), (2048, 132, 64)])
def test_gemm_tiles_against_the_plain_product(shape):
    """This library's own product of many rows (tiles of 128 x 128 on the matrix cores), at sizes that
    are no multiple of its tiles: bfloat16 and float32 results against the float64 product."""
    from tlie_amd import ops
    m, n, k = shape
    torch.manual_seed(m * 7 + n)
    x = torch.randn(m, k, device=DEV).bfloat16()
    w = (torch.randn(n, k, device=DEV) / math.sqrt(k)).bfloat16()
    want = plain_linear(x.cpu().double(), w.cpu().double())
    assert rel_err(ops.gemm_tiles(x, w, torch.float32).cpu(), want) < 5e-6
    got = ops.gemm_tiles(x, w)
    assert got.dtype == torch.bfloat16 and rel_err(got.cpu(), want) < 6e-3                 # one rounding to bfloat16
    for bad_n, bad_k in ((n + 1, k), (n, k + 8)):
        with pytest.raises(ops.EngineError):
            ops.gemm_tiles(torch.zeros(m, bad_k, device=DEV).bfloat16(), torch.zeros(bad_n, bad_k, device=DEV).bfloat16())


def test_library_mm_without_the_library_takes_the_tiled_kernel_and_says_so(monkeypatch):
    """Where the vendor's library cannot be called, a product of many rows takes this library's tiled
    kernel (or, for sizes that one refuses, the plain 32-bit kernel), counts it and warns once per shape."""
    import warnings
    from tlie_amd import ops
    torch.manual_seed(3)
    x = torch.randn(200, 256, device=DEV).bfloat16()
    w = (torch.randn(96, 256, device=DEV) / 16).bfloat16()
    odd = (torch.randn(97, 256, device=DEV) / 16).bfloat16()                  # 97 rows: not the tiled kernel's
    ops.library_mm(x, w)                                                     # (the library is set up, if it is there)
    monkeypatch.setitem(ops._library_gemm, "state", False)
    monkeypatch.setitem(ops._library_gemm, "warned", set())
    before = ops.library_fallbacks()
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        got, again, plain = ops.library_mm(x, w), ops.library_mm(x, w, torch.float32), ops.library_mm(x, odd)
    assert ops.library_fallbacks() == before + 3
    assert len(caught) == 2 and "tiled kernel" in str(caught[0].message) and "32-bit kernel" in str(caught[1].message)
    assert torch.equal(got, ops.gemm_tiles(x, w)) and torch.equal(again, ops.gemm_tiles(x, w, torch.float32))
    assert rel_err(plain.cpu(), plain_linear(x.cpu().double(), odd.cpu().double())) < 6e-3


def test_gemm_skinny_refuses():
    from tlie_amd import EngineError, ops
    w = torch.randn(32, 64, device=DEV).bfloat16()
    with pytest.raises(EngineError):
        ops.gemm_skinny(torch.randn(65, 64, device=DEV).bfloat16(), w, None)                  # too many rows
    with pytest.raises(EngineError):
        ops.gemm_skinny(torch.randn(2, 12, device=DEV).bfloat16(), torch.randn(8, 12, device=DEV).bfloat16(), None)   # K % 8
    with pytest.raises(EngineError):
        ops.gemm_skinny(torch.randn(2, 64, device=DEV), w, None)                              # float32
    assert not ops.attention_mfma_takes(torch.bfloat16, 64, 8)          # pages below 16 rows go to the plain kernel
    assert not ops.attention_mfma_takes(torch.bfloat16, 72, 16) and not ops.attention_mfma_takes(torch.float32, 64, 16)
    with pytest.raises(EngineError):
        ops.attention_mfma(torch.zeros(1, 64, device=DEV).bfloat16(), torch.zeros(2, 2, 1, 8 * 64, device=DEV).bfloat16(),
                           torch.zeros(1, 1, dtype=torch.int32, device=DEV), None, torch.zeros(1, dtype=torch.int32, device=DEV),
                           1, 1, 64, None, 0.125)
    assert not ops.gemm_skinny_takes(torch.randn(2, 12, device=DEV).bfloat16(), torch.randn(8, 12, device=DEV).bfloat16())


def run_attention_mfma(q, k, v, page, window, nsplit, token_list=None, shuffle_seed=0, col_tiles=None, waves=1, shared=False):
    """One sequence through the tiled kernel: q rows for the positions in token_list (default all).
    waves > 1: so many waves share each tile's keys, and the tiles come longest first.  shared: the
    waves take columns of their own instead, and the keys reach them through LDS."""
    from tlie_amd import ops
    import numpy as np
    tokens, nq, d = q.shape
    nkv = k.shape[1]
    cache, pages = build_cache(k, v, page, torch.bfloat16, shuffle_seed=shuffle_seed)
    token_list = list(range(tokens)) if token_list is None else token_list
    # the step brings a run of consecutive positions of the one sequence
    assert token_list == list(range(token_list[0], token_list[0] + len(token_list)))
    table = torch.tensor([[0] * len(pages), pages], dtype=torch.int32, device=DEV)
    col_tiles = col_tiles or ops.attention_col_tiles(d)
    tiles = ops.attention_tiles(np.asarray([0, len(token_list)]), nq // nkv, col_tiles * (waves if shared else 1),
                                np.asarray([token_list[-1] + 1]) if waves > 1 else None)
    if waves > 1 and tiles.shape[0] > 1:
        # the tiles that see the most keys come first (a tile's last column decides)
        groups, columns = col_tiles * (waves if shared else 1), len(token_list) * (nq // nkv)
        reach = [(min(int(col0) + 16 * groups, columns) - 1) // (nq // nkv) for col0 in tiles[:, 3]]
        assert reach == sorted(reach, reverse=True)
    tiles[:, 0] = 1                                                            # the sequence is row 1 of the table
    split_len = ((tokens + nsplit - 1) // nsplit + 31) // 32 * 32
    rows = q[token_list].bfloat16().reshape(len(token_list), nq * d).contiguous().to(DEV)
    positions = torch.tensor(token_list, dtype=torch.int32, device=DEV)
    out = ops.attention_mfma(rows, cache.to(DEV), table, torch.from_numpy(tiles).to(DEV), positions, nq, nkv, d, window,
                             1.0 / math.sqrt(d), nsplit, split_len, col_tiles, waves, shared)
    if len(token_list) == 1 and waves == 1:
        # the same step as a decode step: no work list, the kernel derives the tiles; the sequence must be row 0
        decode = ops.attention_mfma(rows, cache.to(DEV), table[1:].contiguous(), None, positions, nq, nkv, d, window,
                                    1.0 / math.sqrt(d), nsplit, split_len)
        assert torch.equal(decode, out)
        # several waves of a workgroup sharing the keys: the same result within rounding (the sums run in another order)
        waves = 2
        while waves <= ops.attention_max_waves(d):
            shared = ops.attention_mfma(rows, cache.to(DEV), table[1:].contiguous(), None, positions, nq, nkv, d, window,
                                        1.0 / math.sqrt(d), nsplit, split_len, 1, waves)
            assert rel_err(shared, out.double()) < 1e-2, f"{waves} waves"
            waves *= 2
    return out.view(len(token_list), nq, d)


@pytest.mark.parametrize("case", [
    dict(tokens=3, nq=2, nkv=1, d=16, page=16),
    dict(tokens=77, nq=6, nkv=3, d=48, page=16),
    dict(tokens=300, nq=5, nkv=5, d=80, page=32),
    dict(tokens=700, nq=8, nkv=1, d=128, page=16),
    dict(tokens=333, nq=4, nkv=2, d=16, page=32, window=37),
    dict(tokens=130, nq=3, nkv=1, d=256, page=64),
    dict(tokens=200, nq=32, nkv=4, d=64, page=16),
    dict(tokens=150, nq=40, nkv=2, d=32, page=16, window=50),         # 20 heads a group: more than one tile per token
    dict(tokens=97, nq=7, nkv=7, d=112, page=16),
])
def test_attention_mfma(case):
    from tlie_amd import ops
    tokens, nq, nkv, d, page = case["tokens"], case["nq"], case["nkv"], case["d"], case["page"]
    window = case.get("window")
    torch.manual_seed(tokens)
    q, k, v = torch.randn(tokens, nq, d), torch.randn(tokens, nkv, d), torch.randn(tokens, nkv, d)
    want = plain_attention(rounded(q, torch.bfloat16), rounded(k, torch.bfloat16), rounded(v, torch.bfloat16), window=window)
    whole = run_attention_mfma(q, k, v, page, window, 1, shuffle_seed=tokens)
    assert rel_err(whole, want) < TOL["bfloat16"]
    for col_tiles in (1, 2, 4):                                   # 16, 32, 64 columns a wave, where the head size allows
        if col_tiles * d <= 256:
            narrow = run_attention_mfma(q, k, v, page, window, 1, shuffle_seed=tokens, col_tiles=col_tiles)
            assert rel_err(narrow, want) < TOL["bfloat16"], f"{col_tiles} column groups"
    # 2 and 4 waves of a workgroup share each tile's keys (whole and in 3 parts), the tiles longest first
    for waves, nsplit in ((2, 1), (4, 1), (4, 3)):
        col_tiles = 2 if d <= 128 else 1
        if waves <= ops.attention_max_waves(d, col_tiles):
            shared = run_attention_mfma(q, k, v, page, window, nsplit, shuffle_seed=tokens, col_tiles=col_tiles, waves=waves)
            assert rel_err(shared, want) < TOL["bfloat16"], f"{waves} waves, {nsplit} parts"
    # the waves of a workgroup take columns of their own, keys and values reach them through LDS
    if d <= 128:
        for waves, nsplit, col_tiles in ((4, 1, 2), (8, 1, 2), (4, 3, 2), (4, 1, 1), (8, 2, 1)):
            through_lds = run_attention_mfma(q, k, v, page, window, nsplit, shuffle_seed=tokens, col_tiles=col_tiles, waves=waves,
                                             shared=True)
            assert rel_err(through_lds, want) < TOL["bfloat16"], f"through LDS, {waves} waves of {col_tiles * 16} columns, {nsplit} parts"
    # the last token alone (a decode step), its key range cut in parts that are merged
    for nsplit in (1, 2, 5):
        last = run_attention_mfma(q, k, v, page, window, nsplit, token_list=[tokens - 1], shuffle_seed=tokens)
        assert rel_err(last[0], want[-1]) < TOL["bfloat16"], f"nsplit {nsplit}"
    # a portion in the middle that starts and ends off the page and block boundaries
    first, count = max(0, tokens // 2 - 9), min(21, tokens - max(0, tokens // 2 - 9))
    portion = run_attention_mfma(q, k, v, page, window, 1, token_list=list(range(first, first + count)), shuffle_seed=tokens)
    assert rel_err(portion, want[first:first + count]) < TOL["bfloat16"]
    if d <= 128:
        portion = run_attention_mfma(q, k, v, page, window, 1, token_list=list(range(first, first + count)), shuffle_seed=tokens,
                                     col_tiles=2, waves=4, shared=True)
        assert rel_err(portion, want[first:first + count]) < TOL["bfloat16"], "a portion through LDS"
        portion = run_attention_mfma(q, k, v, page, window, 1, token_list=list(range(first, first + count)), shuffle_seed=tokens,
                                     col_tiles=1, waves=4, shared=True)
        assert rel_err(portion, want[first:first + count]) < TOL["bfloat16"], "a portion through LDS, 16 columns a wave"
    split_portion = run_attention_mfma(q, k, v, page, window, 3, token_list=list(range(first, first + count)), shuffle_seed=tokens)
    assert rel_err(split_portion, want[first:first + count]) < TOL["bfloat16"]


def test_attention_mfma_finds_one_key_among_hundreds():
    tokens, nq, nkv, d, page = 600, 4, 2, 32, 16
    torch.manual_seed(1)
    base_k, v = torch.randn(tokens, nkv, d) * 0.1, torch.randn(tokens, nkv, d)
    q = torch.randn(tokens, nq, d) * 0.1
    direction = torch.zeros(d)
    direction[3] = 1.0
    q[tokens - 1] += 12.0 * direction
    for window, needle, inside in [(None, 0, True), (None, 15, True), (None, 16, True), (None, 31, True), (None, 32, True),
                                   (None, 511, True), (None, 598, True), (None, 599, True), (100, 500, True), (100, 499, False),
                                   (16, 584, True), (16, 583, False)]:
        k = base_k.clone()
        k[needle] += 12.0 * direction
        for nsplit in (1, 4):
            got = run_attention_mfma(q, k, v, page, window, nsplit, token_list=[tokens - 1], shuffle_seed=needle)[0].float().cpu()
            wanted_rows = v[needle].bfloat16().float().repeat_interleave(nq // nkv, dim=0)
            hit = (got - wanted_rows).abs().max().item() < 0.05
            assert hit == inside, f"window {window}, needle at {needle}, nsplit {nsplit}: {'missed' if inside else 'seen'}"


def test_attention_mfma_over_thousands_of_keys():
    """A sequence of more pages than the 128 whose numbers a wave keeps at hand while it brings
    blocks through LDS (2600 positions in pages of 16): the last tokens' queries against all keys, by
    every walk, and needles on both sides of the place where the page numbers are loaded again."""
    tokens, nq, nkv, d, page = 2600, 4, 2, 32, 16
    torch.manual_seed(5)
    k, v = torch.randn(tokens, nkv, d) * 0.1, torch.randn(tokens, nkv, d)
    q = torch.randn(tokens, nq, d) * 0.1
    direction = torch.zeros(d)
    direction[5] = 1.0
    first, count = tokens - 150, 150
    for needle in (0, 2047, 2048, 2080, tokens - 151):
        keys = k.clone()
        keys[needle] += 12.0 * direction
        queries = q.clone()
        queries[first:] += 12.0 * direction
        want = plain_attention(rounded(queries, torch.bfloat16), rounded(keys, torch.bfloat16), rounded(v, torch.bfloat16))[first:]
        assert (want - v[needle].bfloat16().double().repeat_interleave(nq // nkv, dim=0)).abs().max() < 0.05   # the needle decides
        for col_tiles, waves, shared, nsplit in ((2, 4, True, 1), (1, 4, True, 1), (2, 8, True, 2), (2, 4, False, 1), (1, 1, False, 3)):
            got = run_attention_mfma(queries, keys, v, page, None, nsplit, token_list=list(range(first, first + count)),
                                     shuffle_seed=needle, col_tiles=col_tiles, waves=waves, shared=shared)
            assert rel_err(got, want) < TOL["bfloat16"], f"needle {needle}: {col_tiles} groups, {waves} waves, shared {shared}, {nsplit} parts"


def test_attention_mfma_finds_one_key_among_tens_of_thousands():
    """33000 positions in pages of 16 (a block table of 2063 entries, 17 times the 128 that a wave keeps
    at hand): the last token alone, as a decode step with the keys in one part and in sixteen, and the last
    40 tokens as a portion that walks all keys through LDS; a key that stands out at the sequence's
    start, at places where parts and table windows meet, and at its end decides the result."""
    tokens, nq, nkv, d, page = 33000, 4, 2, 64, 16
    torch.manual_seed(9)
    base_k, v = torch.randn(tokens, nkv, d) * 0.1, torch.randn(tokens, nkv, d)
    q = torch.randn(tokens, nq, d) * 0.1
    direction = torch.zeros(d)
    direction[7] = 1.0
    q[tokens - 40:] += 14.0 * direction
    for needle in (0, 2047, 2048, 2063, 16383, 16384, 20625, 32767, 32959):
        k = base_k.clone()
        k[needle] += 14.0 * direction
        wanted_rows = v[needle].bfloat16().float().repeat_interleave(nq // nkv, dim=0)
        for nsplit in (1, 16):
            got = run_attention_mfma(q, k, v, page, None, nsplit, token_list=[tokens - 1], shuffle_seed=needle)[0].float().cpu()
            assert (got - wanted_rows).abs().max().item() < 0.05, f"decode, needle at {needle}, {nsplit} parts: missed"
        got = run_attention_mfma(q, k, v, page, None, 1, token_list=list(range(tokens - 40, tokens)), shuffle_seed=needle,
                                 col_tiles=2, waves=4, shared=True).float().cpu()
        assert (got - wanted_rows).abs().max().item() < 0.05, f"portion, needle at {needle}: missed"


def test_attention_mfma_mixed_step():
    """Three sequences in one step: a portion of a prompt, one decoded token, a whole short prompt;
    each must equal what it gives alone."""
    from tlie_amd import ops
    import numpy as np
    nq, nkv, d, page = 6, 2, 64, 16
    torch.manual_seed(9)
    lengths, brings = [90, 200, 11], [(50, 40), (199, 1), (0, 11)]             # (first position, count) brought by the step
    qs, ks, vs = zip(*[(torch.randn(n, nq, d), torch.randn(n, nkv, d), torch.randn(n, nkv, d)) for n in lengths])
    caches, tables, offset = [], [], 0
    for index in range(3):
        cache, pages = build_cache(ks[index], vs[index], page, torch.bfloat16, shuffle_seed=index)
        tables.append([page_index + offset for page_index in pages])
        offset += cache.shape[0]
        caches.append(cache)
    width = max(len(t) for t in tables)
    table = torch.tensor([t + [0] * (width - len(t)) for t in tables], dtype=torch.int32, device=DEV)
    q_rows = torch.cat([qs[i][first:first + count] for i, (first, count) in enumerate(brings)]).bfloat16().reshape(-1, nq * d)
    positions = torch.tensor([p for first, count in brings for p in range(first, first + count)], dtype=torch.int32, device=DEV)
    seq_start = np.cumsum([0] + [count for _, count in brings])
    tiles = torch.from_numpy(ops.attention_tiles(seq_start, nq // nkv, 4)).to(DEV)
    for nsplit in (1, 3):
        out = ops.attention_mfma(q_rows.contiguous().to(DEV), torch.cat(caches).to(DEV), table, tiles, positions, nq, nkv, d,
                                 None, 1.0 / math.sqrt(d), nsplit, 96, 4).view(-1, nq, d)
        cursor = 0
        for index, (first, count) in enumerate(brings):
            want = plain_attention(rounded(qs[index], torch.bfloat16), rounded(ks[index], torch.bfloat16),
                                   rounded(vs[index], torch.bfloat16))[first:first + count]
            assert rel_err(out[cursor:cursor + count], want) < TOL["bfloat16"], f"sequence {index}, nsplit {nsplit}"
            cursor += count


# ---- at most 16 rows: products with the norm before and the gate or the residual add after ----------------

def partial_sums_of_squares(rows, columns_per_part=16):
    """[ceil(width / columns_per_part), 16]: per group of columns and per row the sum of squares, as the
    kernels leave it."""
    count, width = rows.shape
    parts = (width + columns_per_part - 1) // columns_per_part
    padded = torch.zeros(count, parts * columns_per_part, dtype=torch.float64)
    padded[:, :width] = rows.double()
    out = torch.zeros(parts, 16, dtype=torch.float64)
    out[:, :count] = (padded.view(count, parts, columns_per_part) ** 2).sum(-1).T
    return out


@pytest.mark.parametrize("shape", [(1, 40, 64), (3, 177, 176), (8, 2560, 2048), (16, 100, 520), (5, 2048, 5632), (11, 50, 8),
                                   (16, 11264, 2048), (2, 4100, 1000)])
def test_gemm_rows(shape):
    from tlie_amd import ops
    m, n, k = shape
    torch.manual_seed(n + m)
    x = torch.randn(m, k).bfloat16()
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    b = torch.randn(n).bfloat16()
    want = plain_linear(x.double(), w.double(), b.double())
    got = ops.gemm_rows(x.to(DEV), w.to(DEV), b.to(DEV)).dense()
    assert got.dtype == torch.float32 and rel_err(got, want) < 5e-6
    for waves in (2, 4, 8, 16):
        for rows_per_block in (2, 6, 8, 10, 12, 16, 32):
            if rows_per_block == 32 and waves == 16:
                with pytest.raises(ops.EngineError):
                    ops.gemm_rows(x.to(DEV), w.to(DEV), b.to(DEV), waves=waves, rows_per_block=rows_per_block)
                continue
            got = ops.gemm_rows(x.to(DEV), w.to(DEV), b.to(DEV), waves=waves, rows_per_block=rows_per_block).dense()
            assert rel_err(got, want) < 5e-6, (waves, rows_per_block)
    # the norm before the product, folded in: the product runs on residual * g, its rows are scaled
    residual = torch.randn(m, k) * 3
    g = (1 + 0.2 * torch.randn(k)).bfloat16()
    eps = 1e-5
    xg = (residual * g.float()).bfloat16()
    scale = 1.0 / torch.sqrt((residual.double() ** 2).mean(-1, keepdim=True) + eps)
    want = plain_linear(xg.double(), w.double()) * scale + b.double()
    for columns in (16, 8):                       # the partial sums may come per 16 columns or per 8
        normed = ops.NormedRows(xg.to(DEV), partial_sums_of_squares(residual, columns).float().to(DEV), eps)
        got = ops.gemm_rows(normed, w.to(DEV), b.to(DEV)).dense()
        assert rel_err(got, want) < 1e-5
    # and it is the norm: against RMSNorm then product, within the rounding of the input to bfloat16
    want_normed = plain_linear(plain_rms_norm(residual, g.double(), eps), w.double(), b.double())
    assert rel_err(got, want_normed) < TOL["bfloat16"]
    if n % 2 == 0:
        # rows of W alternate gate and up
        full = plain_linear(x.double(), w.double())
        for rows_per_block, waves in ((8, None), (16, None), (32, 4), (32, 2), (16, 2), (10, None), (6, 16)):
            act = ops.gemm_rows(x.to(DEV), w.to(DEV), None, "silu", rows_per_block=rows_per_block, waves=waves)
            assert act.shape == (m, n // 2) and rel_err(act, plain_silu_mul(full[:, 0::2], full[:, 1::2])) < TOL["bfloat16"]
        # the same layout through the kernel that adds up partial sums
        parts = ops.gemm_skinny(x.to(DEV), w.to(DEV), None, split_len=64)
        assert rel_err(ops.silu_mul(parts, torch.bfloat16, interleaved=True), plain_silu_mul(full[:, 0::2], full[:, 1::2])) < TOL["bfloat16"]
    # added into the residual, with the next norm's inputs
    target = torch.randn(m, n)
    next_g = (1 + 0.2 * torch.randn(n)).bfloat16()
    for next_weight, rows_per_block in ((next_g, 16), (next_g.float(), 8), (next_g, 32), (next_g, 10)):
        res_dev = target.clone().to(DEV)
        updated = ops.gemm_rows(x.to(DEV), w.to(DEV), b.to(DEV), "residual", residual=res_dev,
                                next_norm=(next_weight.to(DEV), 1e-6), rows_per_block=rows_per_block,
                                waves=2 if rows_per_block == 32 else None)
        want_res = target.double() + plain_linear(x.double(), w.double(), b.double())
        assert rel_err(res_dev, want_res) < 5e-6
        assert rel_err(updated.normed.xg, want_res * next_g.double()) < TOL["bfloat16"]
        columns = min(rows_per_block, 16)                  # a block of 32 rows leaves its two strips' sums apart
        want_ssq = partial_sums_of_squares(res_dev.cpu(), columns)[:, :m]
        assert updated.normed.ssq.shape[0] >= want_ssq.shape[0]
        assert rel_err(updated.normed.ssq[:want_ssq.shape[0], :m], want_ssq) < 1e-5
        assert updated.normed.ssq[want_ssq.shape[0]:, :m].abs().max().item() == 0 if updated.normed.ssq.shape[0] > want_ssq.shape[0] else True
        assert updated.normed.eps == 1e-6
    res_dev = target.clone().to(DEV)
    plain_update = ops.gemm_rows(x.to(DEV), w.to(DEV), None, "residual", residual=res_dev)
    assert plain_update.normed is None and rel_err(res_dev, target.double() + plain_linear(x.double(), w.double())) < 5e-6


def test_embed_rows_and_refusals():
    from tlie_amd import EngineError, ops
    tokens = torch.tensor([0, 300, 17, 17, 5], dtype=torch.int32, device=DEV)
    for hidden, dtype in ((72, torch.bfloat16), (70, torch.bfloat16), (2056, torch.bfloat16), (40, torch.float32)):
        table = torch.randn(301, hidden).to(dtype).to(DEV)       # 70: no multiple of 4, one element a thread
        g = (1 + 0.2 * torch.randn(hidden)).to(dtype).to(DEV)
        residual, normed = ops.embed_rows(tokens, table, (g, 1e-5))
        rows = table.float().cpu()[tokens.long().cpu()]
        assert torch.equal(residual.cpu(), rows)
        assert rel_err(normed.xg, rows.double() * g.double().cpu()) < TOL["bfloat16"]
        assert rel_err(normed.ssq[:, :5], partial_sums_of_squares(rows)[:, :5]) < 1e-5
    with pytest.raises(EngineError):
        ops.gemm_rows(torch.randn(17, 64, device=DEV).bfloat16(), torch.randn(8, 64, device=DEV).bfloat16(), None)
    with pytest.raises(EngineError):
        ops.gemm_rows(torch.randn(2, 64, device=DEV).bfloat16(), torch.randn(7, 64, device=DEV).bfloat16(), None, "silu")
    assert not ops.gemm_rows_takes(4, torch.randn(8, 12, device=DEV).bfloat16(), torch.bfloat16)


@pytest.mark.parametrize("case", [dict(nq=5, nkv=3, d=48, rot=48, page=8), dict(nq=4, nkv=1, d=64, rot=32, page=16),
                                  dict(nq=2, nkv=2, d=16, rot=0, page=16), dict(nq=32, nkv=4, d=64, rot=64, page=16)])
def test_rotation_in_paired_order_and_inside_the_product(case):
    """The fused q/k/v weight's rows may be stored with rotation pairs side by side.  The rotation
    kernel reading such columns, and the product of few rows that rotates and writes the cache
    itself, must give what the plain order through the plain kernels gives."""
    from tlie_amd import ops
    nq, nkv, d, rot, page = case["nq"], case["nkv"], case["d"], case["rot"], case["page"]
    tokens, hidden = 7, 72
    torch.manual_seed(d + rot)
    x = torch.randn(tokens, hidden).bfloat16().to(DEV)
    w = (torch.randn((nq + 2 * nkv) * d, hidden) / math.sqrt(hidden)).bfloat16().to(DEV)
    b = torch.randn((nq + 2 * nkv) * d).bfloat16().to(DEV)
    positions = torch.tensor([0, 1, 77, 4095, 5, 6, 300], dtype=torch.int32, device=DEV)
    slots = torch.tensor([3, 12, -1, 40, 41, 7, 0], dtype=torch.int32, device=DEV)
    inv_freq = None
    if rot:
        inv_freq = torch.pow(torch.tensor(10000.0), -2.0 * torch.arange(rot // 2, dtype=torch.float32) / rot).to(DEV)

    def fresh_cache():
        return torch.full((8, 2, nkv, page * d), -3.0, dtype=torch.bfloat16, device=DEV)
    plain_cache = fresh_cache()
    plain_q = ops.rope_cache(ops.gemm_skinny(x, w, b), positions, slots, inv_freq, rot, plain_cache, nq, nkv, d, torch.bfloat16)
    order = ops.paired_rows(nq, nkv, d, rot).to(DEV)
    assert sorted(order.tolist()) == list(range((nq + 2 * nkv) * d))
    if rot:
        assert order[:4].tolist() == [0, rot // 2, 1, rot // 2 + 1]
    w_paired, b_paired = w[order].contiguous(), b[order].contiguous()
    paired_cache = fresh_cache()
    paired_q = ops.rope_cache(ops.gemm_skinny(x, w_paired, b_paired), positions, slots, inv_freq, rot, paired_cache, nq, nkv, d,
                              torch.bfloat16, paired=True)
    assert torch.equal(paired_q, plain_q) and torch.equal(paired_cache, plain_cache)
    for rows_per_block, waves in ((8, None), (16, None), (10, None), (12, None), (None, None), (32, 4), (32, 8), (32, 2)):
        fused_cache = fresh_cache()
        target = ops.RopeTarget(positions, slots, inv_freq, rot, fused_cache, nq, nkv, d)
        fused_q = ops.gemm_rows(x, w_paired, b_paired, "rope", rope=target, rows_per_block=rows_per_block, waves=waves)
        # the two products sum in another order, so the last bit of a bfloat16 may differ
        assert rel_err(fused_q, plain_q.double()) < 1e-2
        assert rel_err(fused_cache, plain_cache.double()) < 1e-2
        untouched = plain_cache == -3.0
        assert torch.equal(fused_cache[untouched], plain_cache[untouched])


@pytest.mark.parametrize("seed", range(24))
def test_attention_and_products_at_random_sizes(seed):
    """Sizes drawn at random (head sizes in steps of 16, any number of heads and groups, pages of
    16 to 64 rows, windows, key parts, waves; product sizes that are no multiples of the tiles):
    a portion of a sequence and its last token through the tiled attention kernel, and the same
    random product through both kernels for few rows."""
    from tlie_amd import ops
    rng = random.Random(seed)
    torch.manual_seed(seed)
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256])
    nkv, group = rng.randint(1, 4), rng.choice([1, 2, 3, 4, 5, 8, 17])
    nq, tokens, page = nkv * group, rng.randint(1, 420), rng.choice([16, 32, 64])
    window = rng.choice([None, None, rng.randint(1, 200)])
    q, k, v = torch.randn(tokens, nq, d), torch.randn(tokens, nkv, d), torch.randn(tokens, nkv, d)
    want = plain_attention(rounded(q, torch.bfloat16), rounded(k, torch.bfloat16), rounded(v, torch.bfloat16), window=window)
    col_tiles = rng.choice([c for c in (1, 2, 4) if c * d <= 256])
    waves = rng.choice([w for w in (1, 2, 4, 8) if w <= ops.attention_max_waves(d, col_tiles)])
    nsplit = rng.choice([1, 1, 2, 3, 7])
    first = rng.randint(0, tokens - 1)
    count = rng.randint(1, tokens - first)
    what = f"d={d} nq={nq} nkv={nkv} tokens={tokens} page={page} window={window} col_tiles={col_tiles} waves={waves} nsplit={nsplit}"
    got = run_attention_mfma(q, k, v, page, window, nsplit, token_list=list(range(first, first + count)), shuffle_seed=seed,
                             col_tiles=col_tiles, waves=waves)
    assert rel_err(got, want[first:first + count]) < TOL["bfloat16"], what
    last = run_attention_mfma(q, k, v, page, window, nsplit, token_list=[tokens - 1], shuffle_seed=seed)
    assert rel_err(last[0], want[-1]) < TOL["bfloat16"], what

    m, n, inner = rng.randint(1, 64), rng.choice([rng.randint(1, 300), 2 * rng.randint(1, 2000)]), 8 * rng.randint(1, 700)
    x, w, b = torch.randn(m, inner).bfloat16(), (torch.randn(n, inner) / math.sqrt(inner)).bfloat16(), torch.randn(n).bfloat16()
    want = plain_linear(x.double(), w.double(), b.double())
    what = f"m={m} n={n} k={inner}"
    got = ops.gemm_skinny(x.to(DEV), w.to(DEV), b.to(DEV), split_len=rng.choice([None, 64, 128, 512])).dense()
    assert rel_err(got, want) < 1e-5, what
    if m <= 16:
        waves = rng.choice([2, 4, 8, 16])
        rows_per_block = rng.choice([8, 16, 32, 10, 4] if waves <= 8 else [8, 16, 12, 14])
        got = ops.gemm_rows(x.to(DEV), w.to(DEV), b.to(DEV), waves=waves, rows_per_block=rows_per_block).dense()
        assert rel_err(got, want) < 1e-5, (what, waves, rows_per_block)
        if n % 2 == 0:
            full = plain_linear(x.double(), w.double())
            act = ops.gemm_rows(x.to(DEV), w.to(DEV), None, "silu", waves=waves, rows_per_block=rows_per_block)
            assert rel_err(act, plain_silu_mul(full[:, 0::2], full[:, 1::2])) < TOL["bfloat16"], (what, waves, rows_per_block)
