"""The entry point of the kernel library that allocates nothing, called as a C program would call
it (through ctypes): paged attention with the partial results of its key parts in the library's own
device array instead of buffers of the caller's.  Its output is compared, bit for bit, with that of
the entry point that takes buffers, on two calls in a row, the second smaller than the first (the
array still holds the first call's contents), and with the plain attention on the same keys and
values read back out of the pages; and a step beyond the array's size is refused."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def make_case(seed, seqs, length, nq, nkv, d, page_size=16):
    """A decode step: `seqs` sequences of `length` positions (the last one is the step's token)."""
    generator = torch.Generator().manual_seed(seed)
    blocks = (length + page_size - 1) // page_size
    pages = seqs * blocks + 3
    cache = (torch.randn((pages, 2, nkv, page_size * d), generator=generator) * 0.5).to(torch.bfloat16).cuda()
    order = torch.randperm(pages, generator=generator)[:seqs * blocks].to(torch.int32)
    table = order.view(seqs, blocks).contiguous().cuda()
    q = (torch.randn((seqs, nq * d), generator=generator)).to(torch.bfloat16).cuda()
    positions = torch.full((seqs,), length - 1, dtype=torch.int32).cuda()
    return q, cache, table, positions


def plain_decode_attention(q, cache, table, length, nq, nkv, d, page_size=16):
    """The plain attention's answer for the last position of every sequence: keys and values are
    gathered out of the pages (keys [row][dim], values [dim][row]) into whole sequences first."""
    rows = []
    for seq in range(q.shape[0]):
        pages = cache[table[seq].long()].double().cpu()                                   # [blocks, 2, nkv, page_size * d]
        keys = pages[:, 0].reshape(-1, nkv, page_size, d).permute(0, 2, 1, 3).reshape(-1, nkv, d)[:length]
        values = pages[:, 1].reshape(-1, nkv, d, page_size).permute(0, 3, 1, 2).reshape(-1, nkv, d)[:length]
        rows.append(last_row_attention(q[seq].double().cpu().view(nq, d), keys, values, nq // nkv))
    return torch.stack(rows).reshape(q.shape[0], nq * d)


def last_row_attention(query, keys, values, groups):
    """softmax(q . K^T / sqrt(d)) . V for one query per head over all `keys` (src/operators.cpp:117-143)."""
    from plain_llama import plain_softmax
    d = query.shape[-1]
    out = torch.zeros_like(query)
    for head in range(query.shape[0]):
        scores = (keys[:, head // groups] @ query[head]) * (1.0 / d ** 0.5)
        out[head] = plain_softmax(scores) @ values[:, head // groups]
    return out


def call_no_alloc(library, q, cache, table, positions, nq, nkv, d, page_size, scale, nsplit, split_len, waves):
    out = torch.empty_like(q)
    pointer = lambda tensor: ctypes.c_void_p(tensor.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tokens = q.shape[0]
    status = library.tlie_attention_mfma_no_alloc(
        pointer(q), pointer(cache), pointer(table), table.shape[1], ctypes.c_void_p(0), tokens * ((nq // nkv + 15) // 16), 1,
        pointer(positions), pointer(out), nsplit, split_len, tokens, nq, nkv, d, page_size, 0, ctypes.c_float(scale), waves, 0, stream)
    return status, out


def test_attention_without_allocation_equals_the_entry_point_that_takes_buffers():
    from tlie_amd import ops
    library = ops.library()
    library.tlie_attention_mfma_no_alloc.restype = ctypes.c_int
    nq, nkv, d = 8, 2, 64
    scale = d ** -0.5
    # the first call fills most of what the second one will use with other values
    for seqs, length, nsplit in ((6, 700, 8), (3, 300, 4), (5, 1000, 16)):
        split_len = ((length + nsplit - 1) // nsplit + 31) // 32 * 32
        parts = (length + split_len - 1) // split_len
        q, cache, table, positions = make_case(seqs * 1000 + length, seqs, length, nq, nkv, d)
        want = ops.attention_mfma(q, cache, table, None, positions, nq, nkv, d, None, scale, parts, split_len, 1, 2, False)
        torch.cuda.synchronize()
        status, got = call_no_alloc(library, q, cache, table, positions, nq, nkv, d, 16, scale, parts, split_len, 2)
        torch.cuda.synchronize()
        assert status == 0
        assert torch.equal(got, want), f"{seqs} sequences of {length}: the output differs from the entry point with buffers"
        assert torch.isfinite(got.float()).all()
        # and it is the attention: against the plain formulas on the pages' own keys and values
        plain = plain_decode_attention(q, cache, table, length, nq, nkv, d)
        assert (got.double().cpu() - plain).abs().max() <= 2e-2 * plain.abs().max(), f"{seqs} sequences of {length}: not the plain attention"
    # one part: no scratch memory at all
    q, cache, table, positions = make_case(5, 4, 100, nq, nkv, d)
    want = ops.attention_mfma(q, cache, table, None, positions, nq, nkv, d, None, scale, 1, 0, 1, 1, False)
    status, got = call_no_alloc(library, q, cache, table, positions, nq, nkv, d, 16, scale, 1, 0, 1)
    assert status == 0 and torch.equal(got, want)
    # beyond the array's 8 MiB: refused with its own code, nothing launched
    q, cache, table, positions = make_case(6, 256, 40, 32, 4, 64)
    status, _ = call_no_alloc(library, q, cache, table, positions, 32, 4, 64, 16, scale, 16, 32, 1)    # 256 * 32 * 16 * 66 floats = 34.6 MB
    assert status == -4
    torch.cuda.synchronize()
    # sizes the kernel does not take: refused like the other entry point refuses them
    status, _ = call_no_alloc(library, q, cache, table, positions, 32, 5, 64, 16, scale, 1, 0, 1)
    assert status == -1
