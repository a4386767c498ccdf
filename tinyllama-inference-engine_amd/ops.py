"""Python faces of the HIP kernels.

Every function checks on the host that operand shapes, types and index ranges are what the kernel
and its grid assume, raises `EngineError` when they are not, and only then launches on torch's
current stream.  Nothing here computes anything in torch: without the compiled library (and a
GPU) these functions fail.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

import torch

from .csrc import build as _build
from .errors import EngineError, ErrorCode, invalid_argument, invalid_shape

F32, BF16 = 0, 1
ROWS_MAX = 16          # the most rows the products take that fold in the layer's neighbouring arithmetic
ATTENTION_MAX_HEAD_DIM = 256   # the largest head size that both attention kernels take
GENERIC_TILED_MIN_TOKENS = 4   # a sequence's tokens in a step from which the plain attention shares its reads of the keys
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dtype: torch.dtype) -> int:
    if dtype not in _CODES:
        raise EngineError(ErrorCode.INVALID_DTYPE, f"kernels take float32 or bfloat16, not {dtype}")
    return _CODES[dtype]


def library() -> ctypes.CDLL:
    return _build.load()


def _ptr(tensor: torch.Tensor | None):
    return ctypes.c_void_p(tensor.data_ptr()) if tensor is not None else ctypes.c_void_p(0)


def _stream():
    # the current stream of the current device, by the accessors that cost no Python (a step of
    # prompt portions makes some two hundred launches, and torch.cuda.current_stream() alone took
    # a quarter of the time the host needs for them)
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _check(status: int, what: str) -> None:
    if status == 0:
        return
    if status == -1:
        raise invalid_argument(f"{what}: the kernel does not take these sizes or types")
    raise EngineError(ErrorCode.HIP, f"{what}: the launch failed (status {status})")


def _device_tensor(tensor: torch.Tensor, name: str, dtype: torch.dtype | tuple | None = None) -> None:
    if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda:
        raise invalid_argument(f"{name} must be a tensor on the GPU")
    if not tensor.is_contiguous():
        raise invalid_argument(f"{name} must be contiguous")
    if dtype is not None:
        allowed = dtype if isinstance(dtype, tuple) else (dtype,)
        if tensor.dtype not in allowed:
            raise EngineError(ErrorCode.INVALID_DTYPE, f"{name} has dtype {tensor.dtype}, expected one of {allowed}")


@dataclass
class Product:
    """The result of a matrix product: [rows, cols], or `nsplit` float partial sums
    [nsplit, rows, cols] of a split-K kernel that the consumer adds up."""
    data: torch.Tensor
    nsplit: int = 1

    @property
    def rows(self) -> int:
        return self.data.shape[-2]

    @property
    def cols(self) -> int:
        return self.data.shape[-1]

    @property
    def split_stride(self) -> int:
        return self.rows * self.cols

    def dense(self, dtype: torch.dtype | None = None) -> torch.Tensor:
        """The summed result as one tensor (for parts that do not fuse the sum)."""
        if self.nsplit == 1:
            out = self.data.view(self.rows, self.cols)        # nothing to add up: no kernel runs
        else:
            out = self.data.view(self.nsplit, self.rows, self.cols).sum(0)
        return out if dtype is None or out.dtype == dtype else out.to(dtype)


def as_product(value) -> Product:
    if isinstance(value, Product):
        return value
    if isinstance(value, torch.Tensor) and value.dim() == 2:
        return Product(value.contiguous(), 1)
    raise invalid_argument("a part must return a [tokens, width] tensor or a Product")


def _check_product(product: Product, name: str) -> None:
    _device_tensor(product.data, name, (torch.float32, torch.bfloat16))
    if product.nsplit < 1 or product.data.numel() != product.nsplit * product.rows * product.cols:
        raise invalid_shape(f"{name}: {product.nsplit} splits do not fit a tensor of shape {list(product.data.shape)}")
    if product.nsplit > 1 and product.data.dtype != torch.float32:
        raise EngineError(ErrorCode.INVALID_DTYPE, f"{name}: partial sums must be float32")


# ---------------------------------------------------------------------------------------------
def embed_gather(tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """float32 residual[t, :] = table[tokens[t], :].  The caller has checked 0 <= token < vocab."""
    _device_tensor(tokens, "tokens", torch.int32)
    _device_tensor(table, "embedding table", (torch.float32, torch.bfloat16))
    if tokens.dim() != 1 or table.dim() != 2:
        raise invalid_shape("embed_gather takes tokens [T] and a table [vocab, hidden]")
    out = torch.empty((tokens.shape[0], table.shape[1]), dtype=torch.float32, device=table.device)
    _check(library().tlie_embed_gather(_ptr(tokens), _ptr(table), dtype_code(table.dtype), _ptr(out),
                                       tokens.shape[0], table.shape[1], _stream()), "embed_gather")
    return out


def add_rmsnorm(residual: torch.Tensor, delta: Product | None, weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: torch.Tensor | None = None, want_out: bool = True) -> torch.Tensor | None:
    """residual += delta (all rows, in place) and out = RMSNorm(residual) * weight.

    With `rows` (int32 indices) only those rows are normed, from residual + delta, and the
    residual is left as it was.  `delta` may be None (norm only)."""
    _device_tensor(residual, "residual", torch.float32)
    _device_tensor(weight, "norm weight", (torch.float32, torch.bfloat16))
    if residual.dim() != 2 or weight.shape != (residual.shape[1],):
        raise invalid_shape(f"add_rmsnorm: residual {list(residual.shape)} and weight {list(weight.shape)} do not fit")
    if not eps > 0.0:
        raise EngineError(ErrorCode.NUMERICAL, "RMSNorm requires a positive epsilon")
    tokens, hidden = residual.shape
    delta_code, nsplit, stride = F32, 1, 0
    if delta is not None:
        _check_product(delta, "delta")
        if (delta.rows, delta.cols) != (tokens, hidden):
            raise invalid_shape(f"add_rmsnorm: delta [{delta.rows}, {delta.cols}] does not fit residual {list(residual.shape)}")
        delta_code, nsplit, stride = dtype_code(delta.data.dtype), delta.nsplit, delta.split_stride
    count = tokens
    if rows is not None:
        _device_tensor(rows, "rows", torch.int32)
        count = rows.shape[0]
        if count == 0:
            return torch.empty((0, hidden), dtype=out_dtype, device=residual.device)
    out = torch.empty((count, hidden), dtype=out_dtype, device=residual.device) if want_out else None
    _check(library().tlie_add_rmsnorm(_ptr(residual), _ptr(delta.data if delta is not None else None), delta_code, nsplit,
                                      ctypes.c_longlong(stride), _ptr(weight), dtype_code(weight.dtype),
                                      ctypes.c_float(eps), _ptr(out), dtype_code(out_dtype), _ptr(rows), count, hidden,
                                      _stream()), "add_rmsnorm")
    return out


def silu_mul(gate_up: Product, out_dtype: torch.dtype, interleaved: bool = False) -> torch.Tensor:
    """out[t, i] = silu(gate[t, i]) * up[t, i], with gate_up = [gate | up] side by side or, interleaved,
    g0 u0 g1 u1 ..."""
    _check_product(gate_up, "gate_up")
    if gate_up.cols % 2 != 0:
        raise invalid_shape("silu_mul: the input holds gate and up side by side, its width must be even")
    rows, inter = gate_up.rows, gate_up.cols // 2
    out = torch.empty((rows, inter), dtype=out_dtype, device=gate_up.data.device)
    _check(library().tlie_silu_mul(_ptr(gate_up.data), dtype_code(gate_up.data.dtype), gate_up.nsplit,
                                   ctypes.c_longlong(gate_up.split_stride), _ptr(out), dtype_code(out_dtype), rows, inter,
                                   1 if interleaved else 0, _stream()), "silu_mul")
    return out


def _check_cache(cache: torch.Tensor, num_kv_heads: int, head_dim: int, what: str) -> int:
    """cache: [pages, 2, nkv, page_size * d]; per page and kv head the keys lie as [row][dim] and
    the values transposed, [dim][row].  Returns the page size."""
    if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[2] != num_kv_heads or cache.shape[3] % head_dim != 0:
        raise invalid_shape(f"{what}: cache {list(cache.shape)} is not [pages, 2, nkv, page_size * d]")
    return cache.shape[3] // head_dim


def paired_rows(num_heads: int, num_kv_heads: int, head_dim: int, rot_dim: int) -> torch.Tensor:
    """The order in which the rows of a fused q/k/v weight are stored when rotation pairs are to sit
    side by side: within each q and k head, element i of the rotated part goes to 2i and element
    i + rot_dim / 2 to 2i + 1; everything else stays.  Returns the source row of each stored row."""
    half = rot_dim // 2
    inside = []
    for i in range(half):
        inside += [i, i + half]
    inside += list(range(rot_dim, head_dim))
    order = []
    for head in range(num_heads + num_kv_heads):
        order += [head * head_dim + e for e in inside]
    order += list(range((num_heads + num_kv_heads) * head_dim, (num_heads + 2 * num_kv_heads) * head_dim))
    return torch.tensor(order, dtype=torch.long)


def rope_cache(qkv: Product, positions: torch.Tensor, slot_map: torch.Tensor, inv_freq: torch.Tensor | None,
               rot_dim: int, cache: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
               act_dtype: torch.dtype, paired: bool = False) -> torch.Tensor:
    """Rotates q and k, returns q [T, nq * d], writes k and v into the cache rows of `slot_map`.
    paired: qkv's columns are in the order of `paired_rows`.

    slot_map[t] = page * page_size + row, or -1 to skip.  The slot map comes from the cache
    manager, which hands out only rows of pages it owns."""
    _check_product(qkv, "qkv")
    _device_tensor(positions, "positions", torch.int32)
    _device_tensor(slot_map, "slot_map", torch.int32)
    _device_tensor(cache, "cache", act_dtype)
    tokens = qkv.rows
    if qkv.cols != (num_heads + 2 * num_kv_heads) * head_dim:
        raise invalid_shape(f"rope_cache: qkv width {qkv.cols} is not (nq + 2 nkv) * d")
    if positions.shape != (tokens,) or slot_map.shape != (tokens,):
        raise invalid_shape("rope_cache: positions and slot_map need one entry per token")
    page_size = _check_cache(cache, num_kv_heads, head_dim, "rope_cache")
    if inv_freq is not None:
        _device_tensor(inv_freq, "inv_freq", torch.float32)
        if rot_dim % 2 != 0 or not 0 < rot_dim <= head_dim or inv_freq.shape != (rot_dim // 2,):
            raise invalid_shape("rope_cache: inv_freq needs rot_dim / 2 entries, rot_dim even and at most d")
    else:
        rot_dim = 0
    q_out = torch.empty((tokens, num_heads * head_dim), dtype=act_dtype, device=cache.device)
    _check(library().tlie_rope_cache(_ptr(qkv.data), dtype_code(qkv.data.dtype), qkv.nsplit,
                                     ctypes.c_longlong(qkv.split_stride), _ptr(positions), _ptr(slot_map), _ptr(inv_freq),
                                     rot_dim, _ptr(q_out), _ptr(cache), dtype_code(act_dtype), tokens, num_heads,
                                     num_kv_heads, head_dim, page_size, 1 if paired else 0, _stream()), "rope_cache")
    return q_out


def attention_generic(q: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor, token_seq: torch.Tensor,
                      positions: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                      window: int | None, scale: float, tiled: bool | int = False, seq_start: torch.Tensor | None = None,
                      min_tokens: int = GENERIC_TILED_MIN_TOKENS) -> torch.Tensor:
    """Causal attention of every token over its sequence's cached keys; any number of tokens per
    sequence.  block_table: [sequences, max_blocks] pages; token_seq[t]: the token's row of it.
    tiled 1 (True): the step's sequences bring several tokens each (consecutive in the step, at
    consecutive positions): neighbouring tokens then share each read of the keys (head sizes up to
    64; the result has the same bits either way).  tiled 2: both kernels are launched and every token
    is served by one of them: by the tiled one if its sequence brings `min_tokens` tokens or more
    (seq_start: the step's cumulative token counts [sequences + 1], on the device), by the plain one
    otherwise: for steps that mix portions of prompts with single tokens."""
    _device_tensor(q, "q", (torch.float32, torch.bfloat16))
    _device_tensor(cache, "cache", q.dtype)
    _device_tensor(block_table, "block_table", torch.int32)
    _device_tensor(token_seq, "token_seq", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    tokens = q.shape[0]
    if q.shape != (tokens, num_heads * head_dim):
        raise invalid_shape(f"attention: q {list(q.shape)} is not [tokens, nq * d]")
    page_size = _check_cache(cache, num_kv_heads, head_dim, "attention")
    if block_table.dim() != 2 or token_seq.shape != (tokens,) or positions.shape != (tokens,):
        raise invalid_shape("attention: block_table must be [sequences, max_blocks], token_seq and positions [tokens]")
    if num_heads % num_kv_heads != 0:
        raise invalid_shape("attention: the number of heads must be a multiple of the number of kv heads")
    tiled = int(tiled)
    if tiled == 2:
        _device_tensor(seq_start, "seq_start", torch.int32)
        if seq_start.dim() != 1 or seq_start.shape[0] != block_table.shape[0] + 1 or min_tokens < 1:
            raise invalid_shape("attention: seq_start needs one entry more than the block table has rows, min_tokens at least 1")
    elif tiled not in (0, 1):
        raise invalid_argument("attention: tiled is 0, 1 or 2")
    out = torch.empty_like(q)
    _check(library().tlie_attention_generic(_ptr(q), _ptr(cache), dtype_code(q.dtype), _ptr(block_table),
                                            block_table.shape[1], _ptr(token_seq), _ptr(positions), _ptr(out), tokens,
                                            num_heads, num_kv_heads, head_dim, page_size,
                                            int(window) if window else 0, ctypes.c_float(scale), tiled,
                                            _ptr(seq_start if tiled == 2 else None), int(min_tokens), _stream()),
           "attention_generic")
    return out


def attention_generic_plan(ctx, head_dim: int) -> int:
    """Which form of the plain attention kernel a step takes (the `tiled` of `attention_generic`): the
    one that shares each read of the keys among a sequence's tokens pays from a few tokens a
    sequence on, and costs dearly where a workgroup's 32 columns belong to many sequences of one
    token (it walks each one's context in turn).  A launched step is decided from its host arrays;
    a recorded step of portions, whose cut changes from replay to replay, launches both and lets
    each sequence's token count on the device decide."""
    if head_dim > 64 or ctx.max_new < GENERIC_TILED_MIN_TOKENS:
        return 0
    if ctx.tile_owner is not None:
        return 2
    starts = ctx.host["seq_start"]
    counts = starts[1:] - starts[:-1]
    many = int((counts >= GENERIC_TILED_MIN_TOKENS).sum())
    return 1 if many == len(counts) else (2 if many else 0)


def gemm_generic(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out_dtype: torch.dtype) -> Product:
    """y = x . W^T (+ bias), every product and sum in true 32-bit.  W is [out, in]."""
    _device_tensor(x, "x", (torch.float32, torch.bfloat16))
    _device_tensor(weight, "weight", (torch.float32, torch.bfloat16))
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise invalid_shape(f"gemm: x {list(x.shape)} and weight {list(weight.shape)} do not fit")
    if bias is not None:
        _device_tensor(bias, "bias", weight.dtype)
        if bias.shape != (weight.shape[0],):
            raise invalid_shape("gemm: bias needs one entry per output")
    out = torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=x.device)
    if x.shape[0] == 0:
        return Product(out, 1)
    _check(library().tlie_gemm_generic(_ptr(x), dtype_code(x.dtype), _ptr(weight), dtype_code(weight.dtype), _ptr(bias),
                                       _ptr(out), dtype_code(out_dtype), x.shape[0], weight.shape[0], x.shape[1],
                                       _stream()), "gemm_generic")
    return Product(out, 1)


# state: None (not tried), True, False (not there); fallbacks: products that took this library's plain kernel instead
_library_gemm = {"state": None, "workspace": {}, "fallbacks": 0, "warned": set()}
LIBRARY_WORKSPACE_BYTES = 32 << 20


def library_mm(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """y = x . W^T of bfloat16 operands through the vendor's library (hipBLASLt), for steps of many
    rows; y in bfloat16, or in float32 (the output head's logits).  The library is called
    directly, with its plan for the shape kept (half the host time of torch.mm, which a step of
    prompt portions calls four times a layer); where that is not possible (the library's file
    is not beside torch, or it has no algorithm for the shape) this library's plain kernel makes the
    product."""
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise EngineError(ErrorCode.INVALID_DTYPE, f"library_mm gives bfloat16 or float32, not {out_dtype}")
    _device_tensor(x, "x", torch.bfloat16)
    _device_tensor(weight, "weight", torch.bfloat16)
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise invalid_shape(f"library_mm: x {list(x.shape)} and weight {list(weight.shape)} do not fit")
    state = _library_gemm
    if state["state"] is None:
        import os
        path = os.path.join(os.path.dirname(torch.__file__), "lib", "libhipblaslt.so")
        torch.mm(x[:1], weight[:1].t())                       # torch loads and sets up its copy of the library first
        state["state"] = os.path.isfile(path) and library().tlie_library_gemm_init(path.encode()) == 0
    if state["state"] and x.shape[0] > 0:
        index = x.device.index or 0
        if index not in state["workspace"]:
            state["workspace"][index] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
        workspace = state["workspace"][index]
        out = torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=x.device)
        status = library().tlie_library_gemm(_ptr(x), _ptr(weight), _ptr(out), int(out_dtype == torch.float32), x.shape[0],
                                             weight.shape[0], x.shape[1], _ptr(workspace), ctypes.c_size_t(workspace.numel()),
                                             _stream())
        if status == 0:
            return out
        if status != -3:
            _check(status, "library_gemm")
    # where the library cannot be called directly (its file is not beside torch, or it has no
    # algorithm for the shape) this library's own kernels make the product: the tiled one on the matrix
    # cores (some two thirds of the vendor's speed) for sizes it takes, else the plain 32-bit one (many
    # times slower); one route, recorded or not, so that a step gives the same bits replayed and launched
    # (and safe inside a recording, where a library call that has not been tried may clear a workspace
    # with a memset node)
    if x.shape[0] > 0:
        state["fallbacks"] += 1
        shape = (x.shape[0], weight.shape[0], weight.shape[1])
        if shape not in state["warned"]:
            # said once per shape: nothing else shows why a prompt step is ten times slower than it should be
            state["warned"].add(shape)
            import warnings
            why = "has no algorithm within its workspace for" if state["state"] else "is not available for"
            how = ("this library's tiled kernel, at some two thirds of the speed" if gemm_tiles_takes(weight)
                   else "this library's plain 32-bit kernel, which is many times slower")
            warnings.warn(f"the vendor's matrix library {why} the bfloat16 product {shape[0]} x {shape[1]} x {shape[2]}; "
                          f"it takes {how}", stacklevel=2)
    if gemm_tiles_takes(weight):
        return gemm_tiles(x, weight, out_dtype)
    return gemm_generic(x, weight, None, out_dtype).data


def gemm_tiles_takes(weight: torch.Tensor) -> bool:
    return weight.dtype == torch.bfloat16 and weight.shape[1] % 64 == 0 and weight.shape[0] % 4 == 0


def gemm_tiles(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """y = x . W^T of bfloat16 operands on this library's own tiled kernel for many rows (tiles of 128
    rows of W by 128 tokens on the matrix cores): what `library_mm` runs where the vendor's library
    cannot be called.  The inner size a multiple of 64, W's rows a multiple of 4; y bfloat16 or float32."""
    _device_tensor(x, "x", torch.bfloat16)
    _device_tensor(weight, "weight", torch.bfloat16)
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise invalid_shape(f"gemm_tiles: x {list(x.shape)} and weight {list(weight.shape)} do not fit")
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise EngineError(ErrorCode.INVALID_DTYPE, f"gemm_tiles gives bfloat16 or float32, not {out_dtype}")
    if not gemm_tiles_takes(weight):
        raise invalid_argument("gemm_tiles takes an inner size that is a multiple of 64 and a multiple of 4 of rows of W")
    out = torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=x.device)
    if x.shape[0] == 0:
        return out
    _check(library().tlie_gemm_tiles(_ptr(x), _ptr(weight), _ptr(out), int(out_dtype == torch.float32), x.shape[0],
                                     weight.shape[0], x.shape[1], _stream()), "gemm_tiles")
    return out


def library_fallbacks() -> int:
    """How many products `library_mm` has made with this library's own kernels because the vendor's
    library was not there or offered nothing for the shape (each slower, some many times)."""
    return _library_gemm["fallbacks"]


def add_bias(product: torch.Tensor, bias: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """out = product + bias (one entry per column) for a float32 product that came without its bias;
    the sum is float32 and rounded once to `out_dtype` (float32: in place)."""
    _device_tensor(product, "product", torch.float32)
    _device_tensor(bias, "bias", (torch.float32, torch.bfloat16))
    if product.dim() != 2 or bias.shape != (product.shape[1],):
        raise invalid_shape(f"add_bias: product {list(product.shape)} and bias {list(bias.shape)} do not fit")
    out = product if out_dtype == torch.float32 else torch.empty(product.shape, dtype=out_dtype, device=product.device)
    if product.shape[0] == 0:
        return out
    _check(library().tlie_add_bias(_ptr(product), _ptr(bias), dtype_code(bias.dtype), _ptr(out), dtype_code(out_dtype),
                                   product.shape[0], product.shape[1], _stream()), "add_bias")
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor | None = None, top_p: torch.Tensor | None = None,
           seed: torch.Tensor | None = None, counter: torch.Tensor | None = None,
           out: torch.Tensor | None = None) -> torch.Tensor:
    """One token per row of float32 logits: the first maximum when the row's temperature is not
    positive (or none is given), else a draw from the top-p part of softmax(logits / T) with the
    uniform number of (seed, counter).  A row with a NaN or an infinity gives -1.  `out`: int32
    [rows] to write into (else a new tensor)."""
    _device_tensor(logits, "logits", torch.float32)
    if logits.dim() != 2:
        raise invalid_shape("sample takes logits [rows, vocab]")
    rows = logits.shape[0]
    for name, tensor, dtype in (("temperature", temperature, torch.float32), ("top_p", top_p, torch.float32),
                                ("seed", seed, torch.int64), ("counter", counter, torch.int64)):
        if tensor is not None:
            _device_tensor(tensor, name, dtype)
            if tensor.shape != (rows,):
                raise invalid_shape(f"sample: {name} needs one entry per row")
    if out is None:
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    else:
        _device_tensor(out, "out", torch.int32)
        if out.shape != (rows,):
            raise invalid_shape("sample: out needs one entry per row")
    if rows == 0:
        return out
    _check(library().tlie_sample(_ptr(logits), rows, logits.shape[1], _ptr(temperature), _ptr(top_p), _ptr(seed),
                                 _ptr(counter), _ptr(out), _stream()), "sample")
    return out


def feed_tokens(tokens: torch.Tensor, source: torch.Tensor, sampled: torch.Tensor, vocab: int) -> None:
    """tokens[i] = sampled[source[i]] wherever source[i] >= 0, on the device, brought into the
    vocabulary's range 0 .. vocab - 1 (a sample of -1 marks a row of logits that held a NaN or an
    infinity: the host raises when it reads it, and the step that is already launched takes token 0).
    The caller has checked on the host that every such source is a row of `sampled`."""
    for name, tensor in (("tokens", tokens), ("source", source), ("sampled", sampled)):
        _device_tensor(tensor, name, torch.int32)
    if tokens.dim() != 1 or source.shape != tokens.shape or sampled.dim() != 1 or sampled.shape[0] == 0:
        raise invalid_shape("feed_tokens takes tokens [T], source [T] and sampled [rows]")
    if vocab <= 0:
        raise invalid_argument("feed_tokens: the vocabulary's size must be positive")
    if tokens.shape[0] == 0:
        return
    _check(library().tlie_feed_tokens(_ptr(tokens), _ptr(source), _ptr(sampled), tokens.shape[0], int(vocab), _stream()),
           "feed_tokens")


# ---- bfloat16 kernels on the matrix cores ---------------------------------------------------------
SKINNY_MAX_ROWS = 64
def skinny_split_len(rows: int, out_features: int, in_features: int) -> int:
    """How many k values one split takes when the matrix has work for many workgroups per compute
    unit.  Measured on the MI355X inside whole decode steps: the gated feed-forward's first product
    (11264 rows and more) with 512, and 1024 once the step has more than 32 rows of x, because each
    partial sum is a write and a read of rows x outputs; a long inner size (4096 and more) with 1024
    up to 32 rows and 512 beyond; the others with 256."""
    strips = (out_features + 15) // 16
    if strips >= 512:
        length = 1024 if rows > 32 else 512
    else:
        length = 256
    if in_features >= 4096:
        length = max(length, 1024 if rows <= 32 else 512)
    return min(length, (in_features + 63) // 64 * 64)


_SKINNY_PLANS: dict = {}
_COMPUTE_UNITS: dict = {}


def _compute_units(device: torch.device) -> int:
    index = device.index or 0
    if index not in _COMPUTE_UNITS:
        _COMPUTE_UNITS[index] = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return _COMPUTE_UNITS[index]


def skinny_plan(rows: int, out_features: int, in_features: int, compute_units: int = 256) -> tuple[int, int, int]:
    """The launch shape of `gemm_skinny`: (k values per split, waves a workgroup, strips of 16 rows
    of W a wave).  A compute unit draws some 20 GB/s from memory whatever its waves ask for, so a
    matrix of up to 64 MB is cut into as many equal workgroups as there are compute units, or just
    fewer (the product takes as long as the unit with the most bytes: TinyLlama's q/k/v matrix at 64
    rows 7.4 -> 6.4 us, the output projection 6.9 -> 5.7, gate/up 17.9 -> 16.9, down 11.0 -> 10.3),
    by the number of waves (each takes 16 rows of W) and the number of splits, each split costing a
    write and a read of rows x outputs partial sums (a decode step of the TinyLlama shape at batch
    64 2.10 -> 2.01 ms, at 32 1.69 -> 1.63).  Larger matrices keep many workgroups per compute unit
    (several at once hide each other's waits, which counts for more there)."""
    key = (rows, out_features, in_features, compute_units)
    if key in _SKINNY_PLANS:
        return _SKINNY_PLANS[key]
    plan = (skinny_split_len(rows, out_features, in_features), 4, 2 if rows > 32 else 1)
    if out_features * in_features * 2 <= (64 << 20):
        best = None
        for waves in range(4, 17):
            blocks = -(-out_features // (16 * waves))
            for nsplit in range(1, 33):
                split_len = (-(-in_features // nsplit) + 63) // 64 * 64
                if -(-in_features // split_len) != nsplit:
                    continue
                rounds = -(-blocks * nsplit // compute_units)
                # microseconds: a workgroup's bytes at 20 GB/s and half a microsecond per round; the partial sums at 6 TB/s
                # (the coefficients that gave the fastest whole decode steps at 20, 32 and 64 rows)
                cost = rounds * (16 * waves * split_len * 2 / 20e3 + 0.5) + nsplit * rows * out_features * 8 / 6e6
                if best is None or cost < best[0]:
                    best = (cost, split_len, waves, 1)
        plan = best[1:]
    _SKINNY_PLANS[key] = plan
    return plan


def gemm_skinny_takes(x: torch.Tensor, weight: torch.Tensor) -> bool:
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and 0 < x.shape[0] <= SKINNY_MAX_ROWS
            and weight.shape[1] % 8 == 0)


def skinny_gated_plan(rows: int, out_features: int, in_features: int, compute_units: int = 256) -> tuple[int, int]:
    """(waves a workgroup, strips a wave) of `gemm_skinny` when it keeps all of K in a workgroup and applies
    the SiLU gate itself: as many equal workgroups as compute units, or just fewer (see `skinny_plan`); a
    workgroup's time is its rows of W from memory and all of x from the caches."""
    best = None
    for strips in ((1, 2) if rows > 32 else (1,)):
        for waves in range(3, (8 if strips == 2 else 16) + 1):
            blocks = -(-out_features // (16 * waves * strips))
            rounds = -(-blocks // compute_units)
            cost = rounds * (16 * waves * strips * in_features * 2 / 20e3 + 0.5)
            if best is None or cost < best[0]:
                best = (cost, waves, strips)
    return best[1], best[2]


def gemm_skinny(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, split_len: int | None = None,
                waves: int | None = None, strips: int | None = None, gated: bool = False):
    """y = x . W^T (+ bias) for at most 64 rows of bfloat16 x: float partial sums [nsplit, M, N].
    split_len, waves, strips: the launch shape (see `skinny_plan`, which chooses it when they are not given).
    gated: W's rows alternate gate and up; K is not split, and the kernel stores bfloat16
    silu(gate) * up [M, N / 2], which is returned as a tensor (no partial sums, no activation kernel)."""
    _device_tensor(x, "x", torch.bfloat16)
    _device_tensor(weight, "weight", torch.bfloat16)
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise invalid_shape(f"gemm_skinny: x {list(x.shape)} and weight {list(weight.shape)} do not fit")
    rows, (out_features, in_features) = x.shape[0], weight.shape
    if not 0 < rows <= SKINNY_MAX_ROWS or in_features % 8 != 0:
        raise invalid_argument(f"gemm_skinny takes 1..{SKINNY_MAX_ROWS} rows and an inner size that is a multiple of 8")
    if bias is not None:
        _device_tensor(bias, "bias", torch.bfloat16)
        if bias.shape != (out_features,):
            raise invalid_shape("gemm_skinny: bias needs one entry per output")
    if gated:
        if out_features % 2 != 0:
            raise invalid_shape("gemm_skinny: the gated product needs an even number of rows of W")
        if split_len is not None and split_len < in_features:
            raise invalid_argument("gemm_skinny: the gated product does not split K")
        split_len = (in_features + 63) // 64 * 64
        if waves is None or strips is None:
            waves, strips = skinny_gated_plan(rows, out_features, in_features, _compute_units(x.device))
    elif split_len is None:
        split_len, waves, strips = skinny_plan(rows, out_features, in_features, _compute_units(x.device))
    elif waves is None or strips is None:
        waves, strips = waves or 4, strips or (2 if rows > 32 else 1)
    if split_len <= 0 or split_len % 64 != 0:
        raise invalid_argument("gemm_skinny: a split's length must be a positive multiple of 64")
    if not 3 <= waves <= 16 or strips not in (1, 2) or (strips == 2 and (rows <= 32 or waves > 8)):
        raise invalid_argument("gemm_skinny: 3 to 16 waves; two strips a wave only for more than 32 rows and up to 8 waves")
    nsplit = (in_features + split_len - 1) // split_len
    if gated:
        act = torch.empty((rows, out_features // 2), dtype=torch.bfloat16, device=x.device)
        _check(library().tlie_gemm_skinny(_ptr(x), _ptr(weight), _ptr(bias), _ptr(None), _ptr(act), rows, out_features, in_features,
                                          split_len, waves, strips, _stream()), "gemm_skinny")
        return act
    out = torch.empty((nsplit, rows, out_features), dtype=torch.float32, device=x.device)
    _check(library().tlie_gemm_skinny(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), _ptr(None), rows, out_features, in_features,
                                      split_len, waves, strips, _stream()), "gemm_skinny")
    return Product(out, nsplit)


def attention_col_tiles(head_dim: int) -> int:
    """How many groups of 16 columns a wave of the tiled attention kernel serves in a step that
    brings prompt portions.  The registers hold 4 for head sizes up to 64; 2 measured faster there
    (a prompt of 2048 tokens: 70 us against 92 with 4 waves a tile), the softmax arithmetic of one
    wave then overlapping the products of another."""
    return 2 if head_dim <= 128 else 1


def attention_max_waves(head_dim: int, col_tiles: int = 1) -> int:
    """How many waves of a workgroup of the tiled attention kernel may share a tile's keys."""
    fit, cap = 1024 // (col_tiles * head_dim), 4 if col_tiles * head_dim > 128 else 8
    return max(1, min(fit, cap))


def attention_tiles(seq_start, groups_per_kv: int, col_tiles: int = 1, seq_len=None):
    """The work list of the tiled attention kernel for a step, on the host: for every sequence,
    tiles of 16 * col_tiles columns, a column being a (token, query head of one group) pair.
    seq_start: the step's cumulative token counts [S + 1].  seq_len: the sequences' lengths after
    the step [S]; with it the tiles are ordered by the number of keys they see, most first, so
    that the longest are not the last to start.  Returns an int32 array [tiles, 4]:
    (sequence, its first token's index in the step, its number of tokens, the tile's first column)."""
    import numpy as np
    rows, keys = [], []
    for seq in range(len(seq_start) - 1):
        first, count = int(seq_start[seq]), int(seq_start[seq + 1] - seq_start[seq])
        for col0 in range(0, count * groups_per_kv, 16 * col_tiles):
            rows.append((seq, first, count, col0))
            if seq_len is not None:
                last_token = min(count - 1, (col0 + 16 * col_tiles - 1) // groups_per_kv)
                keys.append(int(seq_len[seq]) - count + last_token + 1)
    rows = np.asarray(rows, dtype=np.int32).reshape(-1, 4)
    if seq_len is not None and len(keys) > 1:
        rows = rows[np.argsort(-np.asarray(keys), kind="stable")]
    return np.ascontiguousarray(rows)


def few_rows_route(rows: int, dtype: torch.dtype) -> bool:
    """Whether a step of `rows` tokens may take the route on which the products of few rows fold in
    the norm before them and the add (or gate, or rotation) after them: bfloat16, at most 16 rows."""
    return dtype == torch.bfloat16 and 0 < rows <= ROWS_MAX


def attention_plan(ctx, groups_per_kv: int, num_kv_heads: int, head_dim: int):
    """How the tiled attention kernel is launched for the step `ctx` describes: its work list (made
    once per step and group size, kept in `ctx.scratch`; None for a decode step, whose tiles the
    kernel derives itself), and how the keys are cut: into as many parts as it takes to give a step
    of few tiles about a thousand waves (measured: at batch 64 and 2048 positions 4 parts reach
    5 TB/s, 16 parts 4 TB/s, and merging more than 16 costs more than it gains), each part a
    multiple of 32 positions and at least 64.  The policy is this kernel's own and measured on the
    MI355X; the step's context only supplies the host arrays, the number of compute units, and, in a
    recorded step, the owner of work lists at fixed addresses.
    Returns (tiles, col_tiles, nsplit, split_len, waves, shared): `waves` of a workgroup share a
    tile's keys, or with `shared` take columns of their own and get the keys through LDS."""
    decode = ctx.max_new == 1 and ctx.num_seqs == ctx.num_tokens
    col_tiles, shared = 1, False
    if decode:
        tiles, count = None, ctx.num_tokens * ((groups_per_kv + 15) // 16)
    else:
        col_tiles = attention_col_tiles(head_dim)
        # sequences of some length with portions of many columns: 4 waves take columns of their own
        # of one tile and every block of keys is brought once for all of them, through LDS (a
        # prompt of 1536 tokens: 34 us against 42; of 8192: 450 against 780; of 512: 15 against
        # 13).  Each wave takes 32 columns, or 16 while that leaves no more tiles than two and a
        # half for every compute unit: the smaller ones then fill the chip better, four
        # workgroups a compute unit (2048 tokens: 51 us against 63; 2560: 74 against 81; 3072:
        # 100 against 98; 4096: 162 against 150)
        shared = (col_tiles == 2 and head_dim <= 128 and ctx.max_context >= 768
                  and ctx.num_tokens * groups_per_kv >= 64 * ctx.num_seqs)

        def tiles_of(groups):
            key = ("attention_tiles", groups_per_kv, groups)
            if key not in ctx.scratch:
                def make(host):
                    return attention_tiles(host["seq_start"], groups_per_kv, groups, host["seq_len"])
                if ctx.tile_owner is not None:
                    # a sequence of n tokens has ceil(n * G / (16 * groups)) tiles
                    capacity = (ctx.num_tokens * groups_per_kv + 16 * groups - 1) // (16 * groups) + ctx.num_seqs
                    ctx.scratch[key] = ctx.tile_owner.tiles_for(key, make, capacity)
                else:
                    ctx.scratch[key] = torch.from_numpy(make(ctx.host)).to(ctx.tokens.device)
            return ctx.scratch[key]
        tiles = tiles_of(col_tiles * (4 if shared else 1))
        if shared and 2 * tiles.shape[0] * num_kv_heads <= 5 * ctx.compute_units:
            col_tiles = 1
            tiles = tiles_of(4)
        count = tiles.shape[0] * (4 if shared else 1)
    tiles_all = count * num_kv_heads
    if not decode:
        # a step of prompt portions has tiles enough; cutting their keys would only add merging,
        # unless few tiles see many keys (a short portion late in a long sequence): then into parts of
        # 256 keys or more (parts of 64 and more made prompts of 64 to 256 tokens 3 to 4% slower: 2.50 ->
        # 2.43 ms at 256 tokens).
        # Up to 4 waves share a tile's keys, each with 128 or more: a tile that sees the whole of
        # a long sequence then takes a quarter of the time, and it is the longest tiles that
        # the step waits for (a prompt of 2048 tokens: 70 us against 87 with one wave a tile)
        nsplit = max(1, min((512 + tiles_all - 1) // tiles_all, 16, ctx.max_context // 256))
        waves = 4 if shared else 1
        while (not shared and waves < 4 and waves * 2 <= attention_max_waves(head_dim, col_tiles)
               and ctx.max_context >= nsplit * waves * 2 * 128):
            waves *= 2
    else:
        # workgroups share a tile's keys until there is one for every compute unit (their sums
        # meet in the merge kernel); then the waves of a workgroup share them, which costs no
        # launch, while a wave keeps 128 keys or more and the step has 2048 waves at most
        # (measured inside whole steps at 2048 positions: batch 1 16 parts x 1 wave, batch 8
        # 8 x 2, batch 64 1 x 8)
        nsplit = max(1, min((256 + tiles_all - 1) // tiles_all, 16, (ctx.max_context + 63) // 64))
        waves = 1
        while (waves * 2 <= attention_max_waves(head_dim) and tiles_all * nsplit * waves * 2 <= 2048
               and ctx.max_context >= nsplit * waves * 2 * 128):
            waves *= 2
        if nsplit > 1 and ctx.max_context <= 256 and attention_max_waves(head_dim) >= 2:
            # up to 256 positions there is nothing to cut: two waves of one workgroup share the keys and the
            # merge launch goes (batch 1 at 200 positions 0.902 ms a step against 0.919, batch 8 0.998
            # against 1.017; at 450 positions the parts win again: 0.928 against 0.944 with 1 x 4)
            nsplit, waves = 1, 2
    if nsplit == 1:
        return tiles, col_tiles, 1, 0, waves, shared
    split_len = ((ctx.max_context + nsplit - 1) // nsplit + 31) // 32 * 32
    nsplit = (ctx.max_context + split_len - 1) // split_len
    return tiles, col_tiles, nsplit, split_len, waves, shared


def attention_mfma_takes(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 0 < head_dim <= ATTENTION_MAX_HEAD_DIM and page_size >= 16
            and page_size & (page_size - 1) == 0)


def attention_mfma(q: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor, tiles: torch.Tensor | None,
                   positions: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, window: int | None,
                   scale: float, nsplit: int = 1, split_len: int = 0, col_tiles: int = 1, waves: int = 1,
                   shared: bool = False) -> torch.Tensor:
    """Causal attention of every token of the step over its sequence's cache, bfloat16.

    tiles: int32 [n, 4] from `attention_tiles` (built from the same step as block_table and
    positions: every tile's sequence is a row of block_table, its tokens are rows of q); None for
    a decode step, in which token i is the one token of sequence i.  nsplit > 1 cuts the keys into
    that many parts of split_len positions (a multiple of 32; nsplit * split_len must reach the
    longest sequence) that run side by side and are merged.  col_tiles: the value the tiles were
    made with.  waves (a power of two up to `attention_max_waves`): so many waves of a
    workgroup share each tile's (or part's) keys and merge their results before writing.
    shared (prompt portions; col_tiles 1 or 2, head size up to 128, 4 or 8 waves): the tiles were made
    with col_tiles * waves column groups, every wave takes col_tiles of them, and each block of keys
    and values is brought once for the whole workgroup."""
    _device_tensor(q, "q", torch.bfloat16)
    _device_tensor(cache, "cache", torch.bfloat16)
    _device_tensor(block_table, "block_table", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    tokens = q.shape[0]
    if q.shape != (tokens, num_heads * head_dim):
        raise invalid_shape(f"attention: q {list(q.shape)} is not [tokens, nq * d]")
    page_size = _check_cache(cache, num_kv_heads, head_dim, "attention")
    if block_table.dim() != 2 or positions.shape != (tokens,):
        raise invalid_shape("attention: block_table must be [sequences, max_blocks], positions [tokens]")
    if num_heads % num_kv_heads != 0:
        raise invalid_shape("attention: the number of heads must be a multiple of the number of kv heads")
    if not scale > 0:
        raise invalid_argument(f"attention: the scale {scale} of the scores is not positive")
    if tiles is not None:
        _device_tensor(tiles, "tiles", torch.int32)
        if tiles.dim() != 2 or tiles.shape[1] != 4 or tiles.shape[0] == 0:
            raise invalid_shape("attention: tiles must be [n, 4]")
        num_tiles = tiles.shape[0]
        if col_tiles not in (1, 2, 4) or col_tiles > (4 if head_dim <= 64 else (2 if head_dim <= 128 else 1)):
            raise invalid_argument(f"attention: {col_tiles} column groups a wave do not fit head size {head_dim}")
    else:
        col_tiles = 1
        if block_table.shape[0] < tokens:
            raise invalid_shape("attention: a decode step needs a block table row per token")
        num_tiles = tokens * ((num_heads // num_kv_heads + 15) // 16)
    if nsplit > 1 and (split_len <= 0 or split_len % 32 != 0):
        raise invalid_argument("attention: split_len must be a positive multiple of 32")
    if shared:
        if tiles is None or col_tiles not in (1, 2) or head_dim > 128 or waves not in (4, 8):
            raise invalid_argument("attention: sharing through LDS takes tiles, 1 or 2 column groups a wave, a head size up to 128 and 4 or 8 waves")
    elif waves not in (1, 2, 4, 8) or waves > attention_max_waves(head_dim, col_tiles):
        raise invalid_argument(f"attention: waves must be a power of two up to {attention_max_waves(head_dim, col_tiles)}")
    if not attention_mfma_takes(q.dtype, head_dim, page_size):
        raise invalid_argument("attention_mfma takes bfloat16, head sizes in steps of 16 up to 256, pages of a power of two of rows (at least 16)")
    out = torch.empty_like(q)
    part_o = part_ml = None
    if nsplit > 1:
        part_o = torch.empty((tokens * num_heads * nsplit, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((tokens * num_heads * nsplit, 2), dtype=torch.float32, device=q.device)
    _check(library().tlie_attention_mfma(_ptr(q), _ptr(cache), _ptr(block_table), block_table.shape[1], _ptr(tiles),
                                         num_tiles, col_tiles, _ptr(positions), _ptr(out), _ptr(part_o), _ptr(part_ml), nsplit,
                                         split_len, tokens, num_heads, num_kv_heads, head_dim, page_size,
                                         int(window) if window else 0, ctypes.c_float(scale), waves, int(bool(shared)), _stream()),
           "attention_mfma")
    return out


# ---- at most 16 rows: products with the layer's neighbouring arithmetic folded in --------------------


@dataclass
class NormedRows:
    """The input of a product, not yet normed: xg = bfloat16(residual * norm weight) [T, width] and
    partial sums of squares of the residual's rows, ssq [parts, 16] (each part covers some of the
    columns; their sum over the parts is the row's sum of squares).  The product applies
    rsqrt(sum(ssq) / width + eps) to its result's rows, which is the same as having normed the
    input."""
    xg: torch.Tensor
    ssq: torch.Tensor
    eps: float

    @property
    def shape(self):
        return self.xg.shape


@dataclass
class ResidualUpdated:
    """A product's result was added into the residual by the kernel that computed it; `normed`
    is the residual as the next norm's product wants it, when that was asked for."""
    normed: NormedRows | None


def gemm_rows_takes(rows: int, weight: torch.Tensor, dtype: torch.dtype) -> bool:
    return (dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and 0 < rows <= ROWS_MAX
            and weight.shape[1] % 8 == 0)


def gemm_rows_shape(out_features: int, in_features: int, epilogue: str = "store", compute_units: int = 256,
                    rows: int = 1) -> tuple[int, int]:
    """(waves that share K, rows of W per workgroup), measured inside whole decode steps on the
    TinyLlama shapes: about four thousand waves in all, 4 to 16 a workgroup (11264 rows: 4 waves a
    strip of 16, 1.15 ms a step against 1.25 with 8; 2560 rows: 16 waves, against 8 another 0.03 ms
    less); strips of 8 rows where 16 waves on strips of 16 are still too few and K is long
    (2048 rows, K = 5632).  Two strips a workgroup and 2 waves gained nothing at these sizes.
    Where strips of 16 rows leave compute units without a workgroup and the product's result feeds
    no norm (whose partial sums would grow in number with the workgroups), the rows are shared out
    evenly over the units instead: 2560 rows on 256 workgroups of 10 rather than 160 of 16, 0.7%
    of a step at batch 1 and 8; the same for the output projection (residual and norm sums) measured
    0.5% slower.
    With 8 rows of x and more, a workgroup's part of x weighs half as much as its 16 rows of W and
    more (both come through the L2): large matrices then take two strips a workgroup, which halves
    that share (Llama-3-8B's output head at 8 rows 239 -> 209 us, at 16 rows 269 -> 229; its gate/up
    61 -> 58, its q/k/v with 8 waves 17.7 -> 16.6; TinyLlama's head at 16 rows 37.6 -> 34.0)."""
    strips = (out_features + 15) // 16
    waves = 4
    while waves < 16 and strips * waves * 2 <= 4096 and in_features >= waves * 2 * 64:
        waves *= 2
    rows_per_block = 8 if (waves == 16 and strips * 16 < 3072 and in_features > 4096) else 16
    if waves == 16 and rows_per_block == 16 and epilogue in ("store", "rope") and compute_units // 2 < strips < compute_units:
        rows_per_block = max(8, (-(-out_features // compute_units) + 1) // 2 * 2)
    if rows >= 8 and ((waves == 4 and strips * rows >= 14336) or (waves == 8 and in_features >= 4096 and strips >= compute_units)):
        rows_per_block = 32
    return waves, rows_per_block


@dataclass
class RopeTarget:
    """What the rotation and cache write need besides the q/k/v product: see `rope_cache`."""
    positions: torch.Tensor
    slot_map: torch.Tensor
    inv_freq: torch.Tensor | None
    rot_dim: int
    cache: torch.Tensor
    num_heads: int
    num_kv_heads: int
    head_dim: int


def gemm_rows(x, weight: torch.Tensor, bias: torch.Tensor | None, epilogue: str = "store",
              residual: torch.Tensor | None = None, next_norm: tuple | None = None, waves: int | None = None,
              rows_per_block: int | None = None, rope: RopeTarget | None = None):
    """y = x . W^T (+ bias) for at most 16 rows.  x: bfloat16 [M, K], or `NormedRows` (then the
    result's rows are scaled as the norm would have scaled the input).
    epilogue "store": float32 [M, N] as a `Product`.  "silu": W's rows alternate gate and up;
    returns bfloat16 silu(gate) * up [M, N / 2].  "residual": residual [M, N] += y in place, returns
    a `ResidualUpdated`, with the next norm's inputs when next_norm = (weight [N], eps) is given.
    "rope": W is a fused q/k/v weight with rows in the order of `paired_rows`; q and k are rotated,
    k and v written to the cache (as `rope_cache` does), bfloat16 q [M, nq * d] is returned."""
    scale = x if isinstance(x, NormedRows) else None
    data = scale.xg if scale is not None else x
    _device_tensor(data, "x", torch.bfloat16)
    _device_tensor(weight, "weight", torch.bfloat16)
    if data.dim() != 2 or weight.dim() != 2 or data.shape[1] != weight.shape[1]:
        raise invalid_shape(f"gemm_rows: x {list(data.shape)} and weight {list(weight.shape)} do not fit")
    rows, (out_features, in_features) = data.shape[0], weight.shape
    if not gemm_rows_takes(rows, weight, data.dtype):
        raise invalid_argument(f"gemm_rows takes 1..{ROWS_MAX} rows of bfloat16 and an inner size that is a multiple of 8")
    if bias is not None:
        _device_tensor(bias, "bias", torch.bfloat16)
        if bias.shape != (out_features,):
            raise invalid_shape("gemm_rows: bias needs one entry per output")
    ssq_in, strips_in, eps = None, 0, 0.0
    if scale is not None:
        _device_tensor(scale.ssq, "ssq", torch.float32)
        if scale.ssq.dim() != 2 or scale.ssq.shape[1] != 16 or scale.ssq.shape[0] == 0:
            raise invalid_shape(f"gemm_rows: ssq {list(scale.ssq.shape)} is not [parts, 16]")
        ssq_in, strips_in, eps = scale.ssq, scale.ssq.shape[0], float(scale.eps)
    default_waves, default_rows = gemm_rows_shape(out_features, in_features, epilogue, _compute_units(data.device), rows)
    waves, rows_per_block = waves or default_waves, rows_per_block or default_rows
    if epilogue == "silu" and rows_per_block % 2 != 0:
        raise invalid_argument("gemm_rows: a gate and its up must fall into one block")
    device = data.device
    y = act = xg = ssq_out = next_weight = None
    next_code = BF16
    if epilogue == "store":
        code = 0
        y = torch.empty((rows, out_features), dtype=torch.float32, device=device)
    elif epilogue == "silu":
        code = 1
        if out_features % 2 != 0:
            raise invalid_shape("gemm_rows: the gated product needs an even number of rows of W")
        act = torch.empty((rows, out_features // 2), dtype=torch.bfloat16, device=device)
    elif epilogue == "residual":
        code = 2
        _device_tensor(residual, "residual", torch.float32)
        if residual.shape != (rows, out_features):
            raise invalid_shape(f"gemm_rows: residual {list(residual.shape)} is not [{rows}, {out_features}]")
        if next_norm is not None:
            next_weight = next_norm[0]
            _device_tensor(next_weight, "next norm weight", (torch.bfloat16, torch.float32))
            if next_weight.shape != (out_features,):
                raise invalid_shape("gemm_rows: the next norm's weight needs one entry per output")
            next_code = dtype_code(next_weight.dtype)
            xg = torch.empty((rows, out_features), dtype=torch.bfloat16, device=device)
            parts = (out_features + rows_per_block - 1) // rows_per_block * max(1, rows_per_block // 16)
            ssq_out = torch.empty((parts, 16), dtype=torch.float32, device=device)
    elif epilogue == "rope":
        code = 3
        if rope is None:
            raise invalid_argument("gemm_rows: the rotation epilogue needs a RopeTarget")
        _device_tensor(rope.positions, "positions", torch.int32)
        _device_tensor(rope.slot_map, "slot_map", torch.int32)
        _device_tensor(rope.cache, "cache", torch.bfloat16)
        if out_features != (rope.num_heads + 2 * rope.num_kv_heads) * rope.head_dim:
            raise invalid_shape(f"gemm_rows: {out_features} rows of W are not (nq + 2 nkv) * d")
        if rope.positions.shape != (rows,) or rope.slot_map.shape != (rows,):
            raise invalid_shape("gemm_rows: positions and slot_map need one entry per token")
        page_size = _check_cache(rope.cache, rope.num_kv_heads, rope.head_dim, "gemm_rows")
        rot_dim = rope.rot_dim if rope.inv_freq is not None else 0
        if rope.inv_freq is not None:
            _device_tensor(rope.inv_freq, "inv_freq", torch.float32)
            if rot_dim % 2 != 0 or not 0 < rot_dim <= rope.head_dim or rope.inv_freq.shape != (rot_dim // 2,):
                raise invalid_shape("gemm_rows: inv_freq needs rot_dim / 2 entries, rot_dim even and at most d")
        if rope.head_dim % 2 != 0:
            raise invalid_shape("gemm_rows: the rotation epilogue needs an even head size")
        q_out = torch.empty((rows, rope.num_heads * rope.head_dim), dtype=torch.bfloat16, device=device)
    else:
        raise invalid_argument(f"gemm_rows: unknown epilogue '{epilogue}'")
    if rope is None or epilogue != "rope":
        rope_args = (_ptr(None), _ptr(None), _ptr(None), 0, 0, 0, 0, 0, _ptr(None), _ptr(None))
    else:
        rope_args = (_ptr(rope.positions), _ptr(rope.slot_map), _ptr(rope.inv_freq), rot_dim, rope.num_heads,
                     rope.num_kv_heads, rope.head_dim, page_size, _ptr(q_out), _ptr(rope.cache))
    _check(library().tlie_gemm_rows(_ptr(data), _ptr(weight), _ptr(bias), rows, out_features, in_features, _ptr(ssq_in),
                                    strips_in, in_features, ctypes.c_float(eps), code, _ptr(y), _ptr(act), _ptr(residual),
                                    _ptr(next_weight), next_code, _ptr(xg), _ptr(ssq_out), *rope_args, waves, rows_per_block,
                                    _stream()), "gemm_rows")
    if epilogue == "rope":
        return q_out
    if epilogue == "store":
        return Product(y, 1)
    if epilogue == "silu":
        return act
    return ResidualUpdated(NormedRows(xg, ssq_out, float(next_norm[1])) if next_norm is not None else None)


def embed_rows(tokens: torch.Tensor, table: torch.Tensor, next_norm: tuple):
    """The embedding for at most 16 tokens with the first norm's inputs: returns (float32
    residual [T, hidden], NormedRows)."""
    _device_tensor(tokens, "tokens", torch.int32)
    _device_tensor(table, "embedding table", (torch.float32, torch.bfloat16))
    next_weight, next_eps = next_norm
    _device_tensor(next_weight, "next norm weight", (torch.bfloat16, torch.float32))
    if tokens.dim() != 1 or table.dim() != 2 or next_weight.shape != (table.shape[1],) or not 0 < tokens.shape[0] <= ROWS_MAX:
        raise invalid_shape("embed_rows takes 1..16 tokens, a table [vocab, hidden] and a norm weight [hidden]")
    count, hidden = tokens.shape[0], table.shape[1]
    residual = torch.empty((count, hidden), dtype=torch.float32, device=table.device)
    xg = torch.empty((count, hidden), dtype=torch.bfloat16, device=table.device)
    ssq = torch.empty(((hidden + 15) // 16, 16), dtype=torch.float32, device=table.device)
    _check(library().tlie_embed_rows(_ptr(tokens), _ptr(table), dtype_code(table.dtype), _ptr(residual), _ptr(next_weight),
                                     dtype_code(next_weight.dtype), _ptr(xg), _ptr(ssq), count, hidden, _stream()),
           "embed_rows")
    return residual, NormedRows(xg, ssq, float(next_eps))


# ---- the machine's own ceilings ---------------------------------------------------------------------
def measured_peaks(device="cuda:0", repeats: int = 5) -> dict:
    """What this GPU delivers to kernels that do nothing else: GB/s of a streaming read of 2 GiB
    (workgroups of 512 threads, four a compute unit, eight 16-byte loads in flight a thread) and
    TFLOP/s of chains of bfloat16 matrix instructions (32 x 32 x 16, eight independent chains a wave,
    eight waves a compute unit); the best of `repeats` timed launches each, after one warm-up."""
    device = torch.device(device)
    units = int(torch.cuda.get_device_properties(device).multi_processor_count)
    sink = torch.zeros(4, dtype=torch.float32, device=device)
    data = torch.empty(1 << 31, dtype=torch.uint8, device=device)
    data.fill_(1)
    blocks = 4 * units
    lib = library()
    lib.tlie_probe_stream_read_bytes.restype = ctypes.c_ulonglong
    read_bytes = lib.tlie_probe_stream_read_bytes(ctypes.c_ulonglong(data.numel()), blocks)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best_read = best_mfma = None
    iterations, mfma_blocks = 4096, 2 * units
    for run in range(repeats + 1):
        start.record()
        _check(lib.tlie_probe_stream_read(_ptr(data), ctypes.c_ulonglong(data.numel()), blocks, _ptr(sink), _stream()), "probe_stream_read")
        stop.record()
        stop.synchronize()
        seconds = start.elapsed_time(stop) / 1e3
        if run > 0:
            best_read = seconds if best_read is None else min(best_read, seconds)
        start.record()
        _check(lib.tlie_probe_mfma_bf16(iterations, mfma_blocks, _ptr(sink), _stream()), "probe_mfma_bf16")
        stop.record()
        stop.synchronize()
        seconds = start.elapsed_time(stop) / 1e3
        if run > 0:
            best_mfma = seconds if best_mfma is None else min(best_mfma, seconds)
    flops = mfma_blocks * 4 * 8 * iterations * 32768.0
    return {"stream_read_gbs": read_bytes / best_read / 1e9, "mfma_bf16_tflops": flops / best_mfma / 1e12}
