"""Typed Python wrappers of the kernel library: they check shapes, types and
devices on the host (a kernel is never launched on operands it was not written
for), allocate outputs with torch, and launch on torch's current stream, so a
step can be recorded into a HIP graph.
"""

from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass

import torch

from tokasaurus_amd.kernels.library import KernelError, call, load

_DT = {torch.float32: 0, torch.bfloat16: 1}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 storage, not {dtype}") from None


def _stream() -> int:
    """torch's current stream on the current device, as the raw handle the kernels launch on
    (the direct query: building a Stream object for it costs the host several microseconds
    a launch, a tenth of an eager step's time)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU; there is no CPU path")


def _i32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():  # (the message is made only when it is needed: this runs ten times a layer)
        raise KernelError(f"{name} must be contiguous int32")


KEY_PIECE = 8  # elements of a key that lie together in a page
VALUE_QUAD = 4  # tokens whose values lie together in a page


def key_pages_shape(pages: int, nkv: int, page_size: int, head_dim: int, padded: bool = False) -> tuple[int, ...]:
    """Keys: [pages, nkv, d / 8, P, 8]: a page holds the 8-element pieces of its P
    keys piece by piece, so that the lanes that feed the matrix cores (16 keys, one
    piece each) read consecutive memory.
    ``padded``: a head size that is no multiple of 8 gets its last piece filled up (only the
    kernels that address pages through ``key_page_elems`` take such a size) instead of a refusal."""
    _need(padded or head_dim % KEY_PIECE == 0, f"the cache keeps keys in pieces of {KEY_PIECE}: head size {head_dim} is no multiple")
    return (pages, nkv, -(-head_dim // KEY_PIECE), page_size, KEY_PIECE)


def value_pages_shape(pages: int, nkv: int, page_size: int, head_dim: int) -> tuple[int, ...]:
    """Values: [pages, nkv, P / 4, d, 4]: a page holds its tokens in groups of 4,
    for each group the d rows of 4 values."""
    _need(page_size % VALUE_QUAD == 0, f"the cache keeps values in groups of {VALUE_QUAD} tokens: page size {page_size} is no multiple")
    return (pages, nkv, page_size // VALUE_QUAD, head_dim, VALUE_QUAD)


def _check_pages(kcache: torch.Tensor, vcache: torch.Tensor, nkv: int, page_size: int, head_dim: int, dtype: torch.dtype, who: str,
                 value_dim: int | None = None) -> None:
    """``value_dim``: the size of a value head where it differs from a key head's."""
    pages = kcache.shape[0]
    vd = head_dim if value_dim is None else value_dim
    # (the shapes are compared in place: this runs twice a layer of an eager step)
    if (kcache.shape != (pages, nkv, -(-head_dim // KEY_PIECE), page_size, KEY_PIECE) or not kcache.is_contiguous()):
        raise KernelError(f"{who}: key pages must be contiguous {key_pages_shape(pages, nkv, page_size, head_dim)}, got {tuple(kcache.shape)}")
    if (vcache.shape != (pages, nkv, page_size // VALUE_QUAD, vd, VALUE_QUAD) or page_size % VALUE_QUAD or not vcache.is_contiguous()):
        raise KernelError(f"{who}: value pages must be contiguous {value_pages_shape(pages, nkv, page_size, vd)}, got {tuple(vcache.shape)}")
    if kcache.dtype != dtype or vcache.dtype != dtype:
        raise KernelError(f"{who}: the cache must be {dtype}")


def embed_gather(
    ids: torch.Tensor, table: torch.Tensor, last_token: torch.Tensor | None = None
) -> torch.Tensor:
    """out[t] = table[ids[t]]; ids[t] < 0 reads the token from last_token[-ids[t]-1]."""
    _gpu(ids, table, last_token)
    _i32(ids, "ids")
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [V, H]")
    if last_token is not None:
        _i32(last_token, "last_token")
    n = ids.numel()
    vocab, hidden = table.shape
    out = torch.empty((n, hidden), dtype=table.dtype, device=table.device)
    call(
        "tk_embed_gather",
        dtype_code(table.dtype),
        ids.data_ptr(),
        last_token.data_ptr() if last_token is not None else None,
        table.data_ptr(),
        out.data_ptr(),
        n,
        hidden,
        vocab,
        _stream(),
    )
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    _gpu(x, weight)
    _need(x.dim() == 2 and x.is_contiguous(), "rmsnorm input must be contiguous [rows, H]")
    rows, hidden = x.shape
    _need(weight.shape == (hidden,) and weight.is_contiguous(), "rmsnorm weight must be [H]")
    _need(
        weight.dtype in (x.dtype, torch.float32),
        f"rmsnorm weight is {weight.dtype}, expected {x.dtype} or float32",
    )
    out = torch.empty_like(x)
    w_f32 = 1 if (weight.dtype == torch.float32 and x.dtype != torch.float32) else 0
    call(
        "tk_rmsnorm",
        dtype_code(x.dtype),
        x.data_ptr(),
        weight.data_ptr(),
        w_f32,
        out.data_ptr(),
        rows,
        hidden,
        float(eps),
        _stream(),
    )
    return out


def add_rmsnorm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float) -> tuple[torch.Tensor, torch.Tensor]:
    """(x + residual rounded to the storage type, its RMSNorm times ``weight``) in one pass."""
    _gpu(x, residual, weight)
    _need(x.dim() == 2 and x.is_contiguous() and residual.shape == x.shape and residual.is_contiguous()
          and residual.dtype == x.dtype, "add_rmsnorm: x and residual must be contiguous [rows, H] of one type")
    rows, hidden = x.shape
    if weight.shape != (hidden,) or not weight.is_contiguous() or weight.dtype not in (x.dtype, torch.float32):
        raise KernelError(f"add_rmsnorm: the weight must be [H] of {x.dtype} or float32")
    stream_out, out = torch.empty_like(x), torch.empty_like(x)
    w_f32 = 1 if (weight.dtype == torch.float32 and x.dtype != torch.float32) else 0
    call("tk_add_rmsnorm", dtype_code(x.dtype), x.data_ptr(), residual.data_ptr(), weight.data_ptr(), w_f32,
         stream_out.data_ptr(), out.data_ptr(), rows, hidden, float(eps), _stream())
    return stream_out, out


def head_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, first_head: int, num_heads: int, head_dim: int) -> None:
    """RMSNorm, in place, of each of the ``num_heads`` heads of ``head_dim`` elements that start at
    head ``first_head`` of every row of ``x`` (2-d, unit inner stride): the per-head norm of queries
    or keys in a stacked q|k|v row, with one weight [head_dim] for all heads."""
    _gpu(x, weight)
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[1] >= (first_head + num_heads) * head_dim and first_head >= 0 and num_heads > 0,
          "head_rmsnorm: x must be 2-d with unit inner stride and hold the heads named")
    _need(weight.shape == (head_dim,) and weight.is_contiguous() and weight.dtype in (x.dtype, torch.float32),
          f"head_rmsnorm: the weight must be [{head_dim}] of {x.dtype} or float32")
    w_f32 = 1 if (weight.dtype == torch.float32 and x.dtype != torch.float32) else 0
    call("tk_head_rmsnorm", dtype_code(x.dtype), x.data_ptr(), x.stride(0), weight.data_ptr(), w_f32, x.shape[0],
         first_head * head_dim, num_heads, head_dim, float(eps), _stream())


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """[rows, 2I] laid out [gate | up] -> silu(gate) * up, [rows, I]."""
    _gpu(gate_up)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0,
          "swiglu input must be contiguous [rows, 2I]")
    rows, two_i = gate_up.shape
    out = torch.empty((rows, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    call("tk_swiglu", dtype_code(gate_up.dtype), gate_up.data_ptr(), out.data_ptr(), rows,
         two_i // 2, _stream())
    return out


def gather_rows(src: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """out[i] = src[idx[i]] for a 2-d ``src`` whose rows may be strided."""
    _gpu(src, idx)
    _i32(idx, "row indices")
    _need(src.dim() == 2 and src.stride(1) == 1, "gather_rows source must be 2-d with unit inner stride")
    n, width = idx.numel(), src.shape[1]
    out = torch.empty((n, width), dtype=src.dtype, device=src.device)
    call("tk_gather_rows", dtype_code(src.dtype), src.data_ptr(), src.stride(0), idx.data_ptr(),
         out.data_ptr(), n, width, _stream())
    return out


def rope_table(inv_freq: torch.Tensor, n_pos: int) -> tuple[torch.Tensor, torch.Tensor]:
    """cos and sin of position * inv_freq, each [n_pos, d/2] in 32-bit."""
    _gpu(inv_freq)
    _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and inv_freq.is_contiguous(),
          "inv_freq must be contiguous float32 [d/2]")
    half = inv_freq.numel()
    cos = torch.empty((n_pos, half), dtype=torch.float32, device=inv_freq.device)
    sin = torch.empty_like(cos)
    call("tk_rope_table", inv_freq.data_ptr(), cos.data_ptr(), sin.data_ptr(), n_pos, half, _stream())
    return cos, sin


def rope_append(
    qkv: torch.Tensor,
    positions: torch.Tensor,
    token_req: torch.Tensor,
    block_table: torch.Tensor | None,
    cos: torch.Tensor | None,
    sin: torch.Tensor | None,
    kcache: torch.Tensor | None,
    vcache: torch.Tensor | None,
    nq: int,
    nkv: int,
    head_dim: int,
    page_size: int,
    write_cache: bool = True,
    rotary_dim: int | None = None,
) -> None:
    """Rotate the query heads of ``qkv`` in place; rotate the key heads and store
    them and the value heads in each token's page.  ``rotary_dim`` (the whole head by
    default): the leading elements of a head that are rotated, element j with element
    j + rotary_dim / 2; the tables then have rotary_dim / 2 entries a position.

    ``kcache`` and ``vcache`` have the shapes of ``key_pages_shape`` and
    ``value_pages_shape``.  ``block_table`` is [requests, width] int32.
    """
    _gpu(qkv, positions, token_req, block_table, cos, sin, kcache, vcache)
    _need(qkv.dim() == 2 and qkv.stride(1) == 1, "qkv must be 2-d with unit inner stride")
    n = qkv.shape[0]
    _i32(positions, "positions")
    _i32(token_req, "token_req")
    _need(positions.numel() == n and token_req.numel() == n, "positions/token_req must have one entry a token")
    rot = head_dim if rotary_dim is None else int(rotary_dim)
    if not (0 <= rot <= head_dim and rot % 2 == 0):
        raise KernelError(f"rope_append: {rot} rotated elements of a head of {head_dim}")
    half = rot // 2
    if cos is not None:
        _need(sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32
              and cos.shape == sin.shape and cos.shape[1] == half and cos.is_contiguous()
              and sin.is_contiguous(), "cos/sin tables must be contiguous float32 [positions, rotary_dim/2]")
    table_stride = 0
    if write_cache:
        _need(block_table is not None and kcache is not None and vcache is not None,
              "rope_append needs the cache and the block table to write")
        _i32(block_table, "block_table")
        _need(block_table.dim() == 2, "block_table must be [requests, width]")
        table_stride = block_table.stride(0)
        _check_pages(kcache, vcache, nkv, page_size, head_dim, qkv.dtype, "rope_append")
    call(
        "tk_rope_append",
        dtype_code(qkv.dtype),
        qkv.data_ptr(),
        qkv.stride(0),
        positions.data_ptr(),
        token_req.data_ptr(),
        block_table.data_ptr() if write_cache else None,
        table_stride,
        cos.data_ptr() if cos is not None else None,
        sin.data_ptr() if sin is not None else None,
        kcache.data_ptr() if write_cache else None,
        vcache.data_ptr() if write_cache else None,
        n,
        nq,
        nkv if write_cache else 0,
        head_dim,
        rot,
        page_size,
        1 if write_cache else 0,
        _stream(),
    )


def gemm_generic(
    a: torch.Tensor,
    w: torch.Tensor,
    residual: torch.Tensor | None = None,
    out_f32: bool = False,
    out: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """a [M, K] times w [N, K] transposed (+ bias [N]) (+ residual [M, N]), 32-bit multiply-adds.
    ``out``: where the result goes (contiguous [M, N] of the result's type) instead of new memory."""
    _gpu(a, w, residual, bias)
    _check_bias(bias, w, "gemm")
    _need(a.dim() == 2 and a.stride(1) == 1, "gemm: A must be 2-d with unit inner stride")
    _need(w.dim() == 2 and w.is_contiguous(), "gemm: W must be contiguous [N, K]")
    _need(a.dtype == w.dtype, f"gemm: A is {a.dtype} but W is {w.dtype}")
    m, k = a.shape
    n = w.shape[0]
    _need(w.shape[1] == k, f"gemm: A has K={k} but W has K={w.shape[1]}")
    out_dtype = torch.float32 if out_f32 else a.dtype
    out = _result_buffer(out, m, n, out_dtype, a.device, "gemm")
    ldr = 0
    if residual is not None:
        _need(not out_f32, "gemm: a residual cannot be combined with 32-bit output")
        _need(residual.shape == (m, n) and residual.stride(1) == 1 and residual.dtype == a.dtype,
              "gemm: residual must be [M, N] of the operand type")
        ldr = residual.stride(0)
    call(
        "tk_gemm_generic",
        dtype_code(a.dtype),
        a.data_ptr(),
        a.stride(0),
        w.data_ptr(),
        out.data_ptr(),
        n,
        residual.data_ptr() if residual is not None else None,
        ldr,
        bias.data_ptr() if bias is not None else None,
        m,
        n,
        k,
        1 if out_f32 else 0,
        _stream(),
    )
    return out


def _check_bias(bias: torch.Tensor | None, w: torch.Tensor, who: str) -> None:
    _need(bias is None or (bias.shape == (w.shape[0],) and bias.dtype == w.dtype and bias.is_contiguous()),
          f"{who}: a bias must be contiguous [{w.shape[0]}] of the weight's type")


def add_bias(out: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """out[m, n] += bias[n] in place, for contiguous 32-bit ``out`` (logits behind a library product)."""
    _gpu(out, bias)
    _need(out.dim() == 2 and out.dtype == torch.float32 and out.is_contiguous(), "add_bias: out must be contiguous float32 [rows, cols]")
    _need(bias.shape == (out.shape[1],) and bias.is_contiguous() and bias.dtype in _DT, "add_bias: the bias must be contiguous [cols]")
    call("tk_add_bias", dtype_code(bias.dtype), out.data_ptr(), bias.data_ptr(), out.shape[0], out.shape[1], _stream())
    return out


def _result_buffer(out: torch.Tensor | None, m: int, n: int, dtype: torch.dtype, device: torch.device, who: str) -> torch.Tensor:
    """The caller's result buffer after a check, or new memory."""
    if out is None:
        return torch.empty((m, n), dtype=dtype, device=device)
    _gpu(out)
    if tuple(out.shape) != (m, n) or out.dtype != dtype or not out.is_contiguous() or out.device != device:
        raise KernelError(f"{who}: the result buffer must be contiguous [{m}, {n}] {dtype} on the operands' device")
    return out


def paged_attention_generic(
    q: torch.Tensor,
    kcache: torch.Tensor,
    vcache: torch.Tensor,
    block_table: torch.Tensor,
    token_req: torch.Tensor,
    positions: torch.Tensor,
    nq: int,
    nkv: int,
    head_dim: int,
    page_size: int,
    window: int = 0,
    scale: float | None = None,
    value_dim: int | None = None,
    sink: torch.Tensor | None = None,
    score_bias: torch.Tensor | None = None,
    softcap: float = 0.0,
    distance_bias: "DistanceBias | None" = None,
) -> torch.Tensor:
    """Attention of every token over its request's pages (see rope_append for
    the page layout).  ``q`` is 2-d, its first nq*d columns are the query heads.
    ``value_dim``: the size of a value head (a key head's by default); the result is
    [tokens, nq * value_dim].  ``sink`` (32-bit, one number a query head): exp(sink) joins the
    softmax's denominator once, with no key and no value.  ``score_bias`` (32-bit, one number a
    query head): no softmax; a visible key's weight is sigmoid(score + score_bias[head]), not normalised.
    ``softcap`` (> 0): a scaled score becomes softcap * tanh(score / softcap).  ``distance_bias``: a learned
    number by (bucket of the distance, head) is added to the score after that."""
    _gpu(q, kcache, vcache, block_table, token_req, positions, sink, score_bias)
    db = _checked_distance_bias(distance_bias, nq)
    vd = head_dim if value_dim is None else int(value_dim)
    _f32_vector(score_bias, nq, "attention: the scores' biases")
    _need(sink is None or (sink.shape == (nq,) and sink.dtype == torch.float32 and sink.is_contiguous()),
          f"attention: the sinks must be contiguous float32 [{nq}]")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nq * head_dim,
          "attention: q must be 2-d with unit inner stride and nq*d leading columns")
    n = q.shape[0]
    _i32(block_table, "block_table")
    _i32(token_req, "token_req")
    _i32(positions, "positions")
    _need(block_table.dim() == 2, "block_table must be [requests, width]")
    _need(positions.numel() == n and token_req.numel() == n, "positions/token_req must have one entry a token")
    _check_pages(kcache, vcache, nkv, page_size, head_dim, q.dtype, "attention", vd)
    out = torch.empty((n, nq * vd), dtype=q.dtype, device=q.device)
    call(
        "tk_paged_attention_generic",
        dtype_code(q.dtype),
        q.data_ptr(),
        q.stride(0),
        out.data_ptr(),
        out.stride(0),
        kcache.data_ptr(),
        vcache.data_ptr(),
        block_table.data_ptr(),
        block_table.stride(0),
        token_req.data_ptr(),
        positions.data_ptr(),
        n,
        nq,
        nkv,
        head_dim,
        vd,
        page_size,
        int(window),
        float(scale if scale is not None else 1.0 / math.sqrt(head_dim)),
        sink.data_ptr() if sink is not None else None,
        score_bias.data_ptr() if score_bias is not None else None,
        float(softcap), *db,
        _stream(),
    )
    return out


@dataclass
class DistanceBias:
    """A learned bias on attention scores by distance: ``rel`` [buckets, heads] (32-bit) and ``bucket_of``
    [far + 1] (int32), the bucket of every distance up to ``far``, which stands for all beyond it."""

    rel: torch.Tensor
    bucket_of: torch.Tensor


def distance_buckets(buckets: int, far: int) -> list[int]:
    """The bucket of every distance 0 .. far: distances below half the buckets have one each, the others
    share the rest on a logarithmic scale that reaches the last bucket at ``far``."""
    half = buckets // 2
    _need(buckets >= 2 and far > half, "distance_buckets: at least two buckets, and distances beyond half of them")
    out = []
    for n in range(int(far) + 1):
        if n < half:
            out.append(n)
        else:
            out.append(min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (buckets - half)))))
    return out


def _checked_distance_bias(db: "DistanceBias | None", nq: int) -> tuple:
    """The kernels' three arguments for a bias by distance (null pointers without one)."""
    if db is None:
        return None, 0, None
    _gpu(db.rel, db.bucket_of)
    _i32(db.bucket_of, "the distances' buckets")
    _need(db.rel.dim() == 2 and db.rel.shape[1] == nq and db.rel.dtype == torch.float32 and db.rel.is_contiguous(),
          f"attention: the bias by distance must be contiguous float32 [buckets, {nq}]")
    _need(db.bucket_of.numel() >= 1, "attention: the table of buckets is empty")
    return db.bucket_of.data_ptr(), db.bucket_of.numel() - 1, db.rel.data_ptr()


def paged_attention_generic_fits(nq: int, nkv: int, head_dim: int, value_dim: int | None = None) -> bool:
    """Whether the plain 32-bit attention kernel takes this many query heads a kv head at these sizes."""
    try:
        call("tk_paged_attention_generic_fits", nq, nkv, head_dim, head_dim if value_dim is None else value_dim)
    except KernelError:
        return False
    return True


def attention_mfma_supports(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    """Whether the matrix-core attention kernel takes this storage type, head size and page size."""
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 128
            and page_size >= 4 and page_size & (page_size - 1) == 0)


def check_attention_shape(dtype: torch.dtype, nq: int, nkv: int, head_dim: int, page_size: int,
                          value_dim: int | None = None, generic_only: bool = False) -> None:
    """Refuse, with the kernel's own reason, head counts and sizes that neither attention
    kernel takes for this storage type and page size.  Called when a cache is made for a
    mixer, so that a model that cannot run is refused before its first step.  ``generic_only``:
    the mixer uses what only the 32-bit-arithmetic kernel has (a value size of its own, sinks)."""
    vd = head_dim if value_dim is None else value_dim
    key_pages_shape(1, nkv, page_size, head_dim, padded=generic_only)
    value_pages_shape(1, nkv, page_size, vd)
    if generic_only or vd != head_dim or not attention_mfma_supports(dtype, head_dim, page_size):
        call("tk_paged_attention_generic_fits", nq, nkv, head_dim, vd)


ATTENTION_GROUP = 4  # wavefronts (of two neighbouring row tiles each) in a workgroup of the grouped prompt kernel
# How the prompt portions of a step are cut for the attention: paired tiles (an early and a late
# row tile a wavefront, every load the wavefront's own), or neighbouring tiles in groups of four
# wavefronts that share every load through LDS, with one set of wavefronts a group or with two that
# take the steps of the group's keys in turn.  What pays depends on how many wavefronts of two row
# tiles the portions fill (W, over all kv heads) and on how many keys the longest walk covers.
# Groups with one set need enough workgroups to fill the chip several times over, since a request's
# last groups walk far longer than its first; two sets halve the longest walk and pay where walks
# are long but groups few; paired tiles (equal walks, no barriers) where walks are short.
# The kernel alone on an MI355X, 8 kv heads of 4 query heads, pages of 16, in microseconds, paired /
# one set / two sets (prompts x tokens, "over n": after a past, n keys in all):
#   head size 64: 1 x 1 536 34 / 45 / 36; 1 x 2 048 47 / 57 / 46; 1 x 2 560 88 / 69 / 59; 1 x 4 096
#   162 / 116 / 123; 1 x 8 192 579 / 376 / 409; 2 x 1 024 29 / 38 / 36; 4 x 512 19 / 23 / 23; 8 x 512
#   33 / 36 / 37; 4 x 1 024 52 / 60 / 50; 2 x 1 536 60 / 53 / 47; 2 x 2 048 90 / 84 / 78; 32 x 256 41 /
#   39 / 47; 1 x 256 over 4 096 81 / 100 / 76; 4 x 256 over 4 096 105 / 107 / 86; 8 x 256 over 4 096
#   144 / 143 / 123; 1 x 2 048 over 8 192 209 / 225 / 198; 1 x 1 024 over 2 048 41 / 54 / 43
#   head size 128: 1 x 1 024 29 / 39 / 33; 1 x 1 536 61 / 58 / 45; 1 x 2 048 85 / 75 / 67; 1 x 4 096 - /
#   195 / 222; 8 x 256 24 / 21 / 29; 4 x 512 34 / 32 / 38; 2 x 1 024 52 / 52 / 43; 8 x 512 61 / 52 / 66;
#   2 x 256 over 4 096 125 / 131 / 100; 1 x 512 over 8 192 237 / 250 / 182; 1 x 1 024 over 2 048 58 /
#   71 / 56.  (Paired tiles of head size 128 need 333 registers: one wavefront a SIMD.)
# Prefill of one prompt, one set against paired: 1B shape 3 072 tokens 8.10 / 8.54 ms, 4 096 tokens
# 9.8 / 10.7 ms, 8 192 tokens 20.3 / 24.7 ms; 8B shape 4 096 tokens 50.2 / 53.8 ms, 8 192 tokens 110 /
# 128 ms; two sets against paired: 3B shape 2 048 tokens 13.5 / 14.4 ms, 8B shape 2 048 tokens 27.4 /
# 28.4 ms.
ATTENTION_GROUPED_FROM = 3072  # wavefronts from which long prompts take groups with one set


def attention_group_sets(wavefronts: int, head_dim: int, page_size: int, longest: int) -> int:
    """How the prompt portions of a step run that fill ``wavefronts`` wavefronts of two row tiles
    (over all kv heads), the longest of their requests having ``longest`` keys: 0 paired tiles, 1
    groups of tiles that share their loads, 2 such groups with their steps dealt out to two sets
    of wavefronts.  (A window is not looked at: it shortens the walks of some layers only, and
    the plan is the same for all.)"""
    if page_size < 16:
        return 0  # a 16-key block of a step would span pages
    walk = -(-longest // 32)  # steps of 32 keys of the longest walk
    if head_dim <= 64:
        if wavefronts >= ATTENTION_GROUPED_FROM and walk >= 96:
            return 1
        if (walk >= 128 and wavefronts >= 256) or (walk >= 64 and wavefronts >= 2048) or (walk >= 32 and wavefronts >= 3072):
            return 2
        return 0
    if wavefronts >= ATTENTION_GROUPED_FROM:
        return 1
    if walk >= 128 and wavefronts >= 256:
        return 2
    if wavefronts >= 1280:
        return 2 if walk >= 32 else 1
    return 2 if walk >= 64 and wavefronts >= 512 else 0


def attention_prompt_split(wavefronts: int, head_dim: int, longest: int) -> int:
    """Keys a split for prompt portions (paired tiles) that fill few wavefronts but walk many keys, 0
    for whole keys.  A wavefront of paired tiles walks every key its rows see, one step of 32 after
    the other: a 64-token portion after 32 768 keys is 64 such walks of a millisecond each, a layer,
    on a chip that has room for 2 048 (1 024 at head sizes above 64, where a wavefront needs more
    than half of a SIMD's registers).  The keys are cut so that the walks fill that room, at 64
    splits at most and 512 keys a split at least, and a second kernel adds the splits' results.
    Measured on an MI355X (1B shape, a layer, whole keys / best of the grouped forms / cut):
    64 tokens after 32 768 keys 992 / - / 57 us, 16 tokens 993 / - / 41, 8 tokens after 131 072 keys
    3 990 / - / 93, 256 tokens after 4 096 keys 81 / 75 / 38, 512 after 8 192 156 / 142 / 86, 1 024 after
    32 768 771 / 613 / 465; at twice the room's wavefronts nothing is gained (1 024 tokens after 8 192
    keys 157 / 146 / 148, 4 x 256 after 4 096 102 / 86 / 94), so two splits are taken for long walks
    only; head size 128: 512 tokens after 8 192 keys 241 / 183 / 147, 2 x 256 after 4 096 121 / 99 / 88."""
    room = 2048 if head_dim <= 64 else 1024
    splits = min(64, room // max(wavefronts, 1))
    if longest < 2048 or splits < 2 or (splits < 4 and head_dim <= 64 and longest < 512 * 32):
        return 0  # (under 2 048 keys the second kernel costs what the shorter walks save)
    split = max(512, -(-(-(-longest // splits)) // 128) * 128)
    return split if split < longest else 0


def attention_tiles(
    q_lens: list[int], group: int, row_tiles: int, requests: list[int] | None = None, pair: bool = False, fill: int = 1
) -> tuple[list[int], list[int], list[int] | None]:
    """The row tiles that cover the (token, head of the group) pairs of ``requests``
    (all by default), ``row_tiles`` tiles of 16 rows a wavefront: (request, first row of
    the first tile, first row of the second tile or -1).  With ``pair`` a request's
    i-th tile shares a wavefront with its i-th last, which evens out the keys a
    wavefront walks under a causal mask; otherwise with its neighbour, and the
    third list is None.  ``fill`` > 1 (two row tiles, no pairs; for the grouped kernel): a
    request's tiles come last rows first (those that see most keys start first) and are filled
    up to a multiple of ``fill`` with empty ones (first row -1), so that a group of ``fill``
    never spans two requests."""
    tile_req: list[int] = []
    tile_row0: list[int] = []
    tile_row1: list[int] = []
    for r in (range(len(q_lens)) if requests is None else requests):
        n = -(-q_lens[r] * group // 16)  # row tiles of the request
        if row_tiles == 1:
            firsts = [(i, -1) for i in range(n)]
        elif pair:
            firsts = [(i, n - 1 - i if n - 1 - i > i else -1) for i in range((n + 1) // 2)]
        else:
            firsts = [(i, i + 1 if i + 1 < n else -1) for i in range(0, n, 2)]
        if fill > 1 and row_tiles == 2 and not pair:
            firsts = firsts[::-1] + [(-1, -1)] * (-len(firsts) % fill)
        for i, j in firsts:
            tile_req.append(r)
            tile_row0.append(16 * i if i >= 0 else -1)
            tile_row1.append(16 * j if j >= 0 else -1)
    return tile_req, tile_row0, (tile_row1 if pair and row_tiles == 2 else None)


def attention_max_waves(head_dim: int, row_tiles: int) -> int:
    """Wavefronts a workgroup of the matrix-core attention may have."""
    return 4 if row_tiles == 2 else (16 if head_dim <= 64 else 8)


def attention_split(max_kv_len: int, n_tiles: int, nkv: int, head_dim: int = 64) -> tuple[int, int]:
    """(keys per split, wavefronts per workgroup) for tiles of one row tile (decode).
    The keys of a tile are cut so that there are about 256 workgroups (one a compute
    unit) or more, into splits of 8 192 keys at most; the wavefronts of a workgroup, which
    adds their results itself, take 64 to 512 keys each, about two thousand wavefronts in all
    or more.
    Measured best on an MI355X at 8192 keys, with the cache read from memory:
    64 keys x 8 wavefronts x 16 splits at batch 1, 256 x 8 x 4 at batch 8,
    512 x 16 x 1 at batch 64."""
    base = max(n_tiles * nkv, 1)
    kv = max(max_kv_len, 1)
    splits = max(1, min(16, -(-256 // base)))
    # at most 8 192 keys a split (2 048 with a thousand tiles and more), however many tiles there are: the bound
    # is that of the longest request, and one long request among short ones must still spread over the chip
    # (63 requests of 2 048 keys beside one of 131 072: 881 us a layer with one split a tile, 168 us with splits of
    # 8 192 keys; 255 of 512 beside one of 32 768: 401 / 114 us; requests of one length lose nothing)
    raw = min(-(-kv // splits), 8192 if base < 1024 else 2048)
    per_wave = min(512, max(64, kv * base // 2048))
    waves = 1
    while waves * 2 <= min(attention_max_waves(head_dim, 1), raw // per_wave):
        waves *= 2
    step = 32 * waves
    return -(-raw // step) * step, waves


# Whether the splits of decoded tokens' tiles are added inside the attention kernel, by the
# workgroup that arrives last at a tile, instead of by a second kernel.
ATTENTION_MERGE_IN_KERNEL = True


class AttentionScratch:
    """Memory for the partial results of split tiles, and the tickets at which the splits of a
    tile of decoded tokens count themselves in (all zero between launches: the kernel leaves them
    so).  The buffers grow on demand and are shared by the launches of one stream, which run one
    after the other."""

    _shared: dict = {}

    def __init__(self, device: torch.device):
        self.device = device
        self.part_o = torch.empty((0,), dtype=torch.float32, device=device)
        self.part_ml = torch.empty((0,), dtype=torch.float32, device=device)
        self.tickets = torch.zeros((0,), dtype=torch.int32, device=device)

    @classmethod
    def shared(cls, device: torch.device) -> "AttentionScratch":
        key = (device.type, device.index)
        if key not in cls._shared:
            cls._shared[key] = cls(device)
        return cls._shared[key]

    def take(self, n_o: int, n_ml: int, n_tickets: int = 0):
        if self.part_o.numel() < n_o:
            self.part_o = torch.empty((n_o,), dtype=torch.float32, device=self.device)
        if self.part_ml.numel() < n_ml:
            self.part_ml = torch.empty((n_ml,), dtype=torch.float32, device=self.device)
        if self.tickets.numel() < n_tickets:
            if torch.cuda.is_current_stream_capturing():
                raise KernelError("attention scratch: the tickets must exist before a step is recorded")
            self.tickets = torch.zeros((n_tickets,), dtype=torch.int32, device=self.device)
        return self.part_o, self.part_ml


def paged_attention_mfma(
    q: torch.Tensor,
    kcache: torch.Tensor,
    vcache: torch.Tensor,
    block_table: torch.Tensor,
    q_start: torch.Tensor,
    kv_len: torch.Tensor,
    tile_req: torch.Tensor,
    tile_row0: torch.Tensor,
    row_tiles: int,
    nq: int,
    nkv: int,
    head_dim: int,
    page_size: int,
    max_kv_len: int,
    split: int,
    window: int = 0,
    scale: float | None = None,
    waves: int = 1,
    out: torch.Tensor | None = None,
    scratch: "AttentionScratch | None" = None,
    tile_row1: torch.Tensor | None = None,
    longest: int | None = None,
    grouped: bool | int = False,
    merge_kernel: bool = False,
) -> torch.Tensor:
    """Attention of every token of the batch over its request's pages on the
    matrix cores (bfloat16).  ``q`` is 2-d and its first nq*d columns are the
    query heads; request r owns tokens q_start[r]..q_start[r+1]-1, the last of
    them at position kv_len[r]-1.  ``max_kv_len`` bounds kv_len (it sizes the
    grid and the scratch, so it may be larger than any request's; ``longest``, if
    given, is the length of the longest request, which the block table must cover).  The tiles
    (see ``attention_tiles``) may cover some of the requests only; rows of ``out``
    that no tile covers are left as they are.

    ``grouped`` (long prompts: two neighbouring row tiles a wavefront, pages of 16 keys or more,
    whole keys): the tiles were made with ``fill=ATTENTION_GROUP``; a workgroup takes a group of
    them and loads the request's keys and values once for all.  As the number 2: two sets of
    wavefronts take the steps over a group's keys in turn (see ``attention_group_sets``).

    The splits of a tile of one row tile (decoded tokens) are added inside the kernel by the
    workgroup that arrives last; ``merge_kernel`` has a second kernel add them instead, as for
    tiles of two row tiles."""
    _gpu(q, kcache, vcache, block_table, q_start, kv_len, tile_req, tile_row0)
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nq * head_dim and q.dtype == torch.bfloat16,
          "attention_mfma: q must be bfloat16, 2-d with unit inner stride and nq*d leading columns")
    n = q.shape[0]
    for t, name in ((block_table, "block_table"), (q_start, "q_start"), (kv_len, "kv_len"),
                    (tile_req, "tile_req"), (tile_row0, "tile_row0")):
        _i32(t, name)
    _need(block_table.dim() == 2, "block_table must be [requests, width]")
    requests = kv_len.numel()
    _need(q_start.numel() == requests + 1 and block_table.shape[0] >= requests,
          "attention_mfma: q_start, kv_len and block_table disagree on the number of requests")
    _need(block_table.shape[1] * page_size >= (max_kv_len if longest is None else longest) or requests == 0,
          "attention_mfma: block table narrower than the longest request")
    _need(longest is None or longest <= max_kv_len, "attention_mfma: the longest request exceeds max_kv_len")
    n_tiles = tile_req.numel()
    _need(tile_row0.numel() == n_tiles, "attention_mfma: tile lists differ in length")
    if tile_row1 is not None:
        _gpu(tile_row1)
        _i32(tile_row1, "tile_row1")
        _need(tile_row1.numel() == n_tiles and row_tiles == 2, "attention_mfma: second row tiles need row_tiles == 2 and one entry a tile")
    _check_pages(kcache, vcache, nkv, page_size, head_dim, torch.bfloat16, "attention_mfma")
    if not attention_mfma_supports(q.dtype, head_dim, page_size):
        raise KernelError(f"attention_mfma: head size {head_dim} / page size {page_size} not supported")
    _need(split > 0 and split % 32 == 0, "attention_mfma: split must be a positive multiple of 32")
    _need(1 <= waves <= attention_max_waves(head_dim, row_tiles) and split % (32 * waves) == 0,
          "attention_mfma: the wavefronts of a workgroup (at most 16; 8 with a head size above 64; 4 with two row tiles) "
          "must cut a split into multiples of 32 keys")
    if out is None:
        out = torch.empty((n, nq * head_dim), dtype=q.dtype, device=q.device)
    else:
        _need(out.shape == (n, nq * head_dim) and out.dtype == q.dtype and out.stride(1) == 1, "attention_mfma: bad out")
    max_splits = max(1, -(-max_kv_len // split))
    _need(not grouped or (row_tiles == 2 and page_size >= 16 and waves == 1 and max_splits == 1 and n_tiles % ATTENTION_GROUP == 0),
          "attention_mfma: grouped tiles are prompts' (two row tiles, filled groups) on pages of 16 keys or more, unsplit")
    if int(grouped) not in (0, 1, 2):
        raise KernelError(f"attention_mfma: {int(grouped)} sets of wavefronts a group (1 or 2)")
    part_o = part_ml = tickets = None
    if max_splits > 1:
        items = n_tiles * nkv * max_splits * 16 * row_tiles
        if scratch is None:
            scratch = AttentionScratch.shared(q.device)
        in_kernel = row_tiles == 1 and not merge_kernel and ATTENTION_MERGE_IN_KERNEL
        part_o, part_ml = scratch.take(items * head_dim, items * 2, n_tiles * nkv if in_kernel else 0)
        tickets = scratch.tickets if in_kernel else None
    call(
        "tk_paged_attention_mfma",
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0),
        kcache.data_ptr(), vcache.data_ptr(), block_table.data_ptr(), block_table.stride(0),
        q_start.data_ptr(), kv_len.data_ptr(), tile_req.data_ptr(), tile_row0.data_ptr(),
        tile_row1.data_ptr() if tile_row1 is not None else None,
        n_tiles, row_tiles, nq, nkv, head_dim, page_size, int(window),
        float(scale if scale is not None else 1.0 / math.sqrt(head_dim)),
        split, waves, max_splits, max_splits,
        part_o.data_ptr() if part_o is not None else None,
        part_ml.data_ptr() if part_ml is not None else None,
        tickets.data_ptr() if tickets is not None else None,
        int(grouped),
        _stream(),
    )
    return out


def sample(
    logits: torch.Tensor,
    temperature: torch.Tensor,
    uniform: torch.Tensor,
    slots: torch.Tensor | None = None,
    last_token: torch.Tensor | None = None,
    want_logprobs: bool = True,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Token ids (int32) and their log-probabilities for each row of ``logits``."""
    _gpu(logits, temperature, uniform, slots, last_token)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1,
          "sample: logits must be float32 [rows, vocab]")
    rows, vocab = logits.shape
    for t, name in ((temperature, "temperature"), (uniform, "uniform")):
        _need(t.dtype == torch.float32 and t.numel() == rows and t.is_contiguous(),
              f"sample: {name} must be float32 [rows]")
    if slots is not None or last_token is not None:
        _need(slots is not None and last_token is not None, "sample: slots and last_token go together")
        _i32(slots, "slots")
        _i32(last_token, "last_token")
        _need(slots.numel() == rows, "sample: one slot a row")
    ids = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    logprobs = torch.empty((rows,), dtype=torch.float32, device=logits.device) if want_logprobs else None
    chunks = load("core").tk_sample_chunks(vocab)
    part = torch.empty((3, max(rows, 1) * chunks), dtype=torch.float32, device=logits.device)
    call(
        "tk_sample",
        logits.data_ptr(),
        logits.stride(0) if rows > 0 else vocab,
        rows,
        vocab,
        temperature.data_ptr(),
        uniform.data_ptr(),
        slots.data_ptr() if slots is not None else None,
        last_token.data_ptr() if last_token is not None else None,
        ids.data_ptr(),
        logprobs.data_ptr() if logprobs is not None else None,
        part[0].data_ptr(),
        part[1].data_ptr(),
        part[2].data_ptr(),
        _stream(),
    )
    return ids, logprobs


TOPK_MAX = 32  # places the top-k kernel ranks (TOPK_MAX of sample.hip)


def topk_logprobs(logits: torch.Tensor, temperature: torch.Tensor, k: int) -> tuple[torch.Tensor, torch.Tensor]:
    """The ``k`` most probable tokens of every row (int32 [rows, k]) and their
    log-probabilities under softmax(logits / T) (float32 [rows, k]; T 0 counts as 1),
    most probable first, the lower index first among equal logits."""
    _gpu(logits, temperature)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1,
          "topk_logprobs: logits must be float32 [rows, vocab]")
    rows, vocab = logits.shape
    _need(temperature.dtype == torch.float32 and temperature.numel() == rows and temperature.is_contiguous(),
          "topk_logprobs: temperature must be float32 [rows]")
    _need(1 <= k <= min(TOPK_MAX, vocab), f"topk_logprobs: k={k} is not between 1 and {min(TOPK_MAX, vocab)}")
    ids = torch.empty((rows, k), dtype=torch.int32, device=logits.device)
    logprobs = torch.empty((rows, k), dtype=torch.float32, device=logits.device)
    chunks = load("core").tk_sample_chunks(vocab)
    n = max(rows, 1) * chunks
    part = torch.empty((2 * n * k + 2 * n,), dtype=torch.float32, device=logits.device)
    call(
        "tk_topk_logprobs",
        logits.data_ptr(),
        logits.stride(0) if rows > 0 else vocab,
        rows,
        vocab,
        temperature.data_ptr(),
        k,
        ids.data_ptr(),
        logprobs.data_ptr(),
        part[: n * k].data_ptr(),
        part[n * k : 2 * n * k].data_ptr(),
        part[2 * n * k : 2 * n * k + n].data_ptr(),
        part[2 * n * k + n :].data_ptr(),
        _stream(),
    )
    return ids, logprobs


# --------------------------------------------------------------------------
# bfloat16 matrix products on the matrix cores
# --------------------------------------------------------------------------

EPI_STORE, EPI_RESIDUAL, EPI_SWIGLU, EPI_F32, EPI_ROPE = 0, 1, 2, 3, 4
SKINNY_MAX_ROWS = 128  # rows the weight-streaming kernel takes
# Rows up to which it is the faster product.  Measured on an MI355X for the layer shapes of a
# 1B model, whole recorded decode steps at a context of 1,024: at 8 and 16 rows 19 and 11 %
# faster than the library product followed by the kernels it fuses away (rotation and append,
# SwiGLU, norms); at 24 and 32 rows 12 % slower, at 64 rows a third.  At the wider 3B and 8B
# shapes it is ahead up to 8 rows (at one row by 21 %, at 8 rows by 10 %) and level with the
# library at 16.
SKINNY_ROWS = 16
# Per product the crossing lies where the rows of A that every workgroup reads (rows x inner size,
# twice that where two weight tiles meet in the epilogue) reach about 80 000 elements: every
# workgroup reads all of A from the caches, which beyond that costs more than the kernels the
# epilogue saves.  Measured on an MI355X, one product at a time with the weights coming from
# memory, library product and epilogue kernels against the fused kernel: output projection
# (inner size 2 048) 11.4 / 6.5 us at 8 rows, 11.7 / 9.6 at 32, 11.7 / 12.9 at 48; down projection
# (8 192) 16.1 / 14.9 at 8 rows, 16.2 / 16.6 at 12, 16.4 / 18.4 at 16; gate and up (2 048, paired)
# 19.8 / 18.4 at 16 rows, 19.8 / 20.7 at 20.  The head keeps SKINNY_ROWS.
SKINNY_A_ELEMENTS = 80_000


def skinny_rows(inner: int, paired: bool = False) -> int:
    """Rows up to which the weight-streaming product is taken for a weight of this inner size."""
    return max(1, min(SKINNY_MAX_ROWS, SKINNY_A_ELEMENTS // (inner * (2 if paired else 1))))
# The stacked q, k, v product with rotation and append in its epilogue replaces two kernels of
# the library path and has a short inner size: it stays ahead up to 32 rows (4 % of a step) at an
# inner size of 2 048, and up to twice the rows of an ordinary paired product at wider ones.
SKINNY_ROPE_ROWS = 32


class _GemmExtra(ctypes.Structure):
    """The optional operands of tk_gemm_skinny_bf16 (struct GemmExtra of gemm_mfma.hip)."""

    _fields_ = [
        ("sumsq_in", ctypes.c_void_p), ("parts_in", ctypes.c_int), ("eps", ctypes.c_float),
        ("emit_w", ctypes.c_void_p), ("emit_w_f32", ctypes.c_int), ("emit_scaled", ctypes.c_void_p),
        ("ld_emit", ctypes.c_int), ("emit_sumsq", ctypes.c_void_p), ("parts_out", ctypes.c_int),
        ("positions", ctypes.c_void_p), ("token_req", ctypes.c_void_p), ("block_table", ctypes.c_void_p),
        ("table_stride", ctypes.c_int), ("cos_t", ctypes.c_void_p), ("sin_t", ctypes.c_void_p),
        ("kcache", ctypes.c_void_p), ("vcache", ctypes.c_void_p),
        ("nq", ctypes.c_int), ("nkv", ctypes.c_int), ("d", ctypes.c_int), ("P", ctypes.c_int),
        ("bias", ctypes.c_void_p), ("glu_limit", ctypes.c_float), ("glu_alpha", ctypes.c_float),
        ("out_scale", ctypes.c_float), ("glu_gelu", ctypes.c_int),
    ]


@dataclass
class Prenorm:
    """What a residual product leaves for the RMSNorm that follows it: the new rows
    times the norm's weight (rounded once) and, per row, partial sums of squares."""

    scaled: torch.Tensor  # [M, N] bfloat16
    sumsq: torch.Tensor  # [M, parts] float32


@dataclass
class RopeAppend:
    """Operands of the rotation-with-append epilogue (see rope_append)."""

    positions: torch.Tensor
    token_req: torch.Tensor
    block_table: torch.Tensor
    cos: torch.Tensor | None
    sin: torch.Tensor | None
    kcache: torch.Tensor
    vcache: torch.Tensor
    nq: int
    nkv: int
    head_dim: int
    page_size: int
    rotary_dim: int | None = None  # leading elements of a head that are rotated (None: the whole head)


def gemm_skinny_bf16(
    a: torch.Tensor,
    w: torch.Tensor,
    residual: torch.Tensor | None = None,
    out_f32: bool = False,
    swiglu: bool = False,
    prenorm: Prenorm | None = None,
    norm_eps: float = 0.0,
    emit_weight: torch.Tensor | None = None,
    rope: RopeAppend | None = None,
    waves_k: int = 0,
    tiles: int = 0,
    staged: int = -1,
    tile_rows: int = 0,
    out: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
    fold: bool = True,
    glu: tuple[float, float] | None = None,
    out_scale: float | None = None,
):
    """a [M <= 128, K] times w [N, K] transposed on the matrix cores, with the
    epilogue fused: + residual, 32-bit output, (``swiglu``: w is [gate | up]
    stacked, 2I rows) silu(gate) * up -> [M, I], or (``rope``: w is [q | k | v]
    stacked) rotation of q and k with the append of k and v to the pages -> q [M, nq*d].

    ``prenorm``: the product of RMSNorm(x): ``a`` must be ``prenorm.scaled`` and the
    rows are divided by their rms (``norm_eps``) in the epilogue.  ``emit_weight``
    (with ``residual``): the weight of the norm that follows; returns
    ``(out, Prenorm)`` for it.  ``out``: where the result goes instead of new memory.
    ``bias`` (one value a row of ``w``): added to the product before the epilogue.
    ``glu`` (with ``swiglu``): (limit, alpha); the gated epilogue is then min(gate, limit) *
    sigmoid(alpha * min(gate, limit)) * (clamp(up, -limit, limit) + 1).
    ``out_scale`` (with ``out_f32``): the 32-bit result is multiplied by it.
    ``waves_k``, ``tiles``, ``staged``, ``tile_rows``, ``fold``: the kernel's own choices overridden (for measurements)."""
    _gpu(a, w, residual, emit_weight, bias)
    _check_bias(bias, w, "gemm_skinny")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.dtype == torch.bfloat16, "gemm_skinny: A must be bfloat16 [M, K]")
    _need(w.dim() == 2 and w.is_contiguous() and w.dtype == torch.bfloat16, "gemm_skinny: W must be contiguous bfloat16 [N, K]")
    m, k = a.shape
    _need(w.shape[1] == k, f"gemm_skinny: A has K={k}, W has K={w.shape[1]}")
    n = w.shape[0]
    n_out = n
    extra = _GemmExtra()
    use_extra = False
    if swiglu:
        _need(residual is None and not out_f32 and rope is None and n % 2 == 0,
              "gemm_skinny: SwiGLU takes a [2I, K] weight, no residual, bfloat16 output")
        n //= 2
        n_out = n
        epi = EPI_SWIGLU
        if glu == "gelu_tanh":  # gelu(gate) * up
            extra.glu_gelu = 1
            use_extra = True
        elif glu is not None:
            _need(glu[0] > 0, "gemm_skinny: the clamp's limit must be positive")
            extra.glu_limit, extra.glu_alpha = float(glu[0]), float(glu[1])
            use_extra = True
    elif rope is not None:
        _need(residual is None and not out_f32, "gemm_skinny: the rotation epilogue stands alone")
        epi = EPI_ROPE
        r = rope
        _gpu(r.positions, r.token_req, r.block_table, r.cos, r.sin, r.kcache, r.vcache)
        _need(n == (r.nq + 2 * r.nkv) * r.head_dim, "gemm_skinny: W is not [q | k | v] of these head counts")
        _need(r.rotary_dim is None or r.rotary_dim == r.head_dim,
              "gemm_skinny: the rotation epilogue rotates whole heads (rope_append rotates a part)")
        for t, name in ((r.positions, "positions"), (r.token_req, "token_req"), (r.block_table, "block_table")):
            _i32(t, name)
        _need(r.positions.numel() == m and r.token_req.numel() == m and r.block_table.dim() == 2,
              "gemm_skinny: positions/token_req need one entry a row, block_table [requests, width]")
        _check_pages(r.kcache, r.vcache, r.nkv, r.page_size, r.head_dim, torch.bfloat16, "gemm_skinny")
        if r.cos is not None:
            half = r.head_dim // 2
            _need(r.sin is not None and r.cos.dtype == torch.float32 and r.sin.dtype == torch.float32
                  and r.cos.shape == r.sin.shape and r.cos.shape[1] == half and r.cos.is_contiguous() and r.sin.is_contiguous(),
                  "gemm_skinny: cos/sin tables must be contiguous float32 [positions, d/2]")
        extra.positions, extra.token_req = r.positions.data_ptr(), r.token_req.data_ptr()
        extra.block_table, extra.table_stride = r.block_table.data_ptr(), r.block_table.stride(0)
        extra.cos_t = r.cos.data_ptr() if r.cos is not None else None
        extra.sin_t = r.sin.data_ptr() if r.sin is not None else None
        extra.kcache, extra.vcache = r.kcache.data_ptr(), r.vcache.data_ptr()
        extra.nq, extra.nkv, extra.d, extra.P = r.nq, r.nkv, r.head_dim, r.page_size
        use_extra = True
        n_out = r.nq * r.head_dim
    elif residual is not None:
        _need(not out_f32, "gemm_skinny: a residual cannot be combined with 32-bit output")
        _need(residual.shape == (m, n) and residual.stride(1) == 1 and residual.dtype == torch.bfloat16,
              "gemm_skinny: residual must be bfloat16 [M, N]")
        epi = EPI_RESIDUAL
    else:
        epi = EPI_F32 if out_f32 else EPI_STORE
    if bias is not None:
        extra.bias = bias.data_ptr()
        use_extra = True
    if out_scale is not None and float(out_scale) != 1.0:
        _need(epi == EPI_F32 and float(out_scale) != 0.0, "gemm_skinny: a factor on the result goes with 32-bit output and is not 0")
        extra.out_scale = float(out_scale)
        use_extra = True
    if prenorm is not None:
        _gpu(prenorm.scaled, prenorm.sumsq)
        _need(residual is None, "gemm_skinny: a norm in front cannot be combined with a residual behind")
        _need(prenorm.scaled.data_ptr() == a.data_ptr() and prenorm.sumsq.dtype == torch.float32
              and prenorm.sumsq.dim() == 2 and prenorm.sumsq.shape[0] == m and prenorm.sumsq.is_contiguous(),
              "gemm_skinny: a norm in front takes the producer's scaled rows as A and its partial sums [M, parts]")
        extra.sumsq_in, extra.parts_in, extra.eps = prenorm.sumsq.data_ptr(), prenorm.sumsq.shape[1], float(norm_eps)
        use_extra = True
    emitted = None
    if emit_weight is not None:
        _need(epi == EPI_RESIDUAL, "gemm_skinny: outputs for a following norm go with the residual epilogue")
        _need(emit_weight.shape == (n,) and emit_weight.is_contiguous() and emit_weight.dtype in (torch.bfloat16, torch.float32),
              "gemm_skinny: the following norm's weight must be contiguous [N], bfloat16 or float32")
        parts = load("mfma").tk_gemm_skinny_parts(m, n, tile_rows)
        emitted = Prenorm(torch.empty((m, n), dtype=torch.bfloat16, device=a.device),
                          torch.empty((m, parts), dtype=torch.float32, device=a.device))
        extra.emit_w, extra.emit_w_f32 = emit_weight.data_ptr(), 1 if emit_weight.dtype == torch.float32 else 0
        extra.emit_scaled, extra.ld_emit = emitted.scaled.data_ptr(), n
        extra.emit_sumsq, extra.parts_out = emitted.sumsq.data_ptr(), parts
        staged = 0  # only the skinny kernel has this epilogue
        use_extra = True
    out = _result_buffer(out, m, n_out, torch.float32 if out_f32 else torch.bfloat16, a.device, "gemm_skinny")
    call(
        "tk_gemm_skinny_bf16",
        a.data_ptr(), a.stride(0), w.data_ptr(), out.data_ptr(), n_out,
        residual.data_ptr() if residual is not None else None,
        residual.stride(0) if residual is not None else 0,
        ctypes.byref(extra) if use_extra else None,
        m, n, k, epi, waves_k, tiles, staged, tile_rows, 1 if fold else 0, _stream(),
    )
    return (out, emitted) if emit_weight is not None else out


def add(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """x + y, each rounded operand added in 32-bit and rounded once."""
    _gpu(x, y)
    _need(x.shape == y.shape and x.dtype == y.dtype and x.is_contiguous() and y.is_contiguous(),
          "add: operands must be contiguous and alike")
    out = torch.empty_like(x)
    call("tk_add", dtype_code(x.dtype), x.data_ptr(), y.data_ptr(), out.data_ptr(), x.numel(), _stream())
    return out


# What the product library's kernels may use for partial sums: its stream-K kernels want up to 64 MB
# (one 256 x 256 tile of 32-bit sums a compute unit); the tensor library gives its products 76 MB too.
LIBRARY_WORKSPACE_BYTES = 76 << 20
_library_workspace: dict[int, torch.Tensor] = {}


def library_workspace() -> torch.Tensor:
    """The current device's workspace for library products: made at the first call (a runner
    makes it before it records steps, so that no recording allocates it) and kept."""
    device = torch._C._cuda_getDevice()
    ws = _library_workspace.get(device)
    if ws is None:
        ws = _library_workspace[device] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=f"cuda:{device}")
    return ws


def gemm_library_direct(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether ``gemm_library_bf16`` is asked for this product: rows of x, w and the result
    that start at multiples of 16 bytes, for which the library has its kernels for certain.
    Other sizes go to the library through the tensor library's product, which knows its way
    round what is missing."""
    return (w.shape[0] % 8 == 0 and w.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def gemm_library_bf16(x: torch.Tensor, w: torch.Tensor, out_f32: bool = False, out: torch.Tensor | None = None) -> torch.Tensor:
    """x [M, K] . w [N, K]^T by the matrix product library (hipBLASLt), bfloat16 operands,
    32-bit accumulation, the result in bfloat16 or (``out_f32``) in 32-bit: the product for
    more rows than the weight-streaming kernel takes, called without the tensor library's
    dispatcher between (the same kernel, half the host's time a call).  ``out``: a buffer
    [M, N] for the result."""
    _gpu(x, w, out)
    if not (x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1] and x.dtype == w.dtype == torch.bfloat16):
        raise KernelError(f"gemm_library: x {tuple(x.shape)} {x.dtype} and w {tuple(w.shape)} {w.dtype} must be bfloat16 [M, K] and [N, K]")
    _need(x.stride(1) == 1 and w.stride(1) == 1 and x.shape[0] > 0 and x.device == w.device, "gemm_library: rows must be contiguous, on one device")
    m, k = x.shape
    n = w.shape[0]
    out = _result_buffer(out, m, n, torch.float32 if out_f32 else torch.bfloat16, x.device, "gemm_library")
    ws = library_workspace()
    call("tk_gemm_library_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
         m, n, k, 1 if out_f32 else 0, ws.data_ptr(), ws.numel(), _stream())
    return out


# --------------------------------------------------------------------------
# a recorded step's traffic with the host
# --------------------------------------------------------------------------


def _pinned_i32(t: torch.Tensor, name: str) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous() and not t.is_cuda and t.is_pinned(),
          f"{name} must be contiguous int32 in pinned host memory")


def stage_step(host_ring: torch.Tensor, counter: torch.Tensor, dev: torch.Tensor) -> None:
    """dev[:] = host_ring[counter % ring]: the step's small arrays from the slot of a ring in
    pinned host memory [ring, words] that its run number names, copied by a kernel of the step."""
    _gpu(counter, dev)
    _pinned_i32(host_ring, "stage_step: the ring")
    _i32(counter, "counter")
    _i32(dev, "the step's buffer")
    _need(host_ring.dim() == 2 and host_ring.shape[1] == dev.numel() and dev.numel() % 4 == 0 and counter.numel() == 1,
          "stage_step: the ring must be [ring, words] with words that of the device buffer, a multiple of 4")
    call("tk_stage_step", host_ring.data_ptr(), counter.data_ptr(), dev.data_ptr(), dev.numel(), host_ring.shape[0], _stream())


def publish_words(rows: int, k: int) -> int:
    """32-bit words of an output slot for ``rows`` sampled rows with ``k`` ranked tokens each."""
    return 1 + (2 + 2 * k) * rows


def publish_step(host_ring: torch.Tensor, counter: torch.Tensor, ids: torch.Tensor, logprobs: torch.Tensor | None,
                 topk_ids: torch.Tensor | None = None, topk_logprobs: torch.Tensor | None = None) -> None:
    """What a step sampled, written by a kernel of the step into slot (counter % ring) of a ring in
    pinned host memory [ring, slot words]: [run number + 1][ids][log-probabilities][ranked ids]
    [their log-probabilities]; the first word is written last.  Adds one to the counter."""
    _gpu(counter, ids, logprobs, topk_ids, topk_logprobs)
    _pinned_i32(host_ring, "publish_step: the ring")
    _i32(counter, "counter")
    _i32(ids, "ids")
    rows = ids.numel()
    _need(host_ring.dim() == 2 and counter.numel() == 1 and rows > 0, "publish_step: the ring must be [ring, slot words]")
    _need(logprobs is None or (logprobs.dtype == torch.float32 and logprobs.numel() == rows and logprobs.is_contiguous()),
          "publish_step: log-probabilities must be float32, one a row")
    k = 0
    if topk_ids is not None:
        _i32(topk_ids, "ranked ids")
        _need(topk_logprobs is not None and topk_ids.dim() == 2 and topk_ids.shape[0] == rows and topk_logprobs.shape == topk_ids.shape
              and topk_logprobs.dtype == torch.float32 and topk_logprobs.is_contiguous(), "publish_step: ranked tokens must be [rows, k]")
        k = topk_ids.shape[1]
    _need(host_ring.shape[1] >= publish_words(rows, k), "publish_step: the ring's slots are too short")
    call("tk_publish_step", host_ring.data_ptr(), counter.data_ptr(), host_ring.shape[0], host_ring.shape[1], ids.data_ptr(),
         logprobs.data_ptr() if logprobs is not None else None, rows,
         topk_ids.data_ptr() if k else None, topk_logprobs.data_ptr() if k else None, k, _stream())


# --------------------------------------------------------------------------
# a residual stream kept in 32-bit
# --------------------------------------------------------------------------

def _f32_vector(t: torch.Tensor | None, n: int, name: str) -> None:
    if t is not None and (t.shape != (n,) or t.dtype != torch.float32 or not t.is_contiguous()):
        raise KernelError(f"{name} must be contiguous float32 [{n}]")


def embed_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float, last_token: torch.Tensor | None = None,
                 pos_table: torch.Tensor | None = None, positions: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = float32(table[ids[t]]) * scale: the first rows of a 32-bit residual stream;
    ids[t] < 0 reads the token from last_token[-ids[t]-1].  ``pos_table`` [positions, H] of the table's type:
    the row of the token's position (``positions``) is added, as it is."""
    _gpu(ids, table, last_token, pos_table, positions)
    if pos_table is not None:
        _need(pos_table.dim() == 2 and pos_table.is_contiguous() and pos_table.shape[1] == table.shape[1] and pos_table.dtype == table.dtype,
              "embed_scaled: the table of positions must be contiguous [positions, H] of the embedding's type")
        _i32(positions, "positions")
        _need(positions.numel() == ids.numel(), "embed_scaled: one position a token")
    _i32(ids, "ids")
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [V, H]")
    if last_token is not None:
        _i32(last_token, "last_token")
    n = ids.numel()
    vocab, hidden = table.shape
    out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
    call("tk_embed_scaled", dtype_code(table.dtype), ids.data_ptr(), last_token.data_ptr() if last_token is not None else None,
         table.data_ptr(), out.data_ptr(), n, hidden, vocab, float(scale),
         pos_table.data_ptr() if pos_table is not None else None, positions.data_ptr() if pos_table is not None else None,
         pos_table.shape[0] if pos_table is not None else 0, _stream())
    return out


def depth_average(hist: torch.Tensor, count: int, weights: torch.Tensor, last: torch.Tensor | None = None,
                  rows: torch.Tensor | None = None, out: torch.Tensor | None = None, norm_weight: torch.Tensor | None = None,
                  unit_offset: bool = False, eps: float = 0.0, out_dtype: torch.dtype = torch.float32,
                  branches: tuple[torch.Tensor | None, torch.Tensor | None] = (None, None), mult: float = 1.0
                  ) -> tuple[torch.Tensor, torch.Tensor | None]:
    """A weighted sum over the streams a model has had so far: ``hist`` [streams, tokens, H] (32-bit) of which the
    first ``count`` count, ``weights`` (32-bit, one number a stream, ``last``'s behind the others); ``rows`` (int32):
    only these rows of the streams are wanted, in this order; ``last`` [len(rows) or tokens, H]: one more stream that
    already has the result's rows.  ``out``: where the result goes (a contiguous 32-bit buffer of its shape).
    ``norm_weight`` (32-bit [H]): also returns the result's rows through an RMS norm with this weight (plus one
    with ``unit_offset``), rounded once to ``out_dtype``.  ``branches`` (32-bit, the result's shape; either may be
    None): the newest stream (``last``, or the last counted of ``hist``) first becomes itself + ``mult`` * (a + b), in
    place: a block's residual sum in the same pass."""
    a, b = branches
    _gpu(hist, weights, last, rows, out, norm_weight, a, b)
    _need(hist.dim() == 3 and hist.dtype == torch.float32 and hist.is_contiguous() and 0 <= count <= hist.shape[0],
          "depth_average: the streams must be contiguous float32 [streams, tokens, H]")
    hidden = hist.shape[2]
    n = rows.numel() if rows is not None else (last.shape[0] if last is not None else hist.shape[1])
    if rows is not None:
        _i32(rows, "rows")
    _need(last is None or (last.shape == (n, hidden) and last.dtype == torch.float32 and last.is_contiguous()),
          "depth_average: the last stream must be contiguous float32 with the result's rows")
    _need(rows is not None or n == hist.shape[1], "depth_average: without chosen rows every stream has the result's rows")
    _f32_vector(weights, count + (1 if last is not None else 0), "depth_average: the weights")
    _f32_vector(norm_weight, hidden, "depth_average: a norm weight")
    for y in (a, b):
        _need(y is None or (y.shape == (n, hidden) and y.dtype == torch.float32 and y.is_contiguous()),
              "depth_average: a branch must be contiguous float32 of the result's shape")
    _need((a is None and b is None) or last is not None or (rows is None and count > 0),
          "depth_average: branches are added to a stream that has the result's rows")
    if out is None:
        out = torch.empty((n, hidden), dtype=torch.float32, device=hist.device)
    _need(out.shape == (n, hidden) and out.dtype == torch.float32 and out.is_contiguous(), "depth_average: the result's buffer")
    normed = torch.empty((n, hidden), dtype=out_dtype, device=hist.device) if norm_weight is not None else None
    if n:
        call("tk_depth_average", dtype_code(out_dtype), hist.data_ptr(), hist.stride(0), int(count),
             last.data_ptr() if last is not None else None, rows.data_ptr() if rows is not None else None, weights.data_ptr(),
             out.data_ptr(), norm_weight.data_ptr() if norm_weight is not None else None, 1.0 if unit_offset else 0.0, float(eps),
             normed.data_ptr() if normed is not None else None, n, hidden, a.data_ptr() if a is not None else None,
             b.data_ptr() if b is not None else None, float(mult), _stream())
    return out, normed


# --------------------------------------------------------------------------
# linear attention with a decay, and what stands around it
# --------------------------------------------------------------------------

def linear_attention(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, state: torch.Tensor, q_start: torch.Tensor,
                     slots: torch.Tensor, heads: int, key_dim: int, value_dim: int, decay: torch.Tensor | None = None,
                     forget_bias: torch.Tensor | None = None, forget_low: torch.Tensor | None = None,
                     longest: int | None = None) -> torch.Tensor:
    """The recurrence ``S_t = diag(a_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` per head over every request's
    tokens of this step, from the 32-bit sums ``proj`` of one stacked product (columns from ``q_off``, ``k_off``
    and ``v_off`` on, head by head).  With ``decay`` (32-bit, one number a head): q, k and v pass silu and a_t is
    the head's decay.  With ``forget_bias`` and ``forget_low`` (32-bit [heads * key_dim]): q passes silu, the
    columns at ``k_off`` are a forget gate's, f = low + (1 - low) * sigmoid(. + bias), a_t = f and k_t = 1 - f, v as
    it is.  ``state`` [slots + 1, heads * value_dim * key_dim] (32-bit) is read and written in the requests'
    ``slots``.  ``longest``: the most tokens a request brings in this step (the launch's form depends on it, the sums
    do not; by default the step's tokens).  Returns o [tokens, heads * value_dim] in 32-bit."""
    _gpu(proj, state, q_start, slots, decay, forget_bias, forget_low)
    _need(proj.dim() == 2 and proj.dtype == torch.float32 and proj.stride(1) == 1, "linear_attention: 32-bit rows with unit inner stride")
    H, dk, dv = int(heads), int(key_dim), int(value_dim)
    n, width = proj.shape
    for off, size in ((q_off, H * dk), (k_off, H * dk), (v_off, H * dv)):
        _need(0 <= off and off + size <= width, "linear_attention: a part lies outside the rows")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous() and state.shape[1] >= H * dk * dv,
          "linear_attention: the state must be contiguous float32 [slots, heads * dv * dk]")
    _i32(q_start, "q_start")
    _i32(slots, "slots")
    _need(q_start.numel() == slots.numel() + 1, "linear_attention: one slot a request")
    constant = decay is not None
    _need(constant != (forget_bias is not None and forget_low is not None), "linear_attention: a decay a head, or a forget gate's bias and bound")
    _f32_vector(decay, H, "linear_attention: the decays")
    _f32_vector(forget_bias, H * dk, "linear_attention: the forget gate's bias")
    _f32_vector(forget_low, H * dk, "linear_attention: the forget gate's lower bound")
    _need(dk <= 512, f"linear_attention: heads of up to 512 key channels, not {dk}")
    o = torch.empty((n, H * dv), dtype=torch.float32, device=proj.device)
    if n:
        longest = max(1, int(n if longest is None else longest))
        # the activated rows that the recurrence reads: one pass over the step's tokens in front of it (a step of single
        # tokens computes them in the recurrence's own kernel)
        rec = (torch.empty((n, load("core").tk_linear_attention_rec_width(H, dk, dv)), dtype=torch.float32, device=proj.device)
               if longest > 1 else None)
        call("tk_linear_attention", 0 if constant else 1, proj.data_ptr(), proj.stride(0), int(q_off), int(k_off), int(v_off),
             decay.data_ptr() if constant else None, forget_bias.data_ptr() if not constant else None,
             forget_low.data_ptr() if not constant else None, state.data_ptr(), state.stride(0), q_start.data_ptr(),
             slots.data_ptr(), rec.data_ptr() if rec is not None else None, o.data_ptr(), n, slots.numel(), H, dk, dv, longest,
             _stream())
    return o


def group_norm_gate(o: torch.Tensor, weight: torch.Tensor, eps: float, groups: int, out_dtype: torch.dtype,
                    gate: torch.Tensor | None = None, scale: float = 1.0, out: torch.Tensor | None = None) -> torch.Tensor:
    """Every group's numbers of a token (``groups`` equal groups a row of the 32-bit ``o``) divided by their root
    mean square, times ``weight`` (32-bit, one group's size, shared by the groups), times sigmoid(``gate``) where
    one is given (32-bit, ``o``'s shape, rows a stride apart), times ``scale``; rounded once to ``out_dtype``.
    ``out``: a 2-d view of that type to write to (rows a stride apart)."""
    _gpu(o, weight, gate, out)
    _need(o.dim() == 2 and o.dtype == torch.float32 and o.is_contiguous() and o.shape[1] % groups == 0,
          "group_norm_gate: contiguous float32 rows of equal groups")
    n, width = o.shape
    size = width // int(groups)
    _f32_vector(weight, size, "group_norm_gate: the weight")
    _need(gate is None or (gate.shape == o.shape and gate.dtype == torch.float32 and gate.stride(1) == 1),
          "group_norm_gate: a 32-bit gate of the rows' shape")
    if out is None:
        out = torch.empty((n, width), dtype=out_dtype, device=o.device)
    _need(out.shape == (n, width) and out.dtype == out_dtype and out.stride(1) == 1, "group_norm_gate: the result's view")
    if n:
        call("tk_group_norm_gate", dtype_code(out_dtype), o.data_ptr(), gate.data_ptr() if gate is not None else None,
             gate.stride(0) if gate is not None else 0, weight.data_ptr(), float(eps), float(scale), out.data_ptr(), out.stride(0),
             n, int(groups), size, _stream())
    return out


def sigmoid_gate(x: torch.Tensor, gate: torch.Tensor, scale: float = 1.0, out: torch.Tensor | None = None) -> torch.Tensor:
    """x * sigmoid(gate) * scale element by element (2-d views of one type and shape, rows a stride apart), 32-bit
    arithmetic, one rounding; into ``out`` (such a view) or a new tensor."""
    _gpu(x, gate, out)
    _need(x.dim() == 2 and gate.shape == x.shape and gate.dtype == x.dtype and x.stride(1) == 1 and gate.stride(1) == 1,
          "sigmoid_gate: rows and gates of one shape and type with unit inner stride")
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _need(out.shape == x.shape and out.dtype == x.dtype and out.stride(1) == 1, "sigmoid_gate: the result's view")
    n, width = x.shape
    for first in range(0, n, 65535):
        m = min(65535, n - first)
        xs, gs, os_ = x[first : first + m], gate[first : first + m], out[first : first + m]
        call("tk_sigmoid_gate", dtype_code(x.dtype), xs.data_ptr(), x.stride(0), gs.data_ptr(), gate.stride(0), float(scale),
             os_.data_ptr(), out.stride(0), m, width, _stream())
    return out


def short_conv(h: torch.Tensor, weight: torch.Tensor, tails: torch.Tensor | None, q_start: torch.Tensor, token_req: torch.Tensor,
               slots: torch.Tensor, single_tokens: bool) -> torch.Tensor:
    """h + conv(h) with a causal convolution over time on every channel, ``conv(h)_t = sum_j weight[j] *
    h_(t - taps + 1 + j)``, zeros before a request's start.  ``weight`` [taps, width] in 32-bit (tap by tap; the last
    row is the current token's); ``tails``
    [slots + 1, (taps - 1) * width] (32-bit) holds every request's last taps - 1 inputs and is moved on.
    ``single_tokens``: every request of the step brings one token (the tails then move in the same kernel)."""
    _gpu(h, weight, tails, q_start, token_req, slots)
    _need(h.dim() == 2 and h.stride(1) == 1, "short_conv: rows with unit inner stride")
    n, width = h.shape
    _need(weight.dim() == 2 and weight.shape[1] == width and weight.dtype == torch.float32 and weight.is_contiguous(),
          "short_conv: taps must be contiguous float32 [taps, width]")
    taps = weight.shape[0]
    if taps > 1:
        _need(tails is not None and tails.dim() == 2 and tails.dtype == torch.float32 and tails.is_contiguous()
              and tails.shape[1] >= (taps - 1) * width, "short_conv: the tails must be contiguous float32 [slots, (taps - 1) * width]")
    for t, name in ((q_start, "q_start"), (token_req, "token_req"), (slots, "slots")):
        _i32(t, name)
    _need(token_req.numel() == n and q_start.numel() == slots.numel() + 1, "short_conv: one request a token, one slot a request")
    out = torch.empty((n, width), dtype=h.dtype, device=h.device)
    if n:
        _need(n < 65536, "short_conv: a step of fewer than 65 536 tokens")
        call("tk_short_conv", dtype_code(h.dtype), h.data_ptr(), h.stride(0), weight.data_ptr(), taps,
             tails.data_ptr() if tails is not None else None, tails.stride(0) if tails is not None else 0, q_start.data_ptr(),
             token_req.data_ptr(), slots.data_ptr(), out.data_ptr(), n, slots.numel(), width, 1 if single_tokens else 0, _stream())
    return out


def gelu_glu(gate_up: torch.Tensor) -> torch.Tensor:
    """[rows, 2I] laid out [gate | up] -> gelu(gate) * up with the tanh form of gelu, [rows, I]; 32-bit arithmetic, one rounding."""
    _gpu(gate_up)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0, "gelu_glu input must be contiguous [rows, 2I]")
    rows, two_i = gate_up.shape
    out = torch.empty((rows, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    for first in range(0, rows, 65535):
        m = min(65535, rows - first)
        call("tk_gelu_glu", dtype_code(gate_up.dtype), gate_up[first:].data_ptr(), out[first:].data_ptr(), m, two_i // 2, _stream())
    return out


def residual_norm(
    x: torch.Tensor,
    branches: tuple[torch.Tensor | None, torch.Tensor | None] = (None, None),
    mult: float = 1.0,
    weights: tuple[torch.Tensor | None, torch.Tensor | None] = (None, None),
    unit_offset: bool = False,
    eps: float = 0.0,
    out_dtype: torch.dtype = torch.float32,
    in_place: bool = True,
) -> tuple[torch.Tensor, torch.Tensor | None, torch.Tensor | None]:
    """The update of a 32-bit residual stream and the norms that read the new stream, in one pass:
    ``x_new = x + mult * (a + b)`` for the 32-bit ``branches`` (either may be None; with neither
    the stream stays), then for each of up to two 32-bit ``weights`` the rows
    ``x_new / sqrt(mean(x_new^2) + eps) * (w + (1 if unit_offset else 0))`` rounded once to
    ``out_dtype``.  Returns (x_new, normed rows for weights[0], for weights[1]).  ``in_place``:
    the new stream overwrites ``x``."""
    a, b = branches
    w1, w2 = weights
    _gpu(x, a, b, w1, w2)
    _need(x.dim() == 2 and x.dtype == torch.float32 and x.is_contiguous(), "residual_norm: the stream must be contiguous float32 [rows, H]")
    rows, hidden = x.shape
    for y in (a, b):
        _need(y is None or (y.shape == x.shape and y.dtype == torch.float32 and y.is_contiguous()),
              "residual_norm: a branch must be contiguous float32 of the stream's shape")
    _f32_vector(w1, hidden, "residual_norm: a norm weight")
    _f32_vector(w2, hidden, "residual_norm: a norm weight")
    changed = a is not None or b is not None
    x_out = (x if in_place else torch.empty_like(x)) if changed else x
    h1 = torch.empty((rows, hidden), dtype=out_dtype, device=x.device) if w1 is not None else None
    h2 = torch.empty((rows, hidden), dtype=out_dtype, device=x.device) if w2 is not None else None
    if rows == 0:
        return x_out, h1, h2
    call("tk_residual_norm", dtype_code(out_dtype), x.data_ptr(), a.data_ptr() if a is not None else None,
         b.data_ptr() if b is not None else None, float(mult), x_out.data_ptr() if changed else None,
         w1.data_ptr() if w1 is not None else None, w2.data_ptr() if w2 is not None else None,
         1.0 if unit_offset else 0.0, float(eps), h1.data_ptr() if h1 is not None else None,
         h2.data_ptr() if h2 is not None else None, rows, hidden, _stream())
    return x_out, h1, h2


def softcap_(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits <- cap * tanh(logits / cap), in place (contiguous float32)."""
    _gpu(logits)
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "softcap: logits must be contiguous float32")
    call("tk_softcap", logits.data_ptr(), logits.numel(), float(cap), _stream())
    return logits


def scale_(logits: torch.Tensor, scale: float) -> torch.Tensor:
    """logits <- logits * scale, in place (contiguous float32)."""
    _gpu(logits)
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "scale: logits must be contiguous float32")
    call("tk_scale_values", logits.data_ptr(), logits.numel(), float(scale), _stream())
    return logits


def cast_rows(x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """A 32-bit stream rounded once to ``out_dtype`` (the stream itself when that is 32-bit)."""
    if out_dtype == torch.float32:
        return x
    _gpu(x)
    _need(x.dtype == torch.float32 and x.is_contiguous(), "cast_rows: contiguous float32 rows")
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    call("tk_cast_rows", dtype_code(out_dtype), x.data_ptr(), out.data_ptr(), x.numel(), _stream())
    return out


def embed_bigram(ctx_ids: torch.Tensor, last_token: torch.Tensor | None, positions: torch.Tensor, token_req: torch.Tensor,
                 q_start: torch.Tensor, slots: torch.Tensor, prev_token: torch.Tensor, table: torch.Tensor, pairs: torch.Tensor,
                 scale: float, mul_prev: int, mul_cur: int, want_cast: bool = True) -> tuple[torch.Tensor, torch.Tensor | None]:
    """The first rows of a 32-bit stream: ``table[id] * scale + pairs[(prev * mul_prev + id * mul_cur) mod buckets]``
    where ``pairs`` has buckets + 1 rows and a request's first token (position 0) takes the last.  ``prev`` is
    the token in front in this step or, for a request's first token of the step, ``prev_token[slot]``, which
    is then set to the request's last token of this step.  Also returns the rows rounded once to the
    table's type (None when that is 32-bit or ``want_cast`` is off)."""
    _gpu(ctx_ids, last_token, positions, token_req, q_start, slots, prev_token, table, pairs)
    for t, name in ((ctx_ids, "ids"), (positions, "positions"), (token_req, "token_req"), (q_start, "q_start"), (slots, "slots"),
                    (prev_token, "prev_token")):
        _i32(t, name)
    if last_token is not None:
        _i32(last_token, "last_token")
    _need(table.dim() == 2 and table.is_contiguous() and pairs.dim() == 2 and pairs.is_contiguous() and pairs.dtype == table.dtype
          and pairs.shape[1] == table.shape[1] and pairs.shape[0] >= 2, "embed_bigram: tables [V, H] and [buckets + 1, H] of one type")
    n = ctx_ids.numel()
    vocab, hidden = table.shape
    _need(positions.numel() == n and token_req.numel() == n, "embed_bigram: one position and one request a token")
    out = torch.empty((n, hidden), dtype=torch.float32, device=table.device)
    cast = torch.empty((n, hidden), dtype=table.dtype, device=table.device) if (want_cast and table.dtype != torch.float32) else None
    call("tk_embed_bigram", dtype_code(table.dtype), ctx_ids.data_ptr(), last_token.data_ptr() if last_token is not None else None,
         positions.data_ptr(), token_req.data_ptr(), q_start.data_ptr(), slots.data_ptr(), prev_token.data_ptr(), table.data_ptr(),
         pairs.data_ptr(), out.data_ptr(), cast.data_ptr() if cast is not None else None, n, hidden, vocab, float(scale),
         pairs.shape[0] - 1, int(mul_prev), int(mul_cur), _stream())
    return out, cast


def clamped_glu(gate_up: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    """[rows, 2I] laid out [gate | up] -> g * sigmoid(alpha * g) * (u + 1) with g = min(gate, limit) and
    u = clamp(up, -limit, limit), [rows, I]; 32-bit arithmetic, one rounding."""
    _gpu(gate_up)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0, "clamped_glu input must be contiguous [rows, 2I]")
    rows, two_i = gate_up.shape
    out = torch.empty((rows, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    call("tk_clamped_glu", dtype_code(gate_up.dtype), gate_up.data_ptr(), out.data_ptr(), rows, two_i // 2, float(limit), float(alpha),
         _stream())
    return out


def min_gru(proj: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor, slots: torch.Tensor, width: int, longest: int,
            out_dtype: torch.dtype, bias: torch.Tensor | None = None) -> torch.Tensor:
    """The gated recurrence ``S <- (1 - z) S + z cand`` per channel over every request's tokens of this
    step, from and to the request's slot of ``state`` [slots, width] (32-bit): ``proj`` holds the 32-bit
    sums (a, u, g) channel by channel ([tokens, width * 3]; z = sigmoid(a), cand = u + 1/2 for u >= 0 and sigmoid(u) below);
    returns S_t * silu(g) rounded once to ``out_dtype``.  ``longest``: the most tokens a request brings.
    ``bias`` (32-bit, [2 width]): added to a and to u here, when the product has not."""
    _gpu(proj, state, q_start, slots, bias)
    _f32_vector(bias, 2 * width, "min_gru: the biases of z and of the candidate")
    _need(proj.dim() == 2 and proj.dtype == torch.float32 and proj.stride(1) == 1 and proj.shape[1] >= 3 * width,
          "min_gru: 32-bit rows of (a, u, g) a channel")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.stride(1) == 1 and state.shape[1] >= width,
          "min_gru: the state is 32-bit [slots, width]")
    _i32(q_start, "q_start")
    _i32(slots, "slots")
    _need(q_start.numel() == slots.numel() + 1, "min_gru: one slot a request")
    out = torch.empty((proj.shape[0], width), dtype=out_dtype, device=proj.device)
    call("tk_min_gru", dtype_code(out_dtype), proj.data_ptr(), proj.stride(0), bias.data_ptr() if bias is not None else None,
         state.data_ptr(), state.stride(0), q_start.data_ptr(),
         slots.data_ptr(), out.data_ptr(), slots.numel(), int(width), int(longest), _stream())
    return out


def unrotate_gate_(o: torch.Tensor, positions: torch.Tensor | None, value_freq: torch.Tensor | None, pair_halves: bool,
                   gate: torch.Tensor | None, nq: int, value_dim: int) -> torch.Tensor:
    """In place on the heads' results [tokens, nq * value_dim]: pair m of every head turned by
    -position * value_freq[m] (pairs as in ``qk_prepare``'s ``value_freq``), then head h times
    sigmoid(gate[token, h]); ``gate`` is a 2-d view (rows may be strided) of the rows' type."""
    _gpu(o, positions, value_freq, gate)
    _need(o.dim() == 2 and o.stride(1) == 1 and o.shape[1] >= nq * value_dim, "unrotate_gate: rows of nq * dv")
    if value_freq is not None:
        _i32(positions, "positions")
        _need(positions.numel() == o.shape[0], "unrotate_gate: one position a token")
        _f32_vector(value_freq, value_dim // 2, "unrotate_gate: the values' frequencies")
    if gate is not None:
        _need(gate.dim() == 2 and gate.stride(1) == 1 and gate.shape == (o.shape[0], nq) and gate.dtype == o.dtype,
              "unrotate_gate: one gate a token and head, of the rows' type")
    call("tk_unrotate_gate", dtype_code(o.dtype), o.data_ptr(), o.stride(0), positions.data_ptr() if value_freq is not None else None,
         value_freq.data_ptr() if value_freq is not None else None, 1 if pair_halves else 0,
         gate.data_ptr() if gate is not None else None, gate.stride(0) if gate is not None else 0, o.shape[0], nq, value_dim, _stream())
    return o


# --------------------------------------------------------------------------
# attention with norms over the whole projection and a rotation of neighbouring elements
# --------------------------------------------------------------------------

def qk_prepare(
    qkv: torch.Tensor,
    positions: torch.Tensor,
    token_req: torch.Tensor,
    block_table: torch.Tensor | None,
    q_weight: torch.Tensor | None,
    k_weight: torch.Tensor | None,
    eps: float,
    freq: torch.Tensor | None,
    kcache: torch.Tensor | None,
    vcache: torch.Tensor | None,
    nq: int,
    nkv: int,
    key_dim: int,
    value_dim: int,
    page_size: int,
    write_cache: bool = True,
    query_dim: int | None = None,
    pair_halves: bool = False,
    values_are_keys: bool = False,
    per_head: bool = False,
    key_skip: int = 0,
    value_freq: torch.Tensor | None = None,
    value_pair_halves: bool = False,
    rotation_scale: float = 1.0,
) -> None:
    """In place on the rows [q: nq*dq | k: nkv*dk | v: nkv*dv] (only q when not ``write_cache``):
    the RMS norm of the whole query row and of the whole key row (32-bit weights of those sizes,
    or None for no norm), the rotation of elements (2i, 2i+1) of every head by position *
    freq[i] for i < len(freq), and the append of keys and values to the token's page.
    ``query_dim``: the size dq of a query head where it is not a key head's.  ``pair_halves``:
    the rotation pairs element i with element i + len(freq) instead of neighbours.
    ``values_are_keys``: the rows hold no values; a token's values are its keys as they are
    before the rotation (after the norm, when there is one).  ``per_head``: the norms take their
    statistics head by head and their weights have one head's size.  ``key_skip``: the leading
    elements of a key head that are neither normed nor weighted; with ``values_are_keys`` the values
    are the elements behind them.  ``value_freq`` (32-bit, half a value head's size): every element of
    a value head is turned before it is cached, pair m by position * value_freq[m], pairs
    (m, m + dv/2) with ``value_pair_halves`` and (2m, 2m+1) without.  ``rotation_scale``: a factor on
    the cosines and sines of the queries' and keys' rotation."""
    _gpu(qkv, positions, token_req, block_table, q_weight, k_weight, freq, kcache, vcache, value_freq)
    _need(qkv.dim() == 2 and qkv.stride(1) == 1, "qk_prepare: rows must be 2-d with unit inner stride")
    n = qkv.shape[0]
    dq = key_dim if query_dim is None else int(query_dim)
    key_skip = int(key_skip)
    _need(not values_are_keys or value_dim == key_dim - key_skip, "qk_prepare: values that are the keys have the keys' size")
    need = nq * dq + (nkv * (key_dim + (0 if values_are_keys else value_dim)) if write_cache else 0)
    _need(qkv.shape[1] >= need, f"qk_prepare: rows of {qkv.shape[1]} hold no {need} elements")
    _i32(positions, "positions")
    _i32(token_req, "token_req")
    _need(positions.numel() == n and token_req.numel() == n, "positions/token_req must have one entry a token")
    _f32_vector(q_weight, dq if per_head else nq * dq, "qk_prepare: the query norm's weight")
    _f32_vector(k_weight, (1 if per_head else nkv) * (key_dim - key_skip), "qk_prepare: the key norm's weight")
    _f32_vector(value_freq, value_dim // 2, "qk_prepare: the values' frequencies")
    rot = 0
    if freq is not None:
        _need(freq.dim() == 1 and freq.dtype == torch.float32 and freq.is_contiguous() and 2 * freq.numel() <= min(key_dim, dq),
              "qk_prepare: frequencies must be contiguous float32, at most half a head's size of them")
        rot = 2 * freq.numel()
    if write_cache:
        _i32(block_table, "block_table")
        _need(block_table.dim() == 2, "block_table must be [requests, width]")
        _check_pages(kcache, vcache, nkv, page_size, key_dim, qkv.dtype, "qk_prepare", value_dim)
    call("tk_qk_prepare", dtype_code(qkv.dtype), qkv.data_ptr(), qkv.stride(0), positions.data_ptr(), token_req.data_ptr(),
         block_table.data_ptr() if write_cache else None, block_table.stride(0) if write_cache else 0,
         q_weight.data_ptr() if q_weight is not None else None, k_weight.data_ptr() if k_weight is not None else None,
         float(eps), freq.data_ptr() if freq is not None else None,
         kcache.data_ptr() if write_cache else None, vcache.data_ptr() if write_cache else None,
         n, nq, nkv if write_cache else 0, dq, key_dim, value_dim, rot, page_size, 1 if write_cache else 0,
         1 if pair_halves else 0, 1 if values_are_keys else 0, 1 if per_head else 0, key_skip,
         value_freq.data_ptr() if value_freq is not None else None, 1 if value_pair_halves else 0, float(rotation_scale),
         _stream())


def gather_keys(kcache: torch.Tensor, block_table: torch.Tensor, req: torch.Tensor, pos: torch.Tensor, key_dim: int,
                page_size: int, head: int = 0) -> torch.Tensor:
    """The keys of kv head ``head`` that request ``req[i]`` (a row of ``block_table``) holds at position
    ``pos[i]``, read back from the pages: [len(req), key_dim]."""
    _gpu(kcache, block_table, req, pos)
    for t, name in ((block_table, "block_table"), (req, "req"), (pos, "pos")):
        _i32(t, name)
    nkv = kcache.shape[1]
    _need(kcache.is_contiguous() and kcache.shape[1:] == key_pages_shape(1, nkv, page_size, key_dim, padded=True)[1:],
          "gather_keys: key pages of this head size and page size")
    _need(block_table.dim() == 2 and req.numel() == pos.numel(), "gather_keys: block_table [requests, width], one request and one position a row")
    out = torch.empty((req.numel(), key_dim), dtype=kcache.dtype, device=kcache.device)
    call("tk_gather_keys", dtype_code(kcache.dtype), kcache.data_ptr(), block_table.data_ptr(), block_table.stride(0), req.data_ptr(),
         pos.data_ptr(), out.data_ptr(), req.numel(), nkv, int(head), key_dim, page_size, _stream())
    return out


def attention_tile_f32_fits(nq: int, nkv: int, key_dim: int, value_dim: int, page_size: int) -> bool:
    """Whether the 32-bit matrix-core attention takes the shape (key size a multiple of 8 up to
    256, value size a multiple of 16 up to 256, pages of a multiple of 16 keys)."""
    return bool(load("core").tk_attention_tile_f32_fits(nq, nkv, key_dim, value_dim, page_size))


def attention_tile_turns_halves(value_dim: int) -> bool:
    """Whether the matrix-core attention can itself turn back the halves of a value head of this size."""
    return bool(load("core").tk_attention_tile_turns_halves(int(value_dim)))


ATTENTION_TILE_SPLIT_BELOW = 2048  # (tile, head block) pairs of a step below which the wavefronts share tiles
ATTENTION_TILE_WORKGROUPS = 512  # workgroups a step with key chunks should have before its chunks grow
ATTENTION_TILE_LONGEST_CHUNK = 2048


def attention_tile_heads(group: int, max_q_len: int) -> int:
    """Query heads of one kv head that share a tile of 16 columns: one for prompt portions (16
    tokens a tile), as many as the group has (the largest power of two that divides it, at most
    16) when every request brings one token."""
    if max_q_len > 1:
        return 1
    gg = 1
    while gg < 16 and group % (gg * 2) == 0:
        gg *= 2
    return gg


def attention_tile_f32(
    q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, block_table: torch.Tensor, q_start: torch.Tensor,
    kv_len: torch.Tensor, tile_req: torch.Tensor, tile_row0: torch.Tensor, nq: int, nkv: int, key_dim: int,
    value_dim: int, page_size: int, heads_a_tile: int, window: int = 0, scale: float = 1.0,
    sink: torch.Tensor | None = None, split: bool | None = None, key_chunk: int = 0, longest: int = 0, first_row: int = 0,
    score_bias: torch.Tensor | None = None, value_freq: torch.Tensor | None = None,
    value_pair_halves: bool = False, gate: torch.Tensor | None = None, softcap: float = 0.0,
    distance_bias: "DistanceBias | None" = None,
) -> torch.Tensor:
    """Attention in 32-bit arithmetic on the matrix cores: every token of the step over its
    request's pages; ``tile_req`` / ``tile_row0`` name each tile's request and its first token's
    row (a tile holds 16 / heads_a_tile neighbouring tokens of one request).  Window, scale,
    value size and sinks as in ``paged_attention_generic``; returns [tokens, nq * value_dim].
    ``split``: the four wavefronts of a workgroup share a tile and take its keys in turn (by
    default when the step has so few tiles that their walks would leave the chip idle).
    ``key_chunk`` (a multiple of 128; with ``longest``, a bound on every request's length that does not
    depend on the batch): a split tile's keys are also cut at absolute multiples of ``key_chunk`` among
    workgroups, whose partial results a second kernel adds in ascending order.
    ``first_row``: ``q`` holds the step's rows from this one on only (the tiles name none before it), and so
    does the result.  ``score_bias``: sigmoid weights as in ``paged_attention_generic``.  ``value_freq``,
    ``value_pair_halves``, ``gate``: what ``unrotate_gate_`` does, in the kernel's own epilogue (halves only where
    ``attention_tile_turns_halves``)."""
    _gpu(q, kcache, vcache, block_table, q_start, kv_len, tile_req, tile_row0, sink, score_bias, value_freq, gate)
    db = _checked_distance_bias(distance_bias, nq)
    _f32_vector(value_freq, value_dim // 2, "attention: the values' frequencies")
    _need(value_freq is None or not value_pair_halves or attention_tile_turns_halves(value_dim),
          "attention: the halves of this value size are turned back by unrotate_gate_")
    _need(gate is None or (gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[1] == nq and gate.dtype == q.dtype
                           and gate.shape[0] == q.shape[0]), "attention: one gate a token and head, of the rows' type")
    _f32_vector(score_bias, nq, "attention: the scores' biases")
    if split is None:
        split = tile_req.numel() * nkv * ((nq // nkv) // int(heads_a_tile)) < ATTENTION_TILE_SPLIT_BELOW
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nq * key_dim,
          "attention: q must be 2-d with unit inner stride and nq*d leading columns")
    for t, name in ((block_table, "block_table"), (q_start, "q_start"), (kv_len, "kv_len"), (tile_req, "tile_req"), (tile_row0, "tile_row0")):
        _i32(t, name)
    _need(block_table.dim() == 2 and tile_req.numel() == tile_row0.numel() and q_start.numel() == kv_len.numel() + 1,
          "attention: block_table [requests, width], one request and one row a tile, one length a request")
    _need(sink is None or (sink.shape == (nq,) and sink.dtype == torch.float32 and sink.is_contiguous()),
          f"attention: the sinks must be contiguous float32 [{nq}]")
    _check_pages(kcache, vcache, nkv, page_size, key_dim, q.dtype, "attention", value_dim)
    out = torch.empty((q.shape[0], nq * value_dim), dtype=q.dtype, device=q.device)
    chunks, part = 0, None
    if split and key_chunk > 0 and longest > key_chunk:
        # longer chunks where the step has workgroups enough without short ones: a chunk's walk should be long
        # enough to hide its first loads
        groups = tile_req.numel() * nkv * ((nq // nkv) // int(heads_a_tile))
        # (behind a window a tile sees at most window + 15 keys, whatever the request's length: they lie in
        # `seen // chunk + 1` chunks at most, one more when they start inside one, and the kernel counts a tile's
        # chunks from the first it sees)
        seen = min(int(longest), int(window) + 15) if window > 0 else int(longest)
        while key_chunk < ATTENTION_TILE_LONGEST_CHUNK and groups * -(-seen // (2 * key_chunk)) >= ATTENTION_TILE_WORKGROUPS:
            key_chunk *= 2
        chunks = -(-int(longest) // int(key_chunk))
        if window > 0:
            chunks = min(chunks, -(-seen // int(key_chunk)) + 1)
        words = load("core").tk_attention_tile_part_words(value_dim)
        part = torch.empty((tile_req.numel() * nkv * ((nq // nkv) // int(heads_a_tile)) * chunks * words,), dtype=torch.float32, device=q.device)
    # the kernel finds a tile's rows by their place in the step
    q_base = q.data_ptr() - int(first_row) * q.stride(0) * q.element_size()
    out_base = out.data_ptr() - int(first_row) * out.stride(0) * out.element_size()
    call("tk_attention_tile_f32", dtype_code(q.dtype), q_base, q.stride(0), out_base, out.stride(0),
         kcache.data_ptr(), vcache.data_ptr(), block_table.data_ptr(), block_table.stride(0), q_start.data_ptr(),
         kv_len.data_ptr(), tile_req.data_ptr(), tile_row0.data_ptr(), tile_req.numel(), nq, nkv, key_dim, value_dim,
         page_size, int(window), float(scale), sink.data_ptr() if sink is not None else None,
         score_bias.data_ptr() if score_bias is not None else None, int(heads_a_tile),
         1 if split else 0, int(key_chunk) if chunks else 0, chunks, part.data_ptr() if part is not None else None,
         value_freq.data_ptr() if value_freq is not None else None, 1 if value_pair_halves else 0,
         (gate.data_ptr() - int(first_row) * gate.stride(0) * gate.element_size()) if gate is not None else None,
         gate.stride(0) if gate is not None else 0, float(softcap), *db, _stream())
    return out


# --------------------------------------------------------------------------
# the gated delta rule with a decay per key channel
# --------------------------------------------------------------------------

def delta_state_size(heads: int, kv_heads: int, key_dim: int, value_dim: int, taps: int) -> int:
    """32-bit numbers a request keeps for one such mixer: the matrices S and the convolutions' tails."""
    return heads * key_dim * value_dim + (taps - 1) * (2 * kv_heads * key_dim + heads * value_dim)


def delta_rec_width(heads: int, kv_heads: int, key_dim: int, value_dim: int) -> int:
    """Numbers a token's row of the recurrence's input holds (q | k | v | decay | beta), filled up to a multiple of 4."""
    return -(-(2 * kv_heads * key_dim + heads * value_dim + heads * key_dim + heads) // 4) * 4


def delta_prepare(
    proj: torch.Tensor,
    col_b: int,
    a_pre: torch.Tensor,
    conv_w: torch.Tensor,
    a_log: torch.Tensor,
    dt_bias: torch.Tensor,
    state: torch.Tensor,
    q_start: torch.Tensor,
    token_req: torch.Tensor,
    slots: torch.Tensor,
    heads: int,
    kv_heads: int,
    key_dim: int,
    value_dim: int,
) -> torch.Tensor:
    """What the recurrence reads, in 32-bit [tokens, q | k | v | decay | beta]: the rows
    ``proj`` [q | k | v | ...] pass their short causal convolutions (``conv_w`` [channels, taps],
    earlier inputs from this step's rows or the tail in the request's ``state`` row) and silu; q
    and k become unit vectors per head (q also times key_dim^-1/2); decay = exp(-exp(a_log) *
    softplus(a_pre + dt_bias)); beta = sigmoid(proj[:, col_b + head]).  The tails in ``state``
    are then moved on by this step's rows."""
    _gpu(proj, a_pre, conv_w, a_log, dt_bias, state, q_start, token_req, slots)
    n = proj.shape[0]
    channels = 2 * kv_heads * key_dim + heads * value_dim
    _need(proj.dim() == 2 and proj.stride(1) == 1 and proj.dtype in _DT, "delta_prepare: rows must be 2-d with unit inner stride")
    _need(conv_w.dim() == 2 and conv_w.shape[0] == channels and conv_w.dtype == torch.float32 and conv_w.is_contiguous(),
          f"delta_prepare: the convolutions' weights must be contiguous float32 [{channels}, taps]")
    taps = conv_w.shape[1]
    _need(a_pre.shape == (n, heads * key_dim) and a_pre.dtype == torch.float32 and a_pre.stride(1) == 1,
          "delta_prepare: the decay's projection must be float32 [tokens, heads * key_dim] with unit inner stride")
    _f32_vector(a_log, heads, "delta_prepare: a_log")
    _f32_vector(dt_bias, heads * key_dim, "delta_prepare: dt_bias")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and state.shape[1] >= delta_state_size(heads, kv_heads, key_dim, value_dim, taps), "delta_prepare: state rows too short")
    for t, name in ((q_start, "q_start"), (token_req, "token_req"), (slots, "slots")):
        _i32(t, name)
    _need(token_req.numel() == n and q_start.numel() == slots.numel() + 1, "delta_prepare: one request a token, one slot a request")
    width = delta_rec_width(heads, kv_heads, key_dim, value_dim)
    rec = torch.empty((n, width), dtype=torch.float32, device=proj.device)
    call("tk_delta_prepare", dtype_code(proj.dtype), proj.data_ptr(), proj.stride(0), int(col_b), a_pre.data_ptr(),
         a_pre.stride(0) if n > 1 else heads * key_dim, conv_w.data_ptr(), taps, a_log.data_ptr(), dt_bias.data_ptr(), state.data_ptr(), state.stride(0),
         heads * key_dim * value_dim, q_start.data_ptr(), token_req.data_ptr(), slots.data_ptr(), rec.data_ptr(), width,
         n, slots.numel(), heads, kv_heads, key_dim, value_dim, _stream())
    return rec


def delta_rule_columns(requests: int, heads: int, key_dim: int, value_dim: int) -> int:
    """Value columns a workgroup of the recurrence owns (16 lanes a column): few, so that the
    chip gets many small workgroups whose wavefronts each have a vector unit to themselves (a
    token's chain of operations is what takes the time); more only when there are so many
    workgroups that they queue up anyway.  A column's arithmetic does not depend on the choice."""
    most = 32 if key_dim <= 128 else 16
    cols = 8 if value_dim > 4 else 4
    while cols * 2 <= most and cols < value_dim and requests * heads * -(-value_dim // cols) > 4096:
        cols *= 2
    return cols


def delta_rule(rec: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor, slots: torch.Tensor,
               heads: int, kv_heads: int, key_dim: int, value_dim: int) -> torch.Tensor:
    """The recurrence over every request's tokens of this step, from and to the matrices in the
    requests' ``state`` rows: o [tokens, heads * value_dim] in 32-bit."""
    _gpu(rec, state, q_start, slots)
    n = rec.shape[0]
    _need(rec.dim() == 2 and rec.dtype == torch.float32 and rec.is_contiguous()
          and rec.shape[1] == delta_rec_width(heads, kv_heads, key_dim, value_dim), "delta_rule: rows of the wrong width")
    _need(state.dim() == 2 and state.dtype == torch.float32 and state.is_contiguous()
          and state.shape[1] >= heads * key_dim * value_dim, "delta_rule: state rows too short")
    _i32(q_start, "q_start")
    _i32(slots, "slots")
    _need(q_start.numel() == slots.numel() + 1, "delta_rule: one slot a request")
    o = torch.empty((n, heads * value_dim), dtype=torch.float32, device=rec.device)
    cols = delta_rule_columns(slots.numel(), heads, key_dim, value_dim)
    call("tk_delta_rule", rec.data_ptr(), rec.stride(0), state.data_ptr(), state.stride(0), q_start.data_ptr(),
         slots.data_ptr(), o.data_ptr(), slots.numel(), heads, kv_heads, key_dim, value_dim, cols, _stream())
    return o


def gated_head_norm(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float, heads: int, value_dim: int,
                    out_dtype: torch.dtype) -> torch.Tensor:
    """Every head's ``value_dim`` numbers divided by their root mean square, times ``weight``
    [value_dim], times sigmoid(gate); 32-bit in, rounded once to ``out_dtype``."""
    _gpu(o, gate, weight)
    n = o.shape[0]
    for t in (o, gate):
        _need(t.shape == (n, heads * value_dim) and t.dtype == torch.float32 and t.stride(1) == 1,
              "gated_head_norm: inputs must be float32 [tokens, heads * value_dim] with unit inner stride")
    _need(o.is_contiguous(), "gated_head_norm: the recurrence's output must be contiguous")
    _f32_vector(weight, value_dim, "gated_head_norm: the weight")
    out = torch.empty((n, heads * value_dim), dtype=out_dtype, device=o.device)
    call("tk_gated_head_norm", dtype_code(out_dtype), o.data_ptr(), gate.data_ptr(), gate.stride(0) if n > 1 else heads * value_dim,
         weight.data_ptr(), float(eps), out.data_ptr(), n, heads, value_dim, _stream())
    return out


# --------------------------------------------------------------------------
# a stream whose branches are normed before they are added
# --------------------------------------------------------------------------

def post_norm_residual(x: torch.Tensor, branch: torch.Tensor, branch_weight: torch.Tensor, branch_eps: float,
                       weight: torch.Tensor | None = None, eps: float = 0.0, out_dtype: torch.dtype = torch.float32,
                       in_place: bool = True, plain_rows: bool = False) -> tuple[torch.Tensor, torch.Tensor | None]:
    """``x_new = x + branch / sqrt(mean(branch^2) + branch_eps) * branch_weight`` on a 32-bit
    stream (the branch 32-bit too), and, when ``weight`` is given, the rows of the norm that
    reads the new stream, ``x_new / sqrt(mean(x_new^2) + eps) * weight`` rounded once to
    ``out_dtype``.  Returns (x_new, those rows or None).  ``in_place``: x_new overwrites x.
    ``plain_rows`` (without ``weight``): the rows returned are x_new itself rounded once to ``out_dtype``
    (x_new when that is 32-bit): for sublayers that read the stream unnormed."""
    _gpu(x, branch, branch_weight, weight)
    _need(x.dim() == 2 and x.dtype == torch.float32 and x.is_contiguous(), "post_norm_residual: the stream must be contiguous float32 [rows, H]")
    _need(branch.shape == x.shape and branch.dtype == torch.float32 and branch.is_contiguous(),
          "post_norm_residual: the branch must be contiguous float32 of the stream's shape")
    rows, hidden = x.shape
    _f32_vector(branch_weight, hidden, "post_norm_residual: the branch norm's weight")
    _f32_vector(weight, hidden, "post_norm_residual: a norm weight")
    x_out = x if in_place else torch.empty_like(x)
    _need(not (plain_rows and weight is not None), "post_norm_residual: plain rows or a norm's rows, not both")
    cast = plain_rows and out_dtype != torch.float32
    h = torch.empty((rows, hidden), dtype=out_dtype, device=x.device) if (weight is not None or cast) else None
    if rows:
        call("tk_post_norm_residual", dtype_code(out_dtype), x.data_ptr(), branch.data_ptr(), branch_weight.data_ptr(),
             float(branch_eps), x_out.data_ptr(), weight.data_ptr() if weight is not None else None, float(eps),
             h.data_ptr() if h is not None else None, rows, hidden, _stream())
    return x_out, (x_out if plain_rows and not cast else h)


def concat_cast(x: torch.Tensor, y: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[x | y] row by row for two 32-bit streams of one shape, rounded once to ``out_dtype``."""
    _gpu(x, y)
    _need(x.dim() == 2 and x.dtype == torch.float32 and x.is_contiguous() and y.shape == x.shape and y.dtype == torch.float32
          and y.is_contiguous(), "concat_cast: two contiguous float32 streams of one shape")
    out = torch.empty((x.shape[0], 2 * x.shape[1]), dtype=out_dtype, device=x.device)
    if x.shape[0]:
        call("tk_concat_cast", dtype_code(out_dtype), x.data_ptr(), y.data_ptr(), out.data_ptr(), x.shape[0], x.shape[1], _stream())
    return out


def squared_relu_(x: torch.Tensor) -> torch.Tensor:
    """x <- max(x, 0)^2, in place."""
    _gpu(x)
    _need(x.is_contiguous(), "squared_relu: the rows must be contiguous")
    call("tk_squared_relu", dtype_code(x.dtype), x.data_ptr(), x.numel(), _stream())
    return x


# --------------------------------------------------------------------------
# a matrix a head; experts of which a token uses a few
# --------------------------------------------------------------------------

GROUPED_TILE = 64  # slots a tile of the grouped matrix-core product (GG_TM of grouped_gemm.hip)
GROUPED_FROM_ROWS = 16  # rows above which the products of experts and of heads run in tiles on the matrix cores


def _grouped_takes(x: torch.Tensor, w: torch.Tensor, inner: int) -> bool:
    """Whether the grouped matrix-core product takes these rows and weights: bfloat16, rows that start at
    multiples of 16 bytes."""
    return (x.dtype == torch.bfloat16 and inner % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def head_linear(x: torch.Tensor, w: torch.Tensor, out_f32: bool = False) -> torch.Tensor:
    """y[t, h, :] = w[h] x[t, h, :] for w [heads, out, in] and the leading heads * in columns of
    the rows of x; returns [tokens, heads * out] in x's type, or 32-bit sums with ``out_f32``."""
    _gpu(x, w)
    _need(w.dim() == 3 and w.is_contiguous() and w.dtype == x.dtype, "head_linear: weights contiguous [heads, out, in] of the rows' type")
    heads, n_out, n_in = w.shape
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[1] >= heads * n_in, "head_linear: rows of unit inner stride that hold heads * in columns")
    y = torch.empty((x.shape[0], heads * n_out), dtype=torch.float32 if out_f32 else x.dtype, device=x.device)
    if x.shape[0] > GROUPED_FROM_ROWS and _grouped_takes(x, w, n_in):
        # many rows: tiles of 32 rows on the matrix cores, the head as the tile's group
        tiles = -(-x.shape[0] // GROUPED_TILE)
        call("tk_grouped_gemm_bf16", x.data_ptr(), x.stride(0), None, None, None, tiles, heads, n_in, n_out, w.data_ptr(),
             n_out * n_in, y.data_ptr(), y.stride(0), n_out, n_in, x.shape[0], 0, 1 if out_f32 else 0, _stream())
        return y
    if x.shape[0]:
        call("tk_head_linear", dtype_code(x.dtype), x.data_ptr(), x.stride(0), w.data_ptr(), y.data_ptr(), y.stride(0),
             1 if (out_f32 and x.dtype != torch.float32) else 0, x.shape[0], heads, n_in, n_out, _stream())
    return y


def expert_route(h: torch.Tensor, w_router: torch.Tensor, correction: torch.Tensor, groups: int, keep: int, top: int,
                 w_gate: torch.Tensor | None = None, normalize_scale: float | None = None,
                 unit_gate: bool = False) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor | None]:
    """The router of a mixture of experts, 32-bit arithmetic: logits ``w_router h`` over all
    experts, their softmax s, the choice by ``s + correction`` among the experts of the ``keep``
    groups of neighbours (of ``groups`` equal ones) whose best choice score is largest, ties to the
    left.  Returns ids [tokens, top] int32 in the order of the choice scores, weights [tokens, top]
    (the chosen experts' s), and, with ``w_gate`` [width], sigmoid(w_gate . h) [tokens].  ``normalize_scale``: the
    weights are divided by their sum (+ 1e-20) and multiplied by this number.  ``unit_gate`` (without ``w_gate``): the
    third result is a gate of ones, for a shared expert that is added as it is."""
    _gpu(h, w_router, correction, w_gate)
    n_all, width = w_router.shape
    _need(h.dim() == 2 and h.stride(1) == 1 and h.shape[1] == width and w_router.dtype == h.dtype and w_router.is_contiguous(),
          "expert_route: rows [tokens, width] and a contiguous router [experts, width] of one type")
    _f32_vector(correction, n_all, "expert_route: the correction")
    _need(w_gate is None or (w_gate.numel() == width and w_gate.dtype == h.dtype and w_gate.is_contiguous()),
          "expert_route: the shared expert's gate must be contiguous [width]")
    n = h.shape[0]
    ids = torch.empty((n, top), dtype=torch.int32, device=h.device)
    weights = torch.empty((n, top), dtype=torch.float32, device=h.device)
    gate = torch.empty((n,), dtype=torch.float32, device=h.device) if (w_gate is not None or unit_gate) else None
    if n == 0:
        return ids, weights, gate
    call("tk_expert_route", dtype_code(h.dtype), h.data_ptr(), h.stride(0), w_router.data_ptr(), correction.data_ptr(),
         w_gate.data_ptr() if w_gate is not None else None, n, width, n_all, int(groups), int(keep), int(top),
         ids.data_ptr(), weights.data_ptr(), gate.data_ptr() if gate is not None else None,
         float(normalize_scale) if normalize_scale else 0.0, _stream())
    return ids, weights, gate


def expert_mix(h: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor,
               shared: torch.Tensor | None = None, shared_gate: torch.Tensor | None = None) -> torch.Tensor:
    """The weighted sum of a token's chosen experts, 32-bit [tokens, width]: expert e is
    ``w_down[e] (silu(gate) * up)`` with [gate | up] = ``w_gate_up[e] h``; an id from
    ``len(w_down)`` on names an identity expert (its output is h), a negative id an empty
    place.  ``shared`` (32-bit [tokens, width]) times ``shared_gate`` [tokens] is added."""
    _gpu(h, w_gate_up, w_down, ids, weights, shared, shared_gate)
    experts, two_ff, width = w_gate_up.shape
    ff = two_ff // 2
    _need(w_gate_up.is_contiguous() and w_down.is_contiguous() and w_down.shape == (experts, width, ff)
          and w_gate_up.dtype == h.dtype and w_down.dtype == h.dtype, "expert_mix: weights [experts, 2 ff, width] and [experts, width, ff] of the rows' type")
    _need(h.dim() == 2 and h.stride(1) == 1 and h.shape[1] == width, "expert_mix: rows [tokens, width]")
    n = h.shape[0]
    _i32(ids, "ids")
    top = ids.shape[1]
    _need(ids.shape == (n, top) and weights.shape == (n, top) and weights.dtype == torch.float32 and weights.is_contiguous(),
          "expert_mix: ids and weights [tokens, top]")
    if shared is not None:
        _need(shared.shape == (n, width) and shared.dtype == torch.float32 and shared.is_contiguous(), "expert_mix: the shared expert's rows must be float32 [tokens, width]")
        _f32_vector(shared_gate, n, "expert_mix: the shared expert's gate")
    out = torch.empty((n, width), dtype=torch.float32, device=h.device)
    if n == 0:
        return out
    if n > GROUPED_FROM_ROWS and _grouped_takes(h, w_gate_up, width) and ff % 8 == 0 and w_down.data_ptr() % 16 == 0:
        # many tokens: the pairs sorted by expert, every expert's rows in tiles on the matrix cores
        max_tiles = -(-(n * top) // GROUPED_TILE) + experts
        slots = max_tiles * GROUPED_TILE
        book = torch.empty((2 * slots + max_tiles,), dtype=torch.int32, device=h.device)
        slot_pair, slot_token, tile_group = book[:slots], book[slots : 2 * slots], book[2 * slots :]
        call("tk_expert_sort", ids.data_ptr(), n * top, top, experts, max_tiles, slot_pair.data_ptr(), slot_token.data_ptr(),
             tile_group.data_ptr(), _stream())
        inter = torch.empty((slots, ff), dtype=h.dtype, device=h.device)
        call("tk_grouped_gemm_bf16", h.data_ptr(), h.stride(0), slot_token.data_ptr(), None, tile_group.data_ptr(), max_tiles, 0,
             0, 0, w_gate_up.data_ptr(), 2 * ff * width, inter.data_ptr(), ff, ff, width, slots, 1, 0, _stream())
        y = torch.empty((n * top, width), dtype=h.dtype, device=h.device)
        call("tk_grouped_gemm_bf16", inter.data_ptr(), ff, None, slot_pair.data_ptr(), tile_group.data_ptr(), max_tiles, 0,
             0, 0, w_down.data_ptr(), width * ff, y.data_ptr(), width, width, ff, slots, 0, 0, _stream())
        call("tk_expert_sum", h.data_ptr(), h.stride(0), y.data_ptr(), ids.data_ptr(), weights.data_ptr(),
             shared.data_ptr() if shared is not None else None, shared_gate.data_ptr() if shared is not None else None,
             out.data_ptr(), n, width, experts, top, _stream())
        return out
    inter = torch.empty((n * top, ff), dtype=h.dtype, device=h.device)
    call("tk_expert_gate_up", dtype_code(h.dtype), h.data_ptr(), h.stride(0), w_gate_up.data_ptr(), ids.data_ptr(),
         inter.data_ptr(), n, width, ff, experts, top, _stream())
    call("tk_expert_combine", dtype_code(h.dtype), h.data_ptr(), h.stride(0), inter.data_ptr(), w_down.data_ptr(),
         ids.data_ptr(), weights.data_ptr(), shared.data_ptr() if shared is not None else None,
         shared_gate.data_ptr() if shared is not None else None, out.data_ptr(), n, width, ff, experts, top, _stream())
    return out
