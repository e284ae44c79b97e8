"""The operations the parts call.  Each wrapper checks shapes, dtypes and
contiguity on the host, then launches the HIP kernel on the current stream.
Tensors are torch tensors on the GPU; torch only provides the memory and the
stream here, every computation is the library's.
"""
from __future__ import annotations

import ctypes

import torch

from . import lib
from .lib import KernelError

_DT = {torch.float32: 0, torch.bfloat16: 1}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype}") from None


_DEVICE = None


def _stream():
    """The current stream's handle (asked for at every launch: under graph capture it is another one).
    torch's own accessor for the raw handle: `torch.cuda.current_stream()` builds a Python object
    and took 9 us a launch, a quarter of the host's time in a step that is not replayed from a graph."""
    global _DEVICE
    if _DEVICE is None:
        _DEVICE = torch.cuda.current_device()
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is None:
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return ctypes.c_void_p(raw(_DEVICE))


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _check(cond, msg):
    if not cond:
        raise KernelError(msg)


def _gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("the kernels take GPU tensors; there is no CPU path")


def _rows2d(t: torch.Tensor, what: str):
    """A 2-D tensor whose rows are contiguous: (rows, cols, leading dimension)."""
    _check(t.dim() == 2 and t.stride(1) == 1, f"{what}: expected a 2-D tensor with contiguous rows")
    return t.shape[0], t.shape[1], t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t, what, n=None):
    _check(t.dtype == torch.int32 and t.is_contiguous(), f"{what}: expected a contiguous int32 tensor")
    if n is not None:
        _check(t.numel() >= n, f"{what}: {t.numel()} entries, {n} needed")


# ------------------------------------------------------------------ simple ops

def embed(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, emit: dict | None = None):
    """out[i, :] = table[ids[i], :] as float32.

    emit: dict(weight, out, shares) as for `linear_fused`: the first half of the norm that
    follows, bfloat16(out * weight) into emit["out"] and the rows' sums of squares in
    `embed_emit_blocks(width)` shares of 64 floats into emit["shares"] (`can_embed_emit` says
    for which tables and rows)."""
    _gpu(out, table, ids)
    n, d, _ = _rows2d(out, "embed out")
    _check(out.dtype == torch.float32 and out.is_contiguous(), "embed: out must be contiguous float32")
    _check(table.dim() == 2 and table.is_contiguous() and table.shape[1] == d, "embed: table shape")
    _i32(ids, "embed ids", n)
    if emit is None:
        lib.core().call("hfee_embed", _ptr(out), _ptr(table), _dt(table), _ptr(ids), n, d, _stream())
        return
    eo, es, ew = emit["out"], emit["shares"], emit["weight"]
    _gpu(eo, es, ew)
    _check(can_embed_emit(table, n), "embed: the norm's first half only with a bfloat16 table of a width that is a "
           "multiple of 8, for at most 64 rows")
    Me, Ne, lde = _rows2d(eo, "embed emit out")
    _check(eo.dtype == torch.bfloat16 and Me >= n and Ne == d, "embed: emit out must be bfloat16 [n, width]")
    _check(ew.numel() == d and ew.is_contiguous(), "embed: emit weight")
    _check(es.dtype == torch.float32 and es.is_contiguous() and es.numel() >= embed_emit_blocks(d) * SS_STRIDE,
           "embed: the shares need embed_emit_blocks(width) * 64 float32")
    lib.core().call("hfee_embed_emit", _ptr(out), _ptr(table), _ptr(ids), n, d, _ptr(ew), _dt(ew), _ptr(eo), lde,
                    _ptr(es), es.numel(), _stream())


EMBED_COLUMNS_A_WORKGROUP = 2048     # of a row, in the embedding kernels for bfloat16 tables


def can_embed_emit(table: torch.Tensor, n: int) -> bool:
    return table.dtype == torch.bfloat16 and table.shape[1] % 8 == 0 and n <= SS_STRIDE


def embed_emit_blocks(width: int) -> int:
    """Shares of a row's sum of squares that `embed(..., emit=...)` leaves."""
    return (width + EMBED_COLUMNS_A_WORKGROUP - 1) // EMBED_COLUMNS_A_WORKGROUP


def rmsnorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float, rows: torch.Tensor | None = None):
    """out[r] = x[rows[r] or r] / sqrt(mean(x^2) + eps) * weight; x float32."""
    _gpu(out, x, weight, rows)
    n, d, _ = _rows2d(out, "rmsnorm out")
    _check(out.is_contiguous() and x.is_contiguous() and x.dtype == torch.float32, "rmsnorm: contiguous float32 x")
    _check(x.dim() == 2 and x.shape[1] == d, "rmsnorm: width mismatch")
    _check(weight.numel() == d and weight.is_contiguous(), "rmsnorm: weight width mismatch")
    if rows is None:
        _check(x.shape[0] >= n, "rmsnorm: fewer input rows than output rows")
    else:
        _i32(rows, "rmsnorm rows", n)
    lib.core().call("hfee_rmsnorm", _ptr(out), _dt(out), _ptr(x), _ptr(weight), _dt(weight), _ptr(rows),
                    float(eps), n, d, _stream())


def cast_rows(out: torch.Tensor, x: torch.Tensor, rows: torch.Tensor | None = None):
    """out[r] = x[rows[r] or r] in out's type; x float32.  (What a model without a norm at some place
    has there.)"""
    _gpu(out, x, rows)
    n, d, _ = _rows2d(out, "cast_rows out")
    _check(out.is_contiguous() and x.is_contiguous() and x.dtype == torch.float32, "cast_rows: contiguous float32 x")
    _check(x.dim() == 2 and x.shape[1] == d, "cast_rows: width mismatch")
    if rows is None:
        _check(x.shape[0] >= n, "cast_rows: fewer input rows than output rows")
    else:
        _i32(rows, "cast_rows rows", n)
    lib.core().call("hfee_cast_rows", _ptr(out), _dt(out), _ptr(x), _ptr(rows), n, d, _stream())


# the activations of a gated feed-forward's gate, as the kernels number them (GATE_SILU ... in csrc/common.h)
GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "gelu": 2, "relu": 3}


def gate_activation(name: str) -> int:
    if name not in GATE_ACTIVATIONS:
        raise KernelError(f"unknown gate activation {name!r}: the kernels have {sorted(GATE_ACTIVATIONS)}")
    return GATE_ACTIVATIONS[name]


def swiglu(out: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, activation: str = "silu"):
    """out = activation(gate) * up ("silu": gate / (1 + exp(-gate))).  gate and up are views of one
    buffer with the same row and column strides (column stride 1: two blocks; 2: alternating columns)."""
    act = gate_activation(activation)
    _gpu(out, gate, up)
    n, w, ldo = _rows2d(out, "swiglu out")
    _check(gate.dim() == 2 and up.dim() == 2 and tuple(gate.shape) == (n, w) == tuple(up.shape), "swiglu: shape mismatch")
    _check(gate.stride() == up.stride() and gate.stride(1) >= 1, "swiglu: gate and up must share their strides")
    _check(out.dtype == gate.dtype == up.dtype, "swiglu: dtype mismatch")
    ld = gate.stride(0) if n > 1 else max(gate.stride(0), (w - 1) * gate.stride(1) + 1)
    lib.core().call("hfee_swiglu", _ptr(out), ldo, _ptr(gate), _ptr(up), ld, gate.stride(1), _dt(out), n, w, act, _stream())


def random_fill(out: torch.Tensor, key: int, kind: str, std: float = 1.0, bound: int = 0):
    """Fills `out` with element i = f(key, i): kind "normal" (N(0, std)), "one_plus_normal"
    (1 + N(0, std)) into a float32 or bfloat16 tensor, "integers" (in [0, bound)) into an int32
    tensor.  The host twin is weights/random_stream.py: the same bits."""
    _gpu(out)
    _check(out.is_contiguous(), "random_fill: the tensor must be contiguous")
    if kind == "integers":
        _check(out.dtype == torch.int32, "random_fill: integers go into an int32 tensor")
        lib.core().call("hfee_random_fill", _ptr(out), 0, out.numel(), key, 2, 0.0, int(bound), _stream())
        return
    _check(kind in ("normal", "one_plus_normal"), f"random_fill: unknown kind {kind!r}")
    lib.core().call("hfee_random_fill", _ptr(out), _dt(out), out.numel(), key, 1 if kind == "one_plus_normal" else 0,
                    float(std), 0, _stream())


def residual_add(x: torch.Tensor, y: torch.Tensor):
    """x (float32) += y."""
    _gpu(x, y)
    _check(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous(), "residual_add: contiguity")
    _check(x.shape == y.shape, "residual_add: shape mismatch")
    lib.core().call("hfee_residual_add", _ptr(x), _ptr(y), _dt(y), x.numel(), _stream())


def read_stream(t: torch.Tensor, workgroups: int = 2048, keep_out_of_l2: bool = False):
    """Reads every byte of t once and keeps nothing: the read-only yardstick of the memory,
    and a prefetch (what is read stays in the memory-side cache for the kernel that comes
    for it next; keep_out_of_l2 for a prefetch that runs beside another kernel)."""
    _gpu(t)
    _check(t.is_contiguous(), "read_stream: a contiguous tensor expected")
    nbytes = t.numel() * t.element_size()
    _check(nbytes % 16 == 0 and t.data_ptr() % 16 == 0, "read_stream: 16-byte alignment expected")
    lib.core().call("hfee_read_stream", _ptr(t), nbytes, None, int(workgroups), int(keep_out_of_l2), _stream())


def mfma_loop(iterations: int, workgroups: int) -> float:
    """Launches a loop of nothing but bfloat16 matrix instructions; returns the flops it does."""
    lib.core().call("hfee_mfma_loop", None, int(iterations), int(workgroups), _stream())
    return float(workgroups) * 4 * iterations * 64 * 2 * 16 * 16 * 32


# ---------------------------------------------------------------- matrix product

def linear_scratch(m: int, n: int, k: int) -> int:
    """float32 words of scratch that `linear` can use for a bfloat16 product of m rows with an
    [n, k] weight (0: none): with too few tiles for the chip, K is cut over more workgroups,
    which leave their partial products there for a second kernel to add up."""
    return int(lib.core().raw("hfee_gemm_bf16_scratch")(int(m), int(n), int(k)))


def linear_cuts(x: torch.Tensor, weight: torch.Tensor, scratch) -> int:
    """x @ weight.T (bfloat16) cut along K over workgroups, the partial products left in scratch
    as that many float32 matrices [M, N] one after the other, for a kernel that adds them up on
    its way (`rope_cache_write_cuts`).  Returns the number of cuts; 0 (and nothing launched)
    where the product is not one that is cut (`linear_scratch`) or scratch is missing."""
    if scratch is None:
        return 0
    _gpu(x, weight, scratch)
    M, K, lda = _rows2d(x, "linear_cuts x")
    N, Kw, ldw = _rows2d(weight, "linear_cuts weight")
    _check(x.dtype == weight.dtype == torch.bfloat16 and Kw == K, "linear_cuts: bfloat16 x and weight of one width")
    _check(scratch.dtype == torch.float32 and scratch.is_contiguous(), "linear_cuts: float32 scratch expected")
    cuts = ctypes.c_int(0)
    lib.core().call("hfee_gemm_bf16_cuts", _ptr(x), lda, _ptr(weight), ldw, M, N, K, _ptr(scratch), scratch.numel(),
                    ctypes.byref(cuts), _stream())
    return cuts.value


def rope_cache_write_cuts(q, partial, cuts: int, positions, token_segment, block_tables, cos, sin, cache_layer,
                          num_heads: int, kv_heads: int, head_dim: int, page_size: int, max_position: int,
                          portions: bool = True):
    """`rope_cache_write` for q, k and v that lie as the `cuts` partial products of `linear_cuts`
    ([n, (num_heads + 2 kv_heads) * head_dim] float32 each): they are added up in their order and
    rounded to bfloat16, rotated (adjacent pairs), q written to `q` (bfloat16 [n, num_heads *
    head_dim], any leading dimension), k and v into the pages of `cache_layer` (bfloat16)."""
    _gpu(q, partial, positions, cos, sin, cache_layer)
    n, wq, ldq = _rows2d(q, "rope q")
    _check(wq == num_heads * head_dim and q.dtype == torch.bfloat16 and cache_layer.dtype == torch.bfloat16,
           "rope_cache_write_cuts: bfloat16 q of num_heads * head_dim columns and a bfloat16 cache")
    _check(partial.dtype == torch.float32 and partial.is_contiguous() and
           partial.numel() >= cuts * n * (num_heads + 2 * kv_heads) * head_dim, "rope_cache_write_cuts: partial products too short")
    _check(cache_layer.is_contiguous() and cache_layer.dim() == 4 and
           tuple(cache_layer.shape[1:]) == (2, kv_heads, page_size * head_dim), "rope: cache layer shape")
    _i32(token_segment, "rope token_segment", n)
    _i32(positions, "rope positions", n)
    _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1, "rope: block tables")
    half = table_positions = 0
    if cos is not None:
        _check(cos.shape == sin.shape and cos.dim() == 2 and cos.is_contiguous() and sin.is_contiguous()
               and cos.dtype == sin.dtype == torch.float32, "rope: cos/sin tables")
        table_positions, half = cos.shape
    lib.core().call("hfee_rope_cache_write_cuts", _ptr(q), ldq, _ptr(partial), int(cuts), _ptr(positions),
                    _ptr(token_segment), _ptr(block_tables), block_tables.stride(0), _ptr(cos), _ptr(sin), half,
                    table_positions, max_position, _ptr(cache_layer), num_heads, kv_heads, head_dim, page_size, n,
                    1 if portions else 0, _stream())


def linear_add_norm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, normed: torch.Tensor,
                    norm_weight: torch.Tensor, eps: float, scratch=None):
    """out (float32, the residual stream) += x @ weight.T, and normed (bfloat16) = the RMS norm of the
    new rows of out times norm_weight.  bfloat16 x and weight.  Where the product's K is cut over
    workgroups (`linear_scratch` > 0 and scratch given) the kernel that adds the partial products
    up does the norm as well; otherwise it is the product and the norm, one after the other."""
    _gpu(out, x, weight, normed, norm_weight)
    M, K, lda = _rows2d(x, "linear_add_norm x")
    N, Kw, ldw = _rows2d(weight, "linear_add_norm weight")
    _check(x.dtype == weight.dtype == torch.bfloat16 and out.dtype == torch.float32 and normed.dtype == torch.bfloat16,
           "linear_add_norm: bfloat16 x, weight and normed, float32 out")
    _check(Kw == K and tuple(out.shape) == (M, N) == tuple(normed.shape) and out.is_contiguous() and normed.is_contiguous(),
           f"linear_add_norm: shapes x{list(x.shape)} w{list(weight.shape)} out{list(out.shape)} normed{list(normed.shape)}")
    _check(norm_weight.numel() == N and norm_weight.is_contiguous() and norm_weight.dtype in (torch.float32, torch.bfloat16),
           "linear_add_norm: the norm's weight must have the width of out, float32 or bfloat16")
    if scratch is not None:
        _gpu(scratch)
        _check(scratch.dtype == torch.float32 and scratch.is_contiguous(), "linear_add_norm: float32 scratch expected")
    lib.core().call("hfee_gemm_bf16_add_norm", _ptr(out), _ptr(x), lda, _ptr(weight), ldw, M, N, K, _ptr(scratch),
                    0 if scratch is None else scratch.numel(), _ptr(normed), _ptr(norm_weight),
                    1 if norm_weight.dtype == torch.float32 else 0, float(eps), _stream())


def linear(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, accumulate: bool = False, kernel: int = 0,
           gate: bool = False, scratch=None, activation: str = "silu"):
    """out (+)= x @ weight.T, weight stored [out_features, in_features].
    scratch (bfloat16 products): float32, `linear_scratch(M, N, K)` words, or None.

    float32 x and weight: the true 32-bit product, out float32.
    bfloat16 x and weight: matrix cores with float32 accumulation; out bfloat16, or
    float32 (required when accumulating: the residual stream).
    gate (bfloat16, aligned shapes): the rows of weight alternate gate/up and
    out[m, j] = activation(row 2j) * row 2j+1, out [M, N/2].
    kernel (bfloat16 only): 0 automatic, 1 skinny, 2 tiled 128x128, 3 the simple tiled
    kernel, 4 tiled 256x256, 5 tiled 256x128, 6 tiled 256x192, 7 and 8 tiled 128x128 and 128x192
    loaded straight into LDS."""
    _gpu(out, x, weight)
    M, K, lda = _rows2d(x, "linear x")
    N, Kw, ldw = _rows2d(weight, "linear weight")
    Mo, No, ldc = _rows2d(out, "linear out")
    _check(Kw == K and Mo == M and No == (N // 2 if gate else N),
           f"linear: shapes x{list(x.shape)} w{list(weight.shape)} out{list(out.shape)}")
    if gate:
        _check(x.dtype == weight.dtype == out.dtype == torch.bfloat16 and not accumulate and N % 2 == 0,
               "linear: the gate epilogue takes bfloat16 operands and an even number of weight rows")
        lib.core().call("hfee_gemm_bf16", _ptr(out), 3, ldc, _ptr(x), lda, _ptr(weight), ldw, M, N, K, kernel,
                        None, 0, gate_activation(activation), _stream())
        return
    _check(x.dtype == weight.dtype, "linear: x and weight dtypes differ")
    if x.dtype == torch.float32:
        _check(out.dtype == torch.float32, "linear: float32 product needs a float32 out")
        lib.core().call("hfee_gemm_f32", _ptr(out), ldc, _ptr(x), lda, _ptr(weight), ldw, M, N, K,
                        1 if accumulate else 0, _stream())
    elif x.dtype == torch.bfloat16:
        if accumulate:
            _check(out.dtype == torch.float32, "linear: accumulation needs a float32 out")
            mode = 2
        else:
            mode = 0 if out.dtype == torch.bfloat16 else 1
            _check(out.dtype in (torch.bfloat16, torch.float32), "linear: out dtype")
        if scratch is not None:
            _gpu(scratch)
            _check(scratch.dtype == torch.float32 and scratch.is_contiguous(), "linear: float32 scratch expected")
        lib.core().call("hfee_gemm_bf16", _ptr(out), mode, ldc, _ptr(x), lda, _ptr(weight), ldw, M, N, K,
                        kernel, _ptr(scratch), 0 if scratch is None else scratch.numel(), 0, _stream())
    else:
        raise KernelError(f"linear: unsupported dtype {x.dtype}")


def tiled_plan(m: int, n: int, k: int) -> tuple:
    """(kernel of the first n1 weight rows, n1, kernel of the rest or 0): how `linear`
    lays an aligned bfloat16 product of more than 64 rows over the tiled kernels."""
    import ctypes
    first, n1, second = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    lib.core().call("hfee_gemm_bf16_plan", m, n, k, ctypes.byref(first), ctypes.byref(n1), ctypes.byref(second))
    return first.value, n1.value, second.value


# --------------------------------------------------------- rotation and the cache

def rope_cache_write(q, k, v, positions, token_segment, block_tables, cos, sin, pairing: int,
                     cache_layer, num_heads: int, kv_heads: int, head_dim: int, page_size: int,
                     max_position: int, portions: bool = True):
    """Rotates q in place, writes rotated k and v into the pages of `cache_layer`.
    portions: the tokens hold runs of consecutive positions (portions of prompts); False for
    single tokens of many sequences, whose values are then written by each token's own workgroup.
    q, k, v: 2-D views [n, heads * head_dim] (any leading dimension), or None.
    cos/sin: [positions, half] float32 or None (no rotation).  cache_layer:
    [pages, 2, kv_heads, page_size * head_dim] or None (no write)."""
    _gpu(q, k, v, positions, cos, sin, cache_layer)
    some = q if q is not None else k
    _check(some is not None, "rope_cache_write: nothing to do")
    n = some.shape[0]
    ldq = ldk = ldv = 0
    if q is not None:
        nq, wq, ldq = _rows2d(q, "rope q")
        _check(nq == n and wq == num_heads * head_dim, "rope: q shape")
    if k is not None:
        _check(v is not None and cache_layer is not None, "rope: k, v and the cache come together")
        nk, wk, ldk = _rows2d(k, "rope k")
        nv, wv, ldv = _rows2d(v, "rope v")
        _check(nk == n and nv == n and wk == wv == kv_heads * head_dim, "rope: k/v shape")
        _check(k.dtype == v.dtype == cache_layer.dtype and (q is None or q.dtype == k.dtype), "rope: dtype mismatch")
        _check(cache_layer.is_contiguous() and cache_layer.dim() == 4 and
               tuple(cache_layer.shape[1:]) == (2, kv_heads, page_size * head_dim), "rope: cache layer shape")
        _i32(token_segment, "rope token_segment", n)
        _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
               "rope: block tables")
    _i32(positions, "rope positions", n)
    half = 0
    table_positions = 0
    if cos is not None:
        _check(cos.shape == sin.shape and cos.dim() == 2 and cos.is_contiguous() and sin.is_contiguous()
               and cos.dtype == sin.dtype == torch.float32, "rope: cos/sin tables")
        table_positions, half = cos.shape
    lib.core().call("hfee_rope_cache_write", _ptr(q), ldq, _ptr(k), ldk, _ptr(v), ldv, _dt(some),
                    _ptr(positions), _ptr(token_segment if k is not None else None),
                    _ptr(block_tables if k is not None else None),
                    block_tables.stride(0) if k is not None else 0,
                    _ptr(cos), _ptr(sin), half, pairing, table_positions, max_position,
                    _ptr(cache_layer if k is not None else None), num_heads, kv_heads, head_dim, page_size,
                    n, int(portions), _stream())


def attention_plain(out, q, cache_layer, positions, token_segment, block_tables, num_heads: int,
                    kv_heads: int, head_dim: int, page_size: int, scale: float, window: int = 0):
    """One wave per (token, head): the 32-bit path's attention and the slow twin of
    the matrix-core kernels.  Token t reads keys max(0, pos-window+1)..pos of its
    segment's pages."""
    _gpu(out, q, cache_layer, positions, token_segment, block_tables)
    n, w, ldq = _rows2d(q, "attention q")
    no, wo, ldo = _rows2d(out, "attention out")
    _check(no == n and wo == w == num_heads * head_dim, "attention: q/out shape")
    _check(q.dtype == out.dtype == cache_layer.dtype, "attention: dtype mismatch")
    _check(cache_layer.is_contiguous() and tuple(cache_layer.shape[1:]) == (2, kv_heads, page_size * head_dim),
           "attention: cache layer shape")
    _i32(positions, "attention positions", n)
    _i32(token_segment, "attention token_segment", n)
    _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
           "attention: block tables")
    lib.core().call("hfee_attention_ref", _ptr(out), ldo, _ptr(q), ldq, _ptr(cache_layer), _dt(q),
                    _ptr(positions), _ptr(token_segment), _ptr(block_tables), block_tables.stride(0),
                    num_heads, kv_heads, head_dim, page_size, float(scale), int(window), n, _stream())


# ------------------------------------------------------------------- sampling

ARGMAX_PARTS = 64


def argmax(out: torch.Tensor, logits: torch.Tensor, partial=None, counters=None):
    """out[r] = id of the first maximum of logits[r].  partial (float32, rows x ARGMAX_PARTS x 2)
    and counters (int32 zeros, one a row; zero again afterwards) let the kernel spread a row
    over several workgroups."""
    _gpu(out, logits, partial, counters)
    rows, V, ld = _rows2d(logits, "argmax logits")
    _check(logits.dtype == torch.float32, "argmax: float32 logits")
    _i32(out, "argmax out", rows)
    if partial is not None or counters is not None:
        _check(partial is not None and counters is not None and partial.dtype == torch.float32
               and partial.is_contiguous() and counters.dtype == torch.int32 and counters.is_contiguous(),
               "argmax: float32 partial results and int32 counters go together")
    lib.core().call("hfee_argmax", _ptr(out), _ptr(logits), ld, rows, V, _ptr(partial),
                    0 if partial is None else partial.numel() // 2, _ptr(counters),
                    0 if counters is None else counters.numel(), _stream())


def sample(out: torch.Tensor, logits: torch.Tensor, params: torch.Tensor, history: torch.Tensor,
           scratch: torch.Tensor, latest=None):
    """out[r] = sampled id for row r; params is [rows, 12] int32 (see sampling/params.py).
    latest: int32 on the device, one id a row that the repeat penalty counts as the newest
    of the row's history (it may be `out` itself: it is read before `out` is written)."""
    _gpu(out, logits, params, history, scratch, latest)
    _, V, ld = _rows2d(logits, "sample logits")
    rows = params.shape[0]
    _check(logits.dtype == torch.float32 and scratch.dtype == torch.float32, "sample: float32 logits and scratch")
    _check(params.dtype == torch.int32 and params.is_contiguous() and params.dim() == 2 and params.shape[1] == 12,
           "sample: params must be [rows, 12] int32")
    rs, Vs, lds = _rows2d(scratch, "sample scratch")
    _check(rs >= rows and Vs >= V, "sample: scratch too small")
    _i32(out, "sample out", rows)
    _check(history.dtype == torch.int32 and history.is_contiguous(), "sample: history must be int32")
    if latest is not None:
        _i32(latest, "sample latest", rows)
    lib.core().call("hfee_sample", _ptr(out), _ptr(logits), ld, rows, V, _ptr(params), _ptr(history),
                    _ptr(latest), _ptr(scratch), lds, _stream())


# ------------------------------------------------- matrix-core attention (bfloat16)

def _attention_common(out, q, cache_layer, block_tables, num_heads, kv_heads, head_dim, page_size):
    _gpu(out, q, cache_layer, block_tables)
    n, w, ldq = _rows2d(q, "attention q")
    no, wo, ldo = _rows2d(out, "attention out")
    _check(no == n and wo == w == num_heads * head_dim, "attention: q/out shape")
    _check(q.dtype == out.dtype == cache_layer.dtype == torch.bfloat16, "attention: bfloat16 tensors expected")
    _check(cache_layer.is_contiguous() and tuple(cache_layer.shape[1:]) == (2, kv_heads, page_size * head_dim),
           "attention: cache layer shape")
    _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
           "attention: block tables")
    return n, ldq, ldo


def attention_run_tiles(head_dim: int) -> int:
    """The most row tiles that a run of `attention_bf16_prefill`'s `runs` may hold."""
    return int(lib.attention_bf16(head_dim).raw("hfee_attention_bf16_run_tiles")())


def attention_halves_fit(head_dim: int, heads_per_kv_head: int, cache_layer=None) -> bool:
    """Whether `attention_bf16_prefill(kernel=3)` takes this shape: a row tile's keys in two halves
    (and this cache layer, if one is given: that kernel reaches every page through a 32-bit offset)."""
    dll = lib.attention_bf16(head_dim)
    if cache_layer is not None and cache_layer.numel() * cache_layer.element_size() >= 1 << int(dll.raw("hfee_attention_bf16_layer_limit_log2")()):
        return False
    return heads_per_kv_head % 4 == 0 and bool(dll.raw("hfee_attention_bf16_halves")())


def prefill_attention_kernel(tiles, window: int, kv_heads: int, heads_per_kv_head: int, head_dim: int) -> int:
    """The `kernel` argument of `attention_bf16_prefill` for a step's row tiles (first row, rows,
    first position, block-table row), on the host.  A workgroup walks the key tiles of its row tile
    one after the other, and two workgroups share a CU: where the longest row tile has many more
    key tiles than a workgroup slot's share of all of them (a prompt read from its start: the last
    row tile of 2,048 tokens has 64, the share is 32), the kernel that walks a row tile's keys in
    two halves side by side is as long as half the longest (3); where the row tiles are alike (a
    portion deep in a long context) two independent workgroups a CU do better (0)."""
    if not tiles or not attention_halves_fit(head_dim, heads_per_kv_head):
        return 0
    steps = []
    for _, rows, pos, _ in tiles:
        first = (max(0, pos - window + 1) >> 5) if window > 0 else 0
        steps.append(((pos + rows - 1) >> 5) + 1 - first)
    share = sum(steps) * kv_heads * (heads_per_kv_head // 4) / (2 * compute_units())
    return 3 if max(steps) >= 4 and max(steps) > 1.4 * max(share, 1.0) else 0


def attention_runs(tiles, head_dim: int) -> list:
    """The runs of a step's row tiles, on the host: tiles is the list of (first row, rows, first
    position, block-table row) that `attention_bf16_prefill` takes; a run is (first tile, count) of
    tiles of one sequence whose rows and positions go on where the tile before ended, at most
    `attention_run_tiles` of them, every tile in exactly one run."""
    most = attention_run_tiles(head_dim)
    runs = []
    for t, (row, rows, pos, table) in enumerate(tiles):
        if runs and runs[-1][1] < most:
            first, count = runs[-1]
            prow, prows, ppos, ptable = tiles[first + count - 1]
            if ptable == table and prow + prows == row and ppos + prows == pos:
                runs[-1] = (first, count + 1)
                continue
        runs.append((t, 1))
    return runs


def attention_bf16_prefill(out, q, cache_layer, tiles, block_tables, num_heads: int, kv_heads: int,
                           head_dim: int, page_size: int, scale: float, window: int = 0, kernel: int = 0, runs=None):
    """tiles: [num_tiles, 4] int32 (first row, rows <= 32, first position, block-table row).
    kernel: 0 automatic, 1 one wave per (tile, head), 2 the heads of a KV head share its
    key tiles through LDS, 3 the same with a row tile's keys in two halves that eight waves
    walk side by side (four heads or a multiple to a KV head, head sizes up to 128).
    runs: [num_runs, 2] int32 (first tile, count <= attention_run_tiles) or None: every tile in
    exactly one run of tiles that follow one another in `tiles` and in one sequence, rows and
    positions going on where the tile before ended (`attention_runs` makes them; a longer run
    would leave row tiles without output).  For heads that share no keys with another head (kv_heads ==
    num_heads) the row tiles of a run then share the head's key tiles through LDS."""
    n, ldq, ldo = _attention_common(out, q, cache_layer, block_tables, num_heads, kv_heads, head_dim, page_size)
    _check(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous(),
           "attention: tiles must be [num_tiles, 4] int32")
    if runs is not None:
        _gpu(runs)
        _check(runs.dtype == torch.int32 and runs.dim() == 2 and runs.shape[1] == 2 and runs.is_contiguous() and runs.shape[0] > 0,
               "attention: runs must be [num_runs, 2] int32")
    lib.attention_bf16(head_dim).call(
        "hfee_attention_bf16_prefill", _ptr(out), ldo, _ptr(q), ldq, _ptr(cache_layer), cache_layer.shape[0], _ptr(tiles),
        tiles.shape[0], _ptr(runs), 0 if runs is None else runs.shape[0], _ptr(block_tables), block_tables.stride(0),
        num_heads, kv_heads, page_size, float(scale), int(window), int(kernel), _stream())


def attention_bf16_decode(out, q, cache_layer, seg_rows, seg_positions, seg_tables, block_tables,
                          num_heads: int, kv_heads: int, head_dim: int, page_size: int, scale: float,
                          window: int, partial, num_splits: int, waves: int = 4, counters=None):
    """One query token per listed segment.  A workgroup of `waves` waves (at most 4)
    shares the keys of one (segment, KV head, split) and joins them in LDS; with
    num_splits > 1 the splits are joined by a second kernel, or, given `counters` (at
    least segments x kv_heads int32 that are zero, and are zero again afterwards), by
    the workgroup of each (segment, KV head) that finishes last.  seg_rows or seg_tables
    None: segment i is row i of q and out, or has row i of block_tables (the kernel then
    reaches its first keys one load sooner)."""
    n, ldq, ldo = _attention_common(out, q, cache_layer, block_tables, num_heads, kv_heads, head_dim, page_size)
    count = seg_positions.numel()
    _i32(seg_positions, "attention seg_positions", count)
    if seg_rows is not None:
        _i32(seg_rows, "attention seg_rows", count)
    else:
        _check(count <= n, "attention: more segments than rows")
    if seg_tables is not None:
        _i32(seg_tables, "attention seg_tables", count)
    else:
        _check(count <= block_tables.shape[0], "attention: more segments than block tables")
    if num_splits > 1:
        _check(partial is not None and partial.dtype == torch.float32 and partial.is_contiguous(),
               "attention: float32 partial buffer expected")
    if counters is not None:
        _check(counters.dtype == torch.int32 and counters.is_contiguous() and counters.is_cuda,
               "attention: int32 counters expected")
    lib.attention_bf16(head_dim).call(
        "hfee_attention_bf16_decode", _ptr(out), ldo, _ptr(q), ldq, _ptr(cache_layer), _ptr(seg_rows),
        _ptr(seg_positions), _ptr(seg_tables), count, _ptr(block_tables), block_tables.stride(0),
        num_heads, kv_heads, page_size, float(scale), int(window), _ptr(partial),
        0 if partial is None else partial.numel(), int(num_splits), int(waves),
        _ptr(counters), 0 if counters is None else counters.numel(), _stream())


# ------------------------------------------------------- fused decode products (M <= 64)

SKINNY_MAX_ROWS = 64
FUSED_NORM_MAX_ROWS = 16
# folding the norm into the product makes every workgroup convert the activations
# itself; beyond this many weight rows a separate norm kernel is cheaper
FUSED_NORM_MAX_N = 8192
_cus = None


def compute_units() -> int:
    """CUs of the device (256 on an MI355X)."""
    global _cus
    if _cus is None:
        _cus = torch.cuda.get_device_properties(0).multi_processor_count
    return _cus


def norm_fusion_pays(n_rows: int, k: int) -> bool:
    """Whether folding the norm into a product with n_rows weight rows is cheaper than
    a norm kernel of its own: narrow products, and the wide ones that the persistent
    kernel takes (there the activations are converted once per workgroup)."""
    wide = n_rows > 16 * compute_units() and k % 1024 == 0 and k <= 4096
    return wide or n_rows <= FUSED_NORM_MAX_N
_EPI = {"bf16": 0, "f32": 1, "add": 2, "swiglu": 3, "qkv": 4}


class TiledWeight:
    """A bfloat16 weight [n, k] in tiles of 16 rows x 32 columns, the form that the products of
    up to 64 rows stream (`linear_fused`): a tile is a kilobyte in the order in which a wave
    holds it as a matrix operand ([column group of 8][row][8 columns]), the tiles of 16 rows
    follow one another along k, and n and k are filled up with zeros to whole tiles."""

    def __init__(self, tiles: torch.Tensor, n: int, k: int):
        self.tiles, self.n, self.k = tiles, n, k
        self.row_stride = ((k + 31) // 32) * 512          # elements from one row of tiles to the next

    @property
    def shape(self):
        return (self.n, self.k)

    def rows(self) -> torch.Tensor:
        """The weight as rows again, [n, k] (for tests)."""
        nt, kt = self.tiles.shape[0], self.tiles.shape[1]
        return self.tiles.view(nt, kt, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(nt * 16, kt * 32)[:self.n, :self.k]


def tile_weight(weight: torch.Tensor) -> TiledWeight:
    """weight [n, k] bfloat16 (rows as they lie in a checkpoint) -> the same in tiles."""
    _check(weight.dim() == 2 and weight.dtype == torch.bfloat16, "tile_weight: a 2-D bfloat16 weight expected")
    n, k = weight.shape
    nt, kt = (n + 15) // 16, (k + 31) // 32
    if nt * 16 != n or kt * 32 != k:
        padded = torch.zeros((nt * 16, kt * 32), dtype=weight.dtype, device=weight.device)
        padded[:n, :k] = weight
        weight = padded
    tiles = weight.view(nt, 16, kt, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(nt, kt, 512)
    return TiledWeight(tiles, n, k)


# The part of the device's memory that the second copies of the weights leave free (for the cache,
# the workspace, and whatever else the process holds).
TILES_LEAVE_FREE = 0.2


def tile_weights_if_room(*weights: torch.Tensor):
    """The weights' second copies in tiles (`tile_weight`), all of them or none: None where they
    would leave less than TILES_LEAVE_FREE of the device's memory free.  A model too large to lie
    in memory twice then has the layers that were bound last without tiles; their steps of at
    most 64 rows go through the kernels that read the rows as they lie."""
    device = weights[0].device
    if device.type == "cuda":
        free, total = torch.cuda.mem_get_info(device)
        if not room_for_tiles(sum(w.numel() * w.element_size() for w in weights), free, total):
            return None
    return tuple(tile_weight(w) for w in weights)


def room_for_tiles(need: int, free: int, total: int) -> bool:
    """Whether copies of `need` bytes leave TILES_LEAVE_FREE of the `total` bytes free, `free` being free now."""
    return free - need >= TILES_LEAVE_FREE * total


SS_STRIDE = 64     # rows of a table of sum-of-squares shares (one row of the table per 16 weight rows)


def mid_rows_scratch(n_rows: int, n_weight_rows: int, k: int) -> int:
    """float32 words of scratch that a product of 17 to 64 rows wants for its faster kernel
    (0: it has no use for scratch)."""
    if n_rows <= 16 or n_rows > SKINNY_MAX_ROWS or k % 256 or k <= 1024:
        return 0
    return ((n_weight_rows + 15) // 16) * ((k + 1023) // 1024) * ((n_rows + 15) // 16) * 256 + SS_STRIDE


def linear_fused(out, x, weight, epilogue: str, norm_weight=None, eps: float = 0.0, rows=None, m=None, qkv=None,
                 emit=None, row_scale=None, scratch=None, force_mid_rows=False):
    """out = epilogue(norm(x) @ weight.T) in one launch, for at most 64 rows; weight: a
    `TiledWeight`.  ("qkv" with a weight as rows [N, K]: any number of rows, through the tiled
    kernels with the same epilogue; nothing else is fused there.)

    emit (with "add"): dict(weight, out, shares): the norm that follows the residual add, in
    two halves: this product also writes bfloat16(out_new * weight) to emit["out"] [M, N] and
    its shares of the rows' sums of squares to emit["shares"] (float32, at least
    ceil(N / 16) * 64).  row_scale: dict(shares, blocks, eps): the other half: x is such an
    emitted tensor, and the finished sums are scaled by 1 / sqrt(sum of shares / K + eps).
    scratch (float32, `mid_rows_scratch` words): lets products of 17 to 64 rows over
    K % 256 == 0 take a kernel that keeps the batch in LDS and cuts K over workgroups, and a
    second one that adds the slices up, where that pays.  Products with weight rows enough to
    fill the chip take a kernel that cuts nothing and needs no scratch.  (force_mid_rows, for
    tests: 1 takes the first wherever it applies, 2 the second.)

    x: bfloat16 [M, K]; or, with norm_weight, the float32 residual stream (at most 16
    rows; `rows` optionally gathers them, then `m` is their number).
    epilogue: "bf16" | "f32" | "add" (out float32 += ...) | "swiglu" (weight rows
    alternate gate/up; out [M, N/2] = silu(gate) * up: the reference's activation; another one is
    "bf16" into [M, N] and `swiglu` over its alternating columns) | "qkv" (rotation + cache write; see
    parts/attention.py; qkv = dict(positions, token_segment, block_tables, cos, sin,
    cache_layer, num_heads, kv_heads, head_dim, page_size))."""
    if not isinstance(weight, TiledWeight):
        _check(epilogue == "qkv" and norm_weight is None and emit is None and row_scale is None,
               "linear_fused: the weight must be a TiledWeight (ops.tile_weight); only the plain q/k/v product "
               "takes a weight as rows")
        return _qkv_rows(out, x, weight, qkv)
    _gpu(out, x, weight.tiles, norm_weight, rows)
    N, K, ldw = weight.n, weight.k, weight.row_stride
    Mx, Kx, lda = _rows2d(x, "linear_fused x")
    M = Mx if m is None else m
    _check(Kx == K, "linear_fused: inner sizes differ")
    _check(M <= SKINNY_MAX_ROWS, f"linear_fused: at most {SKINNY_MAX_ROWS} rows, got {M}")
    weight = weight.tiles
    fused_norm = norm_weight is not None
    if fused_norm:
        _check(x.dtype == torch.float32 and M <= FUSED_NORM_MAX_ROWS, "linear_fused: the fused norm takes <= 16 float32 rows")
        _check(norm_weight.numel() == K and norm_weight.is_contiguous(), "linear_fused: norm weight width")
        if rows is not None:
            _i32(rows, "linear_fused rows", M)
    else:
        _check(x.dtype == torch.bfloat16 and rows is None, "linear_fused: bfloat16 x expected")
    Mo, No, ldc = _rows2d(out, "linear_fused out")
    _check(Mo >= M, "linear_fused: out has too few rows")
    epi = _EPI[epilogue]
    want = {"bf16": torch.bfloat16, "f32": torch.float32, "add": torch.float32, "swiglu": torch.bfloat16,
            "qkv": torch.bfloat16}[epilogue]
    _check(out.dtype == want, f"linear_fused: out must be {want} for {epilogue!r}")
    e_args = [None, 0, None, 0, None]
    if emit is not None:
        _gpu(emit["weight"], emit["out"], emit["shares"])
        _check(epilogue == "add" and not fused_norm, "linear_fused: only the accumulating product emits a norm")
        eo, es, ew = emit["out"], emit["shares"], emit["weight"]
        Me, Ne, lde = _rows2d(eo, "linear_fused emit out")
        _check(eo.dtype == torch.bfloat16 and Me >= M and Ne == N, "linear_fused: emit out must be bfloat16 [M, N]")
        _check(ew.numel() == N and ew.is_contiguous() and ew.dtype in (torch.float32, torch.bfloat16),
               "linear_fused: emit weight")
        _check(es.dtype == torch.float32 and es.is_contiguous() and es.numel() >= ((N + 15) // 16) * SS_STRIDE,
               "linear_fused: the shares need ceil(N / 16) * 64 float32")
        e_args = [_ptr(ew), int(ew.dtype == torch.float32), _ptr(eo), lde, _ptr(es)]
    s_args = [None, 0, 0.0]
    if row_scale is not None:
        _gpu(row_scale["shares"])
        _check(not fused_norm, "linear_fused: a row scale and a fused norm exclude each other")
        ss, blocks = row_scale["shares"], int(row_scale["blocks"])
        _check(ss.dtype == torch.float32 and ss.is_contiguous() and blocks > 0 and ss.numel() >= blocks * SS_STRIDE,
               "linear_fused: row scale shares")
        s_args = [_ptr(ss), blocks, float(row_scale["eps"])]
    w_args = [None, 0, int(force_mid_rows)]
    if scratch is not None:
        _gpu(scratch)
        _check(scratch.dtype == torch.float32 and scratch.is_contiguous(), "linear_fused: float32 scratch expected")
        w_args = [_ptr(scratch), scratch.numel(), int(force_mid_rows)]
    q = qkv or {}
    if epilogue == "qkv":
        H, KV, hd, ps = q["num_heads"], q["kv_heads"], q["head_dim"], q["page_size"]
        _check(N == (H + 2 * KV) * hd and No == H * hd, "linear_fused: q/k/v shapes")
        cache = q.get("cache_layer")
        if cache is not None:
            _check(cache.is_contiguous() and tuple(cache.shape[1:]) == (2, KV, ps * hd) and cache.dtype == torch.bfloat16,
                   "linear_fused: cache layer shape")
            _i32(q["token_segment"], "linear_fused token_segment", M)
            bt = q["block_tables"]
            _check(bt.dtype == torch.int32 and bt.dim() == 2 and bt.stride(1) == 1, "linear_fused: block tables")
        _i32(q["positions"], "linear_fused positions", M)
        cos, sin = q.get("cos"), q.get("sin")
        half, table_positions = (cos.shape[1], cos.shape[0]) if cos is not None else (0, 0)
        bt = q.get("block_tables")
        lib.core().call("hfee_gemm_skinny", _ptr(out), ldc, _ptr(x), int(fused_norm), lda, _ptr(weight), ldw, M, N, K,
                        epi, _ptr(norm_weight), int(fused_norm and norm_weight.dtype == torch.float32), float(eps),
                        _ptr(rows), _ptr(q["positions"]), _ptr(q.get("token_segment")), _ptr(bt),
                        0 if bt is None else bt.stride(0), _ptr(cos), _ptr(sin), half, table_positions,
                        _ptr(cache), H, KV, hd, ps, *e_args, *s_args, *w_args, _stream())
        return
    _check(No == (N // 2 if epilogue == "swiglu" else N), "linear_fused: out width")
    lib.core().call("hfee_gemm_skinny", _ptr(out), ldc, _ptr(x), int(fused_norm), lda, _ptr(weight), ldw, M, N, K, epi,
                    _ptr(norm_weight), int(fused_norm and norm_weight.dtype == torch.float32), float(eps), _ptr(rows),
                    None, None, None, 0, None, None, 0, 0, None, 0, 0, 0, 0, *e_args, *s_args, *w_args, _stream())


def _qkv_rows(out, x, weight, q):
    """The q/k/v product with rotation and cache write for a weight as rows [N, K]."""
    _gpu(out, x, weight)
    N, K, ldw = _rows2d(weight, "linear_fused weight")
    M, Kx, lda = _rows2d(x, "linear_fused x")
    Mo, No, ldc = _rows2d(out, "linear_fused out")
    _check(Kx == K and Mo >= M, "linear_fused: shapes")
    _check(x.dtype == weight.dtype == out.dtype == torch.bfloat16, "linear_fused: bfloat16 tensors expected")
    H, KV, hd, ps = q["num_heads"], q["kv_heads"], q["head_dim"], q["page_size"]
    _check(N == (H + 2 * KV) * hd and No == H * hd, "linear_fused: q/k/v shapes")
    cache = q.get("cache_layer")
    if cache is not None:
        _check(cache.is_contiguous() and tuple(cache.shape[1:]) == (2, KV, ps * hd) and cache.dtype == torch.bfloat16,
               "linear_fused: cache layer shape")
        _i32(q["token_segment"], "linear_fused token_segment", M)
        bt = q["block_tables"]
        _check(bt.dtype == torch.int32 and bt.dim() == 2 and bt.stride(1) == 1, "linear_fused: block tables")
    _i32(q["positions"], "linear_fused positions", M)
    cos, sin = q.get("cos"), q.get("sin")
    half, table_positions = (cos.shape[1], cos.shape[0]) if cos is not None else (0, 0)
    bt = q.get("block_tables")
    lib.core().call("hfee_gemm_qkv_rows", _ptr(out), ldc, _ptr(x), lda, _ptr(weight), ldw, M, N, K,
                    _ptr(q["positions"]), _ptr(q.get("token_segment")), _ptr(bt), 0 if bt is None else bt.stride(0),
                    _ptr(cos), _ptr(sin), half, table_positions, _ptr(cache), H, KV, hd, ps, _stream())
