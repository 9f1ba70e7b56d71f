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

def embed(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, emit: dict | None = None, scale: float = 1.0):
    """out[i, :] = table[ids[i], :] * scale as float32.

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
        lib.core().call("hfee_embed", _ptr(out), _ptr(table), _dt(table), _ptr(ids), n, d, float(scale), _stream())
        return
    _check(scale == 1.0, "embed: a scaled lookup does not begin the norm that follows")
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


# ------------------------------- attention with keys and values of sizes of their own, and a sink

def _kv_cache(cache_layer, kv_heads, dk, dv, page_size, what):
    _check(cache_layer.is_contiguous() and cache_layer.dim() == 3 and
           tuple(cache_layer.shape[1:]) == (kv_heads, page_size * (dk + dv)),
           f"{what}: the cache layer must be [pages, kv_heads, page_size * (key size + value size)]")


def kv_write(q, k, v, positions, token_segment, block_tables, cos, sin, cache_layer, num_heads: int, kv_heads: int,
             q_dim: int, dk: int, dv: int, page_size: int, max_position: int, q_rot_offset: int = 0,
             k_rot_offset: int = 0, v_first=None, v_first_mode: int = 0, v_mix=None):
    """Rotates q in place and writes k (rotated) and v into the pages of `cache_layer`
    ([pages, kv_heads, page_size * (dk + dv)]: keys [slot][dk], then values [dv][slot]).
    q: [n, num_heads * q_dim] or None; k: [n, kv_heads * dk], v: [n, kv_heads * dv] or both None.
    The rotated dims of a q head are [q_rot_offset, q_rot_offset + 2 * half), of a k head
    [k_rot_offset, ...), pairs (i, i + half); cos/sin: float32 [positions, half] or None.
    v_first_mode 1: v is also copied to v_first ([n, kv_heads * dv], contiguous); 2: what is written
    is (1 - v_mix) v + v_mix v_first, v_mix a tensor of one element on the device."""
    _gpu(q, k, v, positions, cos, sin, cache_layer, v_first, v_mix)
    some = q if q is not None else k
    _check(some is not None, "kv_write: nothing to do")
    n = some.shape[0]
    ldq = ldk = ldv = 0
    if q is not None:
        nq, wq, ldq = _rows2d(q, "kv_write q")
        _check(nq == n and wq == num_heads * q_dim, "kv_write: q shape")
    if k is not None:
        _check(v is not None and cache_layer is not None, "kv_write: k, v and the cache come together")
        nk, wk, ldk = _rows2d(k, "kv_write k")
        nv, wv, ldv = _rows2d(v, "kv_write v")
        _check(nk == n and nv == n and wk == kv_heads * dk and wv == kv_heads * dv, "kv_write: k/v shape")
        _check(k.dtype == v.dtype == cache_layer.dtype and (q is None or q.dtype == k.dtype), "kv_write: dtype mismatch")
        _kv_cache(cache_layer, kv_heads, dk, dv, page_size, "kv_write")
        _i32(token_segment, "kv_write token_segment", n)
        _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
               "kv_write: block tables")
        if v_first_mode:
            _check(v_first is not None and v_first.is_contiguous() and v_first.dtype == v.dtype
                   and tuple(v_first.shape) == (n, kv_heads * dv), "kv_write: v_first must be [n, kv_heads * dv]")
        if v_first_mode == 2:
            _check(v_mix is not None and v_mix.numel() == 1 and v_mix.dtype == v.dtype, "kv_write: v_mix is one element")
    _i32(positions, "kv_write positions", n)
    half = table_positions = 0
    if cos is not None:
        _check(cos.shape == sin.shape and cos.dim() == 2 and cos.is_contiguous() and sin.is_contiguous()
               and cos.dtype == sin.dtype == torch.float32, "kv_write: cos/sin tables")
        table_positions, half = cos.shape
    has_k = k is not None
    lib.core().call("hfee_kv_write", _ptr(q), ldq, num_heads, q_dim, q_rot_offset, _ptr(k), ldk, k_rot_offset,
                    _ptr(v), ldv, _ptr(v_first if has_k else None), v_first_mode if has_k else 0,
                    _ptr(v_mix if has_k else None), _dt(some), _ptr(positions),
                    _ptr(token_segment if has_k else None), _ptr(block_tables if has_k else None),
                    block_tables.stride(0) if has_k else 0, _ptr(cos), _ptr(sin), half, table_positions,
                    int(max_position), _ptr(cache_layer if has_k else None), kv_heads, dk, dv, page_size, n, _stream())


KEY_WEIGHTS = {"softmax": 0, "sigmoid": 1}


def _sight(window: int, pool: int, softcap: float, pooled, pool_tables, cache_layer, segments: int, what: str):
    """(the pooled layer, its block tables, their row stride) for the entry points; pooled blocks are a cache layer of
    the tokens' shape and dtype with block tables of its own, a row a segment."""
    _check(window >= 0 and pool >= 0 and softcap >= 0, f"{what}: bad window, pool or softcap")
    if not (pool and window):
        return None, None, 0
    _check(pooled is not None and pool_tables is not None, f"{what}: pooled blocks need their cache layer and its block tables")
    _check(pooled.is_contiguous() and pooled.dtype == cache_layer.dtype and tuple(pooled.shape[1:]) == tuple(cache_layer.shape[1:]),
           f"{what}: the pooled layer must have the tokens' page shape and dtype")
    _check(pool_tables.dtype == torch.int32 and pool_tables.dim() == 2 and pool_tables.stride(1) == 1
           and pool_tables.shape[0] >= segments, f"{what}: the pooled layer's block tables")
    return pooled, pool_tables, pool_tables.stride(0)


def attention_kv_plain(out, q, cache_layer, positions, token_segment, block_tables, num_heads: int, kv_heads: int,
                       dk: int, dv: int, page_size: int, scale: float, sinks=None, weights: str = "softmax",
                       window: int = 0, pool: int = 0, softcap: float = 0.0, pooled=None, pool_tables=None, gate=None):
    """One wave per (token, head), any sizes, both dtypes: token t of head h reads the keys
    0..pos of its sequence; `sinks` (float32 [num_heads] or None) joins the softmax's denominator.
    weights "sigmoid": no softmax, a key weighs sigmoid(score + sinks[head]) and nothing is normalized.
    window > 0: only the last `window` positions, the token's own included; pool > 0: also one key and
    value (entry b of the cache layer `pooled`, which has block tables of its own, `pool_tables`) for every
    block b of `pool` positions that lies wholly before the window; softcap > 0: a score s counts as
    softcap * tanh(s / softcap).
    gate ([n, num_heads] in the tensors' dtype): head h's result is multiplied by sigmoid(gate[t, h])."""
    _check(weights in KEY_WEIGHTS, f"attention_kv: the weights are {sorted(KEY_WEIGHTS)}, not {weights!r}")
    _gpu(out, q, cache_layer, positions, token_segment, block_tables, sinks, gate, pooled, pool_tables)
    n, w, ldq = _rows2d(q, "attention_kv q")
    no, wo, ldo = _rows2d(out, "attention_kv out")
    _check(no == n and w == num_heads * dk and wo == num_heads * dv, "attention_kv: q/out shape")
    _check(q.dtype == out.dtype == cache_layer.dtype, "attention_kv: dtype mismatch")
    _kv_cache(cache_layer, kv_heads, dk, dv, page_size, "attention_kv")
    pooled, pool_tables, pool_stride = _sight(window, pool, softcap, pooled, pool_tables, cache_layer, block_tables.shape[0],
                                              "attention_kv")
    _i32(positions, "attention_kv positions", n)
    _i32(token_segment, "attention_kv token_segment", n)
    _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
           "attention_kv: block tables")
    if sinks is not None:
        _check(sinks.dtype == torch.float32 and sinks.is_contiguous() and sinks.numel() == num_heads,
               "attention_kv: sinks must be float32 [num_heads]")
    ldg = 0
    if gate is not None:
        ng, wg, ldg = _rows2d(gate, "attention_kv gate")
        _check(ng == n and wg == num_heads and gate.dtype == q.dtype, "attention_kv: gate [n, num_heads] in q's dtype")
    lib.core().call("hfee_attention_kv_plain", _ptr(out), ldo, _ptr(q), ldq, _ptr(cache_layer), _dt(q),
                    _ptr(positions), _ptr(token_segment), _ptr(block_tables), block_tables.stride(0),
                    num_heads, kv_heads, dk, dv, page_size, float(scale), _ptr(sinks), KEY_WEIGHTS[weights],
                    int(window), int(pool), float(softcap), _ptr(pooled), _ptr(pool_tables), pool_stride, _ptr(gate), ldg, n,
                    _stream())


def rotate_norm_write(q_out, q, k, v, positions, token_segment, block_tables, cos, sin, cache_layer, num_heads: int,
                      kv_heads: int, dk: int, dv: int, page_size: int, max_position: int, value_eps=None):
    """From float32 projections (behind a short convolution): q ([n, num_heads * dk]) rotated into q_out (the
    cache's dtype), k rotated and v into the token's slot of `cache_layer`, v divided by its root mean square
    over each head where value_eps is a number.  The first 2 * half dims of a head are rotated, pairs
    (i, i + half); cos/sin float32 [positions, half] or None.  k and v None: the queries only."""
    _gpu(q_out, q, k, v, positions, token_segment, block_tables, cos, sin, cache_layer)
    n, wq, ldq = _f32rows(q, "rotate_norm_write q")
    no, wo, ldqo = _rows2d(q_out, "rotate_norm_write q_out")
    _check(no == n and wq == wo == num_heads * dk, "rotate_norm_write: q shapes")
    _i32(positions, "rotate_norm_write positions", n)
    ldk = ldv = 0
    if k is not None:
        nk, wk, ldk = _f32rows(k, "rotate_norm_write k")
        nv, wv, ldv = _f32rows(v, "rotate_norm_write v")
        _check(nk == nv == n and wk == kv_heads * dk and wv == kv_heads * dv and q_out.dtype == cache_layer.dtype,
               "rotate_norm_write: k/v shapes, or the cache's dtype")
        _kv_cache(cache_layer, kv_heads, dk, dv, page_size, "rotate_norm_write")
        _i32(token_segment, "rotate_norm_write token_segment", n)
        _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
               "rotate_norm_write: block tables")
    half = table_positions = 0
    if cos is not None:
        _check(cos.shape == sin.shape and cos.dim() == 2 and cos.is_contiguous() and sin.is_contiguous()
               and cos.dtype == sin.dtype == torch.float32, "rotate_norm_write: cos/sin tables")
        table_positions, half = cos.shape
    has_k = k is not None
    lib.core().call("hfee_rotate_norm_write", _ptr(q_out), ldqo, _ptr(q), ldq, num_heads, _ptr(k), ldk, _ptr(v), ldv,
                    -1.0 if value_eps is None else float(value_eps), _dt(q_out), _ptr(cos), _ptr(sin), half, table_positions,
                    int(max_position), _ptr(positions), _ptr(token_segment if has_k else None),
                    _ptr(block_tables if has_k else None), block_tables.stride(0) if has_k else 0,
                    _ptr(cache_layer if has_k else None), kv_heads, dk, dv, page_size, n, _stream())


def kv_pool_write(cache_layer, pooled, pool: int, positions, token_segment, block_tables, pool_tables, kv_heads: int, dk: int,
                  dv: int, page_size: int):
    """Behind the launch that wrote a step's keys and values: every token at the last position of a block of
    `pool` positions leaves the means of the block's keys and values, as `cache_layer` holds them, in entry
    (position // pool) of the cache layer `pooled` (the tokens' page shape, block tables `pool_tables`)."""
    _gpu(cache_layer, pooled, positions, token_segment, block_tables, pool_tables)
    n = positions.numel()
    _check(pool >= 1, "kv_pool_write: a block holds at least one position")
    _kv_cache(cache_layer, kv_heads, dk, dv, page_size, "kv_pool_write")
    _i32(positions, "kv_pool_write positions", n)
    _i32(token_segment, "kv_pool_write token_segment", n)
    _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
           "kv_pool_write: block tables")
    pooled, pool_tables, pool_stride = _sight(1, pool, 0.0, pooled, pool_tables, cache_layer, block_tables.shape[0], "kv_pool_write")
    lib.core().call("hfee_kv_pool_write", _ptr(cache_layer), _ptr(pooled), _dt(cache_layer), int(pool), _ptr(positions),
                    _ptr(token_segment), _ptr(block_tables), block_tables.stride(0), _ptr(pool_tables), pool_stride, kv_heads, dk,
                    dv, page_size, n, _stream())


def qk_norm_write(q, k, v, positions, token_segment, block_tables, cache_layer, q_weight, k_weight, eps: float,
                  num_heads: int, kv_heads: int, dk: int, dv: int, page_size: int, temperature=None):
    """q (in place) and k (into the cache) are divided by their root mean square over each head and
    multiplied by q_weight / k_weight (float32 [dk], shared by the heads); v goes into the cache as it is.
    temperature (coef, every): q is also multiplied by 1 + coef * ln(floor((p + 1) / every) + 1) at
    position p.  k and v None: the queries only."""
    _gpu(q, k, v, positions, token_segment, block_tables, cache_layer, q_weight, k_weight)
    n, wq, ldq = _rows2d(q, "qk_norm_write q")
    _check(wq == num_heads * dk, "qk_norm_write: q width")
    _check(q_weight.dtype == torch.float32 and q_weight.is_contiguous() and q_weight.numel() == dk, "qk_norm_write: q_weight float32 [dk]")
    _i32(positions, "qk_norm_write positions", n)
    ldk = ldv = 0
    if k is not None:
        nk, wk, ldk = _rows2d(k, "qk_norm_write k")
        nv, wv, ldv = _rows2d(v, "qk_norm_write v")
        _check(nk == nv == n and wk == kv_heads * dk and wv == kv_heads * dv and k.dtype == v.dtype == q.dtype == cache_layer.dtype,
               "qk_norm_write: k/v shapes and dtypes")
        _check(k_weight is not None and k_weight.dtype == torch.float32 and k_weight.is_contiguous() and k_weight.numel() == dk,
               "qk_norm_write: k_weight float32 [dk]")
        _kv_cache(cache_layer, kv_heads, dk, dv, page_size, "qk_norm_write")
        _i32(token_segment, "qk_norm_write token_segment", n)
        _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1, "qk_norm_write: block tables")
    coef, every = (float(temperature[0]), int(temperature[1])) if temperature else (0.0, 0)
    _check(every >= 0, "qk_norm_write: the temperature's step must be positive")
    lib.core().call("hfee_qk_norm_write", _ptr(q), ldq, num_heads, _ptr(k), ldk, _ptr(v), ldv, _dt(q), _ptr(q_weight),
                    _ptr(k_weight), float(eps), coef, every, _ptr(positions), _ptr(token_segment), _ptr(block_tables),
                    block_tables.stride(0) if k is not None else 0, _ptr(cache_layer if k is not None else None),
                    kv_heads, dk, dv, page_size, n, _stream())


def attention_kv_sizes_fit(dk: int, dv: int) -> bool:
    """Whether the matrix-core kernels take these key and value sizes (else: the plain kernel)."""
    from . import build
    return dk % 16 == 0 and dv % 16 == 0 and 16 <= dk <= build.ATTENTION_KV_MOST[0] and 16 <= dv <= build.ATTENTION_KV_MOST[1]


def attention_kv_rows(dk: int, dv: int, heads_per_kv_head: int = 1, weights: str = "softmax") -> int:
    """The most rows that an item of `attention_kv_bf16`'s mode 0 may hold for these sizes and this
    many query heads a key/value head."""
    return int(lib.attention_kv_bf16(dk, dv, weights).raw("hfee_attention_kv_bf16_rows")(int(heads_per_kv_head)))


def attention_kv_partial_words(num_items: int, num_heads: int, dv: int, splits: int) -> int:
    return num_items * num_heads * splits * (4 + dv) if splits > 1 else 0


def attention_kv_bf16(out, q, cache_layer, items, mode: int, block_tables, num_heads: int, kv_heads: int, dk: int,
                      dv: int, page_size: int, scale: float, sinks=None, partial=None, splits: int = 1,
                      weights: str = "softmax", window: int = 0, pool: int = 0, softcap: float = 0.0, pooled=None,
                      pool_tables=None, gate=None):
    """Matrix-core attention, bfloat16 (weights: as in `attention_kv_plain`).  items: int32 [count, 4] on the device (first row, rows,
    first position, block-table row).  mode 0: an item is up to `attention_kv_rows` consecutive tokens of a portion;
    mode 1: an item is a single token (rows = 1), whose keys may be split over `splits` waves that
    leave partial results in `partial` (float32, `attention_kv_partial_words`) for a joining kernel.
    window, pool, softcap, pooled, pool_tables, gate: as in `attention_kv_plain`."""
    _gpu(out, q, cache_layer, items, block_tables, sinks, partial, gate, pooled, pool_tables)
    n, w, ldq = _rows2d(q, "attention_kv q")
    no, wo, ldo = _rows2d(out, "attention_kv out")
    _check(no == n and w == num_heads * dk and wo == num_heads * dv, "attention_kv: q/out shape")
    _check(q.dtype == out.dtype == cache_layer.dtype == torch.bfloat16, "attention_kv: bfloat16 tensors expected")
    _kv_cache(cache_layer, kv_heads, dk, dv, page_size, "attention_kv")
    pooled, pool_tables, pool_stride = _sight(window, pool, softcap, pooled, pool_tables, cache_layer, block_tables.shape[0],
                                              "attention_kv")
    ldg = 0
    if gate is not None:
        ng, wg, ldg = _rows2d(gate, "attention_kv gate")
        _check(ng == n and wg == num_heads and gate.dtype == torch.bfloat16, "attention_kv: gate bfloat16 [n, num_heads]")
    _check(items.dtype == torch.int32 and items.dim() == 2 and items.shape[1] == 4 and items.is_contiguous(),
           "attention_kv: items must be [count, 4] int32")
    _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
           "attention_kv: block tables")
    if sinks is not None:
        _check(sinks.dtype == torch.float32 and sinks.is_contiguous() and sinks.numel() == num_heads,
               "attention_kv: sinks must be float32 [num_heads]")
    if partial is not None:
        _check(partial.dtype == torch.float32 and partial.is_contiguous(), "attention_kv: float32 partial buffer expected")
    lib.attention_kv_bf16(dk, dv, weights).call(
        "hfee_attention_kv_bf16", _ptr(out), ldo, _ptr(q), ldq, _ptr(cache_layer), _ptr(items), items.shape[0], int(mode),
        _ptr(block_tables), block_tables.stride(0), num_heads, kv_heads, page_size, float(scale), _ptr(sinks),
        _ptr(partial), 0 if partial is None else partial.numel(), int(splits), int(window), int(pool), float(softcap),
        _ptr(pooled), _ptr(pool_tables), pool_stride, _ptr(gate), ldg, _stream())


def head_linear(out, x, weight, heads: int, n_in: int, n_out: int, tail: int = 0, x_head_stride: int | None = None,
                out_head_stride: int | None = None):
    """Per head: out[t, h, :n_out] = weight[h].T @ x[t, h, :n_in] (weight [heads, n_in, n_out]), then
    x[t, h, n_in : n_in + tail] copied behind.  x and out are 2-D with contiguous rows; a head's
    elements start every x_head_stride / out_head_stride (default: n_in + tail, n_out + tail)."""
    _gpu(out, x, weight)
    xs = n_in + tail if x_head_stride is None else x_head_stride
    os_ = n_out + tail if out_head_stride is None else out_head_stride
    n, wx, ldx = _rows2d(x, "head_linear x")
    no, wo, ldo = _rows2d(out, "head_linear out")
    _check(no == n and wx >= (heads - 1) * xs + n_in + tail and wo >= (heads - 1) * os_ + n_out + tail,
           "head_linear: rows too short for the heads")
    _check(weight.is_contiguous() and tuple(weight.shape) == (heads, n_in, n_out), "head_linear: weight [heads, n_in, n_out]")
    _check(x.dtype == out.dtype == weight.dtype, "head_linear: dtype mismatch")
    lib.core().call("hfee_head_linear", _ptr(out), ldo, os_, _ptr(x), ldx, xs, _ptr(weight), _dt(x), heads, n_in, n_out,
                    tail, n, _stream())


# ----------------------------------------------- blocks that norm a sub-layer's output; biases

ROW_ACTIVATIONS = {"none": 0, "relu2": 1, "relu": 2, "gelu_tanh": 3, "silu": 4, "xielu": 5}


def norm_add(x, y, weight, eps: float, bias=None, next_out=None, next_weight=None, next_eps: float = 0.0):
    """x (float32, the residual stream) += norm(y + bias) * weight, norm(z) = z / sqrt(mean(z^2) + eps);
    with next_out also next_out = norm(x_new) * next_weight (eps next_eps), the input of the sub-layer
    that follows.  y: [n, d] float32 or bfloat16, contiguous; both weights of one dtype."""
    _gpu(x, y, weight, bias, next_out, next_weight)
    n, d, _ = _rows2d(x, "norm_add x")
    _check(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and tuple(y.shape) == (n, d),
           "norm_add: contiguous x (float32) and y of one shape")
    _check(weight.numel() == d and weight.is_contiguous(), "norm_add: weight width")
    if bias is not None:
        _check(bias.numel() == d and bias.is_contiguous(), "norm_add: bias width")
    if next_out is not None:
        _check(next_weight is not None and next_weight.numel() == d and next_weight.is_contiguous()
               and next_weight.dtype == weight.dtype, "norm_add: the following norm's weight")
        _check(next_out.is_contiguous() and tuple(next_out.shape) == (n, d), "norm_add: next_out shape")
    lib.core().call("hfee_norm_add", _ptr(x), _ptr(y), _dt(y), _ptr(bias), 0 if bias is None else _dt(bias),
                    _ptr(weight), _dt(weight), 0.0, float(eps), _ptr(next_out), 0 if next_out is None else _dt(next_out),
                    _ptr(next_weight), float(next_eps), n, d, _stream())


def add_table_rows(x, table, index):
    """x[r] (float32 [n, d]) += table[index[r]] (a learned vector a position, a segment, ...)."""
    _gpu(x, table, index)
    n, d, _ = _rows2d(x, "add_table_rows x")
    _check(x.dtype == torch.float32 and x.is_contiguous() and table.dim() == 2 and table.is_contiguous() and table.shape[1] == d,
           "add_table_rows: contiguous float32 x and a table of its width")
    _i32(index, "add_table_rows index", n)
    lib.core().call("hfee_add_table_rows", _ptr(x), n, d, _ptr(table), _dt(table), _ptr(index), _stream())


def scaled_add(x, y, a: float = 1.0, y2=None, b: float = 1.0):
    """x += a * y + b * y2 (y2 optional); float32, contiguous, one shape."""
    _gpu(x, y, y2)
    _check(x.dtype == y.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and x.shape == y.shape,
           "scaled_add: contiguous float32 x and y of one shape")
    if y2 is not None:
        _check(y2.dtype == torch.float32 and y2.is_contiguous() and y2.shape == x.shape, "scaled_add: y2 like y")
    lib.core().call("hfee_scaled_add", _ptr(x), _ptr(y), float(a), _ptr(y2), float(b), x.numel(), _stream())


def scaled_add_norm(x, y, a: float, next_out, next_weight, next_eps: float):
    """x += a * y (float32, contiguous, one shape), and next_out (the engine's dtype, contiguous) = the RMS norm of
    the new rows, x / sqrt(mean(x^2) + next_eps) * next_weight (float32 [width])."""
    _gpu(x, y, next_out, next_weight)
    _check(x.dtype == y.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and x.shape == y.shape and x.dim() == 2,
           "scaled_add_norm: contiguous float32 rows x and y of one shape")
    _check(next_out.is_contiguous() and next_out.shape == x.shape, "scaled_add_norm: next_out like x")
    _check(next_weight.dtype == torch.float32 and next_weight.is_contiguous() and next_weight.numel() == x.shape[1],
           "scaled_add_norm: next_weight float32 [width]")
    lib.core().call("hfee_scaled_add_norm", _ptr(x), _ptr(y), float(a), _ptr(next_out), _dt(next_out), _ptr(next_weight),
                    float(next_eps), x.shape[0], x.shape[1], _stream())


def gated_norm_add(x, y, weight, eps: float, y2=None, scales=(1.0, 1.0), gate=None, gate_bias=None, next_out=None,
                   next_weight=None, next_eps: float = 0.0):
    """With v = (scales[0] * y + scales[1] * y2) * sigmoid(gate + gate_bias) (y2 and the gate optional):
    x (float32, the residual stream) += v / sqrt(mean(v^2) + eps) * weight; with next_out also
    next_out = norm(x_new) * next_weight (eps next_eps).  y, y2 float32 [n, d] contiguous; gate [n, d] in
    either dtype (rows of a wider buffer allowed); the weights and the gate's bias float32."""
    _gpu(x, y, weight, y2, gate, gate_bias, next_out, next_weight)
    n, d, _ = _rows2d(x, "gated_norm_add x")
    _check(x.dtype == y.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and tuple(y.shape) == (n, d),
           "gated_norm_add: contiguous float32 x and y of one shape")
    if y2 is not None:
        _check(y2.dtype == torch.float32 and y2.is_contiguous() and tuple(y2.shape) == (n, d), "gated_norm_add: y2 like y")
    ldg = 0
    if gate is not None:
        ng, wg, ldg = _rows2d(gate, "gated_norm_add gate")
        _check(ng == n and wg == d, "gated_norm_add: gate shape")
    for t, what in ((weight, "weight"), (gate_bias, "gate_bias"), (next_weight, "next_weight")):
        if t is not None:
            _check(t.dtype == torch.float32 and t.is_contiguous() and t.numel() == d, f"gated_norm_add: {what} float32 [d]")
    if next_out is not None:
        _check(next_weight is not None and next_out.is_contiguous() and tuple(next_out.shape) == (n, d), "gated_norm_add: next_out")
    lib.core().call("hfee_gated_norm_add", _ptr(x), _ptr(y), _ptr(y2), float(scales[0]), float(scales[1]), _ptr(gate),
                    0 if gate is None else _dt(gate), ldg, _ptr(gate_bias), _ptr(weight), float(eps), _ptr(next_out),
                    0 if next_out is None else _dt(next_out), _ptr(next_weight), float(next_eps), n, d, _stream())


def bias_act(out, x, bias, activation: str = "none", numbers=(0.0, 0.0)):
    """out = activation(x + bias), row by row; "relu2" is the square of relu; "xielu" with its two
    `numbers` (a, b) is a z^2 + z / 2 above zero and b (exp(z) - 1 - z) + z / 2 at and below it."""
    _gpu(out, x, bias)
    _check(activation in ROW_ACTIVATIONS, f"bias_act: the activations are {sorted(ROW_ACTIVATIONS)}, not {activation!r}")
    n, w, ldi = _rows2d(x, "bias_act x")
    no, wo, ldo = _rows2d(out, "bias_act out")
    _check(no == n and wo == w and out.dtype == x.dtype, "bias_act: shapes and dtypes of x and out")
    if bias is not None:
        _check(bias.numel() == w and bias.is_contiguous() and bias.dtype == x.dtype, "bias_act: bias")
    lib.core().call("hfee_bias_act", _ptr(out), ldo, _ptr(x), ldi, _ptr(bias), _dt(x), n, w, ROW_ACTIVATIONS[activation],
                    float(numbers[0]), float(numbers[1]), _stream())


def rmsnorm_cols(out, x, weight, eps: float):
    """out[r] = x[r] / sqrt(mean(x[r]^2) + eps) * weight over the columns of x, a 2-D view in the
    engine's dtype with contiguous rows (a block of columns of a wider buffer); out may be x."""
    _gpu(out, x, weight)
    n, w, ldx = _rows2d(x, "rmsnorm_cols x")
    no, wo, ldo = _rows2d(out, "rmsnorm_cols out")
    _check(no == n and wo == w and out.dtype == x.dtype, "rmsnorm_cols: shapes and dtypes of x and out")
    _check(weight.numel() == w and weight.is_contiguous(), "rmsnorm_cols: weight width")
    lib.core().call("hfee_rmsnorm_cols", _ptr(out), ldo, _ptr(x), ldx, _dt(x), _ptr(weight), _dt(weight), 0.0, float(eps),
                    n, w, _stream())


def layernorm(out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float, rows: torch.Tensor | None = None):
    """out[r] = (x[rows[r] or r] - mean) / sqrt(variance + eps) * weight, the variance the mean of the
    squared deviations; x float32, no bias."""
    _gpu(out, x, weight, rows)
    n, d, _ = _rows2d(out, "layernorm out")
    _check(out.is_contiguous() and x.is_contiguous() and x.dtype == torch.float32, "layernorm: contiguous float32 x")
    _check(x.dim() == 2 and x.shape[1] == d, "layernorm: width mismatch")
    _check(weight.numel() == d and weight.is_contiguous(), "layernorm: weight width mismatch")
    if rows is None:
        _check(x.shape[0] >= n, "layernorm: fewer input rows than output rows")
    else:
        _i32(rows, "layernorm rows", n)
    lib.core().call("hfee_layernorm", _ptr(out), _dt(out), _ptr(x), _ptr(weight), _dt(weight), _ptr(rows), float(eps),
                    n, d, _stream())


# --------------------------------- attention whose heads' scores are mixed, over keys that are the values

def _mix_cache(cache_layer, kv_heads, dim, page_size, what):
    _check(cache_layer.is_contiguous() and cache_layer.dim() == 3 and
           tuple(cache_layer.shape[1:]) == (kv_heads, page_size * 2 * dim),
           f"{what}: the cache layer must be [pages, kv_heads, page_size * 2 * dim]")


def _tables(block_tables, what):
    _check(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1, f"{what}: block tables")


def attention_mix_prepare(q, k, positions, token_segment, block_tables, cos, sin, cache_layer, num_heads: int,
                          kv_heads: int, dim: int, page_size: int, max_position: int, norm: bool = True,
                          eps: float = 0.0):
    """q ([n, num_heads * dim], in place) and k ([n, kv_heads * dim]) rotated in their first 2 * half
    dims (cos/sin float32 [positions, half], pairs (i, i + half)) and then, with `norm`, divided by
    their root mean square over each head; the key as it is scored and the key as it was projected
    go into the token's slot of `cache_layer` ([pages, kv_heads, page_size * 2 * dim]: the scored keys of a
    (page, head) as [slot][dim], then the values transposed as [dim][slot]).  k None: only q is made ready."""
    _gpu(q, k, positions, cos, sin, cache_layer)
    some = q if q is not None else k
    _check(some is not None, "attention_mix_prepare: nothing to do")
    n = some.shape[0]
    ldq = ldk = 0
    if q is not None:
        nq, wq, ldq = _rows2d(q, "attention_mix_prepare q")
        _check(wq == num_heads * dim, "attention_mix_prepare: q shape")
    if k is not None:
        nk, wk, ldk = _rows2d(k, "attention_mix_prepare k")
        _check(nk == n and wk == kv_heads * dim and k.dtype == cache_layer.dtype and (q is None or q.dtype == k.dtype),
               "attention_mix_prepare: k shape or dtype")
        _mix_cache(cache_layer, kv_heads, dim, page_size, "attention_mix_prepare")
        _i32(token_segment, "attention_mix_prepare token_segment", n)
        _tables(block_tables, "attention_mix_prepare")
    _i32(positions, "attention_mix_prepare positions", n)
    half = table_positions = 0
    if cos is not None:
        _check(cos.shape == sin.shape and cos.dim() == 2 and cos.is_contiguous() and sin.is_contiguous()
               and cos.dtype == sin.dtype == torch.float32, "attention_mix_prepare: cos/sin tables")
        table_positions, half = cos.shape
    has_k = k is not None
    lib.core().call("hfee_attention_mix_prepare", _ptr(q), ldq, _ptr(k), ldk, _dt(some), num_heads, kv_heads, dim,
                    _ptr(positions), _ptr(token_segment if has_k else None), _ptr(block_tables if has_k else None),
                    block_tables.stride(0) if has_k else 0, _ptr(cos), _ptr(sin), half, table_positions,
                    int(max_position), 1 if norm else 0, float(eps), _ptr(cache_layer if has_k else None), page_size, n,
                    _stream())


def attention_mix(out, q, cache_layer, positions, token_segment, block_tables, num_heads: int, kv_heads: int, dim: int,
                  page_size: int, scale: float, mix=None, chunk: int = 0, sink=None):
    """Token t at position p reads the keys of its sequence from the start of p's chunk (chunk 0: from
    position 0) up to p; the heads' scores q . k * scale are mixed by `mix` (float32 [heads, heads],
    score_h = sum_g mix[h, g] score_g; None: not mixed); sink: None, "zero" (one more term exp(0) in
    the softmax's denominator) or a float32 tensor [heads] of learned scores; the values are the
    second half of each (page, head) of the cache."""
    _gpu(out, q, cache_layer, positions, token_segment, block_tables, mix)
    n, w, ldq = _rows2d(q, "attention_mix q")
    no, wo, ldo = _rows2d(out, "attention_mix out")
    _check(no == n and w == num_heads * dim and wo == num_heads * dim, "attention_mix: q/out shape")
    _check(q.dtype == out.dtype == cache_layer.dtype, "attention_mix: dtype mismatch")
    _mix_cache(cache_layer, kv_heads, dim, page_size, "attention_mix")
    _i32(positions, "attention_mix positions", n)
    _i32(token_segment, "attention_mix token_segment", n)
    _tables(block_tables, "attention_mix")
    if mix is not None:
        _check(mix.dtype == torch.float32 and mix.is_contiguous() and tuple(mix.shape) == (num_heads, num_heads),
               "attention_mix: mix must be float32 [heads, heads]")
    sinks, mode = None, 0
    if isinstance(sink, str):
        _check(sink == "zero", "attention_mix: sink is None, 'zero' or a tensor")
        mode = 1
    elif sink is not None:
        _gpu(sink)
        _check(sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == num_heads,
               "attention_mix: sinks must be float32 [heads]")
        sinks, mode = sink, 2
    lib.core().call("hfee_attention_mix", _ptr(out), ldo, _ptr(q), ldq, _ptr(cache_layer), _dt(q), _ptr(positions),
                    _ptr(token_segment), _ptr(block_tables), block_tables.stride(0), num_heads, kv_heads, dim, page_size,
                    float(scale), _ptr(mix), int(chunk), mode, _ptr(sinks), n, _stream())


def attention_mix_fits(num_heads: int, dim: int) -> bool:
    """Whether the matrix-core kernels take these sizes (else: `attention_mix`)."""
    from . import build
    return build.attention_mix_fits(num_heads, dim)


ATTENTION_MIX_ROWS = 16


def attention_mix_partial_words(num_items: int, num_heads: int, dim: int, splits: int) -> int:
    return num_items * splits * num_heads * ATTENTION_MIX_ROWS * (dim + 2) if splits > 1 else 0


def attention_mix_bf16(out, q, cache_layer, items, block_tables, num_heads: int, kv_heads: int, dim: int, page_size: int,
                       scale: float, mix_t=None, chunk: int = 0, sink=None, splits: int = 1, partial=None):
    """`attention_mix` on the matrix cores, bfloat16.  items: int32 [count, 4] on the device (first row,
    rows (1 to 16), first position, block-table row), the rows of an item consecutive positions of one
    sequence within one chunk; mix_t: the mixing matrix transposed, float32 [heads, heads]
    (score_h = sum_g mix_t[g, h] score_g), or None.  splits > 1: the key tiles of every item are shared out
    over so many workgroups, which leave their parts in `partial` (float32, `attention_mix_partial_words`)
    for a joining kernel."""
    _gpu(out, q, cache_layer, items, block_tables, mix_t, partial)
    if partial is not None:
        _check(partial.dtype == torch.float32 and partial.is_contiguous(), "attention_mix: float32 partial buffer expected")
    n, w, ldq = _rows2d(q, "attention_mix q")
    no, wo, ldo = _rows2d(out, "attention_mix out")
    _check(no == n and w == num_heads * dim and wo == num_heads * dim, "attention_mix: q/out shape")
    _check(q.dtype == out.dtype == cache_layer.dtype == torch.bfloat16, "attention_mix: bfloat16 tensors expected")
    _mix_cache(cache_layer, kv_heads, dim, page_size, "attention_mix")
    _check(items.dtype == torch.int32 and items.dim() == 2 and items.shape[1] == 4 and items.is_contiguous(),
           "attention_mix: items must be [count, 4] int32")
    _tables(block_tables, "attention_mix")
    if mix_t is not None:
        _check(mix_t.dtype == torch.float32 and mix_t.is_contiguous() and tuple(mix_t.shape) == (num_heads, num_heads),
               "attention_mix: mix_t must be float32 [heads, heads]")
    sinks, mode = None, 0
    if isinstance(sink, str):
        _check(sink == "zero", "attention_mix: sink is None, 'zero' or a tensor")
        mode = 1
    elif sink is not None:
        _gpu(sink)
        _check(sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == num_heads,
               "attention_mix: sinks must be float32 [heads]")
        sinks, mode = sink, 2
    lib.attention_mix_bf16(num_heads, kv_heads, dim).call(
        "hfee_attention_mix_bf16", _ptr(out), ldo, _ptr(q), ldq, _ptr(cache_layer), _ptr(items), items.shape[0],
        _ptr(block_tables), block_tables.stride(0), kv_heads, page_size, float(scale), _ptr(mix_t), int(chunk), mode,
        _ptr(sinks), int(splits), _ptr(partial), 0 if partial is None else partial.numel(), _stream())


# ------------------------------------------------ mixers with a state of fixed size a request

def _f32rows(t, what):
    n, w, ld = _rows2d(t, what)
    _check(t.dtype == torch.float32, f"{what}: float32 expected")
    return n, w, ld


def short_conv_silu(y, x, state, taps, token_segment, segment_rows, segment_slots, in_bias=None, out_bias=None,
                    activation: str = "silu"):
    """y (float32 [n, C]) = silu of the causal convolution of x ([n, C], the step's rows) with taps
    (float32 [C, K], the last column the current token's) per channel; the K - 1 inputs before a
    portion's first token come from state[slot] ([slots, K - 1, C] in x's dtype, the newest last).
    in_bias (float32 [C]) is added to every input that exists (before a sequence's start stand zeros),
    out_bias (float32 [C]) to the sum; activation "silu" or "none"."""
    _gpu(y, x, state, taps, token_segment, segment_rows, segment_slots, in_bias, out_bias)
    _check(activation in ("silu", "none"), "short_conv: the activation is 'silu' or 'none'")
    for b in (in_bias, out_bias):
        if b is not None:
            _check(b.dtype == torch.float32 and b.is_contiguous() and b.numel() == x.shape[1], "short_conv: a bias is float32 [C]")
    n, C, ldx = _rows2d(x, "short_conv_silu x")
    ny, wy, ldy = _f32rows(y, "short_conv_silu y")
    K = taps.shape[1]
    _check(ny == n and wy == C and tuple(taps.shape) == (C, K) and taps.dtype == torch.float32 and taps.is_contiguous(),
           "short_conv_silu: shapes of y and taps")
    _check(state.dtype == x.dtype and state.is_contiguous() and tuple(state.shape[1:]) == (K - 1, C),
           "short_conv_silu: the state must be [slots, K - 1, C] in x's dtype")
    _i32(token_segment, "short_conv_silu token_segment", n)
    _i32(segment_rows, "short_conv_silu segment_rows")
    _i32(segment_slots, "short_conv_silu segment_slots")
    lib.core().call("hfee_short_conv_silu", _ptr(y), ldy, _ptr(x), ldx, _ptr(state), _dt(x), _ptr(taps),
                    _ptr(token_segment), _ptr(segment_rows), _ptr(segment_slots), C, K, n, _ptr(in_bias), _ptr(out_bias),
                    1 if activation == "silu" else 0, _stream())


def short_conv_keep(state, x, segment_rows, segment_lengths, segment_slots, in_bias=None):
    """state[slot] <- the last K - 1 inputs of each segment's sequence (the step's rows x with in_bias,
    and what the state held before where a portion is shorter than K - 1)."""
    _gpu(state, x, segment_rows, segment_lengths, segment_slots, in_bias)
    if in_bias is not None:
        _check(in_bias.dtype == torch.float32 and in_bias.is_contiguous() and in_bias.numel() == x.shape[1], "short_conv_keep: in_bias float32 [C]")
    n, C, ldx = _rows2d(x, "short_conv_keep x")
    _check(state.dtype == x.dtype and state.is_contiguous() and state.dim() == 3 and state.shape[2] == C,
           "short_conv_keep: the state must be [slots, K - 1, C] in x's dtype")
    segments = segment_rows.numel()
    _i32(segment_rows, "short_conv_keep segment_rows")
    _i32(segment_lengths, "short_conv_keep segment_lengths", segments)
    _i32(segment_slots, "short_conv_keep segment_slots", segments)
    lib.core().call("hfee_short_conv_keep", _ptr(state), _ptr(x), ldx, _dt(x), _ptr(segment_rows), _ptr(segment_lengths),
                    _ptr(segment_slots), C, state.shape[1] + 1, segments, _ptr(in_bias), _stream())


def unit_heads(x, heads: int, dim: int, eps: float, factor: float = 1.0):
    """x (float32 [n, heads * dim], in place) <- x / sqrt(sum(x^2) + eps) * factor over each head."""
    _gpu(x)
    n, w, ldx = _f32rows(x, "unit_heads x")
    _check(w == heads * dim, "unit_heads: width")
    lib.core().call("hfee_unit_heads", _ptr(x), ldx, heads, dim, float(eps), float(factor), n, _stream())


def rotate_rows(out, x, positions, cos, sin, heads: int, dim: int, max_position: int, scaled_from: int | None = None,
                factor: float = 1.0):
    """out (float32 [n, heads * dim]) = x (the engine's dtype) with the first 2 * half dims of every head turned by
    the token's position (pairs (i, i + half); cos/sin float32 [positions, half], or None for no rotation), and the
    heads from `scaled_from` on multiplied by `factor` behind it."""
    _gpu(out, x, positions, cos, sin)
    n, w, ldx = _rows2d(x, "rotate_rows x")
    no, wo, ldo = _f32rows(out, "rotate_rows out")
    _check(no == n and w == wo == heads * dim, "rotate_rows: shapes")
    _i32(positions, "rotate_rows positions", n)
    half = table_positions = 0
    if cos is not None:
        _check(cos.shape == sin.shape and cos.dim() == 2 and cos.is_contiguous() and sin.is_contiguous()
               and cos.dtype == sin.dtype == torch.float32, "rotate_rows: cos/sin tables")
        table_positions, half = cos.shape
    lib.core().call("hfee_rotate_rows", _ptr(out), ldo, _ptr(x), ldx, _dt(x), _ptr(positions), _ptr(cos), _ptr(sin), half,
                    table_positions, int(max_position), heads, dim, heads if scaled_from is None else int(scaled_from),
                    float(factor), n, _stream())


SCAN_GATES = {"step_decay": 0, "root_sigmoid": 1, "sigmoid": 2, "cast": 3, "softplus": 4}


def scan_gate(out, z, kind: str, bias=None, per_head=None, head_width: int = 0, number: float = 1.0, first_columns: int = 0):
    """out (float32) from a projection z (engine dtype), column by column:
    "step_decay": exp(-exp(per_head[column // head_width]) * softplus(z + bias));
    "root_sigmoid": sigmoid(z + bias) ** (1 / number);  "sigmoid": sigmoid(z + bias);
    "cast": z * number in the first `first_columns` columns, z in the others;  "softplus": softplus(z + bias)."""
    _gpu(out, z, bias, per_head)
    n, w, ldz = _rows2d(z, "scan_gate z")
    no, wo, ldo = _f32rows(out, "scan_gate out")
    _check(kind in SCAN_GATES and no == n and wo == w, "scan_gate: kind or shapes")
    for t, what in ((bias, "bias"), (per_head, "per_head")):
        if t is not None:
            _check(t.dtype == torch.float32 and t.is_contiguous(), f"scan_gate: {what} must be contiguous float32")
    if bias is not None:
        _check(bias.numel() == w, "scan_gate: bias width")
    if kind == "step_decay":
        _check(per_head is not None and head_width > 0 and per_head.numel() * head_width == w, "scan_gate: one number a head")
    lib.core().call("hfee_scan_gate", _ptr(out), ldo, _ptr(z), ldz, _dt(z), _ptr(bias), _ptr(per_head), int(head_width),
                    SCAN_GATES[kind], float(number), int(first_columns), n, w, _stream())


SCAN_COLUMNS, SCAN_PARTS = 4, 16


def _scan_rows_a_lane(dim: int) -> int:
    per = (dim + SCAN_PARTS - 1) // SCAN_PARTS
    return 1 << max(0, (per - 1).bit_length())


def scan_state_shape(dim: int, vdim: int) -> tuple:
    """How `linear_scan` keeps a head's matrix S [dim, vdim]: blocks of four columns, each as the 64 lanes
    of a wave hold it: [blocks, rows a lane, 4 columns, 16 parts], row d = rows a lane * part + i."""
    return ((vdim + SCAN_COLUMNS - 1) // SCAN_COLUMNS, _scan_rows_a_lane(dim), SCAN_COLUMNS, SCAN_PARTS)


def scan_state_matrix(state: torch.Tensor, dim: int, vdim: int) -> torch.Tensor:
    """[..., blocks, rows a lane, 4, 16] as `linear_scan` keeps it -> [..., dim, vdim]."""
    s = state.permute(*range(state.dim() - 4), -1, -3, -4, -2)         # [..., part, i, block, column]
    return s.reshape(*s.shape[:-4], s.shape[-4] * s.shape[-3], s.shape[-2] * s.shape[-1])[..., :dim, :vdim]


def linear_scan(out, state, q, k, v, decay, beta, segment_rows, segment_lengths, segment_slots, heads: int,
                qk_heads: int, dim: int, vdim: int, rule: str, decay_per_head: bool = False):
    """Walks each segment's rows in order from state[slot] (float32 [slots, heads, `scan_state_shape`],
    updated in place: a head's matrix in blocks of four columns).  rule "decay_add": S <- diag(decay) S + k v^T; "delta": S <- diag(decay) S,
    S <- S + k (beta (v - S^T k))^T; "scaled_add": S <- diag(decay) S + k (beta v)^T; out = S^T q.
    q, k: float32 [n, qk_heads * dim] (head h reads q/k head h // (heads / qk_heads)); v, out:
    [n, heads * vdim]; decay: [n, heads * dim], or with decay_per_head [n, heads], one number for all
    of a head's rows (or [heads]: the same decays for every token); beta [n, heads]."""
    _gpu(out, state, q, k, v, decay, beta, segment_rows, segment_lengths, segment_slots)
    n, wq, ldq = _f32rows(q, "linear_scan q")
    nk, wk, ldk = _f32rows(k, "linear_scan k")
    nv, wv, ldv = _f32rows(v, "linear_scan v")
    if decay.dim() == 1:        # one row for every token
        _check(decay_per_head and decay.dtype == torch.float32 and decay.is_contiguous(), "linear_scan: constant decays are float32 [heads]")
        nd, wd, ldd = n, decay.numel(), 0
    else:
        nd, wd, ldd = _f32rows(decay, "linear_scan decay")
    no, wo, ldo = _f32rows(out, "linear_scan out")
    rules = {"decay_add": 0, "delta": 1, "scaled_add": 2}
    _check(rule in rules, f"linear_scan: rule is one of {sorted(rules)}")
    _check(nk == nv == nd == no == n and wq == wk == qk_heads * dim and wv == wo == heads * vdim
           and wd == (heads if decay_per_head else heads * dim), "linear_scan: shapes")
    _check(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (heads, *scan_state_shape(dim, vdim)),
           "linear_scan: the state must be float32 [slots, heads, *scan_state_shape(dim, vdim)]")
    ldb = 0
    if rule != "decay_add":
        nb, wb, ldb = _f32rows(beta, "linear_scan beta")
        _check(nb == n and wb == heads, "linear_scan: beta [n, heads]")
    segments = segment_rows.numel()
    _i32(segment_rows, "linear_scan segment_rows")
    _i32(segment_lengths, "linear_scan segment_lengths", segments)
    _i32(segment_slots, "linear_scan segment_slots", segments)
    lib.core().call("hfee_linear_scan", _ptr(out), ldo, _ptr(state), _ptr(q), ldq, _ptr(k), ldk, _ptr(v), ldv, _ptr(decay),
                    ldd, _ptr(beta if rule != "decay_add" else None), ldb, _ptr(segment_rows), _ptr(segment_lengths),
                    _ptr(segment_slots), segments, heads, qk_heads, dim, vdim, rules[rule], 1 if decay_per_head else 0, _stream())


RGLRU_CHUNK = 32        # tokens a chunk of the recurrent unit's kernels for long portions


def rglru_scan_scratch(longest: int, segments: int, width: int) -> int:
    """float32 words that `rglru_scan` needs for a step whose longest portion has `longest` tokens."""
    if longest <= 2 * RGLRU_CHUNK:
        return 0
    return (segments * (-(-longest // RGLRU_CHUNK)) * 2 + segments) * width


def rglru_scan(out, state, gates, gate_bias, u, rate, y, y_bias, segment_rows, segment_lengths, segment_slots, block: int,
               longest: int = 0, scratch=None):
    """The real-gated linear recurrent unit, a number a channel: with r, i the gates of a token (gates:
    float32 [n, blocks, 2 * block] before bias and sigmoid, a block's r, then its i; gate_bias float32 of
    that width), a = exp(rate * sigmoid(r)) (rate float32 [W], not positive),
    S <- a S + sqrt(1 - a^2) sigmoid(i) u, out = S * gelu_tanh(y + y_bias) in y's dtype.  state: float32
    [slots, W], walked from and left in each segment's slot; u float32 [n, W]; y [n, W].  longest: the
    longest portion of the step, if known; with `scratch` (float32, `rglru_scan_scratch` words) long
    portions are walked in chunks by many threads a channel."""
    _gpu(out, state, gates, gate_bias, u, rate, y, y_bias, segment_rows, segment_lengths, segment_slots)
    n, W, ldu = _f32rows(u, "rglru_scan u")
    ng, wg, ldg = _f32rows(gates, "rglru_scan gates")
    ny, wy, ldy = _rows2d(y, "rglru_scan y")
    no, wo, ldo = _rows2d(out, "rglru_scan out")
    _check(ng == ny == no == n and wg == 2 * W and wy == wo == W and out.dtype == y.dtype and W % block == 0, "rglru_scan: shapes")
    _check(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 2 and state.shape[1] == W, "rglru_scan: state float32 [slots, W]")
    for t, w, what in ((gate_bias, 2 * W, "gate_bias"), (rate, W, "rate"), (y_bias, W, "y_bias")):
        if t is not None:
            _check(t.dtype == torch.float32 and t.is_contiguous() and t.numel() == w, f"rglru_scan: {what} float32 [{w}]")
    segments = segment_rows.numel()
    _i32(segment_rows, "rglru_scan segment_rows")
    _i32(segment_lengths, "rglru_scan segment_lengths", segments)
    _i32(segment_slots, "rglru_scan segment_slots", segments)
    words = 0
    if scratch is not None:
        _gpu(scratch)
        _check(scratch.dtype == torch.float32 and scratch.is_contiguous(), "rglru_scan: scratch float32")
        _check(0 < longest <= n, "rglru_scan: scratch comes with the longest portion's length")
        words = scratch.numel()
    lib.core().call("hfee_rglru_scan", _ptr(out), ldo, _dt(out), _ptr(state), _ptr(gates), ldg, _ptr(gate_bias), _ptr(u), ldu,
                    _ptr(rate), _ptr(y), ldy, _ptr(y_bias), _ptr(segment_rows), _ptr(segment_lengths), _ptr(segment_slots),
                    segments, W, int(block), int(longest), _ptr(scratch), words, _stream())


def gate_group_norm(out, o, x, skip, z, weight, heads: int, parts: int, eps: float):
    """out = norm((o + skip[head] * x) * silu(z)) * weight, the norm (root mean square, eps) over each of
    `parts` equal parts of a row; o, x float32 [n, inner], skip float32 [heads], z and out in the engine's
    dtype, weight float32 [inner]."""
    _gpu(out, o, x, skip, z, weight)
    n, inner, ldi = _f32rows(o, "gate_group_norm o")
    nx, wx, ldx = _f32rows(x, "gate_group_norm x")
    nz, wz, ldz = _rows2d(z, "gate_group_norm z")
    no, wo, ldo = _rows2d(out, "gate_group_norm out")
    _check(nx == nz == no == n and wx == wz == wo == inner and z.dtype == out.dtype and inner % heads == 0 and inner % parts == 0,
           "gate_group_norm: shapes")
    _check(skip.dtype == weight.dtype == torch.float32 and skip.is_contiguous() and weight.is_contiguous()
           and skip.numel() == heads and weight.numel() == inner, "gate_group_norm: skip float32 [heads], weight float32 [inner]")
    lib.core().call("hfee_gate_group_norm", _ptr(out), ldo, _dt(out), _ptr(o), ldi, _ptr(x), ldx, _ptr(skip), inner // heads,
                    _ptr(z), ldz, _ptr(weight), int(parts), inner, float(eps), n, _stream())


def head_norm_gate(out, o, gate, weight, heads: int, vdim: int, eps: float, activation: str):
    """out[t, h] = o[t, h] / sqrt(mean(o[t, h]^2) + eps) * weight * act(gate[t, h]) over each head's vdim
    values; o float32, gate and out in the engine's dtype, weight float32 [vdim]; act "sigmoid" or "silu"."""
    _gpu(out, o, gate, weight)
    n, w, ldi = _f32rows(o, "head_norm_gate o")
    ng, wg, ldg = _rows2d(gate, "head_norm_gate gate")
    no, wo, ldo = _rows2d(out, "head_norm_gate out")
    _check(ng == no == n and wg == wo == w == heads * vdim and gate.dtype == out.dtype, "head_norm_gate: shapes and dtypes")
    _check(weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() == vdim, "head_norm_gate: weight float32 [vdim]")
    _check(activation in ("sigmoid", "silu"), "head_norm_gate: the gate's activation is 'sigmoid' or 'silu'")
    lib.core().call("hfee_head_norm_gate", _ptr(out), ldo, _ptr(o), ldi, _ptr(gate), ldg, _dt(out), _ptr(weight), heads, vdim,
                    float(eps), 0 if activation == "sigmoid" else 1, n, _stream())


# ------------------------------------------------------------------ experts

def _experts_of(chosen, table, token_ids, n, top, what):
    if chosen is not None:
        _check(chosen.dtype == torch.int32 and chosen.is_contiguous() and tuple(chosen.shape) == (n, top), f"{what}: chosen int32 [n, top]")
        return
    _check(table is not None and token_ids is not None and table.dtype == torch.int32 and table.is_contiguous()
           and table.dim() == 2 and table.shape[1] == top, f"{what}: a table int32 [vocabulary, top] and the token ids")
    _i32(token_ids, f"{what} token_ids", n)


def _in_weights(in_weights, w_gate, n, top, what):
    if in_weights is not None:
        _check(w_gate is None, f"{what}: only experts without a gate take a weight on their input")
        _check(in_weights.dtype == torch.float32 and in_weights.is_contiguous() and tuple(in_weights.shape) == (n, top),
               f"{what}: in_weights float32 [n, top]")


def moe_up(act, h, w_gate, w_up, top: int, chosen=None, table=None, token_ids=None, in_weights=None):
    """act[t * top + j] = silu(w_gate[e] @ h[t]) * (w_up[e] @ h[t]), e the j-th expert of token t
    (chosen[t, j], or table[token_ids[t], j]); w_gate, w_up: [experts, ff, width].  w_gate None: experts
    without a gate, act = relu(in_weights[t, j] * (w_up[e] @ h[t]))^2 (in_weights float32 or None for one)."""
    _gpu(act, h, w_gate, w_up, chosen, table, token_ids, in_weights)
    n, width, ldh = _rows2d(h, "moe_up h")
    E, F, W = w_up.shape
    _check(W == width and w_up.is_contiguous() and (w_gate is None or (w_gate.shape == w_up.shape and w_gate.is_contiguous()
                                                                      and w_gate.dtype == w_up.dtype)),
           "moe_up: weights [experts, ff, width]")
    _check(act.is_contiguous() and tuple(act.shape) == (n * top, F) and act.dtype == h.dtype == w_up.dtype,
           "moe_up: act [n * top, ff], one dtype")
    _experts_of(chosen, table, token_ids, n, top, "moe_up")
    _in_weights(in_weights, w_gate, n, top, "moe_up")
    lib.core().call("hfee_moe_up", _ptr(act), _ptr(h), ldh, _ptr(w_gate), _ptr(w_up), _dt(h), _ptr(chosen), _ptr(table),
                    _ptr(token_ids), top, E, F, width, n, _ptr(in_weights), _stream())


ROUTER_SCORES = {"sigmoid": 0, "softmax": 1}


def router_topk(chosen, weights, logits, top: int, score: str = "sigmoid", correction=None):
    """chosen (int32 [n, top]) = the experts with the `top` largest choice scores of each row of logits
    (float32 [n, experts]; of equal ones the lower number), weights (float32 [n, top]) their scores.  A score
    is sigmoid(logit), or with score "softmax" the softmax over the row; the choice score is the score plus
    correction (float32 [experts]) where one is given, and the weights never hold it."""
    _gpu(chosen, weights, logits, correction)
    n, E, ld = _f32rows(logits, "router_topk logits")
    _check(score in ROUTER_SCORES, f"router_topk: the scores are {sorted(ROUTER_SCORES)}")
    _check(chosen.dtype == torch.int32 and chosen.is_contiguous() and tuple(chosen.shape) == (n, top), "router_topk: chosen int32 [n, top]")
    _check(weights.dtype == torch.float32 and weights.is_contiguous() and tuple(weights.shape) == (n, top), "router_topk: weights float32 [n, top]")
    if correction is not None:
        _check(correction.dtype == torch.float32 and correction.is_contiguous() and correction.numel() == E,
               "router_topk: correction float32 [experts]")
    lib.core().call("hfee_router_topk", _ptr(logits), ld, n, E, int(top), _ptr(chosen), _ptr(weights), ROUTER_SCORES[score],
                    _ptr(correction), _stream())


def moe_down(x, act, w_down, top: int, weight: float = 1.0, pair_weights=None, chosen=None, table=None, token_ids=None,
             accumulate: bool = True):
    """x[t] (+)= sum_j weight_tj * (w_down[e_j] @ act[t * top + j]); x float32 [n, width], w_down
    [experts, width, ff]; weight_tj = pair_weights[t, j] (float32) or the one number `weight`."""
    _gpu(x, act, w_down, pair_weights, chosen, table, token_ids)
    n, width, ldx = _f32rows(x, "moe_down x")
    E, W, F = w_down.shape
    _check(W == width and w_down.is_contiguous() and act.is_contiguous() and tuple(act.shape) == (n * top, F)
           and act.dtype == w_down.dtype, "moe_down: w_down [experts, width, ff], act [n * top, ff]")
    if pair_weights is not None:
        _check(pair_weights.dtype == torch.float32 and pair_weights.is_contiguous() and tuple(pair_weights.shape) == (n, top),
               "moe_down: pair_weights float32 [n, top]")
    _experts_of(chosen, table, token_ids, n, top, "moe_down")
    lib.core().call("hfee_moe_down", _ptr(x), ldx, _ptr(act), _ptr(w_down), _dt(act), _ptr(chosen), _ptr(table),
                    _ptr(token_ids), _ptr(pair_weights), float(weight), top, E, F, width, 1 if accumulate else 0, n, _stream())


MOE_TILE_PAIRS = 64


def moe_group_tiles(n: int, top: int, experts: int) -> int:
    """The most tiles of 64 (token, expert) pairs of one expert that a step of n tokens can make."""
    return (n * top + MOE_TILE_PAIRS - 1) // MOE_TILE_PAIRS + experts


def moe_grouped_fits(dtype, width: int, ff: int) -> bool:
    return dtype == torch.bfloat16 and width % 32 == 0 and ff % 32 == 0


def moe_grouped(x, h, w_gate, w_up, w_down, top: int, order, tiles, act, y=None, weight: float = 1.0, pair_weights=None,
                chosen=None, table=None, token_ids=None, in_weights=None):
    """x[t] += sum_j weight_tj * w_down[e_j] @ (silu(w_gate[e_j] @ h[t]) * (w_up[e_j] @ h[t])), bfloat16, with the
    step's (token, expert) pairs grouped by expert on the device and multiplied in tiles on the matrix cores.
    order: int32 [n * top]; tiles: int32 [3 * moe_group_tiles(n, top, experts) + 1]; act: bfloat16
    [n * top, ff]; y: float32 [n * top, width] (where top > 1): scratch.  w_gate None: experts without a gate,
    relu(in_weights[t, j] * (w_up[e_j] @ h[t]))^2 in the gate's place (then without pair_weights)."""
    _gpu(x, h, w_gate, w_up, w_down, order, tiles, act, y, pair_weights, chosen, table, token_ids, in_weights)
    n, width, ldh = _rows2d(h, "moe_grouped h")
    nx, wx, ldx = _f32rows(x, "moe_grouped x")
    E, F, W = w_up.shape
    _check(nx == n and wx == width == W and tuple(w_down.shape) == (E, width, F) and w_up.is_contiguous() and w_down.is_contiguous()
           and (w_gate is None or (w_gate.shape == w_up.shape and w_gate.is_contiguous() and w_gate.dtype == torch.bfloat16)),
           "moe_grouped: shapes")
    _check(h.dtype == w_up.dtype == w_down.dtype == act.dtype == torch.bfloat16, "moe_grouped: bfloat16 operands")
    _in_weights(in_weights, w_gate, n, top, "moe_grouped")
    _check(w_gate is not None or pair_weights is None, "moe_grouped: experts without a gate take their weights on the input")
    _check(act.is_contiguous() and act.numel() >= n * top * F, "moe_grouped: act [n * top, ff]")
    _check(order.dtype == tiles.dtype == torch.int32 and order.is_contiguous() and tiles.is_contiguous()
           and order.numel() >= n * top and tiles.numel() >= 3 * moe_group_tiles(n, top, E) + 1, "moe_grouped: order and tiles")
    if top > 1:
        _check(y is not None and y.dtype == torch.float32 and y.is_contiguous() and y.numel() >= n * top * width,
               "moe_grouped: y float32 [n * top, width]")
    if pair_weights is not None:
        _check(pair_weights.dtype == torch.float32 and pair_weights.is_contiguous() and tuple(pair_weights.shape) == (n, top),
               "moe_grouped: pair_weights float32 [n, top]")
    _experts_of(chosen, table, token_ids, n, top, "moe_grouped")
    lib.core().call("hfee_moe_grouped", _ptr(x), ldx, _ptr(h), ldh, _ptr(w_gate), _ptr(w_up), _ptr(w_down), _ptr(chosen),
                    _ptr(table), _ptr(token_ids), _ptr(pair_weights), float(weight), top, E, F, width, n, _ptr(order),
                    _ptr(tiles), _ptr(act), _ptr(y), _ptr(in_weights), _stream())
