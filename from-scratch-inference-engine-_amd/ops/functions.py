"""Host-side checks and launches of the kernels."""

from __future__ import annotations

import ctypes

from typing import Optional

import torch

from .library import KernelError, check, load

F32, BF16 = 0, 1
ATTN_ITEM_INTS = 8
ATTN_MERGE_INTS = 4
ATTN_POOL_WALK = 1 << 29  # the item also reads the pooled blocks before its queries' windows
ATTN_KEEP_WALK = 1 << 30  # in an item's last field, beside the number of kept first keys: read them before the item's range
GEMM_SKINNY_MAX_M = 8
GEMM_MFMA_SKINNY_MAX_M = 64
GEMM_MFMA_WIDE_MAX_M = 128  # the product that shares x through LDS, on a fragment-ordered weight
GEMM_MFMA_SKINNY_BEST_M = 16
GEMM_SPLITS = (2, 4, 8)  # slices of K that the few-rows product may leave as partial sums
GEMM_MAX_SPLITS = 16     # most slices of the product that shares x through LDS, and most that a norm adds up
GEMM_AUTO, GEMM_TILED, GEMM_SKINNY, GEMM_NARROW = 0, 1, 2, 3


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16, not {dtype}")


# the current stream's handle straight from the runtime where torch offers it: the Stream object that
# torch.cuda.current_stream() builds costs some 10 us, and every kernel launch asks for it
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _need(t: torch.Tensor, name: str, dtype=None, shape=None, ndim=None) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: must be a tensor on the GPU")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, found {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise KernelError(f"{name}: expected {ndim} dimensions, found shape {tuple(t.shape)}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: expected shape {tuple(shape)}, found {tuple(t.shape)}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def embedding(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """float32 rows of ``table`` [V, H] at ``ids`` (int32 [T]), times ``scale``.  The caller has checked the ids."""
    _need(table, "embedding table", ndim=2)
    _need(ids, "embedding ids", dtype=torch.int32, ndim=1)
    v, h = table.shape
    t = ids.shape[0]
    if out is None:
        out = torch.empty((t, h), dtype=torch.float32, device=table.device)
    _need(out, "embedding out", dtype=torch.float32, shape=(t, h))
    check(load().fsie_embedding(table.data_ptr(), dtype_code(table.dtype), ids.data_ptr(), out.data_ptr(),
                                t, h, v, float(scale), _stream()))
    return out


def rmsnorm(residual: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
            write_back: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm of ``residual (+ delta)`` (float32 stream) times ``weight`` (float32).  ``delta``
    is [T, H] in ``out_dtype``, or float32 [S, T, H] with S in (2, 4, 8): partial sums that are
    added in order.  ``write_back`` stores the sum into ``residual``; ``rows`` (int32) selects rows."""
    _need(residual, "rmsnorm residual", dtype=torch.float32, ndim=2)
    t, h = residual.shape
    _need(weight, "rmsnorm weight", dtype=torch.float32, shape=(h,))
    n_parts = 0
    if delta is not None and delta.ndim == 3:
        n_parts = delta.shape[0]
        _need(delta, "rmsnorm delta parts", dtype=torch.float32, shape=(n_parts, t, h))
        if not 2 <= n_parts <= GEMM_MAX_SPLITS:
            raise KernelError(f"rmsnorm: {n_parts} partial sums; 2 to {GEMM_MAX_SPLITS} are taken")
    elif delta is not None:
        _need(delta, "rmsnorm delta", dtype=out_dtype, shape=(t, h))
    n_rows = t
    if rows is not None:
        _need(rows, "rmsnorm rows", dtype=torch.int32, ndim=1)
        n_rows = rows.shape[0]
    if out is None:
        out = torch.empty((n_rows, h), dtype=out_dtype, device=residual.device)
    _need(out, "rmsnorm out", dtype=out_dtype, shape=(n_rows, h))
    check(load().fsie_rmsnorm(residual.data_ptr(), _ptr(delta), weight.data_ptr(), out.data_ptr(), _ptr(rows),
                              n_rows, h, float(eps), dtype_code(out_dtype), int(write_back), n_parts, t, _stream()))
    return out


def rmsnorm_plain(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm of a plain tensor ``x`` [T, W] (no residual stream), float32 sums: every run of
    ``weight.shape[0]`` values of a row is normalised by itself and multiplied by ``weight``
    (float32), so a weight as long as a head normalises every head of a row.  ``x`` may be a view
    whose rows are a stride apart (the q columns of a q/k/v row); ``out`` may be ``x``."""
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dim() != 2 or x.stride(1) != 1:
        raise KernelError("rmsnorm_plain x: must be a 2-d tensor on the GPU whose rows are contiguous")
    _need(weight, "rmsnorm_plain weight", dtype=torch.float32, ndim=1)
    t, w = x.shape
    width = weight.shape[0]
    if width == 0 or w % width:
        raise KernelError(f"rmsnorm_plain: rows of {w} values are not whole runs of {width}")
    if out is None:
        out = torch.empty((t, w), dtype=x.dtype, device=x.device)
    if out.shape != x.shape or out.dtype != x.dtype or out.stride(1) != 1 or not out.is_cuda:
        raise KernelError("rmsnorm_plain out: must have the shape and type of x and contiguous rows")
    check(load().fsie_rmsnorm_plain(x.data_ptr(), x.stride(0), weight.data_ptr(), out.data_ptr(), out.stride(0), t,
                                    w // width, width, float(eps), dtype_code(x.dtype), _stream()))
    return out


def zero_rows(table: torch.Tensor, slots: torch.Tensor) -> torch.Tensor:
    """``table[slots[i]] = 0`` for every non-negative entry of ``slots`` (int32); rows are whole
    multiples of four bytes."""
    _need(table, "zero_rows table")
    _need(slots, "zero_rows slots", dtype=torch.int32, ndim=1)
    if table.dim() < 1:
        raise KernelError("zero_rows: the table needs a first dimension of slots")
    row_bytes = (table.numel() // max(table.shape[0], 1)) * table.element_size()
    if row_bytes % 4:
        raise KernelError(f"zero_rows: rows of {row_bytes} bytes are not whole 4-byte words")
    check(load().fsie_zero_rows(table.data_ptr(), slots.data_ptr(), slots.shape[0], row_bytes, table.shape[0], _stream()))
    return table


def zero_pages(pool_a: torch.Tensor, pool_b: torch.Tensor, pages: torch.Tensor) -> None:
    """Pages ``pages`` (int32, negative = none) of two pools [planes, n_pages, ...] of equal page
    size set to zero in every plane."""
    _need(pool_a, "zero_pages pool")
    _need(pool_b, "zero_pages pool", dtype=pool_a.dtype)
    _need(pages, "zero_pages pages", dtype=torch.int32, ndim=1)
    if pool_a.dim() < 3 or pool_b.dim() < 3 or pool_a.shape[:2] != pool_b.shape[:2] or pool_a[0, 0].numel() != pool_b[0, 0].numel():
        raise KernelError(f"zero_pages: pools of shapes {tuple(pool_a.shape)} and {tuple(pool_b.shape)} do not go together")
    page_bytes = pool_a[0, 0].numel() * pool_a.element_size()
    check(load().fsie_zero_pages(pool_a.data_ptr(), pool_b.data_ptr(), pages.data_ptr(), pages.shape[0], pool_a.shape[0],
                                 pool_a.shape[1], page_bytes, _stream()))


def random_fill(out: torch.Tensor, key: int, init: str, std: float = 0.0) -> torch.Tensor:
    """Fill ``out`` (float32, or int32 for ``init == 'int'``) with the counter-based random values
    of the sequence ``key``: ``std * z`` ('weight', 'bias'), ``1 + std * z`` ('norm'), 15 random
    bits ('int'); element i is a function of (key, i) alone."""
    kind = {"weight": 0, "bias": 0, "norm": 1, "int": 2}.get(init)
    if kind is None:
        raise KernelError(f"random_fill: unknown init '{init}'")
    _need(out, "random_fill out", dtype=torch.int32 if kind == 2 else torch.float32)
    check(load().fsie_random_fill(out.data_ptr(), out.numel(), int(key) & ((1 << 64) - 1), kind, float(std), _stream()))
    return out


GATE_ACTS = {"silu": 0, "gelu_tanh": 1, "relu": 2}  # the activations of a gate that the kernels know


def gate_act_code(act: str) -> int:
    try:
        return GATE_ACTS[act]
    except KeyError:
        raise KernelError(f"unknown gate activation '{act}' (known: {sorted(GATE_ACTS)})") from None


def swiglu(x: torch.Tensor, out: Optional[torch.Tensor] = None, act: str = "silu") -> torch.Tensor:
    """act(x[:, 0::2]) * x[:, 1::2] for x [T, 2I] (gate and up interleaved); ``act``: "silu" or "gelu_tanh"."""
    _need(x, "swiglu input", ndim=2)
    t, two_i = x.shape
    if two_i % 2:
        raise KernelError(f"swiglu: the input width {two_i} must be even")
    inter = two_i // 2
    if out is None:
        out = torch.empty((t, inter), dtype=x.dtype, device=x.device)
    _need(out, "swiglu out", dtype=x.dtype, shape=(t, inter))
    check(load().fsie_gated_act(x.data_ptr(), out.data_ptr(), t, inter, dtype_code(x.dtype), gate_act_code(act), _stream()))
    return out


def residual_add(residual: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _need(residual, "residual", dtype=torch.float32)
    _need(delta, "delta", shape=residual.shape)
    check(load().fsie_residual_add(residual.data_ptr(), delta.data_ptr(), residual.numel(),
                                   dtype_code(delta.dtype), _stream()))
    return residual


def bias_add(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """y[r, :] += bias (float32) in place."""
    _need(y, "bias_add y", ndim=2)
    _need(bias, "bias", dtype=torch.float32, shape=(y.shape[1],))
    check(load().fsie_bias_add(y.data_ptr(), bias.data_ptr(), y.shape[0], y.shape[1], dtype_code(y.dtype), _stream()))
    return y


def sum_round(parts: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bfloat16 [M, N] from float32 partial sums [S, M, N] (or one plane [M, N]): added in their order, plus ``bias``
    (float32 [N]), rounded once.  N a multiple of 4."""
    if parts.ndim == 2:
        parts = parts.unsqueeze(0)
    _need(parts, "sum_round parts", dtype=torch.float32, ndim=3)
    s, m, n = parts.shape
    if n % 4:
        raise KernelError(f"sum_round: rows of {n} values are not a multiple of four")
    if bias is not None:
        _need(bias, "sum_round bias", dtype=torch.float32, shape=(n,))
    y = torch.empty((m, n), dtype=torch.bfloat16, device=parts.device)
    check(load().fsie_sum_round(parts.data_ptr(), s, _ptr(bias), y.data_ptr(), m, n, _stream()))
    return y


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                  inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor] = None,
                  k_pool: Optional[torch.Tensor] = None, v_pool: Optional[torch.Tensor] = None,
                  page_size: int = 0, bias: Optional[torch.Tensor] = None,
                  cos_sin: Optional[torch.Tensor] = None, parts: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate the q and k heads of ``qkv`` [T, (n_heads + 2 n_kv) head_dim] in place by the angles
    ``positions * inv_freq`` (float64 table of rotary_dim/2 entries; ``None`` = no rotation) and
    copy k and v to the cache slots ``slots`` (int32 [T], negative = not stored) of the pools: keys
    [pages, n_kv, page_size, head_dim], values [pages, n_kv, head_dim, page_size].  ``cos_sin``
    (``rope_table`` of these positions and frequencies): where the whole head is rotated and
    head_dim is a multiple of 8, the kernel reads the angles' cosines and sines there; the table
    alone, without ``inv_freq``, says that the whole head is rotated by it.
    ``parts`` (float32 [S, T, width], only with ``cos_sin``): the projection as the partial sums of a
    product cut along its inner dimension; they are added in order, ``qkv`` is then only written: its
    q columns get the rotated q heads, k and v go to the pools alone."""
    _need(qkv, "qkv", ndim=2)
    t = qkv.shape[0]
    if qkv.shape[1] != (n_heads + 2 * n_kv) * head_dim:
        raise KernelError(f"qkv: width {qkv.shape[1]} != (heads {n_heads} + 2 * kv heads {n_kv}) * {head_dim}")
    _need(positions, "positions", dtype=torch.int32, shape=(t,))
    rotary_dim = 0
    if inv_freq is not None:
        _need(inv_freq, "inv_freq", dtype=torch.float64, ndim=1)
        rotary_dim = 2 * inv_freq.shape[0]
    elif cos_sin is not None:
        if head_dim % 8:
            raise KernelError("rope_kv_write: a table of cosines and sines alone needs a head of a multiple of 8 dimensions")
        rotary_dim = head_dim
    if bias is not None:
        _need(bias, "qkv bias", dtype=torch.float32, shape=(qkv.shape[1],))
    pool_slots = 0
    if k_pool is not None:
        if v_pool is None or slots is None:
            raise KernelError("rope_kv_write: k_pool needs v_pool and slots")
        _need(slots, "slots", dtype=torch.int32, shape=(t,))
        _need(k_pool, "k_pool", dtype=qkv.dtype, ndim=4)
        _need(v_pool, "v_pool", dtype=qkv.dtype, shape=(k_pool.shape[0], n_kv, head_dim, page_size))
        if tuple(k_pool.shape[1:]) != (n_kv, page_size, head_dim):
            raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} is not [pages, {n_kv}, {page_size}, {head_dim}]")
        pool_slots = k_pool.shape[0] * page_size
    n_parts = 0
    if parts is not None:
        if cos_sin is None or rotary_dim != head_dim or head_dim % 8:
            raise KernelError("rope_kv_write: partial sums need the table of cosines and sines and a whole head "
                              "of a multiple of 8 dimensions rotated")
        n_parts = parts.shape[0] if parts.dim() == 3 else 0
        _need(parts, "qkv partial sums", dtype=torch.float32, shape=(n_parts, t, qkv.shape[1]))
        if not 1 <= n_parts <= GEMM_MAX_SPLITS:
            raise KernelError(f"rope_kv_write: {n_parts} partial sums; 1 to {GEMM_MAX_SPLITS} are taken")
    if cos_sin is not None and rotary_dim == head_dim and head_dim % 8 == 0:
        _need(cos_sin, "cos_sin", dtype=torch.float32, shape=(t, head_dim // 2, 2))
        check(load().fsie_rope_kv_write_table(qkv.data_ptr(), cos_sin.data_ptr(), _ptr(slots), _ptr(bias),
                                              _ptr(k_pool), _ptr(v_pool), t, n_heads, n_kv, head_dim, page_size,
                                              pool_slots, dtype_code(qkv.dtype), _ptr(parts), n_parts, _stream()))
        return qkv
    check(load().fsie_rope_kv_write(qkv.data_ptr(), positions.data_ptr(), _ptr(slots), _ptr(inv_freq),
                                    _ptr(bias), _ptr(k_pool), _ptr(v_pool), t, n_heads, n_kv, head_dim, rotary_dim,
                                    page_size, pool_slots, dtype_code(qkv.dtype), _stream()))
    return qkv


def gemm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
         out_dtype: Optional[torch.dtype] = None, kind: int = GEMM_AUTO,
         out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [M, K] . weight [N, K]^T + bias [N] (float32) with float32 accumulation."""
    _need(x, "gemm x", ndim=2)
    _need(weight, "gemm weight", dtype=x.dtype, ndim=2)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"gemm: weight inner size {weight.shape[1]} does not match x's {k}")
    if bias is not None:
        _need(bias, "gemm bias", dtype=torch.float32, shape=(n,))
    out_dtype = out_dtype or x.dtype
    if out_dtype not in (x.dtype, torch.float32):
        raise KernelError(f"gemm: output {out_dtype} from {x.dtype} operands is not offered")
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _need(out, "gemm out", dtype=out_dtype, shape=(m, n))
    check(load().fsie_gemm(x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), m, n, k,
                           dtype_code(x.dtype), int(out_dtype == torch.float32), kind, _stream()))
    return out


def gemm_mfma_fp32(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, waves: int = 0,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [M, K] . weight [N, K]^T + bias in true float32 on the matrix cores, for up to 64 rows and K a
    multiple of 4 (the 32-bit path's decoding).  A row's sums do not depend on the other rows."""
    _need(x, "gemm x", dtype=torch.float32, ndim=2)
    _need(weight, "gemm weight", dtype=torch.float32, ndim=2)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"gemm: weight inner size {weight.shape[1]} does not match x's {k}")
    if bias is not None:
        _need(bias, "gemm bias", dtype=torch.float32, shape=(n,))
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _need(out, "gemm out", dtype=torch.float32, shape=(m, n))
    check(load().fsie_gemm_mfma_fp32(x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), m, n, k, waves, _stream()))
    return out


def gemm_mfma_skinny(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
                     out_dtype: Optional[torch.dtype] = None, waves: int = 0, blocks: int = 0,
                     out: Optional[torch.Tensor] = None, epilogue: str = "plain", splits: int = 1) -> torch.Tensor:
    """The same product on the matrix cores for bfloat16 operands (K a multiple of 8): at most 16
    rows for a bfloat16 result, at most 64 for a float32 one.
    ``epilogue="swiglu"``: the rows of ``weight`` are gate and up interleaved and the result is
    silu(gate) * up, [M, N/2].  ``splits`` in (2, 4, 8): K is cut into that many slices and the
    result is their float32 partial sums [splits, M, N] (no bias), for ``rmsnorm`` to add up."""
    _need(x, "gemm x", dtype=torch.bfloat16, ndim=2)
    _need(weight, "gemm weight", dtype=torch.bfloat16, ndim=2)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"gemm: weight inner size {weight.shape[1]} does not match x's {k}")
    if bias is not None:
        _need(bias, "gemm bias", dtype=torch.float32, shape=(n,))
    out_dtype = out_dtype or x.dtype
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"gemm: output {out_dtype} is not offered")
    if epilogue not in ("plain", "swiglu", "geglu_tanh", "reglu"):
        raise KernelError(f"gemm: unknown epilogue '{epilogue}'")
    gated = epilogue != "plain"  # "geglu_tanh": the same with GELU (tanh form) on the gate
    if gated and n % 2:
        raise KernelError(f"gemm: the swiglu epilogue needs an even number of weight rows, found {n}")
    n_out = n // 2 if gated else n
    shape = (m, n_out)
    if splits != 1:
        if splits not in GEMM_SPLITS or epilogue != "plain" or bias is not None:
            raise KernelError(f"gemm: partial sums come in {GEMM_SPLITS} slices, without bias or epilogue")
        out_dtype, shape = torch.float32, (splits, m, n)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    _need(out, "gemm out", dtype=out_dtype, shape=shape)
    check(load().fsie_gemm_mfma_skinny(x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), m, n, k,
                                       int(out_dtype == torch.float32), waves, blocks,
                                       {"plain": 0, "swiglu": 1, "geglu_tanh": 2, "reglu": 3}[epilogue],
                                       splits, _stream()))
    return out


class FragmentOrdered:
    """The copy of a bfloat16 matrix [rows, cols] in the order of the matrix instruction's A
    fragments (``fragment_order``): the 64 16-byte units of a block of 16 rows and 32 columns lie
    together in the order of the lanes that hold them, so that a wave's load of the weight is one
    piece of 1 KB and can be a streaming load.  ``gemm_mfma_wide`` and ``gemm_mfma_wide_swiglu``
    take it in place of the matrix."""

    __slots__ = ("data", "rows", "cols")

    def __init__(self, data: torch.Tensor, rows: int, cols: int):
        self.data, self.rows, self.cols = data, rows, cols

    @property
    def shape(self):
        return (self.rows, self.cols)


def fragment_order(weight: torch.Tensor) -> FragmentOrdered:
    """The copy of ``weight`` [N, K] (bfloat16, K a multiple of 32) in fragment order; the rows that
    fill N up to a multiple of 16 are zeros."""
    _need(weight, "fragment_order weight", dtype=torch.bfloat16, ndim=2)
    n, k = weight.shape
    size = int(load().fsie_fragment_order_size(n, k))
    if size <= 0:
        raise KernelError(f"fragment_order: the inner size {k} must be a multiple of 32")
    data = torch.empty(size, dtype=torch.bfloat16, device=weight.device)
    check(load().fsie_fragment_order(weight.data_ptr(), data.data_ptr(), n, k, _stream()))
    return FragmentOrdered(data, n, k)


def _wide_weight(weight, k: int):
    """(pointer, N, whether it is in fragment order) of a weight given to the wide products."""
    if isinstance(weight, FragmentOrdered):
        _need(weight.data, "gemm weight", dtype=torch.bfloat16, ndim=1)
        n, kw, ptr, frags = weight.rows, weight.cols, weight.data.data_ptr(), 1
    else:
        _need(weight, "gemm weight", dtype=torch.bfloat16, ndim=2)
        n, kw, ptr, frags = weight.shape[0], weight.shape[1], weight.data_ptr(), 0
    if kw != k:
        raise KernelError(f"gemm: weight inner size {kw} does not match x's {k}")
    return ptr, n, frags


def gemm_mfma_wide_takes(m: int, weight, splits: int = 1, gate_up: bool = False) -> bool:
    """Whether ``gemm_mfma_wide`` (``gate_up``: ``gemm_mfma_wide_swiglu``) takes ``m`` rows against this
    weight in ``splits`` slices: up to 64 rows wherever it takes the inner size; 65 to 128 rows only on a
    ``FragmentOrdered`` copy, for the launch shapes that have kernels of five to eight tiles of rows."""
    n, k = weight.shape
    return bool(load().fsie_gemm_mfma_wide_takes(int(m), int(n), int(k), int(splits), int(gate_up),
                                                 int(isinstance(weight, FragmentOrdered))))


def gemm_mfma_wide_splits_ok(k: int, splits: int) -> bool:
    """Whether ``gemm_mfma_wide`` can cut an inner size ``k`` into ``splits`` slices (whole stages
    of 128 values each)."""
    return load().fsie_gemm_mfma_wide_slice(int(k), int(splits)) > 0


def gemm_mfma_wide_swiglu(x: torch.Tensor, weight: torch.Tensor, waves: int = 0, blocks: int = 0,
                          out: Optional[torch.Tensor] = None, act: str = "silu") -> torch.Tensor:
    """silu(gate) * up [M, N/2] (bfloat16) of x [M, K] and a weight [N, K] whose rows are gate and up
    in turn (or its ``FragmentOrdered`` copy), by the kernel that shares x through LDS; up to 64
    rows, N a multiple of 4, K of 128."""
    _need(x, "gemm x", dtype=torch.bfloat16, ndim=2)
    m, k = x.shape
    wptr, n, frags = _wide_weight(weight, k)
    if n % 4:
        raise KernelError(f"gemm_mfma_wide_swiglu: the number of weight rows {n} must be a multiple of 4")
    if out is None:
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    _need(out, "gemm out", dtype=torch.bfloat16, shape=(m, n // 2))
    check(load().fsie_gemm_mfma_wide_gated(x.data_ptr(), wptr, out.data_ptr(), m, n, k, waves, blocks, frags,
                                           gate_act_code(act), _stream()))
    return out


def gemm_mfma_wide_best_splits(m: int, n: int, k: int) -> int:
    """Into how many slices of K ``gemm_mfma_wide`` best cuts a product of ``m`` rows that leaves
    partial sums (1: it does not cut, or does not take this K)."""
    return int(load().fsie_gemm_mfma_wide_best_splits(int(m), int(n), int(k)))


def gemm_mfma_wide(x: torch.Tensor, weight: torch.Tensor, splits: int = 1, waves: int = 0,
                   out: Optional[torch.Tensor] = None, blocks: int = 0) -> torch.Tensor:
    """x [M, K] . weight [N, K]^T for bfloat16 operands and up to 64 rows, the rows of x shared by
    a workgroup's waves through LDS (made for 17 rows and more); ``weight`` may be the matrix's
    ``FragmentOrdered`` copy.  The result is float32: [M, N],
    or with ``splits`` of 2 to 16 the partial sums [splits, M, N] of the slices of K, for
    ``rmsnorm`` to add up.  K must be a multiple of 128 that the slices cover in whole stages
    (``gemm_mfma_wide_splits_ok``)."""
    _need(x, "gemm x", dtype=torch.bfloat16, ndim=2)
    m, k = x.shape
    wptr, n, frags = _wide_weight(weight, k)
    if not 1 <= splits <= GEMM_MAX_SPLITS:
        raise KernelError(f"gemm_mfma_wide: splits must be 1 to {GEMM_MAX_SPLITS}, got {splits}")
    shape = (m, n) if splits == 1 else (splits, m, n)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32, device=x.device)
    _need(out, "gemm out", dtype=torch.float32, shape=shape)
    check(load().fsie_gemm_mfma_wide(x.data_ptr(), wptr, out.data_ptr(), m, n, k, splits, waves, blocks, frags,
                                     _stream()))
    return out


def gemm_mfma_skinny_rope(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                          positions: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                          inv_freq: Optional[torch.Tensor], slots: Optional[torch.Tensor] = None,
                          k_pool: Optional[torch.Tensor] = None, v_pool: Optional[torch.Tensor] = None,
                          page_size: int = 0, cos_sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The fused q/k/v projection x [M, K] . weight [(n_heads + 2 n_kv) head_dim, K]^T of at most 64
    rows (bfloat16) with the position encoding in its epilogue: bias, rotation of the q and k
    heads over the whole head (``inv_freq``: float64 [head_dim / 2], ``None`` = none) and the
    write of k and v into the cache pools at ``slots``.  ``cos_sin``: what ``rope_table`` made of
    these positions and frequencies (the kernel then reads the cosines and sines instead of
    computing them; the table may come without ``inv_freq``).  Returns [M, N] whose q columns are filled; the k and v columns are not
    written."""
    _need(x, "gemm x", dtype=torch.bfloat16, ndim=2)
    _need(weight, "gemm weight", dtype=torch.bfloat16, ndim=2)
    m, k = x.shape
    n = (n_heads + 2 * n_kv) * head_dim
    if tuple(weight.shape) != (n, k):
        raise KernelError(f"gemm: weight shape {tuple(weight.shape)} is not [{n}, {k}]")
    if bias is not None:
        _need(bias, "qkv bias", dtype=torch.float32, shape=(n,))
    _need(positions, "positions", dtype=torch.int32, shape=(m,))
    if inv_freq is not None:
        _need(inv_freq, "inv_freq", dtype=torch.float64, shape=(head_dim // 2,))
    if cos_sin is not None:
        _need(cos_sin, "cos_sin", dtype=torch.float32, shape=(m, head_dim // 2, 2))
    pool_slots = 0
    if k_pool is not None:
        if v_pool is None or slots is None:
            raise KernelError("gemm_mfma_skinny_rope: k_pool needs v_pool and slots")
        _need(slots, "slots", dtype=torch.int32, shape=(m,))
        _need(k_pool, "k_pool", dtype=torch.bfloat16, ndim=4)
        _need(v_pool, "v_pool", dtype=torch.bfloat16, shape=(k_pool.shape[0], n_kv, head_dim, page_size))
        if tuple(k_pool.shape[1:]) != (n_kv, page_size, head_dim):
            raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} is not [pages, {n_kv}, {page_size}, {head_dim}]")
        pool_slots = k_pool.shape[0] * page_size
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    check(load().fsie_gemm_mfma_skinny_rope(x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(), m, k,
                                            positions.data_ptr(), _ptr(slots), _ptr(inv_freq), _ptr(cos_sin),
                                            _ptr(k_pool), _ptr(v_pool), n_heads, n_kv, head_dim, page_size, pool_slots,
                                            _stream()))
    return out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, magnitude: float = 1.0) -> torch.Tensor:
    """float32 [T, half, 2]: cos and sin of positions[t] * inv_freq[i] (the angle in float64, as in
    the kernels that rotate), each times ``magnitude``.  The angles of a step are the same in every
    layer: a step makes the table once."""
    _need(positions, "positions", dtype=torch.int32, ndim=1)
    _need(inv_freq, "inv_freq", dtype=torch.float64, ndim=1)
    t, half = positions.shape[0], inv_freq.shape[0]
    table = torch.empty((t, half, 2), dtype=torch.float32, device=positions.device)
    check(load().fsie_rope_table_scaled(positions.data_ptr(), inv_freq.data_ptr(), t, half, float(magnitude),
                                        table.data_ptr(), _stream()))
    return table


def attention_tile_tokens(n_heads: int, n_kv: int) -> int:
    n = load().fsie_attention_scalar_tile_tokens(n_heads, n_kv)
    if n <= 0:
        raise KernelError(f"attention: heads {n_heads} must be a positive multiple of kv heads {n_kv}")
    return n


def attention_scalar(q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                     block_tables: torch.Tensor, items: torch.Tensor, n_items: int, out: torch.Tensor,
                     partials: Optional[torch.Tensor], n_heads: int, n_kv: int, head_dim: int,
                     window: Optional[int], scale: float, n_query_rows: int,
                     sinks: Optional[torch.Tensor] = None, softcap: float = 0.0, pooled=None) -> torch.Tensor:
    """Attention of the work items over the paged cache (float32 arithmetic).  ``sinks`` (float32 [n_heads],
    here and in the other attention functions): exp(sinks[h]) is one more term of the denominator of
    head h's softmax, with no key and no value.  ``pooled`` = (k_pool, v_pool, block_tables, block_tokens) of the
    pools of pooled blocks (one mean key and value for every ``block_tokens`` positions): items flagged
    ``ATTN_POOL_WALK`` also read the blocks that lie wholly before their queries' windows.

    ``q`` is a view into rows of stride ``q_stride`` elements whose first n_heads*head_dim columns
    are the queries; ``out`` is [n_query_rows, n_heads*head_dim]."""
    if not q.is_cuda:
        raise KernelError("attention q: must be on the GPU")
    _need(k_pool, "k_pool", dtype=q.dtype, ndim=4)
    _need(v_pool, "v_pool", dtype=q.dtype, shape=(k_pool.shape[0], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]))
    _need(block_tables, "block_tables", dtype=torch.int32, ndim=2)
    _need(items, "attention items", dtype=torch.int32, ndim=2)
    if items.shape[1] != ATTN_ITEM_INTS or items.shape[0] < n_items:
        raise KernelError(f"attention items: shape {tuple(items.shape)} does not hold {n_items} items")
    _need(out, "attention out", dtype=q.dtype, shape=(n_query_rows, n_heads * head_dim))
    pages, kvh, page_size, hd = k_pool.shape
    if kvh != n_kv or hd != head_dim:
        raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} does not match kv heads {n_kv}, head_dim {head_dim}")
    if q_stride < n_heads * head_dim:
        raise KernelError("attention: q_stride is smaller than the query width")
    if partials is not None:
        _need(partials, "attention partials", dtype=torch.float32, ndim=1)
    pooled_args = (None, None, None, 0, 0, 0)
    if pooled is not None:
        pk, pv, ptab, block_tokens = pooled
        _need(pk, "pooled k_pool", dtype=q.dtype, ndim=4)
        _need(pv, "pooled v_pool", dtype=q.dtype, shape=(pk.shape[0], pk.shape[1], pk.shape[3], pk.shape[2]))
        _need(ptab, "pooled block_tables", dtype=torch.int32, ndim=2)
        if pk.shape[1] != n_kv or pk.shape[3] != head_dim or ptab.shape[0] != block_tables.shape[0] or not window:
            raise KernelError("attention: the pools of pooled blocks do not fit the layer (heads, head size, requests, a window)")
        pooled_args = (pk.data_ptr(), pv.data_ptr(), ptab.data_ptr(), ptab.shape[1], pk.shape[2], int(block_tokens))
    check(load().fsie_attention_scalar(q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                                       block_tables.data_ptr(), block_tables.shape[1], items.data_ptr(),
                                       n_items, out.data_ptr(), _ptr(partials), n_heads, n_kv, head_dim,
                                       page_size, int(window or 0), float(scale), dtype_code(q.dtype),
                                       _sinks_ptr(sinks, n_heads), float(softcap or 0.0), *pooled_args, _stream()))
    return out


def pool_blocks(k_pool: torch.Tensor, v_pool: torch.Tensor, block_tables: torch.Tensor, k_pooled: torch.Tensor,
                v_pooled: torch.Tensor, pooled_tables: torch.Tensor, jobs: torch.Tensor, n_jobs: int, block_tokens: int) -> None:
    """The mean key and value of every block of ``block_tokens`` positions that ``jobs`` int32 [n, 2] names (request of
    the step, block; request -1: nothing), read from the pages of keys and values and written to the pools of pooled
    blocks at the entry of the block (float32 sums in the order of the positions)."""
    _need(k_pool, "k_pool", ndim=4)
    units, n_kv, page_size, hd = k_pool.shape
    _need(v_pool, "v_pool", dtype=k_pool.dtype, shape=(units, n_kv, hd, page_size))
    _need(k_pooled, "pooled k_pool", dtype=k_pool.dtype, ndim=4)
    if k_pooled.shape[1] != n_kv or k_pooled.shape[3] != hd:
        raise KernelError("pool_blocks: the pools of pooled blocks hold other heads")
    _need(v_pooled, "pooled v_pool", dtype=k_pool.dtype, shape=(k_pooled.shape[0], n_kv, hd, k_pooled.shape[2]))
    _need(block_tables, "block_tables", dtype=torch.int32, ndim=2)
    _need(pooled_tables, "pooled block_tables", dtype=torch.int32, ndim=2)
    _need(jobs, "pool_blocks jobs", dtype=torch.int32, ndim=2)
    if jobs.shape[1] != 2 or jobs.shape[0] < n_jobs or pooled_tables.shape[0] != block_tables.shape[0]:
        raise KernelError("pool_blocks: bad tables")
    check(load().fsie_pool_blocks(k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(), block_tables.shape[1],
                                  page_size, k_pooled.data_ptr(), v_pooled.data_ptr(), pooled_tables.data_ptr(),
                                  pooled_tables.shape[1], k_pooled.shape[2], jobs.data_ptr(), int(n_jobs), int(block_tokens),
                                  n_kv, hd, dtype_code(k_pool.dtype), _stream()))


def round_to(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The float32 tensor ``x`` in ``dtype`` (rounded to nearest even; a copy for float32)."""
    _need(x, "round_to x", dtype=torch.float32)
    y = torch.empty(x.shape, dtype=dtype, device=x.device)
    check(load().fsie_round_to(x.data_ptr(), y.data_ptr(), x.numel(), dtype_code(dtype), _stream()))
    return y


def scaled_sum(x1: torch.Tensor, a: float, x2: torch.Tensor, b: float) -> torch.Tensor:
    """a * x1 + b * x2 in float32, rounded once to the operands' type."""
    _need(x1, "scaled_sum x1")
    _need(x2, "scaled_sum x2", dtype=x1.dtype, shape=tuple(x1.shape))
    y = torch.empty_like(x1)
    check(load().fsie_scaled_sum(x1.data_ptr(), float(a), x2.data_ptr(), float(b), y.data_ptr(), x1.numel(),
                                 dtype_code(x1.dtype), _stream()))
    return y


def attention_mfma_rows(head_dim: int, large: bool) -> int:
    """Query rows (tokens x heads of a kv head's group) that one work item of the matrix-core
    attention holds; 0 if the head size is not offered."""
    return 16 * load().fsie_attention_mfma_tiles(head_dim, int(large))


def compute_units() -> int:
    """Compute units of the current device; 0 where there is none to ask."""
    return load().fsie_device_compute_units()


def attention_mfma_max_waves(head_dim: int) -> int:
    return load().fsie_attention_mfma_max_waves(head_dim)


def attention_mfma(q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                   block_tables: torch.Tensor, items: torch.Tensor, n_items: int, out: torch.Tensor,
                   partials: Optional[torch.Tensor], n_heads: int, n_kv: int, head_dim: int,
                   window: Optional[int], scale: float, n_query_rows: int, large: bool, waves: int = 1,
                   sinks: Optional[torch.Tensor] = None, softcap: float = 0.0) -> torch.Tensor:
    """Attention of the work items over the paged cache on the matrix cores (bfloat16; head_dim a
    multiple of 16; page size a multiple of 4).  ``items`` may be a view into a longer table.
    ``waves`` waves of a workgroup split each item's keys and combine inside the workgroup."""
    if not q.is_cuda or q.dtype != torch.bfloat16:
        raise KernelError("attention_mfma q: must be bfloat16 on the GPU")
    _need(k_pool, "k_pool", dtype=q.dtype, ndim=4)
    _need(v_pool, "v_pool", dtype=q.dtype, shape=(k_pool.shape[0], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]))
    _need(block_tables, "block_tables", dtype=torch.int32, ndim=2)
    _need(items, "attention items", dtype=torch.int32, ndim=2)
    if items.shape[1] != ATTN_ITEM_INTS or items.shape[0] < n_items:
        raise KernelError(f"attention items: shape {tuple(items.shape)} does not hold {n_items} items")
    _need(out, "attention out", dtype=q.dtype, shape=(n_query_rows, n_heads * head_dim))
    pages, kvh, page_size, hd = k_pool.shape
    if kvh != n_kv or hd != head_dim:
        raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} does not match kv heads {n_kv}, head_dim {head_dim}")
    if q_stride < n_heads * head_dim:
        raise KernelError("attention: q_stride is smaller than the query width")
    if partials is not None:
        _need(partials, "attention partials", dtype=torch.float32, ndim=1)
    check(load().fsie_attention_mfma(q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                                     block_tables.data_ptr(), block_tables.shape[1], items.data_ptr(), n_items,
                                     out.data_ptr(), _ptr(partials), n_heads, n_kv, head_dim, page_size,
                                     int(window or 0), float(scale), int(large), int(waves),
                                     _sinks_ptr(sinks, n_heads), float(softcap or 0.0), _stream()))
    return out


def attention_mfma_qkv_ok(head_dim: int, page_size: int) -> bool:
    """Whether the attention kernel that finishes the q/k/v product itself takes this geometry."""
    return bool(load().fsie_attention_mfma_qkv_ok(head_dim, page_size))


def attention_mfma_qkv(sums: torch.Tensor, bias: Optional[torch.Tensor], cos_sin: torch.Tensor, slots: torch.Tensor,
                       k_pool: torch.Tensor, v_pool: torch.Tensor, block_tables: torch.Tensor, items: torch.Tensor,
                       n_items: int, out: torch.Tensor, partials: Optional[torch.Tensor], n_heads: int, n_kv: int,
                       head_dim: int, window: Optional[int], scale: float, waves: int = 1) -> torch.Tensor:
    """Attention of a step of one token a request (every item: one query row a head) from the q/k/v
    product's float32 partial sums [S, T, (heads + 2 kv heads) head_dim]: the kernel adds them up, adds
    ``bias``, rotates queries and keys by ``cos_sin`` [T, head_dim / 2, 2], scores each request's new key
    from registers and writes it and the value to ``slots[t]`` of the pools (negative: nowhere)."""
    width = (n_heads + 2 * n_kv) * head_dim
    _need(sums, "q/k/v sums", dtype=torch.float32, ndim=3)
    n_parts, t = sums.shape[0], sums.shape[1]
    if sums.shape[2] != width or t < 1:
        raise KernelError(f"q/k/v sums: shape {tuple(sums.shape)} does not hold rows of {width}")
    if bias is not None:
        _need(bias, "q/k/v bias", dtype=torch.float32, shape=(width,))
    _need(cos_sin, "cos_sin", dtype=torch.float32)
    if cos_sin.numel() != t * head_dim:
        raise KernelError(f"cos_sin: {cos_sin.numel()} values for {t} tokens of head_dim {head_dim}")
    _need(slots, "slots", dtype=torch.int32, shape=(t,))
    _need(k_pool, "k_pool", dtype=torch.bfloat16, ndim=4)
    _need(v_pool, "v_pool", dtype=torch.bfloat16,
          shape=(k_pool.shape[0], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]))
    _need(block_tables, "block_tables", dtype=torch.int32, ndim=2)
    _need(items, "attention items", dtype=torch.int32, ndim=2)
    if items.shape[1] != ATTN_ITEM_INTS or items.shape[0] < n_items:
        raise KernelError(f"attention items: shape {tuple(items.shape)} does not hold {n_items} items")
    _need(out, "attention out", dtype=torch.bfloat16, shape=(t, n_heads * head_dim))
    pages, kvh, page_size, hd = k_pool.shape
    if kvh != n_kv or hd != head_dim:
        raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} does not match kv heads {n_kv}, head_dim {head_dim}")
    if partials is not None:
        _need(partials, "attention partials", dtype=torch.float32, ndim=1)
    check(load().fsie_attention_mfma_qkv(sums.data_ptr(), n_parts, t, _ptr(bias), cos_sin.data_ptr(), slots.data_ptr(),
                                         k_pool.data_ptr(), v_pool.data_ptr(), pages * page_size,
                                         block_tables.data_ptr(), block_tables.shape[1], items.data_ptr(), n_items,
                                         out.data_ptr(), _ptr(partials), n_heads, n_kv, head_dim, page_size,
                                         int(window or 0), float(scale), int(waves), _stream()))
    return out


def attention_mfma_lds_ok(head_dim: int, page_size: int) -> bool:
    """Whether the kernel that shares a block of keys among four waves takes this geometry."""
    return bool(load().fsie_attention_mfma_lds_ok(head_dim, page_size))


def attention_mfma_lds(q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                       block_tables: torch.Tensor, items: torch.Tensor, groups: torch.Tensor, n_groups: int,
                       out: torch.Tensor, n_heads: int, n_kv: int, head_dim: int, window: Optional[int], scale: float,
                       n_query_rows: int, sinks: Optional[torch.Tensor] = None, softcap: float = 0.0) -> torch.Tensor:
    """Attention of large work items (long portions) with the keys and values of a block staged in
    LDS for four tiles at once.  ``groups`` int32 [n, 2]: index in ``items`` of a group's first
    tile and its number of tiles (1..4, consecutive tiles of one request)."""
    if not q.is_cuda or q.dtype != torch.bfloat16:
        raise KernelError("attention_mfma_lds q: must be bfloat16 on the GPU")
    _need(k_pool, "k_pool", dtype=q.dtype, ndim=4)
    _need(v_pool, "v_pool", dtype=q.dtype, shape=(k_pool.shape[0], k_pool.shape[1], k_pool.shape[3], k_pool.shape[2]))
    _need(block_tables, "block_tables", dtype=torch.int32, ndim=2)
    _need(items, "attention items", dtype=torch.int32, ndim=2)
    _need(groups, "attention groups", dtype=torch.int32, ndim=2)
    if items.shape[1] != ATTN_ITEM_INTS or groups.shape[1] != 2 or groups.shape[0] < n_groups:
        raise KernelError(f"attention: items {tuple(items.shape)} / groups {tuple(groups.shape)} do not hold {n_groups} groups")
    _need(out, "attention out", dtype=q.dtype, shape=(n_query_rows, n_heads * head_dim))
    pages, kvh, page_size, hd = k_pool.shape
    if kvh != n_kv or hd != head_dim:
        raise KernelError(f"k_pool: shape {tuple(k_pool.shape)} does not match kv heads {n_kv}, head_dim {head_dim}")
    if q_stride < n_heads * head_dim:
        raise KernelError("attention: q_stride is smaller than the query width")
    check(load().fsie_attention_mfma_lds(q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                                         block_tables.data_ptr(), block_tables.shape[1], items.data_ptr(),
                                         groups.data_ptr(), n_groups, out.data_ptr(), n_heads, n_kv, head_dim,
                                         page_size, int(window or 0), float(scale), _sinks_ptr(sinks, n_heads),
                                         float(softcap or 0.0), _stream()))
    return out


def _sinks_ptr(sinks: Optional[torch.Tensor], n_heads: int) -> Optional[int]:
    if sinks is None:
        return None
    _need(sinks, "attention sinks", dtype=torch.float32, shape=(n_heads,))
    return sinks.data_ptr()


def attention_merge(partials: torch.Tensor, merges: torch.Tensor, n_merges: int, out: torch.Tensor,
                    n_heads: int, head_dim: int, sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``sinks``: added to the denominator once, after the splits (the items that left the records ignored it)."""
    _need(partials, "attention partials", dtype=torch.float32, ndim=1)
    _need(merges, "attention merges", dtype=torch.int32, ndim=2)
    if merges.shape[1] != ATTN_MERGE_INTS or merges.shape[0] < n_merges:
        raise KernelError(f"attention merges: shape {tuple(merges.shape)} does not hold {n_merges} items")
    _need(out, "attention out", ndim=2)
    check(load().fsie_attention_merge(partials.data_ptr(), merges.data_ptr(), n_merges, out.data_ptr(),
                                      n_heads, head_dim, dtype_code(out.dtype), _sinks_ptr(sinks, n_heads), _stream()))
    return out


def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           top_k: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
           uniform: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token id per row of float32 ``logits`` [n, V]: argmax where temperature <= 0 (or no
    temperatures are given), else temperature/top-k/top-p sampling against ``uniform`` (float64)."""
    _need(logits, "logits", dtype=torch.float32, ndim=2)
    n, v = logits.shape
    if temperature is not None:
        _need(temperature, "temperature", dtype=torch.float32, shape=(n,))
        if uniform is None:
            raise KernelError("sample: temperatures need uniform numbers")
        _need(uniform, "uniform", dtype=torch.float64, shape=(n,))
    if top_k is not None:
        _need(top_k, "top_k", dtype=torch.int32, shape=(n,))
    if top_p is not None:
        _need(top_p, "top_p", dtype=torch.float32, shape=(n,))
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _need(out, "sample out", dtype=torch.int32, shape=(n,))
    check(load().fsie_sample(logits.data_ptr(), n, v, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                             _ptr(uniform), out.data_ptr(), _stream()))
    return out


# ---------------------------------------------------------------------------------------------
# a layer with a norm before and after every sublayer; norms of heads with a gate; the logits' cap
# ---------------------------------------------------------------------------------------------
def sandwich_norm(residual: torch.Tensor, delta: torch.Tensor, post_weight: torch.Tensor, post_eps: float,
                  weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                  write_back: bool = False) -> torch.Tensor:
    """``v = residual + rmsnorm(delta; post_weight, post_eps)``, then ``rmsnorm(v; weight, eps)`` in
    ``out_dtype``, one pass.  ``delta`` as for ``rmsnorm``; ``write_back`` stores v into ``residual``
    (not with ``rows``, which selects the rows to work on)."""
    _need(residual, "sandwich_norm residual", dtype=torch.float32, ndim=2)
    t, h = residual.shape
    if weight is not None:  # (None: the result is v itself, rounded to ``out_dtype``)
        _need(weight, "sandwich_norm weight", dtype=torch.float32, shape=(h,))
    _need(post_weight, "sandwich_norm post weight", dtype=torch.float32, shape=(h,))
    n_parts = 0
    if delta.ndim == 2 and delta.dtype == torch.float32 and out_dtype != torch.float32:
        delta = delta.unsqueeze(0)  # a float32 delta beside 16-bit activations (the experts' sum): one plane of sums
    if delta.ndim == 3:
        n_parts = delta.shape[0]
        _need(delta, "sandwich_norm delta parts", dtype=torch.float32, shape=(n_parts, t, h))
        if not 1 <= n_parts <= GEMM_MAX_SPLITS:
            raise KernelError(f"sandwich_norm: {n_parts} partial sums; up to {GEMM_MAX_SPLITS} are taken")
    else:
        _need(delta, "sandwich_norm delta", dtype=out_dtype, shape=(t, h))
    n_rows = t
    if rows is not None:
        _need(rows, "sandwich_norm rows", dtype=torch.int32, ndim=1)
        n_rows = rows.shape[0]
        if write_back:
            raise KernelError("sandwich_norm: chosen rows are not written back")
    out = torch.empty((n_rows, h), dtype=out_dtype, device=residual.device)
    check(load().fsie_sandwich_norm(residual.data_ptr(), delta.data_ptr(), post_weight.data_ptr(), float(post_eps),
                                    _ptr(weight), float(eps), out.data_ptr(), _ptr(rows), n_rows, h,
                                    dtype_code(out_dtype), int(write_back), n_parts, t, _stream()))
    return out


def _columns_of(out: Optional[torch.Tensor], t: int, width: int, dtype, device, name: str) -> torch.Tensor:
    """``out`` (or a new tensor) as the place of a result [t, width]: it may be a run of columns of wider rows."""
    if out is None:
        return torch.empty((t, width), dtype=dtype, device=device)
    if (not out.is_cuda or out.dim() != 2 or tuple(out.shape) != (t, width) or out.dtype != dtype or out.stride(1) != 1
            or out.stride(0) < width):
        raise KernelError(f"{name} out: must be [{t}, {width}] of {dtype} on the GPU, rows contiguous (columns of wider rows may do)")
    return out


def gated_headnorm(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float, heads: int,
                   act: str = "silu", out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """``rmsnorm(o[t, h]; weight, eps) * act(gate[t, h])`` for every token and head: ``o`` float32
    [T, heads * width] (or [P, T, heads * width]: planes that are added in order first), ``weight`` float32
    [width] (shared by the heads), ``gate`` [T, heads * width] in the activations' type (it may be columns of
    wider rows); the result has the gate's type.  ``out``: where it goes (columns of wider rows may do); ``scale``: a
    factor on it, applied before the one rounding."""
    if o.dim() == 2:
        o = o.unsqueeze(0)
    _need(o, "gated_headnorm o", dtype=torch.float32, ndim=3)
    _need(weight, "gated_headnorm weight", dtype=torch.float32, ndim=1)
    planes, t, total = o.shape
    width = weight.shape[0]
    if total != heads * width:
        raise KernelError(f"gated_headnorm: rows of {total} values are not {heads} heads of {width}")
    if not gate.is_cuda or gate.dim() != 2 or gate.stride(1) != 1 or tuple(gate.shape) != (t, total):
        raise KernelError("gated_headnorm gate: must be [T, heads * width] on the GPU with contiguous rows")
    out = _columns_of(out, t, total, gate.dtype, o.device, "gated_headnorm")
    check(load().fsie_gated_headnorm(o.data_ptr(), planes, gate.data_ptr(), gate.stride(0), weight.data_ptr(), out.data_ptr(), t,
                                     heads, width, float(eps), gate_act_code(act), dtype_code(gate.dtype), out.stride(0) if t else total,
                                     float(scale), _stream()))
    return out


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x <- cap * tanh(x / cap)`` in place (float32)."""
    _need(x, "softcap x", dtype=torch.float32)
    check(load().fsie_softcap(x.data_ptr(), x.numel(), float(cap), _stream()))
    return x


# ---------------------------------------------------------------------------------------------
# gated linear attention
# ---------------------------------------------------------------------------------------------
def gla_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, z: torch.Tensor, state: torch.Tensor,
             q_starts: torch.Tensor, seq_slots: torch.Tensor, heads: int, dim: int, vdim: int, q_scale: float,
             inv_tau: float, chunked: bool = True, head_decay: Optional[torch.Tensor] = None,
             qk: Optional[torch.Tensor] = None, cos_sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """S <- diag(sigmoid(z_t)^inv_tau) S + k_t v_t^T, o_t = S^T (q_scale q_t) over the tokens of every
    request of the step, from and to ``state`` float32 [slots, heads, dim, vdim].  ``proj`` [T, W] holds the
    q, k (heads x dim) and v (heads x vdim) columns from ``q_off``, ``k_off``, ``v_off``; ``z`` float32
    [T, heads * dim]; ``q_starts`` int32 [n + 1], ``seq_slots`` int32 [n].  Returns o float32 [P, T, heads * vdim]:
    the shares of the P groups of key channels that the kernel deals a head's state to (P follows from the
    sizes alone); their sum in order is o, and ``gated_headnorm`` takes them as they are.  Long portions are
    computed chunk by chunk on the matrix cores (the same sums in another order); ``chunked=False`` walks
    every portion token by token."""
    _need(proj, "gla proj", ndim=2)
    t, w = proj.shape
    if head_decay is not None:
        # a fixed decay a head (float32 [heads]) instead of the decays of every token and key channel
        _need(head_decay, "gla head decay", dtype=torch.float32, shape=(heads,))
    else:
        _need(z, "gla z", dtype=torch.float32, shape=(t, heads * dim))
    _need(state, "gla state", dtype=torch.float32, ndim=4)
    if tuple(state.shape[1:]) != (heads, dim, vdim):
        raise KernelError(f"gla state: shape {tuple(state.shape)} is not [slots, {heads}, {dim}, {vdim}]")
    _need(q_starts, "gla q_starts", dtype=torch.int32, ndim=1)
    _need(seq_slots, "gla seq_slots", dtype=torch.int32, ndim=1)
    n = seq_slots.shape[0]
    if q_starts.shape[0] != n + 1:
        raise KernelError("gla: q_starts must have one entry more than seq_slots")
    if qk is not None:
        # q and k in rows of their own [T, W'] (the same column offsets): what a caller has turned by the positions
        _need(qk, "gla q and k", dtype=proj.dtype, ndim=2)
        if qk.shape[0] != t:
            raise KernelError("gla: a row of q and k a token")
    rot_pairs = 0
    if cos_sin is not None:
        # the step's cosines and sines [T, pairs, 2]: the first 2 * pairs channels of every q and k head are turned as
        # they are read, channel i with channel i + pairs
        _need(cos_sin, "gla cos/sin", dtype=torch.float32, ndim=3)
        rot_pairs = cos_sin.shape[1]
        if tuple(cos_sin.shape) != (t, rot_pairs, 2) or 2 * rot_pairs > dim:
            raise KernelError(f"gla: cosines and sines {tuple(cos_sin.shape)} do not fit {t} tokens and heads of {dim}")
    per_token, planes, chunk_tokens, chunk_min = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    chunk_floats = ctypes.c_int64(0)
    check(load().fsie_gla_scan_shape(heads, dim, vdim, ctypes.byref(per_token), ctypes.byref(planes),
                                     ctypes.byref(chunk_tokens), ctypes.byref(chunk_min), ctypes.byref(chunk_floats)))
    prep = torch.empty((t * per_token.value,), dtype=torch.float32, device=proj.device)
    out = torch.empty((planes.value, t, heads * vdim), dtype=torch.float32, device=proj.device)
    # a step of single tokens (t == n, as every captured decode step is) has no portion to cut into chunks
    max_chunks = t // chunk_tokens.value + n if chunked and t > n and t >= chunk_min.value else 0
    work = torch.empty((max_chunks * chunk_floats.value,), dtype=torch.float32, device=proj.device) if max_chunks else None
    check(load().fsie_gla_scan(proj.data_ptr(), w, q_off, k_off, v_off, _ptr(z), state.data_ptr(), q_starts.data_ptr(),
                               seq_slots.data_ptr(), n, t, prep.data_ptr(), out.data_ptr(),
                               work.data_ptr() if work is not None else None, max_chunks, heads, dim, vdim, float(q_scale),
                               float(inv_tau), state.shape[0], dtype_code(proj.dtype), _ptr(head_decay), _ptr(qk),
                               qk.shape[1] if qk is not None else 0, _ptr(cos_sin), rot_pairs, _stream()))
    return out


# ---------------------------------------------------------------------------------------------
# attention through a latent
# ---------------------------------------------------------------------------------------------
def latent_prep(proj: torch.Tensor, dq_off: int, q_rank: int, dkv_off: int, kv_rank: int, rot_dim: int, rot_pairs: int,
                g_off: int, heads: int, q_weight: torch.Tensor, kv_weight: Optional[torch.Tensor], eps: float,
                cos_sin: Optional[torch.Tensor], slots: Optional[torch.Tensor] = None,
                k_pool: Optional[torch.Tensor] = None, v_pool: Optional[torch.Tensor] = None):
    """From the fused projection ``proj`` [T, W]: the normed query latent [T, q_rank] (type of ``proj``), the
    sigmoid of the heads' gates (float32 [T, heads]) and, if pools are given, every token's cache row
    [normed latent | key part with its first ``rot_pairs`` pairs of neighbours rotated (a negative number: that
    many pairs of value i with value i + pairs) | zeros] written at
    ``slots`` into ``k_pool`` [units, 1, page, width] and (transposed) ``v_pool`` [units, 1, width, page]."""
    _need(proj, "latent proj", ndim=2)
    t, w = proj.shape
    _need(q_weight, "latent q norm weight", dtype=torch.float32, shape=(q_rank,))
    width = page_size = pool_slots = 0
    if k_pool is not None:
        _need(k_pool, "k_pool", dtype=proj.dtype, ndim=4)
        units, kvh, page_size, width = k_pool.shape
        _need(v_pool, "v_pool", dtype=proj.dtype, shape=(units, kvh, width, page_size))
        if kvh != 1:
            raise KernelError("latent_prep: the latent cache has one kv head")
        _need(slots, "latent slots", dtype=torch.int32, shape=(t,))
        _need(kv_weight, "latent kv norm weight", dtype=torch.float32, shape=(kv_rank,))
        pool_slots = units * page_size
        if rot_pairs:
            _need(cos_sin, "latent cos/sin", dtype=torch.float32, shape=(t, abs(rot_pairs), 2))
    cq = torch.empty((t, q_rank), dtype=proj.dtype, device=proj.device)
    gate = torch.empty((t, heads), dtype=torch.float32, device=proj.device)
    check(load().fsie_latent_prep(proj.data_ptr(), w, dq_off, q_rank, dkv_off, kv_rank, rot_dim, rot_pairs, g_off, heads,
                                  q_weight.data_ptr(), _ptr(kv_weight), float(eps), _ptr(cos_sin), cq.data_ptr(),
                                  gate.data_ptr(), _ptr(slots), _ptr(k_pool), _ptr(v_pool), width, page_size, pool_slots, t,
                                  dtype_code(proj.dtype), _stream()))
    return cq, gate


def rope_pairs(x: torch.Tensor, in_off: int, in_head_stride: int, out: torch.Tensor, out_off: int, out_head_stride: int,
               heads: int, width: int, rot_pairs: int, out_width: int, cos_sin: Optional[torch.Tensor]) -> torch.Tensor:
    """Of every token and head the run of ``width`` values at column ``in_off + h * in_head_stride`` of ``x``,
    its first ``rot_pairs`` pairs of neighbours (2i, 2i + 1) rotated by ``cos_sin`` [T, rot_pairs, 2] (a negative
    ``rot_pairs``: that many pairs of value i with value i + pairs), written to
    column ``out_off + h * out_head_stride`` of ``out`` and filled up with zeros to ``out_width`` values."""
    _need(x, "rope_pairs x", ndim=2)
    _need(out, "rope_pairs out", dtype=x.dtype, ndim=2)
    t = x.shape[0]
    if out.shape[0] != t:
        raise KernelError("rope_pairs: x and out must have a row a token")
    if rot_pairs:
        _need(cos_sin, "rope_pairs cos/sin", dtype=torch.float32, shape=(t, abs(rot_pairs), 2))
    check(load().fsie_rope_pairs(x.data_ptr(), x.shape[1], in_off, in_head_stride, out.data_ptr(), out.shape[1], out_off,
                                 out_head_stride, heads, width, rot_pairs, out_width, _ptr(cos_sin), t,
                                 dtype_code(x.dtype), _stream()))
    return out


def head_gemm(x: torch.Tensor, x_off: int, x_head_stride: int, weight: torch.Tensor, out: torch.Tensor, out_off: int,
              out_head_stride: int, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t, h, n] = (sum_k x[t, h, k] weight[h, n, k]) * gate[t, h]``: a matrix of its own for every head.
    ``x`` [T, W] holds head h's K values from column ``x_off + h * x_head_stride``, ``out`` [T, V] receives its N
    values from column ``out_off + h * out_head_stride``; ``weight`` [heads, N, K]; ``gate`` float32 [T, heads]."""
    _need(x, "head_gemm x", ndim=2)
    _need(weight, "head_gemm weight", dtype=x.dtype, ndim=3)
    _need(out, "head_gemm out", dtype=x.dtype, ndim=2)
    heads, n, k = weight.shape
    t = x.shape[0]
    if out.shape[0] != t:
        raise KernelError("head_gemm: x and out must have a row a token")
    if gate is not None:
        _need(gate, "head_gemm gate", dtype=torch.float32, shape=(t, heads))
    check(load().fsie_head_gemm(x.data_ptr(), x.shape[1], x_off, x_head_stride, weight.data_ptr(), out.data_ptr(),
                                out.shape[1], out_off, out_head_stride, _ptr(gate), t, heads, n, k, dtype_code(x.dtype),
                                _stream()))
    return out


def _delta_parts(delta: Optional[torch.Tensor], t: int, h: int, out_dtype: torch.dtype, name: str) -> int:
    """How a pending delta comes: 0 = one array [T, H] of the activations' type, n = float32 partial sums [n, T, H]."""
    if delta is None:
        return 0
    if delta.ndim == 3:
        n = delta.shape[0]
        _need(delta, f"{name} delta parts", dtype=torch.float32, shape=(n, t, h))
        if not 1 <= n <= GEMM_MAX_SPLITS:
            raise KernelError(f"{name}: {n} partial sums; up to {GEMM_MAX_SPLITS} are taken")
        return n
    _need(delta, f"{name} delta", dtype=out_dtype, shape=(t, h))
    return 0


def layer_norm(residual: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float, out_dtype: torch.dtype,
               delta: Optional[torch.Tensor] = None, delta2: Optional[torch.Tensor] = None,
               weight2: Optional[torch.Tensor] = None, bias2: Optional[torch.Tensor] = None,
               rows: Optional[torch.Tensor] = None, write_back: bool = False):
    """Layer norm of ``residual + delta + delta2`` (float32 stream; each delta [T, H] in ``out_dtype`` or float32
    partial sums [S, T, H] added in order), ``(v - mean) / sqrt(var + eps) * weight + bias`` with the variance the
    mean of the squared deviations, all in float32.  With ``weight2`` and ``bias2`` a second output from the same
    statistics: the function then returns both.  ``write_back`` stores the sum into ``residual``; ``rows`` (int32)
    selects rows."""
    _need(residual, "layer_norm residual", dtype=torch.float32, ndim=2)
    t, h = residual.shape
    _need(weight, "layer_norm weight", dtype=torch.float32, shape=(h,))
    _need(bias, "layer_norm bias", dtype=torch.float32, shape=(h,))
    two = weight2 is not None
    if two:
        _need(weight2, "layer_norm second weight", dtype=torch.float32, shape=(h,))
        _need(bias2, "layer_norm second bias", dtype=torch.float32, shape=(h,))
    parts_a = _delta_parts(delta, t, h, out_dtype, "layer_norm")
    parts_b = _delta_parts(delta2, t, h, out_dtype, "layer_norm")
    n_rows = t
    if rows is not None:
        _need(rows, "layer_norm rows", dtype=torch.int32, ndim=1)
        n_rows = rows.shape[0]
    out = torch.empty((n_rows, h), dtype=out_dtype, device=residual.device)
    out2 = torch.empty((n_rows, h), dtype=out_dtype, device=residual.device) if two else None
    check(load().fsie_layer_norm(residual.data_ptr(), _ptr(delta), parts_a, _ptr(delta2), parts_b, weight.data_ptr(),
                                 bias.data_ptr(), out.data_ptr(), _ptr(weight2), _ptr(bias2), _ptr(out2), _ptr(rows), n_rows,
                                 h, float(eps), dtype_code(out_dtype), int(write_back), t, _stream()))
    return (out, out2) if two else out


def pair_embedding(table: torch.Tensor, pairs: torch.Tensor, ids: torch.Tensor, q_starts: torch.Tensor,
                   seq_slots: torch.Tensor, last: torch.Tensor, mul_prev: int, mul_cur: int, scale: float) -> torch.Tensor:
    """float32 rows ``table[id] * scale + pairs[(previous id * mul_prev + id * mul_cur) mod buckets]`` with
    ``buckets = pairs.shape[0] - 1``; a request's first token takes the last row of ``pairs``.  ``q_starts`` int32
    [requests + 1] and ``seq_slots`` int32 [requests] describe the step; ``last`` int32 [slots, 1] keeps every
    request's latest id + 1 between steps (0: none yet) and is brought up to date."""
    _need(table, "pair_embedding table", ndim=2)
    _need(pairs, "pair_embedding pairs", dtype=table.dtype, ndim=2)
    _need(ids, "pair_embedding ids", dtype=torch.int32, ndim=1)
    _need(q_starts, "pair_embedding q_starts", dtype=torch.int32, ndim=1)
    _need(seq_slots, "pair_embedding seq_slots", dtype=torch.int32, shape=(q_starts.shape[0] - 1,))
    _need(last, "pair_embedding last tokens", dtype=torch.int32)
    v, h = table.shape
    if pairs.shape[1] != h or pairs.shape[0] < 2:
        raise KernelError(f"pair_embedding: the pairs' table {tuple(pairs.shape)} does not go with rows of {h}")
    t = ids.shape[0]
    out = torch.empty((t, h), dtype=torch.float32, device=table.device)
    check(load().fsie_pair_embedding(table.data_ptr(), pairs.data_ptr(), dtype_code(table.dtype), ids.data_ptr(),
                                     q_starts.data_ptr(), seq_slots.data_ptr(), seq_slots.shape[0], last.data_ptr(),
                                     last.numel(), out.data_ptr(), t, h, v, pairs.shape[0] - 1, int(mul_prev), int(mul_cur),
                                     float(scale), _stream()))
    return out


def attention_prep(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, g_off: int, heads: int, kv_heads: int, dim: int,
                   vdim: int, padded: int, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                   pairs: int, cos_sin: Optional[torch.Tensor], gated: bool, v_other: Optional[torch.Tensor] = None,
                   v_other_stride: int = 0, mix: Optional[torch.Tensor] = None, slots: Optional[torch.Tensor] = None,
                   k_pool: Optional[torch.Tensor] = None, v_pool: Optional[torch.Tensor] = None,
                   v_unit_norm_eps: Optional[float] = None):
    """``v_unit_norm_eps`` (a number or None): every kv head's values are divided by sqrt(mean(v^2) + eps) before they
    are cached.  From the fused projection ``proj`` [T, W] (q, k, v and one gate logit a head at their column offsets): the
    queries [T, heads * padded] after the heads' RMS norm (weights float32 [dim] or None) and the rotation of their
    first ``pairs`` pairs (i, i + pairs) by ``cos_sin`` [T, pairs, 2] (``q_weight`` may also be [heads, dim]: a weight
    of its own for every query head); the gates' sigmoid (float32 [T, heads], or
    None); and, if pools are given, keys (normed, rotated) and values written at ``slots``, the values mixed with
    ``v_other`` (a view of the same type whose rows are ``v_other_stride`` apart) by the weight ``mix`` (float32 [1])
    where it is given.  Heads are ``padded`` values wide in the queries and the pools, zeros at their end."""
    _need(proj, "attention_prep proj", ndim=2)
    t, w = proj.shape
    if max(q_off + heads * dim, k_off + kv_heads * dim, v_off + kv_heads * vdim, g_off + (heads if gated else 0)) > w:
        raise KernelError("attention_prep: the projection's rows are shorter than q, k, v and the gates")
    q_weight_stride = 0
    if q_weight is not None and q_weight.ndim == 2:
        # a weight of its own for every query head
        _need(q_weight, "attention_prep q norm weights", dtype=torch.float32, shape=(heads, dim))
        q_weight_stride = dim
    elif q_weight is not None:
        _need(q_weight, "attention_prep q norm weight", dtype=torch.float32, shape=(dim,))
    if k_weight is not None:
        _need(k_weight, "attention_prep k norm weight", dtype=torch.float32, shape=(dim,))
    if pairs:
        _need(cos_sin, "attention_prep cos/sin", dtype=torch.float32, shape=(t, pairs, 2))
    page_size = pool_slots = 0
    if k_pool is not None:
        _need(k_pool, "k_pool", dtype=proj.dtype, ndim=4)
        units, kvh, page_size, hd = k_pool.shape
        _need(v_pool, "v_pool", dtype=proj.dtype, shape=(units, kvh, hd, page_size))
        if kvh != kv_heads or hd != padded:
            raise KernelError(f"attention_prep: pools {tuple(k_pool.shape)} do not hold {kv_heads} heads of {padded}")
        _need(slots, "attention_prep slots", dtype=torch.int32, shape=(t,))
        pool_slots = units * page_size
    if v_other is not None:
        if v_other.dtype != proj.dtype or not v_other.is_cuda or v_other.stride(-1) != 1:
            raise KernelError("attention_prep: the other layer's values must be of the projection's type")
        _need(mix, "attention_prep mix", dtype=torch.float32)
    q = torch.empty((t, heads * padded), dtype=proj.dtype, device=proj.device)
    gate = torch.empty((t, heads), dtype=torch.float32, device=proj.device) if gated else None
    check(load().fsie_attention_prep(proj.data_ptr(), w, q_off, k_off, v_off, g_off, heads, kv_heads, dim, vdim, padded,
                                     _ptr(q_weight), _ptr(k_weight), float(eps), pairs, _ptr(cos_sin), _ptr(v_other),
                                     int(v_other_stride), _ptr(mix), q.data_ptr(), _ptr(gate), _ptr(slots), _ptr(k_pool),
                                     _ptr(v_pool), page_size, pool_slots, t, dtype_code(proj.dtype), q_weight_stride,
                                     int(v_unit_norm_eps is not None), float(v_unit_norm_eps or 0.0), _stream()))
    return q, gate


def gate_heads(x: torch.Tensor, padded: int, vdim: int, heads: int, gate: Optional[torch.Tensor],
               out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """[T, heads * vdim]: of every head of ``x`` [T, heads * padded] its first ``vdim`` values times ``gate``
    (float32 [T, heads]; None: as they are) times ``scale``.  ``out``: where it goes (columns of wider rows may do)."""
    _need(x, "gate_heads x", ndim=2)
    t = x.shape[0]
    if x.shape[1] != heads * padded or padded < vdim:
        raise KernelError(f"gate_heads: rows of {x.shape[1]} are not {heads} heads of {padded}")
    if gate is not None:
        _need(gate, "gate_heads gate", dtype=torch.float32, shape=(t, heads))
    y = _columns_of(out, t, heads * vdim, x.dtype, x.device, "gate_heads")
    check(load().fsie_gate_heads(x.data_ptr(), padded, _ptr(gate), y.data_ptr(), t, heads, vdim, dtype_code(x.dtype),
                                 y.stride(0) if t else heads * vdim, float(scale), _stream()))
    return y


def group_rmsnorm(residual: torch.Tensor, weight: torch.Tensor, eps: float, groups: int, out_dtype: torch.dtype,
                  delta: Optional[torch.Tensor] = None, delta2: Optional[torch.Tensor] = None, delta_scale: float = 1.0,
                  weight2: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None, write_back: bool = False):
    """RMS norm in ``groups`` equal consecutive parts of ``residual + delta_scale * (delta + delta2)`` (float32 stream
    [T, H]; each delta [T, H] in float32 or bfloat16, or None), every part divided by its own root mean square, times
    ``weight`` (float32).  ``write_back`` stores the sum into ``residual``; ``rows`` (int32) selects rows.  With
    ``weight2`` the result is a pair: the same normed rows times either weight."""
    _need(residual, "group_rmsnorm residual", dtype=torch.float32, ndim=2)
    t, h = residual.shape
    _need(weight, "group_rmsnorm weight", dtype=torch.float32, shape=(h,))
    if weight2 is not None:
        _need(weight2, "group_rmsnorm second weight", dtype=torch.float32, shape=(h,))
    for name, d in (("delta", delta), ("delta2", delta2)):
        if d is not None:
            _need(d, f"group_rmsnorm {name}", shape=(t, h))
    n_rows = t
    if rows is not None:
        _need(rows, "group_rmsnorm rows", dtype=torch.int32, ndim=1)
        n_rows = rows.shape[0]
    out = torch.empty((n_rows, h), dtype=out_dtype, device=residual.device)
    out2 = torch.empty((n_rows, h), dtype=out_dtype, device=residual.device) if weight2 is not None else None
    check(load().fsie_group_rmsnorm(residual.data_ptr(), _ptr(delta), dtype_code(delta.dtype) if delta is not None else 0,
                                    _ptr(delta2), dtype_code(delta2.dtype) if delta2 is not None else 0, float(delta_scale),
                                    weight.data_ptr(), _ptr(weight2), out.data_ptr(), _ptr(out2), _ptr(rows), n_rows, h,
                                    int(groups), float(eps), dtype_code(out_dtype), int(write_back), _stream()))
    return out if weight2 is None else (out, out2)


def causal_conv(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, q_starts: torch.Tensor, seq_slots: torch.Tensor,
                out_dtype: torch.dtype, x2: Optional[torch.Tensor] = None, weight2: Optional[torch.Tensor] = None,
                state2: Optional[torch.Tensor] = None):
    """``x + conv(x)``: a causal convolution over time within every request, channel by channel.  ``x`` float32 [T, H];
    ``weight`` float32 [H, taps], the last tap on the token itself; ``state`` float32 [slots, ..., taps - 1, H], a view
    whose first dimension are the requests' slots: the inputs before a portion's first token (oldest first), brought
    up to date by this call.  The result has ``out_dtype``.  With ``x2``, ``weight2`` and ``state2`` (a view of the
    same slots' records, behind ``state``) a second convolution of the same sizes goes through the same launches, and
    the result is the pair."""
    _need(x, "causal_conv x", dtype=torch.float32, ndim=2)
    t, h = x.shape
    _need(weight, "causal_conv weight", dtype=torch.float32, ndim=2)
    taps = weight.shape[1]
    if weight.shape[0] != h or taps < 1:
        raise KernelError(f"causal_conv: weight {tuple(weight.shape)} does not fit rows of {h}")

    def state_ok(st):
        return (isinstance(st, torch.Tensor) and st.is_cuda and st.dtype == torch.float32 and st.ndim == 3
                and tuple(st.shape[1:]) == (taps - 1, h) and st.stride(2) == 1 and st.stride(1) == h)

    if taps > 1 and not state_ok(state):
        raise KernelError(f"causal_conv: the state must be float32 [slots, {taps - 1}, {h}] with contiguous records")
    _need(q_starts, "causal_conv q_starts", dtype=torch.int32, ndim=1)
    _need(seq_slots, "causal_conv seq_slots", dtype=torch.int32, ndim=1)
    y = torch.empty((t, h), dtype=out_dtype, device=x.device)
    y2, second = None, 0
    if x2 is not None:
        _need(x2, "causal_conv x2", dtype=torch.float32, shape=(t, h))
        _need(weight2, "causal_conv weight2", dtype=torch.float32, shape=(h, taps))
        if taps > 1:
            if not state_ok(state2) or state2.stride(0) != state.stride(0) or state2.shape[0] != state.shape[0]:
                raise KernelError("causal_conv: the second state must be a view of the same slots' records")
            second = (state2.data_ptr() - state.data_ptr()) // 4
            if second < (taps - 1) * h or second + (taps - 1) * h > state.stride(0):
                raise KernelError("causal_conv: the second state must lie behind the first in a slot's record")
        y2 = torch.empty((t, h), dtype=out_dtype, device=x.device)
    check(load().fsie_causal_conv(x.data_ptr(), weight.data_ptr(), y.data_ptr(), _ptr(x2), _ptr(weight2), _ptr(y2),
                                  state.data_ptr() if taps > 1 else None, state.stride(0) if taps > 1 else 2 * max(taps - 1, 0) * h,
                                  second, state.shape[0] if taps > 1 else 1, q_starts.data_ptr(), seq_slots.data_ptr(),
                                  seq_slots.shape[0], t, h, taps, dtype_code(out_dtype), _stream()))
    return y if x2 is None else (y, y2)


def mlstm_state_floats(dim: int, vdim: int) -> int:
    """float32 numbers of one head's record of the mLSTM state: S [dim, vdim], n [dim], m and three unused ones."""
    return int(load().fsie_mlstm_state_floats(dim, vdim))


def mlstm_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, gates: torch.Tensor, gate_cap: float, q_scale: float,
               state: torch.Tensor, q_starts: torch.Tensor, seq_slots: torch.Tensor, heads: int, dim: int, vdim: int,
               chunked: bool = True):
    """The matrix memory over the step's tokens, request by request in order.  ``proj`` [T, W] holds q, k (heads * dim
    each) and v (heads * vdim) at their column offsets; ``gates`` float32 [T, 2 * heads]: the input gates' logits, then
    the forget gates'; ``state`` float32 [slots, heads, mlstm_state_floats(dim, vdim)], updated in place.  Returns
    (num [T, heads, vdim], den [T, heads], coef [T, heads, 4]), all float32: S^T q, n . q and (f, i, m before the token,
    m).  Long portions are computed chunk by chunk on the matrix cores (the same sums in another order);
    ``chunked=False`` walks every portion token by token."""
    _need(proj, "mlstm proj", ndim=2)
    t, w = proj.shape
    if max(q_off + heads * dim, k_off + heads * dim, v_off + heads * vdim) > w:
        raise KernelError("mlstm_scan: the projection's rows are shorter than q, k and v")
    _need(gates, "mlstm gates", dtype=torch.float32, shape=(t, 2 * heads))
    _need(state, "mlstm state", dtype=torch.float32, ndim=3)
    if tuple(state.shape[1:]) != (heads, mlstm_state_floats(dim, vdim)):
        raise KernelError(f"mlstm_scan: state {tuple(state.shape)} is not [slots, {heads}, {mlstm_state_floats(dim, vdim)}]")
    _need(q_starts, "mlstm q_starts", dtype=torch.int32, ndim=1)
    _need(seq_slots, "mlstm seq_slots", dtype=torch.int32, ndim=1)
    num = torch.empty((t, heads, vdim), dtype=torch.float32, device=proj.device)
    den = torch.empty((t, heads), dtype=torch.float32, device=proj.device)
    coef = torch.empty((t, heads, 4), dtype=torch.float32, device=proj.device)
    n = seq_slots.shape[0]
    if q_starts.shape[0] != n + 1:
        raise KernelError("mlstm_scan: q_starts must have one entry more than seq_slots")
    chunk_tokens, chunk_min, chunk_floats = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int64(0)
    check(load().fsie_mlstm_scan_shape(heads, dim, vdim, ctypes.byref(chunk_tokens), ctypes.byref(chunk_min),
                                       ctypes.byref(chunk_floats)))
    # a step of single tokens (t == n, as every captured decode step is) has no portion to cut into chunks
    max_chunks = t // chunk_tokens.value + n if chunked and chunk_floats.value and t > n and t >= chunk_min.value else 0
    work = torch.empty((max_chunks * chunk_floats.value,), dtype=torch.float32, device=proj.device) if max_chunks else None
    check(load().fsie_mlstm_scan(proj.data_ptr(), w, q_off, k_off, v_off, dtype_code(proj.dtype), gates.data_ptr(),
                                 float(gate_cap), float(q_scale), state.data_ptr(), state.shape[0], q_starts.data_ptr(),
                                 seq_slots.data_ptr(), n, t, heads, dim, vdim, coef.data_ptr(),
                                 num.data_ptr(), den.data_ptr(), work.data_ptr() if work is not None else None, max_chunks,
                                 _stream()))
    return num, den, coef


def mlstm_out(num: torch.Tensor, den: torch.Tensor, coef: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float,
              out_dtype: torch.dtype) -> torch.Tensor:
    """[T, heads * vdim] in ``out_dtype``: every head's num / (max(|den|, exp(-m)) + 1e-6) divided by its root mean square,
    times ``weight`` (float32 [heads * vdim]) and the sigmoid of ``gate`` ([T, heads * vdim], a view whose rows may be
    a stride apart)."""
    _need(num, "mlstm num", dtype=torch.float32, ndim=3)
    t, heads, vdim = num.shape
    _need(den, "mlstm den", dtype=torch.float32, shape=(t, heads))
    _need(coef, "mlstm coef", dtype=torch.float32, shape=(t, heads, 4))
    _need(weight, "mlstm norm weight", dtype=torch.float32, shape=(heads * vdim,))
    if not gate.is_cuda or gate.dtype != out_dtype or tuple(gate.shape) != (t, heads * vdim) or gate.stride(1) != 1:
        raise KernelError("mlstm_out: the gate must be [T, heads * vdim] of the output's type with contiguous rows")
    y = torch.empty((t, heads * vdim), dtype=out_dtype, device=num.device)
    check(load().fsie_mlstm_out(num.data_ptr(), den.data_ptr(), coef.data_ptr(), gate.data_ptr(), gate.stride(0),
                                weight.data_ptr(), y.data_ptr(), t, heads, vdim, float(eps), dtype_code(out_dtype), _stream()))
    return y


def moe_tile_rows(n_pairs: int, experts: int) -> int:
    """Rows of a tile of the experts' products for a step of this many (token, choice) pairs: 16, 32, 64 or 128."""
    return int(load().fsie_moe_tile_rows(int(n_pairs), int(experts)))


def moe_route(x: torch.Tensor, router: torch.Tensor, correction: Optional[torch.Tensor], top: int, scale: float,
              scores: str = "sigmoid", groups: int = 1, keep: int = 1, renorm: bool = True):
    """(ids int32 [T, top], weights float32 [T, top]): the ``top`` experts with the largest sigmoid(x . router^T) +
    correction (ties: the lower index) and their weights, the chosen sigmoids divided by their sum times ``scale``.
    ``x`` [T, H] and ``router`` [E, H] share a type; the logits are summed in float32.  ``scores="softmax"``: the scores
    are the softmax of the logits over all experts.  ``groups`` > 1: the experts form that many equal groups of
    neighbours and only those of the ``keep`` groups with the largest best score can be chosen.  ``renorm=False``: the
    weights are the chosen scores themselves times ``scale``.  ``correction`` may be None."""
    _need(x, "moe_route x", ndim=2)
    t, h = x.shape
    _need(router, "moe_route router", dtype=x.dtype, ndim=2)
    e = router.shape[0]
    if router.shape[1] != h:
        raise KernelError(f"moe_route: router {tuple(router.shape)} does not fit rows of {h}")
    if correction is not None:
        _need(correction, "moe_route correction", dtype=torch.float32, shape=(e,))
    if scores not in ("sigmoid", "softmax"):
        raise KernelError(f"moe_route: unknown scores '{scores}'")
    ids = torch.empty((t, top), dtype=torch.int32, device=x.device)
    weights = torch.empty((t, top), dtype=torch.float32, device=x.device)
    check(load().fsie_moe_route(x.data_ptr(), router.data_ptr(), _ptr(correction), dtype_code(x.dtype), ids.data_ptr(),
                                weights.data_ptr(), t, h, e, int(top), float(scale), int(scores == "softmax"), int(groups),
                                int(keep), int(bool(renorm)), _stream()))
    return ids, weights


def moe_group(ids: torch.Tensor, experts: int, tile_rows: Optional[int] = None):
    """The (token, choice) pairs of ``ids`` [T, top] grouped by expert: (order int32 [pairs]: the pair in every slot,
    slot_of int32 [pairs], tiles int32 [max_tiles, 3]: (expert, first slot, slots) of every tile of ``tile_rows``
    slots (default: what ``moe_tile_rows`` names for the step); unused tiles have no slots)."""
    _need(ids, "moe_group ids", dtype=torch.int32, ndim=2)
    n = ids.numel()
    tile_rows = moe_tile_rows(n, experts) if tile_rows is None else int(tile_rows)
    max_tiles = -(-n // tile_rows) + experts
    order = torch.empty((n,), dtype=torch.int32, device=ids.device)
    slot_of = torch.empty((n,), dtype=torch.int32, device=ids.device)
    tiles = torch.empty((max_tiles, 3), dtype=torch.int32, device=ids.device)
    check(load().fsie_moe_group(ids.data_ptr(), n, int(experts), tile_rows, order.data_ptr(), slot_of.data_ptr(),
                                tiles.data_ptr(), max_tiles, _stream()))
    return order, slot_of, tiles


def moe_gemm(a: torch.Tensor, weight: torch.Tensor, tiles: torch.Tensor, order: torch.Tensor, gather_div: int = 0,
             pair_weight: Optional[torch.Tensor] = None, tile_rows: Optional[int] = None,
             gated: Optional[str] = None) -> torch.Tensor:
    """One product per expert: out[slot] = a[row(slot)] . weight[expert of slot]^T with ``weight`` [E, N, K].
    ``gather_div`` > 0: row(slot) = order[slot] // gather_div (``a`` holds tokens); 0: row(slot) = slot.  Without
    ``pair_weight`` the result is the exact GELU of the product in ``a``'s type; with it (float32 [pairs]) the product
    times the pair's weight, float32.  ``tile_rows``: the rows of a tile of ``tiles`` (default: what ``moe_tile_rows``
    names for the step, as ``moe_group``'s default is).  ``gated`` (a gate activation's name): the rows of every
    expert's matrix are gate and up in turn and the result is act(gate) * up, [slots, N / 2]."""
    _need(a, "moe_gemm a", ndim=2)
    _need(weight, "moe_gemm weight", dtype=a.dtype, ndim=3)
    _, n, k = weight.shape
    if a.shape[1] != k:
        raise KernelError(f"moe_gemm: rows of {a.shape[1]} against weights {tuple(weight.shape)}")
    _need(tiles, "moe_gemm tiles", dtype=torch.int32, ndim=2)
    _need(order, "moe_gemm order", dtype=torch.int32, ndim=1)
    slots = order.shape[0]
    tile_rows = moe_tile_rows(slots, weight.shape[0]) if tile_rows is None else int(tile_rows)
    if not gather_div and a.shape[0] != slots:
        raise KernelError("moe_gemm: without a gather the rows are the slots")
    if pair_weight is not None:
        _need(pair_weight, "moe_gemm pair weights", dtype=torch.float32)
        if pair_weight.numel() != slots:
            raise KernelError("moe_gemm: one weight a pair")
    if gated is not None and (pair_weight is not None or n % 2):
        raise KernelError("moe_gemm: a gated product has an even number of rows and no pair weights")
    epilogue = 2 + gate_act_code(gated) if gated is not None else (1 if pair_weight is not None else 0)
    out = torch.empty((slots, n // 2 if gated is not None else n), dtype=torch.float32 if pair_weight is not None else a.dtype,
                      device=a.device)
    check(load().fsie_moe_gemm(a.data_ptr(), weight.data_ptr(), out.data_ptr(), tiles.data_ptr(), tiles.shape[0],
                               order.data_ptr(), int(gather_div), _ptr(pair_weight), n, k, epilogue,
                               dtype_code(a.dtype), tile_rows, _stream()))
    return out


def moe_combine(rows: torch.Tensor, slot_of: torch.Tensor, n_tokens: int, top: int) -> torch.Tensor:
    """float32 [T, H]: for every token the sum of its ``top`` rows (``rows`` [pairs, H] by slot), in the order of its choices."""
    _need(rows, "moe_combine rows", dtype=torch.float32, ndim=2)
    _need(slot_of, "moe_combine slot_of", dtype=torch.int32, shape=(n_tokens * top,))
    y = torch.empty((n_tokens, rows.shape[1]), dtype=torch.float32, device=rows.device)
    check(load().fsie_moe_combine(rows.data_ptr(), slot_of.data_ptr(), y.data_ptr(), n_tokens, top, rows.shape[1], _stream()))
    return y
