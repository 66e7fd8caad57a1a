"""Checked calls into the HIP kernels.

Every wrapper checks on the host that the operands are on the GPU, contiguous where the kernel
assumes it, of a type the kernel has, and of shapes that fit each other and the kernel's limits,
BEFORE anything is launched; a kernel never sees a size it was not written for. Refusals raise
``KernelArgumentError`` with the offending value.
"""
from __future__ import annotations

import contextlib
import ctypes
from ctypes import c_float, c_int, c_longlong, c_void_p

import torch

from tokenmill_amd.hip.library import library

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


class KernelArgumentError(ValueError):
    pass


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelArgumentError(msg)


def code(dtype: torch.dtype) -> int:
    _need(dtype in _CODES, f"kernels exist for float32 and bfloat16, not {dtype}")
    return _CODES[dtype]


def _gpu(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel operand is not on the GPU (there is no CPU path)")


def _p(t: torch.Tensor | None) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def _stream() -> c_void_p:
    # the current stream of the current device, straight from the C layer: the Python-level
    # torch.cuda.current_stream() costs more than a launch
    return c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _check(rc: int, name: str) -> None:
    if rc == 1:
        raise KernelArgumentError(f"{name}: the kernel refused its arguments")
    if rc != 0:
        raise RuntimeError(f"{name}: launch failed (code {rc})")


def _check_pools(k_pool: torch.Tensor, v_pool: torch.Tensor, KVH: int, D: int, dtype, who: str) -> int:
    """K pool [pages, page, KVH, D], V pool [pages, KVH, D, page]; returns the page size."""
    _need(k_pool.dim() == 4 and v_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous(),
          f"{who}: the cache pools must be contiguous 4-d tensors")
    pages, page = k_pool.shape[0], k_pool.shape[1]
    _need(tuple(k_pool.shape) == (pages, page, KVH, D), f"{who}: k_pool must be [pages, page, {KVH}, {D}]")
    _need(tuple(v_pool.shape) == (pages, KVH, D, page), f"{who}: v_pool must be [pages, {KVH}, {D}, page]")
    _need(k_pool.dtype == dtype and v_pool.dtype == dtype, f"{who}: the cache pools must have the type {dtype}")
    return page


def _ints(t: torch.Tensor, n: int, name: str) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n, f"{name} must be contiguous int32 [{n}]")


# --------------------------------------------------------------------------------------------

def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale as 32-bit rows. table [V, hidden], ids int32 [T], out float32 [T, hidden]."""
    _gpu(table, ids, out)
    T = ids.numel()
    V, hidden = table.shape
    _need(table.is_contiguous() and out.is_contiguous(), "embed_gather: operands must be contiguous")
    _need(out.dtype == torch.float32 and tuple(out.shape) == (T, hidden), "embed_gather: out must be float32 [T, hidden]")
    _ints(ids, T, "ids")
    if scale != 1.0:
        _check(library().tm_embed_gather_scaled(_p(table), code(table.dtype), _p(ids), _p(out), c_int(T), c_int(hidden), c_int(V),
                                                c_float(scale), _stream()), "embed_gather_scaled")
        return out
    _check(library().tm_embed_gather(_p(table), code(table.dtype), _p(ids), _p(out), c_int(T), c_int(hidden),
                                     c_int(V), _stream()), "embed_gather")
    return out


def add_rmsnorm(resid: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: torch.Tensor | None = None) -> torch.Tensor:
    """rows None: resid += delta (in place, 32-bit), out = rmsnorm(resid) * weight, all rows.
    rows given: out[r] = rmsnorm(resid[rows[r]] + delta[rows[r]]) * weight; resid is not written."""
    _gpu(resid, delta, weight, out, rows)
    T, hidden = resid.shape
    R = T if rows is None else rows.numel()
    _need(resid.dtype == torch.float32 and resid.is_contiguous(), "add_rmsnorm: the residual stream is contiguous float32")
    _need(tuple(out.shape) == (R, hidden) and out.is_contiguous(), f"add_rmsnorm: out must be [{R}, {hidden}]")
    if delta is not None:
        _need(delta.dtype == out.dtype and tuple(delta.shape) == (T, hidden) and delta.is_contiguous(),
              "add_rmsnorm: delta must match the residual's shape and out's type")
    _need(tuple(weight.shape) == (hidden,) and weight.is_contiguous(), "add_rmsnorm: weight must be [hidden]")
    _need(out.dtype == torch.bfloat16 or weight.dtype == torch.float32, "add_rmsnorm: a float32 output needs float32 weights")
    if rows is not None:
        _ints(rows, R, "rows")
    _need(eps > 0, "add_rmsnorm: eps must be positive")
    _check(library().tm_add_rmsnorm(_p(resid), _p(delta), _p(rows), _p(weight), code(weight.dtype), _p(out),
                                    code(out.dtype), c_int(R), c_int(hidden), c_float(eps), _stream()), "add_rmsnorm")
    return out


def rope_kv_write(qkv: torch.Tensor, H: int, KVH: int, D: int, cos: torch.Tensor | None, sin: torch.Tensor | None,
                  positions: torch.Tensor | None, slots: torch.Tensor | None, k_pool: torch.Tensor | None,
                  v_pool: torch.Tensor | None) -> None:
    """Rotate q and k of qkv [T, (H + 2 KVH) D] in place by each token's position and store k, v at
    the tokens' cache slots. cos/sin float32 [max_pos, rot/2] or None (store only); k_pool
    [pages, page, KVH, D] and v_pool [pages, KVH, D, page], or None (rotate only). A slot < 0 is
    not stored."""
    _gpu(qkv, cos, sin, positions, slots, k_pool, v_pool)
    T = qkv.shape[0]
    _need(qkv.is_contiguous() and qkv.shape[1] == (H + 2 * KVH) * D, "rope_kv_write: qkv must be contiguous [T, (H+2KVH)D]")
    rot = 0
    if cos is not None:
        _need(sin is not None and positions is not None, "rope_kv_write: cos needs sin and positions")
        _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
              and cos.shape == sin.shape and cos.dim() == 2, "rope_kv_write: cos/sin must be float32 [max_pos, rot/2]")
        rot = 2 * cos.shape[1]
        _need(0 < rot <= D, f"rope_kv_write: rotary width {rot} does not fit head size {D}")
        _ints(positions, T, "positions")
    write = k_pool is not None
    page = 0
    if write:
        _need(v_pool is not None and slots is not None, "rope_kv_write: a cache write needs both pools and slots")
        page = _check_pools(k_pool, v_pool, KVH, D, qkv.dtype, "rope_kv_write")
        _ints(slots, T, "slots")
    _check(library().tm_rope_kv_write(_p(qkv), code(qkv.dtype), c_int(T), c_int(H), c_int(KVH), c_int(D), c_int(rot),
                                      _p(cos), _p(sin), _p(positions), _p(slots), _p(k_pool), _p(v_pool),
                                      c_int(page), c_int(1 if write else 0), _stream()), "rope_kv_write")


def silu_mul(gu: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, i] = silu(gu[t, i]) * gu[t, I + i]; gu [T, 2I], out [T, I]."""
    _gpu(gu, out)
    T, two_i = gu.shape
    _need(two_i % 2 == 0 and tuple(out.shape) == (T, two_i // 2) and gu.is_contiguous() and out.is_contiguous()
          and gu.dtype == out.dtype, "silu_mul: gu [T, 2I] and out [T, I] of one type, contiguous")
    _check(library().tm_silu_mul(_p(gu), _p(out), code(gu.dtype), c_int(T), c_int(two_i // 2), _stream()), "silu_mul")
    return out


def gelu_mul(gu: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, i] = gelu_tanh(gu[t, i]) * gu[t, I + i], computed in 32-bit; gu [T, 2I], out [T, I]."""
    _gpu(gu, out)
    T, two_i = gu.shape
    _need(two_i % 2 == 0 and tuple(out.shape) == (T, two_i // 2) and gu.is_contiguous() and out.is_contiguous()
          and gu.dtype == out.dtype, "gelu_mul: gu [T, 2I] and out [T, I] of one type, contiguous")
    _check(library().tm_gelu_mul(_p(gu), _p(out), code(gu.dtype), c_int(T), c_int(two_i // 2), _stream()), "gelu_mul")
    return out


def convert(src: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(src, out)
    _need(src.is_contiguous() and out.is_contiguous() and src.numel() == out.numel(), "convert: same size, contiguous")
    _check(library().tm_convert(_p(src), code(src.dtype), _p(out), code(out.dtype), c_longlong(src.numel()),
                                _stream()), "convert")
    return out


def gemm_nt_tiled(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias[N]) with 32-bit multiply-adds in ascending k.
    a and out may be row-strided views (unit stride in the last dimension)."""
    _gpu(a, w, bias, out)
    M, K = a.shape
    N = w.shape[0]
    _need(w.shape[1] == K and w.is_contiguous() and w.dtype == a.dtype, "gemm: w must be contiguous [N, K] of a's type")
    _need(a.stride(1) == 1 and out.stride(1) == 1 and tuple(out.shape) == (M, N), "gemm: a [M, K], out [M, N], unit inner stride")
    _need(not (a.dtype == torch.float32 and out.dtype != torch.float32), "gemm: float32 inputs give float32 outputs")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm: bias must be [N]")
        _need(not (a.dtype == torch.float32 and bias.dtype != torch.float32), "gemm: float32 inputs need a float32 bias")
    _need(M <= 64 * 65535, "gemm: too many rows for one launch")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    _check(library().tm_gemm_nt_tiled(_p(a), c_int(lda), _p(w), _p(bias),
                                      c_int(code(bias.dtype) if bias is not None else -1), _p(out), c_int(ldc),
                                      c_int(M), c_int(N), c_int(K), code(a.dtype), code(out.dtype), _stream()),
           "gemm_nt_tiled")
    return out


LIBRARY_WORKSPACE_BYTES = 32 << 20
_library_workspace: dict[int, torch.Tensor] = {}


def library_workspace(device: torch.device) -> torch.Tensor:
    """The device memory the library products may use; made once per device (call it before any
    graph capture, so that the capture allocates nothing for it)."""
    ws = _library_workspace.get(device.index)
    if ws is None:
        ws = _library_workspace[device.index] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return ws


TUNE_AFTER_CALLS = 3        # a shape's candidates are timed when it is called this often (most shapes of a serving run come once)
_tune_now: tuple[int, int, bool] | None = None


@contextlib.contextmanager
def tuning(candidates: int, after: int = TUNE_AFTER_CALLS, every: bool = False):
    """Inside, the library products that this module's ``linear`` and ``gemm_library`` launch time up to
    ``candidates`` of the library's algorithms on their own operands when a shape is called the ``after``-th
    time with the same matrix (outside a graph capture) and keep the fastest (``every``: a shape timed at its
    first call also tries every algorithm the library holds for the operand types: about a second a shape,
    and an algorithm found that way is kept only if it gives the first choice's result). Timing is a
    property of the caller, not of the process: an engine that asks for it wraps its own steps in this, and
    the plans of timed callers are kept apart from the plans of the others."""
    global _tune_now
    _need(0 <= candidates <= 32 and after >= 1, "tuning: 0 to 32 candidates, after >= 1 calls")
    _need(not every or candidates >= 2, "tuning: every algorithm is tried beside at least 2 candidates")
    saved, _tune_now = _tune_now, (candidates, after, every)
    try:
        yield
    finally:
        _tune_now = saved


def _tune_arg(tune: tuple[int, int, bool] | None):
    """The TmTune argument of a library product: ``tune`` if given, else what an open ``tuning()`` says, else null."""
    from tokenmill_amd.hip.abi import TmTune
    t = tune if tune is not None else _tune_now
    if t is None or t[0] < 2:
        return None
    return ctypes.byref(TmTune(int(t[0]), int(t[1]), 1 if t[2] else 0))


def rule(name: str) -> int:
    """A number of the library's kernel-choosing rules (``csrc/choose.h``), for sizing a buffer or checking an
    argument: "skinny_rows", "panel_qkv_rows", "stream_rows", "skinny_max_rows", "gemv_f32_rows", "decode_chunk",
    "decode_split_pairs". The rules themselves are applied inside the library only."""
    value = _rules.get(name)
    if value is None:
        from tokenmill_amd.hip.abi import bound
        value = bound().tm_rule(name.encode())
        _need(value >= 0, f"the kernel library has no rule named {name!r}")
        _rules[name] = value
    return value


_rules: dict[str, int] = {}


def gemm_library(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor,
                 tune: tuple[int, int, bool] | None = None) -> bool:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias[N]) by hipBLASLt: bfloat16 inputs, 32-bit sums, out
    bfloat16 or float32. The plan for a shape is made on its first call and kept. Returns False
    (nothing written) if the library has no algorithm for this product. ``tune``: (candidates, after, every)
    as for ``tuning()``, which it overrides."""
    _gpu(a, w, bias, out)
    M, K = a.shape
    N = w.shape[0]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype in (torch.bfloat16, torch.float32),
          "gemm_library: bfloat16 inputs, bfloat16 or float32 output")
    _need(w.shape[1] == K and w.is_contiguous(), "gemm_library: w must be contiguous [N, K]")
    _need(a.stride(1) == 1 and out.stride(1) == 1 and tuple(out.shape) == (M, N),
          "gemm_library: a [M, K], out [M, N], unit inner stride")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous() and bias.dtype in (torch.bfloat16, torch.float32),
              "gemm_library: bias must be contiguous [N], bfloat16 or float32")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    ws = library_workspace(a.device)
    rc = library().tm_gemm_library(_p(a), c_int(lda), _p(w), c_int(K), _p(bias),
                                   c_int(code(bias.dtype) if bias is not None else -1), _p(out), c_int(ldc),
                                   c_int(1 if out.dtype == torch.float32 else 0), c_int(M), c_int(N), c_int(K),
                                   _p(ws), ctypes.c_size_t(LIBRARY_WORKSPACE_BYTES), _tune_arg(tune), _stream())
    if rc == 3:
        return False
    _check(rc, "gemm_library")
    return True


def gemv_f32_ok(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> bool:
    M, K = a.shape
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    return (a.dtype == torch.float32 and w.dtype == torch.float32 and out.dtype == torch.float32
            and (bias is None or bias.dtype == torch.float32) and 0 < M <= rule("gemv_f32_rows") and K % 4 == 0
            and lda % 4 == 0 and a.stride(1) == 1 and out.stride(1) == 1 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def gemv_f32(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias[N]), everything float32, M <= 16: 32-bit multiply-adds
    in an order that depends on K only."""
    _gpu(a, w, bias, out)
    M, K = a.shape
    N = w.shape[0]
    _need(gemv_f32_ok(a, w, bias, out), "gemv_f32: float32 operands, at most 16 rows, K a multiple of 4, 16-byte aligned")
    _need(w.shape[1] == K and w.is_contiguous() and tuple(out.shape) == (M, N), "gemv_f32: w [N, K] contiguous, out [M, N]")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemv_f32: bias must be [N]")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    _check(library().tm_gemv_f32(_p(a), c_int(lda), _p(w), _p(bias), _p(out), c_int(ldc), c_int(M), c_int(N),
                                 c_int(K), _stream()), "gemv_f32")
    return out


def gemm_f32_mfma_ok(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> bool:
    """Does the float32 product on the 32-bit matrix unit take these operands?"""
    if not (a.dtype == w.dtype == out.dtype == torch.float32 and (bias is None or bias.dtype == torch.float32)
            and a.dim() == 2 and a.stride(1) == 1 and out.stride(1) == 1 and w.is_contiguous()):
        return False
    M, K = a.shape
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(w.shape[0], out.stride(0))
    return bool(library().tm_gemm_f32_mfma_fits(_p(a), c_int(lda), _p(w), _p(bias), _p(out), c_int(ldc), c_int(M),
                                                c_int(w.shape[0]), c_int(K)))


def gemm_f32_mfma(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias[N]), everything float32, on the 32-bit matrix unit: 32-bit
    products and sums in an order that depends on K only. K must be a multiple of 16, N and the row strides of 4,
    and the operands 16-byte aligned."""
    _gpu(a, w, bias, out)
    _need(gemm_f32_mfma_ok(a, w, bias, out), "gemm_f32_mfma: float32 operands, K a multiple of 16, N and row strides of 4, 16-byte aligned")
    M, K = a.shape
    N = w.shape[0]
    _need(w.shape[1] == K and tuple(out.shape) == (M, N), "gemm_f32_mfma: w [N, K], out [M, N]")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm_f32_mfma: bias must be [N]")
    _need(M <= 64 * 65535, "gemm_f32_mfma: too many rows for one launch")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    _check(library().tm_gemm_f32_mfma(_p(a), c_int(lda), _p(w), _p(bias), _p(out), c_int(ldc), c_int(M), c_int(N),
                                      c_int(K), _stream()), "gemm_f32_mfma")
    return out


def attn_paged_generic(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                       block_tables: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                       H: int, KVH: int, D: int, scale: float, window: int = 0) -> torch.Tensor:
    """Attention of every token of the step over its request's cached keys (its own included).
    q: [T, >= H*D] view with unit inner stride (q heads first in each row); out [T, H*D];
    k_pool [pages, page, KVH, D], v_pool [pages, KVH, D, page]; block_tables int32 [S, W];
    seq_of_token, positions int32 [T]."""
    _gpu(q, out, k_pool, v_pool, block_tables, seq_of_token, positions)
    T = q.shape[0]
    _need(q.stride(1) == 1 and q.shape[1] >= H * D and out.is_contiguous() and tuple(out.shape) == (T, H * D),
          "attention: q [T, >=H*D] unit inner stride, out contiguous [T, H*D]")
    _need(q.dtype == out.dtype, "attention: q and out share one type")
    _need(H % KVH == 0 and D % 4 == 0 and 0 < D <= 256, f"attention(generic): head size {D} must be a multiple of 4 up to 256")
    _check_pools(k_pool, v_pool, KVH, D, q.dtype, "attention")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attention: block_tables must be contiguous int32 [S, W]")
    _ints(seq_of_token, T, "seq_of_token")
    _ints(positions, T, "positions")
    _need(window >= 0, "attention: window must be >= 0 (0 = every key)")
    q_stride = q.stride(0) if T > 1 else max(q.stride(0), H * D)
    _check(library().tm_attn_paged_generic(_p(q), c_int(q_stride), _p(out), c_int(H * D), _p(k_pool), _p(v_pool),
                                           _p(block_tables), c_int(block_tables.shape[1]), _p(seq_of_token),
                                           _p(positions), c_int(T), c_int(H), c_int(KVH), c_int(D),
                                           c_int(k_pool.shape[1]), c_float(scale), c_int(window), code(q.dtype),
                                           _stream()), "attn_paged_generic")
    return out


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(logits, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "argmax: logits must be contiguous float32 [R, V]")
    _ints(out, R, "out")
    nb = library().tm_argmax_work_chunks(c_int(V))
    work_v = work_i = None
    if nb > 1:                                   # a wide vocabulary: every row is cut over nb blocks
        work_v = torch.empty(R * nb, dtype=torch.float32, device=logits.device)
        work_i = torch.empty(R * nb, dtype=torch.int32, device=logits.device)
    _check(library().tm_argmax_rows(_p(logits), c_int(R), c_int(V), _p(out), _p(work_v), _p(work_i), _stream()),
           "argmax_rows")
    return out


_sample_work: dict[int, torch.Tensor] = {}


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                u: torch.Tensor, out: torch.Tensor, uses_top_k: bool = True, uses_top_p: bool = True) -> torch.Tensor:
    """One token per row: argmax where temperature <= 1e-5 or top_k == 1, else the inverse CDF at
    u of softmax(logits / temperature) after the top-k / top-p filters, in vocabulary order.
    ``uses_top_k`` / ``uses_top_p``: False if the caller knows that no row asks for that filter (its
    launches are then left out; a row that asks for none skips their work either way)."""
    _gpu(logits, temperature, top_k, top_p, u, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "sample: logits must be contiguous float32 [R, V]")
    for t, name in ((temperature, "temperature"), (top_p, "top_p"), (u, "u")):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() == R, f"sample: {name} must be float32 [R]")
    _ints(top_k, R, "top_k")
    _ints(out, R, "out")
    _need(V <= 1 << 20, f"sample: at most 2^20 logits a row, got {V}")
    lib = library()
    lib.tm_sample_work_bytes.restype = ctypes.c_size_t
    need = lib.tm_sample_work_bytes(c_int(R), c_int(V))
    work = _sample_work.get(logits.device.index)
    if work is None or work.numel() < need:            # kept and grown: one sampling call at a time per device
        work = _sample_work[logits.device.index] = torch.empty(need, dtype=torch.uint8, device=logits.device)
    _check(lib.tm_sample_rows(_p(logits), c_int(R), c_int(V), _p(temperature), _p(top_k), _p(top_p), _p(u), _p(out),
                              _p(work), ctypes.c_size_t(work.numel()), c_int((1 if uses_top_k else 0) | (2 if uses_top_p else 0)),
                              _stream()), "sample_rows")
    return out


class PackedWeight:
    """A bfloat16 matrix [N, K] (or several stacked parts of one K) in the strip order the decode-step
    products read: ``data[((s * KS + ks) * 4 + g) * rows + r, i] = W[s * rows + r, 32 ks + 8 g + i]`` with
    KS = ceil(K / 32), zero where the row or the k does not exist, so that a wavefront's load of a k-step
    of a strip is one run of rows * 64 bytes. Each part of ``parts`` (rows per part) starts a strip of its
    own: the strips of the second part lie behind those of the first."""

    def __init__(self, data: torch.Tensor, n: int, k: int, rows: int, parts: tuple[int, ...]):
        self.data, self.n, self.k, self.rows, self.parts = data, n, k, rows, parts


def pack_weight(w: torch.Tensor, rows: int, parts: list[int] | None = None) -> PackedWeight:
    """w bfloat16 [N, K] on the GPU -> its strip order in strips of ``rows`` (16, 8 or 4) rows."""
    _gpu(w)
    _need(w.dim() == 2 and w.dtype == torch.bfloat16 and rows in (4, 8, 16), "pack_weight: bfloat16 [N, K], strips of 4, 8 or 16 rows")
    N, K = w.shape
    parts = [N] if parts is None else list(parts)
    _need(sum(parts) == N and all(p > 0 for p in parts), "pack_weight: the parts must add up to the matrix's rows")
    ks = -(-K // 32)
    out, row0 = [], 0
    for n in parts:
        strips = -(-n // rows)
        padded = torch.zeros((strips * rows, ks * 32), dtype=w.dtype, device=w.device)
        padded[:n, :K] = w[row0:row0 + n]
        # [s, r, ks, g, i] -> [s, ks, g, r, i]
        out.append(padded.view(strips, rows, ks, 4, 8).permute(0, 2, 3, 1, 4).reshape(-1))
        row0 += n
    data = torch.cat(out) if len(out) > 1 else out[0].contiguous()
    return PackedWeight(data, N, K, rows, tuple(parts))


def linear_desc(w: torch.Tensor, packed: "PackedWeight | None", bias: torch.Tensor | None, library_first: bool = False,
                relu2: bool = False):
    """A matrix as the library's product rule takes it (a ``TmLinear``; the caller keeps the tensors alive)."""
    from tokenmill_amd.hip.abi import TmLinear
    _gpu(w, bias)
    _need(w.dim() == 2 and w.is_contiguous(), "linear: the matrix must be contiguous [N, K]")
    if bias is not None:
        _need(tuple(bias.shape) == (w.shape[0],) and bias.is_contiguous(), "linear: bias must be [N]")
    if packed is not None:
        _packed_operand(packed, None, "linear")
        _need((packed.n, packed.k) == tuple(w.shape), "linear: the packed copy is of another matrix")
    return TmLinear(w.data_ptr(), packed.data.data_ptr() if packed is not None else None,
                    bias.data_ptr() if bias is not None else None, packed.rows if packed is not None else 0,
                    len(packed.parts) if packed is not None else 0, code(bias.dtype) if bias is not None else -1,
                    w.shape[0], w.shape[1], code(w.dtype), 1 if library_first else 0, 1 if relu2 else 0)


def _linear_input(desc, x: torch.Tensor) -> int:
    _gpu(x)
    _need(x.dim() == 2 and x.shape[1] == desc.K and x.stride(1) == 1, f"linear: x must be [M, {desc.K}] with unit inner stride")
    _need(code(x.dtype) == desc.dtype, "linear: x must have the matrix's type (widen it for a 32-bit matrix)")
    return x.stride(0) if x.shape[0] > 1 else max(desc.K, x.stride(0))


def linear_accumulates(desc, x: torch.Tensor) -> bool:
    """Is there a kernel that adds round(x W^T + b) into a 32-bit tensor in its own epilogue, for these operands?"""
    from tokenmill_amd.hip.abi import bound
    ldx = _linear_input(desc, x)
    return bool(bound().tm_linear_accumulates(ctypes.byref(desc), code(x.dtype), _p(x), ldx, x.shape[0]))


def linear(desc, x: torch.Tensor, out: torch.Tensor | None, accum: torch.Tensor | None = None,
           tune: tuple[int, int, bool] | None = None) -> torch.Tensor:
    """out[M, N] = x[M, K] W^T (+ bias) by the kernel the library's product rule chooses for the row count and
    types (``desc``: ``linear_desc``). With ``accum`` (float32 [M, N]; only where ``linear_accumulates``) the
    result, rounded to the matrix's type, is added there instead and ``out`` stays unwritten."""
    from tokenmill_amd.hip.abi import bound
    ldx = _linear_input(desc, x)
    M = x.shape[0]
    ws = library_workspace(x.device)
    if accum is not None:
        _gpu(accum)
        _need(accum.dtype == torch.float32 and tuple(accum.shape) == (M, desc.N) and accum.stride(1) == 1,
              f"linear: accum must be float32 [{M}, {desc.N}]")
        ldacc = accum.stride(0) if M > 1 else max(desc.N, accum.stride(0))
        _check(bound().tm_linear_run(ctypes.byref(desc), code(x.dtype), _p(x), ldx, M, None, 0, 0, _p(accum), ldacc, _p(ws),
                                     LIBRARY_WORKSPACE_BYTES, _tune_arg(tune), _stream()), "linear")
        return accum
    _gpu(out)
    _need(out is not None and tuple(out.shape) == (M, desc.N) and out.stride(1) == 1, f"linear: out must be [{M}, {desc.N}]")
    _need(not (x.dtype == torch.float32 and out.dtype != torch.float32), "linear: float32 inputs give float32 outputs")
    ldc = out.stride(0) if M > 1 else max(desc.N, out.stride(0))
    _check(bound().tm_linear_run(ctypes.byref(desc), code(x.dtype), _p(x), ldx, M, _p(out), ldc, code(out.dtype), None, 0,
                                 _p(ws), LIBRARY_WORKSPACE_BYTES, _tune_arg(tune), _stream()), "linear")
    return out


def skinny_strip_rows(N: int, K: int) -> int:
    """Rows of a strip the skinny product wants an [N, K] matrix packed in."""
    return int(library().tm_skinny_strip_rows(c_int(N), c_int(K)))


def fused_qkv_strip_rows(H: int, KVH: int, D: int, K: int) -> int:
    """Rows of a strip the norm-fused q|k|v product wants its matrix packed in."""
    return int(library().tm_fused_qkv_strip_rows(c_int(H), c_int(KVH), c_int(D), c_int(K)))


def _packed_operand(w: PackedWeight, rows_expected: int | None, who: str) -> None:
    _need(isinstance(w, PackedWeight) and w.data.is_cuda and w.data.dtype == torch.bfloat16 and w.data.is_contiguous()
          and w.data.data_ptr() % 16 == 0, f"{who}: the matrix must be a PackedWeight on the GPU")
    if rows_expected is not None:
        _need(w.rows == rows_expected, f"{who}: the matrix is packed in strips of {w.rows} rows, the kernel reads {rows_expected}")


def gemm_skinny(a: torch.Tensor, w: "torch.Tensor | PackedWeight", bias: torch.Tensor | None,
                out: torch.Tensor | None, silu: bool = False, accum: torch.Tensor | None = None) -> torch.Tensor:
    """MFMA product for at most 64 rows of bfloat16 activations: out[M, N] = a @ w^T (+ bias), or with
    ``silu`` out[M, N] = silu(a @ w[:N]^T) * (a @ w[N:]^T) for a stacked [gate; up] matrix w [2N, K].
    out is bfloat16 or float32 (float32 not with silu). With ``accum`` (float32 [M, N]) nothing is
    stored to out: the result, rounded to bfloat16, is added into accum (the residual stream).
    w may be a ``PackedWeight`` (at most 16 rows of a then; with silu packed as two parts of 16-row
    strips): the same bits, read faster."""
    if isinstance(w, PackedWeight):
        return _gemm_skinny_packed(a, w, bias, out, silu, accum)
    _gpu(a, w, bias, out, accum)
    M, K = a.shape
    if accum is not None:
        _need(out is None and not silu and accum.dtype == torch.float32 and accum.dim() == 2 and accum.shape[0] == M
              and accum.stride(1) == 1, "gemm_skinny: accum must be float32 [M, N], and excludes out and silu")
        N = accum.shape[1]
        _need(tuple(w.shape) == (N, K) and w.is_contiguous() and a.dtype == w.dtype == torch.bfloat16 and 0 < M <= 64
              and a.stride(1) == 1, "gemm_skinny: bfloat16 a [M<=64, K], contiguous w [N, K]")
        lda = a.stride(0) if M > 1 else max(K, a.stride(0))
        _need(K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0,
              "gemm_skinny: K and the row stride must be multiples of 8 and the operands 16-byte aligned")
        if bias is not None:
            _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm_skinny: bias must be [N]")
        ldacc = accum.stride(0) if M > 1 else max(N, accum.stride(0))
        _check(library().tm_gemm_skinny(_p(a), c_int(lda), _p(w), _p(bias),
                                        c_int(code(bias.dtype) if bias is not None else -1), _p(None), c_int(N),
                                        c_int(M), c_int(N), c_int(K), c_int(BF16), c_int(0), _p(accum), c_int(ldacc),
                                        _stream()), "gemm_skinny")
        return accum
    N = out.shape[1]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_skinny: bfloat16 inputs")
    _need(0 < M <= 64, f"gemm_skinny: at most 64 rows, got {M}")
    _need(w.is_contiguous() and tuple(w.shape) == ((2 * N if silu else N), K), "gemm_skinny: w must be contiguous [N, K]")
    _need(a.stride(1) == 1 and out.stride(1) == 1 and out.shape[0] == M, "gemm_skinny: unit inner strides")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    ldc = out.stride(0) if M > 1 else max(N, out.stride(0))
    _need(K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0,
          "gemm_skinny: K and the row stride must be multiples of 8 and the operands 16-byte aligned")
    _need(out.dtype in (torch.bfloat16, torch.float32) and not (silu and out.dtype != torch.bfloat16),
          "gemm_skinny: out is bfloat16, or float32 without silu")
    if bias is not None:
        _need(not silu and tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm_skinny: bias must be [N], not with silu")
    _check(library().tm_gemm_skinny(_p(a), c_int(lda), _p(w), _p(bias),
                                    c_int(code(bias.dtype) if bias is not None else -1), _p(out), c_int(ldc),
                                    c_int(M), c_int(N), c_int(K), code(out.dtype), c_int(1 if silu else 0),
                                    _p(None), c_int(0), _stream()), "gemm_skinny")
    return out


def _gemm_skinny_packed(a, w: PackedWeight, bias, out, silu: bool, accum) -> torch.Tensor:
    _gpu(a, bias, out, accum)
    _packed_operand(w, 16 if silu else None, "gemm_skinny")
    M, K = a.shape
    N = w.n // 2 if silu else w.n
    _need(a.dtype == torch.bfloat16 and a.dim() == 2 and a.stride(1) == 1 and 0 < M <= rule("skinny_rows") and K == w.k,
          f"gemm_skinny: bfloat16 a [M<={rule('skinny_rows')}, {w.k}] for a packed matrix")
    _need(w.parts == ((N, N) if silu else (w.n,)), "gemm_skinny: with silu the matrix is packed as its two halves, else as one part")
    lda = a.stride(0) if M > 1 else max(K, a.stride(0))
    _need(K % 8 == 0 and lda % 8 == 0 and a.data_ptr() % 16 == 0,
          "gemm_skinny: K and the row stride must be multiples of 8 and the activations 16-byte aligned")
    if bias is not None:
        _need(not silu and tuple(bias.shape) == (N,) and bias.is_contiguous(), "gemm_skinny: bias must be [N], not with silu")
    if accum is not None:
        _need(out is None and not silu and accum.dtype == torch.float32 and tuple(accum.shape) == (M, N)
              and accum.stride(1) == 1, "gemm_skinny: accum must be float32 [M, N], and excludes out and silu")
        ldacc = accum.stride(0) if M > 1 else max(N, accum.stride(0))
        c, ldc, out_code = None, N, BF16
    else:
        _need(out is not None and tuple(out.shape) == (M, N) and out.stride(1) == 1
              and out.dtype in (torch.bfloat16, torch.float32) and not (silu and out.dtype != torch.bfloat16),
              "gemm_skinny: out [M, N] bfloat16, or float32 without silu")
        ldacc = 0
        c, ldc, out_code = out, (out.stride(0) if M > 1 else max(N, out.stride(0))), code(out.dtype)
    _check(library().tm_gemm_skinny_packed(_p(a), c_int(lda), _p(w.data), c_int(w.rows), _p(bias),
                                           c_int(code(bias.dtype) if bias is not None else -1), _p(c), c_int(ldc),
                                           c_int(M), c_int(N), c_int(K), c_int(out_code), c_int(1 if silu else 0),
                                           _p(accum), c_int(ldacc), _stream()), "gemm_skinny_packed")
    return accum if accum is not None else out


def attn_decode_mfma_supported(dtype, H: int, KVH: int, D: int, page: int) -> bool:
    return (dtype == torch.bfloat16 and D in (32, 64, 96, 128) and page >= 16 and page & (page - 1) == 0
            and H % KVH == 0 and H // KVH <= 16)


def attn_decode_mfma(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                     block_tables: torch.Tensor, context_lens: torch.Tensor, H: int, KVH: int, D: int, scale: float,
                     window: int, max_context: int, workspace: tuple[torch.Tensor, torch.Tensor] | None = None,
                     split: bool | None = None, softcap: float = 0.0):
    """Attention of one new token per request over its cache (the token's own key included); ``softcap`` > 0: a scaled
    score s becomes softcap * tanh(s / softcap).
    q: [S, >= H*D] rows (unit inner stride), out [S, H*D] view; block_tables int32 [S, W];
    context_lens int32 [S] (new token counted); max_context >= every context length. ``split``: None runs
    the kernel the library's rule names for this many requests (contexts split over blocks and merged, or one
    block a request and kv head); True / False name it (each kernel alone, in tests)."""
    _gpu(q, out, k_pool, v_pool, block_tables, context_lens)
    S = q.shape[0]
    page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "attn_decode")
    _need(attn_decode_mfma_supported(q.dtype, H, KVH, D, page), "attn_decode: unsupported head size, group or page size")
    _need(q.stride(1) == 1 and out.stride(1) == 1 and out.dtype == torch.bfloat16 and out.shape[0] == S
          and q.shape[1] >= H * D and out.shape[1] >= H * D, "attn_decode: q, out [S, >= H*D] with unit inner stride")
    q_stride = q.stride(0) if S > 1 else max(q.stride(0), H * D)
    out_stride = out.stride(0) if S > 1 else max(out.stride(0), H * D)
    _need(q_stride % 8 == 0 and q.data_ptr() % 16 == 0, "attn_decode: q rows must be 16-byte aligned")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= S
          and block_tables.stride(1) == 1, "attn_decode: block_tables must be int32 [S, W]")
    W = block_tables.shape[1]
    _need(block_tables.stride(0) == W or S == 1, "attn_decode: block_tables rows must be contiguous")
    _ints(context_lens, S, "context_lens")
    _need(0 < max_context <= W * page, "attn_decode: max_context exceeds what the block tables hold")
    from tokenmill_amd.hip.abi import bound
    chunks = -(-max_context // rule("decode_chunk"))
    part_o = part_ml = None
    if split is None:                                             # few (request, kv head) pairs: contexts split over blocks
        split = bool(bound().tm_decode_split_chunks(S, KVH, max_context))
    if split and chunks > 1:
        if workspace is None:
            workspace = (torch.empty((S, H, chunks, D), dtype=torch.float32, device=q.device),
                         torch.empty((S, H, chunks, 2), dtype=torch.float32, device=q.device))
        part_o, part_ml = workspace
        _need(part_o.numel() >= S * H * chunks * D and part_ml.numel() >= S * H * chunks * 2
              and part_o.dtype == torch.float32 and part_ml.dtype == torch.float32, "attn_decode: workspace too small")
    _need(out_stride % 4 == 0 and out.data_ptr() % 8 == 0, "attn_decode: out rows must be 8-byte aligned")
    _check(library().tm_attn_decode_mfma_cap(_p(q), c_int(q_stride), _p(out), c_int(out_stride), _p(k_pool), _p(v_pool),
                                             _p(block_tables), c_int(W), _p(context_lens), _p(part_o), _p(part_ml),
                                             c_int(chunks), c_int(S), c_int(H), c_int(KVH), c_int(D), c_int(page),
                                             c_float(scale), c_int(window), c_float(softcap), _stream()), "attn_decode_mfma")
    return out


PREFILL_TILE = 16           # query tokens per tile of the MFMA prefill attention


def attn_prefill_mfma_supported(dtype, H: int, KVH: int, D: int, page: int) -> bool:
    return (dtype == torch.bfloat16 and D in (32, 64, 96, 128) and page >= 16 and page & (page - 1) == 0
            and H % KVH == 0)


def attn_prefill_mfma(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                      block_tables: torch.Tensor, tiles: torch.Tensor, H: int, KVH: int, D: int, scale: float,
                      window: int, shared: bool = False, softcap: float = 0.0) -> torch.Tensor:
    """Attention of prompt portions over the cache (``softcap`` > 0: a scaled score s becomes softcap * tanh(s / softcap)). q: [T, >= H*D] rows, out [T, H*D]; tiles int32
    [n, 4] = (request index, first row, tokens (1..16), position of the first token) cover the rows
    to compute; every row of a tile belongs to one request at consecutive positions. ``shared``: the kernel
    that stages a tile's keys and values through LDS for all heads of a kv head, instead of the one whose
    wavefronts split the key blocks (each kernel alone, in tests; a step's choice is the library's)."""
    _gpu(q, out, k_pool, v_pool, block_tables, tiles)
    T = q.shape[0]
    page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "attn_prefill")
    _need(attn_prefill_mfma_supported(q.dtype, H, KVH, D, page), "attn_prefill: unsupported head size or page size")
    _need(q.stride(1) == 1 and out.stride(1) == 1 and out.dtype == torch.bfloat16 and out.shape[0] == T
          and q.shape[1] >= H * D and out.shape[1] >= H * D, "attn_prefill: q, out [T, >= H*D] with unit inner stride")
    q_stride = q.stride(0) if T > 1 else max(q.stride(0), H * D)
    out_stride = out.stride(0) if T > 1 else max(out.stride(0), H * D)
    _need(q_stride % 8 == 0 and q.data_ptr() % 16 == 0 and out_stride % 2 == 0 and out.data_ptr() % 4 == 0,
          "attn_prefill: q rows must be 16-byte aligned and out rows 4-byte aligned")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attn_prefill: block_tables must be contiguous int32 [S, W]")
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous(),
          "attn_prefill: tiles must be contiguous int32 [n, 4]")
    if shared:
        _need(bool(library().tm_attn_prefill_shared_takes(c_int(H), c_int(KVH), c_int(D))) and out_stride % 4 == 0
              and out.data_ptr() % 8 == 0, "attn_prefill: the shared-keys kernel takes up to 16 query heads a kv head "
              "and out rows aligned to 8 bytes")
    entry = library().tm_attn_prefill_shared_cap if shared else library().tm_attn_prefill_mfma_cap
    _check(entry(_p(q), c_int(q_stride), _p(out), c_int(out_stride), _p(k_pool), _p(v_pool),
                 _p(block_tables), c_int(block_tables.shape[1]), _p(tiles),
                 c_int(tiles.shape[0]), c_int(H), c_int(KVH), c_int(D), c_int(page),
                 c_float(scale), c_int(window), c_float(softcap), _stream()), "attn_prefill_shared" if shared else "attn_prefill_mfma")
    return out


def attn_prefill_f32_supported(dtype, H: int, KVH: int, D: int, page: int) -> bool:
    return (dtype == torch.float32 and D % 16 == 0 and 16 <= D <= 128 and page >= 16 and page & (page - 1) == 0
            and H % KVH == 0)


def attn_prefill_f32(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                     block_tables: torch.Tensor, tiles: torch.Tensor, H: int, KVH: int, D: int, scale: float,
                     window: int, softcap: float = 0.0) -> torch.Tensor:
    """Attention of prompt portions over the cache in true 32-bit (32-bit MFMA). Operands as for
    ``attn_prefill_mfma``, all float32."""
    _gpu(q, out, k_pool, v_pool, block_tables, tiles)
    T = q.shape[0]
    page = _check_pools(k_pool, v_pool, KVH, D, torch.float32, "attn_prefill_f32")
    _need(attn_prefill_f32_supported(q.dtype, H, KVH, D, page), "attn_prefill_f32: unsupported head size or page size")
    _need(q.stride(1) == 1 and out.stride(1) == 1 and out.dtype == torch.float32 and out.shape[0] == T
          and q.shape[1] >= H * D and out.shape[1] >= H * D, "attn_prefill_f32: q, out [T, >= H*D] with unit inner stride")
    q_stride = q.stride(0) if T > 1 else max(q.stride(0), H * D)
    out_stride = out.stride(0) if T > 1 else max(out.stride(0), H * D)
    _need(q_stride % 4 == 0 and out_stride % 4 == 0 and q.data_ptr() % 16 == 0 and out.data_ptr() % 16 == 0,
          "attn_prefill_f32: q and out rows must be 16-byte aligned")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attn_prefill_f32: block_tables must be contiguous int32 [S, W]")
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous(),
          "attn_prefill_f32: tiles must be contiguous int32 [n, 4]")
    _check(library().tm_attn_prefill_f32_cap(_p(q), c_int(q_stride), _p(out), c_int(out_stride), _p(k_pool), _p(v_pool),
                                             _p(block_tables), c_int(block_tables.shape[1]), _p(tiles),
                                             c_int(tiles.shape[0]), c_int(H), c_int(KVH), c_int(D), c_int(page),
                                             c_float(scale), c_int(window), c_float(softcap), _stream()), "attn_prefill_f32")
    return out


def fused_norm_qkv_rope(resid: torch.Tensor, norm_w: torch.Tensor, eps: float, w: PackedWeight,
                        bias: torch.Tensor | None, q_out: torch.Tensor, H: int, KVH: int, D: int, cos: torch.Tensor,
                        sin: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                        k_pool: torch.Tensor | None, v_pool: torch.Tensor | None) -> torch.Tensor:
    """q_out[M, H*D] and the cache <- rope(rmsnorm(resid) * norm_w @ w^T + bias) for at most 16 tokens.
    resid float32 [M, K]; w the [(H + 2 KVH) D, K] matrix packed in strips of
    ``fused_qkv_strip_rows(H, KVH, D, K)`` rows; cos/sin float32 [max_pos, D/2]."""
    _gpu(resid, norm_w, bias, q_out, cos, sin, positions, slots, k_pool, v_pool)
    M, K = resid.shape
    _need(0 < M <= rule("skinny_rows"), f"fused qkv: at most {rule('skinny_rows')} tokens, got {M}")
    _need(resid.dtype == torch.float32 and resid.is_contiguous() and resid.data_ptr() % 16 == 0, "fused qkv: resid float32 [M, K]")
    _need(D % 32 == 0, f"fused qkv: head size {D} must be a multiple of 32")
    _packed_operand(w, fused_qkv_strip_rows(H, KVH, D, K), "fused qkv")
    _need((w.n, w.k) == ((H + 2 * KVH) * D, K) and len(w.parts) == 1 and K % 8 == 0,
          "fused qkv: w must be the packed [(H+2KVH)D, K] matrix, K a multiple of 8")
    _need(tuple(norm_w.shape) == (K,) and norm_w.is_contiguous() and norm_w.data_ptr() % 16 == 0, "fused qkv: norm weight [K]")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
          and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] * 2 == D,
          "fused qkv: cos/sin must be float32 [max_pos, D/2] (rotation over the whole head)")
    _need(q_out.dtype == torch.bfloat16 and q_out.is_contiguous() and tuple(q_out.shape) == (M, H * D), "fused qkv: q_out [M, H*D]")
    _ints(positions, M, "positions")
    page = 16
    if slots is not None:
        _need(k_pool is not None and v_pool is not None, "fused qkv: slots need the cache pools")
        page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "fused qkv")
        _need(page & (page - 1) == 0, "fused qkv: the page size must be a power of two")
        _ints(slots, M, "slots")
    if bias is not None:
        _need(tuple(bias.shape) == (w.n,) and bias.is_contiguous() and bias.data_ptr() % 16 == 0,
              "fused qkv: bias [rows], 16-byte aligned")
    _need(eps > 0, "fused qkv: eps must be positive")
    _check(library().tm_fused_norm_qkv_rope(_p(resid), _p(norm_w), code(norm_w.dtype), c_float(eps), c_int(M), c_int(K),
                                            _p(w.data), _p(bias), c_int(code(bias.dtype) if bias is not None else -1),
                                            _p(q_out), c_int(H), c_int(KVH), c_int(D), _p(cos), _p(sin), _p(positions),
                                            _p(slots), _p(k_pool if slots is not None else None),
                                            _p(v_pool if slots is not None else None), c_int(page), _stream()),
           "fused_norm_qkv_rope")
    return q_out


def fused_norm_gate_up_silu(resid: torch.Tensor, norm_w: torch.Tensor, eps: float, w: PackedWeight,
                            out: torch.Tensor) -> torch.Tensor:
    """out[M, I] <- silu(x Wg^T) * (x Wu^T), x = rmsnorm(resid) * norm_w, w = [Wg; Wu] [2I, K] packed as
    its two halves in strips of 16 rows."""
    _gpu(resid, norm_w, out)
    M, K = resid.shape
    I = out.shape[1]
    _need(0 < M <= rule("skinny_rows"), f"fused gate-up: at most {rule('skinny_rows')} tokens, got {M}")
    _need(resid.dtype == torch.float32 and resid.is_contiguous() and resid.data_ptr() % 16 == 0, "fused gate-up: resid float32 [M, K]")
    _packed_operand(w, 16, "fused gate-up")
    _need((w.n, w.k) == (2 * I, K) and w.parts == (I, I) and K % 8 == 0 and I % 4 == 0,
          "fused gate-up: w must be the packed [2I, K] matrix in two parts of I rows; K % 8 == 0, I % 4 == 0")
    _need(tuple(norm_w.shape) == (K,) and norm_w.is_contiguous() and norm_w.data_ptr() % 16 == 0, "fused gate-up: norm weight [K]")
    _need(out.dtype == torch.bfloat16 and out.is_contiguous() and out.shape[0] == M, "fused gate-up: out bfloat16 [M, I]")
    _need(eps > 0, "fused gate-up: eps must be positive")
    _check(library().tm_fused_norm_gate_up_silu(_p(resid), _p(norm_w), code(norm_w.dtype), c_float(eps), c_int(M),
                                                c_int(K), _p(w.data), _p(out), c_int(I), _stream()),
           "fused_norm_gate_up_silu")
    return out


def panel_fits(M: int, K: int) -> bool:
    """Do the panel products (q|k|v + rotary + cache write, gate|up + SiLU·up for up to 64 tokens behind a
    norm that ran by itself) take M tokens of width K?"""
    return bool(library().tm_gemm_panel_fits(c_int(M), c_int(K)))


def _panel_input(x: torch.Tensor, who: str) -> int:
    M, K = x.shape
    _need(x.dtype == torch.bfloat16 and x.stride(1) == 1 and x.data_ptr() % 16 == 0 and M > 0
          and panel_fits(M, K), f"{who}: x bfloat16 [M, K] with x and the partial sums fitting a block's LDS")
    ldx = x.stride(0) if M > 1 else max(K, x.stride(0))
    _need(ldx % 8 == 0, f"{who}: rows of x must be 16-byte aligned")
    return ldx


def panel_qkv_rope(x: torch.Tensor, w: PackedWeight, bias: torch.Tensor | None, q_out: torch.Tensor, H: int, KVH: int,
                   D: int, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                   k_pool: torch.Tensor | None, v_pool: torch.Tensor | None) -> torch.Tensor:
    """q_out[M, H*D] and the cache <- rope(x @ w^T + bias) for up to 64 tokens; x bfloat16 [M, K] is the normed
    input, everything else as for ``fused_norm_qkv_rope``."""
    _gpu(x, bias, q_out, cos, sin, positions, slots, k_pool, v_pool)
    M, K = x.shape
    ldx = _panel_input(x, "panel qkv")
    _need(D % 32 == 0, f"panel qkv: head size {D} must be a multiple of 32")
    _packed_operand(w, fused_qkv_strip_rows(H, KVH, D, K), "panel qkv")
    _need((w.n, w.k) == ((H + 2 * KVH) * D, K) and len(w.parts) == 1, "panel qkv: w must be the packed [(H+2KVH)D, K] matrix")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
          and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] * 2 == D,
          "panel qkv: cos/sin must be float32 [max_pos, D/2] (rotation over the whole head)")
    _need(q_out.dtype == torch.bfloat16 and q_out.is_contiguous() and tuple(q_out.shape) == (M, H * D), "panel qkv: q_out [M, H*D]")
    _ints(positions, M, "positions")
    page = 16
    if slots is not None:
        _need(k_pool is not None and v_pool is not None, "panel qkv: slots need the cache pools")
        page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "panel qkv")
        _need(page & (page - 1) == 0, "panel qkv: the page size must be a power of two")
        _ints(slots, M, "slots")
    if bias is not None:
        _need(tuple(bias.shape) == (w.n,) and bias.is_contiguous() and bias.data_ptr() % 16 == 0,
              "panel qkv: bias [rows], 16-byte aligned")
    _check(library().tm_panel_qkv_rope(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), _p(bias),
                                       c_int(code(bias.dtype) if bias is not None else -1), _p(q_out), c_int(H),
                                       c_int(KVH), c_int(D), _p(cos), _p(sin), _p(positions), _p(slots),
                                       _p(k_pool if slots is not None else None),
                                       _p(v_pool if slots is not None else None), c_int(page), _stream()),
           "panel_qkv_rope")
    return q_out


def stream_fits(M: int, K: int) -> bool:
    """Do the products that stream a packed matrix once for up to 64 tokens take M tokens of width K?"""
    return bool(library().tm_gemm_stream_fits(c_int(M), c_int(K)))


def _stream_input(x: torch.Tensor, w: PackedWeight, who: str) -> int:
    M, K = x.shape
    _need(x.dtype == torch.bfloat16 and x.stride(1) == 1 and x.data_ptr() % 16 == 0 and stream_fits(M, K) and K == w.k,
          f"{who}: x bfloat16 [M<=64, {w.k}], 16-byte aligned")
    ldx = x.stride(0) if M > 1 else max(K, x.stride(0))
    _need(ldx % 8 == 0, f"{who}: rows of x must be 16-byte aligned")
    return ldx


def stream_qkv_rope(x: torch.Tensor, w: PackedWeight, bias: torch.Tensor | None, q_out: torch.Tensor, H: int, KVH: int,
                    D: int, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor | None,
                    k_pool: torch.Tensor | None, v_pool: torch.Tensor | None) -> torch.Tensor:
    """q_out[M, H*D] and the cache <- rope(x @ w^T + bias) for up to 64 tokens of any width; x bfloat16 [M, K] is the
    normed input, w the [(H + 2 KVH) D, K] matrix packed in strips of 16, 8 or 4 rows; the rest as for
    ``fused_norm_qkv_rope``."""
    _gpu(x, bias, q_out, cos, sin, positions, slots, k_pool, v_pool)
    M, K = x.shape
    _packed_operand(w, None, "stream qkv")
    ldx = _stream_input(x, w, "stream qkv")
    _need(D % 32 == 0, f"stream qkv: head size {D} must be a multiple of 32")
    _need((w.n, w.k) == ((H + 2 * KVH) * D, K) and len(w.parts) == 1, "stream qkv: w must be the packed [(H+2KVH)D, K] matrix")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
          and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] * 2 == D and cos.data_ptr() % 16 == 0
          and sin.data_ptr() % 16 == 0, "stream qkv: cos/sin must be float32 [max_pos, D/2] (rotation over the whole head)")
    _need(q_out.dtype == torch.bfloat16 and q_out.is_contiguous() and tuple(q_out.shape) == (M, H * D), "stream qkv: q_out [M, H*D]")
    _ints(positions, M, "positions")
    page = 16
    if slots is not None:
        _need(k_pool is not None and v_pool is not None, "stream qkv: slots need the cache pools")
        page = _check_pools(k_pool, v_pool, KVH, D, torch.bfloat16, "stream qkv")
        _need(page & (page - 1) == 0, "stream qkv: the page size must be a power of two")
        _ints(slots, M, "slots")
    if bias is not None:
        _need(tuple(bias.shape) == (w.n,) and bias.is_contiguous(), "stream qkv: bias [rows]")
    _check(library().tm_stream_qkv_rope(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), c_int(w.rows), _p(bias),
                                        c_int(code(bias.dtype) if bias is not None else -1), _p(q_out), c_int(H),
                                        c_int(KVH), c_int(D), _p(cos), _p(sin), _p(positions), _p(slots),
                                        _p(k_pool if slots is not None else None),
                                        _p(v_pool if slots is not None else None), c_int(page), _stream()),
           "stream_qkv_rope")
    return q_out


def stream_gate_up_silu(x: torch.Tensor, w: PackedWeight, out: torch.Tensor) -> torch.Tensor:
    """out[M, I] <- silu(x Wg^T) * (x Wu^T) for up to 64 tokens of any width; w as for ``fused_norm_gate_up_silu``."""
    _gpu(x, out)
    M, K = x.shape
    I = out.shape[1]
    _packed_operand(w, 16, "stream gate-up")
    ldx = _stream_input(x, w, "stream gate-up")
    _need((w.n, w.k) == (2 * I, K) and w.parts == (I, I) and I % 4 == 0,
          "stream gate-up: w must be the packed [2I, K] matrix in two parts of I rows; I % 4 == 0")
    _need(out.dtype == torch.bfloat16 and out.is_contiguous() and out.shape[0] == M, "stream gate-up: out bfloat16 [M, I]")
    _check(library().tm_stream_gate_up_silu(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), _p(out), c_int(I),
                                            _stream()), "stream_gate_up_silu")
    return out


def stream_linear(x: torch.Tensor, w: PackedWeight, bias: torch.Tensor | None, out: torch.Tensor | None,
                  accum: torch.Tensor | None = None) -> torch.Tensor:
    """out[M, N] = x @ w^T (+ bias) for up to 64 tokens of any width, out bfloat16 or float32; or with ``accum``
    (float32 [M, N]) the result, rounded to bfloat16, is added there and out stays unwritten. w: the [N, K]
    matrix packed as one part in strips of 16, 8 or 4 rows."""
    _gpu(x, bias, out, accum)
    M, K = x.shape
    _packed_operand(w, None, "stream linear")
    ldx = _stream_input(x, w, "stream linear")
    N = w.n
    _need(len(w.parts) == 1, "stream linear: the matrix is packed as one part")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "stream linear: bias must be [N]")
    if accum is not None:
        _need(out is None and accum.dtype == torch.float32 and tuple(accum.shape) == (M, N) and accum.stride(1) == 1,
              "stream linear: accum must be float32 [M, N], and excludes out")
        ldacc = accum.stride(0) if M > 1 else max(N, accum.stride(0))
        c, ldc, f32 = None, N, 0
    else:
        _need(out is not None and tuple(out.shape) == (M, N) and out.stride(1) == 1
              and out.dtype in (torch.bfloat16, torch.float32), "stream linear: out [M, N] bfloat16 or float32")
        ldacc = 0
        c, ldc, f32 = out, (out.stride(0) if M > 1 else max(N, out.stride(0))), 1 if out.dtype == torch.float32 else 0
    _check(library().tm_stream_linear(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), c_int(w.rows), c_int(N), _p(bias),
                                      c_int(code(bias.dtype) if bias is not None else -1), _p(c), c_int(ldc), c_int(f32),
                                      _p(accum), c_int(ldacc), _stream()), "stream_linear")
    return accum if accum is not None else out


def stream_linear_split(x: torch.Tensor, w: PackedWeight, bias: torch.Tensor | None) -> torch.Tensor:
    """The plain product of up to 64 rows with K split over groups of blocks: returns float32 [parts, M, N], the
    partial sums (bias in part 0) that ``add_rmsnorm_parts`` or ``sum_parts`` add up. The number of parts follows
    from the matrix's shape alone."""
    _gpu(x, bias)
    M, K = x.shape
    _packed_operand(w, None, "stream linear")
    ldx = _stream_input(x, w, "stream linear")
    N = w.n
    _need(len(w.parts) == 1, "stream linear: the matrix is packed as one part")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous(), "stream linear: bias must be [N]")
    n_parts = library().tm_stream_linear_parts(c_int(N), c_int(K))
    parts = torch.empty((n_parts, M, N), dtype=torch.float32, device=x.device)
    _check(library().tm_stream_linear_split(_p(x), c_int(ldx), c_int(M), c_int(K), _p(w.data), c_int(w.rows), c_int(N),
                                            _p(bias), c_int(code(bias.dtype) if bias is not None else -1), _p(parts),
                                            _stream()), "stream_linear_split")
    return parts


def sum_parts(parts: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = round(parts[0] + parts[1] + ...) in out's type; parts float32 [P, ...]."""
    _gpu(parts, out)
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and out.is_contiguous()
          and tuple(parts.shape[1:]) == tuple(out.shape), "sum_parts: parts float32 [P, *out.shape]")
    _check(library().tm_sum_parts(_p(parts), c_int(parts.shape[0]), ctypes.c_size_t(out.numel()), _p(out), code(out.dtype),
                                  ctypes.c_size_t(out.numel()), _stream()), "sum_parts")
    return out


def add_rmsnorm_parts(resid: torch.Tensor, parts: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                      rows: torch.Tensor | None = None) -> torch.Tensor:
    """``add_rmsnorm`` with what is to be added given as float32 partial sums [P, T, hidden]: added in their order and
    rounded to out's type before they meet the residual."""
    _gpu(resid, parts, weight, out, rows)
    T, hidden = resid.shape
    R = T if rows is None else rows.numel()
    _need(resid.dtype == torch.float32 and resid.is_contiguous(), "add_rmsnorm: the residual stream is contiguous float32")
    _need(tuple(out.shape) == (R, hidden) and out.is_contiguous(), f"add_rmsnorm: out must be [{R}, {hidden}]")
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and parts.dim() == 3 and tuple(parts.shape[1:]) == (T, hidden)
          and 1 <= parts.shape[0] <= 16, "add_rmsnorm: parts must be float32 [P <= 16, T, hidden]")
    _need(tuple(weight.shape) == (hidden,) and weight.is_contiguous(), "add_rmsnorm: weight must be [hidden]")
    _need(out.dtype == torch.bfloat16 or weight.dtype == torch.float32, "add_rmsnorm: a float32 output needs float32 weights")
    if rows is not None:
        _ints(rows, R, "rows")
    _need(eps > 0, "add_rmsnorm: eps must be positive")
    _check(library().tm_add_rmsnorm_parts(_p(resid), _p(parts), c_int(parts.shape[0]), ctypes.c_size_t(T * hidden), _p(rows),
                                          _p(weight), code(weight.dtype), _p(out), code(out.dtype), c_int(R), c_int(hidden),
                                          c_float(eps), _stream()), "add_rmsnorm_parts")
    return out


def fused_lds_fits(M: int, K: int) -> bool:
    """Does the normed input of M tokens (4, 8 or 16 rows of K + 8 bfloat16), beside the partial sums of
    the block's 4 (K < 2048) or 8 wavefronts, fit the 160 KB of LDS a block of the norm-fused products may use?"""
    rows = 4 if M <= 4 else (8 if M <= 8 else 16)
    waves = 8 if K >= 2048 else 4
    return rows * (K + 8) * 2 + 4 * waves * 2 * 64 * 5 + 1024 <= 160 * 1024


def argmax_rows_static(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``argmax_rows`` without any allocation: the chunk candidates go to a fixed array the library holds on
    each GPU. For callers that cannot allocate; calls that may overlap on one GPU must not be made."""
    _gpu(logits, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous(), "argmax: logits must be contiguous float32 [R, V]")
    _ints(out, R, "out")
    lib = library()
    pairs, most = R * lib.tm_argmax_work_chunks(c_int(V)), lib.tm_argmax_rows_static_max_pairs()
    _need(pairs <= most or lib.tm_argmax_work_chunks(c_int(V)) == 1,
          f"argmax (static): {R} rows of {V} logits need {pairs} chunk candidates; the fixed array holds {most}")
    _need(logits.device.index == torch.cuda.current_device(), "argmax (static): the logits' GPU must be the current device")
    _check(lib.tm_argmax_rows_static(_p(logits), c_int(R), c_int(V), _p(out), _stream()), "argmax_rows_static")
    return out


# -------------------------------------------------------------------------------------------- learned positions, gelu

def embed_gather_pos(table: torch.Tensor, places: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor,
                     out: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]] + places[positions[t]] as 32-bit rows. table [V, hidden] and places [P, hidden] of one
    type, ids and positions int32 [T], out float32 [T, hidden]."""
    _gpu(table, places, ids, positions, out)
    T = ids.numel()
    V, hidden = table.shape
    _need(table.is_contiguous() and places.is_contiguous() and out.is_contiguous(), "embed_gather_pos: operands must be contiguous")
    _need(places.dim() == 2 and places.shape[1] == hidden and places.dtype == table.dtype,
          f"embed_gather_pos: the position table must be [positions, {hidden}] of the token table's type")
    _need(out.dtype == torch.float32 and tuple(out.shape) == (T, hidden), "embed_gather_pos: out must be float32 [T, hidden]")
    _ints(ids, T, "ids")
    _ints(positions, T, "positions")
    _check(library().tm_embed_gather_pos(_p(table), _p(places), code(table.dtype), _p(ids), _p(positions), _p(out), c_int(T),
                                         c_int(hidden), c_int(V), c_int(places.shape[0]), _stream()), "embed_gather_pos")
    return out


def gelu_tanh(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))), computed in 32-bit; ``out`` may be ``x``."""
    _gpu(x, out)
    _need(x.is_contiguous() and out.is_contiguous() and x.shape == out.shape and x.dtype == out.dtype,
          "gelu_tanh: x and out must be contiguous, of one shape and type")
    _check(library().tm_gelu_tanh(_p(x), _p(out), code(x.dtype), c_longlong(x.numel()), _stream()), "gelu_tanh")
    return out


def relu2(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = relu(x)^2, computed in 32-bit; ``out`` may be ``x``."""
    _gpu(x, out)
    _need(x.is_contiguous() and out.is_contiguous() and x.shape == out.shape and x.dtype == out.dtype,
          "relu2: x and out must be contiguous, of one shape and type")
    _check(library().tm_relu2(_p(x), _p(out), code(x.dtype), c_longlong(x.numel()), _stream()), "relu2")
    return out


# -------------------------------------------------------------------------------------------- norm in groups

GROUP_NORM_MAX_FLOATS = 16384 - 64        # what a row and its group sums may take of a block's 64 KiB of LDS


def group_norm(resid: torch.Tensor, y: torch.Tensor | None, post_w: torch.Tensor | None, pre_w: torch.Tensor | None,
               out: torch.Tensor | None, groups: int, eps: float, rows: torch.Tensor | None = None) -> torch.Tensor | None:
    """RMS norm in ``groups`` equal consecutive parts of a row, around a sublayer:
    resid += norm(y; post_w) (``post_w`` None: y as it is; ``y`` None: nothing is added), then
    out = norm(resid; pre_w) (``out`` None: no second norm; ``pre_w`` None with an ``out``: out = resid, rounded). With ``rows``: only those rows, out row r from resid row
    rows[r], and resid is not written. resid float32 [T, hidden]; y, out of the model's type; weights [hidden]."""
    _gpu(resid, y, post_w, pre_w, out, rows)
    T, hidden = resid.shape
    R = T if rows is None else rows.numel()
    _need(resid.dtype == torch.float32 and resid.is_contiguous(), "group_norm: the residual stream is contiguous float32")
    _need(groups >= 1 and hidden % groups == 0, f"group_norm: {groups} groups do not divide the width {hidden}")
    _need(hidden + 5 * groups <= GROUP_NORM_MAX_FLOATS, f"group_norm: a row of {hidden} does not fit the kernel's LDS")
    _need(pre_w is None or out is not None, "group_norm: a second norm needs somewhere to put its result")
    _need(post_w is None or y is not None, "group_norm: a norm of y needs y")
    dtype = out.dtype if out is not None else y.dtype if y is not None else None
    _need(dtype is not None, "group_norm: nothing to do")
    if y is not None:
        _need(y.dtype == dtype and tuple(y.shape) == (T, hidden) and y.is_contiguous(), f"group_norm: y must be {dtype} [{T}, {hidden}]")
    if out is not None:
        _need(tuple(out.shape) == (R, hidden) and out.is_contiguous(), f"group_norm: out must be [{R}, {hidden}]")
    w_dtype = None
    for w in (post_w, pre_w):
        if w is not None:
            _need(tuple(w.shape) == (hidden,) and w.is_contiguous(), "group_norm: a weight must be [hidden]")
            _need(w_dtype in (None, w.dtype), "group_norm: both weights share one type")
            w_dtype = w.dtype
    _need(w_dtype is None or dtype == torch.bfloat16 or w_dtype == torch.float32, "group_norm: a float32 result needs float32 weights")
    if rows is not None:
        _ints(rows, R, "rows")
    _need(eps > 0, "group_norm: eps must be positive")
    _check(library().tm_group_norm(_p(resid), _p(y), _p(post_w), _p(rows), _p(pre_w), c_int(code(w_dtype or dtype)), _p(out),
                                   c_int(code(dtype)), c_int(R), c_int(hidden), c_int(groups), c_float(eps), _stream()),
           "group_norm")
    return out


# -------------------------------------------------------------------------------------------- sigmoid attention

def _check_pools_kv(k_pool: torch.Tensor, v_pool: torch.Tensor, G: int, D: int, Dv: int, dtype, who: str) -> int:
    """K pool [pages, page, G, D], V pool [pages, G, Dv, page]; returns the page size."""
    _need(k_pool.dim() == 4 and v_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous(),
          f"{who}: the cache pools must be contiguous 4-d tensors")
    pages, page = k_pool.shape[0], k_pool.shape[1]
    _need(tuple(k_pool.shape) == (pages, page, G, D), f"{who}: k_pool must be [pages, page, {G}, {D}]")
    _need(tuple(v_pool.shape) == (pages, G, Dv, page), f"{who}: v_pool must be [pages, {G}, {Dv}, page]")
    _need(k_pool.dtype == dtype and v_pool.dtype == dtype, f"{who}: the cache pools must have the type {dtype}")
    return page


def qk_norm_rope_store(qkv: torch.Tensor, H: int, G: int, D: int, Dv: int, q_w: torch.Tensor | None, k_w: torch.Tensor | None,
                       eps: float, cos: torch.Tensor | None, sin: torch.Tensor | None, positions: torch.Tensor | None,
                       slots: torch.Tensor | None, k_pool: torch.Tensor | None, v_pool: torch.Tensor | None) -> None:
    """In place on qkv [T, H*D + G*D + G*Dv]: every head of q and k is divided by its root mean square and multiplied by
    q_w / k_w (float32 [D], shared by the heads; both None: no norm), then its first 2 * cos.shape[1] channels are
    rotated by the token's position (cos/sin float32 [max_pos, rot/2]; None: no rotation); k and v go to the tokens'
    cache slots (pools None: not stored; a slot < 0 is not stored)."""
    _gpu(qkv, q_w, k_w, cos, sin, positions, slots, k_pool, v_pool)
    T = qkv.shape[0]
    width = (H + G) * D + G * Dv
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == width, f"qk_norm_rope_store: qkv must be [T, {width}]")
    _need(0 < D <= 256 and 0 < Dv, "qk_norm_rope_store: head sizes up to 256")
    _need((q_w is None) == (k_w is None), "qk_norm_rope_store: q and k are normed together or not at all")
    for w in (q_w, k_w):
        if w is not None:
            _need(w.dtype == torch.float32 and tuple(w.shape) == (D,) and w.is_contiguous(), f"qk_norm_rope_store: norm weights are float32 [{D}]")
    rot = 0
    if cos is not None:
        rot = 2 * cos.shape[1]
        _need(sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape
              and cos.is_contiguous() and sin.is_contiguous() and rot <= D, "qk_norm_rope_store: cos/sin float32 [max_pos, rot/2], rot <= D")
        _ints(positions, T, "positions")
    write = k_pool is not None
    page = 0
    if write:
        page = _check_pools_kv(k_pool, v_pool, G, D, Dv, qkv.dtype, "qk_norm_rope_store")
        _ints(slots, T, "slots")
    ld = qkv.stride(0) if T > 1 else max(width, qkv.stride(0))
    _check(library().tm_qk_norm_rope_store(_p(qkv), c_int(ld), c_int(code(qkv.dtype)), c_int(T), c_int(H), c_int(G), c_int(D),
                                           c_int(Dv), c_int(rot), _p(q_w), _p(k_w), c_float(eps), _p(cos), _p(sin),
                                           _p(positions), _p(slots), _p(k_pool), _p(v_pool), c_int(page), c_int(1 if write else 0),
                                           _stream()), "qk_norm_rope_store")


def attn_sigmoid_paged(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                       block_tables: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                       head_bias: torch.Tensor | None, H: int, G: int, D: int, Dv: int, scale: float, chunk: int = 0,
                       window: int = 0, split_keys: int = 0, most_keys: int = 0) -> torch.Tensor:
    """out[t, h] = sum over visible keys j of sigmoid(scale * q[t, h] . k[j] + head_bias[h]) * v[j]: every token of the step
    over its request's cache (its own key included), from the start of its chunk of ``chunk`` positions (0: from the
    first) and at most ``window`` back (0: any). q [T, >= H*D] with unit inner stride, out [T, H*Dv].
    ``split_keys`` > 0: a token's visible keys are dealt in runs of that many (counted from its first visible key) to
    ceil(most_keys / split_keys) wavefronts whose 32-bit sums are added in their order; ``most_keys``: the most keys any
    token of the call sees. Few tokens with long contexts then fill the chip."""
    _gpu(q, out, k_pool, v_pool, block_tables, seq_of_token, positions, head_bias)
    T = q.shape[0]
    _need(q.stride(1) == 1 and q.shape[1] >= H * D and out.is_contiguous() and tuple(out.shape) == (T, H * Dv),
          f"attention(sigmoid): q [T, >={H * D}] unit inner stride, out contiguous [T, {H * Dv}]")
    _need(q.dtype == out.dtype, "attention(sigmoid): q and out share one type")
    _need(H % G == 0 and 0 < D <= 256 and 0 < Dv <= 256, "attention(sigmoid): head sizes up to 256, heads a multiple of kv heads")
    page = _check_pools_kv(k_pool, v_pool, G, D, Dv, q.dtype, "attention(sigmoid)")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attention(sigmoid): block_tables must be contiguous int32 [S, W]")
    _ints(seq_of_token, T, "seq_of_token")
    _ints(positions, T, "positions")
    if head_bias is not None:
        _need(head_bias.dtype == torch.float32 and tuple(head_bias.shape) == (H,) and head_bias.is_contiguous(),
              f"attention(sigmoid): head_bias is float32 [{H}]")
    _need(chunk >= 0 and window >= 0, "attention(sigmoid): chunk and window must be >= 0")
    q_stride = q.stride(0) if T > 1 else max(q.stride(0), H * D)
    n_splits, parts = 0, None
    if split_keys > 0 and T > 0:
        _need(most_keys > 0, "attention(sigmoid): split keys need the most keys a token sees")
        n_splits = -(-most_keys // split_keys)
        _need(n_splits <= 65535, "attention(sigmoid): too many runs of keys")
        parts = torch.empty((n_splits, T, H * Dv), dtype=torch.float32, device=q.device)
    _check(library().tm_attn_sigmoid_paged(_p(q), c_int(q_stride), _p(out), c_int(H * Dv), _p(k_pool), _p(v_pool), _p(block_tables),
                                           c_int(block_tables.shape[1]), _p(seq_of_token), _p(positions), _p(head_bias), c_int(T),
                                           c_int(H), c_int(G), c_int(D), c_int(Dv), c_int(page), c_float(scale), c_int(chunk),
                                           c_int(window), c_int(code(q.dtype)), c_int(split_keys if n_splits else 0), c_int(n_splits),
                                           _p(parts), _stream()), "attn_sigmoid_paged")
    if parts is not None:
        sum_parts(parts, out)
    return out


# -------------------------------------------------------------------------------------------- gated linear attention

def gla_decay(z: torch.Tensor, tau: float, out: torch.Tensor | None = None) -> torch.Tensor:
    """sigmoid(z)^(1/tau) as exp(logsigmoid(z) / tau), float32; in place unless ``out`` is given."""
    out = z if out is None else out
    _gpu(z, out)
    _need(z.dtype == torch.float32 and out.dtype == torch.float32 and z.is_contiguous() and out.is_contiguous()
          and z.shape == out.shape, "gla_decay: contiguous float32 tensors of one shape")
    _need(tau > 0, "gla_decay: tau must be positive")
    _check(library().tm_gla_decay(_p(z), _p(out), c_float(tau), c_longlong(z.numel()), _stream()), "gla_decay")
    return out


def gla_scan_states_only(proj: torch.Tensor, q_off: int, k_off: int, decay: torch.Tensor, D: int) -> bool:
    """Can ``gla_scan`` run these operands without results (``o`` None), advancing the states only?"""
    ld = proj.stride(0) if proj.shape[0] > 1 else max(proj.shape[1], proj.stride(0))
    return bool(library().tm_gla_scan_in_pieces(c_int(code(proj.dtype)), _p(proj), c_int(ld), c_int(q_off), c_int(k_off), _p(decay), c_int(D)))


def gla_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, decay: torch.Tensor, o: torch.Tensor | None, state: torch.Tensor,
             cu_q_lens: torch.Tensor, state_slots: torch.Tensor, num_seqs: int, H: int, D: int, Dv: int, q_scale: float) -> torch.Tensor:
    """The recurrence S = diag(decay_t) S + k_t v_t^T, o_t = S^T (q_scale * q_t) over the rows of each request of the
    step in order, from and to the request's state row (``o`` None where ``gla_scan_states_only``: the states alone). proj [T, ld] holds q, k [H*D] and v [H*Dv] at the given column
    offsets; decay float32 [T, H*D]; o float32 [T, H*Dv]; state float32 [slots, H, D, Dv]; cu_q_lens int32 [S+1];
    state_slots int32 [S]."""
    _gpu(proj, decay, o, state, cu_q_lens, state_slots)
    T, ld_cols = proj.shape
    _need(proj.stride(1) == 1, "gla_scan: proj rows have unit inner stride")
    _need(0 < D <= 256 and Dv > 0 and H > 0, "gla_scan: key size up to 256")
    for off, n in ((q_off, H * D), (k_off, H * D), (v_off, H * Dv)):
        _need(0 <= off and off + n <= ld_cols, "gla_scan: q, k, v lie inside a row of proj")
    _need(decay.dtype == torch.float32 and decay.is_contiguous() and tuple(decay.shape) == (T, H * D), f"gla_scan: decay float32 [{T}, {H * D}]")
    if o is not None:
        _need(o.dtype == torch.float32 and o.is_contiguous() and tuple(o.shape) == (T, H * Dv), f"gla_scan: o float32 [{T}, {H * Dv}]")
    else:
        _need(gla_scan_states_only(proj, q_off, k_off, decay, D), "gla_scan: these operands are not scanned without results")
    _need(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, D, Dv),
          f"gla_scan: state float32 [slots, {H}, {D}, {Dv}]")
    _ints(cu_q_lens, num_seqs + 1, "cu_q_lens")
    _ints(state_slots, num_seqs, "state_slots")
    _need(num_seqs <= 65535, "gla_scan: at most 65,535 requests a step")
    ld = proj.stride(0) if T > 1 else max(ld_cols, proj.stride(0))
    _check(library().tm_gla_scan(_p(proj), c_int(ld), c_int(q_off), c_int(k_off), c_int(v_off), c_int(code(proj.dtype)), _p(decay),
                                 _p(o), _p(state), _p(cu_q_lens), _p(state_slots), c_int(num_seqs), c_int(H), c_int(D), c_int(Dv),
                                 c_float(q_scale), _stream()), "gla_scan")
    return o


def gla_out_gate(o: torch.Tensor, gate: torch.Tensor, w: torch.Tensor, y: torch.Tensor, H: int, Dv: int, eps: float) -> torch.Tensor:
    """y[t, h] = w * o[t, h] / rms(o[t, h]) * silu(gate[t, h]). o float32 [T, H*Dv]; gate [T, >= H*Dv] (a view with unit
    inner stride) and y [T, H*Dv] of the model's type; w float32 [Dv]."""
    _gpu(o, gate, w, y)
    T = o.shape[0]
    _need(o.dtype == torch.float32 and o.is_contiguous() and tuple(o.shape) == (T, H * Dv), f"gla_out_gate: o float32 [{T}, {H * Dv}]")
    _need(gate.stride(1) == 1 and gate.shape[0] == T and gate.shape[1] >= H * Dv and gate.dtype == y.dtype, "gla_out_gate: gate [T, >= H*Dv] of y's type")
    _need(y.is_contiguous() and tuple(y.shape) == (T, H * Dv), f"gla_out_gate: y [{T}, {H * Dv}]")
    _need(w.dtype == torch.float32 and tuple(w.shape) == (Dv,) and w.is_contiguous(), f"gla_out_gate: w float32 [{Dv}]")
    _need(eps > 0, "gla_out_gate: eps must be positive")
    ldg = gate.stride(0) if T > 1 else max(gate.stride(0), H * Dv)
    _check(library().tm_gla_out_gate(_p(o), _p(gate), c_int(ldg), c_int(code(y.dtype)), _p(w), _p(y), c_int(T), c_int(H), c_int(Dv),
                                     c_float(eps), _stream()), "gla_out_gate")
    return y


def attn_sigmoid_prefill_takes(dtype, D: int, Dv: int, page: int, q_stride: int) -> bool:
    """Does the matrix-unit kernel for prompt portions run these sizes?"""
    return dtype == torch.bfloat16 and bool(library().tm_attn_sigmoid_prefill_takes(c_int(D), c_int(Dv), c_int(page), c_int(q_stride)))


def attn_sigmoid_prefill(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                         block_tables: torch.Tensor, tiles: torch.Tensor, head_bias: torch.Tensor | None, H: int, G: int,
                         D: int, Dv: int, scale: float, chunk: int = 0, window: int = 0) -> torch.Tensor:
    """``attn_sigmoid_paged`` for the rows of a step's prompt portions, given as tiles int32 [n, 4] = (request, first row,
    tokens (1..16), position of the first token); bfloat16 on the matrix unit. Rows that belong to no tile are not written."""
    _gpu(q, out, k_pool, v_pool, block_tables, tiles, head_bias)
    T = q.shape[0]
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "attention(sigmoid, prefill): bfloat16 only")
    _need(q.stride(1) == 1 and q.shape[1] >= H * D and out.is_contiguous() and tuple(out.shape) == (T, H * Dv),
          f"attention(sigmoid, prefill): q [T, >={H * D}] unit inner stride, out contiguous [T, {H * Dv}]")
    page = _check_pools_kv(k_pool, v_pool, G, D, Dv, q.dtype, "attention(sigmoid, prefill)")
    q_stride = q.stride(0) if T > 1 else max(q.stride(0), H * D)
    _need(H % G == 0 and attn_sigmoid_prefill_takes(q.dtype, D, Dv, page, q_stride) and q.data_ptr() % 16 == 0,
          f"attention(sigmoid, prefill): sizes {D}/{Dv}, page {page}, row stride {q_stride} are not taken")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attention(sigmoid, prefill): block_tables must be contiguous int32 [S, W]")
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous(),
          "attention(sigmoid, prefill): tiles must be contiguous int32 [n, 4]")
    if head_bias is not None:
        _need(head_bias.dtype == torch.float32 and tuple(head_bias.shape) == (H,) and head_bias.is_contiguous(),
              f"attention(sigmoid, prefill): head_bias is float32 [{H}]")
    _need(chunk >= 0 and window >= 0, "attention(sigmoid, prefill): chunk and window must be >= 0")
    _check(library().tm_attn_sigmoid_prefill(_p(q), c_int(q_stride), _p(out), c_int(H * Dv), _p(k_pool), _p(v_pool),
                                             _p(block_tables), c_int(block_tables.shape[1]), _p(tiles), c_int(tiles.shape[0]),
                                             _p(head_bias), c_int(H), c_int(G), c_int(D), c_int(Dv), c_int(page), c_float(scale),
                                             c_int(chunk), c_int(window), _stream()), "attn_sigmoid_prefill")
    return out


def gla_gate_decay(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, tau: float, out: torch.Tensor) -> torch.Tensor:
    """out[t, n] = sigmoid(sum_k x[t, k] w[n, k] + bias[n])^(1/tau), the sum and what follows in 32-bit. x [T, K] (a view
    with unit inner stride), w [N, K] and bias [N] of one type, out float32 [T, N]."""
    _gpu(x, w, bias, out)
    T, K = x.shape
    N = w.shape[0]
    _need(x.stride(1) == 1 and w.is_contiguous() and tuple(w.shape) == (N, K) and w.dtype == x.dtype, f"gla_gate_decay: x [T, {K}], w [N, {K}] of one type")
    if bias is not None:
        _need(tuple(bias.shape) == (N,) and bias.is_contiguous() and bias.dtype == x.dtype, f"gla_gate_decay: bias [{N}] of x's type")
    _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (T, N), f"gla_gate_decay: out float32 [{T}, {N}]")
    _need(tau > 0, "gla_gate_decay: tau must be positive")
    ldx = x.stride(0) if T > 1 else max(K, x.stride(0))
    _check(library().tm_gla_gate_decay(_p(x), c_int(ldx), _p(w), _p(bias), c_int(code(x.dtype)), _p(out), c_int(T), c_int(N), c_int(K),
                                       c_float(tau), _stream()), "gla_gate_decay")
    return out


def gla_segment_decay(decay: torch.Tensor, cu_seg: torch.Tensor, n_seg: int, out: torch.Tensor) -> torch.Tensor:
    """out[c, j] = product over the rows cu_seg[c] .. cu_seg[c + 1] - 1 of decay[t, j]. decay float32 [T, HD]."""
    _gpu(decay, cu_seg, out)
    T, HD = decay.shape
    _need(decay.dtype == torch.float32 and decay.is_contiguous(), "gla_segment_decay: decay is contiguous float32 [T, HD]")
    _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (n_seg, HD), f"gla_segment_decay: out float32 [{n_seg}, {HD}]")
    _ints(cu_seg, n_seg + 1, "cu_seg")
    _need(n_seg <= 65535, "gla_segment_decay: at most 65,535 segments")
    _check(library().tm_gla_segment_decay(_p(decay), _p(cu_seg), _p(out), c_int(n_seg), c_int(HD), _stream()), "gla_segment_decay")
    return out


def gla_combine(state: torch.Tensor, state_slots: torch.Tensor, first_seg: torch.Tensor, seg_decay: torch.Tensor,
                local: torch.Tensor, start: torch.Tensor, num_seqs: int) -> None:
    """For request s with segments first_seg[s] .. first_seg[s + 1] - 1: start[c] = B, B = diag(seg_decay[c]) B + local[c] in
    their order, from B = state[state_slots[s]], which receives the last B. state [slots, H, D, Dv]; local, start
    [n_seg, H, D, Dv]; seg_decay [n_seg, H * D]; all float32."""
    _gpu(state, state_slots, first_seg, seg_decay, local, start)
    n_seg = local.shape[0]
    H, D, Dv = state.shape[1:]
    for t, shape, name in ((state, None, "state"), (local, (n_seg, H, D, Dv), "local"), (start, (n_seg, H, D, Dv), "start"),
                           (seg_decay, (n_seg, H * D), "seg_decay")):
        _need(t.dtype == torch.float32 and t.is_contiguous() and (shape is None or tuple(t.shape) == shape), f"gla_combine: {name} float32 {shape}")
    _ints(state_slots, num_seqs, "state_slots")
    _ints(first_seg, num_seqs + 1, "first_seg")
    _need(num_seqs <= 65535, "gla_combine: at most 65,535 requests a step")
    _check(library().tm_gla_combine(_p(state), _p(state_slots), _p(first_seg), _p(seg_decay), _p(local), _p(start), c_int(num_seqs),
                                    c_int(H * D), c_int(Dv), _stream()), "gla_combine")


# -------------------------------------------------------------------------------------------- layer norm, short convolution, PolyNorm

def layer_norm(resid: torch.Tensor, y: torch.Tensor | None, gate: torch.Tensor | None, mult: float, w: torch.Tensor | None,
               b: torch.Tensor | None, out: torch.Tensor | None, eps: float, rows: torch.Tensor | None = None, dtype=None):
    """v = resid + mult * y * sigmoid(gate) (gate None: no gate; y None: nothing is added); with ``rows`` None every row runs
    and v is written back to resid (float32 [T, hidden]); out = (v - mean) / sqrt(var + eps) * w + b (out None: the add
    alone). With ``rows`` (int32 [R]) only those rows are read, resid stays as it is and out is [R, hidden]. y, gate and out
    share one type; w, b are float32 [hidden]."""
    _gpu(resid, y, gate, w, b, out, rows)
    T, hidden = resid.shape
    R = T if rows is None else rows.numel()
    _need(resid.dtype == torch.float32 and resid.is_contiguous(), "layer_norm: the residual stream is contiguous float32")
    _need(hidden <= 16384, "layer_norm: rows of up to 16,384 elements")
    dt = dtype
    for t, name in ((y, "y"), (gate, "gate")):
        if t is not None:
            _need(tuple(t.shape) == (T, hidden) and t.is_contiguous(), f"layer_norm: {name} must be contiguous [{T}, {hidden}]")
            _need(dt in (None, t.dtype), "layer_norm: y, gate and out share one type")
            dt = t.dtype
    if out is not None:
        _need(tuple(out.shape) == (R, hidden) and out.is_contiguous(), f"layer_norm: out must be contiguous [{R}, {hidden}]")
        _need(dt in (None, out.dtype), "layer_norm: y, gate and out share one type")
        dt = out.dtype
        for t in (w, b):
            _need(t is not None and t.dtype == torch.float32 and tuple(t.shape) == (hidden,) and t.is_contiguous(),
                  f"layer_norm: weight and bias are float32 [{hidden}]")
    _need(gate is None or y is not None, "layer_norm: a gate needs something to gate")
    _need(dt is not None, "layer_norm: nothing to do")
    if rows is not None:
        _ints(rows, R, "rows")
    _need(eps > 0, "layer_norm: eps must be positive")
    _check(library().tm_layer_norm(_p(resid), _p(y), _p(gate), c_float(mult), _p(rows), _p(w), _p(b), _p(out), c_int(code(dt)),
                                   c_int(R), c_int(hidden), c_float(eps), _stream()), "layer_norm")
    return out


SHORT_CONV_WALK_ROWS = 8        # up to this many rows a request, a step's convolution and its new state are one launch


def short_conv(h: torch.Tensor, w: torch.Tensor, state: torch.Tensor | None, cu_q_lens: torch.Tensor, state_slots: torch.Tensor,
               seq_of_token: torch.Tensor, num_seqs: int, out: torch.Tensor, most_rows: int = 0) -> torch.Tensor:
    """out[t] = h[t] + sum_j w[:, j] * h[t - taps + 1 + j] within each request (rows cu_q_lens[s] .. cu_q_lens[s + 1] - 1 of h),
    the rows before the step's first taken from state[state_slots[s]] ([taps - 1, width]); afterwards that state holds the
    last taps - 1 rows the request has seen. h, w [width, taps], state [slots, taps - 1, width] and out share one type.
    ``most_rows``: the most rows any request brings, if known: few rows a request (single tokens) take one launch in which a
    thread walks a request's rows, otherwise the convolution and the state's update are two; both give the same bits."""
    _gpu(h, w, state, cu_q_lens, state_slots, seq_of_token, out)
    T, width = h.shape
    taps = w.shape[1]
    _need(h.is_contiguous() and out.is_contiguous() and out.shape == h.shape and out.dtype == h.dtype and out.data_ptr() != h.data_ptr(),
          "short_conv: h and out are two contiguous tensors of one shape and type")
    _need(tuple(w.shape) == (width, taps) and w.is_contiguous() and w.dtype == h.dtype and 1 <= taps <= 16,
          "short_conv: w must be [width, taps] of h's type, taps up to 16")
    if taps > 1:
        _need(state is not None and state.dim() == 3 and tuple(state.shape[1:]) == (taps - 1, width) and state.is_contiguous()
              and state.dtype == h.dtype, f"short_conv: state must be [slots, {taps - 1}, {width}] of h's type")
    _ints(cu_q_lens, num_seqs + 1, "cu_q_lens")
    _ints(state_slots, num_seqs, "state_slots")
    _ints(seq_of_token, T, "seq_of_token")
    lib = library()
    if taps > 1 and 0 < most_rows <= SHORT_CONV_WALK_ROWS:
        _check(lib.tm_short_conv_walk(_p(h), _p(out), _p(w), _p(state), _p(cu_q_lens), _p(state_slots), c_int(num_seqs), c_int(width),
                                      c_int(taps), c_int(code(h.dtype)), _stream()), "short_conv_walk")
        return out
    _check(lib.tm_short_conv(_p(h), _p(out), _p(w), _p(state), _p(cu_q_lens), _p(state_slots), _p(seq_of_token), c_int(T),
                             c_int(width), c_int(taps), c_int(code(h.dtype)), _stream()), "short_conv")
    if taps > 1:
        _check(lib.tm_short_conv_state(_p(h), _p(state), _p(cu_q_lens), _p(state_slots), c_int(num_seqs), c_int(width), c_int(taps),
                                       c_int(code(h.dtype)), _stream()), "short_conv_state")
    return out


def poly_norm(z: torch.Tensor, coef: torch.Tensor, out: torch.Tensor, eps: float) -> torch.Tensor:
    """out = a N(z) + b N(z^2) + c N(z^3) + e, (a, b, c, e) = coef (float32 [4] on the device), N(v) = v / sqrt(mean(v^2) + eps)
    over a row; z float32 [T, F]."""
    _gpu(z, coef, out)
    _need(z.dtype == torch.float32 and z.dim() == 2 and z.is_contiguous(), "poly_norm: z is contiguous float32 [T, F]")
    _need(coef.dtype == torch.float32 and coef.numel() == 4 and coef.is_contiguous(), "poly_norm: four float32 coefficients")
    _need(out.shape == z.shape and out.is_contiguous(), "poly_norm: out has z's shape")
    _need(eps > 0, "poly_norm: eps must be positive")
    _check(library().tm_poly_norm(_p(z), _p(coef), _p(out), c_int(code(out.dtype)), c_int(z.shape[0]), c_int(z.shape[1]),
                                  c_float(eps), _stream()), "poly_norm")
    return out


# -------------------------------------------------------------------------------------------- attention over a shared latent

def _check_latent_pool(pool: torch.Tensor, Dk: int, dtype, who: str) -> int:
    """The cached rows [pages, page, 1, Dk]; returns the page size."""
    _need(pool.dim() == 4 and pool.is_contiguous() and pool.shape[2] == 1 and pool.shape[3] == Dk and pool.dtype == dtype,
          f"{who}: the pool must be contiguous [pages, page, 1, {Dk}] of type {dtype}")
    return pool.shape[1]


def _angles(cos, sin, rot: int, positions, T: int, who: str) -> None:
    if rot:
        _need(cos is not None and sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32
              and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == rot // 2 and cos.is_contiguous() and sin.is_contiguous(),
              f"{who}: cos/sin float32 [positions, {rot // 2}]")
        _ints(positions, T, "positions")


def latent_prepare(low: torch.Tensor, Lq: int, Lk: int, Dr: int, wq: torch.Tensor | None, wk: torch.Tensor | None, eps: float,
                   cos: torch.Tensor | None, sin: torch.Tensor | None, positions: torch.Tensor | None, slots: torch.Tensor | None,
                   cq: torch.Tensor | None, pool: torch.Tensor | None, half_pairs: bool = False) -> None:
    """low float32 [T, >= Lq + Lk + Dr] = [query latent | key/value latent | shared key]: cq [T, Lq] = rms_norm(query latent) * wq;
    the cache row of token t (slot slots[t] of pool; < 0: not stored) = [rms_norm(latent) * wk | shared key with its first
    2 * cos.shape[1] channels rotated in pairs (2i, 2i + 1), or (i, i + half) with ``half_pairs``, by the token's position].
    Lk = 0 (with Dr = 0 and no slots): a layer that has only queries of its own."""
    _gpu(low, wq, wk, cos, sin, positions, slots, cq, pool)
    T = low.shape[0]
    _need(low.dtype == torch.float32 and low.dim() == 2 and low.stride(1) == 1 and low.shape[1] >= Lq + Lk + Dr,
          f"latent_prepare: low is float32 [T, >= {Lq + Lk + Dr}]")
    if Lk:
        _need(wk is not None and wk.dtype == torch.float32 and tuple(wk.shape) == (Lk,) and wk.is_contiguous(),
              f"latent_prepare: wk is float32 [{Lk}]")
    else:
        _need(Dr == 0 and slots is None and Lq > 0, "latent_prepare: without a key/value latent there is nothing to store")
    dt = None
    if Lq:
        _need(wq is not None and wq.dtype == torch.float32 and tuple(wq.shape) == (Lq,) and wq.is_contiguous(),
              f"latent_prepare: wq is float32 [{Lq}]")
        _need(cq is not None and tuple(cq.shape) == (T, Lq) and cq.is_contiguous(), f"latent_prepare: cq is contiguous [T, {Lq}]")
        dt = cq.dtype
    rot = 2 * cos.shape[1] if (cos is not None and Dr) else 0
    _need(rot <= Dr, "latent_prepare: more rotated channels than the shared key has")
    _angles(cos, sin, rot, positions, T, "latent_prepare")
    if slots is not None:
        _need(pool is not None, "latent_prepare: slots without a pool")
        _check_latent_pool(pool, Lk + Dr, dt or pool.dtype, "latent_prepare")
        dt = pool.dtype
        _ints(slots, T, "slots")
    _need(dt is not None, "latent_prepare: nothing to do")
    ld = low.stride(0) if T > 1 else max(low.stride(0), low.shape[1])
    _check(library().tm_latent_prepare(_p(low), c_int(ld), c_int(Lq), c_int(Lk), c_int(Dr), c_int(rot), _p(wq), _p(wk), c_float(eps),
                                       _p(cos if rot else None), _p(sin if rot else None), _p(positions if rot else None), _p(slots), _p(cq),
                                       _p(pool if slots is not None else None), c_int(code(dt)), c_int(T), c_int(1 if half_pairs else 0),
                                       _stream()), "latent_prepare")


def heads_matmul(a: torch.Tensor, a_head: int, b: torch.Tensor, c: torch.Tensor, c_head: int,
                 gate: torch.Tensor | None = None) -> torch.Tensor:
    """c[t, h * c_head + n] = sum_k a[t, h * a_head + k] * b[h, k, n] for n < N, k < K (b [H, K, N]); with ``gate`` (float32
    [T, >= H], rows may be strided) the result is multiplied by sigmoid(gate[t, h]). a, b, c share one type; rows may be strided."""
    _gpu(a, b, c, gate)
    T = a.shape[0]
    H, K, N = b.shape
    _need(a.dim() == 2 and c.dim() == 2 and a.stride(1) == 1 and c.stride(1) == 1 and c.shape[0] == T and b.is_contiguous(),
          "heads_matmul: a, c [T, .] with unit inner stride, b contiguous [H, K, N]")
    _need(a.dtype == b.dtype == c.dtype, "heads_matmul: one type")
    _need(a_head >= K and c_head >= N and a.shape[1] >= (H - 1) * a_head + K and c.shape[1] >= (H - 1) * c_head + N,
          "heads_matmul: the heads do not fit the rows")
    gate_stride = 0
    if gate is not None:
        _need(gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == T and gate.shape[1] >= H and gate.stride(1) == 1,
              "heads_matmul: gate is float32 [T, >= H]")
        gate_stride = gate.stride(0) if T > 1 else max(gate.stride(0), H)
    lda = a.stride(0) if T > 1 else max(a.stride(0), a.shape[1])
    ldc = c.stride(0) if T > 1 else max(c.stride(0), c.shape[1])
    _check(library().tm_heads_matmul(_p(a), c_int(lda), c_int(a_head), _p(b), _p(c), c_int(ldc), c_int(c_head), _p(gate),
                                     c_int(gate_stride), c_int(T), c_int(H), c_int(K), c_int(N), c_int(code(a.dtype)), _stream()),
           "heads_matmul")
    return c


def heads_matmul_mfma_takes(a: torch.Tensor, a_head: int, w: torch.Tensor) -> bool:
    """Does the matrix-unit kernel take this per-head product (bfloat16, whole 16-byte pieces)? w [H, N, K]."""
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or not a.is_cuda:
        return False
    lda = a.stride(0) if a.shape[0] > 1 else max(a.stride(0), a.shape[1])
    return bool(library().tm_heads_matmul_mfma_takes(_p(a), c_int(lda), c_int(a_head), _p(w), c_int(w.shape[2])))


def heads_matmul_mfma(a: torch.Tensor, a_head: int, w: torch.Tensor, c: torch.Tensor, c_head: int,
                      gate: torch.Tensor | None = None, tail: int = 0, cos: torch.Tensor | None = None,
                      sin: torch.Tensor | None = None, positions: torch.Tensor | None = None, half_pairs: bool = False) -> torch.Tensor:
    """``heads_matmul`` on the matrix unit, with the matrices given as w [H, N, K] (k contiguous): c[t, h * c_head + n] =
    sum_k a[t, h * a_head + k] * w[h, n, k], times sigmoid(gate[t, h]) if ``gate`` (float32 [T, >= H]). ``tail`` > 0: the
    ``tail`` channels behind a head's K input channels are copied behind its N output channels, the first 2 * cos.shape[1]
    of them rotated in pairs (2i, 2i + 1), or (i, i + half) with ``half_pairs``, by the row's position (``rotate_heads`` in the
    same launch)."""
    _gpu(a, w, c, gate)
    T = a.shape[0]
    H, N, K = w.shape
    _need(a.dim() == 2 and c.dim() == 2 and a.stride(1) == 1 and c.stride(1) == 1 and c.shape[0] == T and w.is_contiguous(),
          "heads_matmul: a, c [T, .] with unit inner stride, w contiguous [H, N, K]")
    _need(a.dtype == w.dtype == c.dtype == torch.bfloat16, "heads_matmul (matrix unit): bfloat16")
    _need(tail >= 0 and a_head >= K + tail and c_head >= N + tail and a.shape[1] >= (H - 1) * a_head + K + tail
          and c.shape[1] >= (H - 1) * c_head + N + tail, "heads_matmul: the heads do not fit the rows")
    _need(heads_matmul_mfma_takes(a, a_head, w), "heads_matmul (matrix unit): operands not in whole 16-byte pieces")
    rot = 2 * cos.shape[1] if (cos is not None and tail) else 0
    _need(rot <= tail, "heads_matmul: more rotated channels than the tail has")
    _angles(cos, sin, rot, positions, T, "heads_matmul")
    _gpu(cos, sin, positions)
    gate_stride = 0
    if gate is not None:
        _need(gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == T and gate.shape[1] >= H and gate.stride(1) == 1,
              "heads_matmul: gate is float32 [T, >= H]")
        gate_stride = gate.stride(0) if T > 1 else max(gate.stride(0), H)
    lda = a.stride(0) if T > 1 else max(a.stride(0), a.shape[1])
    ldc = c.stride(0) if T > 1 else max(c.stride(0), c.shape[1])
    _check(library().tm_heads_matmul_mfma(_p(a), c_int(lda), c_int(a_head), _p(w), _p(c), c_int(ldc), c_int(c_head), _p(gate),
                                          c_int(gate_stride), c_int(T), c_int(H), c_int(K), c_int(N), c_int(tail), c_int(rot),
                                          _p(cos if rot else None), _p(sin if rot else None), _p(positions if rot else None),
                                          c_int(1 if half_pairs else 0), _stream()), "heads_matmul_mfma")
    return c


def rotate_heads(src: torch.Tensor, src_head: int, dst: torch.Tensor, dst_head: int, H: int, Dr: int, cos: torch.Tensor | None,
                 sin: torch.Tensor | None, positions: torch.Tensor | None, half_pairs: bool = False) -> None:
    """dst[t, h * dst_head + c] = src[t, h * src_head + c] for c < Dr, the first 2 * cos.shape[1] channels of every head rotated in
    pairs (2i, 2i + 1) by the token's position. src and dst are views that start at the heads' first rotated channel."""
    _gpu(src, dst, cos, sin, positions)
    T = src.shape[0]
    _need(src.dim() == 2 and dst.dim() == 2 and src.stride(1) == 1 and dst.stride(1) == 1 and dst.shape[0] == T and src.dtype == dst.dtype,
          "rotate_heads: src, dst [T, .] of one type with unit inner stride")
    _need(src_head >= Dr and dst_head >= Dr and src.shape[1] >= (H - 1) * src_head + Dr and dst.shape[1] >= (H - 1) * dst_head + Dr,
          "rotate_heads: the heads do not fit the rows")
    rot = 2 * cos.shape[1] if cos is not None else 0
    _need(rot <= Dr, "rotate_heads: more rotated channels than a head has")
    _angles(cos, sin, rot, positions, T, "rotate_heads")
    lds = src.stride(0) if T > 1 else max(src.stride(0), src.shape[1])
    ldd = dst.stride(0) if T > 1 else max(dst.stride(0), dst.shape[1])
    _check(library().tm_rotate_heads(_p(src), c_int(lds), c_int(src_head), _p(dst), c_int(ldd), c_int(dst_head), c_int(T), c_int(H),
                                     c_int(Dr), c_int(rot), _p(cos), _p(sin), _p(positions), c_int(code(src.dtype)),
                                     c_int(1 if half_pairs else 0), _stream()), "rotate_heads")


LATENT_MAX_ROW, LATENT_MAX_RANK = 704, 512


def _check_sink(sink: torch.Tensor | None, H: int) -> None:
    if sink is not None:
        _need(sink.dtype == torch.float32 and tuple(sink.shape) == (H,) and sink.is_contiguous(), f"attention: sink is float32 [{H}]")


def attn_latent(qa: torch.Tensor, out: torch.Tensor, pool: torch.Tensor, block_tables: torch.Tensor, seq_of_token: torch.Tensor,
                positions: torch.Tensor, H: int, Lk: int, Dk: int, scale: float, window: int = 0,
                sink: torch.Tensor | None = None) -> torch.Tensor:
    """out[t, h, :Lk] = sum_j softmax_j(scale * qa[t, h, :Dk] . row[j]) * row[j, :Lk] over the cached rows j of the token's
    request with 0 <= position - j < window (0: every row up to the token's own). qa [T, H * Dk], out [T, H * Lk]. ``sink``
    (float32 [H]): one more term exp(sink[h]) in the softmax's denominator, with no row behind it."""
    _gpu(qa, out, pool, block_tables, seq_of_token, positions, sink)
    _check_sink(sink, H)
    T = qa.shape[0]
    _need(qa.is_contiguous() and tuple(qa.shape) == (T, H * Dk) and out.is_contiguous() and tuple(out.shape) == (T, H * Lk)
          and qa.dtype == out.dtype, f"attention(latent): qa [T, {H * Dk}] and out [T, {H * Lk}] contiguous, of one type")
    _need(0 < Lk <= Dk <= LATENT_MAX_ROW and Lk <= LATENT_MAX_RANK, f"attention(latent): rows of up to {LATENT_MAX_ROW} with a latent of up to {LATENT_MAX_RANK}")
    page = _check_latent_pool(pool, Dk, qa.dtype, "attention(latent)")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attention(latent): block_tables must be contiguous int32 [S, W]")
    _ints(seq_of_token, T, "seq_of_token")
    _ints(positions, T, "positions")
    _need(window >= 0, "attention(latent): window must be >= 0")
    _check(library().tm_attn_latent(_p(qa), c_int(H * Dk), _p(out), c_int(H * Lk), _p(pool), _p(block_tables), c_int(block_tables.shape[1]),
                                    _p(seq_of_token), _p(positions), c_int(T), c_int(H), c_int(Lk), c_int(Dk), c_int(page),
                                    c_float(scale), c_int(window), _p(sink), c_int(code(qa.dtype)), _stream()), "attn_latent")
    return out


def attn_latent_mfma_takes(dtype, Lk: int, Dk: int, H: int) -> bool:
    """Does the matrix-unit kernel run these sizes (bfloat16, latent and row in whole 16-byte pieces)?"""
    return dtype == torch.bfloat16 and bool(library().tm_attn_latent_mfma_takes(c_int(Lk), c_int(Dk), c_int(H * Dk), c_int(H * Lk)))


def attn_latent_mfma(qa: torch.Tensor, out: torch.Tensor, pool: torch.Tensor, block_tables: torch.Tensor, tiles: torch.Tensor | None,
                     seq_of_token: torch.Tensor, positions: torch.Tensor, first_single: int, n_single: int, H: int, Lk: int, Dk: int,
                     scale: float, window: int = 0, most_context: int = 0, bound: int = 0,
                     sink: torch.Tensor | None = None) -> torch.Tensor:
    """``attn_latent`` on the matrix unit for bfloat16: with ``tiles`` (int32 [n, 4]: request, first row, tokens, first position)
    the prompt portions of the step, tile by tile; with ``tiles`` None the ``n_single`` single tokens that start at row
    ``first_single``, none of which sits beyond position ``most_context`` - 1 (their visible rows are dealt in chunks to blocks
    of their own and merged in chunk order; ``bound``: the most rows the model lets any token see, its window or its longest
    context, which sets the chunks' size). Rows of qa / out that neither names are left alone."""
    _gpu(qa, out, pool, block_tables, tiles, seq_of_token, positions, sink)
    _check_sink(sink, H)
    T = qa.shape[0]
    _need(qa.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "attention(latent, matrix unit): bfloat16 only")
    _need(qa.is_contiguous() and tuple(qa.shape) == (T, H * Dk) and out.is_contiguous() and tuple(out.shape) == (T, H * Lk),
          f"attention(latent, matrix unit): qa [T, {H * Dk}] and out [T, {H * Lk}] contiguous")
    _need(attn_latent_mfma_takes(qa.dtype, Lk, Dk, H), "attention(latent, matrix unit): sizes the kernel does not run")
    page = _check_latent_pool(pool, Dk, qa.dtype, "attention(latent, matrix unit)")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attention(latent, matrix unit): block_tables must be contiguous int32 [S, W]")
    _ints(seq_of_token, T, "seq_of_token")
    _ints(positions, T, "positions")
    _need(window >= 0, "attention(latent, matrix unit): window must be >= 0")
    n_tiles, n_chunks, chunk_runs, part_o, part_ml = 0, 0, 0, None, None
    if tiles is not None:
        _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 4 and tiles.is_contiguous(), "tiles must be int32 [n, 4]")
        n_tiles, n_single = tiles.shape[0], 0
    elif n_single > 0:
        _need(0 <= first_single and first_single + n_single <= T, "attention(latent, matrix unit): the single tokens lie outside the step")
        _need(most_context > 0, "attention(latent, matrix unit): single tokens need the longest context among them")
        chunk_runs = int(library().tm_attn_latent_chunk_runs(c_int(window if window else max(bound, most_context))))
        n_chunks = int(library().tm_attn_latent_chunks(c_int(min(window, most_context) if window else most_context), c_int(chunk_runs)))
        part_o = torch.empty((n_single * H, n_chunks, Lk), dtype=torch.float32, device=qa.device)
        part_ml = torch.empty((n_single * H, n_chunks, 2), dtype=torch.float32, device=qa.device)
    _check(library().tm_attn_latent_mfma(_p(qa), c_int(H * Dk), _p(out), c_int(H * Lk), _p(pool), _p(block_tables),
                                         c_int(block_tables.shape[1]), _p(tiles), c_int(n_tiles), _p(seq_of_token), _p(positions),
                                         c_int(first_single), c_int(n_single), _p(part_o), _p(part_ml), c_int(n_chunks), c_int(chunk_runs), c_int(H),
                                         c_int(Lk), c_int(Dk), c_int(page), c_float(scale), c_int(window), _p(sink), _stream()),
           "attn_latent_mfma")
    return out


# -------------------------------------------------------------------------------------------- experts by table

MOE_TILE_ROWS = 32
MOE_MAX_EXPERTS = 1024


def moe_max_tiles(pairs: int, experts: int, tile_rows: int = MOE_TILE_ROWS) -> int:
    """The most tiles of ``tile_rows`` rows that ``pairs`` (token, expert) pairs can fall into."""
    return min(pairs, pairs // tile_rows + experts)


def moe_tile_rows(pairs: int, experts: int, dtype) -> int:
    """Rows of a tile for a step of ``pairs`` pairs: 32, or 64 / 128 where the matrix-unit products (bfloat16) have that many
    rows an expert on average, so that an expert's matrices are read fewer times. A row's result does not depend on it."""
    if dtype != torch.bfloat16:
        return MOE_TILE_ROWS
    per_expert = pairs // max(experts, 1)
    return 128 if per_expert >= 96 else (64 if per_expert >= 48 else MOE_TILE_ROWS)


def moe_route(token_ids: torch.Tensor, table: torch.Tensor, experts: int, tile_rows: int = MOE_TILE_ROWS):
    """Sorts the step's (token, choice) pairs by expert. Returns int32 tensors (slot_pair [P], pair_slot [P], tiles [max, 3],
    n_tiles [1]) and the tiles' rows; see ``csrc/moe.hip``."""
    _gpu(token_ids, table)
    T = token_ids.numel()
    _need(table.dtype == torch.int32 and table.dim() == 2 and table.is_contiguous(), "moe_route: table is contiguous int32 [vocab, top]")
    _ints(token_ids, T, "token_ids")
    top = table.shape[1]
    _need(0 < experts <= MOE_MAX_EXPERTS, f"moe_route: up to {MOE_MAX_EXPERTS} experts")
    P = T * top
    _need(tile_rows in (32, 64, 128), "moe_route: tiles of 32, 64 or 128 rows")
    most = moe_max_tiles(P, experts, tile_rows)
    work = torch.empty(2 * P + 3 * most + 1, dtype=torch.int32, device=token_ids.device)
    slot_pair, pair_slot, tiles, n_tiles = work[:P], work[P:2 * P], work[2 * P:2 * P + 3 * most].view(most, 3), work[2 * P + 3 * most:]
    _check(library().tm_moe_route(_p(token_ids), _p(table), c_int(T), c_int(top), c_int(experts), c_int(tile_rows), _p(slot_pair),
                                  _p(pair_slot), _p(tiles), _p(n_tiles), _stream()), "moe_route")
    return slot_pair, pair_slot, tiles, n_tiles, tile_rows


def moe_experts(x: torch.Tensor, routed, w_gate_up: torch.Tensor, w_down: torch.Tensor, top: int, weight: float,
                out: torch.Tensor) -> torch.Tensor:
    """out[t] = sum over the token's ``top`` experts e of weight * Wd[e] (silu(Wg[e] x[t]) * (Wu[e] x[t])), in the order of
    its choices. w_gate_up [E, 2F, K] (gate rows, then up rows), w_down [E, N, F]; ``routed`` from ``moe_route``."""
    slot_pair, pair_slot, tiles, n_tiles, tile_rows = routed
    _gpu(x, w_gate_up, w_down, out)
    T, K = x.shape
    E, F2, K2 = w_gate_up.shape
    F = F2 // 2
    N = w_down.shape[1]
    P = T * top
    _need(x.stride(1) == 1 and K2 == K and F2 == 2 * F and tuple(w_down.shape) == (E, N, F) and w_gate_up.is_contiguous()
          and w_down.is_contiguous(), "moe_experts: x [T, K], w_gate_up [E, 2F, K], w_down [E, N, F]")
    _need(x.dtype == w_gate_up.dtype == w_down.dtype == out.dtype, "moe_experts: one type")
    _need(tuple(out.shape) == (T, N) and out.is_contiguous(), f"moe_experts: out is contiguous [{T}, {N}]")
    _need(slot_pair.numel() == P and pair_slot.numel() == P, "moe_experts: the routing belongs to another step")
    most = tiles.shape[0]
    act = torch.empty((P, F), dtype=x.dtype, device=x.device)
    part = torch.empty((P, N), dtype=torch.float32, device=x.device)
    lib, dt = library(), c_int(code(x.dtype))
    ldx = x.stride(0) if T > 1 else max(x.stride(0), K)
    if x.dtype == torch.bfloat16 and lib.tm_moe_mfma_takes(_p(x), c_int(ldx), _p(w_gate_up), _p(w_down), _p(act), c_int(K), c_int(F)):
        # the matrix unit takes the same tiles
        _check(lib.tm_moe_gate_up_mfma(_p(x), c_int(ldx), _p(slot_pair), c_int(top), _p(w_gate_up), _p(act), _p(tiles), _p(n_tiles),
                                       c_int(most), c_int(tile_rows), c_int(K), c_int(F), _stream()), "moe_gate_up_mfma")
        _check(lib.tm_moe_down_mfma(_p(act), _p(w_down), _p(part), _p(tiles), _p(n_tiles), c_int(most), c_int(tile_rows), c_int(F),
                                    c_int(N), _stream()), "moe_down_mfma")
        _check(lib.tm_moe_combine(_p(part), _p(pair_slot), _p(out), c_int(T), c_int(top), c_float(weight), c_int(N), dt, _stream()),
               "moe_combine")
        return out
    _need(tile_rows == MOE_TILE_ROWS, "moe_experts: these products take tiles of 32 rows")
    _check(lib.tm_moe_gate_up(_p(x), c_int(ldx), _p(slot_pair), c_int(top), _p(w_gate_up), _p(act), _p(tiles), _p(n_tiles), c_int(most),
                              c_int(K), c_int(F), dt, _stream()), "moe_gate_up")
    _check(lib.tm_moe_down(_p(act), _p(w_down), _p(part), _p(tiles), _p(n_tiles), c_int(most), c_int(F), c_int(N), dt, _stream()),
           "moe_down")
    _check(lib.tm_moe_combine(_p(part), _p(pair_slot), _p(out), c_int(T), c_int(top), c_float(weight), c_int(N), dt, _stream()),
           "moe_combine")
    return out


# -------------------------------------------------------------------------------------------- softmax attention with extras

def whole_norm_rope_store(proj: torch.Tensor, q_out: torch.Tensor, H: int, G: int, D: int, Dv: int, q_w: torch.Tensor | None,
                          k_w: torch.Tensor | None, eps: float, cos: torch.Tensor | None, sin: torch.Tensor | None, interleaved: bool,
                          positions: torch.Tensor | None, slots: torch.Tensor | None, k_pool: torch.Tensor | None,
                          v_pool: torch.Tensor | None, has_kv: bool = True, per_head: bool = False) -> torch.Tensor:
    """proj float32 [T, >= H*D (+ G*D + G*Dv)]: q (and k) are divided by the root mean square of the whole projection (all
    heads of a token at once) and multiplied by q_w [H*D] / k_w [G*D] (float32; None: no norm), the first 2 * cos.shape[1]
    channels of every head rotated by the token's position (pairs (j, j + rot/2), or (2j, 2j + 1) if ``interleaved``); q goes
    to q_out [T, H*D], k and v to the tokens' cache slots. ``has_kv`` False: the row holds no k and v (a layer that reads
    another layer's cache). ``per_head``: every head of q and of k is normed by itself over its D channels, with weights [D] that
    the heads share."""
    _gpu(proj, q_out, q_w, k_w, cos, sin, positions, slots, k_pool, v_pool)
    T = proj.shape[0]
    width = H * D + (G * (D + Dv) if has_kv else 0)
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= width,
          f"whole_norm_rope_store: proj is float32 [T, >= {width}]")
    _need(tuple(q_out.shape) == (T, H * D) and q_out.is_contiguous(), f"whole_norm_rope_store: q_out is contiguous [T, {H * D}]")
    for w, n in ((q_w, D if per_head else H * D), (k_w, D if per_head else G * D)):
        if w is not None:
            _need(w.dtype == torch.float32 and tuple(w.shape) == (n,) and w.is_contiguous(), f"whole_norm_rope_store: a norm weight is float32 [{n}]")
    _need(not per_head or H + G <= 1024, "whole_norm_rope_store: up to 1024 heads of q and k are normed by themselves")
    _need(not has_kv or (q_w is None) == (k_w is None), "whole_norm_rope_store: q and k are normed together or not at all")
    rot = 0
    if cos is not None:
        rot = 2 * cos.shape[1]
        _need(sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape
              and cos.is_contiguous() and sin.is_contiguous() and rot <= D, "whole_norm_rope_store: cos/sin float32 [max_pos, rot/2], rot <= D")
        _ints(positions, T, "positions")
    write = has_kv and k_pool is not None
    page = 0
    if write:
        page = _check_pools_kv(k_pool, v_pool, G, D, Dv, q_out.dtype, "whole_norm_rope_store")
        _ints(slots, T, "slots")
    ld = proj.stride(0) if T > 1 else max(width, proj.stride(0))
    _check(library().tm_whole_norm_rope_store(_p(proj), c_int(ld), _p(q_out), c_int(code(q_out.dtype)), c_int(T), c_int(H), c_int(G),
                                              c_int(D), c_int(Dv), c_int(rot), c_int(1 if interleaved else 0), _p(q_w), _p(k_w),
                                              c_float(eps), _p(cos), _p(sin), _p(positions), _p(slots if write else None),
                                              _p(k_pool if write else None), _p(v_pool if write else None), c_int(page),
                                              c_int(1 if has_kv else 0), c_int(1 if per_head else 0), _stream()), "whole_norm_rope_store")
    return q_out


def attn_paged_softmax(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, block_tables: torch.Tensor,
                       seq_of_token: torch.Tensor, positions: torch.Tensor, H: int, G: int, D: int, Dv: int, scale: float,
                       window: int = 0, softcap: float = 0.0, gate: torch.Tensor | None = None) -> torch.Tensor:
    """Softmax attention of every token of the step over its request's cached keys (its own included), a token and a head a
    wavefront: keys of D channels, values of Dv; a score s becomes softcap * tanh(s / softcap) if ``softcap`` > 0; head h of
    token t is multiplied by sigmoid(gate[t, h]) (gate: a float32 view [T, >= H] with unit inner stride; None: no gate).
    q [T, >= H*D] with unit inner stride, out [T, H*Dv]."""
    _gpu(q, out, k_pool, v_pool, block_tables, seq_of_token, positions, gate)
    T = q.shape[0]
    _need(q.stride(1) == 1 and q.shape[1] >= H * D and out.is_contiguous() and tuple(out.shape) == (T, H * Dv),
          f"attention: q [T, >={H * D}] unit inner stride, out contiguous [T, {H * Dv}]")
    _need(q.dtype == out.dtype, "attention: q and out share one type")
    _need(H % G == 0 and D % 4 == 0 and 0 < D <= 256 and 0 < Dv <= 256, "attention(generic): key size a multiple of 4, sizes up to 256")
    page = _check_pools_kv(k_pool, v_pool, G, D, Dv, q.dtype, "attention")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "attention: block_tables must be contiguous int32 [S, W]")
    _ints(seq_of_token, T, "seq_of_token")
    _ints(positions, T, "positions")
    _need(window >= 0 and softcap >= 0, "attention: window and softcap must be >= 0 (0 = none)")
    ldg = 0
    if gate is not None:
        _need(gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == T and gate.shape[1] >= H and gate.stride(1) == 1,
              f"attention: gate is float32 [T, >= {H}]")
        ldg = gate.stride(0) if T > 1 else max(gate.stride(0), H)
    q_stride = q.stride(0) if T > 1 else max(q.stride(0), H * D)
    _check(library().tm_attn_paged_generic_ext(_p(q), c_int(q_stride), _p(out), c_int(H * Dv), _p(k_pool), _p(v_pool), _p(block_tables),
                                               c_int(block_tables.shape[1]), _p(seq_of_token), _p(positions), c_int(T), c_int(H),
                                               c_int(G), c_int(D), c_int(Dv), c_int(page), c_float(scale), c_int(window),
                                               c_float(softcap), _p(gate), c_int(ldg), code(q.dtype), _stream()), "attn_paged_generic_ext")
    return out


# -------------------------------------------------------------------------------------------- experts by router

def moe_router(z: torch.Tensor, experts: int, top: int, correction: torch.Tensor | None = None, over_chosen: bool = False):
    """z: float32 view [T, >= experts] (the router's outputs). s = softmax over the first ``experts`` columns; the ``top``
    largest of s + correction are chosen (descending; of equals the lower index). Returns (chosen int32 [T, top], weight
    float32 [T, top] = the chosen experts' s divided by their sum + 1e-20). ``over_chosen``: the ``top`` largest z themselves are
    chosen and the weights are the softmax over the chosen z only (no correction)."""
    _gpu(z, correction)
    T = z.shape[0]
    _need(z.dtype == torch.float32 and z.dim() == 2 and z.stride(1) == 1 and z.shape[1] >= experts, f"moe_router: z is float32 [T, >= {experts}]")
    _need(0 < top <= experts <= MOE_MAX_EXPERTS, f"moe_router: {top} of {experts} experts (up to {MOE_MAX_EXPERTS})")
    _need(not (over_chosen and correction is not None), "moe_router: a correction shifts a choice among softmax scores only")
    if correction is not None:
        _need(correction.dtype == torch.float32 and tuple(correction.shape) == (experts,) and correction.is_contiguous(),
              f"moe_router: correction is float32 [{experts}]")
    chosen = torch.empty((T, top), dtype=torch.int32, device=z.device)
    weight = torch.empty((T, top), dtype=torch.float32, device=z.device)
    ldz = z.stride(0) if T > 1 else max(z.stride(0), experts)
    _check(library().tm_moe_router(_p(z), c_int(ldz), _p(correction), c_int(T), c_int(experts), c_int(top), _p(chosen), _p(weight),
                                   c_int(1 if over_chosen else 0), _stream()), "moe_router")
    return chosen, weight


def moe_route_chosen(chosen: torch.Tensor, experts: int, real: int, tile_rows: int = MOE_TILE_ROWS):
    """As ``moe_route`` for pairs whose experts a router chose (``chosen`` int32 [T, top]); experts ``real`` .. experts - 1
    have no matrices, and a pair that names one gets no slot (pair_slot = -1)."""
    _gpu(chosen)
    _need(chosen.dtype == torch.int32 and chosen.dim() == 2 and chosen.is_contiguous(), "moe_route_chosen: chosen is contiguous int32 [T, top]")
    T, top = chosen.shape
    _need(0 <= real <= experts <= MOE_MAX_EXPERTS and experts > 0, f"moe_route_chosen: up to {MOE_MAX_EXPERTS} experts")
    _need(tile_rows in (32, 64, 128), "moe_route_chosen: tiles of 32, 64 or 128 rows")
    P = T * top
    most = moe_max_tiles(P, max(real, 1), tile_rows)
    work = torch.empty(2 * P + 3 * most + 1, dtype=torch.int32, device=chosen.device)
    slot_pair, pair_slot, tiles, n_tiles = work[:P], work[P:2 * P], work[2 * P:2 * P + 3 * most].view(most, 3), work[2 * P + 3 * most:]
    _check(library().tm_moe_route_chosen(None, _p(chosen), c_int(T), c_int(top), c_int(experts), c_int(real), c_int(tile_rows),
                                         _p(slot_pair), _p(pair_slot), _p(tiles), _p(n_tiles), _stream()), "moe_route_chosen")
    return slot_pair, pair_slot, tiles, n_tiles, tile_rows


def moe_experts_weighted(x: torch.Tensor, routed, weight: torch.Tensor, w_up: torch.Tensor | None, w_down: torch.Tensor | None, top: int,
                         out: torch.Tensor, shared: torch.Tensor | None = None, shared_gate: torch.Tensor | None = None,
                         gated: bool = False) -> torch.Tensor:
    """out[t] = sum over the token's ``top`` pairs of weight[t, k] * (Wd[e] relu(Wu[e] x[t])^2, or x[t] itself for a pair
    without a slot) + sigmoid(shared_gate[t]) * shared[t]. w_up [E, F, K], w_down [E, N, F] (both None: every expert stands
    for the input); ``routed`` from ``moe_route_chosen``; shared float32 [T, N] or None; shared_gate a float32 view [T, >= 1].
    ``gated``: an expert is Wd[e] (silu(Wg[e] x) * (Wu[e] x)) and w_up is [E, 2F, K], an expert's gate rows, then its up rows."""
    slot_pair, pair_slot, tiles, n_tiles, tile_rows = routed
    _gpu(x, w_up, w_down, out, weight, shared, shared_gate)
    T, K = x.shape
    P = T * top
    N = out.shape[1]
    _need(x.stride(1) == 1 and N == K and tuple(out.shape) == (T, N) and out.is_contiguous() and x.dtype == out.dtype,
          "moe_experts_weighted: x [T, K], out contiguous [T, K], one type")
    _need(weight.dtype == torch.float32 and tuple(weight.shape) == (T, top) and weight.is_contiguous(), "moe_experts_weighted: weight is float32 [T, top]")
    _need(slot_pair.numel() == P and pair_slot.numel() == P, "moe_experts_weighted: the routing belongs to another step")
    if shared is not None:
        _need(shared.dtype == torch.float32 and tuple(shared.shape) == (T, N) and shared.is_contiguous(), "moe_experts_weighted: shared is float32 [T, N]")
    ldg = 0
    if shared_gate is not None:
        _need(shared is not None and shared_gate.dtype == torch.float32 and shared_gate.dim() == 2 and shared_gate.shape[0] == T
              and shared_gate.stride(1) == 1, "moe_experts_weighted: shared_gate is a float32 view [T, >= 1] beside a shared result")
        ldg = shared_gate.stride(0) if T > 1 else max(shared_gate.stride(0), 1)
    lib, dt = library(), c_int(code(x.dtype))
    ldx = x.stride(0) if T > 1 else max(x.stride(0), K)
    most = tiles.shape[0]
    part = torch.empty((max(P, 1), N), dtype=torch.float32, device=x.device)
    if w_up is not None and most > 0:
        E, F, K2 = w_up.shape
        if gated:
            _need(F % 2 == 0, "moe_experts_weighted: gate rows and up rows come in equal numbers")
            F //= 2
        _need(K2 == K and tuple(w_down.shape) == (E, N, F) and w_up.is_contiguous() and w_down.is_contiguous()
              and x.dtype == w_up.dtype == w_down.dtype, "moe_experts_weighted: w_up [E, F, K], w_down [E, N, F], one type")
        act = torch.empty((P, F), dtype=x.dtype, device=x.device)
        if x.dtype == torch.bfloat16 and lib.tm_moe_mfma_takes(_p(x), c_int(ldx), _p(w_up), _p(w_down), _p(act), c_int(K), c_int(F)):
            first = lib.tm_moe_gate_up_mfma if gated else lib.tm_moe_up_act_mfma
            _check(first(_p(x), c_int(ldx), _p(slot_pair), c_int(top), _p(w_up), _p(act), _p(tiles), _p(n_tiles),
                         c_int(most), c_int(tile_rows), c_int(K), c_int(F), _stream()), "moe_up_act_mfma")
            _check(lib.tm_moe_down_mfma(_p(act), _p(w_down), _p(part), _p(tiles), _p(n_tiles), c_int(most), c_int(tile_rows), c_int(F),
                                        c_int(N), _stream()), "moe_down_mfma")
        else:
            _need(tile_rows == MOE_TILE_ROWS, "moe_experts_weighted: these products take tiles of 32 rows")
            first = lib.tm_moe_gate_up if gated else lib.tm_moe_up_act
            _check(first(_p(x), c_int(ldx), _p(slot_pair), c_int(top), _p(w_up), _p(act), _p(tiles), _p(n_tiles), c_int(most),
                         c_int(K), c_int(F), dt, _stream()), "moe_up_act")
            _check(lib.tm_moe_down(_p(act), _p(w_down), _p(part), _p(tiles), _p(n_tiles), c_int(most), c_int(F), c_int(N), dt, _stream()),
                   "moe_down")
    _check(lib.tm_moe_combine_weighted(_p(part), _p(pair_slot), _p(weight), _p(x), c_int(ldx), _p(shared), _p(shared_gate), c_int(ldg),
                                       _p(out), c_int(T), c_int(top), c_int(N), dt, _stream()), "moe_combine_weighted")
    return out


# -------------------------------------------------------------------------------------------- the gated delta rule

DELTA_MAX_KEY_DIM = 256
DELTA_MAX_CHANNELS = 1 << 22        # convolved channels of a token (q | k | v)


def delta_row_width(H: int, G: int, D: int, Dv: int) -> int:
    """Floats of a prepared row [q | k | v | beta | g | k.q], rounded up to whole 16-byte pieces."""
    return -(-(2 * G * D + H * Dv + 2 * H + G) // 4) * 4


def delta_prepare(proj: torch.Tensor, conv_w: torch.Tensor, conv_state: torch.Tensor | None, ba: torch.Tensor, a_log: torch.Tensor,
                  dt_bias: torch.Tensor, cu_q_lens: torch.Tensor, state_slots: torch.Tensor, seq_of_token: torch.Tensor, num_seqs: int,
                  out: torch.Tensor, H: int, G: int, D: int, Dv: int, unit_eps: float = 1e-6) -> torch.Tensor:
    """The rows the delta-rule recurrence reads, from the projections of a step. proj [T, >= C] (C = 2 G D + H Dv: the q, k and v
    channels first) in the model's type; conv_w [C, taps] and conv_state [slots, taps - 1, C] of the same type (the rows before a
    request's first row of the step come from its state; the state itself is advanced by ``delta_conv_state``); ba float32
    [T, >= 2H] = [b | a]; a_log, dt_bias float32 [H]. Per token: y = silu(conv(.)), q = y_q / sqrt(sum y_q^2 + eps) / sqrt(D),
    k = y_k / sqrt(sum y_k^2 + eps), beta = sigmoid(b), g = exp(-exp(a_log) softplus(a + dt_bias)); out float32
    [T, delta_row_width] = [q | k | v | beta | g | k.q]."""
    _gpu(proj, conv_w, conv_state, ba, a_log, dt_bias, cu_q_lens, state_slots, seq_of_token, out)
    T = proj.shape[0]
    C = 2 * G * D + H * Dv
    taps = conv_w.shape[1]
    _need(proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= C, f"delta_prepare: proj is [T, >= {C}]")
    _need(H % G == 0 and 0 < D <= DELTA_MAX_KEY_DIM and C <= DELTA_MAX_CHANNELS, "delta_prepare: sizes the kernels do not take")
    _need(tuple(conv_w.shape) == (C, taps) and conv_w.is_contiguous() and conv_w.dtype == proj.dtype and 1 <= taps <= 16,
          f"delta_prepare: conv_w is [{C}, taps] of proj's type, taps up to 16")
    if taps > 1:
        _need(conv_state is not None and conv_state.dim() == 3 and tuple(conv_state.shape[1:]) == (taps - 1, C)
              and conv_state.is_contiguous() and conv_state.dtype == proj.dtype, f"delta_prepare: conv_state is [slots, {taps - 1}, {C}] of proj's type")
    _need(ba.dtype == torch.float32 and ba.dim() == 2 and ba.shape[0] == T and ba.shape[1] >= 2 * H and ba.stride(1) == 1,
          f"delta_prepare: ba is float32 [T, >= {2 * H}]")
    for name, v in (("a_log", a_log), ("dt_bias", dt_bias)):
        _need(v.dtype == torch.float32 and tuple(v.shape) == (H,) and v.is_contiguous(), f"delta_prepare: {name} is float32 [{H}]")
    ldo = out.shape[1] if out.dim() == 2 else 0
    _need(out.dtype == torch.float32 and out.dim() == 2 and out.shape[0] == T and out.is_contiguous() and ldo >= C + 2 * H + G,
          "delta_prepare: out is contiguous float32 [T, >= C + 2H + G]")
    _ints(cu_q_lens, num_seqs + 1, "cu_q_lens")
    _ints(state_slots, num_seqs, "state_slots")
    _ints(seq_of_token, T, "seq_of_token")
    ld = proj.stride(0) if T > 1 else max(proj.stride(0), proj.shape[1])
    ldba = ba.stride(0) if T > 1 else max(ba.stride(0), ba.shape[1])
    _check(library().tm_delta_prepare(_p(proj), c_int(ld), _p(conv_w), _p(conv_state), _p(ba), c_int(ldba), _p(a_log), _p(dt_bias),
                                      _p(cu_q_lens), _p(state_slots), _p(seq_of_token), _p(out), c_int(ldo), c_int(T), c_int(H), c_int(G),
                                      c_int(D), c_int(Dv), c_int(taps), c_float(unit_eps), c_int(code(proj.dtype)), _stream()),
           "delta_prepare")
    return out


def delta_conv_state(proj: torch.Tensor, C: int, conv_state: torch.Tensor, cu_q_lens: torch.Tensor, state_slots: torch.Tensor,
                     num_seqs: int) -> None:
    """Every request's convolution state [taps - 1, C] becomes the last taps - 1 rows it has seen (the first C columns of proj)."""
    _gpu(proj, conv_state, cu_q_lens, state_slots)
    T = proj.shape[0]
    _need(conv_state.dim() == 3 and conv_state.shape[2] == C and conv_state.is_contiguous() and conv_state.dtype == proj.dtype,
          f"delta_conv_state: the state is [slots, taps - 1, {C}] of proj's type")
    _need(proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= C, f"delta_conv_state: proj is [T, >= {C}]")
    _ints(cu_q_lens, num_seqs + 1, "cu_q_lens")
    _ints(state_slots, num_seqs, "state_slots")
    ld = proj.stride(0) if T > 1 else max(proj.stride(0), proj.shape[1])
    _check(library().tm_delta_conv_state(_p(proj), c_int(ld), _p(conv_state), _p(cu_q_lens), _p(state_slots), c_int(num_seqs), c_int(C),
                                         c_int(conv_state.shape[1] + 1), c_int(code(proj.dtype)), _stream()), "delta_conv_state")


def delta_scan(rows: torch.Tensor, o: torch.Tensor | None, state: torch.Tensor, cu_q_lens: torch.Tensor, state_slots: torch.Tensor,
               num_seqs: int, H: int, G: int, D: int, Dv: int, transitions_of: int | None = None) -> torch.Tensor | None:
    """The recurrence over the rows of ``delta_prepare``, request by request in the order of the step's rows:
    S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q. state float32 [slots, H, D, Dv] (row state_slots[s] is read and
    written); o float32 [T, H * Dv], or None where only the states are wanted. ``transitions_of`` = the rows' value size: the
    values count as zero and the state has ``Dv`` columns of its own (from the identity, Dv = D, a run of tokens leaves the
    product of its transitions g (I - beta k k^T))."""
    _gpu(rows, o, state, cu_q_lens, state_slots)
    T = rows.shape[0]
    row_dv = Dv if transitions_of is None else transitions_of
    _need(rows.dtype == torch.float32 and rows.dim() == 2 and rows.is_contiguous() and rows.shape[1] >= 2 * G * D + H * row_dv + 2 * H + G,
          "delta_scan: rows are those of delta_prepare")
    if o is not None:
        _need(transitions_of is None, "delta_scan: a scan without values has no results")
        _need(o.dtype == torch.float32 and o.is_contiguous() and tuple(o.shape) == (T, H * Dv), f"delta_scan: o is float32 [{T}, {H * Dv}]")
    _need(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, D, Dv),
          f"delta_scan: state is float32 [slots, {H}, {D}, {Dv}]")
    _need(H % G == 0 and 0 < D <= DELTA_MAX_KEY_DIM, "delta_scan: sizes the kernel does not take")
    _ints(cu_q_lens, num_seqs + 1, "cu_q_lens")
    _ints(state_slots, num_seqs, "state_slots")
    _check(library().tm_delta_scan(_p(rows), c_int(rows.shape[1]), _p(o), _p(state), _p(cu_q_lens), _p(state_slots), c_int(num_seqs),
                                   c_int(H), c_int(G), c_int(D), c_int(Dv), c_int(row_dv), c_int(0 if transitions_of is not None else 1),
                                   _stream()), "delta_scan")
    return o


def delta_combine(trans: torch.Tensor, local: torch.Tensor, start: torch.Tensor, state: torch.Tensor, state_slots: torch.Tensor,
                  first_seg: torch.Tensor, num_seqs: int) -> None:
    """Chains the segments of every request: start[j] = S, S <- trans[j] S + local[j] for its segments j = first_seg[s] ..
    first_seg[s + 1] - 1 in order, from S = state[state_slots[s]], which becomes the last S. trans float32 [n, H, D, D], local and
    start [n, H, D, Dv], state [slots, H, D, Dv]."""
    _gpu(trans, local, start, state, state_slots, first_seg)
    n, H, D, Dv = local.shape
    for name, t, shape in (("trans", trans, (n, H, D, D)), ("local", local, (n, H, D, Dv)), ("start", start, (n, H, D, Dv))):
        _need(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == shape, f"delta_combine: {name} is float32 {list(shape)}")
    _need(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, D, Dv),
          f"delta_combine: state is float32 [slots, {H}, {D}, {Dv}]")
    _need(0 < D <= DELTA_MAX_KEY_DIM, "delta_combine: sizes the kernel does not take")
    _ints(state_slots, num_seqs, "state_slots")
    _ints(first_seg, num_seqs + 1, "first_seg")
    _check(library().tm_delta_combine(_p(trans), _p(local), _p(start), _p(state), _p(state_slots), _p(first_seg), c_int(num_seqs), c_int(H),
                                      c_int(D), c_int(Dv), _stream()), "delta_combine")


def pair_norm_mean(a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, out: torch.Tensor, eps: float) -> torch.Tensor:
    """out = (a / rms(a) * wa + b / rms(b) * wb) / 2 row by row, statistics and sums in 32-bit; a, b, out [T, W] of one type,
    wa, wb float32 [W]."""
    _gpu(a, b, wa, wb, out)
    T, W = a.shape
    _need(a.is_contiguous() and b.is_contiguous() and out.is_contiguous() and a.shape == b.shape == out.shape
          and a.dtype == b.dtype == out.dtype, "pair_norm_mean: a, b and out are contiguous, of one shape and type")
    for w in (wa, wb):
        _need(w.dtype == torch.float32 and tuple(w.shape) == (W,) and w.is_contiguous(), f"pair_norm_mean: the weights are float32 [{W}]")
    _need(eps > 0, "pair_norm_mean: eps must be positive")
    _check(library().tm_pair_norm_mean(_p(a), _p(b), _p(wa), _p(wb), _p(out), c_int(T), c_int(W), c_float(eps), c_int(code(a.dtype)),
                                       _stream()), "pair_norm_mean")
    return out
