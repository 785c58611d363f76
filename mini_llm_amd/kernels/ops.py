"""The engine's device operations: thin, checked wrappers over the HIP kernels.

Every op takes torch tensors that live on the GPU, checks on the host that shapes,
strides and dtypes match what the kernel and its grid assume, and launches on the
current HIP stream (so the calls can be captured in a HIP graph). There is no CPU
path: a tensor that is not on the GPU, or a kernel library that cannot be built and
loaded, raises.

Parts look ops up as ``ops.<name>`` at call time.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from ..build import load_library

EPILOGUES = {"store": 0, "gelu_tanh": 1, "gelu_erf": 2, "add_residual": 3, "store_f32": 4}
_DT = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


def _dt(t: torch.Tensor) -> int:
    if t.dtype not in _DT:
        raise KernelError(f"unsupported dtype {t.dtype} (float32 or bfloat16)")
    return _DT[t.dtype]


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError(
                "tensor is not on the GPU: the engine has no CPU path "
                f"(device={t.device}, shape={tuple(t.shape)})")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> ctypes.c_void_p:
    """The current HIP stream of the current device (the raw handle: building a Stream object
    for every launch costs more than many of the launches)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _check(rc: int, what: str) -> None:
    if rc == 0:
        return
    if rc < 0:
        raise KernelError(f"{what}: the kernel refuses these sizes (code {rc})")
    raise KernelError(f"{what}: HIP error {rc} at launch")


def _rows2d(t: torch.Tensor, name: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{name} must be 2-D with a contiguous last dimension, got shape "
                          f"{tuple(t.shape)} strides {t.stride()}")


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{name} must be a contiguous int32 tensor")
    if n is not None and t.numel() < n:
        raise KernelError(f"{name} has {t.numel()} entries, {n} needed")


# ---------------------------------------------------------------------------------

def embed(ids: torch.Tensor, positions: Optional[torch.Tensor], wte: torch.Tensor,
          wpe: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    """out[t,:] = wte[ids[t],:] + wpe[positions[t],:] in fp32. ids/positions must be in range
    (the caller checks them on the host)."""
    _gpu(ids, positions, wte, wpe, out)
    T = ids.numel()
    _rows2d(wte, "wte")
    D = wte.shape[1]
    _i32(ids, "ids")
    if not wte.is_contiguous():
        raise KernelError("wte must be contiguous")
    if wpe is not None:
        if positions is None:
            raise KernelError("positions are needed with a position table")
        _i32(positions, "positions", T)
        if wpe.dtype != wte.dtype or wpe.dim() != 2 or wpe.shape[1] != D or not wpe.is_contiguous():
            raise KernelError("wpe must be contiguous [P, D] in wte's dtype")
    if out.dtype != torch.float32 or out.shape != (T, D) or not out.is_contiguous():
        raise KernelError(f"out must be contiguous fp32 [{T}, {D}]")
    lib = load_library("elementwise")
    _check(lib.mllm_embed(_p(ids), _p(positions if wpe is not None else None), _p(wte), _p(wpe), _p(out),
                          T, D, _dt(wte), _stream()), "embed")
    return out


def select_tokens(ids: torch.Tensor, src: torch.Tensor, prev: torch.Tensor) -> torch.Tensor:
    """ids[i] = prev[src[i]] where src[i] >= 0, in place: token ids that an earlier step sampled
    on the device and the host has not read yet."""
    _gpu(ids, src, prev)
    n = ids.numel()
    _i32(ids, "ids")
    _i32(src, "src", n)
    _i32(prev, "prev")
    lib = load_library("elementwise")
    _check(lib.mllm_select_tokens(_p(ids), _p(src), _p(prev), n, prev.numel(), _stream()), "select_tokens")
    return ids


def reset_state(state: torch.Tensor, slots: torch.Tensor, starts: torch.Tensor) -> None:
    """Clears row ``slots[b]`` of ``state`` ([n_slots, ...]) for every b with ``starts[b] == 0`` and
    ``slots[b] >= 0``: the fixed-size state of requests that begin in this step."""
    _gpu(state, slots, starts)
    B = slots.numel()
    _i32(slots, "slots")
    _i32(starts, "starts", B)
    if not state.is_contiguous() or state.dim() < 1:
        raise KernelError("state must be contiguous [n_slots, ...]")
    slot_bytes = (state.numel() // max(state.shape[0], 1)) * state.element_size()
    lib = load_library("elementwise")
    rc = lib.mllm_reset_state(_p(state), ctypes.c_size_t(slot_bytes), state.shape[0], _p(slots), _p(starts), B,
                              _stream())
    if rc == -1:
        raise KernelError(f"reset_state: a slot of {slot_bytes} bytes is no multiple of 4 bytes")
    _check(rc, "reset_state")


def layernorm(x: torch.Tensor, gamma: torch.Tensor, beta: Optional[torch.Tensor], eps: float,
              out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[i,:] = LayerNorm(x[rows[i] if rows else i,:]); statistics in fp32."""
    _gpu(x, gamma, beta, out, rows)
    if x.dtype != torch.float32 or x.dim() != 2 or not x.is_contiguous():
        raise KernelError("layernorm input must be contiguous fp32 [rows, D]")
    D = x.shape[1]
    n = rows.numel() if rows is not None else x.shape[0]
    if rows is not None:
        _i32(rows, "rows")
    if gamma.dtype != torch.float32 or gamma.numel() != D or not gamma.is_contiguous():
        raise KernelError(f"gamma must be fp32 [{D}]")
    if beta is not None and (beta.dtype != torch.float32 or beta.numel() != D or not beta.is_contiguous()):
        raise KernelError(f"beta must be fp32 [{D}]")
    if out.shape != (n, D) or not out.is_contiguous():
        raise KernelError(f"out must be contiguous [{n}, {D}]")
    lib = load_library("elementwise")
    _check(lib.mllm_layernorm(_p(x), _p(rows), _p(gamma), _p(beta), _p(out), n, D, ctypes.c_float(eps),
                              _dt(out), _stream()), "layernorm")
    return out


def _scatter_is_fused(dtype: torch.dtype, rows: int) -> bool:
    """Whether the product kernel that runs for these rows writes a fused QKV product's keys and
    values to the pages in its epilogue: the many-row bf16 kernel does."""
    return dtype == torch.bfloat16 and rows > 64


class AttentionSplits:
    """The output of decode attention that has not been merged yet: every (token, head) pair's keys
    were split over ``nsplit`` workgroups, whose states (running maximum, sum, unnormalised output)
    lie in the attention scratch. ``linear`` takes it in place of a tensor and merges while it loads
    (``tensor()`` merges into an ordinary activation). Valid until the next attention launch."""

    def __init__(self, ws: torch.Tensor, n_tokens: int, n_heads: int, head_dim: int, nsplit: int, dtype):
        self.ws, self.n_tokens, self.n_heads, self.head_dim, self.nsplit = ws, n_tokens, n_heads, head_dim, nsplit
        self.dtype, self.device = dtype, ws.device
        self.shape = (n_tokens, n_heads * head_dim)

    def tensor(self, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if out is None:
            out = torch.empty(self.shape, dtype=self.dtype, device=self.device)
        lib = load_library("attention_decode")
        _check(lib.mllm_merge_attention_splits(_p(self.ws), self.n_tokens, self.n_heads, self.head_dim, self.nsplit,
                                               _p(out), out.stride(0), _DT[self.dtype], _stream()), "merge_splits")
        return out


MERGE_MAX_ROWS = 16        # tokens whose attention splits a product merges while loading (one row block)
MERGE_MAX_SPLITS = 4       # and the most splits per (token, head) pair it takes


def _linear_from_splits(a: AttentionSplits, w, bias, out, epilogue: str) -> Optional[torch.Tensor]:
    """The product fed by unmerged attention splits, or None if its kernel does not take these sizes."""
    M, K = a.shape
    N = w.shape[0]
    lib = load_library("gemm_bf16")
    ml = a.ws[M * a.n_heads * a.nsplit * a.head_dim:]
    rc = lib.mllm_gemm_bf16_merged(_p(a.ws), _p(ml), a.nsplit, a.n_heads, a.head_dim, _p(w), w.stride(0), _p(bias),
                                   _p(out), out.stride(0), M, N, EPILOGUES[epilogue], _stream())
    if rc == -2:
        return None
    _check(rc, "linear (merging attention splits)")
    return out


def linear(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           epilogue: str = "store", kv_scatter: Optional[tuple] = None) -> torch.Tensor:
    """out = epilogue(a @ w.T + bias). a: [M,K] (or the unmerged ``AttentionSplits`` of decode attention),
    w: [N,K] (same dtype), bias: fp32 [N].

    epilogue: "store" | "gelu_tanh" | "gelu_erf" (out in a's dtype), "add_residual"
    (out fp32, accumulated in place), "store_f32" (out fp32).

    ``kv_scatter=(slots, k_pages, v_pages, q_cols)`` (only with "store"): the columns after the
    first q_cols are keys, then values, of kv_dim = k_pages.shape[1] columns each, and row m's also
    go to row slots[m] (>= 0) of the pages: in the product's epilogue where the kernel that runs
    for these sizes has one, otherwise by a copy kernel after it.
    """
    splits = a if isinstance(a, AttentionSplits) else None
    _gpu(None if splits else a, w, bias, out)
    if splits is None:
        _rows2d(a, "a")
    _rows2d(w, "w")
    _rows2d(out, "out")
    M, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or w.dtype != a.dtype:
        raise KernelError(f"linear: a is {tuple(a.shape)} {a.dtype}, w is {tuple(w.shape)} {w.dtype}")
    if epilogue not in EPILOGUES:
        raise KernelError(f"unknown epilogue '{epilogue}'")
    if splits is not None:
        want = torch.float32 if epilogue in ("add_residual", "store_f32") else a.dtype
        ok = (kv_scatter is None and a.dtype == torch.bfloat16 and out.shape == (M, N) and out.dtype == want
              and (bias is None or (bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous()))
              and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0)
        if ok and _linear_from_splits(a, w, bias, out, epilogue) is not None:
            return out
        a = splits.tensor()
    want = torch.float32 if epilogue in ("add_residual", "store_f32") else a.dtype
    if out.shape != (M, N) or out.dtype != want:
        raise KernelError(f"linear({epilogue}): out must be [{M}, {N}] {want}, got {tuple(out.shape)} {out.dtype}")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N or not bias.is_contiguous()):
        raise KernelError(f"bias must be contiguous fp32 [{N}]")
    mode = EPILOGUES[epilogue]
    if kv_scatter is not None:
        if epilogue != "store":
            raise KernelError("linear: the key/value scatter needs the plain store")
        if not _scatter_is_fused(a.dtype, M):
            slots, k_pages, v_pages, q_cols = kv_scatter
            kv_dim = k_pages.shape[1]
            if N != q_cols + 2 * kv_dim:
                raise KernelError(f"linear: {N} columns are not {q_cols} + 2 x {kv_dim}")
            linear(a, w, bias, out, epilogue)
            kv_append(out, q_cols, q_cols + kv_dim, kv_dim, k_pages, v_pages, slots)
            return out
    if a.dtype == torch.float32:
        lib = load_library("gemm_f32")
        rc = lib.mllm_gemm_f32(_p(a), a.stride(0), _p(w), w.stride(0), _p(bias), _p(out), out.stride(0),
                               M, N, K, mode, _stream())
    elif a.dtype == torch.bfloat16:
        lib = load_library("gemm_bf16")
        if kv_scatter is not None:
            slots, k_pages, v_pages, q_cols = kv_scatter
            _gpu(slots, k_pages, v_pages)
            kv_dim = k_pages.shape[1]
            _i32(slots, "slots", M)
            for name, pg in (("k_pages", k_pages), ("v_pages", v_pages)):
                if pg.dim() != 2 or pg.shape[1] != kv_dim or not pg.is_contiguous() or pg.dtype != a.dtype:
                    raise KernelError(f"{name} must be contiguous [rows, {kv_dim}] {a.dtype}")
            if q_cols % 4 or kv_dim % 4 or N != q_cols + 2 * kv_dim:
                raise KernelError(f"linear: {N} columns are not {q_cols} + 2 x {kv_dim} (multiples of 4)")
            rc = lib.mllm_gemm_bf16_kv(_p(a), a.stride(0), _p(w), w.stride(0), _p(bias), _p(out), out.stride(0),
                                       M, N, K, _p(slots), _p(k_pages), _p(v_pages), int(q_cols), int(kv_dim),
                                       _stream())
        else:
            ws = _gemm_workspace(a.device) if M <= 256 else None
            rc = lib.mllm_gemm_bf16(_p(a), a.stride(0), _p(w), w.stride(0), _p(bias), _p(out), out.stride(0),
                                    M, N, K, mode, _p(ws), ctypes.c_size_t(GEMM_WORKSPACE_BYTES if M <= 256 else 0),
                                    _stream())
        if rc == -1:
            raise KernelError(
                f"linear(bf16): K={K} and the row strides ({a.stride(0)}, {w.stride(0)}) must be multiples "
                "of 8 elements and the operands 16-byte aligned")
    else:
        raise KernelError(f"linear: unsupported dtype {a.dtype}")
    _check(rc, "linear")
    return out


GEMM_WORKSPACE_BYTES = 16 * 1024 + 256 * 1024     # counters, then 1 KB per workgroup of a shared-tile launch
_GEMM_WS = {}


def _gemm_workspace(device) -> torch.Tensor:
    """Scratch of the few-row products that share a tile among workgroups: zeroed once per device
    (the kernel leaves its counters at zero); launches on one stream use it one after the other."""
    ws = _GEMM_WS.get(device)
    if ws is None:
        ws = _GEMM_WS[device] = torch.zeros(GEMM_WORKSPACE_BYTES // 4, dtype=torch.int32, device=device)
    return ws


LN_FUSE_MAX_ROWS = 32      # above this many rows the norm is faster as a kernel of its own (measured: 1-2 % of a
                           # decode step gained at 24 and 32 rows, 3 % lost at 64)


def ln_linear(x: torch.Tensor, gamma: torch.Tensor, beta: Optional[torch.Tensor], eps: float,
              w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, epilogue: str = "store",
              rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = epilogue(LayerNorm(x) @ w.T + bias) with x the fp32 stream [*,K] and w [N,K]; with
    ``rows`` (int32 [M]) row m of the input is x[rows[m]].

    For bfloat16 weights, at most 32 rows and fewer than 16384 columns the norm is fused into the
    product (one kernel);
    otherwise the norm and the product run one after the other. Same numerics either way:
    statistics in fp32, the normalised rows rounded to w's dtype before the product.
    """
    _gpu(x, gamma, beta, w, bias, out, rows)
    K = x.shape[1]
    M = x.shape[0] if rows is None else rows.numel()
    N = w.shape[0]
    if rows is not None:
        _i32(rows, "rows")
    if (w.dtype == torch.bfloat16 and M <= LN_FUSE_MAX_ROWS and x.dtype == torch.float32 and x.is_contiguous()
            and gamma.data_ptr() % 16 == 0 and (beta is None or beta.data_ptr() % 16 == 0)):
        _rows2d(w, "w")
        _rows2d(out, "out")
        if w.shape[1] != K or gamma.numel() != K or gamma.dtype != torch.float32:
            raise KernelError(f"ln_linear: x is {tuple(x.shape)}, w is {tuple(w.shape)}, gamma {tuple(gamma.shape)}")
        if beta is not None and (beta.numel() != K or beta.dtype != torch.float32):
            raise KernelError("ln_linear: beta must be fp32 [K]")
        if epilogue not in EPILOGUES:
            raise KernelError(f"unknown epilogue '{epilogue}'")
        want = torch.float32 if epilogue in ("add_residual", "store_f32") else w.dtype
        if out.shape != (M, N) or out.dtype != want:
            raise KernelError(f"ln_linear({epilogue}): out must be [{M}, {N}] {want}")
        if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N or not bias.is_contiguous()):
            raise KernelError(f"bias must be contiguous fp32 [{N}]")
        lib = load_library("gemm_bf16")
        rc = lib.mllm_ln_gemm_bf16(_p(x), x.stride(0), _p(rows), _p(gamma), _p(beta), ctypes.c_float(eps), _p(w),
                                   w.stride(0), _p(bias), _p(out), out.stride(0), M, N, K, EPILOGUES[epilogue],
                                   _stream())
        if rc == 0:
            return out
        if rc != -2:
            _check(rc, "ln_linear")
    h = torch.empty((M, K), dtype=w.dtype, device=x.device)
    layernorm(x, gamma, beta, eps, h, rows)
    return linear(h, w, bias, out, epilogue)


def kv_append(src: torch.Tensor, k_col: int, v_col: int, kv_dim: int, k_pages: torch.Tensor,
              v_pages: torch.Tensor, slots: torch.Tensor) -> None:
    """Copies columns [k_col, k_col+kv_dim) and [v_col, v_col+kv_dim) of each row of ``src``
    into row ``slots[t]`` of the key and value pages (slot < 0: skipped)."""
    _gpu(src, k_pages, v_pages, slots)
    _rows2d(src, "src")
    T = src.shape[0]
    _i32(slots, "slots", T)
    for name, pg in (("k_pages", k_pages), ("v_pages", v_pages)):
        if pg.dim() != 2 or pg.shape[1] != kv_dim or not pg.is_contiguous() or pg.dtype != src.dtype:
            raise KernelError(f"{name} must be contiguous [rows, {kv_dim}] {src.dtype}")
    if max(k_col, v_col) + kv_dim > src.shape[1] or min(k_col, v_col) < 0:
        raise KernelError("key/value columns lie outside the source rows")
    lib = load_library("elementwise")
    _check(lib.mllm_kv_append(_p(src), src.stride(0), k_col, v_col, _p(k_pages), _p(v_pages), kv_dim,
                              _p(slots), T, _dt(src), _stream()), "kv_append")


def paged_attention(q: torch.Tensor, q_col: int, n_heads: int, n_kv_heads: int, head_dim: int,
                    k_pages: torch.Tensor, v_pages: torch.Tensor, page_size: int,
                    block_tables: torch.Tensor, token_seq: torch.Tensor, positions: torch.Tensor,
                    scale: float, window: int, out: torch.Tensor, *, cu_q: Optional[torch.Tensor] = None,
                    ctx_len: Optional[torch.Tensor] = None, max_q_len: int = 0, max_ctx_len: int = 0,
                    append: Optional[tuple] = None, n_single: int = 0, may_split: bool = False):
    """Causal attention of the step's queries over the pages.

    q: [T, >= q_col + n_heads*head_dim] (queries of token t start at column q_col);
    block_tables: int32 [B, max_blocks]; token_seq[t]: row of block_tables; positions[t]:
    position of token t in its sequence. A query at position p sees keys
    [max(0, p-window+1) if window else 0, p]. out: [T, n_heads*head_dim].

    ``append=(k_col, v_col, slots)``: the step's own keys and values are still in q's rows
    (columns k_col, v_col) and this op writes them to row ``slots[t]`` of the pages first
    (fused into the decode kernel where that runs); without it they are in the pages already.

    ``n_single``: the first n_single sequences of the batch bring one token each (decoded tokens stand
    first in a mixed step). They then go to the single-query kernel and only the portions behind them
    to the 64-query tiles of the matrix cores, where a lone query would leave 63 of 64 lanes idle.

    ``may_split``: the caller hands the result to ``linear`` next and accepts an ``AttentionSplits``
    in place of ``out`` (returned when a few single tokens' keys were split over several workgroups
    each; ``out`` is then left unwritten).
    """
    _gpu(q, k_pages, v_pages, block_tables, token_seq, positions, out)
    _rows2d(q, "q")
    _rows2d(out, "out")
    T = q.shape[0]
    kv_dim = n_kv_heads * head_dim
    if q_col < 0 or q_col + n_heads * head_dim > q.shape[1]:
        raise KernelError("query columns lie outside q's rows")
    if out.shape[0] != T or out.shape[1] != n_heads * head_dim or out.dtype != q.dtype:
        raise KernelError(f"out must be [{T}, {n_heads * head_dim}] {q.dtype}")
    for name, pg in (("k_pages", k_pages), ("v_pages", v_pages)):
        if pg.dim() != 2 or pg.shape[1] != kv_dim or not pg.is_contiguous() or pg.dtype != q.dtype:
            raise KernelError(f"{name} must be contiguous [rows, {kv_dim}] {q.dtype}")
    if k_pages.shape[0] % page_size != 0:
        raise KernelError("the page pool is not a whole number of pages")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise KernelError("block_tables must be contiguous int32 [B, max_blocks]")
    _i32(token_seq, "token_seq", T)
    _i32(positions, "positions", T)
    if head_dim % 8 != 0 or head_dim > 256:
        raise KernelError(f"head_dim={head_dim} is not supported (multiples of 8 up to 256)")
    if n_heads % n_kv_heads != 0:
        raise KernelError(f"n_heads={n_heads} is not a multiple of n_kv_heads={n_kv_heads}")
    esz = q.element_size()
    if (q.stride(0) * esz) % 16 or (q_col * esz) % 16 or (head_dim * esz) % 16 or q.data_ptr() % 16:
        raise KernelError("query rows and heads must be 16-byte aligned")
    lpk = head_dim * esz // 16
    decode = (max_q_len == 1 and lpk >= 2 and (lpk & (lpk - 1)) == 0
              and page_size & (page_size - 1) == 0 and block_tables.shape[1] <= 4096)
    k_col = v_col = 0
    slots = None
    if append is not None:
        k_col, v_col, slots = append
        if not decode:
            kv_append(q, k_col, v_col, kv_dim, k_pages, v_pages, slots)
            slots = None
        else:
            _i32(slots, "slots", T)
            if max(k_col, v_col) + kv_dim > q.shape[1] or min(k_col, v_col) < 0 or (k_col * esz) % 16 or (v_col * esz) % 16:
                raise KernelError("key/value columns lie outside q's rows or are not 16-byte aligned")
    tiles_ok = (q.dtype == torch.bfloat16 and head_dim in (32, 64, 128) and max_q_len > 1
                and cu_q is not None and ctx_len is not None
                and page_size & (page_size - 1) == 0 and page_size >= head_dim // 16
                and block_tables.shape[1] <= 2048)
    if (tiles_ok and 0 < n_single < block_tables.shape[0] and lpk >= 2 and (lpk & (lpk - 1)) == 0
            and block_tables.shape[1] <= 4096):
        # a mixed step: the leading single tokens, then the portions, two launches over disjoint rows
        # (every row's keys and values are in the pages by now)
        paged_attention(q[:n_single], q_col, n_heads, n_kv_heads, head_dim, k_pages, v_pages, page_size,
                        block_tables[:n_single], token_seq[:n_single], positions[:n_single], scale, window,
                        out[:n_single], max_q_len=1, max_ctx_len=max_ctx_len, n_single=n_single)
        B = block_tables.shape[0] - n_single
        _i32(cu_q, "cu_q", block_tables.shape[0] + 1)
        _i32(ctx_len, "ctx_len", block_tables.shape[0])
        if out.data_ptr() % 16 or (out.stride(0) * esz) % 8:
            raise KernelError("attention output rows must be 8-byte aligned")
        lib = load_library("attention_prefill")
        # (row numbers in cu_q are absolute, so q and out are passed whole and the per-sequence arrays from
        # the first portion on)
        _check(lib.mllm_prefill_attention_bf16(
            _p(q), q.stride(0), q_col, _p(k_pages), _p(v_pages), kv_dim, _p(block_tables[n_single:]),
            block_tables.shape[1], _p(cu_q[n_single:]), _p(ctx_len[n_single:]), B, (T - n_single) // 64 + B,
            n_heads, n_kv_heads, head_dim, page_size, ctypes.c_float(scale), int(window or 0), _p(out),
            out.stride(0), _stream()), "prefill_attention")
        return out
    if decode:
        # every query is a single decoded token: split its keys over workgroups
        pairs = T * n_heads
        unmerged = (may_split and q.dtype == torch.bfloat16 and T <= MERGE_MAX_ROWS and head_dim % 8 == 0
                    and DECODE_SHAPE_OVERRIDE is None)
        nsplit, waves = _decode_launch_shape(pairs, max_ctx_len, unmerged)
        unmerged = unmerged and nsplit > 1
        ws, counters = _decode_workspace(q.device, pairs, nsplit, head_dim)
        lib = load_library("attention_decode")
        # every sequence of the batch brings one token (the caller says so): token t is sequence t, and the
        # kernel need not load that
        seq_of_token = None if n_single == T == block_tables.shape[0] else token_seq
        _check(lib.mllm_decode_attention(
            _p(q), q.stride(0), q_col, _p(k_pages), _p(v_pages), kv_dim, _p(block_tables), block_tables.shape[1],
            _p(seq_of_token), _p(positions), T, n_heads, n_kv_heads, head_dim, page_size, ctypes.c_float(scale),
            int(window or 0), nsplit, waves, _p(out), out.stride(0), _p(ws), _p(counters), k_col, v_col, _p(slots),
            1 if unmerged else 0, _dt(q), _stream()),
            "decode_attention")
        if unmerged:
            return AttentionSplits(ws, T, n_heads, head_dim, nsplit, q.dtype)
        return out
    if tiles_ok:
        # prompt portions: tiles of 64 queries on the matrix cores
        B = block_tables.shape[0]
        _i32(cu_q, "cu_q", B + 1)
        _i32(ctx_len, "ctx_len", B)
        if out.data_ptr() % 16 or (out.stride(0) * esz) % 8:
            raise KernelError("attention output rows must be 8-byte aligned")
        lib = load_library("attention_prefill")
        _check(lib.mllm_prefill_attention_bf16(
            _p(q), q.stride(0), q_col, _p(k_pages), _p(v_pages), kv_dim, _p(block_tables), block_tables.shape[1],
            _p(cu_q), _p(ctx_len), B, T // 64 + B, n_heads, n_kv_heads, head_dim, page_size,
            ctypes.c_float(scale), int(window or 0), _p(out), out.stride(0), _stream()), "prefill_attention")
        return out
    lib = load_library("attention")
    _check(lib.mllm_paged_attention_generic(
        _p(q), q.stride(0), q_col, _p(k_pages), _p(v_pages), kv_dim, _p(block_tables), block_tables.shape[1],
        _p(token_seq), _p(positions), T, n_heads, n_kv_heads, head_dim, page_size, ctypes.c_float(scale),
        int(window or 0), _p(out), out.stride(0), _dt(q), _stream()), "paged_attention")
    return out


DECODE_SHAPE_OVERRIDE = None      # (nsplit, waves): set by tests of the split path and by tuning scripts
DECODE_MAX_SPLIT = 8              # most workgroups that share one (token, head) pair's keys


# ---------------------------------------------------------------------------------
# Scratch buffers: device memory that a kernel needs beyond its inputs and outputs
# (argmax partial results, partial outputs and counters of the split decode attention).
# One set per device. A captured HIP graph keeps the raw address of the buffer it was
# captured with, so a buffer is never replaced behind a graph's back: callers that
# capture graphs reserve room for their largest launch first (``reserve_scratch``),
# and if a buffer must grow after all, everyone registered with ``on_scratch_growth``
# is told, and drops the graphs it holds.
# ---------------------------------------------------------------------------------
_SCRATCH: dict = {}               # (device, name) -> tensor
_GROWTH_LISTENERS: list = []      # weak references to bound methods


def on_scratch_growth(method) -> None:
    """Registers a bound method that is called (with no arguments) whenever a scratch buffer has
    been replaced by a larger one. Held weakly."""
    import weakref
    _GROWTH_LISTENERS.append(weakref.WeakMethod(method))


def _scratch(device, name: str, numel: int, dtype: torch.dtype, zero: bool = False) -> torch.Tensor:
    key = (torch.device(device), name)
    t = _SCRATCH.get(key)
    if t is not None and t.numel() >= numel:
        return t
    grown = (torch.zeros if zero else torch.empty)(numel, dtype=dtype, device=device)
    _SCRATCH[key] = grown
    if t is not None:
        alive = []
        for ref in _GROWTH_LISTENERS:
            fn = ref()
            if fn is not None:
                fn()
                alive.append(ref)
        _GROWTH_LISTENERS[:] = alive
    return grown


def scratch_address(device, name: str) -> int:
    """Address of a scratch buffer (0 if it does not exist yet): tests check that it stays put."""
    t = _SCRATCH.get((torch.device(device), name))
    return 0 if t is None else t.data_ptr()


def reserve_scratch(device, rows: int, vocab: int, n_heads: int = 0, head_dim: int = 0) -> None:
    """Makes the scratch buffers large enough for ``rows`` sampled rows of ``vocab`` logits and for
    decode attention over ``rows`` tokens of ``n_heads`` heads, so that no later launch up to these
    sizes replaces them."""
    if torch.device(device).type != "cuda":
        return
    chunks = load_library("sampling").mllm_argmax_chunks(int(vocab))
    _argmax_scratch(device, rows * chunks)
    if n_heads and head_dim:
        _decode_workspace(device, rows * n_heads, DECODE_MAX_SPLIT, head_dim)


DECODE_UNMERGED_SHAPE = None     # (nsplit, waves) for splits that the next product merges: tuning scripts


def _decode_launch_shape(pairs: int, max_ctx_len: int, unmerged: bool = False):
    """How many workgroups share one (token, head) pair's keys, and wavefronts per workgroup."""
    if DECODE_SHAPE_OVERRIDE is not None:
        return DECODE_SHAPE_OVERRIDE
    if unmerged:
        # The splits cost nothing to merge here (the next product does it while it loads), so few pairs
        # are spread over the compute units: a unit streams keys at 35 to 90 GB/s, and a pair's keys
        # and values at 768 tokens are 200 KB. Every split keeps at least 128 keys.
        if DECODE_UNMERGED_SHAPE is not None:
            return DECODE_UNMERGED_SHAPE
        # (measured at GPT-2 small sizes, 768 keys: 12 pairs x 4 splits of 4 wavefronts and 96 pairs x 2 splits
        # of 8 wavefronts are the fastest shapes; more workgroups than compute units lose again)
        nsplit = max(1, min(MERGE_MAX_SPLITS, 256 // max(pairs, 1), max_ctx_len // 128))
        if nsplit > 1:
            keys = -(-max_ctx_len // nsplit)
            return nsplit, max(2, min(12, -(-keys // 64)))
    # One workgroup per pair: merging splits (fences, a second merge) costs about 3 us, more than
    # the parallelism gains below about 2,000 keys (measured at 12 to 96 pairs). Few pairs get more
    # wavefronts each instead (measured: 12 are 1 to 3 % of a decode step faster than 8 up to 200
    # pairs at GPT-2 small to XL sizes, 3 % slower from 384 pairs).
    return 1, (4 if pairs >= 512 else 6 if pairs > 256 else 12)



def _decode_workspace(device, pairs: int, nsplit: int, head_dim: int):
    """Scratch of the split decode attention: partial outputs and a zeroed counter per
    (token, head) (the kernel leaves the counters at zero). Launches on one stream use it one
    after the other."""
    if nsplit <= 1:
        need_f = 1                      # one workgroup per pair exchanges nothing
    else:
        need_f = pairs * nsplit * (head_dim + 2)
    ws = _scratch(device, "decode_partials", max(need_f, 1 << 16), torch.float32)
    counters = _scratch(device, "decode_counters", max(pairs, 4096), torch.int32, zero=True)
    return ws, counters


def _argmax_scratch(device, n: int):
    """Partial results of the first stage of argmax: a value and an index per (row, chunk)."""
    return (_scratch(device, "argmax_values", max(n, 4096), torch.float32),
            _scratch(device, "argmax_indices", max(n, 4096), torch.int32))


def argmax(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[i] = index of the largest logits[i,:], the lowest index on ties."""
    _gpu(logits, out)
    _rows2d(logits, "logits")
    if logits.dtype != torch.float32:
        raise KernelError("logits must be fp32")
    n, V = logits.shape
    _i32(out, "out", n)
    lib = load_library("sampling")
    chunks = lib.mllm_argmax_chunks(V)
    pv, pi = _argmax_scratch(logits.device, n * chunks)
    _check(lib.mllm_argmax(_p(logits), logits.stride(0), n, V, _p(out), _p(pv), _p(pi), _stream()), "argmax")
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, u: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """Row i: temperature[i] <= 0 takes the argmax; otherwise draws from
    softmax(logits[i]/temperature[i]) by inverse CDF at u[i] in [0,1)."""
    _gpu(logits, temperature, u, out)
    _rows2d(logits, "logits")
    if logits.dtype != torch.float32:
        raise KernelError("logits must be fp32")
    n, V = logits.shape
    for name, t in (("temperature", temperature), ("u", u)):
        if t.dtype != torch.float32 or t.numel() < n or not t.is_contiguous():
            raise KernelError(f"{name} must be contiguous fp32 [{n}]")
    _i32(out, "out", n)
    lib = load_library("sampling")
    _check(lib.mllm_sample(_p(logits), logits.stride(0), n, V, _p(temperature), _p(u), _p(out), _stream()),
           "sample")
    return out
