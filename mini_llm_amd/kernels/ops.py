"""The engine's device operations, seen from Python: a thin face over the native ops
(csrc/engine/ops.cc), which check shapes, strides and dtypes, choose among the kernels of an
operation by size and launch on torch's current HIP stream. The engine's parts call the same
functions natively; this face serves the tests of a kernel alone and tuning scripts.

There is no CPU path: a tensor that is not on the GPU, or a library that cannot be built and
loaded, raises.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .. import native

EPILOGUES = {"store": 0, "gelu_tanh": 1, "gelu_erf": 2, "add_residual": 3, "store_f32": 4}
_DT = {torch.float32: 0, torch.bfloat16: 1}
_DT_BACK = {0: torch.float32, 1: torch.bfloat16}


class KernelError(RuntimeError):
    pass


# -- the native structures (csrc/engine/ops.h) ---------------------------------------------------
_vp, _i, _i64, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float


class Tensor2(ctypes.Structure):
    _fields_ = [("data", _vp), ("dtype", _i), ("rows", _i64), ("cols", _i64), ("stride", _i64)]


class KvScatterC(ctypes.Structure):
    _fields_ = [("slots", _vp), ("k_pages", Tensor2), ("v_pages", Tensor2), ("q_cols", _i)]


class AttentionSplitsC(ctypes.Structure):
    _fields_ = [("ws", _vp), ("n_tokens", _i), ("n_heads", _i), ("head_dim", _i), ("nsplit", _i), ("dtype", _i)]


class AttentionArgsC(ctypes.Structure):
    _fields_ = [("q", Tensor2), ("q_col", _i), ("n_heads", _i), ("n_kv_heads", _i), ("head_dim", _i),
                ("k_pages", Tensor2), ("v_pages", Tensor2), ("page_size", _i), ("block_tables", _vp),
                ("n_seqs", _i), ("max_blocks", _i), ("token_seq", _vp), ("positions", _vp), ("scale", _f),
                ("window", _i), ("out", Tensor2), ("cu_q", _vp), ("ctx_len", _vp), ("max_q_len", _i),
                ("max_ctx_len", _i), ("append", _i), ("k_col", _i), ("v_col", _i), ("slots", _vp),
                ("n_single", _i), ("may_split", _i)]


_lib = None


def engine_library():
    """The native engine library, with its functions' types declared."""
    global _lib
    if _lib is not None:
        return _lib
    lib = native.lib()
    T2p, sz = ctypes.POINTER(Tensor2), ctypes.c_size_t
    sigs = {
        "mllm_op_embed": (_i, [_vp, _vp, T2p, T2p, T2p, _vp, _vp, _i, _vp]),
        "mllm_op_select_tokens": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
        "mllm_op_reset_state": (_i, [_vp, sz, _i, _vp, _vp, _i, _vp]),
        "mllm_op_layernorm": (_i, [T2p, _vp, _vp, _f, T2p, _vp, _vp]),
        "mllm_op_kv_append": (_i, [T2p, _i, _i, T2p, T2p, _vp, _vp]),
        "mllm_op_linear": (_i, [T2p, T2p, _vp, T2p, _i, ctypes.POINTER(KvScatterC), _vp]),
        "mllm_op_linear_from_splits": (_i, [ctypes.POINTER(AttentionSplitsC), T2p, _vp, T2p, _i, _vp, _vp]),
        "mllm_op_merge_splits": (_i, [ctypes.POINTER(AttentionSplitsC), T2p, _vp]),
        "mllm_op_ln_linear": (_i, [T2p, _vp, _vp, _f, T2p, _vp, T2p, _i, _vp, _vp, _vp, _vp]),
        "mllm_op_paged_attention": (_i, [ctypes.POINTER(AttentionArgsC), ctypes.POINTER(AttentionSplitsC),
                                         ctypes.POINTER(_i), _vp]),
        "mllm_op_argmax": (_i, [T2p, _vp, _vp]),
        "mllm_op_sample": (_i, [T2p, _vp, _vp, _vp, _vp]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def _ok(rc: int) -> None:
    if rc != 0:
        raise KernelError(engine_library().mllm_last_error().decode("utf-8", "replace"))


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


def _dt(t: torch.Tensor) -> int:
    if t.dtype not in _DT:
        raise KernelError(f"unsupported dtype {t.dtype} (float32 or bfloat16)")
    return _DT[t.dtype]


def t2(t: Optional[torch.Tensor], name: str = "tensor") -> Tensor2:
    """A 2-D native view of a tensor (a 1-D tensor is one row)."""
    if t is None:
        return Tensor2(None, 0, 0, 0, 0)
    if t.dim() == 1:
        t = t.view(1, -1)
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{name} must be 2-D with a contiguous last dimension, got shape "
                          f"{tuple(t.shape)} strides {t.stride()}")
    stride = t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])
    return Tensor2(t.data_ptr(), _dt(t), t.shape[0], t.shape[1], stride)


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{name} must be a contiguous int32 tensor")
    if n is not None and t.numel() < n:
        raise KernelError(f"{name} has {t.numel()} entries, {n} needed")


def _f32vec(t: Optional[torch.Tensor], name: str, n: int) -> None:
    if t is not None and (t.dtype != torch.float32 or t.numel() != n or not t.is_contiguous()):
        raise KernelError(f"{name} must be contiguous fp32 [{n}]")


# -- scratch and tuning -----------------------------------------------------------------------------
# Scratch buffers (device memory that a kernel needs beyond its inputs and outputs: argmax partial
# results, the states of split decode attention, shared-tile sums) are kept per stream by the native
# side; ops called from here use the set of torch's current stream.

def scratch_address(name: str) -> int:
    """Address of a scratch buffer of the current stream (0 if it does not exist yet)."""
    return engine_library().mllm_scratch_address(name.encode(), _stream()) or 0


def scratch_bytes() -> int:
    """Bytes of scratch that all streams of the current device hold."""
    return int(engine_library().mllm_scratch_bytes())


def seen(name: str) -> int:
    """What the ops chose since ``reset_seen()``: "max_decode_splits", "merge_kernel_launches",
    "prefill_tile_launches", "generic_attention_launches"."""
    v = engine_library().mllm_get_seen(name.encode())
    if v < 0:
        raise KernelError(f"unknown counter '{name}'")
    return int(v)


def reset_seen() -> None:
    _ok(engine_library().mllm_set_tuning(b"reset_seen", 0, 0))


# Tuning hooks: tests and tuning scripts set these module attributes; they reach the native side at the
# next op that they concern.
DECODE_SHAPE_OVERRIDE = None      # (nsplit, waves): forced launch shape of decode attention merged in its kernel
DECODE_UNMERGED_SHAPE = None      # (nsplit, waves): forced shape of splits that the next product merges
MERGE_MAX_ROWS = 16               # tokens whose attention splits a product merges while loading (one row block)
LONG_CONTEXT_SPLITS = True        # few pairs with long contexts: keys split over up to 256 workgroups, merged by a small kernel
LN_FUSE_MAX_ROWS = 32             # rows up to which the few-row product normalises its input itself (measured: 1-2 % of
                                  # a decode step gained at 24 and 32 rows, 3 % lost at 64)
_pushed_tuning = None


def push_tuning() -> None:
    """Hands the module's tuning values to the native side if they have changed."""
    global _pushed_tuning
    now = (DECODE_SHAPE_OVERRIDE, DECODE_UNMERGED_SHAPE, MERGE_MAX_ROWS, LN_FUSE_MAX_ROWS, LONG_CONTEXT_SPLITS)
    if now == _pushed_tuning:
        return
    lib = engine_library()
    a, b = DECODE_SHAPE_OVERRIDE or (0, 0)
    _ok(lib.mllm_set_tuning(b"decode_shape", int(a), int(b)))
    a, b = DECODE_UNMERGED_SHAPE or (0, 0)
    _ok(lib.mllm_set_tuning(b"unmerged_shape", int(a), int(b)))
    _ok(lib.mllm_set_tuning(b"merge_max_rows", int(MERGE_MAX_ROWS), 0))
    _ok(lib.mllm_set_tuning(b"ln_fuse_max_rows", int(LN_FUSE_MAX_ROWS), 0))
    _ok(lib.mllm_set_tuning(b"long_context_splits", 1 if LONG_CONTEXT_SPLITS else 0, 0))
    _pushed_tuning = now


# -- the ops -----------------------------------------------------------------------------------------

def embed(ids: torch.Tensor, positions: Optional[torch.Tensor], wte: torch.Tensor,
          wpe: Optional[torch.Tensor], out: torch.Tensor, src: Optional[torch.Tensor] = None,
          prev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t,:] = wte[ids[t],:] + wpe[positions[t],:] in fp32. ids/positions must be in range
    (the caller checks them on the host). With ``src`` and ``prev``: where src[t] >= 0, token t's id is
    prev[src[t]] (a token that an earlier step sampled on the device) instead of ids[t]."""
    _gpu(ids, positions, wte, wpe, out, src, prev)
    if src is not None:
        _i32(src, "src", ids.numel())
        _i32(prev, "prev")
    T = ids.numel()
    _i32(ids, "ids")
    if wpe is not None:
        if positions is None:
            raise KernelError("positions are needed with a position table")
        _i32(positions, "positions", T)
    if out.dim() != 2 or out.shape[0] != T:
        raise KernelError(f"out must be contiguous fp32 [{T}, {wte.shape[1]}]")
    _ok(engine_library().mllm_op_embed(_p(ids), _p(positions), ctypes.byref(t2(wte, "wte")),
                                       ctypes.byref(t2(wpe, "wpe")) if wpe is not None else None,
                                       ctypes.byref(t2(out, "out")), _p(src), _p(prev),
                                       0 if prev is None else prev.numel(), _stream()))
    return out


def select_tokens(ids: torch.Tensor, src: torch.Tensor, prev: torch.Tensor) -> torch.Tensor:
    """ids[i] = prev[src[i]] where src[i] >= 0, in place: token ids that an earlier step sampled
    on the device and the host has not read yet."""
    _gpu(ids, src, prev)
    n = ids.numel()
    _i32(ids, "ids")
    _i32(src, "src", n)
    _i32(prev, "prev")
    _ok(engine_library().mllm_op_select_tokens(_p(ids), _p(src), _p(prev), n, prev.numel(), _stream()))
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
    _ok(engine_library().mllm_op_reset_state(_p(state), slot_bytes, state.shape[0], _p(slots), _p(starts), B,
                                             _stream()))


def layernorm(x: torch.Tensor, gamma: torch.Tensor, beta: Optional[torch.Tensor], eps: float,
              out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[i,:] = LayerNorm(x[rows[i] if rows else i,:]); statistics in fp32."""
    _gpu(x, gamma, beta, out, rows)
    if x.dim() != 2:
        raise KernelError("layernorm input must be contiguous fp32 [rows, D]")
    D = x.shape[1]
    n = rows.numel() if rows is not None else x.shape[0]
    if rows is not None:
        _i32(rows, "rows")
    _f32vec(gamma, "gamma", D)
    _f32vec(beta, "beta", D)
    if out.shape != (n, D):
        raise KernelError(f"out must be contiguous [{n}, {D}]")
    _ok(engine_library().mllm_op_layernorm(ctypes.byref(t2(x, "x")), _p(gamma), _p(beta), eps,
                                           ctypes.byref(t2(out, "out")), _p(rows), _stream()))
    return out


class AttentionSplits:
    """The output of decode attention that has not been merged yet: every (token, head) pair's keys
    were split over ``nsplit`` workgroups, whose states (running maximum, sum, unnormalised output)
    lie in the attention scratch. ``linear`` takes it in place of a tensor and merges while it loads
    (``tensor()`` merges into an ordinary activation). Valid until the next attention launch."""

    def __init__(self, c: AttentionSplitsC, device):
        self.c = c
        self.n_tokens, self.n_heads, self.head_dim, self.nsplit = c.n_tokens, c.n_heads, c.head_dim, c.nsplit
        self.dtype, self.device = _DT_BACK[c.dtype], device
        self.shape = (c.n_tokens, c.n_heads * c.head_dim)

    def tensor(self, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if out is None:
            out = torch.empty(self.shape, dtype=self.dtype, device=self.device)
        _ok(engine_library().mllm_op_merge_splits(ctypes.byref(self.c), ctypes.byref(t2(out, "out")), _stream()))
        return out


def linear(a, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
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
    if epilogue not in EPILOGUES:
        raise KernelError(f"unknown epilogue '{epilogue}'")
    _f32vec(bias, "bias", w.shape[0])
    lib = engine_library()
    if splits is not None:
        if kv_scatter is not None:
            raise KernelError("linear: attention splits and a key/value scatter do not go together")
        tmp = torch.empty(splits.shape, dtype=splits.dtype, device=splits.device)
        _ok(lib.mllm_op_linear_from_splits(ctypes.byref(splits.c), ctypes.byref(t2(w, "w")), _p(bias),
                                           ctypes.byref(t2(out, "out")), EPILOGUES[epilogue], _p(tmp), _stream()))
        return out
    kv = None
    if kv_scatter is not None:
        slots, k_pages, v_pages, q_cols = kv_scatter
        _gpu(slots, k_pages, v_pages)
        _i32(slots, "slots", a.shape[0])
        kv = ctypes.byref(KvScatterC(slots.data_ptr(), t2(k_pages, "k_pages"), t2(v_pages, "v_pages"), int(q_cols)))
    _ok(lib.mllm_op_linear(ctypes.byref(t2(a, "a")), ctypes.byref(t2(w, "w")), _p(bias), ctypes.byref(t2(out, "out")),
                           EPILOGUES[epilogue], kv, _stream()))
    return out


def ln_linear(x: torch.Tensor, gamma: torch.Tensor, beta: Optional[torch.Tensor], eps: float,
              w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, epilogue: str = "store",
              rows: Optional[torch.Tensor] = None, kv_scatter: Optional[tuple] = None) -> torch.Tensor:
    """out = epilogue(LayerNorm(x) @ w.T + bias) with x the fp32 stream [*,K] and w [N,K]; with
    ``rows`` (int32 [M]) row m of the input is x[rows[m]]; ``kv_scatter`` as for ``linear``.

    For bfloat16 weights, at most 32 rows and fewer than 16384 columns the norm is fused into the
    product (one kernel); otherwise the norm and the product run one after the other. Same numerics
    either way: statistics in fp32, the normalised rows rounded to w's dtype before the product.
    """
    _gpu(x, gamma, beta, w, bias, out, rows)
    if epilogue not in EPILOGUES:
        raise KernelError(f"unknown epilogue '{epilogue}'")
    K = x.shape[1]
    M = x.shape[0] if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, "rows")
    _f32vec(gamma, "gamma", K)
    _f32vec(beta, "beta", K)
    _f32vec(bias, "bias", w.shape[0])
    if out.shape[0] != M:
        raise KernelError(f"ln_linear({epilogue}): out must have {M} rows")
    push_tuning()
    # (room for the normalised rows, used when the fused kernel does not take these sizes)
    tmp = torch.empty((M, K), dtype=w.dtype, device=x.device)
    kv = None
    if kv_scatter is not None:
        slots, k_pages, v_pages, q_cols = kv_scatter
        _gpu(slots, k_pages, v_pages)
        _i32(slots, "slots", M)
        kv = ctypes.byref(KvScatterC(slots.data_ptr(), t2(k_pages, "k_pages"), t2(v_pages, "v_pages"), int(q_cols)))
    _ok(engine_library().mllm_op_ln_linear(ctypes.byref(t2(x, "x")), _p(gamma), _p(beta), eps, ctypes.byref(t2(w, "w")),
                                           _p(bias), ctypes.byref(t2(out, "out")), EPILOGUES[epilogue], _p(rows),
                                           _p(tmp), kv, _stream()))
    return out


def kv_append(src: torch.Tensor, k_col: int, v_col: int, kv_dim: int, k_pages: torch.Tensor,
              v_pages: torch.Tensor, slots: torch.Tensor) -> None:
    """Copies columns [k_col, k_col+kv_dim) and [v_col, v_col+kv_dim) of each row of ``src``
    into row ``slots[t]`` of the key and value pages (slot < 0: skipped)."""
    _gpu(src, k_pages, v_pages, slots)
    _i32(slots, "slots", src.shape[0])
    if k_pages.dim() != 2 or k_pages.shape[1] != kv_dim:
        raise KernelError(f"k_pages must be contiguous [rows, {kv_dim}] {src.dtype}")
    _ok(engine_library().mllm_op_kv_append(ctypes.byref(t2(src, "src")), int(k_col), int(v_col),
                                           ctypes.byref(t2(k_pages, "k_pages")), ctypes.byref(t2(v_pages, "v_pages")),
                                           _p(slots), _stream()))


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
    _gpu(q, k_pages, v_pages, block_tables, token_seq, positions, out, cu_q, ctx_len)
    T = q.shape[0]
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise KernelError("block_tables must be contiguous int32 [B, max_blocks]")
    B = block_tables.shape[0]
    _i32(token_seq, "token_seq", T)
    _i32(positions, "positions", T)
    if cu_q is not None:
        _i32(cu_q, "cu_q", B + 1)
    if ctx_len is not None:
        _i32(ctx_len, "ctx_len", B)
    a = AttentionArgsC()
    a.q, a.q_col, a.n_heads, a.n_kv_heads, a.head_dim = t2(q, "q"), int(q_col), int(n_heads), int(n_kv_heads), int(head_dim)
    a.k_pages, a.v_pages, a.page_size = t2(k_pages, "k_pages"), t2(v_pages, "v_pages"), int(page_size)
    a.block_tables, a.n_seqs, a.max_blocks = block_tables.data_ptr(), B, block_tables.shape[1]
    a.token_seq, a.positions, a.scale, a.window = token_seq.data_ptr(), positions.data_ptr(), float(scale), int(window or 0)
    a.out = t2(out, "out")
    a.cu_q = cu_q.data_ptr() if cu_q is not None else None
    a.ctx_len = ctx_len.data_ptr() if ctx_len is not None else None
    a.max_q_len, a.max_ctx_len = int(max_q_len), int(max_ctx_len)
    if append is not None:
        k_col, v_col, slots = append
        _gpu(slots)
        _i32(slots, "slots", T)
        a.append, a.k_col, a.v_col, a.slots = 1, int(k_col), int(v_col), slots.data_ptr()
    a.n_single, a.may_split = int(n_single), 1 if may_split else 0
    push_tuning()
    splits, unmerged = AttentionSplitsC(), _i(0)
    _ok(engine_library().mllm_op_paged_attention(ctypes.byref(a), ctypes.byref(splits), ctypes.byref(unmerged), _stream()))
    if unmerged.value:
        return AttentionSplits(splits, q.device)
    return out


def argmax(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[i] = index of the largest logits[i,:], the lowest index on ties."""
    _gpu(logits, out)
    _i32(out, "out", logits.shape[0])
    _ok(engine_library().mllm_op_argmax(ctypes.byref(t2(logits, "logits")), _p(out), _stream()))
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, u: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """Row i: temperature[i] <= 0 takes the argmax; otherwise draws from
    softmax(logits[i]/temperature[i]) by inverse CDF at u[i] in [0,1)."""
    _gpu(logits, temperature, u, out)
    n = logits.shape[0]
    for name, t in (("temperature", temperature), ("u", u)):
        if t.dtype != torch.float32 or t.numel() < n or not t.is_contiguous():
            raise KernelError(f"{name} must be contiguous fp32 [{n}]")
    _i32(out, "out", n)
    _ok(engine_library().mllm_op_sample(ctypes.byref(t2(logits, "logits")), _p(temperature), _p(u), _p(out), _stream()))
    return out
