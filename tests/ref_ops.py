"""Python face of the plain C++ twins of the device operations (csrc/ref/ref_ops.cc): same signatures
as ``plain_ops``, CPU tensors, results in float32 (sums in double inside). The kernel tests compare the
HIP kernels with these as well as with the plain Python references."""
import ctypes

import torch

from mini_llm_amd.build import load_library

_EPI = {"store": 0, "gelu_tanh": 1, "gelu_erf": 2, "add_residual": 3, "store_f32": 4}


def _lib():
    return load_library("ref")


def _f(t):
    return t.detach().to(torch.float32).contiguous()


def _p(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def embed(ids, positions, wte, wpe):
    ids, wte = ids.to(torch.int32).contiguous(), _f(wte)
    wpe = None if wpe is None else _f(wpe)
    pos = None if positions is None else positions.to(torch.int32).contiguous()
    out = torch.empty((ids.numel(), wte.shape[1]), dtype=torch.float32)
    _lib().ref_embed(_p(ids), _p(pos), _p(wte), _p(wpe), _p(out), ids.numel(), wte.shape[1])
    return out


def layernorm(x, gamma, beta, eps, rows=None):
    x, gamma = _f(x), _f(gamma)
    beta = None if beta is None else _f(beta)
    rows = None if rows is None else rows.to(torch.int32).contiguous()
    n = x.shape[0] if rows is None else rows.numel()
    out = torch.empty((n, x.shape[1]), dtype=torch.float32)
    _lib().ref_layernorm(_p(x), _p(rows), _p(gamma), _p(beta), ctypes.c_float(eps), _p(out), n, x.shape[1])
    return out


def linear(a, w, bias, out0=None, epilogue="store"):
    a, w = _f(a), _f(w)
    bias = None if bias is None else _f(bias)
    out = torch.zeros((a.shape[0], w.shape[0]), dtype=torch.float32) if out0 is None else _f(out0).clone()
    assert _lib().ref_linear(_p(a), _p(w), _p(bias), _p(out), a.shape[0], w.shape[0], a.shape[1], _EPI[epilogue]) == 0
    return out


def kv_append(src, k_col, v_col, kv_dim, k_pages, v_pages, slots):
    """In place on float32 pages."""
    s = _f(src)
    assert k_pages.dtype == torch.float32 and v_pages.dtype == torch.float32 and k_pages.is_contiguous()
    sl = slots.to(torch.int32).contiguous()
    _lib().ref_kv_append(_p(s), s.stride(0), k_col, v_col, _p(k_pages), _p(v_pages), kv_dim, _p(sl), s.shape[0])


def paged_attention(q, q_col, n_heads, n_kv_heads, head_dim, k_pages, v_pages, page_size, block_tables, token_seq,
                    positions, scale, window):
    q, k, v = _f(q), _f(k_pages), _f(v_pages)
    k, v = torch.nan_to_num(k, nan=0.0), torch.nan_to_num(v, nan=0.0)      # (rows never read may hold NaN)
    bt = block_tables.to(torch.int32).contiguous()
    ts, ps = token_seq.to(torch.int32).contiguous(), positions.to(torch.int32).contiguous()
    out = torch.empty((q.shape[0], n_heads * head_dim), dtype=torch.float32)
    _lib().ref_paged_attention(_p(q), q.stride(0), q_col, n_heads, n_kv_heads, head_dim, _p(k), _p(v), page_size,
                               _p(bt), bt.shape[1], _p(ts), _p(ps), ctypes.c_float(scale), int(window or 0), _p(out),
                               q.shape[0])
    return out


def argmax(logits):
    l = _f(logits)
    out = torch.empty(l.shape[0], dtype=torch.int32)
    _lib().ref_argmax(_p(l), l.shape[0], l.shape[1], _p(out))
    return out


def sample(logits, temperature, u):
    l, t, uu = _f(logits), _f(temperature), _f(u)
    out = torch.empty(l.shape[0], dtype=torch.int32)
    _lib().ref_sample(_p(l), l.shape[0], l.shape[1], _p(t), _p(uu), _p(out))
    return out


def gelu(x, exact=False):
    x = _f(x)
    out = torch.empty_like(x)
    _lib().ref_gelu(_p(x), _p(out), ctypes.c_long(x.numel()), 1 if exact else 0)
    return out


def add_bias(x, bias):
    out = _f(x).clone()
    _lib().ref_add_bias(_p(out), _p(_f(bias)), out.shape[0], out.shape[1])
    return out


def residual_add(x, y):
    out, y = _f(x).clone(), _f(y)
    _lib().ref_residual_add(_p(out), _p(y), ctypes.c_long(out.numel()))
    return out
