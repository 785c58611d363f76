"""Plain torch references of the engine's device ops, one per kernel, same signatures.

GPU tests compare each kernel with its reference here, and CPU tests compare these with the
plain C++ twins (csrc/ref/ref_ops.cc). They are not part of the product path.
Accumulation is done in float64 (``PRECISE``) so that the reference is the more
accurate side of every comparison.
"""
from __future__ import annotations

import math

import torch

PRECISE = torch.float64


def embed(ids, positions, wte, wpe, out, src=None, prev=None):
    if src is not None:
        ids = torch.where((src >= 0) & (src < prev.numel()), prev[src.clamp(0, prev.numel() - 1).long()], ids)
    x = wte[ids.long()].to(PRECISE)
    if wpe is not None:
        x = x + wpe[positions.long()[: ids.numel()]].to(PRECISE)
    out.copy_(x.to(out.dtype))
    return out


def select_tokens(ids, src, prev):
    for i in range(ids.numel()):
        if int(src[i]) >= 0:
            ids[i] = prev[int(src[i])]
    return ids


def layernorm(x, gamma, beta, eps, out, rows=None):
    src = x if rows is None else x[rows.long()]
    s = src.to(PRECISE)
    mean = s.mean(-1, keepdim=True)
    var = ((s - mean) ** 2).mean(-1, keepdim=True)
    y = (s - mean) / torch.sqrt(var + eps) * gamma.to(PRECISE)
    if beta is not None:
        y = y + beta.to(PRECISE)
    out.copy_(y.to(out.dtype))
    return out


def _gelu_tanh(v):
    return 0.5 * v * (1.0 + torch.tanh(0.7978845608 * (v + 0.044715 * v ** 3)))


def _gelu_erf(v):
    return 0.5 * v * (1.0 + torch.erf(v / math.sqrt(2.0)))


def reset_state(state, slots, starts):
    for b in range(slots.numel()):
        if int(slots[b]) >= 0 and int(starts[b]) == 0:
            state[int(slots[b])] = 0


def linear(a, w, bias, out, epilogue="store", kv_scatter=None):
    y = a.to(PRECISE) @ w.to(PRECISE).T
    if bias is not None:
        y = y + bias.to(PRECISE)
    if epilogue == "gelu_tanh":
        y = _gelu_tanh(y)
    elif epilogue == "gelu_erf":
        y = _gelu_erf(y)
    if epilogue == "add_residual":
        out.add_(y.to(out.dtype))
    else:
        out.copy_(y.to(out.dtype))
    if kv_scatter is not None:
        slots, k_pages, v_pages, q_cols = kv_scatter
        kv_append(out, q_cols, q_cols + k_pages.shape[1], k_pages.shape[1], k_pages, v_pages, slots)
    return out


def ln_linear(x, gamma, beta, eps, w, bias, out, epilogue="store", rows=None, kv_scatter=None):
    n = x.shape[0] if rows is None else rows.numel()
    h = layernorm(x, gamma, beta, eps, torch.empty((n, x.shape[1]), dtype=w.dtype), rows)
    return linear(h, w, bias, out, epilogue, kv_scatter=kv_scatter)


def kv_append(src, k_col, v_col, kv_dim, k_pages, v_pages, slots):
    T = src.shape[0]
    s = slots[:T].long()
    keep = s >= 0
    k_pages[s[keep]] = src[keep, k_col:k_col + kv_dim]
    v_pages[s[keep]] = src[keep, v_col:v_col + kv_dim]


def paged_attention(q, q_col, n_heads, n_kv_heads, head_dim, k_pages, v_pages, page_size, block_tables,
                    token_seq, positions, scale, window, out, append=None, **_):
    # (the hints n_single and may_split change nothing here: the result is always merged into `out`)
    T = q.shape[0]
    if append is not None:
        kv_append(q, append[0], append[1], n_kv_heads * head_dim, k_pages, v_pages, append[2])
    rep = n_heads // n_kv_heads
    for t in range(T):
        b, p = int(token_seq[t]), int(positions[t])
        lo = max(0, p - window + 1) if window else 0
        js = torch.arange(lo, p + 1)
        rows = block_tables[b].long()[js // page_size] * page_size + js % page_size
        for h in range(n_heads):
            hk = h // rep
            qv = q[t, q_col + h * head_dim: q_col + (h + 1) * head_dim].to(PRECISE)
            k = k_pages[rows, hk * head_dim:(hk + 1) * head_dim].to(PRECISE)
            v = v_pages[rows, hk * head_dim:(hk + 1) * head_dim].to(PRECISE)
            s = (k @ qv) * scale
            w = torch.softmax(s, dim=0)
            out[t, h * head_dim:(h + 1) * head_dim] = (w @ v).to(out.dtype)
    return out


def argmax(logits, out):
    n = logits.shape[0]
    for i in range(n):
        row = logits[i]
        out[i] = int(torch.nonzero(row == row.max())[0])
    return out


def sample(logits, temperature, u, out):
    n = logits.shape[0]
    for i in range(n):
        t = float(temperature[i])
        row = logits[i].to(PRECISE)
        if t <= 0:
            out[i] = int(torch.nonzero(row == row.max())[0])
            continue
        p = torch.exp((row - row.max()) / t)
        c = torch.cumsum(p, 0)
        target = float(u[i]) * float(c[-1])
        idx = int(torch.searchsorted(c, torch.tensor(target, dtype=PRECISE), right=True))
        out[i] = min(idx, row.numel() - 1)
    return out
