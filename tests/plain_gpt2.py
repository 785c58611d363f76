"""A plain, slow GPT-2: whole sequences, no cache, one function for each part.

Written from the reference's formulas (cited per function); it shares no code with
the engine: it parses config.json itself and reads the checkpoint with the
``safetensors`` package. Everything is computed in float64 by default.
The reference is read, not run.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List

import torch
from safetensors import safe_open


def read_model(model_dir: str, dtype=torch.float64):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w: Dict[str, torch.Tensor] = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            short = name[len("transformer."):] if name.startswith("transformer.") else name
            w[short] = f.get_tensor(name).to(dtype)
    return cfg, w


def embedding(wte, wpe, ids, positions):
    """x[t,:] = wte[id[t],:] + wpe[pos[t],:]  -- /root/reference/src/kernels/embedding.cu:23-43"""
    return wte[ids] + wpe[positions]


def layer_norm(x, gamma, beta, eps):
    """mean; biased variance of (x - mean); (x - mean) * rsqrt(var + eps) * gamma + beta
    -- /root/reference/src/kernels/layernorm.cu:32-49"""
    mean = x.sum(-1, keepdim=True) / x.shape[-1]
    c = x - mean
    var = (c * c).sum(-1, keepdim=True) / x.shape[-1]
    return c / torch.sqrt(var + eps) * gamma + beta


def conv1d_linear(x, w, b):
    """y = x W + b with W stored [in, out], used untransposed
    -- /root/reference/scripts/export_weights.py:47-52, /root/reference/src/kernels/linear.cu:8-40"""
    return x @ w + b


def gelu_tanh(v):
    """0.5 v (1 + tanh(0.7978845608 (v + 0.044715 v^3)))  -- /root/reference/src/kernels/gelu.cu:7-9"""
    return 0.5 * v * (1.0 + torch.tanh(0.7978845608 * (v + 0.044715 * v * v * v)))


def gelu_erf(v):
    """0.5 v (1 + erf(v / sqrt 2)); the exact form that config value "gelu" names.
    The reference has only the tanh form."""
    return 0.5 * v * (1.0 + torch.erf(v / math.sqrt(2.0)))


ACTIVATIONS = {"gelu_new": gelu_tanh, "gelu_pytorch_tanh": gelu_tanh, "gelu_fast": gelu_tanh, "gelu": gelu_erf}


def causal_attention(q, k, v, n_head, window=None):
    """Per head h (columns [h*dh, (h+1)*dh) of q, k, v): s_ij = (q_i . k_j) / sqrt(dh) for j <= i,
    softmax over j with the maximum subtracted, o_i = sum_j w_ij v_j; heads concatenated.
    -- /root/reference/src/kernels/prefill/flashattention.cu:71-79,129-178 (causal skip, softmax),
       scale 1/sqrt(dh) at /root/reference/src/model/gpt2_model.cu:308,
       naive form /root/reference/tests/cpp/test_flashattention.cu:39-105."""
    n, d = q.shape
    dh = d // n_head
    out = torch.zeros_like(q)
    for h in range(n_head):
        qh, kh, vh = (t[:, h * dh:(h + 1) * dh] for t in (q, k, v))
        for i in range(n):
            lo = 0 if not window else max(0, i - window + 1)
            s = (kh[lo:i + 1] @ qh[i]) / math.sqrt(dh)
            s = s - s.max()
            e = torch.exp(s)
            w = e / e.sum()
            out[i, h * dh:(h + 1) * dh] = w @ vh[lo:i + 1]
    return out


def attention_block(x, w, i, n_head):
    """qkv = x W_attn + b; q,k,v = columns [0,D), [D,2D), [2D,3D); attention; then the output
    projection -- /root/reference/src/model/gpt2_model.cu:289-334,
    column split /root/reference/src/kernels/prefill/append_kv.cu:31-33."""
    D = x.shape[-1]
    qkv = conv1d_linear(x, w[f"h.{i}.attn.c_attn.weight"], w[f"h.{i}.attn.c_attn.bias"])
    q, k, v = qkv[:, :D], qkv[:, D:2 * D], qkv[:, 2 * D:]
    a = causal_attention(q, k, v, n_head)
    return conv1d_linear(a, w[f"h.{i}.attn.c_proj.weight"], w[f"h.{i}.attn.c_proj.bias"])


def mlp_block(x, w, i, act):
    """act(x W_fc + b) W_proj + b  -- /root/reference/src/model/gpt2_model.cu:345-363"""
    h = act(conv1d_linear(x, w[f"h.{i}.mlp.c_fc.weight"], w[f"h.{i}.mlp.c_fc.bias"]))
    return conv1d_linear(h, w[f"h.{i}.mlp.c_proj.weight"], w[f"h.{i}.mlp.c_proj.bias"])


def block(x, w, i, cfg):
    """Pre-norm: x += attn(ln_1(x)); x += mlp(ln_2(x))  -- /root/reference/src/model/gpt2_model.cu:279-363"""
    eps = cfg["layer_norm_epsilon"]
    act = ACTIVATIONS[cfg.get("activation_function", "gelu_new")]
    x = x + attention_block(layer_norm(x, w[f"h.{i}.ln_1.weight"], w[f"h.{i}.ln_1.bias"], eps), w, i,
                            cfg["n_head"])
    x = x + mlp_block(layer_norm(x, w[f"h.{i}.ln_2.weight"], w[f"h.{i}.ln_2.bias"], eps), w, i, act)
    return x


def logits_head(x, w, cfg):
    """ln_f, then logits = h wte^T (tied, no bias) -- /root/reference/src/model/gpt2_model.cu:408-428"""
    h = layer_norm(x, w["ln_f.weight"], w["ln_f.bias"], cfg["layer_norm_epsilon"])
    return h @ w["wte.weight"].T


def forward_logits(cfg, w, ids: List[int]) -> torch.Tensor:
    """Logits [len(ids), vocab] of one whole sequence."""
    ids_t = torch.tensor(ids, dtype=torch.long)
    x = embedding(w["wte.weight"], w["wpe.weight"], ids_t, torch.arange(len(ids)))
    for i in range(cfg["n_layer"]):
        x = block(x, w, i, cfg)
    return logits_head(x, w, cfg)


def greedy_generate(cfg, w, prompt: List[int], n_new: int) -> List[int]:
    """Argmax with the lowest index on ties -- /root/reference/src/kernels/argmax.cu:12-20.
    The whole sequence is recomputed for every token."""
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        row = forward_logits(cfg, w, ids)[-1]
        tok = int(torch.nonzero(row == row.max())[0])
        out.append(tok)
        ids.append(tok)
    return out
