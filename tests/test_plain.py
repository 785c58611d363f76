"""Pins the plain implementation (tests/plain_gpt2.py) by what fixes it beside the reference's
text: vectors the reference's own tests hold, special cases that reduce to a library routine,
and invariants, each chosen so that a plausible mistake fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_gpt2 as P
from conftest import TINY_A, TINY_B

D64 = torch.float64


def test_embedding_reference_vector():
    # /root/reference/tests/kernels/embedding/gen.py:13-27
    V, S, D = 64, 32, 768
    wte = torch.arange(V, dtype=D64)[:, None] * 0.01 + torch.arange(D, dtype=D64)[None] * 0.0001
    wpe = torch.arange(S, dtype=D64)[:, None] * 0.001 + torch.arange(D, dtype=D64)[None] * 0.00001
    ids = torch.tensor([3, 5, 7, 5, 11, 13, 17])
    x = P.embedding(wte, wpe, ids, torch.arange(7))
    assert x[3, 10].item() == pytest.approx(5 * 0.01 + 10 * 0.0001 + 3 * 0.001 + 10 * 0.00001, abs=1e-12)
    assert torch.equal(x, F.embedding(ids, wte) + wpe[:7])
    assert not torch.equal(x[1], x[3])          # same token, other position


def test_layer_norm_reference_vector_and_invariants():
    # /root/reference/tests/kernels/layernorm/gen.py:8-21
    rng = np.random.default_rng(0)
    x = rng.normal(0.0, 1.0, size=(17, 768)).astype(np.float32)
    gamma = rng.normal(1.0, 0.1, size=(768,)).astype(np.float32)
    beta = rng.normal(0.0, 0.1, size=(768,)).astype(np.float32)
    mean = x.mean(axis=1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=1, keepdims=True)
    expected = ((x - mean) / np.sqrt(var + 1e-5)) * gamma + beta
    xt, gt, bt = (torch.from_numpy(a).double() for a in (x, gamma, beta))
    y = P.layer_norm(xt, gt, bt, 1e-5)
    assert np.abs(y.numpy() - expected).max() <= 1e-4
    assert (y - F.layer_norm(xt, (768,), gt, bt, 1e-5)).abs().max() <= 1e-12
    # biased variance: an unbiased one differs by a factor sqrt(767/768)
    plain = P.layer_norm(xt, torch.ones(768, dtype=D64), torch.zeros(768, dtype=D64), 0.0)
    assert plain.mean(-1).abs().max() <= 1e-12 and (plain.pow(2).mean(-1) - 1).abs().max() <= 1e-9
    assert (P.layer_norm(xt + 3.5, gt, bt, 1e-5) - y).abs().max() <= 1e-9          # shift invariance
    const = torch.full((1, 768), 2.0, dtype=D64)
    assert torch.equal(P.layer_norm(const, gt, bt, 1e-5), bt[None])                  # constant row -> beta
    tiny = xt[:1] * 1e-3
    assert (P.layer_norm(tiny, gt, bt, 1e-5) - P.layer_norm(tiny, gt, bt, 1e-6)).abs().max() > 1e-2   # eps counts


def test_conv1d_linear_uses_in_out_layout():
    # /root/reference/tests/kernels/linear/gen.py:8-16
    rng = np.random.default_rng(0)
    x = rng.normal(0, 0.02, size=(5, 768)).astype(np.float32)
    w = rng.normal(0, 0.02, size=(768, 2304)).astype(np.float32)
    b = rng.normal(0, 0.02, size=(2304,)).astype(np.float32)
    y = P.conv1d_linear(*(torch.from_numpy(a).double() for a in (x, w, b)))
    assert y.shape == (5, 2304) and np.abs(y.numpy() - (x @ w + b)).max() <= 1e-3
    assert torch.allclose(y, F.linear(torch.from_numpy(x).double(), torch.from_numpy(w).double().T,
                                      torch.from_numpy(b).double()))


def test_gelu_forms():
    # /root/reference/tests/kernels/gelu/gen.py:5-12
    x = torch.arange(1027, dtype=D64) * 0.01 - 5.0
    assert (P.gelu_tanh(x) - F.gelu(x, approximate="tanh")).abs().max() <= 1e-9
    assert (P.gelu_erf(x) - F.gelu(x)).abs().max() <= 1e-12
    xr = np.arange(1027, dtype=np.float32) * 0.01
    expected = 0.5 * xr * (1.0 + np.tanh(0.7978845608 * (xr + 0.044715 * np.power(xr, 3))))
    assert np.abs(P.gelu_tanh(torch.from_numpy(xr).double()).numpy() - expected).max() <= 1e-5
    assert (P.gelu_tanh(x) - P.gelu_erf(x)).abs().max() > 1e-4       # a swapped activation is seen
    assert P.ACTIVATIONS["gelu_new"] is P.gelu_tanh and P.ACTIVATIONS["gelu"] is P.gelu_erf


def _sdpa(q, k, v, n_head):
    n, d = q.shape
    sp = lambda t: t.view(n, n_head, d // n_head).transpose(0, 1)
    return F.scaled_dot_product_attention(sp(q), sp(k), sp(v), is_causal=True).transpose(0, 1).reshape(n, d)


@pytest.mark.parametrize("n_head,dh", [(4, 16), (3, 32), (1, 8)])
def test_attention_reduces_to_the_library_routine(n_head, dh):
    g = torch.Generator().manual_seed(n_head)
    q, k, v = (torch.randn(37, n_head * dh, generator=g, dtype=D64) for _ in range(3))
    out = P.causal_attention(q, k, v, n_head)
    assert (out - _sdpa(q, k, v, n_head)).abs().max() <= 1e-12
    assert torch.allclose(out[0], v[0])                                        # the first token sees itself only
    perm = torch.cat([torch.arange(20), 20 + torch.randperm(17, generator=g)])
    out_p = P.causal_attention(q[perm], k[perm], v[perm], n_head)
    assert torch.equal(out_p[:20], out[:20])                                   # the future does not leak back
    if n_head > 1:
        assert (P.causal_attention(q, k, v, 1) - out).abs().max() > 1e-3       # heads are not one big head


def test_attention_reference_vector():
    # the analytic q, k, v of /root/reference/tests/cpp/test_flashattention.cu:15-37 (seq 37, scale 1/8)
    S, H, Dh = 37, 12, 64
    D = H * Dh
    t = torch.arange(1, S + 1, dtype=D64)[:, None]
    d = torch.arange(1, D + 1, dtype=D64)[None]
    q = 0.20 * torch.sin(0.013 * t + 0.007 * d)
    k = 0.20 * torch.cos(0.011 * (t + 1.0) - 0.005 * (d + 2.0))
    v = 0.10 * torch.sin(0.017 * (t + 2.0) + 0.003 * (d + 4.0))
    out = P.causal_attention(q, k, v, H)
    assert (out - _sdpa(q, k, v, H)).abs().max() <= 1e-4
    w = torch.softmax((q[5, :Dh] @ k[:6, :Dh].T) / 8.0, 0)                      # row 5 of head 0 by hand
    assert torch.allclose(out[5, :Dh], w @ v[:6, :Dh])


def test_window_attention():
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(20, 32, generator=g, dtype=D64) for _ in range(3))
    assert torch.allclose(P.causal_attention(q, k, v, 2, window=64), P.causal_attention(q, k, v, 2))
    w1 = P.causal_attention(q, k, v, 2, window=1)
    assert torch.allclose(w1, v)                                               # only itself
    w5 = P.causal_attention(q, k, v, 2, window=5)
    assert torch.allclose(w5[:5], P.causal_attention(q, k, v, 2)[:5]) and not torch.allclose(w5[9], P.causal_attention(q, k, v, 2)[9])


def _library_forward(cfg, w, ids):
    """The same model arranged from torch's library routines only."""
    D, H = cfg["n_embd"], cfg["n_head"]
    eps = cfg["layer_norm_epsilon"]
    approx = "tanh" if cfg["activation_function"] == "gelu_new" else "none"
    ids = torch.tensor(ids)
    x = F.embedding(ids, w["wte.weight"]) + F.embedding(torch.arange(len(ids)), w["wpe.weight"])
    for i in range(cfg["n_layer"]):
        p = f"h.{i}."
        h = F.layer_norm(x, (D,), w[p + "ln_1.weight"], w[p + "ln_1.bias"], eps)
        qkv = F.linear(h, w[p + "attn.c_attn.weight"].T, w[p + "attn.c_attn.bias"])
        a = _sdpa(*qkv.split(D, dim=1), H)
        x = x + F.linear(a, w[p + "attn.c_proj.weight"].T, w[p + "attn.c_proj.bias"])
        h = F.layer_norm(x, (D,), w[p + "ln_2.weight"], w[p + "ln_2.bias"], eps)
        h = F.gelu(F.linear(h, w[p + "mlp.c_fc.weight"].T, w[p + "mlp.c_fc.bias"]), approximate=approx)
        x = x + F.linear(h, w[p + "mlp.c_proj.weight"].T, w[p + "mlp.c_proj.bias"])
    return F.linear(F.layer_norm(x, (D,), w["ln_f.weight"], w["ln_f.bias"], eps), w["wte.weight"])


@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_model_against_library_routines(tiny_model_dirs, name):
    cfg, w = P.read_model(tiny_model_dirs[name])
    ids = torch.randint(0, cfg["vocab_size"], (29,), generator=torch.Generator().manual_seed(0)).tolist()
    mine = P.forward_logits(cfg, w, ids)
    assert mine.shape == (29, cfg["vocab_size"])
    assert (mine - _library_forward(cfg, w, ids)).abs().max() <= 1e-10
    # causality of the whole model: a later token does not change earlier logits
    ids2 = ids[:20] + [(t + 1) % cfg["vocab_size"] for t in ids[20:]]
    assert torch.equal(P.forward_logits(cfg, w, ids2)[:20], mine[:20])
    # positions count: the same token at another place gives other logits
    assert not torch.allclose(P.forward_logits(cfg, w, [ids[0], ids[0]])[1], mine[0])


def test_block_arrangement_is_pinned_by_invariants(tiny_model_dirs):
    """Where the norms and the residual sums stand, fixed by two cases that need no second arrangement
    of the whole model to compare with.

    (1) Both residual projections (attention c_proj, MLP c_proj) zero, weights and biases: every layer
        adds nothing, so logits = ln_f(embedding) wte^T. A model without the final norm, or with a norm
        ON the stream (post-norm), fails.
    (2) One layer whose attention c_proj has zero weights and a bias b: the attention sub-layer adds
        exactly b to every row, so ln_2 must see x + b (pre-norm, sequential), and the result is
        x + b + MLP(ln_2(x + b)), computed here with library routines. A parallel arrangement
        (ln_2 sees x) or a post-norm one fails."""
    cfg, w = P.read_model(tiny_model_dirs["b"])
    D, eps = cfg["n_embd"], cfg["layer_norm_epsilon"]
    ids = [7, 7, 900, 41, 3, 512, 88, 7, 19]
    emb = F.embedding(torch.tensor(ids), w["wte.weight"]) + w["wpe.weight"][:len(ids)]
    head = lambda x: F.linear(F.layer_norm(x, (D,), w["ln_f.weight"], w["ln_f.bias"], eps), w["wte.weight"])

    w1 = dict(w)
    for i in range(cfg["n_layer"]):
        for part in ("attn", "mlp"):
            w1[f"h.{i}.{part}.c_proj.weight"] = torch.zeros_like(w[f"h.{i}.{part}.c_proj.weight"])
            w1[f"h.{i}.{part}.c_proj.bias"] = torch.zeros_like(w[f"h.{i}.{part}.c_proj.bias"])
    assert (P.forward_logits(cfg, w1, ids) - head(emb)).abs().max() <= 1e-12
    assert (P.forward_logits(cfg, w, ids) - head(emb)).abs().max() > 1e-3       # the layers do count otherwise

    one = dict(cfg, n_layer=1)
    w2 = dict(w)
    w2["h.0.attn.c_proj.weight"] = torch.zeros_like(w["h.0.attn.c_proj.weight"])
    b = 0.1 * torch.sin(torch.arange(D, dtype=D64))                               # a few times the stream
    w2["h.0.attn.c_proj.bias"] = b
    x1 = emb + b
    h = F.layer_norm(x1, (D,), w["h.0.ln_2.weight"], w["h.0.ln_2.bias"], eps)
    inner = F.gelu(F.linear(h, w["h.0.mlp.c_fc.weight"].T, w["h.0.mlp.c_fc.bias"]))      # config b: the erf form
    x2 = x1 + F.linear(inner, w["h.0.mlp.c_proj.weight"].T, w["h.0.mlp.c_proj.bias"])
    got = P.forward_logits(one, w2, ids)
    assert (got - head(x2)).abs().max() <= 1e-10
    # what the wrong arrangements would give is far away
    h_par = F.layer_norm(emb, (D,), w["h.0.ln_2.weight"], w["h.0.ln_2.bias"], eps)
    par = x1 + F.linear(F.gelu(F.linear(h_par, w["h.0.mlp.c_fc.weight"].T, w["h.0.mlp.c_fc.bias"])),
                        w["h.0.mlp.c_proj.weight"].T, w["h.0.mlp.c_proj.bias"])
    assert (got - head(par)).abs().max() > 1e-2, (got - head(par)).abs().max()
    post = F.layer_norm(x1, (D,), w["h.0.ln_1.weight"], w["h.0.ln_1.bias"], eps)            # a norm on the stream
    assert (got - head(post + F.linear(inner, w["h.0.mlp.c_proj.weight"].T, w["h.0.mlp.c_proj.bias"]))).abs().max() > 1e-2


def test_parts_in_the_wrong_place_are_seen(tiny_model_dirs):
    """Post-norm instead of pre-norm, a missing final norm, an untied or biased head, a wrong
    activation: each moves the logits far beyond any tolerance the engine is held to."""
    cfg, w = P.read_model(tiny_model_dirs["b"])
    ids = list(range(3, 40, 3))
    base = P.forward_logits(cfg, w, ids)
    x = P.embedding(w["wte.weight"], w["wpe.weight"], torch.tensor(ids), torch.arange(len(ids)))
    for i in range(cfg["n_layer"]):
        x = P.block(x, w, i, cfg)
    no_final_norm = x @ w["wte.weight"].T
    assert (no_final_norm - base).abs().max() > 1e-2
    other_act = P.forward_logits(dict(cfg, activation_function="gelu_new"), w, ids)
    assert 1e-6 < (other_act - base).abs().max()
    other_eps = P.forward_logits(dict(cfg, layer_norm_epsilon=1e-2), w, ids)
    assert (other_eps - base).abs().max() > 1e-4
    fewer_heads = P.forward_logits(dict(cfg, n_head=1), w, ids)
    assert (fewer_heads - base).abs().max() > 1e-4


def test_tied_head_and_greedy_tie_break(tiny_model_dirs):
    cfg, w = P.read_model(tiny_model_dirs["a"])
    hidden = torch.randn(2, cfg["n_embd"], dtype=D64, generator=torch.Generator().manual_seed(1))
    w2 = dict(w)
    w2["wte.weight"] = torch.cat([w["wte.weight"], w["wte.weight"][7:8]])       # one more row, a copy of row 7
    l1, l2 = P.logits_head(hidden, w, cfg), P.logits_head(hidden, w2, cfg)
    assert torch.equal(l2[:, :-1], l1) and torch.equal(l2[:, -1], l1[:, 7])
    # greedy takes the lowest index on ties (/root/reference/src/kernels/argmax.cu:12-20)
    row = torch.tensor([0.0, 2.0, 2.0, 1.0])
    assert int(torch.nonzero(row == row.max())[0]) == 1
