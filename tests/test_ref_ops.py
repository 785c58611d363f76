"""The plain C++ twins of the device operations (csrc/ref/ref_ops.cc) against the plain Python references
and against library routines: two independent statements of every operation's meaning agree, so either can
stand as a kernel's oracle."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_ops
import ref_ops


def test_embed_and_layernorm():
    g = torch.Generator().manual_seed(0)
    wte, wpe = torch.randn(50, 24, generator=g), torch.randn(16, 24, generator=g)
    ids, pos = torch.tensor([3, 5, 7, 5, 11]), torch.tensor([0, 1, 2, 9, 15])
    assert torch.equal(ref_ops.embed(ids, pos, wte, wpe), wte[ids] + wpe[pos])
    assert torch.equal(ref_ops.embed(ids, None, wte, None), wte[ids])
    x = torch.randn(9, 100, generator=g) * 3 + 1
    gamma, beta = torch.randn(100, generator=g), torch.randn(100, generator=g)
    for eps in (1e-5, 1e-2):
        assert (ref_ops.layernorm(x, gamma, beta, eps) - F.layer_norm(x.double(), (100,), gamma.double(), beta.double(), eps)).abs().max() <= 1e-6
    rows = torch.tensor([8, 0, 3])
    assert torch.equal(ref_ops.layernorm(x, gamma, None, 1e-5, rows), ref_ops.layernorm(x[rows], gamma, None, 1e-5))


@pytest.mark.parametrize("epi", ["store", "gelu_tanh", "gelu_erf", "add_residual", "store_f32"])
def test_linear_and_its_epilogues(epi):
    g = torch.Generator().manual_seed(1)
    a, w, b = torch.randn(9, 73, generator=g), torch.randn(37, 73, generator=g) / math.sqrt(73), torch.randn(37, generator=g)
    out0 = torch.randn(9, 37, generator=g)
    got = ref_ops.linear(a, w, b, out0, epi)
    want = plain_ops.linear(a, w, b, out0.double().clone(), epi)
    assert (got.double() - want).abs().max() <= 1e-6
    lib = {"store": lambda y: y, "store_f32": lambda y: y, "gelu_tanh": lambda y: F.gelu(y, approximate="tanh"),
           "gelu_erf": F.gelu, "add_residual": lambda y: y + out0.double()}[epi]
    assert (got.double() - lib(F.linear(a.double(), w.double(), b.double()))).abs().max() <= 1e-6


def test_pages_and_attention():
    g = torch.Generator().manual_seed(2)
    H, Hkv, dh, page = 6, 2, 16, 4
    seqs = [(0, 9), (5, 1), (3, 6)]                       # (tokens cached before, new tokens)
    ctx = [s + n for s, n in seqs]
    nblk = [-(-c // page) for c in ctx]
    perm = torch.randperm(sum(nblk) + 2, generator=g).tolist()
    tables = torch.zeros(3, max(nblk), dtype=torch.int32)
    kp = torch.full(((sum(nblk) + 2) * page, Hkv * dh), float("nan"))
    vp = kp.clone()
    T = sum(n for _, n in seqs)
    q = torch.randn(T, H * dh + 8, generator=g)
    token_seq, positions, used = [], [], 0
    for b, (s, n) in enumerate(seqs):
        for j in range(nblk[b]):
            tables[b, j] = perm[used]
            used += 1
        js = torch.arange(ctx[b])
        rows = tables[b].long()[js // page] * page + js % page
        kp[rows], vp[rows] = torch.randn(ctx[b], Hkv * dh, generator=g), torch.randn(ctx[b], Hkv * dh, generator=g)
        token_seq += [b] * n
        positions += list(range(s, s + n))
    token_seq, positions = torch.tensor(token_seq, dtype=torch.int32), torch.tensor(positions, dtype=torch.int32)
    for window in (0, 3):
        got = ref_ops.paged_attention(q, 8, H, Hkv, dh, kp, vp, page, tables, token_seq, positions, dh ** -0.5, window)
        want = torch.zeros(T, H * dh, dtype=torch.float64)
        plain_ops.paged_attention(q, 8, H, Hkv, dh, kp, vp, page, tables, token_seq, positions, dh ** -0.5, window, want)
        assert (got.double() - want).abs().max() <= 1e-6
    # the first sequence alone, no window: the library's causal attention (grouped heads expanded)
    k0 = kp[tables[0].long()[torch.arange(9) // page] * page + torch.arange(9) % page]
    v0 = vp[tables[0].long()[torch.arange(9) // page] * page + torch.arange(9) % page]
    rep = H // Hkv
    ex = lambda t: t.view(9, Hkv, 1, dh).expand(9, Hkv, rep, dh).reshape(9, H, dh).transpose(0, 1)
    lib = F.scaled_dot_product_attention(q[:9, 8:].view(9, H, dh).transpose(0, 1).double(), ex(k0).double(), ex(v0).double(),
                                         is_causal=True).transpose(0, 1).reshape(9, H * dh)
    got = ref_ops.paged_attention(q, 8, H, Hkv, dh, kp, vp, page, tables, token_seq, positions, dh ** -0.5, 0)
    assert (got[:9].double() - lib).abs().max() <= 1e-6
    # the page write
    src = torch.randn(4, 3 * Hkv * dh, generator=g)
    slots = torch.tensor([5, -1, 0, 9], dtype=torch.int32)
    k1, v1 = torch.zeros(12, Hkv * dh), torch.zeros(12, Hkv * dh)
    k2, v2 = k1.clone(), v1.clone()
    ref_ops.kv_append(src, Hkv * dh, 2 * Hkv * dh, Hkv * dh, k1, v1, slots)
    plain_ops.kv_append(src, Hkv * dh, 2 * Hkv * dh, Hkv * dh, k2, v2, slots)
    assert torch.equal(k1, k2) and torch.equal(v1, v2) and k1[1].abs().sum() == 0


def test_token_choice():
    row = torch.tensor([[0.0, 2.0, 2.0, 1.0], [5.0, 5.0, 5.0, 5.0], [-1.0, -3.0, -0.5, -0.5]])
    assert ref_ops.argmax(row).tolist() == [1, 0, 2]                    # the lowest index on ties
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(6, 1000, generator=g) * 2
    temp = torch.tensor([0.0, 0.7, 1.0, 1.3, 0.2, 5.0])
    u = torch.tensor([0.3, 0.0, 0.999, 0.5, 0.25, 0.75])
    want = torch.empty(6, dtype=torch.int32)
    plain_ops.sample(logits, temp, u, want)
    assert torch.equal(ref_ops.sample(logits, temp, u), want)
    assert ref_ops.sample(logits, temp, u)[0] == logits[0].argmax()


def test_unfused_epilogues():
    # the reference's vector for its GELU: x = 0.01 i, 1027 values, tolerance 1e-5 (/root/reference/tests/kernels/gelu/gen.py:5-12)
    x = 0.01 * torch.arange(1027, dtype=torch.float32) - 5.0
    assert (ref_ops.gelu(x) - F.gelu(x.double(), approximate="tanh")).abs().max() <= 1e-6
    assert (ref_ops.gelu(x, exact=True) - F.gelu(x.double())).abs().max() <= 1e-6
    assert (ref_ops.gelu(x) - ref_ops.gelu(x, exact=True)).abs().max() > 1e-4          # the two forms are told apart
    g = torch.Generator().manual_seed(4)
    a, b, bias = torch.randn(5, 7, generator=g), torch.randn(5, 7, generator=g), torch.randn(7, generator=g)
    assert torch.equal(ref_ops.add_bias(a, bias), a + bias) and torch.equal(ref_ops.residual_add(a, b), a + b)
    # the fused epilogue of the product is these, one after the other
    w = torch.randn(7, 7, generator=g)
    fused = ref_ops.linear(a, w, bias, None, "gelu_tanh")
    assert (fused - ref_ops.gelu(ref_ops.add_bias(ref_ops.linear(a, w, None), bias))).abs().max() <= 1e-6
