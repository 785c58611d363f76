"""Each HIP kernel alone against its plain reference (tests/plain_ops.py), at sizes other
than the engine's tiny models: widths and vocabularies that are no power of two,
ragged row counts, several head sizes and group counts."""
import math

import pytest
import torch

import plain_ops
import ref_ops

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from mini_llm_amd.kernels import ops as o
    return o


def _tol(dtype, scale=1.0):
    return (2e-5 if dtype == torch.float32 else 1.6e-2) * scale


def _rand(shape, dtype, gen, std=1.0):
    return (torch.randn(shape, generator=gen, dtype=torch.float32) * std).to(dtype)


def test_loaded_libraries_are_in_tree(ops):
    """After an op has run, the native code mapped into this process is the in-tree build: the engine
    library and the kernel libraries it links, all from the package's own folder and nowhere else."""
    import os
    from mini_llm_amd import build
    out = torch.empty(2, dtype=torch.int32, device=DEV)
    ops.argmax(torch.tensor([[0.0, 2.0, 1.0], [3.0, 2.0, 1.0]], device=DEV), out)
    assert out.tolist() == [1, 0]
    with open("/proc/self/maps") as f:
        mapped = {line.split()[-1] for line in f if "libmllm_" in line}
    names = {os.path.basename(m) for m in mapped}
    for lib in ("engine", "elementwise", "gemm_bf16", "gemm_f32", "attention_decode", "attention_prefill", "sampling"):
        assert os.path.basename(build.lib_path(lib)) in names, (lib, names)
    here = os.path.realpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "_lib"))     # the tests' own
    assert all(os.path.dirname(os.path.realpath(m)) in (os.path.realpath(build.LIB_DIR), here) for m in mapped), mapped


def test_lane_exchange_between_rows(ops):
    """The reductions over one lane of each 16-lane row (built on gfx950's row swaps) against their meaning."""
    import ctypes
    import toy  # noqa: F401  (registers the test-only library)
    from mini_llm_amd import build
    lib = build.load_library("lane_check")
    g = torch.Generator().manual_seed(3)
    v = torch.randn(64, generator=g)
    out = torch.zeros(384, device=DEV)
    rc = lib.mllm_rows_check(ctypes.c_void_p(v.to(DEV).data_ptr()), ctypes.c_void_p(out.data_ptr()),
                             ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    groups = v.view(4, 16)
    assert torch.equal(out[:64].cpu().view(4, 16), groups.max(0).values.expand(4, 16))
    want = (groups[0] + groups[1]) + (groups[2] + groups[3])
    assert torch.equal(out[64:128].cpu().view(4, 16), want.expand(4, 16))
    lanes = torch.arange(64)
    for i, off in enumerate((8, 16, 32, 4)):
        assert torch.equal(out[128 + 64 * i:192 + 64 * i].cpu(), v[lanes ^ off]), off


def test_ops_refuse_cpu_tensors(ops):
    x = torch.zeros(2, 8)
    with pytest.raises(ops.KernelError, match="not on the GPU"):
        ops.layernorm(x, torch.ones(8), None, 1e-5, torch.empty(2, 8))


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_reference_vector(ops, dtype):
    # /root/reference/tests/kernels/embedding/gen.py:13-27
    V, P, D = 64, 32, 768
    wte = (torch.arange(V)[:, None] * 0.01 + torch.arange(D)[None, :] * 0.0001).to(dtype)
    wpe = (torch.arange(P)[:, None] * 0.001 + torch.arange(D)[None, :] * 0.00001).to(dtype)
    ids = torch.tensor([3, 5, 7, 5, 11, 13, 17], dtype=torch.int32)
    pos = torch.arange(7, dtype=torch.int32)
    out = torch.empty(7, D, dtype=torch.float32, device=DEV)
    ops.embed(ids.to(DEV), pos.to(DEV), wte.to(DEV), wpe.to(DEV), out)
    ref = wte[ids.long()].float() + wpe[pos.long()].float()
    assert (out.cpu() - ref).abs().max() <= 1e-6
    # without a position table
    ops.embed(ids.to(DEV), None, wte.to(DEV), None, out)
    assert torch.equal(out.cpu(), wte[ids.long()].float())
    # tokens taken on the device from what an earlier step sampled: rows 1, 4 and 6 (a source beyond the
    # sampled tokens is ignored, as by select_tokens)
    src = torch.tensor([-1, 2, -1, -1, 0, 9, 1], dtype=torch.int32)
    prev = torch.tensor([60, 61, 62], dtype=torch.int32)
    ops.embed(ids.to(DEV), pos.to(DEV), wte.to(DEV), wpe.to(DEV), out, src=src.to(DEV), prev=prev.to(DEV))
    fed = torch.tensor([3, 62, 7, 5, 60, 13, 61])
    assert (out.cpu() - (wte[fed].float() + wpe[pos.long()].float())).abs().max() <= 1e-6
    want = plain_ops.embed(ids, pos, wte, wpe, torch.empty(7, D, dtype=torch.float64), src=src, prev=prev)
    assert (out.cpu().double() - want).abs().max() <= 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,D,eps", [(17, 768, 1e-5), (5, 100, 1e-6), (3, 1600, 1e-5), (1, 16, 1e-3),
                                        (2050, 768, 1e-5), (6, 2048, 1e-5), (5, 2052, 1e-5), (4, 98, 1e-6)])
def test_layernorm(ops, dtype, rows, D, eps):
    g = torch.Generator().manual_seed(0)
    x = _rand((rows, D), torch.float32, g) + 0.5
    gamma = 1 + 0.1 * _rand((D,), torch.float32, g)
    beta = 0.1 * _rand((D,), torch.float32, g)
    out = torch.empty(rows, D, dtype=dtype, device=DEV)
    ops.layernorm(x.to(DEV), gamma.to(DEV), beta.to(DEV), eps, out)
    ref = plain_ops.layernorm(x, gamma, beta, eps, torch.empty(rows, D, dtype=torch.float64))
    assert (out.cpu().double() - ref).abs().max() <= _tol(dtype, 4)
    # selected rows, no bias
    sel = torch.tensor([rows - 1, 0], dtype=torch.int32)
    out2 = torch.empty(2, D, dtype=dtype, device=DEV)
    ops.layernorm(x.to(DEV), gamma.to(DEV), None, eps, out2, rows=sel.to(DEV))
    ref2 = plain_ops.layernorm(x, gamma, None, eps, torch.empty(2, D, dtype=torch.float64), rows=sel)
    assert (out2.cpu().double() - ref2).abs().max() <= _tol(dtype, 4)


def test_layernorm_constant_row_gives_beta(ops):
    D = 96
    x = torch.full((2, D), 3.25)
    beta = torch.linspace(-1, 1, D)
    out = torch.empty(2, D, dtype=torch.float32, device=DEV)
    ops.layernorm(x.to(DEV), torch.ones(D, device=DEV), beta.to(DEV), 1e-6, out)
    assert (out.cpu() - beta).abs().max() <= 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(67, 79, 40), (5, 2304, 768), (1, 1000, 96), (130, 320, 96),
                                   (9, 73, 320), (200, 50257, 64), (33, 96, 3072), (257, 257, 264),
                                   (300, 4800, 1600), (100, 1600, 6400)])
@pytest.mark.parametrize("epi", ["store", "gelu_tanh", "gelu_erf", "add_residual", "store_f32"])
def test_linear(ops, dtype, M, N, K, epi):
    if N == 50257 and epi not in ("store_f32", "store"):
        pytest.skip("the wide case is the logits head")
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    a = _rand((M, K), dtype, g)
    w = _rand((N, K), dtype, g, std=1.0 / math.sqrt(K))
    bias = 0.5 * _rand((N,), torch.float32, g)
    f32_out = epi in ("add_residual", "store_f32")
    out0 = _rand((M, N), torch.float32 if f32_out else dtype, g)
    out = out0.clone().to(DEV)
    ops.linear(a.to(DEV), w.to(DEV), bias.to(DEV), out, epi)
    ref = plain_ops.linear(a, w, bias, out0.double().clone(), epi)
    err = (out.cpu().double() - ref).abs().max().item()
    tol = 3e-5 if dtype == torch.float32 else (2e-5 + 2e-5 * math.sqrt(K) if f32_out else 4e-2)
    assert err <= tol, (err, tol)
    # no bias, strided input rows
    a2 = _rand((M, K + 8), dtype, g).to(DEV)[:, :K]
    out = out0.clone().to(DEV)
    ops.linear(a2, w.to(DEV), None, out, epi)
    ref = plain_ops.linear(a2.cpu(), w, None, out0.double().clone(), epi)
    assert (out.cpu().double() - ref).abs().max().item() <= tol


@pytest.mark.parametrize("M,N,K", [(2000, 2300, 776),      # 128x192 tiles, one round, ragged in M, N and K
                                   (2048, 3072, 768),      # 128x192 tiles, no edge
                                   (2900, 3000, 72),       # 128x192 tiles, two rounds, ragged
                                   (2040, 4090, 136),      # 128x256 tiles, ragged
                                   (2040, 1800, 200),      # 128x128 tiles, one round, ragged
                                   (2040, 1000, 200),      # 64x128 tiles, ragged
                                   (2040, 760, 136),       # 64x96 tiles, one round, ragged
                                   (2048, 768, 3072),      # 64x96 tiles, long K: two wavefront groups per workgroup
                                   (2040, 1800, 2056),     # 128x128 tiles, two groups, K not a multiple of their k tile
                                   (1000, 1000, 2056),     # 64x64 tiles, two groups, ragged
                                   (300, 500, 4104),       # 64x32 tiles (few workgroups), long ragged K
                                   (1000, 1000, 40),       # 64x64 tiles, K below one k tile
                                   (257, 257, 264)])       # 64x32 tiles, few workgroups
@pytest.mark.parametrize("epi", ["store", "add_residual"])
def test_linear_bf16_tile_choices(ops, M, N, K, epi):
    """Every tile shape of the many-row product, with edges in all three dimensions."""
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K)
    a = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, std=1.0 / math.sqrt(K))
    bias = 0.5 * _rand((N,), torch.float32, g)
    f32_out = epi == "add_residual"
    out0 = _rand((M, N), torch.float32 if f32_out else torch.bfloat16, g)
    out = out0.clone().to(DEV)
    ops.linear(a.to(DEV), w.to(DEV), bias.to(DEV), out, epi)
    ref = plain_ops.linear(a, w, bias, out0.double().clone(), epi)
    err = (out.cpu().double() - ref).abs().max().item()
    assert err <= (2e-5 + 2e-5 * math.sqrt(K) if f32_out else 4e-2), err


@pytest.mark.parametrize("M,H,Hkv,dh,K", [(2048, 12, 12, 64, 768),      # 128x192 tiles
                                          (300, 6, 2, 16, 96),         # 64x64 tiles, ragged, grouped heads
                                          (70, 3, 3, 48, 144),         # just above the few-row kernel
                                          (1000, 16, 4, 32, 520)])
def test_linear_bf16_scatters_keys_and_values(ops, M, H, Hkv, dh, K):
    """The fused QKV product with the page write in its epilogue: output as without, and the key
    and value columns of every row with a slot arrive in that row of the pages, nothing else."""
    g = torch.Generator().manual_seed(M + K)
    q_cols, kv_dim = H * dh, Hkv * dh
    N = q_cols + 2 * kv_dim
    a = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, std=1.0 / math.sqrt(K))
    bias = 0.5 * _rand((N,), torch.float32, g)
    rows = M + 37
    perm = torch.randperm(rows, generator=g)[:M].to(torch.int32)
    perm[::7] = -1                                   # rows that write nothing
    k0 = _rand((rows, kv_dim), torch.bfloat16, g)
    v0 = _rand((rows, kv_dim), torch.bfloat16, g)
    kp, vp = k0.clone().to(DEV), v0.clone().to(DEV)
    out = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    ops.linear(a.to(DEV), w.to(DEV), bias.to(DEV), out, "store", kv_scatter=(perm.to(DEV), kp, vp, q_cols))
    plain = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    ops.linear(a.to(DEV), w.to(DEV), bias.to(DEV), plain, "store")
    if M > 256:
        assert torch.equal(out, plain)               # the same kernel with and without the page write
    else:                                            # without, fewer rows may take the weight-streaming kernel
        assert (out.float() - plain.float()).abs().max().item() <= 4e-2
    ref = plain_ops.linear(a, w, bias, torch.empty((M, N), dtype=torch.float64))
    assert (out.cpu().double() - ref).abs().max().item() <= 4e-2
    kr, vr = k0.clone(), v0.clone()
    plain_ops.kv_append(out.cpu(), q_cols, q_cols + kv_dim, kv_dim, kr, vr, perm)
    assert torch.equal(kp.cpu(), kr) and torch.equal(vp.cpu(), vr)
    # few rows: the product's kernel has no such epilogue and a copy kernel follows it; same contract
    kp8, vp8 = k0.clone().to(DEV), v0.clone().to(DEV)
    ops.linear(a[:8].to(DEV), w.to(DEV), bias.to(DEV), out[:8], "store", kv_scatter=(perm[:8].to(DEV), kp8, vp8, q_cols))
    kr, vr = k0.clone(), v0.clone()
    plain_ops.kv_append(out[:8].cpu(), q_cols, q_cols + kv_dim, kv_dim, kr, vr, perm[:8])
    assert torch.equal(kp8.cpu(), kr) and torch.equal(vp8.cpu(), vr)
    with pytest.raises(ops.KernelError, match="scatter"):
        ops.linear(a.to(DEV), w.to(DEV), None, torch.empty((M, N), dtype=torch.float32, device=DEV), "store_f32",
                   kv_scatter=(perm.to(DEV), kp, vp, q_cols))


@pytest.mark.parametrize("M,H,Hkv,dh,K", [(65, 12, 12, 64, 768), (256, 25, 25, 64, 1600), (100, 6, 2, 32, 200), (8, 4, 4, 16, 64),
                                          (64, 12, 12, 64, 768), (300, 3, 3, 32, 96)])
def test_ln_linear_scatters_keys_and_values(ops, M, H, Hkv, dh, K):
    """The norm, the QKV product and the page write in one call: the output of the norm followed by the
    product, and the key and value columns in their slots."""
    g = torch.Generator().manual_seed(M + K)
    q_cols, kv_dim = H * dh, Hkv * dh
    N = q_cols + 2 * kv_dim
    x = _rand((M, K), torch.float32, g, std=2.0) + 0.3
    gamma, beta = 1 + 0.1 * _rand((K,), torch.float32, g), 0.1 * _rand((K,), torch.float32, g)
    w = _rand((N, K), torch.bfloat16, g, std=1.0 / math.sqrt(K))
    bias = 0.5 * _rand((N,), torch.float32, g)
    rows = M + 37
    slots = torch.randperm(rows, generator=g)[:M].to(torch.int32)
    slots[::7] = -1
    k0, v0 = _rand((rows, kv_dim), torch.bfloat16, g), _rand((rows, kv_dim), torch.bfloat16, g)
    kp, vp = k0.clone().to(DEV), v0.clone().to(DEV)
    out = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    ops.ln_linear(x.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5, w.to(DEV), bias.to(DEV), out, "store",
                  kv_scatter=(slots.to(DEV), kp, vp, q_cols))
    h = plain_ops.layernorm(x, gamma, beta, 1e-5, torch.empty(M, K, dtype=torch.bfloat16))
    ref = plain_ops.linear(h, w, bias, torch.empty((M, N), dtype=torch.float64))
    assert (out.cpu().double() - ref).abs().max().item() <= 4e-2
    kr, vr = k0.clone(), v0.clone()
    plain_ops.kv_append(out.cpu(), q_cols, q_cols + kv_dim, kv_dim, kr, vr, slots)
    assert torch.equal(kp.cpu(), kr) and torch.equal(vp.cpu(), vr)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 48, 64])
@pytest.mark.parametrize("N,K", [(2304, 768), (768, 3072), (1000, 96), (50257, 768), (72, 1600), (4800, 1600),
                                 (1600, 6400), (1024, 4096),
                                 # more than 256 tiles of 16 columns: two tiles per workgroup, the second narrower
                                 (4104, 72), (6400, 1600), (8190, 200)])
def test_linear_bf16_few_rows(ops, M, N, K):
    """The weight-streaming kernel of decode steps (M <= 64), every wavefront count and m-tile count."""
    g = torch.Generator().manual_seed(M + N + K)
    a = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, std=1.0 / math.sqrt(K))
    bias = 0.5 * _rand((N,), torch.float32, g)
    for epi in ("store_f32", "add_residual", "gelu_tanh"):
        f32_out = epi != "gelu_tanh"
        out0 = _rand((M, N), torch.float32 if f32_out else torch.bfloat16, g)
        out = out0.clone().to(DEV)
        ops.linear(a.to(DEV), w.to(DEV), bias.to(DEV), out, epi)
        ref = plain_ops.linear(a, w, bias, out0.double().clone(), epi)
        err = (out.cpu().double() - ref).abs().max().item()
        assert err <= (2e-5 + 2e-5 * math.sqrt(K) if f32_out else 4e-2), (epi, err)


@pytest.mark.parametrize("M,N,K", [(65, 768, 768), (96, 2304, 768), (100, 1000, 96), (128, 768, 3072), (200, 72, 1600),
                                   (256, 768, 768), (256, 1024, 4096), (250, 40, 6400), (129, 2304, 768), (64, 6400, 1600)])
def test_linear_bf16_up_to_256_rows(ops, M, N, K):
    """Between 65 and 256 rows the weight-streaming kernel (many 16-row blocks) or the tiled kernel
    runs, by the number of workgroups the former would need."""
    g = torch.Generator().manual_seed(M + N + K)
    a = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, std=1.0 / math.sqrt(K))
    bias = 0.5 * _rand((N,), torch.float32, g)
    for epi in ("store", "add_residual", "gelu_erf"):
        f32_out = epi == "add_residual"
        out0 = _rand((M, N), torch.float32 if f32_out else torch.bfloat16, g)
        out = out0.clone().to(DEV)
        ops.linear(a.to(DEV), w.to(DEV), bias.to(DEV), out, epi)
        ref = plain_ops.linear(a, w, bias, out0.double().clone(), epi)
        err = (out.cpu().double() - ref).abs().max().item()
        assert err <= (2e-5 + 2e-5 * math.sqrt(K) if f32_out else 4e-2), (epi, err)


@pytest.mark.parametrize("M,N,K", [(8, 1600, 6400), (1, 1280, 5120), (16, 72, 8192), (5, 200, 5192), (32, 40, 6400),
                                   (64, 24, 5128)])
def test_linear_bf16_few_rows_long_k_shares_tiles(ops, M, N, K):
    """Narrow products with a long K: several workgroups share a tile and the last to arrive adds their
    parts. Every call gives the same bits (the parts are added in a fixed order, the counters are
    left at zero), on any stream."""
    g = torch.Generator().manual_seed(M + N + K)
    a = _rand((M, K), torch.bfloat16, g).to(DEV)
    w = _rand((N, K), torch.bfloat16, g, std=1.0 / math.sqrt(K)).to(DEV)
    bias = (0.5 * _rand((N,), torch.float32, g)).to(DEV)
    x0 = _rand((M, N), torch.float32, g)
    ref = plain_ops.linear(a.cpu(), w.cpu(), bias.cpu(), x0.double().clone(), "add_residual")
    outs = []
    for _ in range(3):
        x = x0.clone().to(DEV)
        ops.linear(a, w, bias, x, "add_residual")
        outs.append(x.cpu())
    assert (outs[0].double() - ref).abs().max().item() <= 2e-5 + 2e-5 * math.sqrt(K)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    # another epilogue between two runs, and a second stream with scratch of its own: the same bits again
    y = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.linear(a, w, bias, y, "gelu_tanh")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        x = x0.clone().to(DEV)
        ops.linear(a, w, bias, x, "add_residual")
        assert ops.scratch_address("gemm_workspace") != 0
    side.synchronize()
    assert torch.equal(x.cpu(), outs[0])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 2304, 768), (8, 3072, 768), (16, 320, 96), (5, 200, 1600), (17, 96, 64),
                                   (3, 64, 4096), (16, 6400, 1600), (9, 50257, 1024), (16, 3072, 1024), (33, 2304, 768),
                                   (64, 50257, 768), (64, 104, 1600), (65, 96, 64),
                                   # more than 256 tiles: two per workgroup
                                   (8, 4800, 1600), (3, 4104, 72), (16, 8190, 200),
                                   # more than 32 rows: the norm runs as a kernel of its own
                                   (64, 3072, 768), (48, 4096, 1024), (50, 136, 200), (100, 320, 96), (200, 4800, 1600),
                                   (256, 3072, 776), (17, 40, 72), (31, 1000, 2048), (300, 320, 96)])
@pytest.mark.parametrize("epi", ["store", "gelu_tanh", "gelu_erf", "store_f32"])
def test_ln_linear(ops, dtype, M, N, K, epi):
    """LayerNorm fused into the product (bf16, few rows) and its unfused form give the plain result."""
    g = torch.Generator().manual_seed(M * 7 + N + K)
    x = _rand((M, K), torch.float32, g, std=2.0) + 0.3
    gamma = 1 + 0.1 * _rand((K,), torch.float32, g)
    beta = 0.1 * _rand((K,), torch.float32, g)
    w = _rand((N, K), dtype, g, std=1.0 / math.sqrt(K))
    bias = 0.5 * _rand((N,), torch.float32, g)
    odt = torch.float32 if epi == "store_f32" else dtype
    out = torch.zeros(M, N, dtype=odt, device=DEV)
    ops.ln_linear(x.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5, w.to(DEV), bias.to(DEV), out, epi)
    h = plain_ops.layernorm(x, gamma, beta, 1e-5, torch.empty(M, K, dtype=dtype))     # rounded as the kernel rounds
    ref = plain_ops.linear(h, w, bias, torch.zeros(M, N, dtype=torch.float64), epi)
    tol = 3e-5 if dtype == torch.float32 else (2e-2 if epi == "store_f32" else 4e-2)
    assert (out.cpu().double() - ref).abs().max().item() <= tol
    # no bias, rows gathered in another order
    sel = torch.tensor(list(range(M - 1, -1, -1)), dtype=torch.int32)
    out2 = torch.zeros(M, N, dtype=odt, device=DEV)
    ops.ln_linear(x.to(DEV), gamma.to(DEV), None, 1e-5, w.to(DEV), None, out2, epi, rows=sel.to(DEV))
    h = plain_ops.layernorm(x, gamma, None, 1e-5, torch.empty(M, K, dtype=dtype), rows=sel)
    ref = plain_ops.linear(h, w, None, torch.zeros(M, N, dtype=torch.float64), epi)
    assert (out2.cpu().double() - ref).abs().max().item() <= tol


def test_linear_fp32_is_true_fp32(ops):
    """Values that bf16 or tf32 inputs would destroy: 1 + 2^-20 differs from 1 only in true fp32."""
    K = 64
    a = torch.ones(4, K)
    a[:, 0] = 1 + 2.0 ** -20
    w = torch.zeros(3, K)
    w[0, 0], w[0, 1] = 1.0, -1.0
    out = torch.empty(4, 3, device=DEV)
    ops.linear(a.to(DEV), w.to(DEV), None, out, "store")
    assert out[0, 0].item() == 2.0 ** -20


@pytest.mark.parametrize("M,N,K,pad", [(5, 70, 42, 0),        # K no multiple of 4: the tiled kernel
                                         (7, 33, 1028, 3),      # row strides no multiple of 4 floats
                                         (8, 50257, 64, 0),     # the few-row kernel, one pass, wide
                                         (64, 130, 1600, 0),    # four passes of 16 rows, k chunks with a rest
                                         (17, 5, 8, 4)])        # fewer columns than a workgroup has wavefronts
def test_linear_fp32_few_rows(ops, M, N, K, pad):
    """The 32-bit product of few rows streams the weights, one column per wavefront, where the operands
    are 16-byte aligned, and falls back to the tiled kernel where they are not."""
    g = torch.Generator().manual_seed(M + N + K)
    a = _rand((M, K + pad), torch.float32, g).to(DEV)[:, :K]
    w = _rand((N, K + pad), torch.float32, g, std=1.0 / math.sqrt(K)).to(DEV)[:, :K]
    bias = 0.5 * _rand((N,), torch.float32, g)
    for epi in ("store", "add_residual", "gelu_tanh"):
        out0 = _rand((M, N), torch.float32, g)
        out = out0.clone().to(DEV)
        ops.linear(a, w, bias.to(DEV), out, epi)
        ref = plain_ops.linear(a.cpu(), w.cpu(), bias, out0.double().clone(), epi)
        assert (out.cpu().double() - ref).abs().max().item() <= 3e-5


def test_linear_bf16_refuses_odd_k(ops):
    a = torch.zeros(4, 36, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(8, 36, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.KernelError, match="multiples of 8"):
        ops.linear(a, w, None, torch.empty(4, 8, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("dtype", DTYPES)
def test_kv_append_reference_vector(ops, dtype):
    # /root/reference/tests/kernels/append_kv/gen.py:12-24: blocks [3,3,7,7,7,9], offsets [0,1,0,1,2,4]
    D, BS, NB = 768, 16, 12
    blocks = torch.tensor([3, 3, 7, 7, 7, 9])
    offs = torch.tensor([0, 1, 0, 1, 2, 4])
    qkv = torch.zeros(6, 3 * D)
    for t in range(6):
        for part, base in enumerate((10000, 20000, 30000)):
            qkv[t, part * D:(part + 1) * D] = (base + t * 100 + torch.arange(D)) / 64.0
    qkv = qkv.to(dtype)
    kp = torch.full((NB * BS, D), -1.0, dtype=dtype, device=DEV)
    vp = torch.full((NB * BS, D), -1.0, dtype=dtype, device=DEV)
    slots = (blocks * BS + offs).to(torch.int32)
    slots_skip = torch.cat([slots, torch.tensor([-1], dtype=torch.int32)])
    src = torch.cat([qkv, torch.ones(1, 3 * D, dtype=dtype)])
    ops.kv_append(src.to(DEV), D, 2 * D, D, kp, vp, slots_skip.to(DEV))
    assert torch.equal(kp.cpu()[slots.long()], qkv[:, D:2 * D])
    assert torch.equal(vp.cpu()[slots.long()], qkv[:, 2 * D:])
    untouched = torch.ones(NB * BS, dtype=torch.bool)
    untouched[slots.long()] = False
    assert (kp.cpu()[untouched] == -1).all() and (vp.cpu()[untouched] == -1).all()


def _attention_case(ops, dtype, H, Hkv, dh, page, seqs, window, gen, boost=None, n_single=0):
    """seqs: list of (start, q_len). Builds pages in scrambled order, garbage elsewhere."""
    B = len(seqs)
    ctx = [s + n for s, n in seqs]
    nblk = [-(-c // page) for c in ctx]
    n_pages = sum(nblk) + 3
    perm = torch.randperm(n_pages, generator=gen).tolist()
    kv_dim = Hkv * dh
    kp = torch.full((n_pages * page, kv_dim), float("nan"), dtype=dtype)
    vp = torch.full((n_pages * page, kv_dim), float("nan"), dtype=dtype)
    tables = torch.zeros(B, max(nblk), dtype=torch.int32)
    T = sum(n for _, n in seqs)
    q = _rand((T, H * dh + 16), dtype, gen)
    token_seq, positions = [], []
    used = 0
    for b, (s, n) in enumerate(seqs):
        for j in range(nblk[b]):
            tables[b, j] = perm[used]
            used += 1
        k = _rand((ctx[b], kv_dim), dtype, gen)
        v = _rand((ctx[b], kv_dim), dtype, gen)
        if boost is not None and ctx[b] > boost[0]:
            # one far key stands out: its score dominates for the last query
            far = boost[0]
            k[far] = k[far] * 0 + (q[len(token_seq) + n - 1, 8:8 + H * dh].float().view(H, dh)[::H // Hkv]
                                   .reshape(-1) * boost[1]).to(dtype)
        js = torch.arange(ctx[b])
        rows = tables[b].long()[js // page] * page + js % page
        kp[rows] = k
        vp[rows] = v
        token_seq += [b] * n
        positions += list(range(s, s + n))
    token_seq = torch.tensor(token_seq, dtype=torch.int32)
    positions = torch.tensor(positions, dtype=torch.int32)
    scale = dh ** -0.5
    out = torch.zeros(T, H * dh, dtype=dtype, device=DEV)
    cu = torch.tensor([0] + list(torch.tensor([n for _, n in seqs]).cumsum(0)), dtype=torch.int32)
    ops.paged_attention(q.to(DEV), 8, H, Hkv, dh, kp.to(DEV), vp.to(DEV), page, tables.to(DEV),
                        token_seq.to(DEV), positions.to(DEV), scale, window, out,
                        cu_q=cu.to(DEV), ctx_len=torch.tensor(ctx, dtype=torch.int32).to(DEV),
                        max_q_len=max(n for _, n in seqs), max_ctx_len=max(ctx), n_single=n_single)
    ref = torch.zeros(T, H * dh, dtype=torch.float64)
    plain_ops.paged_attention(q, 8, H, Hkv, dh, kp, vp, page, tables, token_seq, positions, scale, window, ref)
    if sum(c * n for c, (_, n) in zip(ctx, seqs)) * H * dh <= 2e8:
        # the second oracle, the plain C++ twin, says the same
        twin = ref_ops.paged_attention(q, 8, H, Hkv, dh, kp, vp, page, tables, token_seq, positions, scale, window)
        assert (twin.double() - ref).abs().max() <= 2e-6
    return out.cpu().double(), ref


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,dh,page", [(12, 12, 64, 16), (4, 4, 16, 4), (3, 3, 32, 8), (6, 2, 48, 16),
                                           (5, 1, 128, 32), (2, 2, 256, 64)])
def test_paged_attention_mixed_batch(ops, dtype, H, Hkv, dh, page):
    g = torch.Generator().manual_seed(H * 100 + dh)
    seqs = [(0, 37), (130, 1), (64, 2), (5, 70), (0, 1), (199, 1)]
    out, ref = _attention_case(ops, dtype, H, Hkv, dh, page, seqs, 0, g)
    assert torch.isfinite(out).all()
    assert (out - ref).abs().max() <= _tol(dtype, 2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,dh,page", [(12, 12, 64, 16), (4, 4, 16, 4), (3, 3, 32, 8), (6, 2, 128, 16),
                                           (2, 1, 256, 64), (5, 5, 48, 16)])
@pytest.mark.parametrize("window", [0, 33])
@pytest.mark.parametrize("shape", [None, (3, 4), (8, 2), (1, 6), (1, 16)])
def test_paged_attention_decode_only(ops, dtype, H, Hkv, dh, page, window, shape):
    """Every query a single token: the decode kernel (power-of-two head sizes; others fall back),
    in its default launch shape and with the keys of a query split over 3 and 8 workgroups whose
    partial results the last one merges; contexts from 1 token to a thousand so that splits are
    empty, partial and full."""
    g = torch.Generator().manual_seed(H * 10 + dh + window)
    ops.DECODE_SHAPE_OVERRIDE = shape
    try:
        for seqs in ([(0, 1)], [(1023, 1), (0, 1), (63, 1), (64, 1), (500, 1), (17, 1), (129, 1), (255, 1)],
                     [(s, 1) for s in range(3, 300, 7)]):
            out, ref = _attention_case(ops, dtype, H, Hkv, dh, page, seqs, window, g)
            assert torch.isfinite(out).all()
            assert (out - ref).abs().max() <= _tol(dtype, 2)
        # run twice in a row: the split counters must be back at zero
        out, ref = _attention_case(ops, dtype, H, Hkv, dh, page, [(700, 1), (2, 1)], window, g)
        assert (out - ref).abs().max() <= _tol(dtype, 2)
    finally:
        ops.DECODE_SHAPE_OVERRIDE = None


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,dh,page,qlens", [(12, 12, 64, 16, (1, 1, 1)), (6, 2, 32, 8, (1, 1, 1)),
                                                   (5, 5, 48, 16, (1, 1, 1)), (4, 2, 64, 4, (3, 1, 9))])
def test_paged_attention_appends_own_keys(ops, dtype, H, Hkv, dh, page, qlens):
    """With append=..., the step's keys/values come from the q rows and land in the pages:
    fused into the decode kernel (single-token queries, power-of-two heads) or copied first."""
    g = torch.Generator().manual_seed(H + dh + sum(qlens))
    starts = (200, 0, 31)
    kv_dim, qd = Hkv * dh, H * dh
    n_pages = sum(-(-(s + n) // page) for s, n in zip(starts, qlens)) + 2
    kp = torch.full((n_pages * page, kv_dim), float("nan"), dtype=dtype)
    vp = torch.full((n_pages * page, kv_dim), float("nan"), dtype=dtype)
    ref_kp, ref_vp = kp.clone(), vp.clone()
    maxb = max(-(-(s + n) // page) for s, n in zip(starts, qlens))
    tables = torch.zeros(3, maxb, dtype=torch.int32)
    T = sum(qlens)
    qkv = _rand((T, qd + 2 * kv_dim), dtype, g)
    token_seq, positions, slots = [], [], []
    used = t = 0
    for b, (s, n) in enumerate(zip(starts, qlens)):
        nb = -(-(s + n) // page)
        tables[b, :nb] = torch.arange(used, used + nb, dtype=torch.int32)
        used += nb
        js = torch.arange(s + n)
        rows = tables[b].long()[js // page] * page + js % page
        k, v = _rand((s + n, kv_dim), dtype, g), _rand((s + n, kv_dim), dtype, g)
        k[s:], v[s:] = qkv[t:t + n, qd:qd + kv_dim], qkv[t:t + n, qd + kv_dim:]
        ref_kp[rows], ref_vp[rows] = k, v
        kp[rows[:s]], vp[rows[:s]] = k[:s], v[:s]             # the step's own rows are still empty
        token_seq += [b] * n
        positions += list(range(s, s + n))
        slots += rows[s:].tolist()
        t += n
    token_seq, positions, slots = (torch.tensor(a, dtype=torch.int32) for a in (token_seq, positions, slots))
    kp_d, vp_d = kp.to(DEV), vp.to(DEV)
    out = torch.zeros(T, qd, dtype=dtype, device=DEV)
    ops.paged_attention(qkv.to(DEV), 0, H, Hkv, dh, kp_d, vp_d, page, tables.to(DEV), token_seq.to(DEV),
                        positions.to(DEV), dh ** -0.5, 0, out, max_q_len=max(qlens), max_ctx_len=210,
                        append=(qd, qd + kv_dim, slots.to(DEV)))
    ref = torch.zeros(T, qd, dtype=torch.float64)
    plain_ops.paged_attention(qkv, 0, H, Hkv, dh, ref_kp, ref_vp, page, tables, token_seq, positions, dh ** -0.5, 0, ref)
    assert (out.cpu().double() - ref).abs().max() <= _tol(dtype, 2)
    written = slots.long()
    assert torch.equal(kp_d.cpu()[written], ref_kp[written]) and torch.equal(vp_d.cpu()[written], ref_vp[written])


@pytest.mark.parametrize("H,Hkv,dh,page", [(12, 12, 64, 16), (3, 3, 32, 8), (4, 1, 128, 16), (6, 2, 64, 4)])
@pytest.mark.parametrize("window", [0, 1, 50, 64, 200])
def test_paged_attention_prefill_tiles(ops, H, Hkv, dh, page, window):
    """The MFMA prefill kernel (bf16, head sizes 32/64/128): query tiles that are full, partial and
    a single row; portions that start mid-sequence and mid-page; windows that cut inside a key tile."""
    g = torch.Generator().manual_seed(H + dh + window)
    seqs = [(0, 64), (0, 150), (37, 2), (100, 129), (511, 1), (64, 64), (5, 63)]
    out, ref = _attention_case(ops, torch.bfloat16, H, Hkv, dh, page, seqs, window, g)
    assert torch.isfinite(out).all()
    assert (out - ref).abs().max() <= _tol(torch.bfloat16, 2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,dh,page", [(12, 12, 64, 16), (4, 4, 16, 4), (6, 2, 48, 12), (5, 1, 80, 8), (3, 3, 128, 20),
                                           (2, 1, 256, 64), (7, 7, 32, 1)])
@pytest.mark.parametrize("window", [0, 1, 50, 64, 200])
def test_paged_attention_tiles_in_true_32_bit(ops, dtype, H, Hkv, dh, page, window):
    """The prompt-portion kernel that shares key tiles among 64 queries at any head size (steps of 16 up to 256),
    any page size (12 and 20 are no powers of two; 1), grouped heads, float32 and bfloat16 storage: query tiles that
    are full, partial and a single row; portions that start mid-sequence and mid-page; windows that cut inside a key
    tile. Read back from the ops: this kernel ran wherever the bfloat16 matrix-core kernel does not take the sizes."""
    g = torch.Generator().manual_seed(H + dh + window + page)
    seqs = [(0, 64), (0, 150), (37, 2), (100, 129), (511, 1), (64, 64), (5, 63)]
    ops.reset_seen()
    out, ref = _attention_case(ops, dtype, H, Hkv, dh, page, seqs, window, g)
    mfma_bf16 = dtype == torch.bfloat16 and dh in (32, 64, 128) and page & (page - 1) == 0 and page >= dh // 16
    assert ops.seen("tiled_f32_launches") == (0 if mfma_bf16 else 1) and ops.seen("generic_attention_launches") == 0
    assert torch.isfinite(out).all()
    assert (out - ref).abs().max() <= _tol(dtype, 2)
    # single tokens in front of the portions (a mixed step): at page sizes the decode kernel refuses they go to the
    # one-wavefront-per-query kernel, the portions to the tiles
    seqs = [(300, 1), (0, 1), (77, 1), (0, 70), (130, 3), (64, 129)]
    ops.reset_seen()
    out, ref = _attention_case(ops, dtype, H, Hkv, dh, page, seqs, window, g, n_single=3)
    assert ops.seen("tiled_f32_launches") == (0 if mfma_bf16 else 1)
    assert torch.isfinite(out).all()
    assert (out - ref).abs().max() <= _tol(dtype, 2)


@pytest.mark.parametrize("T", [1, 8, 16])
@pytest.mark.parametrize("H,Hkv,dh,page,N", [(12, 12, 64, 16, 768), (25, 25, 64, 16, 1600), (3, 3, 32, 8, 96),
                                             (4, 2, 128, 16, 200), (16, 16, 64, 16, 1024)])
@pytest.mark.parametrize("shape", [(2, 4), (3, 2), (4, 12), None])
def test_decode_attention_splits_merged_by_the_next_product(ops, T, H, Hkv, dh, page, N, shape):
    """Single tokens whose keys are split over several workgroups per (token, head): the attention op
    hands back the splits unmerged and the product that follows merges them while it loads. Equal to
    attention followed by the product on merged rows; contexts from one key (most splits empty) to
    several hundred; the tokens' own keys come from their qkv rows and reach the pages."""
    g = torch.Generator().manual_seed(T * 31 + H + dh)
    ctx = [1, 700, 130, 2, 64, 65, 300, 17, 1000, 5, 129, 511, 33, 256, 90, 3][:T]
    nblk = [-(-c // page) for c in ctx]
    n_pages = sum(nblk) + 2
    perm = torch.randperm(n_pages, generator=g).tolist()
    kv_dim, D = Hkv * dh, H * dh
    kp = torch.full((n_pages * page, kv_dim), float("nan"), dtype=torch.bfloat16)
    vp = torch.full((n_pages * page, kv_dim), float("nan"), dtype=torch.bfloat16)
    tables = torch.zeros(T, max(nblk), dtype=torch.int32)
    qkv = _rand((T, D + 2 * kv_dim), torch.bfloat16, g)
    slots = torch.zeros(T, dtype=torch.int32)
    used = 0
    for b in range(T):
        for j in range(nblk[b]):
            tables[b, j] = perm[used]
            used += 1
        js = torch.arange(ctx[b] - 1)                   # the last key is the token's own, not in the pages yet
        rows = tables[b].long()[js // page] * page + js % page
        kp[rows] = _rand((ctx[b] - 1, kv_dim), torch.bfloat16, g)
        vp[rows] = _rand((ctx[b] - 1, kv_dim), torch.bfloat16, g)
        slots[b] = int(tables[b, (ctx[b] - 1) // page]) * page + (ctx[b] - 1) % page
    token_seq = torch.arange(T, dtype=torch.int32)
    positions = torch.tensor([c - 1 for c in ctx], dtype=torch.int32)
    w = _rand((N, D), torch.bfloat16, g, std=1.0 / math.sqrt(D))
    bias = 0.5 * _rand((N,), torch.float32, g)
    x0 = _rand((T, N), torch.float32, g)
    # reference: append, attention, product, all plain
    rk, rv = kp.clone(), vp.clone()
    att = torch.zeros(T, D, dtype=torch.float64)
    plain_ops.paged_attention(qkv, 0, H, Hkv, dh, rk, rv, page, tables, token_seq, positions, dh ** -0.5, 0, att,
                              append=(D, D + kv_dim, slots))
    ref = plain_ops.linear(att, w.double(), bias, x0.double().clone(), "add_residual")
    kd, vd = kp.to(DEV), vp.to(DEV)
    out = torch.empty(T, D, dtype=torch.bfloat16, device=DEV)
    ops.DECODE_UNMERGED_SHAPE = shape
    try:
        a = ops.paged_attention(qkv.to(DEV), 0, H, Hkv, dh, kd, vd, page, tables.to(DEV), token_seq.to(DEV),
                                positions.to(DEV), dh ** -0.5, 0, out, max_q_len=1, max_ctx_len=max(ctx),
                                append=(D, D + kv_dim, slots.to(DEV)), may_split=True)
    finally:
        ops.DECODE_UNMERGED_SHAPE = None
    if shape is not None or (max(ctx) >= 256 and T * H <= 128):
        assert isinstance(a, ops.AttentionSplits) and a.nsplit == (shape[0] if shape else a.nsplit) and a.nsplit > 1
    x = x0.clone().to(DEV)
    ops.linear(a, w.to(DEV), bias.to(DEV), x, "add_residual")
    assert torch.isfinite(x).all()
    assert (x.cpu().double() - ref).abs().max() <= 3e-2
    written = slots.long()
    assert torch.equal(kd.cpu()[written], rk[written]) and torch.equal(vd.cpu()[written], rv[written])
    if isinstance(a, ops.AttentionSplits):
        # merged into an ordinary activation by the kernel of its own: the same rows
        merged = a.tensor()
        assert (merged.cpu().double() - att).abs().max() <= 2e-2
        y = torch.empty(T, N, dtype=torch.bfloat16, device=DEV)
        ops.linear(a, w.to(DEV), bias.to(DEV), y, "gelu_tanh")
        ref_y = plain_ops.linear(att, w.double(), bias, torch.empty(T, N, dtype=torch.float64), "gelu_tanh")
        assert (y.cpu().double() - ref_y).abs().max() <= 3e-2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,dh,page,window", [(12, 12, 64, 16, 0), (3, 3, 32, 8, 0), (4, 1, 128, 16, 40), (4, 4, 16, 4, 0)])
def test_paged_attention_single_tokens_before_portions(ops, dtype, H, Hkv, dh, page, window):
    """A scheduler's mixed step: decoded tokens first, then prompt portions. The leading single tokens
    (`n_single` of them) go to the single-query kernel and the rest to the query tiles; a single token
    that stands among the portions stays with them. Same result as without the hint."""
    g = torch.Generator().manual_seed(H + dh)
    seqs = [(130, 1), (0, 1), (299, 1), (64, 1), (0, 37), (17, 1), (5, 70), (100, 130)]
    out, ref = _attention_case(ops, dtype, H, Hkv, dh, page, seqs, window, g, n_single=4)
    assert torch.isfinite(out).all()
    assert (out - ref).abs().max() <= _tol(dtype, 2)
    g = torch.Generator().manual_seed(H + dh)
    plain, _ = _attention_case(ops, dtype, H, Hkv, dh, page, seqs, window, g)
    assert (out - plain).abs().max() <= _tol(dtype, 2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,dh,page", [(4, 4, 64, 4), (2, 1, 128, 16)])
def test_paged_attention_long_contexts(ops, dtype, H, Hkv, dh, page):
    """Contexts far beyond the tiny models': block tables longer than the prefill kernel stages in
    LDS (2048 blocks), decode over 20,000 keys, a portion that ends a long prompt, with and without
    a window."""
    g = torch.Generator().manual_seed(dh + page)
    for seqs, window in (([(9000, 1), (5, 1)], 0), ([(8300, 200)], 0), ([(0, 2300)], 777), ([(20000, 1)], 0),
                         ([(8190, 3), (100, 40)], 777), ([(8000, 192)], 0)):        # (the last: 2048 blocks of 4 exactly)
        out, ref = _attention_case(ops, dtype, H, Hkv, dh, page, seqs, window, g)
        assert torch.isfinite(out).all()
        assert (out - ref).abs().max() <= _tol(dtype, 2), (seqs, window)


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_attention_splits_long_contexts_over_the_chip(ops, dtype):
    """Few pairs with thousands of keys: the keys of a pair are split over up to 256 workgroups and a small
    kernel merges their states. Same result as one workgroup a pair, with a short sequence beside the long
    ones (splits that hold no key) and with a window."""
    g = torch.Generator().manual_seed(5)
    for seqs, window in (([(6000, 1), (3, 1), (4500, 1)], 0), ([(9000, 1)], 0), ([(7000, 1), (5000, 1)], 1300)):
        results = []
        for on in (True, False):
            ops.LONG_CONTEXT_SPLITS = on
            try:
                gg = torch.Generator().manual_seed(int(g.initial_seed()) + len(seqs))
                out, ref = _attention_case(ops, dtype, 6, 2, 64, 16, seqs, window, gg)
            finally:
                ops.LONG_CONTEXT_SPLITS = True
            assert (out - ref).abs().max() <= _tol(dtype, 2), (seqs, window, on)
            results.append(out)
        assert (results[0] - results[1]).abs().max() <= _tol(dtype, 2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_far_key_stands_out(ops, dtype):
    """One key hundreds of positions back carries almost all the weight of the last query."""
    g = torch.Generator().manual_seed(7)
    out, ref = _attention_case(ops, dtype, 4, 2, 64, 16, [(600, 3), (0, 300)], 0, g, boost=(3, 4.0))
    assert (out - ref).abs().max() <= _tol(dtype, 2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 7, 64, 65])
def test_paged_attention_window_edge(ops, dtype, window):
    g = torch.Generator().manual_seed(window)
    out, ref = _attention_case(ops, dtype, 4, 2, 32, 8, [(0, 80), (130, 1), (63, 3)], window, g)
    assert (out - ref).abs().max() <= _tol(dtype, 2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_kernels_against_their_cpp_twins(ops, dtype):
    """Every kernel against the plain C++ statement of its operation (csrc/ref/ref_ops.cc)."""
    g = torch.Generator().manual_seed(11)
    V, P, D, T = 301, 40, 200, 37
    wte, wpe = _rand((V, D), dtype, g), _rand((P, D), dtype, g)
    ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    pos = torch.randint(0, P, (T,), generator=g, dtype=torch.int32)
    x = torch.empty(T, D, dtype=torch.float32, device=DEV)
    ops.embed(ids.to(DEV), pos.to(DEV), wte.to(DEV), wpe.to(DEV), x)
    assert (x.cpu() - ref_ops.embed(ids, pos, wte, wpe)).abs().max() <= 1e-6
    gamma, beta = 1 + 0.1 * _rand((D,), torch.float32, g), 0.1 * _rand((D,), torch.float32, g)
    h = torch.empty(T, D, dtype=dtype, device=DEV)
    ops.layernorm(x, gamma.to(DEV), beta.to(DEV), 1e-5, h)
    assert (h.cpu().float() - ref_ops.layernorm(x.cpu(), gamma, beta, 1e-5)).abs().max() <= _tol(dtype, 4)
    for M, N, K, epi in [(T, 3 * D, D, "store"), (5, 72, D, "gelu_tanh"), (T, D, D, "add_residual"), (70, V, D, "store_f32"),
                         (3, 90, D, "gelu_erf")]:
        a, w, bias = _rand((M, K), dtype, g), _rand((N, K), dtype, g, std=K ** -0.5), 0.5 * _rand((N,), torch.float32, g)
        f32_out = epi in ("add_residual", "store_f32")
        out0 = _rand((M, N), torch.float32 if f32_out else dtype, g)
        out = out0.clone().to(DEV)
        ops.linear(a.to(DEV), w.to(DEV), bias.to(DEV), out, epi)
        tol = 3e-5 if dtype == torch.float32 else (2e-5 + 2e-5 * math.sqrt(K) if f32_out else 4e-2)
        assert (out.cpu().float() - ref_ops.linear(a, w, bias, out0, epi)).abs().max() <= tol, (M, N, K, epi)
        if epi != "add_residual":
            xs = _rand((M, K), torch.float32, g) + 0.3
            out = out0.clone().to(DEV)
            ops.ln_linear(xs.to(DEV), gamma.to(DEV), beta.to(DEV), 1e-5, w.to(DEV), bias.to(DEV), out, epi)
            hn = ref_ops.layernorm(xs, gamma, beta, 1e-5).to(dtype)
            # (a normalised value next to a bf16 rounding boundary may round the other way in the kernel)
            tol_ln = 3e-5 if dtype == torch.float32 else (2e-2 if epi == "store_f32" else 4e-2)
            assert (out.cpu().float() - ref_ops.linear(hn, w, bias, out0, epi)).abs().max() <= tol_ln, (M, N, K, epi)
    H, Hkv, dh, page = 6, 2, 32, 8
    src = _rand((9, 3 * Hkv * dh), dtype, g)
    slots = torch.tensor([5, -1, 0, 9, 70, 71, 72, 3, 11], dtype=torch.int32)
    kp, vp = torch.zeros(80, Hkv * dh, dtype=dtype, device=DEV), torch.zeros(80, Hkv * dh, dtype=dtype, device=DEV)
    ops.kv_append(src.to(DEV), Hkv * dh, 2 * Hkv * dh, Hkv * dh, kp, vp, slots.to(DEV))
    k2, v2 = torch.zeros(80, Hkv * dh), torch.zeros(80, Hkv * dh)
    ref_ops.kv_append(src, Hkv * dh, 2 * Hkv * dh, Hkv * dh, k2, v2, slots)
    assert torch.equal(kp.cpu().float(), k2) and torch.equal(vp.cpu().float(), v2)
    _attention_case(ops, dtype, H, Hkv, dh, page, [(40, 1), (0, 70), (9, 5), (130, 1)], 0, g)   # (compares both oracles)
    logits = _rand((6, 1000), torch.float32, g, std=2.0)
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    ops.argmax(logits.to(DEV), out)
    assert torch.equal(out.cpu(), ref_ops.argmax(logits))
    temp, u = torch.tensor([0.0, 0.7, 1.0, 1.3, 0.2, 5.0]), torch.tensor([0.3, 0.0, 0.999, 0.5, 0.25, 0.75])
    ops.sample(logits.to(DEV), temp.to(DEV), u.to(DEV), out)
    got, want = out.cpu(), ref_ops.sample(logits, temp, u)
    for r in range(6):                  # next to a boundary of the cumulative mass either neighbour is right
        assert abs(int(got[r]) - int(want[r])) <= 1, (r, got, want)


def test_argmax_ties_take_lowest_index(ops):
    V = 50257
    g = torch.Generator().manual_seed(3)
    logits = _rand((5, V), torch.float32, g)
    logits[0, 40000] = logits[0, 123] = 9.0
    logits[1, V - 1] = 10.0
    logits[2, 0] = 10.0
    logits[3, :] = 0.5
    out = torch.empty(5, dtype=torch.int32, device=DEV)
    ops.argmax(logits.to(DEV), out)
    ref = plain_ops.argmax(logits, torch.empty(5, dtype=torch.int32))
    assert out.cpu().tolist() == ref.tolist()
    assert out.cpu().tolist()[:4] == [123, V - 1, 0, 0]


@pytest.mark.parametrize("V", [4, 1000, 50257])
def test_sample_inverse_cdf(ops, V):
    g = torch.Generator().manual_seed(V)
    n = 64
    logits = _rand((n, V), torch.float32, g, std=2.0)
    temps = torch.rand(n, generator=g) * 1.5 + 0.2
    temps[::7] = 0.0
    u = torch.rand(n, generator=g)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV), temps.to(DEV), u.to(DEV), out)
    got = out.cpu().tolist()
    for i in range(n):
        row = logits[i].double()
        if temps[i] <= 0:
            assert got[i] == int(row.argmax())
            continue
        p = torch.softmax(row / temps[i].double(), 0)
        c = torch.cumsum(p, 0)
        lo = float(c[got[i] - 1]) if got[i] > 0 else 0.0
        hi = float(c[got[i]])
        assert lo - 1e-5 <= float(u[i]) <= hi + 1e-5, (i, got[i], lo, float(u[i]), hi)


def test_sample_edge_rows(ops):
    """All mass on one entry, a flat row, u at both ends, masses that underflow to zero."""
    V = 5000
    logits = torch.full((6, V), -50.0)
    logits[0, 4321] = 30.0
    logits[1] = 0.0
    logits[2] = 0.0
    logits[3, V - 1] = 30.0
    logits[4, 0] = 30.0
    logits[5, 2047:2050] = 5.0                      # the mass straddles a tile edge
    u = torch.tensor([0.5, 0.0, 0.99999994, 0.99999994, 0.0, 0.5])
    temps = torch.full((6,), 1.0)
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV), temps.to(DEV), u.to(DEV), out)
    got = out.cpu().tolist()
    assert got[0] == 4321 and got[1] == 0 and got[2] == V - 1 and got[3] == V - 1 and got[4] == 0
    assert got[5] == 2048


def test_sample_frequencies_follow_softmax(ops):
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0]]).repeat(4096, 1)
    g = torch.Generator().manual_seed(11)
    u = torch.rand(4096, generator=g)
    temps = torch.full((4096,), 0.8)
    out = torch.empty(4096, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV), temps.to(DEV), u.to(DEV), out)
    freq = torch.bincount(out.cpu().long(), minlength=4).double() / 4096
    p = torch.softmax(logits[0].double() / 0.8, 0)
    assert (freq - p).abs().max() < 4 * math.sqrt(0.25 / 4096)
