"""Each part alone on the GPU against the plain implementation's function for it, and the
framework's generality: toy parts and toy architectures that are defined under tests/ (a plugin,
tests/native/toy_plugin.hip: a mixer with state of its own, a norm of another kind, a layer without
feed-forward, a position encoding that turns queries and keys, a feed-forward with routing, an untied
head) are registered, built, stepped and served without a change to the framework's files."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_gpt2 as P
import toy

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
NAME = {torch.float32: "float32", torch.bfloat16: "bfloat16"}
TOL = {torch.float32: 3e-5, torch.bfloat16: 3e-2}
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _randn(g, *shape, mean=0.0, std=1.0, dtype=None):
    t = torch.empty(shape).normal_(mean, std, generator=g)
    return t.to(dtype).float() if dtype is not None else t       # (what the part holds, exactly)


@pytest.mark.parametrize("dtype", DTYPES)
def test_layernorm_part(dtype):
    import parts_face as pf
    g = torch.Generator().manual_seed(0)
    gamma, beta = _randn(g, 100, mean=1.0, std=0.1), _randn(g, 100, std=0.05)
    ln = pf.Norm("layernorm", pf.Params(size=100, eps=1e-6, dtype=pf.DT[dtype], gamma=gamma.to(DEV), beta=beta.to(DEV)))
    x = torch.randn(9, 100, generator=g) * 3 + 1
    y = ln.forward(x.to(DEV), dtype)
    ref = P.layer_norm(x.double(), gamma.double(), beta.double(), 1e-6)
    assert (y.cpu().double() - ref).abs().max() <= TOL[dtype] * 4
    rows = torch.tensor([8, 0, 3], dtype=torch.int32, device=DEV)
    y = ln.forward(x.to(DEV), dtype, rows)
    assert (y.cpu().double() - ref[[8, 0, 3]]).abs().max() <= TOL[dtype] * 4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", ["gelu_tanh", "gelu_erf"])
def test_dense_mlp_part(dtype, act):
    import parts_face as pf
    g = torch.Generator().manual_seed(1)
    up, down = _randn(g, 200, 48, std=0.05, dtype=dtype), _randn(g, 48, 200, std=0.05, dtype=dtype)
    b1, b2 = _randn(g, 200, std=0.05), _randn(g, 48, std=0.05)
    ff = pf.FeedForward("dense_mlp", pf.Params(activation=act, dtype=pf.DT[dtype], up__weight=up.to(dtype).to(DEV),
                                               up__bias=b1.to(DEV), down__weight=down.to(dtype).to(DEV),
                                               down__bias=b2.to(DEV)))
    h = torch.randn(7, 48, generator=g).to(dtype)
    x0 = torch.randn(7, 48, generator=g)
    x = ff.forward(h.to(DEV), x0.clone().to(DEV))
    fn = P.gelu_tanh if act == "gelu_tanh" else P.gelu_erf
    # (the plain block takes the reference's [in, out] layout)
    w = {"h.0.mlp.c_fc.weight": up.double().T, "h.0.mlp.c_fc.bias": b1.double(),
         "h.0.mlp.c_proj.weight": down.double().T, "h.0.mlp.c_proj.bias": b2.double()}
    ref = x0.double() + P.mlp_block(h.double(), w, 0, fn)
    assert (x.cpu().double() - ref).abs().max() <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_position_and_head_parts(dtype):
    import parts_face as pf
    g = torch.Generator().manual_seed(2)
    wte, wpe = _randn(g, 301, 40, std=0.05, dtype=dtype), _randn(g, 50, 40, std=0.05, dtype=dtype)
    emb = pf.Embedding("token_table", pf.Params(table=wte.to(dtype).to(DEV)))
    pos = pf.Params(table=wpe.to(dtype).to(DEV))
    ids = torch.tensor([300, 0, 7, 7, 19], dtype=torch.int32, device=DEV)
    positions = torch.tensor([0, 1, 49, 3, 4], dtype=torch.int32, device=DEV)
    x = emb.forward(ids, positions, 40, "learned_absolute", pos)
    ref = P.embedding(wte.double(), wpe.double(), ids.cpu().long(), positions.cpu().long())
    assert x.dtype == torch.float32 and (x.cpu().double() - ref).abs().max() <= 1e-6
    # without a position encoding: the table's rows alone
    x0 = emb.forward(ids, positions, 40)
    assert (x0.cpu().double() - wte.double()[ids.cpu().long()]).abs().max() <= 1e-6
    # a head tied to the table, and one with a matrix and a bias of its own
    gamma, beta = _randn(g, 40, mean=1.0, std=0.1), _randn(g, 40, std=0.05)
    ln = pf.Norm("layernorm", pf.Params(size=40, eps=1e-5, dtype=pf.DT[dtype], gamma=gamma.to(DEV), beta=beta.to(DEV)))
    xs = torch.randn(6, 40, generator=g)
    rows = torch.tensor([5, 1, 2], dtype=torch.int32, device=DEV)
    normed = P.layer_norm(xs.double(), gamma.double(), beta.double(), 1e-5)[[5, 1, 2]]
    tied = pf.Head("linear", pf.Params(weight=wte.to(dtype).to(DEV), dtype=pf.DT[dtype]))
    logits = tied.forward(xs.to(DEV), ln, 301, rows)
    assert logits.shape == (3, 301) and (logits.cpu().double() - normed @ wte.double().T).abs().max() <= TOL[dtype]
    own, bias = _randn(g, 77, 40, std=0.05, dtype=dtype), _randn(g, 77, std=0.05)
    untied = pf.Head("linear", pf.Params(weight=own.to(dtype).to(DEV), bias=bias.to(DEV), dtype=pf.DT[dtype]))
    logits = untied.forward(xs.to(DEV), ln, 77, rows)
    assert (logits.cpu().double() - (normed @ own.double().T + bias.double())).abs().max() <= TOL[dtype]


def _save_model(d, cfg, tensors):
    from safetensors.torch import save_file
    os.makedirs(d, exist_ok=True)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(d, "model.safetensors"))
    return d


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,dh,window", [(4, 4, 16, 0), (3, 3, 32, 0), (6, 2, 16, 0), (4, 2, 32, 5)])
def test_attention_part_in_portions_over_page_edges(tmp_path, dtype, H, Hkv, dh, window):
    """The mixer alone (the toy architecture around it is identities: the embedding table holds the mixer's
    input rows, the norms only cast, the untied head is the unit matrix): a sequence fed in portions that
    start and end at, before and after page edges equals the plain whole-sequence attention."""
    from mini_llm_amd import Runner, StepEntry
    toy.load()
    D, n = H * dh, 41
    g = torch.Generator().manual_seed(H + dh)
    h = _randn(g, n, D, dtype=dtype)
    w = {"emb.weight": h, "qkv.weight": _randn(g, D + 2 * Hkv * dh, D, std=0.05, dtype=dtype),
         "o.weight": _randn(g, D, D, std=0.05, dtype=dtype), "qkv.bias": _randn(g, D + 2 * Hkv * dh, std=0.05),
         "o.bias": _randn(g, D, std=0.05), "head.weight": torch.eye(D)}
    cfg = dict(architectures=["ToyBareMixer"], rows=n, heads=H, kv_heads=Hkv, head_dim=dh, outputs=D, bias=True, window=window)
    d = _save_model(str(tmp_path / "bare"), cfg, w)
    runner = Runner(model_dir=d, dtype=NAME[dtype], page_size=8, n_pages=8, max_num_seqs=2)
    runner.poison_cache()
    got, i = [], 0
    for size in (7, 1, 8, 9, 2, 14):          # 7 | 8 | 16 | 25 | 27 | 41: edges at 8, 16, 24, 32, 40
        got.append(runner.step([StepEntry(1, list(range(i, i + size)), list(range(size)))]))
        i += size
    x = torch.from_numpy(np.concatenate(got)).double()       # = h + attention(h), through the unit head
    wd = {k: v.double() for k, v in w.items()}
    qkv = h.double() @ wd["qkv.weight"].T + wd["qkv.bias"]
    q, k, v = qkv[:, :D], qkv[:, D:D + Hkv * dh], qkv[:, D + Hkv * dh:]
    rep = H // Hkv
    expand = lambda t: t.view(n, Hkv, 1, dh).expand(n, Hkv, rep, dh).reshape(n, D)
    a = P.causal_attention(q, expand(k), expand(v), H, window=window or None)
    ref = h.double() + a @ wd["o.weight"].T + wd["o.bias"]
    # (in bfloat16 the identity norm in front of the unit head rounds the result itself to bfloat16: half a unit
    # in the last place of each value, on top of the mixer's own error)
    cast = ref.abs() * 2.0 ** -8 if dtype == torch.bfloat16 else 0.0
    assert ((x - ref).abs() <= TOL[dtype] * 2 + cast).all(), (x - ref).abs().max()


# ---------------------------------------------------------------------------------------------
# ToyLM: one attention layer and one layer whose mixer keeps a running mean in a fixed-size state
# slot, run in an order that names the attention layer twice (the second call only reads the cache
# the first one wrote). The attention layer's two norms differ in kind and the other layer has no
# feed-forward.
# ---------------------------------------------------------------------------------------------
TOY_CFG = dict(architectures=["ToyLM"], vocab=203, width=48, heads=3, decay=0.75, eps=1e-5)


def _weights(d):
    from safetensors import safe_open
    with safe_open(d + "/model.safetensors", framework="pt") as f:
        return {k: f.get_tensor(k).double() for k in f.keys()}


def _toy_plain(w, cfg, ids):
    """Whole sequence, no cache, float64."""
    D, H = cfg["width"], cfg["heads"]
    dh = D // H
    x = w["emb.weight"][torch.tensor(ids)]
    ln = lambda x, p: P.layer_norm(x, w[p + ".weight"], w[p + ".bias"], cfg["eps"])
    ffn = lambda h, p: P.gelu_erf(h @ w[p + "up.weight"].T) @ w[p + "down.weight"].T
    kv_first = None
    for layer, write in ((0, True), (1, True), (0, False)):
        p = f"l{layer}."
        h = ln(x, p + "n1")
        if layer == 0:
            qkv = h @ w[p + "qkv.weight"].T
            q = qkv[:, :D]
            if write:
                kv_first = (qkv[:, D:D + dh], qkv[:, D + dh:])
            k, v = kv_first                              # the second call reads the first call's keys
            x = x + P.causal_attention(q, k.repeat(1, H), v.repeat(1, H), H) @ w[p + "o.weight"].T
        else:
            s = torch.zeros(D, dtype=torch.float64)
            add = []
            for t in range(len(ids)):
                s = cfg["decay"] * s + (1 - cfg["decay"]) * h[t]
                add.append(w[p + "mean.gain"] * s)
            x = x + torch.stack(add)
            continue                                     # this layer has no feed-forward
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 10 * cfg["eps"]) * w[p + "n2.gain"]
        x = x + ffn(h, p)
    return ln(x, "final") @ w["emb.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_a_stateful_mixer(tmp_path, dtype):
    from mini_llm_amd import Runner, StepEntry, write_random_model
    toy.load()
    d = write_random_model(TOY_CFG, str(tmp_path / "toy"), seed=3)
    runner = Runner(model_dir=d, dtype=dtype, page_size=4, n_pages=24, max_num_seqs=3)
    runner.poison_cache()
    info = runner.info()
    # two layers, three calls, two caches: one of pages (one group), one of state slots
    assert (info["architecture"], info["n_layers"], info["n_calls"], info["n_caches"], info["n_groups"]) == ("ToyLM", 2, 3, 2, 1)
    assert info["max_positions"] == 0                     # no position encoding: unbounded
    w = _weights(d)
    g = torch.Generator().manual_seed(0)
    seqs = {1: torch.randint(0, 203, (30,), generator=g).tolist(), 2: torch.randint(0, 203, (19,), generator=g).tolist(),
            3: torch.randint(0, 203, (9,), generator=g).tolist()}
    got = {r: [] for r in seqs}
    fed = {r: 0 for r in seqs}
    plan = [{1: 7, 2: 3}, {1: 1, 2: 9}, {2: 1, 3: 4}, {1: 12, 2: 1, 3: 1}, {1: 10, 2: 5, 3: 4}]
    for step in plan:
        entries = [StepEntry(r, seqs[r][fed[r]:fed[r] + n], list(range(n))) for r, n in step.items()]
        logits = runner.step(entries)
        i = 0
        for r, n in step.items():
            got[r].append(logits[i:i + n].copy())
            i += n
            fed[r] += n
    tol = 3e-5 if dtype == "float32" else 4e-2
    for r, ids in seqs.items():
        assert fed[r] == len(ids)
        ref = _toy_plain(w, TOY_CFG, ids)
        assert (torch.from_numpy(np.concatenate(got[r])).double() - ref).abs().max() <= tol, r
    # a slot that is used again starts from an empty state (the storage clears it on the device)
    runner.end_request(3)
    runner.poison_cache()
    out = runner.step([StepEntry(4, seqs[3], list(range(9)))])
    assert (torch.from_numpy(out).double() - _toy_plain(w, TOY_CFG, seqs[3])).abs().max() <= tol
    assert runner.check() == ""


def _plain_greedy(w, cfg, ids, new):
    ids, out = list(ids), []
    for _ in range(new):
        logits = _toy_plain(w, cfg, ids)[-1]
        top = torch.topk(logits, 2).values
        out.append((int(logits.argmax()), float(top[0] - top[1])))
        ids.append(out[-1][0])
    return out


def test_toy_architecture_is_served_by_the_engine_and_the_command_line(tmp_path):
    """The engine (scheduler, continuous batching, sampling on the device, steps run ahead) and the program
    `mini-llm generate` serve the plugin's architecture: 9 requests through batches of up to 12 with the state
    slots of finished requests used again in a second round, tokens equal to greedy decoding of the plain
    whole-sequence implementation."""
    from mini_llm_amd import Engine, EngineOptions, SamplingParams, write_random_model
    path = toy.load()
    d = write_random_model(TOY_CFG, str(tmp_path / "toy"), seed=5)
    w = _weights(d)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, 203, (3 + i,), generator=g).tolist() for i in range(9)]
    new = 7
    plain = [_plain_greedy(w, TOY_CFG, p, new) for p in prompts]

    def same(outs, label):
        for p, o, ref in zip(prompts, outs, plain):
            assert len(o) == new
            for i, (tok, gap) in enumerate(ref):
                assert o[i] == tok or gap < 1e-4, (label, p, i, o, tok)
                if o[i] != tok:
                    break

    engine = Engine.from_pretrained(d, dtype="float32", options=EngineOptions(
        kv_block_size=4, total_kv_blocks=64, max_batch_num=12, max_tokens_per_step=64, prefill_chunk=8))
    engine.runner.poison_cache()
    for round_ in range(2):                       # the second round reuses slots that hold old states
        same(engine.generate(prompts, SamplingParams(max_new_tokens=new, ignore_eos=True)), f"engine round {round_}")
    assert engine.stats()["free_pages"] == 64
    # the program, with the plugin named on its command line
    cmd = [sys.executable, os.path.join(ROOT, "bin", "mini-llm"), "generate", "--plugin", path, "--model", d, "--dtype", "float32",
           "--max-new-tokens", str(new), "--ignore-eos", "--kv-block-size", "4", "--total-kv-blocks", "64",
           "--max-batch-num", "12", "--prefill-chunk", "8"]
    for p in prompts:
        cmd += ["--prompt-ids", " ".join(map(str, p))]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    assert len(lines) == len(prompts) and all(l.endswith("[DONE]") for l in lines)
    same([[int(t) for t in l.split()[:-1]] for l in lines], "program")
    # without the plugin the architecture is unknown, and the error says what is registered
    r = subprocess.run([c for c in cmd if c not in ("--plugin", path)], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "ToyLM" in r.stderr and "GPT2LMHeadModel" in r.stderr
    # ... unless the environment names it
    r = subprocess.run([c for c in cmd if c not in ("--plugin", path)], capture_output=True, text=True, timeout=300,
                       env=dict(os.environ, MINI_LLM_PLUGINS=path))
    assert r.returncode == 0, r.stderr


def test_toy_architecture_through_the_benchmark(tmp_path):
    """bench.py measures the plugin's architecture through the same engine and the same accounting (bytes and flops
    from the model's parts, whatever they are)."""
    path = toy.load()
    (tmp_path / "toy.json").write_text(json.dumps(TOY_CFG))
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--plugin", path, "--config", str(tmp_path / "toy.json"),
                        "--positions", "256", "--prompt-len", "64", "--batch", "4", "--steps", "16", "--warmup", "4"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr
    rec = json.loads(r.stdout.strip().splitlines()[-1])
    assert rec["config"]["model"] == "ToyLM-sizes" and rec["config"]["vocab_size"] == 203 and rec["value"] > 0
    # weights a step reads: the attention layer's, the stateful layer's, the final norm's and the tied head's (bf16
    # matrices, fp32 vectors); the cache: one layer of one key/value head of 16
    D, dh = 48, 16
    matrices = (D + 2 * dh) * D + D * D + 2 * D * D * 2 + 203 * D
    vectors = 2 * D + D + 2 * D + D + 2 * D
    live = 4 * rec["config"]["mean_context"] * 2 * dh * 2
    assert rec["roofline"]["bytes_per_step"] == int(2 * matrices + 4 * vectors + live)


def test_toy_architecture_through_trace_replay(tmp_path):
    """bin/trace_run replays a trace on the plugin's architecture (the plugin named by the environment)."""
    import replay_util as ru
    from mini_llm_amd import write_random_model
    path = toy.load()
    d = write_random_model(TOY_CFG, str(tmp_path / "toy"), seed=8)
    w = _weights(d)
    reqs = ru.random_requests(203, [21, 33, 9, 64], seed=3)
    steps, _ = ru.trace_mixed(reqs, seed=3)
    out = ru.run_trace_run(d, "float32", steps, str(tmp_path / "out"), ru.peak_tokens(steps),
                           env=dict(os.environ, MINI_LLM_PLUGINS=path))
    got = ru.collect(steps, out, 203)
    for rid, toks in reqs.items():
        ref = _toy_plain(w, TOY_CFG, toks).numpy()
        for pos in range(len(toks)):
            assert np.abs(got[rid][pos] - ref[pos]).max() <= 3e-5, (rid, pos)


# ---------------------------------------------------------------------------------------------
# ToyRoutedLM: a position encoding that turns queries and keys inside the mixer (no table at the
# embedding), a feed-forward that routes every token to one of several experts in the first layer
# and a dense one in the second, grouped heads, a window in the second layer.
# ---------------------------------------------------------------------------------------------
def _routed_plain(w, cfg, ids):
    """Whole sequence, no cache, float64. Returns the logits and the smallest gap between the
    two largest router logits of any token (a tie there would make the comparison meaningless)
    and the set of experts that were chosen."""
    D, H, G = cfg["width"], cfg["heads"], cfg["groups"]
    dh, n = D // H, len(ids)
    x = w["emb.weight"][torch.tensor(ids)]
    ln = lambda x, p: P.layer_norm(x, w[p + ".weight"], w[p + ".bias"], cfg["eps"])
    pos = torch.arange(n, dtype=torch.float64)
    turn_by = torch.polar(torch.ones(n, dh // 2, dtype=torch.float64),
                          pos[:, None] * cfg["base"] ** (-torch.arange(dh // 2, dtype=torch.float64) / (dh // 2)))

    def turn(t, heads):
        t = t.view(n, heads, dh)
        z = torch.complex(t[..., :dh // 2], t[..., dh // 2:]) * turn_by[:, None, :]
        return torch.cat([z.real, z.imag], dim=-1)

    gap, used = float("inf"), set()
    for layer in (0, 1):
        p = f"l{layer}."
        qkv = ln(x, p + "n1") @ w[p + "qkv.weight"].T + w[p + "qkv.bias"]
        q = turn(qkv[:, :D], H).reshape(n, D)
        k = turn(qkv[:, D:D + G * dh], G)
        v = qkv[:, D + G * dh:].view(n, G, dh)
        wide = lambda t: t[:, :, None, :].expand(n, G, H // G, dh).reshape(n, D)
        a = P.causal_attention(q, wide(k), wide(v), H, window=cfg["window"] if layer == 1 else None)
        x = x + a @ w[p + "o.weight"].T + w[p + "o.bias"]
        h = ln(x, p + "n2")
        if layer == 0:
            scores = h @ w[p + "router"].T
            top = scores.topk(2, dim=-1).values
            gap = min(gap, float((top[:, 0] - top[:, 1]).min()))
            prob = torch.softmax(scores, dim=-1)
            rows = []
            for t in range(n):
                e = int(prob[t].argmax())
                used.add(e)
                rows.append(prob[t, e] * (P.gelu_erf(h[t] @ w[f"{p}expert.{e}.up"].T) @ w[f"{p}expert.{e}.down"].T))
            x = x + torch.stack(rows)
        else:
            x = x + P.gelu_tanh(h @ w[p + "up.weight"].T + w[p + "up.bias"]) @ w[p + "down.weight"].T + w[p + "down.bias"]
    return ln(x, "final") @ w["emb.weight"].T, gap, used


ROUTED_CFG = dict(architectures=["ToyRoutedLM"], vocab=157, width=64, heads=4, groups=2, experts=3, window=6,
                  base=50.0, eps=1e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_turned_keys_and_routed_experts(tmp_path, dtype):
    from mini_llm_amd import Runner, StepEntry, write_random_model
    toy.load()
    # a seed whose router logits have no near tie and whose tokens use at least two experts
    for seed in range(30, 60):
        d = write_random_model(ROUTED_CFG, str(tmp_path / f"routed{seed}"), seed=seed)
        w = _weights(d)
        g = torch.Generator().manual_seed(seed)
        seqs = {1: torch.randint(0, 157, (26,), generator=g).tolist(), 2: torch.randint(0, 157, (15,), generator=g).tolist()}
        refs = {r: _routed_plain(w, ROUTED_CFG, ids) for r, ids in seqs.items()}
        if all(ref[1] > 0.3 for ref in refs.values()) and len(set().union(*(ref[2] for ref in refs.values()))) >= 2:
            break
    else:
        pytest.fail("no seed without a near tie between experts")
    runner = Runner(model_dir=d, dtype=dtype, page_size=4, n_pages=14, max_num_seqs=2)
    runner.poison_cache()
    assert runner.info()["n_groups"] == 2                 # the window gives the second layer pages of its own
    got, fed = {r: [] for r in seqs}, {r: 0 for r in seqs}
    plan = [{1: 9, 2: 2}, {1: 1, 2: 6}, {1: 1}, {1: 13, 2: 1}, {1: 2, 2: 6}]
    for step in plan:
        entries = [StepEntry(r, seqs[r][fed[r]:fed[r] + n], list(range(n))) for r, n in step.items()]
        logits = runner.step(entries)
        i = 0
        for r, n in step.items():
            got[r].append(logits[i:i + n].copy())
            i += n
            fed[r] += n
    tol = 3e-5 if dtype == "float32" else 4e-2
    for r, ids in seqs.items():
        assert fed[r] == len(ids)
        assert (torch.from_numpy(np.concatenate(got[r])).double() - refs[r][0]).abs().max() <= tol, r
    assert runner.check() == ""
