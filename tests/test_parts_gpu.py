"""Each part alone on the GPU against the plain implementation's function for it, and the
framework's generality: a toy mixer with state of its own, defined here, is registered, built
and stepped without a change to the framework's files."""
import dataclasses
import math
from typing import List, Optional

import numpy as np
import pytest
import torch

import plain_gpt2 as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 3e-5, torch.bfloat16: 3e-2}


def _fill(part, prefix, gen, dtype):
    """Random tensors for a part's parameters; returns them as the checkpoint would hold them."""
    stored = {}
    for s in part.param_specs(prefix):
        mean, std = s.init
        t = torch.empty(s.shape).normal_(mean, max(std, 0.05), generator=gen)
        if s.role == "matrix":
            t = t.to(dtype).float()
        stored[s.name] = t.double()
        v = t.t().contiguous() if s.layout == "transpose" else t
        s.assign((v.to(dtype) if s.role == "matrix" else v.float()).to(DEV))
    return stored


def _ctx(runner, rid, tokens):
    from mini_llm_amd.engine.step import StepEntry
    runner.ensure_request(rid)
    runner.manager.reserve(rid, runner.manager.length(rid) + len(tokens))
    return runner.build_context([StepEntry(rid, tokens, [len(tokens) - 1])])


@pytest.mark.parametrize("dtype", DTYPES)
def test_layernorm_part(dtype):
    from mini_llm_amd.parts.norms import LayerNorm
    g = torch.Generator().manual_seed(0)
    ln = LayerNorm(size=100, eps=1e-6, dtype=dtype, device=DEV)
    w = _fill(ln, "n", g, dtype)
    x = torch.randn(9, 100, generator=g) * 3 + 1
    y = ln.forward(x.to(DEV))
    assert y.dtype == dtype
    ref = P.layer_norm(x.double(), w["n.weight"], w["n.bias"], 1e-6)
    assert (y.cpu().double() - ref).abs().max() <= TOL[dtype] * 4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("act", ["gelu_tanh", "gelu_erf"])
def test_dense_mlp_part(dtype, act):
    from mini_llm_amd.parts.mlp import DenseMLP
    g = torch.Generator().manual_seed(1)
    ff = DenseMLP(hidden_size=48, inner_size=200, activation=act, bias=True, weight_layout="in_out",
                  names={"up": "mlp.c_fc", "down": "mlp.c_proj"}, dtype=dtype, device=DEV)
    w = _fill(ff, "h.0.", g, dtype)
    h = torch.randn(7, 48, generator=g).to(dtype)
    x0 = torch.randn(7, 48, generator=g)
    x = x0.clone().to(DEV)
    ff.forward(h.to(DEV), None, x)
    fn = P.gelu_tanh if act == "gelu_tanh" else P.gelu_erf
    ref = x0.double() + P.mlp_block(h.double(), w, 0, fn)
    assert (x.cpu().double() - ref).abs().max() <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_tied_head_parts(dtype):
    from mini_llm_amd.parts.embedding import LearnedAbsolutePositions, TiedHead, TokenEmbedding
    g = torch.Generator().manual_seed(2)
    emb = TokenEmbedding(vocab_size=301, size=40, name="wte", dtype=dtype, device=DEV)
    pos = LearnedAbsolutePositions(n_positions=50, size=40, name="wpe", dtype=dtype, device=DEV)
    w = {**_fill(emb, "", g, dtype), **_fill(pos, "", g, dtype)}

    class Ctx:
        n_tokens = 5
        token_ids = torch.tensor([300, 0, 7, 7, 19], dtype=torch.int32, device=DEV)
        positions = torch.tensor([0, 1, 49, 3, 4], dtype=torch.int32, device=DEV)
    x = emb.forward(Ctx, pos)
    ref = P.embedding(w["wte.weight"], w["wpe.weight"], Ctx.token_ids.cpu().long(), Ctx.positions.cpu().long())
    assert x.dtype == torch.float32 and (x.cpu().double() - ref).abs().max() <= 1e-6
    h = torch.randn(3, 40, generator=g).to(dtype)
    logits = TiedHead(emb, dtype, DEV).forward(h.to(DEV))
    assert logits.dtype == torch.float32 and logits.shape == (3, 301)
    assert (logits.cpu().double() - h.double() @ w["wte.weight"].T).abs().max() <= TOL[dtype]


class _OneLayer:
    """The least a ModelRunner needs, around one attention part."""

    def __init__(self, mixer, dtype):
        self.mixer, self.dtype, self.device = mixer, dtype, torch.device(DEV)
        self.vocab_size, self.max_positions = 1000, None

    def cache_specs(self):
        return [self.mixer.cache_spec()]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,dh,window", [(4, 4, 16, None), (3, 3, 32, None), (6, 2, 16, None), (4, 2, 32, 5)])
def test_attention_part_in_portions_over_page_edges(dtype, H, Hkv, dh, window):
    """The mixer alone: a sequence fed in portions that start and end at, before and after page
    edges equals the plain whole-sequence attention."""
    from mini_llm_amd.engine.step import ModelRunner
    from mini_llm_amd.parts.attention import CausalSelfAttention
    D = H * dh
    g = torch.Generator().manual_seed(H + dh)
    att = CausalSelfAttention(hidden_size=D, n_heads=H, n_kv_heads=Hkv, head_dim=dh, scale=dh ** -0.5,
                              window=window, bias=True, weight_layout="out_in",
                              names={"qkv": "qkv", "out": "o"}, dtype=dtype, device=DEV)
    w = _fill(att, "", g, dtype)
    runner = ModelRunner(_OneLayer(att, dtype), page_size=8, n_pages=8, max_num_seqs=2)
    runner.cache.poison()
    n = 41
    h = torch.randn(n, D, generator=g).to(dtype)
    x = torch.zeros(n, D, device=DEV)
    i = 0
    for size in (7, 1, 8, 9, 2, 14):          # 7 | 8 | 16 | 25 | 27 | 41: edges at 8, 16, 24, 32, 40
        ctx = _ctx(runner, 1, [0] * size)
        att.forward(h[i:i + size].to(DEV), ctx, runner.cache.view(0), x[i:i + size])
        runner.manager.commit(1, i + size)
        i += size
    # plain: q, k, v from the same weights (stored [out, in] here), grouped heads expanded
    qkv = h.double() @ w["qkv.weight"].T + w["qkv.bias"]
    q, k, v = qkv[:, :D], qkv[:, D:D + Hkv * dh], qkv[:, D + Hkv * dh:]
    rep = H // Hkv
    expand = lambda t: t.view(n, Hkv, 1, dh).expand(n, Hkv, rep, dh).reshape(n, D)
    a = P.causal_attention(q, expand(k), expand(v), H, window=window)
    ref = a @ w["o.weight"].T + w["o.bias"]
    assert (x.cpu().double() - ref).abs().max() <= TOL[dtype] * 2


# ---------------------------------------------------------------------------------------------
# A toy architecture defined entirely in this test: one attention layer and one layer whose
# mixer keeps a running mean in a fixed-size state slot, run in an order that names the
# attention layer twice (the second call only reads the cache the first one wrote). The attention
# layer's two norms differ in kind (the second is defined here too) and the other layer has no
# feed-forward: a layer's make-up is the specification's business, not the framework's.
# ---------------------------------------------------------------------------------------------

def _define_toy():
    from mini_llm_amd.cache.manager import StateCacheSpec
    from mini_llm_amd.config.base import LayerCall, LayerSpec, ModelConfig, PartSpec
    from mini_llm_amd.config.registry import register_architecture
    from mini_llm_amd.models.decoder import DecoderModel, build_layers
    from mini_llm_amd.parts.base import MIXERS, Mixer, Norm, ParamSpec, register_mixer, register_norm
    from mini_llm_amd.parts.embedding import NoPositions, TiedHead, TokenEmbedding
    from mini_llm_amd.parts.norms import LayerNorm

    @register_mixer("toy_running_mean", replace=True)
    class RunningMean(Mixer):
        """state <- decay * state + (1 - decay) * h_t, token by token; x_t += gain * state.

        All on the device (torch operations over the step's index arrays, nothing read on the
        host), so decode steps of a model that holds it can be captured as a graph. A request's
        slot is empty when it begins: the cache storage clears it, not the mixer. Rows whose
        state slot is < 0 are padding and touch no state."""

        def __init__(self, size, decay, dtype, device):
            super().__init__(dtype, device)
            self.size, self.decay, self.gain = size, decay, None

        def param_specs(self, prefix):
            return [ParamSpec(prefix + "mean.gain", (self.size,), "vector", self._set, (1.0, 0.1))]

        def _set(self, t):
            self.gain = t

        def cache_spec(self):
            return StateCacheSpec((self.size,), torch.float32)

        def forward(self, h, ctx, cache_view, x, write=True):
            state = cache_view.slots                                   # [n_slots, size]
            n_slots = state.shape[0]
            lo, hi = ctx.cu_q[:-1].long(), ctx.cu_q[1:].long()
            slot = ctx.state_slots.long()
            which = torch.arange(n_slots, device=state.device)
            for k in range(ctx.max_q_len):                             # the k-th token of every sequence
                t = lo + k
                live = (t < hi) & (slot >= 0)
                t = torch.where(live, t, torch.zeros_like(t))
                before = state[slot.clamp(min=0)]                      # rows of padding entries are not used
                s = torch.where(live[:, None], self.decay * before + (1 - self.decay) * h[t].float(),
                                torch.zeros_like(before))
                own = ((slot[:, None] == which[None, :]) & live[:, None]).float()      # [B, n_slots], one-hot rows
                state.copy_(torch.where(own.sum(0)[:, None] > 0, own.T @ s, state))
                x.index_add_(0, t, self.gain * s)

    @register_norm("toy_scale_norm", replace=True)
    class ScaleNorm(Norm):
        """x / sqrt(mean(x^2) + eps) * gain: another norm kind than the first position's."""

        def __init__(self, size, eps, dtype, device):
            super().__init__(dtype, device)
            self.size, self.eps, self.gain = size, eps, None

        def param_specs(self, prefix):
            return [ParamSpec(prefix + ".gain", (self.size,), "vector", self._set, (1.0, 0.1))]

        def _set(self, t):
            self.gain = t

        def forward(self, x, rows=None):
            x = x if rows is None else x[rows.long()]
            return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps) * self.gain).to(self.dtype)

    @dataclasses.dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        vocab: int
        width: int
        heads: int
        decay: float
        eps: float
        architecture = "ToyLM"

        @property
        def vocab_size(self):
            return self.vocab

        @property
        def hidden_size(self):
            return self.width

        @classmethod
        def from_dict(cls, d):
            return cls(d["vocab"], d["width"], d["heads"], d["decay"], d["eps"])

        def to_dict(self):
            return dict(dataclasses.asdict(self), architectures=["ToyLM"])

        def layer_specs(self):
            norm = PartSpec("layernorm", {"size": self.width, "eps": self.eps})
            ff = PartSpec("dense_mlp", dict(hidden_size=self.width, inner_size=2 * self.width, activation="gelu_erf",
                                            bias=False, weight_layout="out_in", names={"up": "up", "down": "down"}))
            att = PartSpec("causal_attention", dict(
                hidden_size=self.width, n_heads=self.heads, n_kv_heads=1, head_dim=self.width // self.heads,
                scale=1.0 / math.sqrt(self.width // self.heads), window=None, bias=False, weight_layout="out_in",
                names={"qkv": "qkv", "out": "o"}))
            mean = PartSpec("toy_running_mean", {"size": self.width, "decay": self.decay})
            scale_norm = PartSpec("toy_scale_norm", {"size": self.width, "eps": 10 * self.eps})
            # the first layer's two norms differ in kind; the second layer has no feed-forward
            return [LayerSpec("pre_norm", att, ff, (norm, scale_norm), "l0.", ("n1", "n2")),
                    LayerSpec("pre_norm", mean, None, norm, "l1.", ("n1", "n2"))]

        def layer_order(self):
            return [LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 0, write=False)]

    def build(config, dtype, device):
        emb = TokenEmbedding(config.vocab, config.width, "emb", dtype, device)
        layers, prefixes = build_layers(config.layer_specs(), dtype, device)
        final = LayerNorm(size=config.width, eps=config.eps, dtype=dtype, device=device)
        return DecoderModel(config, emb, NoPositions(dtype, device), layers, prefixes, config.layer_order(),
                            final, "final", TiedHead(emb, dtype, device), dtype, device)

    register_architecture("ToyLM", ToyConfig, build, replace=True)
    return ToyConfig


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
    from safetensors import safe_open
    from mini_llm_amd import write_random_model
    from mini_llm_amd.cache.manager import KVCacheSpec, StateCacheSpec
    from mini_llm_amd.engine.step import ModelRunner, StepEntry
    from mini_llm_amd.models import load_model
    _define_toy()
    cfg = dict(architectures=["ToyLM"], vocab=203, width=48, heads=3, decay=0.75, eps=1e-5)
    d = write_random_model(cfg, str(tmp_path / "toy"), seed=3)
    model = load_model(d, dtype, DEV)
    assert [type(s) for s in model.cache_specs()] == [KVCacheSpec, StateCacheSpec]
    runner = ModelRunner(model, page_size=4, n_pages=24, max_num_seqs=3)
    runner.cache.poison()
    assert runner.cache.n_groups == 1 and runner.cache.view(1).slots.shape == (3, 48)
    with safe_open(d + "/model.safetensors", framework="pt") as f:
        w = {k: f.get_tensor(k).double() for k in f.keys()}
    g = torch.Generator().manual_seed(0)
    seqs = {1: torch.randint(0, 203, (30,), generator=g).tolist(), 2: torch.randint(0, 203, (19,), generator=g).tolist(),
            3: torch.randint(0, 203, (9,), generator=g).tolist()}
    got = {r: [] for r in seqs}
    fed = {r: 0 for r in seqs}
    plan = [{1: 7, 2: 3}, {1: 1, 2: 9}, {2: 1, 3: 4}, {1: 12, 2: 1, 3: 1}, {1: 10, 2: 5, 3: 4}]
    for step in plan:
        entries = [StepEntry(r, seqs[r][fed[r]:fed[r] + n], list(range(n))) for r, n in step.items()]
        logits = runner.step(entries).float().cpu()
        i = 0
        for r, n in step.items():
            got[r].append(logits[i:i + n])
            i += n
            fed[r] += n
    tol = 3e-5 if dtype == "float32" else 4e-2
    for r, ids in seqs.items():
        assert fed[r] == len(ids)
        ref = _toy_plain(w, cfg, ids)
        assert (torch.cat(got[r]).double() - ref).abs().max() <= tol, r
    assert model.graph_safe and runner.use_graphs
    # a slot that is used again starts from an empty state (the storage clears it on the device)
    runner.end_request(3)
    runner.cache.poison()
    out = runner.step([StepEntry(4, seqs[3], list(range(9)))]).float().cpu()
    assert (out.double() - _toy_plain(w, cfg, seqs[3])).abs().max() <= tol


def test_stateful_toy_mixer_decodes_through_captured_graphs(tmp_path):
    """The toy model's decode steps run as HIP graphs of 16 rows for 9 requests: the 7 padding rows
    and the run that precedes the capture must leave every request's state alone, a state slot
    must be empty when its request begins, and tokens must equal greedy decoding of the plain
    whole-sequence implementation."""
    from safetensors import safe_open
    from mini_llm_amd import Engine, EngineOptions, SamplingParams, write_random_model
    from mini_llm_amd.models import load_model
    _define_toy()
    cfg = dict(architectures=["ToyLM"], vocab=203, width=48, heads=3, decay=0.75, eps=1e-5)
    d = write_random_model(cfg, str(tmp_path / "toy"), seed=5)
    with safe_open(d + "/model.safetensors", framework="pt") as f:
        w = {k: f.get_tensor(k).double() for k in f.keys()}
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, 203, (3 + i,), generator=g).tolist() for i in range(9)]
    new = 7

    def plain_greedy(ids):
        ids, out = list(ids), []
        for _ in range(new):
            logits = _toy_plain(w, cfg, ids)[-1]
            top = torch.topk(logits, 2).values
            out.append((int(logits.argmax()), float(top[0] - top[1])))
            ids.append(out[-1][0])
        return out

    engine = Engine(load_model(d, "float32", DEV), EngineOptions(kv_block_size=4, total_kv_blocks=64, max_batch_num=12,
                                                                max_tokens_per_step=64, prefill_chunk=8))
    engine.runner.cache.poison()
    assert engine.runner.use_graphs
    for round_ in range(2):                       # the second round reuses slots that hold old states
        outs = engine.generate(prompts, SamplingParams(max_new_tokens=new, ignore_eos=True))
        assert any(k[0] == 16 for k in engine.runner._graphs), "no 16-row decode graph was used"
        for p, o in zip(prompts, outs):
            for i, (tok, gap) in enumerate(plain_greedy(p)):
                assert o[i] == tok or gap < 1e-4, (round_, p, i, o, tok)
                if o[i] != tok:
                    break


# ---------------------------------------------------------------------------------------------
# A second toy architecture: a position encoding that turns queries and keys inside the mixer
# (no table at the embedding), a feed-forward that routes every token to one of several experts
# in the first layer and a dense one in the second, grouped heads, a window in the second layer.
# The toy parts compute with torch; the framework's own parts around them run their kernels.
# ---------------------------------------------------------------------------------------------

def _define_routed_toy():
    from mini_llm_amd.config.base import LayerCall, LayerSpec, ModelConfig, PartSpec
    from mini_llm_amd.config.registry import register_architecture
    from mini_llm_amd.models.decoder import DecoderModel, build_layers
    from mini_llm_amd.parts.base import (FeedForward, ParamSpec, PositionEncoding, register_feed_forward,
                                         register_position)
    from mini_llm_amd.parts.embedding import TiedHead, TokenEmbedding
    from mini_llm_amd.parts.norms import LayerNorm

    @register_position("toy_half_turn", replace=True)
    class HalfTurn(PositionEncoding):
        """Per head, the pair (v[i], v[i + dh/2]) is turned by the angle pos * base^(-i / (dh/2))."""
        applies_in_mixer = True
        max_positions = None

        def __init__(self, base, dtype, device):
            super().__init__(dtype, device)
            self.base = base

        def in_mixer(self, qkv, mixer, ctx):
            dh, half = mixer.head_dim, mixer.head_dim // 2
            rate = self.base ** (-torch.arange(half, device=qkv.device, dtype=torch.float32) / half)
            angle = ctx.positions[:qkv.shape[0]].float()[:, None, None] * rate
            cos, sin = angle.cos(), angle.sin()
            qk = qkv[:, :mixer.q_dim + mixer.kv_dim].view(qkv.shape[0], -1, dh)
            a, b = qk[..., :half].float(), qk[..., half:].float()
            turned = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)   # before qk is written
            qk.copy_(turned)

    @register_feed_forward("toy_one_of_n", replace=True)
    class OneOfN(FeedForward):
        """p = softmax(h R^T) in fp32; the token goes to expert e = argmax p and
        x += p_e * W2_e gelu(W1_e h)."""

        def __init__(self, size, inner, n_experts, dtype, device):
            super().__init__(dtype, device)
            self.size, self.inner, self.n = size, inner, n_experts
            self.router, self.up, self.down = None, [None] * n_experts, [None] * n_experts

        def param_specs(self, prefix):
            def put(lst, e):
                return lambda t: lst.__setitem__(e, t)
            specs = [ParamSpec(prefix + "router", (self.n, self.size), "vector",
                               lambda t: setattr(self, "router", t), (0.0, 1.0))]
            for e in range(self.n):
                specs.append(ParamSpec(f"{prefix}expert.{e}.up", (self.inner, self.size), "matrix", put(self.up, e)))
                specs.append(ParamSpec(f"{prefix}expert.{e}.down", (self.size, self.inner), "matrix", put(self.down, e)))
            return specs

        def forward(self, h, ctx, x):
            p = torch.softmax(h.float() @ self.router.t(), dim=-1)
            gate, chosen = p.max(dim=-1)
            for e in range(self.n):
                y = torch.nn.functional.gelu(h @ self.up[e].t()) @ self.down[e].t()
                x += (gate * (chosen == e))[:, None] * y.float()

    @dataclasses.dataclass(frozen=True)
    class RoutedConfig(ModelConfig):
        vocab: int
        width: int
        heads: int
        groups: int
        experts: int
        window: int
        base: float
        eps: float
        architecture = "ToyRoutedLM"

        @property
        def vocab_size(self):
            return self.vocab

        @property
        def hidden_size(self):
            return self.width

        @classmethod
        def from_dict(cls, d):
            return cls(*(d[k] for k in ("vocab", "width", "heads", "groups", "experts", "window", "base", "eps")))

        def to_dict(self):
            return dict(dataclasses.asdict(self), architectures=["ToyRoutedLM"])

        def layer_specs(self):
            dh = self.width // self.heads
            norm = PartSpec("layernorm", {"size": self.width, "eps": self.eps})
            dense = PartSpec("dense_mlp", dict(hidden_size=self.width, inner_size=3 * self.width, activation="gelu_tanh",
                                               bias=True, weight_layout="out_in", names={"up": "up", "down": "down"}))
            routed = PartSpec("toy_one_of_n", dict(size=self.width, inner=2 * self.width, n_experts=self.experts))
            att = lambda window: PartSpec("causal_attention", dict(
                hidden_size=self.width, n_heads=self.heads, n_kv_heads=self.groups, head_dim=dh,
                scale=1.0 / math.sqrt(dh), window=window, bias=True, weight_layout="out_in",
                names={"qkv": "qkv", "out": "o"}))
            return [LayerSpec("pre_norm", att(None), routed, norm, "l0.", ("n1", "n2")),
                    LayerSpec("pre_norm", att(self.window), dense, norm, "l1.", ("n1", "n2"))]

        def layer_order(self):
            return [LayerCall(0, 0), LayerCall(1, 1)]

    def build(config, dtype, device):
        emb = TokenEmbedding(config.vocab, config.width, "emb", dtype, device)
        turn = HalfTurn(config.base, dtype, device)
        layers, prefixes = build_layers(config.layer_specs(), dtype, device, position=turn)
        final = LayerNorm(size=config.width, eps=config.eps, dtype=dtype, device=device)
        return DecoderModel(config, emb, turn, layers, prefixes, config.layer_order(),
                            final, "final", TiedHead(emb, dtype, device), dtype, device)

    register_architecture("ToyRoutedLM", RoutedConfig, build, replace=True)


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
ROUTED_SEED = 35


def _routed_sequences():
    g = torch.Generator().manual_seed(ROUTED_SEED)
    return {1: torch.randint(0, 157, (26,), generator=g).tolist(), 2: torch.randint(0, 157, (15,), generator=g).tolist()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_turned_keys_and_routed_experts(tmp_path, dtype):
    from safetensors import safe_open
    from mini_llm_amd import write_random_model
    from mini_llm_amd.engine.step import ModelRunner, StepEntry
    from mini_llm_amd.models import load_model
    _define_routed_toy()
    d = write_random_model(ROUTED_CFG, str(tmp_path / "routed"), seed=ROUTED_SEED)
    model = load_model(d, dtype, DEV)
    assert all(layer.mixer.position is model.position for layer in model.layers)
    runner = ModelRunner(model, page_size=4, n_pages=14, max_num_seqs=2)
    runner.cache.poison()
    with safe_open(d + "/model.safetensors", framework="pt") as f:
        w = {k: f.get_tensor(k).double() for k in f.keys()}
    seqs = _routed_sequences()
    got, fed = {r: [] for r in seqs}, {r: 0 for r in seqs}
    plan = [{1: 9, 2: 2}, {1: 1, 2: 6}, {1: 1}, {1: 13, 2: 1}, {1: 2, 2: 6}]
    for step in plan:
        entries = [StepEntry(r, seqs[r][fed[r]:fed[r] + n], list(range(n))) for r, n in step.items()]
        logits = runner.step(entries).float().cpu()
        i = 0
        for r, n in step.items():
            got[r].append(logits[i:i + n])
            i += n
            fed[r] += n
    tol = 3e-5 if dtype == "float32" else 4e-2
    for r, ids in seqs.items():
        assert fed[r] == len(ids)
        ref, gap, used = _routed_plain(w, ROUTED_CFG, ids)
        assert gap > 0.3 and len(used) >= 2, "the seed gives a near tie between experts, or one expert only"
        assert (torch.cat(got[r]).double() - ref).abs().max() <= tol, r
