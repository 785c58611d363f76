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
# attention layer twice (the second call only reads the cache the first one wrote).
# ---------------------------------------------------------------------------------------------

def _define_toy():
    from mini_llm_amd.cache.manager import StateCacheSpec
    from mini_llm_amd.config.base import LayerCall, LayerSpec, ModelConfig, PartSpec
    from mini_llm_amd.config.registry import register_architecture
    from mini_llm_amd.models.decoder import DecoderModel, build_layers
    from mini_llm_amd.parts.base import MIXERS, Mixer, ParamSpec, register_mixer
    from mini_llm_amd.parts.embedding import NoPositions, TiedHead, TokenEmbedding
    from mini_llm_amd.parts.norms import LayerNorm

    @register_mixer("toy_running_mean", replace=True)
    class RunningMean(Mixer):
        """state <- decay * state + (1 - decay) * h_t, token by token; x_t += gain * state."""
        graph_safe = False           # it walks the batch on the host

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
            for b in range(ctx.n_seqs):
                lo, hi = int(ctx.h_cu_q[b]), int(ctx.h_cu_q[b + 1])
                slot = int(ctx.h_state_slots[b])
                s = cache_view.slots[slot]
                if int(ctx.h_starts[b]) == 0:
                    s.zero_()                      # a new request starts from an empty state
                for t in range(lo, hi):
                    s.mul_(self.decay).add_(h[t].float(), alpha=1 - self.decay)
                    x[t] += self.gain * s

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
            return [LayerSpec("pre_norm", att, ff, norm, "l0.", ("n1", "n2")),
                    LayerSpec("pre_norm", mean, ff, norm, "l1.", ("n1", "n2"))]

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
        x = x + ffn(ln(x, p + "n2"), p)
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
    assert not model.graph_safe and not runner.use_graphs
    # a slot that is used again starts from an empty state
    runner.end_request(3)
    out = runner.step([StepEntry(4, seqs[3], list(range(9)))]).float().cpu()
    assert (out.double() - _toy_plain(w, cfg, seqs[3])).abs().max() <= tol
