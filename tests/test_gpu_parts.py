"""Each part alone against the plain implementation, and a model put together from other
parts than Llama's: a toy mixer with state of its own (defined here, registered from outside),
a windowed attention layer, a learned position table, a layer that runs twice and a layer that
reads another layer's cache.  None of this touches the framework's files."""
import json
import math
import os
from dataclasses import dataclass
from typing import Dict

import numpy as np
import pytest
import torch

import plain_llama as P
from helpers import TOL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def rt32():
    from rustinfer_amd.engine import make_runtime
    return make_runtime("float32", DEV)


@pytest.fixture(scope="module")
def rt16():
    from rustinfer_amd.engine import make_runtime
    return make_runtime("bfloat16", DEV)


def t64(a):
    return torch.tensor(a, dtype=torch.float64)


class OnePart:
    """The least a 'model' must be for the engine to build a step context around one mixer."""
    vocab_size = 100

    def __init__(self, mixer, pos_encs=()):
        self.mixer, self.pos_encs = mixer, list(pos_encs)

    def prepare(self, rt, max_positions):
        for pe in self.pos_encs:
            pe.prepare(rt, max_positions)

    def cache_needs(self):
        return {0: self.mixer.cache_need()}


def test_rmsnorm_part(rt32, rt16):
    from rustinfer_amd.parts import RMSNorm
    for rt, tol in ((rt32, 1e-5), (rt16, 2e-2)):
        norm = RMSNorm(200, 1e-6)
        assert norm.param_specs()["weight"].shape == (200,)
        w = 1 + 0.1 * torch.randn(200)
        norm.load({"weight": w}, rt)
        assert norm.weight.dtype == torch.float32          # stored in 32-bit, stays 32-bit
        x = torch.randn(5, 200, device=DEV)
        out = torch.empty(5, 200, device=DEV, dtype=rt.dtype)
        norm.forward(None, x, None, out)
        ref = P.rmsnorm(x.double().cpu().numpy(), w.double().numpy(), 1e-6)
        assert np.max(np.abs(out.double().cpu().numpy() - ref)) < tol
        norm.load({"weight": w.to(torch.bfloat16)}, rt)
        assert norm.weight.dtype == rt.dtype


def test_swiglu_mlp_part(rt32, rt16):
    from rustinfer_amd.engine import Workspace
    from rustinfer_amd.parts import SwiGLUMLP
    from types import SimpleNamespace
    g = torch.Generator().manual_seed(1)
    wt = {n: (torch.randn(s, generator=g) * 0.1).to(torch.bfloat16) for n, s in
          (("gate_proj.weight", (72, 40)), ("up_proj.weight", (72, 40)), ("down_proj.weight", (40, 72)))}
    x = torch.randn(11, 40, generator=g).to(torch.bfloat16)
    ref = P.swiglu_mlp(*(a.double().numpy() for a in (x, wt["gate_proj.weight"], wt["up_proj.weight"], wt["down_proj.weight"])))
    for rt, tol in ((rt32, 1e-5), (rt16, 2e-2)):
        mlp = SwiGLUMLP(40, 72)
        assert {k: v.shape for k, v in mlp.param_specs().items()} == {k: tuple(v.shape) for k, v in wt.items()}
        mlp.load(wt, rt)
        ctx = SimpleNamespace(workspace=Workspace(rt.device))
        out = mlp.forward(ctx, x.to(DEV, rt.dtype))
        assert np.max(np.abs(out.double().cpu().numpy() - ref)) < tol


def test_embedding_and_output_head_parts(rt32, rt16):
    """The embedding writes rows of its table into the 32-bit residual stream; the head gives
    32-bit logits, from a matrix of its own or (tied) from the embedding's table."""
    from rustinfer_amd.parts import Embedding, LMHead
    from types import SimpleNamespace
    g = torch.Generator().manual_seed(2)
    V, d = 301, 72
    table = (torch.randn(V, d, generator=g) * 0.5).to(torch.bfloat16)
    head_w = (torch.randn(V, d, generator=g) * 0.1).to(torch.bfloat16)
    ids = torch.tensor([5, 0, 300, 5, 17], dtype=torch.int32, device=DEV)
    x_in = torch.randn(4, d, generator=g).to(torch.bfloat16)
    for rt, tol in ((rt32, 1e-5), (rt16, 2e-2)):
        emb = Embedding(V, d)
        assert emb.param_specs()["weight"].shape == (V, d)
        emb.load({"weight": table}, rt)
        x = torch.full((5, d), 9.0, device=DEV)
        emb.forward(SimpleNamespace(), ids, x)
        assert torch.equal(x.cpu(), table.float()[ids.long().cpu()])           # exact: a copy
        own = LMHead(V, d)
        assert own.param_specs()["weight"].shape == (V, d)
        own.load({"weight": head_w}, rt)
        tied = LMHead(V, d, tied_to=emb)
        assert tied.param_specs() == {}
        tied.load({}, rt)
        for head, w in ((own, head_w), (tied, table)):
            logits = torch.empty(4, V, device=DEV)
            head.forward(None, x_in.to(DEV, rt.dtype), logits)
            ref = x_in.double().numpy() @ w.double().numpy().T
            assert logits.dtype == torch.float32
            assert np.max(np.abs(logits.double().cpu().numpy() - ref)) < tol * max(1.0, np.abs(ref).max())


def test_block_part_keeps_the_sum_pending(rt32):
    """The pre-norm block alone: x <- x + mixer(norm1(x)); x <- x + ffn(norm2(x)), with the second
    sub-layer's output left pending for whoever normalises next; and the same block cut down to
    chosen rows after its mixer."""
    from rustinfer_amd.engine import Workspace
    from rustinfer_amd.parts import Mixer, ParamSpec, PreNormBlock, RMSNorm, SwiGLUMLP
    from rustinfer_amd.parts.block import Hidden
    from types import SimpleNamespace

    class Doubler(Mixer):                      # a mixer without weights or cache: 2 * its input
        def param_specs(self): return {}
        def load(self, tensors, rt): self.rt = rt
        def cache_need(self): return None
        def forward(self, ctx, normed, cache): return (normed * 2).contiguous()

    g = torch.Generator().manual_seed(3)
    d, I, T = 40, 72, 9
    blk = PreNormBlock(d, RMSNorm(d, 1e-5), Doubler(), RMSNorm(d, 1e-6), SwiGLUMLP(d, I))
    specs = blk.param_specs()
    assert sorted(specs) == ["input_layernorm.weight", "mlp.down_proj.weight", "mlp.gate_proj.weight",
                             "mlp.up_proj.weight", "post_attention_layernorm.weight"]
    wt = {n: (1 + 0.1 * torch.randn(sp.shape, generator=g)) if "norm" in n else torch.randn(sp.shape, generator=g) * 0.1
          for n, sp in specs.items()}
    blk.load(wt, rt32)
    w = {n: t.double().numpy() for n, t in wt.items()}
    x0 = torch.randn(T, d, generator=g)
    xn = x0.double().numpy()
    h1 = xn + 2 * P.rmsnorm(xn, w["input_layernorm.weight"], 1e-5)
    delta = P.swiglu_mlp(P.rmsnorm(h1, w["post_attention_layernorm.weight"], 1e-6), w["mlp.gate_proj.weight"],
                         w["mlp.up_proj.weight"], w["mlp.down_proj.weight"])
    ctx = SimpleNamespace(workspace=Workspace(rt32.device))
    hidden = Hidden(x0.to(DEV).clone())
    blk.forward(ctx, hidden, None)
    assert np.max(np.abs(hidden.x.double().cpu().numpy() - h1)) < 1e-5          # the first sum is made
    pend = hidden.pending.double().cpu().numpy()
    assert np.max(np.abs((pend.sum(0) if pend.ndim == 3 else pend) - delta)) < 1e-5   # the second waits
    rows = torch.tensor([7, 2], dtype=torch.int32, device=DEV)
    hidden = Hidden(x0.to(DEV).clone())
    assert blk.can_cut_rows()
    blk.forward(ctx, hidden, None, out_rows=rows)
    assert tuple(hidden.x.shape) == (2, d)
    pend = hidden.pending.double().cpu().numpy()
    got = hidden.x.double().cpu().numpy() + (pend.sum(0) if pend.ndim == 3 else pend)
    assert np.max(np.abs(got - (h1 + delta)[[7, 2]])) < 1e-5


def test_rotary_tables(rt32):
    from rustinfer_amd.config import RopeScaling
    from rustinfer_amd.parts import RotaryEmbedding
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=32)
    pe = RotaryEmbedding(32, 500000.0, RopeScaling(**sc))
    pe.prepare(rt32, 300)
    cos, sin, rot = pe.rotary()
    f = P.rope_frequencies(32, 500000.0, sc)
    ang = np.arange(300)[:, None] * f[None, :]
    assert rot == 32 and cos.shape == (300, 16) and cos.dtype == torch.float32
    assert np.max(np.abs(cos.double().cpu().numpy() - np.cos(ang))) < 1e-7
    assert np.max(np.abs(sin.double().cpu().numpy() - np.sin(ang))) < 1e-7


@pytest.mark.parametrize("H,Hkv,hd,window", [(4, 2, 16, None), (5, 1, 32, None), (6, 3, 48, 7)])
def test_attention_part_over_the_cache(rt32, H, Hkv, hd, window):
    """The attention mixer alone, a sequence cut into three steps, against rotation + causal
    attention + projections computed plainly on the whole sequence."""
    from rustinfer_amd.engine import Engine, StepEntry
    from rustinfer_amd.parts import PagedAttention, RotaryEmbedding
    d, T = 72, 37
    g = torch.Generator().manual_seed(H)
    pe = RotaryEmbedding(hd, 10000.0)
    att = PagedAttention(d, H, Hkv, hd, pos_enc=pe, window=window)
    wt = {n: (torch.randn(s.shape, generator=g) * 0.2) for n, s in att.param_specs().items()}
    att.load(wt, rt32)
    eng = Engine(OnePart(att, [pe]), rt32, page_size=8, num_pages=16, max_requests=2, max_model_len=64)
    x = torch.randn(T, d, generator=g)
    xn = x.double().numpy()
    f = P.rope_frequencies(hd, 10000.0, None)
    q = P.rope((xn @ wt["q_proj.weight"].double().numpy().T).reshape(T, H, hd), np.arange(T), f)
    k = P.rope((xn @ wt["k_proj.weight"].double().numpy().T).reshape(T, Hkv, hd), np.arange(T), f)
    v = (xn @ wt["v_proj.weight"].double().numpy().T).reshape(T, Hkv, hd)
    ref = P.attention(q, k, v, 1 / math.sqrt(hd), window).reshape(T, H * hd) @ wt["o_proj.weight"].double().numpy().T
    eng.cache.add_request("r")
    pos = 0
    for n in (20, 1, 16):
        start = eng.cache.append("r", n)
        ctx = eng._build_context([StepEntry("r", [0] * n, [])], [start])
        out = att.forward(ctx, x[pos:pos + n].to(DEV), eng.cache.view(0))
        # outputs are of size |ref|; 32-bit rounding is relative to that
        assert np.max(np.abs(out.double().cpu().numpy() - ref[pos:pos + n])) < 4e-6 * max(1.0, np.abs(ref).max())
        pos += n


# ---------------------------------------------------------------------------
# a toy architecture, registered from outside
# ---------------------------------------------------------------------------
def define_toy(state_on_device=False, state_last=False):
    """``state_on_device``: the state mixer reads the step's device tensors only (and may be
    captured in a graph) instead of walking the host's lists (and saying that it may not).
    ``state_last``: the layer with the state mixer runs last instead of second."""
    from rustinfer_amd.config import ModelConfig, register_architecture, unregister_architecture
    from rustinfer_amd.models import DecoderModel, LayerCall
    from rustinfer_amd.parts import (Embedding, FeedForward, LMHead, Mixer, PagedAttention, ParamSpec,
                                     PositionEncoding, PreNormBlock, RMSNorm, RotaryEmbedding, StateNeed,
                                     SwiGLUMLP, register_feed_forward, register_mixer, make_part)

    class DecayStateMixer(Mixer):
        """s_t = decay * s_(t-1) + x_t for each request; out_t = s_t W^T.  The state lives in
        the cache manager's slot of the request; the first portion of a request starts from zero."""

        def __init__(self, hidden_size, decay):
            self.d, self.decay = hidden_size, decay
            self.graph_safe = state_on_device       # the host-list form depends on more than the batch's shape

        def param_specs(self):
            # a decay for each channel, drawn uniformly around the configured one: a parameter that is
            # neither a matrix nor a norm weight, so the spec brings its own distribution
            lo, hi = self.decay - 0.15, self.decay + 0.15
            return {"out_proj.weight": ParamSpec((self.d, self.d)),
                    "decay": ParamSpec((self.d,), init=lambda g, shape, device: lo + (hi - lo) * torch.rand(
                        shape, generator=g, device=device, dtype=torch.float32))}

        def cache_need(self):
            return StateNeed((self.d,), torch.float32)

        def load(self, tensors, rt):
            self.rt = rt
            self.w = tensors["out_proj.weight"].to(rt.device, torch.float32)
            self.decay_vec = tensors["decay"].to(rt.device, torch.float32)

        def forward(self, ctx, normed, cache):
            out = ctx.workspace.get("toy.out", normed.shape[0], self.d, self.rt.dtype)
            if state_on_device:
                # the same kernels with the same arguments whatever the rows hold: a token of no
                # request (row -1) works on the slot its row points at, the scratch slot
                T = normed.shape[0]
                rows = ctx.row_of_token[:T].long()
                pad_slot = torch.full_like(rows, cache.state.shape[0] - 1)
                slot = torch.where(rows >= 0, ctx.state_slots.long()[rows.clamp(min=0)], pad_slot)
                keep = (ctx.positions[:T] != 0).float()                  # a request's first token starts from zero
                for i in range(T):
                    s = cache.state.index_select(0, slot[i:i + 1]) * (keep[i] * self.decay_vec) + normed[i].float()
                    cache.state.index_copy_(0, slot[i:i + 1], s)
                    out[i] = (s[0] @ self.w.T).to(out.dtype)
                return out
            t = 0
            for q, start, slot in zip(ctx.host_q_lens, ctx.host_q_start, ctx.host_slots):
                s = cache.state[slot]
                if start == 0:
                    s.zero_()
                for i in range(t, t + q):
                    s.mul_(self.decay_vec).add_(normed[i].float())
                    out[i] = (self.w @ s).to(out.dtype)
                t += q
            return out

    class HeadNorm:
        """What a variant of the attention mixer does between projection and rotation: an RMS norm
        over each head of q and of k with one learned weight of head size (32-bit arithmetic)."""

        def __init__(self, head_dim, eps):
            self.hd, self.eps = head_dim, eps

        def param_specs(self):
            return {"qk_norm.weight": ParamSpec((self.hd,), mean=1.0, std=0.1)}

        def load(self, tensors, rt):
            self.w = tensors["qk_norm.weight"].to(rt.device, torch.float32)

        def __call__(self, ctx, qkv, attn):
            T = qkv.shape[0]
            n = (attn.num_heads + attn.num_kv_heads) * self.hd          # queries and keys, head after head
            x = qkv[:, :n].float().view(T, -1, self.hd)
            x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.eps) * self.w
            qkv[:, :n] = x.view(T, n).to(qkv.dtype)

    class RoutedExperts(FeedForward):
        """A router and a few experts: out_t = sum_e softmax(R n_t)_e * (W_e n_t), the router's
        logits and weights in 32-bit.  (Every expert takes part, weighted: a toy, but with a router's
        and experts' tensors of its own.)"""

        def __init__(self, hidden_size, num_experts):
            self.d, self.E = hidden_size, num_experts

        def param_specs(self):
            specs = {"router.weight": ParamSpec((self.E, self.d))}
            specs.update({f"experts.{e}.weight": ParamSpec((self.d, self.d)) for e in range(self.E)})
            return specs

        def load(self, tensors, rt):
            self.rt = rt
            self.router = tensors["router.weight"].to(rt.device, torch.float32)
            self.experts = [tensors[f"experts.{e}.weight"].to(rt.device, torch.float32) for e in range(self.E)]

        def forward(self, ctx, normed):
            x = normed.float()
            p = torch.softmax(x @ self.router.T * 8.0, dim=-1)
            out = sum(p[:, e:e + 1] * (x @ w.T) for e, w in enumerate(self.experts))
            return out.to(self.rt.dtype)

    class LearnedPositions(PositionEncoding):
        """A table added to the embedded tokens."""

        def __init__(self, max_positions, dim):
            self.n, self.dim = max_positions, dim

        def param_specs(self):
            return {"weight": ParamSpec((self.n, self.dim))}

        def load(self, tensors, rt):
            self.rt = rt
            self.table = tensors["weight"].to(rt.device, torch.float32)

        def on_embedding(self, ctx, x):
            x += self.table[ctx.positions[:x.shape[0]].long()]

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        hidden_size: int = 48
        vocab_size: int = 90
        num_heads: int = 3
        num_kv_heads: int = 1
        head_dim: int = 16
        intermediate_size: int = 56
        window: int = 5
        num_experts: int = 3
        decay: float = 0.75
        eps: float = 1e-5
        max_position_embeddings: int = 96
        architecture: str = "ToyForCausalLM"

        @classmethod
        def from_dict(cls, d, where="config.json"):
            return cls(**{k: v for k, v in d.items() if k in cls.__dataclass_fields__ and k != "architecture"})

        def to_dict(self):
            d = {k: getattr(self, k) for k in self.__dataclass_fields__ if k != "architecture"}
            d["architectures"] = [self.architecture]
            return d

    register_mixer("toy_decay_state", DecayStateMixer, replace=True)
    register_feed_forward("toy_routed_experts", RoutedExperts, replace=True)

    class ToyModel(DecoderModel):
        """Adds the learned position table to the checkpoint names."""

        def _children(self):
            yield from super()._children()
            yield "model.positions", self.position_encodings[1]

    def build_toy(c):
        d = c.hidden_size
        rope = RotaryEmbedding(c.head_dim, 10000.0)
        learned = LearnedPositions(c.max_position_embeddings, d)
        norm = lambda: RMSNorm(d, c.eps)
        attn = lambda **kw: PagedAttention(d, c.num_heads, c.num_kv_heads, c.head_dim, pos_enc=rope, **kw)
        layers = [
            PreNormBlock(d, norm(), attn(), norm(), SwiGLUMLP(d, c.intermediate_size)),
            PreNormBlock(d, norm(), make_part("mixer", "toy_decay_state", hidden_size=d, decay=c.decay),
                         norm(), SwiGLUMLP(d, c.intermediate_size)),
            PreNormBlock(d, norm(), attn(window=c.window, qk_transform=HeadNorm(c.head_dim, c.eps)), norm(),
                         make_part("feed_forward", "toy_routed_experts", hidden_size=d, num_experts=c.num_experts)),
            PreNormBlock(d, norm(), attn(own_kv=False), norm(), SwiGLUMLP(d, c.intermediate_size)),
        ]
        schedule = [LayerCall(0), LayerCall(1), LayerCall(2), LayerCall(0, cache=3),
                    LayerCall(3, cache=0, write=False)]
        if state_last:
            schedule = [schedule[0]] + schedule[2:] + [schedule[1]]
        embed = Embedding(c.vocab_size, d)
        return ToyModel(c, embed, layers, norm(), LMHead(c.vocab_size, d, tied_to=embed),
                        position_encodings=[rope, learned], schedule=schedule)

    register_architecture("ToyForCausalLM", ToyConfig, build_toy, replace=True)
    return ToyConfig, (lambda: unregister_architecture("ToyForCausalLM"))


def toy_plain_forward(c, w, ids, state_last=False):
    """The toy model on a whole sequence, from the plain parts."""
    T, d, H, Hkv, hd = len(ids), c.hidden_size, c.num_heads, c.num_kv_heads, c.head_dim
    pos = np.arange(T)
    f = P.rope_frequencies(hd, 10000.0, None)
    x = P.embedding(w["model.embed_tokens.weight"], ids) + w["model.positions.weight"][:T]
    kv0 = {}

    def attn(x, p, window=None, shared=None, keep=None, head_norm=None):
        n = P.rmsnorm(x, w[p + "input_layernorm.weight"], c.eps)
        hn = (lambda a: P.rmsnorm(a, head_norm, c.eps)) if head_norm is not None else (lambda a: a)
        q = P.rope(hn((n @ w[p + "self_attn.q_proj.weight"].T).reshape(T, H, hd)), pos, f)
        if shared is None:
            k = P.rope(hn((n @ w[p + "self_attn.k_proj.weight"].T).reshape(T, Hkv, hd)), pos, f)
            v = (n @ w[p + "self_attn.v_proj.weight"].T).reshape(T, Hkv, hd)
        else:
            k, v = shared
        if keep is not None:
            keep["kv"] = (k, v)
        o = P.attention(q, k, v, 1 / math.sqrt(hd), window).reshape(T, H * hd)
        return x + o @ w[p + "self_attn.o_proj.weight"].T

    def mlp(x, p):
        n = P.rmsnorm(x, w[p + "post_attention_layernorm.weight"], c.eps)
        return x + P.swiglu_mlp(n, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

    def state_layer(x):
        n = P.rmsnorm(x, w["model.layers.1.input_layernorm.weight"], c.eps)
        s, outs = np.zeros(d), []
        for t in range(T):
            s = w["model.layers.1.self_attn.decay"] * s + n[t]
            outs.append(w["model.layers.1.self_attn.out_proj.weight"] @ s)
        return mlp(x + np.stack(outs), "model.layers.1.")

    x = mlp(attn(x, "model.layers.0.", keep=kv0), "model.layers.0.")
    if not state_last:
        x = state_layer(x)
    x = attn(x, "model.layers.2.", window=c.window, head_norm=w["model.layers.2.self_attn.qk_norm.weight"])
    n = P.rmsnorm(x, w["model.layers.2.post_attention_layernorm.weight"], c.eps)
    p = P.softmax(n @ w["model.layers.2.mlp.router.weight"].T * 8.0)
    x = x + sum(p[:, e:e + 1] * (n @ w[f"model.layers.2.mlp.experts.{e}.weight"].T) for e in range(c.num_experts))
    x = mlp(attn(x, "model.layers.0."), "model.layers.0.")                   # layer 0 again, own cache
    x = mlp(attn(x, "model.layers.3.", shared=kv0["kv"]), "model.layers.3.")  # reads the first call's cache
    if state_last:
        x = state_layer(x)
    return P.rmsnorm(x, w["model.norm.weight"], c.eps) @ w["model.embed_tokens.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_registers_builds_and_steps(tmp_path, dtype):
    from rustinfer_amd.engine import StepEntry, build_engine
    from rustinfer_amd.weights import write_random_model
    ToyConfig, undo = define_toy()
    try:
        c = ToyConfig()
        d = write_random_model(c, 3, str(tmp_path))
        assert json.load(open(os.path.join(d, "config.json")))["architectures"] == ["ToyForCausalLM"]
        w = P.read_safetensors(os.path.join(d, "model.safetensors"))
        assert "model.layers.3.self_attn.k_proj.weight" not in w and "model.positions.weight" in w
        eng = build_engine(d, dtype=dtype, page_size=4, num_pages=40, max_requests=2, max_model_len=96)
        assert len(eng.cache.groups) == 2 and sorted(eng.cache.state_tensors) == [1]   # full + windowed pages, one state
        rng = np.random.default_rng(0)
        seqs = {r: rng.integers(0, c.vocab_size, n).tolist() for r, n in (("a", 41), ("b", 23), ("c", 30))}
        ref = {r: toy_plain_forward(c, w, s) for r, s in seqs.items()}
        tol = TOL[dtype]
        # a and b interleaved in portions; then c takes b's slot and pages (state must restart at zero)
        plan = [[("a", 7), ("b", 2)], [("a", 1), ("b", 9)], [("a", 13)], [("b", 1), ("a", 1)],
                [("b", 11), ("a", 19)], ["end b"], [("c", 5)], [("c", 1)], [("c", 24)]]
        pos = {r: 0 for r in seqs}
        for step in plan:
            if step == ["end b"]:
                eng.release("b")
                continue
            ents = [StepEntry(r, seqs[r][pos[r]:pos[r] + n], list(range(n))) for r, n in step]
            lg = eng.step(ents).double().cpu().numpy()
            row = 0
            for r, n in step:
                diff = np.max(np.abs(lg[row:row + n] - ref[r][pos[r]:pos[r] + n]))
                assert diff <= tol, (dtype, r, pos[r], n, diff)
                row += n
                pos[r] += n
            eng.cache.check()
        assert pos == {r: len(s) for r, s in seqs.items()}
        assert eng.cache.slot("c") == 1                                   # b's slot, used again
        win = eng.cache.table(1, "a")
        assert any(p == -1 for p in win) and all(p >= 0 for p in eng.cache.table(0, "a"))  # the window gave pages back
    finally:
        undo()


@pytest.mark.parametrize("state_last", [False, True])
def test_portions_whose_logits_nobody_wants_still_move_caches_and_state(tmp_path, state_last):
    """A step that wants no logits runs its last block only as far as later steps need it.  The
    toy's last block reads another call's cache and writes none (nothing to do at all); with
    ``state_last`` it is the block with the state mixer, which has no ``update_cache`` and must run
    whole so that its state moves on.  Logits after such steps are the plain ones."""
    from rustinfer_amd.engine import StepEntry, build_engine
    from rustinfer_amd.weights import write_random_model
    ToyConfig, undo = define_toy(state_last=state_last)
    try:
        c = ToyConfig()
        d = write_random_model(c, 5, str(tmp_path))
        w = P.read_safetensors(os.path.join(d, "model.safetensors"))
        eng = build_engine(d, dtype="float32", page_size=4, num_pages=40, max_requests=2, max_model_len=96)
        rng = np.random.default_rng(2)
        seqs = {r: rng.integers(0, c.vocab_size, n).tolist() for r, n in (("a", 37), ("b", 18))}
        ref = {r: toy_plain_forward(c, w, s, state_last) for r, s in seqs.items()}
        pos = {r: 0 for r in seqs}
        # (request, tokens, whether the last token's logits are wanted)
        plan = [[("a", 9, False)], [("a", 12, False), ("b", 6, False)], [("a", 1, True), ("b", 5, False)],
                [("b", 7, True)], [("a", 15, True)]]
        for step in plan:
            ents = [StepEntry(r, seqs[r][pos[r]:pos[r] + n], [n - 1] if want else []) for r, n, want in step]
            lg = eng.step(ents).double().cpu().numpy()
            row = 0
            for r, n, want in step:
                if want:
                    assert np.max(np.abs(lg[row] - ref[r][pos[r] + n - 1])) <= TOL["float32"], (state_last, step, r)
                    row += 1
                pos[r] += n
            eng.cache.check()
    finally:
        undo()


@pytest.mark.parametrize("state_on_device", [True, False])
def test_toy_architecture_generates_through_the_entry_point_with_graphs(tmp_path, state_on_device):
    """The toy model through ``LLM.generate`` with graphs switched on, as for every model.  A
    state mixer that reads device tensors only is captured (on rows of no request, with the
    scratch slot, so no request's state moves twice for one token) and replayed, padding rows
    included; one that walks the host's lists says ``graph_safe = False`` and every step of the
    model runs eagerly.  Both give the plain implementation's tokens."""
    from rustinfer_amd import LLM, SamplingParams
    from rustinfer_amd.weights import write_random_model
    ToyConfig, undo = define_toy(state_on_device)
    try:
        c = ToyConfig()
        d = write_random_model(c, 4, str(tmp_path))
        w = P.read_safetensors(os.path.join(d, "model.safetensors"))
        rng = np.random.default_rng(1)
        prompts = [rng.integers(0, c.vocab_size, n).tolist() for n in (7, 12, 3)]
        lengths = (10, 5, 8)
        want = []
        for p, n in zip(prompts, lengths):
            toks = list(p)
            for _ in range(n):
                toks.append(int(np.argmax(toy_plain_forward(c, w, toks)[-1])))
            want.append(toks[len(p):])
        llm = LLM(model=d, dtype="float32", paged_block_size=4, num_blocks=60, max_batch_seqs=4,
                  max_model_len=96, capture_sizes=[1, 2, 4], mixed_graph_after=1)
        assert llm.engine.model.graph_safe == state_on_device
        res = llm.generate(prompts, [SamplingParams(max_tokens=n, ignore_eos=True) for n in lengths])
        assert [r.token_ids for r in res] == want
        if state_on_device:
            # three rows pad to four, then two rows, then one
            assert llm.engine.graph_replays >= 8
            assert sorted(k[0] for k in llm.engine._graphs if k[0] != "mixed") == [1, 2, 4]
            # the prompts ran as a captured step too: 22 tokens in three rows, padded to 32 in four
            assert ("mixed", 32, 4, 96, 0, 0) in llm.engine._graphs and llm.engine.mixed_graph_replays >= 1
        else:
            assert llm.engine.graph_replays == 0 and not llm.engine._graphs
        llm.engine.cache.check()
        assert llm.engine.cache.free_pages() == 60
    finally:
        undo()
