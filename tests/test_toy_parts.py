"""Generality of the parts: a toy mixer with state of its own, a toy feed-forward that routes
each row to one of a few experts, a toy position encoding and a toy architecture are defined
*here*, registered, built and stepped without a change to the framework's files.  The toy model
mixes kinds of layers, runs one layer twice and lets one layer read another layer's cache.  It
is nobody's model."""
from dataclasses import dataclass, field
from typing import Mapping

import pytest
import torch

from emulated_ops import EmulatedOps
from plain import qwen2_plain as P

from machserve_amd.config import (AttentionSpec, EmbeddingSpec, GatedMlpSpec, HeadSpec, LayerSpec, ModelSpec, NormSpec,
                                  RotarySpec, register_architecture)
from machserve_amd.parts import (FeedForward, Mixer, PositionEncoding, StateRequest, TensorDecl, register_feed_forward,
                                 register_mixer, register_position_encoding)

WIDTH, HEADS, KV, HD, INTER, VOCAB = 48, 3, 1, 16, 80, 90
EXPERTS, EXPERT_INTER = 3, 24


@dataclass(frozen=True)
class RunningMeanSpec:
    kind: str
    width: int
    tensors: Mapping[str, str] = field(default_factory=dict)


@register_mixer("toy_running_mean")
class RunningMean(Mixer):
    """out_t = W * mean(h_0 .. h_t): causal, and its whole memory is a sum and a count per request."""

    def tensor_decls(self):
        return [TensorDecl("w", (self.spec.width, self.spec.width))]

    def load(self, t):
        self.w = t["w"]

    def cache_request(self):
        return StateRequest({"sum": (self.spec.width,), "count": (1,)})

    def bind_cache(self, binding):
        self.state = binding.tensors

    def forward(self, h, stream, ctx):
        out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
        for slot, q0, n in zip(ctx.host["seq_slot"], ctx.host["seq_q_start"], ctx.host["seq_q_len"]):
            rows = h[q0:q0 + n].float()
            run = self.state["sum"][slot] + torch.cumsum(rows, 0)
            cnt = self.state["count"][slot] + torch.arange(1, n + 1, device=h.device, dtype=torch.float32)[:, None]
            out[q0:q0 + n] = run / cnt
            self.state["sum"][slot] = run[-1]
            self.state["count"][slot] = cnt[-1]
        stream.add(out @ self.w.float().t())


@dataclass(frozen=True)
class RoutedSpec:
    kind: str
    width: int
    experts: int
    inter: int
    tensors: Mapping[str, str] = field(default_factory=dict)


@register_feed_forward("toy_routed")
class Routed(FeedForward):
    """Every row goes to the one expert its router logit (32-bit) is largest for; an expert is
    w2 relu(w1 h).  The router and the experts are the part's own business."""

    def tensor_decls(self):
        sp = self.spec
        return [TensorDecl("router", (sp.experts, sp.width), "vector"), TensorDecl("w1", (sp.experts, sp.inter, sp.width)),
                TensorDecl("w2", (sp.experts, sp.width, sp.inter))]

    def load(self, t):
        self.router, self.w1, self.w2 = t["router"], t["w1"], t["w2"]

    def forward(self, h, stream, ctx):
        x = h.float()
        choice = (x @ self.router.float().t()).argmax(-1)
        out = torch.zeros_like(x)
        for e in range(self.spec.experts):
            rows = choice == e
            out[rows] = torch.relu(x[rows] @ self.w1[e].float().t()) @ self.w2[e].float().t()
        stream.add(out)


@register_position_encoding("toy_position_scale")
class PositionScale(PositionEncoding):
    """q and k of the row at position p are multiplied by 1 + p / 64: not a rotation, so the
    attention part must take the unfused path."""

    def apply(self, q, k, ctx):
        f = (1.0 + ctx.positions.float() / 64.0)[:, None, None]
        q *= f
        if k is not None:
            k *= f


@dataclass
class ToyConfig:
    layers: int = 4

    @classmethod
    def from_dict(cls, raw):
        return cls(raw.get("layers", 4))

    def to_spec(self):
        def norm(name):
            return NormSpec("rmsnorm", WIDTH, 1e-5, {"weight": name})

        def att(i, position, **kw):
            p = f"l{i}.att."
            names = {k: p + k for k in ("q.weight", "k.weight", "v.weight", "o.weight", "q.bias", "k.bias", "v.bias")}
            return AttentionSpec("attention", WIDTH, HEADS, KV, HD, position, tensors=names, **kw)

        def layer(i, mixer):
            ff = GatedMlpSpec("gated_mlp", WIDTH, INTER, "silu", {k: f"l{i}.ff.{k}" for k in ("gate.weight", "up.weight", "down.weight")})
            if i == 2:
                ff = RoutedSpec("toy_routed", WIDTH, EXPERTS, EXPERT_INTER, {k: f"l2.moe.{k}" for k in ("router", "w1", "w2")})
            return LayerSpec("prenorm", mixer, ff, norm(f"l{i}.n1"), norm(f"l{i}.n2"))

        layers = [
            layer(0, att(0, RotarySpec("rotary", HD, 1e4))),
            layer(1, RunningMeanSpec("toy_running_mean", WIDTH, {"w": "l1.mean.w"})),
            layer(2, att(2, RotarySpec("toy_position_scale", HD, 0.0), window=9)),
            layer(3, att(3, RotarySpec("rotary", HD, 1e4), kv_source=0)),
        ]
        return ModelSpec("ToyForCausalLM", EmbeddingSpec(VOCAB, WIDTH, {"weight": "emb"}), tuple(layers),
                         order=(0, 1, 2, 1, 3), final_norm=norm("nf"), head=HeadSpec(VOCAB, WIDTH, True), max_positions=512)


register_architecture("ToyForCausalLM", ToyConfig)


def toy_tensors(seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * 0.2
    t = {"emb": r(VOCAB, WIDTH), "nf": 1 + r(WIDTH) * 0.2, "l1.mean.w": r(WIDTH, WIDTH),
         "l2.moe.router": r(EXPERTS, WIDTH) * 5, "l2.moe.w1": r(EXPERTS, EXPERT_INTER, WIDTH), "l2.moe.w2": r(EXPERTS, WIDTH, EXPERT_INTER)}
    for i in range(4):
        t[f"l{i}.n1"], t[f"l{i}.n2"] = 1 + r(WIDTH) * 0.2, 1 + r(WIDTH) * 0.2
        if i != 2:  # layer 2 has the routed feed-forward
            t[f"l{i}.ff.gate.weight"], t[f"l{i}.ff.up.weight"], t[f"l{i}.ff.down.weight"] = r(INTER, WIDTH), r(INTER, WIDTH), r(WIDTH, INTER)
    for i in (0, 2, 3):
        t[f"l{i}.att.q.weight"], t[f"l{i}.att.o.weight"], t[f"l{i}.att.q.bias"] = r(HEADS * HD, WIDTH), r(WIDTH, HEADS * HD), r(HEADS * HD)
        if i != 3:
            t[f"l{i}.att.k.weight"], t[f"l{i}.att.v.weight"] = r(KV * HD, WIDTH), r(KV * HD, WIDTH)
            t[f"l{i}.att.k.bias"] = r(KV * HD)
    return t


def plain_toy(t, toks):
    """The toy model over a whole sequence with the plain parts."""
    T = len(toks)
    pos = torch.arange(T)
    x = t["emb"][torch.tensor(toks)]
    kv0 = {}

    def attention(i, xn, kind):
        q = P.linear(xn, t[f"l{i}.att.q.weight"], t[f"l{i}.att.q.bias"]).view(T, HEADS, HD)
        if i == 3:
            k, v = kv0["k"], kv0["v"]
        else:
            k = P.linear(xn, t[f"l{i}.att.k.weight"], t[f"l{i}.att.k.bias"]).view(T, KV, HD)
            v = P.linear(xn, t[f"l{i}.att.v.weight"]).view(T, KV, HD)
        if kind == "rotary":
            q = P.rope(q, pos, 1e4)
            k = P.rope(k, pos, 1e4) if i != 3 else k
        else:
            f = (1.0 + pos.float() / 64.0)[:, None, None]
            q, k = q * f, k * f
        if i == 0:
            kv0["k"], kv0["v"] = k, v
        o = P.attention(q, k, v, window=9 if i == 2 else None)
        return P.linear(o.reshape(T, -1), t[f"l{i}.att.o.weight"])

    for i in (0, 1, 2, 1, 3):
        xn = P.rms_norm(x, t[f"l{i}.n1"], 1e-5)
        if i == 1:
            # the layer runs twice with the same weights; each run has a state of its own
            mean = torch.cumsum(xn, 0) / torch.arange(1, T + 1, dtype=torch.float32)[:, None]
            x = x + mean @ t["l1.mean.w"].t()
        else:
            x = x + attention(i, xn, "rotary" if i != 2 else "scale")
        xn = P.rms_norm(x, t[f"l{i}.n2"], 1e-5)
        if i == 2:  # one expert a row
            choice = (xn @ t["l2.moe.router"].t()).argmax(-1)
            y = torch.stack([torch.relu(t["l2.moe.w1"][e] @ row) for row, e in zip(xn, choice)])
            x = x + torch.stack([t["l2.moe.w2"][e] @ row for row, e in zip(y, choice)])
            continue
        x = x + P.swiglu(xn, t[f"l{i}.ff.gate.weight"], t[f"l{i}.ff.up.weight"], t[f"l{i}.ff.down.weight"])
    return P.linear(P.rms_norm(x, t["nf"], 1e-5), t["emb"])


def _check(device, ops, dtype=torch.float32):
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import StepEntry, load_model
    t = toy_tensors()
    lm = load_model(config=config_from_dict({"architectures": ["ToyForCausalLM"]}), tensors=t, dtype=dtype,
                    device=device, page_size=16, num_pages=12, max_requests=3, ops=ops)
    assert sorted(lm.cache.groups) == ["full", "window9"] and lm.cache.state_requests.keys() == {1, 3}
    assert not lm.step.use_graphs, "a mixer that reads host lists must keep the step function out of graphs"
    gen = torch.Generator().manual_seed(1)
    seqs = [torch.randint(0, VOCAB, (n,), generator=gen).tolist() for n in (40, 23)]
    # two requests, cut differently and interleaved
    cuts = [[17, 1, 1, 12, 9], [5, 11, 1, 1, 5]]
    refs = [plain_toy(t, s) for s in seqs]
    slots = [lm.cache.admit() for _ in seqs]
    got = [[], []]
    fed = [0, 0]
    for step in range(5):
        entries = []
        for r in range(2):
            n = cuts[r][step]
            entries.append(StepEntry(slots[r], seqs[r][fed[r]:fed[r] + n], list(range(n))))
        logits = lm.step(entries)
        k = 0
        for r in range(2):
            n = cuts[r][step]
            got[r].append(logits[k:k + n].float().cpu())
            k += n
            fed[r] += n
    for r in range(2):
        out = torch.cat(got[r])
        assert (out - refs[r]).abs().max() <= 2e-4 * (1 + refs[r].abs().max()), f"request {r}"
    # a slot that is taken again starts from zero state
    lm.cache.release(slots[0])
    s = lm.cache.admit()
    assert s == slots[0] and all(lm.device_cache.states[p]["sum"][s].abs().max() == 0 for p in (1, 3))


def test_toy_model_on_the_cpu_stand_ins():
    _check("cpu", EmulatedOps())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32])
def test_toy_model_on_the_gpu(dtype):
    _check("cuda:0", None, dtype)
