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
from machserve_amd.parts import (FEED_FORWARDS, MIXERS, NORMS, Block, FeedForward, Head, Mixer, PagedKVRequest, PositionEncoding,
                                 ResidualStream, StateRequest, TensorDecl, register_block, register_feed_forward, register_head,
                                 register_mixer, register_position_encoding)

WIDTH, HEADS, KV, HD, INTER, VOCAB = 48, 3, 1, 16, 80, 90
EXPERTS, EXPERT_INTER = 3, 24
VHD = 8                              # width of a value in the toy latent mixer; its keys are HD wide
EMB_SCALE, HEAD_SCALE = 1.5, 0.5


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
        f = (1.0 + ctx.position_axis(0).float() / 64.0)[:, None, None]
        q *= f
        if k is not None:
            k *= f


def two_axis_factor(positions, hd):
    """[T, 1, hd]: the first half of a head is scaled by 1 + p0 / 64, the second by 1 + p1 / 32."""
    p = positions.float()
    return torch.cat([(1.0 + p[:, 0:1] / 64.0).expand(-1, hd // 2), (1.0 + p[:, 1:2] / 32.0).expand(-1, hd - hd // 2)], 1)[:, None, :]


@register_position_encoding("toy_two_axes")
class TwoAxes(PositionEncoding):
    """A position is a pair of numbers; each scales one half of every head."""
    axes = 2

    def apply(self, q, k, ctx):
        f = two_axis_factor(ctx.positions, q.shape[-1])
        q *= f
        if k is not None:
            k *= f


@dataclass(frozen=True)
class LatentSpec:
    kind: str
    width: int
    heads: int
    key_dim: int
    value_dim: int
    position: object
    tensors: Mapping[str, str] = field(default_factory=dict)


@register_mixer("toy_latent")
class LatentAttention(Mixer):
    """One key/value head whose values are narrower than its keys, and beside the pages a state of fixed size
    (how many tokens the request has had), which damps the output: it asks the cache manager for both at
    once.  Its attention is written with ordinary tensor operations; it reads the step's host lists."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        from machserve_amd.parts import POSITION_ENCODINGS
        self.position = POSITION_ENCODINGS.build(spec.position, rt)

    def sub_parts(self):
        return [self.position]

    def tensor_decls(self):
        sp = self.spec
        return [TensorDecl("q", (sp.heads * sp.key_dim, sp.width)), TensorDecl("k", (sp.key_dim, sp.width)),
                TensorDecl("v", (sp.value_dim, sp.width)), TensorDecl("o", (sp.width, sp.heads * sp.value_dim))]

    def load(self, t):
        self.w = {k: v.float() for k, v in t.items()}

    def cache_request(self):
        return [PagedKVRequest(1, self.spec.key_dim, None, v_head_dim=self.spec.value_dim), StateRequest({"count": (1,)})]

    def bind_cache(self, bindings):
        kv, state = bindings
        self.group, self.kpool, self.vpool, self.count = kv.group, kv.kpool, kv.vpool, state.tensors["count"]

    def forward(self, h, stream, ctx):
        sp, x = self.spec, h.float()
        T = x.shape[0]
        q = (x @ self.w["q"].t()).view(T, sp.heads, sp.key_dim)
        k = (x @ self.w["k"].t()).view(T, 1, sp.key_dim)
        v = (x @ self.w["v"].t())
        self.position.apply(q, k, ctx)
        view = ctx.groups[self.group]
        ps = view.page_size
        where = view.slot_map.long()
        self.kpool[where // ps, 0, where % ps, :] = k[:, 0].to(self.kpool.dtype)
        self.vpool[where // ps, 0, :, where % ps] = v.to(self.vpool.dtype)
        out = torch.empty((T, sp.heads, sp.value_dim), dtype=torch.float32, device=x.device)
        for s, (slot, q0, n, p0) in enumerate(zip(ctx.host["seq_slot"], ctx.host["seq_q_start"], ctx.host["seq_q_len"], ctx.host["seq_pos0"])):
            pages = view.block_table[s, :-(-(p0 + n) // ps)].long()
            keys = self.kpool[pages, 0].reshape(-1, sp.key_dim).float()[:p0 + n]
            vals = self.vpool[pages, 0].transpose(1, 2).reshape(-1, sp.value_dim).float()[:p0 + n]
            scores = torch.einsum("thd,sd->ths", q[q0:q0 + n], keys) * sp.key_dim ** -0.5
            seen = torch.arange(p0 + n, device=x.device)[None, :] <= (p0 + torch.arange(n, device=x.device))[:, None]
            scores = scores.masked_fill(~seen[:, None, :], float("-inf"))
            count = self.count[slot] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
            out[q0:q0 + n] = torch.softmax(scores, -1) @ vals / (1.0 + 0.01 * count)[:, None, None]
            self.count[slot] = count[-1]
        stream.add(out.reshape(T, -1) @ self.w["o"].t())


@dataclass(frozen=True)
class BiasedHeadSpec:
    kind: str
    vocab: int
    width: int
    tied: bool
    scale: float
    tensors: Mapping[str, str] = field(default_factory=dict)


@register_head("toy_biased")
class BiasedHead(Head):
    """The framework's head, and a bias on every logit: another head is a registered class and a spec."""

    def tensor_decls(self):
        return super().tensor_decls() + [TensorDecl("bias", (self.spec.vocab,), "vector")]

    def load(self, t):
        super().load(t)
        self.bias = t["bias"]

    def forward(self, h):
        return super().forward(h) + self.bias


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
            layer(4, LatentSpec("toy_latent", WIDTH, HEADS, HD, VHD, RotarySpec("toy_two_axes", HD, 0.0),
                                {k: f"l4.lat.{k}" for k in ("q", "k", "v", "o")})),
        ]
        return ModelSpec("ToyForCausalLM", EmbeddingSpec(VOCAB, WIDTH, {"weight": "emb"}, scale=EMB_SCALE), tuple(layers),
                         order=(0, 1, 2, 1, 3, 4), final_norm=norm("nf"),
                         head=BiasedHeadSpec("toy_biased", VOCAB, WIDTH, True, HEAD_SCALE, {"bias": "head.bias"}),
                         max_positions=512)


register_architecture("ToyForCausalLM", ToyConfig)


def toy_tensors(seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * 0.2
    t = {"emb": r(VOCAB, WIDTH), "nf": 1 + r(WIDTH) * 0.2, "l1.mean.w": r(WIDTH, WIDTH),
         "l2.moe.router": r(EXPERTS, WIDTH) * 5, "l2.moe.w1": r(EXPERTS, EXPERT_INTER, WIDTH), "l2.moe.w2": r(EXPERTS, WIDTH, EXPERT_INTER)}
    t["head.bias"] = r(VOCAB)
    t["l4.lat.q"], t["l4.lat.k"], t["l4.lat.v"], t["l4.lat.o"] = r(HEADS * HD, WIDTH), r(HD, WIDTH), r(VHD, WIDTH), r(WIDTH, HEADS * VHD)
    for i in range(5):
        t[f"l{i}.n1"], t[f"l{i}.n2"] = 1 + r(WIDTH) * 0.2, 1 + r(WIDTH) * 0.2
        if i != 2:  # layer 2 has the routed feed-forward
            t[f"l{i}.ff.gate.weight"], t[f"l{i}.ff.up.weight"], t[f"l{i}.ff.down.weight"] = r(INTER, WIDTH), r(INTER, WIDTH), r(WIDTH, INTER)
    for i in (0, 2, 3):
        t[f"l{i}.att.q.weight"], t[f"l{i}.att.o.weight"], t[f"l{i}.att.q.bias"] = r(HEADS * HD, WIDTH), r(WIDTH, HEADS * HD), r(HEADS * HD)
        if i != 3:
            t[f"l{i}.att.k.weight"], t[f"l{i}.att.v.weight"] = r(KV * HD, WIDTH), r(KV * HD, WIDTH)
            t[f"l{i}.att.k.bias"] = r(KV * HD)
    return t


def second_axis(n0, n1):
    """The second number of the positions n0 .. n1 - 1 that the tests give the toy model: a row of a picture
    three tokens wide, say."""
    return [j // 3 for j in range(n0, n1)]


def plain_toy(t, toks):
    """The toy model over a whole sequence with the plain parts."""
    T = len(toks)
    pos = torch.arange(T)
    pos2 = torch.stack([pos, torch.tensor(second_axis(0, T))], 1)
    x = t["emb"][torch.tensor(toks)] * EMB_SCALE
    kv0 = {}

    def latent(xn):
        q = (xn @ t["l4.lat.q"].t()).view(T, HEADS, HD) * two_axis_factor(pos2, HD)
        k = (xn @ t["l4.lat.k"].t()).view(T, 1, HD) * two_axis_factor(pos2, HD)
        v = (xn @ t["l4.lat.v"].t()).view(T, 1, VHD)
        scores = torch.einsum("thd,sd->ths", q, k[:, 0]) * HD ** -0.5
        scores = scores.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool))[:, None, :], float("-inf"))
        o = torch.softmax(scores, -1) @ v[:, 0] / (1.0 + 0.01 * torch.arange(1, T + 1, dtype=torch.float32))[:, None, None]
        return o.reshape(T, -1) @ t["l4.lat.o"].t()

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

    for i in (0, 1, 2, 1, 3, 4):
        xn = P.rms_norm(x, t[f"l{i}.n1"], 1e-5)
        if i == 4:
            x = x + latent(xn)
        elif i == 1:
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
    return P.linear(P.rms_norm(x, t["nf"], 1e-5), t["emb"]) * HEAD_SCALE + t["head.bias"]


def _check(device, ops, dtype=torch.float32):
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import StepEntry, load_model
    t = toy_tensors()
    lm = load_model(config=config_from_dict({"architectures": ["ToyForCausalLM"]}), tensors=t, dtype=dtype,
                    device=device, page_size=16, num_pages=12, max_requests=3, ops=ops)
    assert sorted(lm.cache.groups) == ["full", f"full/kv1x{HD}v{VHD}", "window9"] and lm.cache.state_requests.keys() == {1, 3}
    assert lm.step.position_axes == 2
    kv, st = lm.device_cache.binding(5)      # the latent layer asked for pages and a state at once
    assert kv.kpool.shape[-1] == HD and kv.vpool.shape[-2] == VHD and st.tensors["count"].shape == (3 + 1, 1)
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
            positions = [[a, b] for a, b in zip(range(fed[r], fed[r] + n), second_axis(fed[r], fed[r] + n))]
            entries.append(StepEntry(slots[r], seqs[r][fed[r]:fed[r] + n], list(range(n)), positions))
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


# ---------------------------------------------------------------------------- a toy model that may be captured

@register_mixer("toy_running_mean_on_device")
class DeviceRunningMean(RunningMean):
    """The same running mean, reading nothing but device memory from the step: such a mixer may say
    ``graph_safe`` and is then captured into graphs, filled up with rows that belong to no request (they
    update the scratch slot's state, nobody's), and launched a step ahead like the framework's own attention."""
    graph_safe = True

    def forward(self, h, stream, ctx):
        x = h.float()
        T, dev = x.shape[0], x.device
        rows = torch.arange(T, device=dev)
        seq = torch.searchsorted(ctx.seq_q_start.long(), rows, right=True) - 1      # the request of every row
        slot, q0 = ctx.seq_slot.long()[seq], ctx.seq_q_start.long()[seq]
        earlier = ((seq[:, None] == seq[None, :]) & (rows[None, :] <= rows[:, None])).float()
        run = earlier @ x + self.state["sum"][slot]
        cnt = self.state["count"][slot] + (rows - q0 + 1).float()[:, None]
        last = (ctx.seq_q_start + ctx.seq_q_len - 1).long()
        self.state["sum"].index_copy_(0, ctx.seq_slot.long(), run[last])
        self.state["count"].index_copy_(0, ctx.seq_slot.long(), cnt[last])
        stream.add((run / cnt) @ self.w.float().t())


@dataclass
class GraphToyConfig:
    @classmethod
    def from_dict(cls, raw):
        return cls()

    def to_spec(self):
        base = ToyConfig().to_spec()
        mean = LayerSpec("prenorm", RunningMeanSpec("toy_running_mean_on_device", WIDTH, {"w": "l1.mean.w"}), base.layers[1].feed_forward,
                         base.layers[1].mixer_norm, base.layers[1].feed_forward_norm)
        return ModelSpec("GraphToyForCausalLM", EmbeddingSpec(VOCAB, WIDTH, {"weight": "emb"}), (base.layers[0], mean),
                         order=(0, 1, 0), final_norm=base.final_norm, head=HeadSpec(VOCAB, WIDTH, True), max_positions=512)


register_architecture("GraphToyForCausalLM", GraphToyConfig)


def plain_graph_toy(t, toks):
    T = len(toks)
    pos = torch.arange(T)
    x = t["emb"][torch.tensor(toks)]
    for i in (0, 1, 0):
        xn = P.rms_norm(x, t[f"l{i}.n1"], 1e-5)
        if i == 1:
            x = x + (torch.cumsum(xn, 0) / torch.arange(1, T + 1, dtype=torch.float32)[:, None]) @ t["l1.mean.w"].t()
        else:
            q = P.rope(P.linear(xn, t["l0.att.q.weight"], t["l0.att.q.bias"]).view(T, HEADS, HD), pos, 1e4)
            k = P.rope(P.linear(xn, t["l0.att.k.weight"], t["l0.att.k.bias"]).view(T, KV, HD), pos, 1e4)
            v = P.linear(xn, t["l0.att.v.weight"]).view(T, KV, HD)
            x = x + P.linear(P.attention(q, k, v).reshape(T, -1), t["l0.att.o.weight"])
        xn = P.rms_norm(x, t[f"l{i}.n2"], 1e-5)
        x = x + P.swiglu(xn, t[f"l{i}.ff.gate.weight"], t[f"l{i}.ff.up.weight"], t[f"l{i}.ff.down.weight"])
    return P.linear(P.rms_norm(x, t["nf"], 1e-5), t["emb"])


def graph_toy_tensors():
    t = toy_tensors()
    keep = ("emb", "nf", "l0.", "l1.")
    return {k: v for k, v in t.items() if k.startswith(keep)}


def _generate_graph_toy(device, ops, n_new):
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import Engine, load_model
    t = graph_toy_tensors()
    lm = load_model(config=config_from_dict({"architectures": ["GraphToyForCausalLM"]}), tensors=t, dtype=torch.float32,
                    device=device, page_size=16, num_pages=24, max_requests=4, ops=ops)
    gen = torch.Generator().manual_seed(3)
    prompts = [torch.randint(0, VOCAB, (n,), generator=gen).tolist() for n in (7, 19, 12)]
    eng = Engine(lm, max_batch_tokens=64)
    got = eng.generate(prompts, max_new=n_new)
    for p, g in zip(prompts, got):
        seq = list(p)
        for tok in g:   # greedy: every generated token is the plain model's most likely one, by a clear margin or a tie's lowest index
            logits = plain_graph_toy(t, seq)[-1]
            assert tok == P.argmax_first(logits) or logits[tok] >= logits.max() - 2e-4 * (1 + logits.abs().max()), len(seq)
            seq.append(tok)
    return lm


def test_toy_model_with_state_on_the_device_on_the_cpu_stand_ins():
    _generate_graph_toy("cpu", EmulatedOps(), 12)


@pytest.mark.gpu
def test_a_mixer_with_state_is_captured_filled_up_and_launched_ahead():
    """Three requests decode in captured steps of four rows (one belongs to nobody) that are launched a step
    ahead: the state of the requests is what the plain model's is, token for token, for 60 tokens."""
    lm = _generate_graph_toy("cuda:0", None, 60)
    assert lm.step.use_graphs and len(lm.step._graphs) >= 1
    assert any(k[0] == (1, 1, 1, 1) for k in lm.step._graphs), "a step of three requests is captured as one of four rows"


# ---------------------------------------------------------------------------- toy arrangements of a block

@dataclass(frozen=True)
class SandwichSpec:
    """A layer whose two branches are normalised before *and after*: four norms, and a softmax scale of its own."""
    block: str
    mixer: object
    feed_forward: object
    norms: tuple   # before the mixer, after it, before the feed-forward, after it


@register_block("toy_sandwich")
class Sandwich(Block):
    """x += norm(mixer(norm(x))); x += norm(feed_forward(norm(x))): the arrangement builds its four norms and its two
    branches from the fields of its own spec; each branch adds into a stream of its own that starts at zero."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer = MIXERS.build(spec.mixer, rt)
        self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, rt)
        self.norms = [NORMS.build(n, rt) for n in spec.norms]

    def parts(self):
        return self.norms + [self.mixer, self.feed_forward]

    def forward(self, stream, ctx):
        for before, branch_part, after in ((self.norms[0], self.mixer, self.norms[1]),
                                           (self.norms[2], self.feed_forward, self.norms[3])):
            branch = ResidualStream(torch.zeros_like(stream.value()), stream.ops)
            branch_part.forward(before.forward(stream), branch, ctx)
            stream.add(after.forward(branch).float())


@dataclass(frozen=True)
class MixerOnlySpec:
    block: str
    mixer: object
    norm: object


@register_block("toy_mixer_only")
class MixerOnly(Block):
    """x += mixer(norm(x)) and nothing else: a layer without a feed-forward."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer, self.norm = MIXERS.build(spec.mixer, rt), NORMS.build(spec.norm, rt)

    def parts(self):
        return [self.norm, self.mixer]

    def forward(self, stream, ctx):
        self.mixer.forward(self.norm.forward(stream), stream, ctx)


SANDWICH_SCALE = 0.11   # not HD ** -0.5 = 0.25


@dataclass
class SandwichToyConfig:
    @classmethod
    def from_dict(cls, raw):
        return cls()

    def to_spec(self):
        norm = lambda name: NormSpec("rmsnorm", WIDTH, 1e-5, {"weight": name})
        names = lambda i: {k: f"l{i}.att.{k}" for k in ("q.weight", "k.weight", "v.weight", "o.weight", "q.bias", "k.bias", "v.bias")}
        att0 = AttentionSpec("attention", WIDTH, HEADS, KV, HD, RotarySpec("rotary", HD, 1e4), tensors=names(0), scale=SANDWICH_SCALE)
        ff0 = GatedMlpSpec("gated_mlp", WIDTH, INTER, "gelu_tanh", {k: f"l0.ff.{k}" for k in ("gate.weight", "up.weight", "down.weight")})
        layers = (SandwichSpec("toy_sandwich", att0, ff0, (norm("l0.n1"), norm("l0.n2"), norm("l1.n1"), norm("l1.n2"))),
                  MixerOnlySpec("toy_mixer_only", AttentionSpec("attention", WIDTH, HEADS, KV, HD, RotarySpec("rotary", HD, 1e4),
                                                                tensors=names(2)), norm("l2.n1")))
        return ModelSpec("SandwichToyForCausalLM", EmbeddingSpec(VOCAB, WIDTH, {"weight": "emb"}), layers, order=(0, 1, 0),
                         final_norm=norm("nf"), head=HeadSpec(VOCAB, WIDTH, True), max_positions=512)


register_architecture("SandwichToyForCausalLM", SandwichToyConfig)


def plain_sandwich_toy(t, toks, scale0=SANDWICH_SCALE, act=lambda g: torch.nn.functional.gelu(g, approximate="tanh")):
    T = len(toks)
    pos = torch.arange(T)
    x = t["emb"][torch.tensor(toks)]

    def att(i, xn, scale):
        q = P.rope(P.linear(xn, t[f"l{i}.att.q.weight"], t[f"l{i}.att.q.bias"]).view(T, HEADS, HD), pos, 1e4)
        k = P.rope(P.linear(xn, t[f"l{i}.att.k.weight"], t[f"l{i}.att.k.bias"]).view(T, KV, HD), pos, 1e4)
        v = P.linear(xn, t[f"l{i}.att.v.weight"]).view(T, KV, HD)
        # the plain attention scales by HD ** -0.5: another scale is a factor on the queries
        o = P.attention(q * (scale / HD ** -0.5), k, v)
        return P.linear(o.reshape(T, -1), t[f"l{i}.att.o.weight"])

    for i in (0, 1, 0):
        if i == 0:
            x = x + P.rms_norm(att(0, P.rms_norm(x, t["l0.n1"], 1e-5), scale0), t["l0.n2"], 1e-5)
            xn = P.rms_norm(x, t["l1.n1"], 1e-5)
            y = P.linear(act(P.linear(xn, t["l0.ff.gate.weight"])) * P.linear(xn, t["l0.ff.up.weight"]), t["l0.ff.down.weight"])
            x = x + P.rms_norm(y, t["l1.n2"], 1e-5)
        else:
            x = x + att(2, P.rms_norm(x, t["l2.n1"], 1e-5), HD ** -0.5)
    return P.linear(P.rms_norm(x, t["nf"], 1e-5), t["emb"])


def _check_sandwich(device, ops):
    """Blocks that build parts of their own (four norms; no feed-forward), an attention whose scale the spec gives and a
    gated feed-forward whose activation it gives (the tanh form of GELU, the library's own as the plain one): a request
    in portions beside one token by token, against the plain parts."""
    from machserve_amd.config import config_from_dict
    from machserve_amd.engine import StepEntry, load_model
    t = {k: v for k, v in toy_tensors().items() if k.startswith(("emb", "nf", "l0.", "l1.n", "l2.n1", "l2.att"))}
    lm = load_model(config=config_from_dict({"architectures": ["SandwichToyForCausalLM"]}), tensors=t, dtype=torch.float32,
                    device=device, page_size=16, num_pages=12, max_requests=2, ops=ops)
    assert [type(b).__name__ for b in lm.model.blocks] == ["Sandwich", "MixerOnly"]
    assert len(lm.model.blocks[0].parts()) == 6 and lm.model.blocks[0].mixer.scale == SANDWICH_SCALE
    gen = torch.Generator().manual_seed(5)
    seqs = [torch.randint(0, VOCAB, (n,), generator=gen).tolist() for n in (37, 9)]
    refs = [plain_sandwich_toy(t, s) for s in seqs]
    slots = [lm.cache.admit() for _ in seqs]
    cuts = [[20, 2, 6, 9], [1, 1, 1, 6]]
    got, fed = [[], []], [0, 0]
    for step in range(4):
        entries = [StepEntry(slots[r], seqs[r][fed[r]:fed[r] + cuts[r][step]], list(range(cuts[r][step]))) for r in range(2)]
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
    # the test can tell the scale: with the usual one the plain model is far from this
    usual = plain_sandwich_toy(t, seqs[0], HD ** -0.5)
    assert (usual - refs[0]).abs().max() > 50 * 2e-4 * (1 + refs[0].abs().max())
    # ... and the activation
    usual = plain_sandwich_toy(t, seqs[0], act=P.silu)
    assert (usual - refs[0]).abs().max() > 50 * 2e-4 * (1 + refs[0].abs().max())


def test_blocks_that_build_their_own_parts_on_the_cpu_stand_ins():
    _check_sandwich("cpu", EmulatedOps())


@pytest.mark.gpu
def test_blocks_that_build_their_own_parts_on_the_gpu():
    _check_sandwich("cuda:0", None)


def test_toy_model_on_the_cpu_stand_ins():
    _check("cpu", EmulatedOps())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32])
def test_toy_model_on_the_gpu(dtype):
    _check("cuda:0", None, dtype)
