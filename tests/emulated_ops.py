"""CPU stand-ins for the HIP entry points, with the same signatures and memory layouts.

Used only by tests: they let the host logic of the engine (step building, cache manager,
scheduler, replay) run where there is no GPU, and they are the per-kernel references of
the GPU tests.  Nothing in the package imports this file.
"""
from __future__ import annotations

import torch

MASK64 = (1 << 64) - 1


def _act(g, activation):
    """The activation on the gate branch of a gated product, in its textbook form."""
    if activation == "silu":
        return g / (1.0 + torch.exp(-g))
    if activation == "gelu_tanh":
        return 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * (g + 0.044715 * g * g * g)))
    raise ValueError(f"no activation {activation!r}")


class EmulatedOps:

    def __init__(self, dtype=torch.float32, device="cpu"):
        self.dtype = dtype
        self.device = torch.device(device)

    def _r(self, t):  # round to the element type, as a kernel's store does
        return t.to(self.dtype)

    def embed(self, tokens, table, scale=1.0):
        return table[tokens.long()].float() * scale

    SKINNY_ROWS = 64
    DECODE_MAX_GROUP = 16

    def rmsnorm(self, x, weight, eps, rows=None, out_f32=False, partials=None):
        full = x if partials is None else x + partials.sum(0)
        if partials is not None and rows is None:
            x.copy_(full)
        src = full if rows is None else full[rows.long()]
        y = src * (1.0 / torch.sqrt((src * src).sum(-1, keepdim=True) / src.shape[-1] + eps)) * weight
        return y if out_f32 else self._r(y)

    def linear(self, a, w, bias=None, out_f32=False):
        y = a.float() @ w.float().t()
        if bias is not None:
            y = y + bias
        return y if out_f32 else self._r(y)

    def add_partials(self, x, partials):
        x += partials.sum(0)

    def linear_split(self, a, w, allow_partials=True):
        y = a.float() @ w.float().t()
        if a.shape[0] <= self.SKINNY_ROWS and allow_partials:  # two parts, to exercise the consumers
            r = torch.randn(y.shape, generator=torch.Generator().manual_seed(0))
            return torch.stack([y - r, r])
        return y.unsqueeze(0)

    def norm_folds_into(self, M, N, K, n_partials):
        return M <= 16 and N >= 64

    def _normed(self, x, partials, norm_w, eps):
        full = x if partials is None else x + partials.sum(0)
        inv = 1.0 / torch.sqrt((full * full).sum(-1, keepdim=True) / full.shape[-1] + eps)
        return self._r(full * norm_w), inv, (full if partials is not None else None)

    def linear_split_normed(self, x, partials, norm_w, eps, w):
        a, inv, x_new = self._normed(x, partials, norm_w, eps)
        return ((a.float() @ w.float().t()) * inv).unsqueeze(0), x_new

    def linear_swiglu_normed(self, x, partials, norm_w, eps, w_gate_up, intermediate, activation="silu"):
        a, inv, x_new = self._normed(x, partials, norm_w, eps)
        Ip = w_gate_up.shape[0] // 2
        w = w_gate_up.float().view(Ip // 16, 2, 16, -1)
        gate = (a.float() @ w[:, 0].reshape(Ip, -1).t()) * inv
        up = (a.float() @ w[:, 1].reshape(Ip, -1).t()) * inv
        return self._r((_act(gate, activation) * up)[:, :intermediate]), x_new

    def linear_residual(self, a, w, x):
        if a.shape[0] <= self.SKINNY_ROWS:
            return self.linear_split(a, w)
        x += a.float() @ w.float().t()
        return None

    def linear_swiglu(self, a, w_gate_up, intermediate, activation="silu"):
        Ip = w_gate_up.shape[0] // 2
        w = w_gate_up.float().view(Ip // 16, 2, 16, -1)
        gate = a.float() @ w[:, 0].reshape(Ip, -1).t()
        up = a.float() @ w[:, 1].reshape(Ip, -1).t()
        return self._r((_act(gate, activation) * up)[:, :intermediate])

    def rope_kv_write(self, qkv, bias, positions, inv_freq, slot_map, kpool, vpool, H, KV, hd, page_size):
        qkv = qkv if qkv.dim() == 2 else qkv.sum(0)
        if bias is not None:
            qkv = qkv + bias
        T = qkv.shape[0]
        half = hd // 2
        if inv_freq is not None:
            ang = positions.float()[:, None] * inv_freq[None, :]
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        else:
            c = torch.ones(T, 1, half)
            s = torch.zeros(T, 1, half)

        def rot(x):
            a, b = x[..., :half], x[..., half:]
            return torch.cat([a * c - b * s, a * s + b * c], -1)

        q = self._r(rot(qkv[:, :H * hd].reshape(T, H, hd))).reshape(T, H * hd)
        if slot_map is not None:
            k = self._r(rot(qkv[:, H * hd:(H + KV) * hd].reshape(T, KV, hd)))
            v = self._r(qkv[:, (H + KV) * hd:(H + 2 * KV) * hd].reshape(T, KV, hd))
            page, off = (slot_map // page_size).long(), (slot_map % page_size).long()
            for t in range(T):
                kpool[page[t], :, off[t], :] = k[t]
                vpool[page[t], :, :, off[t]] = v[t]
        return q

    rows_per_block = 64  # flat rows of a work item; a test that hands over a GPU library's work list sets that library's

    def attention_rows_per_block(self, hd):
        return self.rows_per_block

    def paged_attention(self, q, kpool, vpool, block_table, seq_q_start, seq_q_len, seq_pos0, work, H, KV, hd,
                        page_size, window, scale):
        T = q.shape[0]
        g = H // KV
        out = torch.zeros(T, H * hd)
        done = set()
        for s, r0 in work.tolist():
            if s < 0:   # an item that only fills the list up
                continue
            qs, ql, p0 = int(seq_q_start[s]), int(seq_q_len[s]), int(seq_pos0[s])
            for r in range(r0, min(r0 + self.rows_per_block, ql * g)):
                tok, j = divmod(r, g)
                pos = p0 + tok
                lo = 0 if not window else max(0, pos - window + 1)
                keys = torch.arange(lo, pos + 1)
                pages = block_table[s].long()[keys // page_size]
                assert (pages >= 0).all(), "attention reads a page that was given back"
                offs = keys % page_size
                for kvh in range(KV):
                    h = kvh * g + j
                    kk = kpool[pages, kvh, offs, :].float()
                    vv = vpool[pages, kvh, :, offs].float()
                    sc = (kk @ q[qs + tok, h * hd:(h + 1) * hd].float()) * scale
                    p = torch.softmax(sc, 0)
                    out[qs + tok, h * hd:(h + 1) * hd] = p @ vv
                    done.add((qs + tok, h))
        assert len(done) == T * H, "the work list does not cover every row and head"
        return self._r(out)

    def decode_attention_fused(self, qkv, bias, inv_freq, slot_map, kpool, vpool, block_table, seq_pos0, H, KV, hd,
                               page_size, window, scale):
        q = self.rope_kv_write(qkv, bias, seq_pos0, inv_freq, slot_map, kpool, vpool, H, KV, hd, page_size)
        return self.decode_attention(q, kpool, vpool, block_table, seq_pos0, H, KV, hd, page_size, window, scale)

    def decode_attention(self, q, kpool, vpool, block_table, seq_pos0, H, KV, hd, page_size, window, scale):
        S = q.shape[0]
        ar = torch.arange(S, dtype=torch.int32)
        work = torch.stack([ar, torch.zeros_like(ar)], 1)
        return self.paged_attention(q, kpool, vpool, block_table, ar, torch.ones_like(ar), seq_pos0, work, H, KV, hd,
                                    page_size, window, scale)

    def sample(self, logits, temperature, top_k, top_p, state, any_greedy=True):
        from plain.qwen2_plain import sample as plain_sample
        toks, lps = [], []
        for r in range(logits.shape[0]):
            st = int(state[r].item()) & MASK64
            tok, st = plain_sample(logits[r].numpy(), float(temperature[r]), int(top_k[r]), float(top_p[r]), st)
            state[r] = st - (1 << 64) if st >= (1 << 63) else st
            toks.append(tok)
            lps.append(0.0)
        return torch.tensor(toks, dtype=torch.int32), torch.tensor(lps)

    def top_logprobs(self, logits, inv_t, k):
        lp = torch.log_softmax(logits.double() * inv_t.double()[:, None], -1)
        order = torch.argsort(-logits.double(), dim=-1, stable=True)[:, :k]
        return order.to(torch.int32), torch.gather(lp, 1, order).float()

    def logit_edit(self, logits, row_of, token, delta):
        for r, t, d in zip(row_of.tolist(), token.tolist(), delta.tolist()):
            logits[r, t] += d
