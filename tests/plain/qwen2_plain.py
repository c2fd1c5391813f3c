"""Plain, slow Qwen2 decoder: whole sequences, no cache, one function per part.

Written from the formulas of gqf2008/machserve (paths below are relative to the
reference checkout).  It shares no code with the engine: it takes a dict of
tensors by checkpoint name and a dict of sizes, and computes everything with
ordinary torch ops on the CPU in the dtype of ``compute`` (float32 or float64).

Every function cites the reference lines it was written from.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """``y_i = x_i * (1 / sqrt(mean(x^2) + eps)) * w_i``: eps inside the root, added
    to the mean, weight multiplied last and not offset by one.

    crates/mach-model/src/ref_model.rs:1180-1188, crates/mach-model/src/kernels.rs:63-80.
    """
    ss = (x * x).sum(dim=-1, keepdim=True)
    inv = 1.0 / torch.sqrt(ss / x.shape[-1] + eps)
    return x * inv * w


def linear(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor | None = None) -> torch.Tensor:
    """``y[n] = sum_k W[n, k] x[k] (+ b[n])``; weight is row-major ``[out, in]`` and
    an absent bias tensor means no add.

    crates/mach-model/src/ref_model.rs:1167-1178 (matvec_t), tools/ref_llama.py:104-115 (bias).
    """
    y = x @ w.t()
    if b is not None:
        y = y + b
    return y


def yarn_of(rope_scaling):
    """``rope_scaling`` of config.json as the reference reads it: None unless its ``type`` is "yarn"; then
    ``(factor, original_max_position_embeddings, beta_fast = 32, beta_slow = 1, mscale = 1, mscale_all_dim = 0)``.
    crates/mach-server/src/startup.rs:172-199."""
    if not rope_scaling or rope_scaling.get("type", rope_scaling.get("rope_type")) != "yarn":
        return None
    return (float(rope_scaling.get("factor", 1.0)), int(rope_scaling.get("original_max_position_embeddings", 0)),
            float(rope_scaling.get("beta_fast", 32.0)), float(rope_scaling.get("beta_slow", 1.0)),
            float(rope_scaling.get("mscale", 1.0)), float(rope_scaling.get("mscale_all_dim", 0.0)))


def rope_freq(head_dim: int, theta: float, dtype=torch.float32, yarn=None) -> torch.Tensor:
    """Inverse frequency of every pair index ``j < head_dim/2``: ``theta^(-2j / head_dim)``; with YaRN
    ``freq_inter * ramp + freq_extra * (1 - ramp)``, ``freq_inter = freq_extra / factor``,
    ``ramp = clamp((j - low) / (high - low), 0, 1)``,
    ``low = floor(head_dim ln(orig / (beta_fast 2 pi)) / (2 ln theta))`` not below 0,
    ``high = ceil(the same with beta_slow)`` not above ``head_dim - 1`` (and 0.001 more if equal to ``low``).

    crates/mach-model/src/ref_model.rs:636-667 (rope_freq).
    """
    j = torch.arange(head_dim // 2, dtype=dtype)
    th = torch.tensor(float(theta), dtype=dtype)
    extra = 1.0 / torch.pow(th, 2.0 * j / head_dim)
    if yarn is None:
        return extra
    factor, orig, beta_fast, beta_slow = yarn[:4]
    inter = 1.0 / (factor * torch.pow(th, 2.0 * j / head_dim))

    def pair(rotations):
        return head_dim * math.log(orig / (rotations * 2.0 * math.pi)) / (2.0 * math.log(theta))
    low, high = max(math.floor(pair(beta_fast)), 0.0), min(math.ceil(pair(beta_slow)), head_dim - 1.0)
    if high == low:
        high += 0.001
    ramp = ((j - low) / (high - low)).clamp(0.0, 1.0)
    return inter * ramp + extra * (1.0 - ramp)


def yarn_attention_factor(yarn) -> float:
    """What YaRN multiplies every cosine and sine by: ``mscale(factor, mscale) / mscale(factor, mscale_all_dim)``
    with ``mscale(f, m) = 0.1 m ln f + 1``.  crates/mach-model/src/config.rs:242-253."""
    if yarn is None:
        return 1.0
    ln = math.log(yarn[0])
    return (0.1 * yarn[4] * ln + 1.0) / (0.1 * yarn[5] * ln + 1.0)


def attn_scale(head_dim: int, yarn=None) -> float:
    """``m^2 / sqrt(head_dim)`` with ``m = 0.1 mscale_all_dim ln(factor) + 1`` under YaRN with ``mscale_all_dim > 0``,
    else ``m = 1``.  crates/mach-model/src/config.rs:218-234."""
    m = 1.0
    if yarn is not None and yarn[5] > 0.0:
        m = 0.1 * yarn[5] * math.log(yarn[0]) + 1.0
    return m * m / math.sqrt(head_dim)


def rope_angles(positions: torch.Tensor, head_dim: int, theta: float, dtype=torch.float32, yarn=None) -> torch.Tensor:
    """``ang[p, j] = float(pos_p) * freq_j`` for ``j < head_dim/2``, every step in ``dtype`` as the
    reference does it in f32.

    crates/mach-model/src/ref_model.rs:636-643 (rope_freq) and 679-681.
    """
    return positions.to(dtype)[:, None] * rope_freq(head_dim, theta, dtype, yarn)[None, :]


def rope(x: torch.Tensor, positions: torch.Tensor, theta: float, yarn=None) -> torch.Tensor:
    """Rotate pairs ``(j, j + head_dim/2)`` (rotate_half pairing, whole head rotated):
    ``a' = a cos - b sin``, ``b' = a sin + b cos``, cosine and sine times YaRN's factor if there is one.
    ``x`` is ``[T, heads, head_dim]``.

    crates/mach-model/src/ref_model.rs:669-704 (apply_rope, interleave=false), tools/ref_llama.py:56-67.
    """
    hd = x.shape[-1]
    half = hd // 2
    ang = rope_angles(positions, hd, theta, x.dtype, yarn)
    f = yarn_attention_factor(yarn)
    c = torch.cos(ang)[:, None, :] * f
    s = torch.sin(ang)[:, None, :] * f
    a = x[..., :half]
    b = x[..., half:]
    return torch.cat([a * c - b * s, a * s + b * c], dim=-1)


def same(x: torch.Tensor) -> torch.Tensor:
    return x


def to_bf16_and_back(x: torch.Tensor) -> torch.Tensor:
    """What storing a value in bfloat16 does to it (round to nearest even, crates/mach-model/src/fp16.rs:84-94)."""
    return x.to(torch.bfloat16).to(x.dtype)


def to_f16_and_back(x: torch.Tensor) -> torch.Tensor:
    """What storing a value in half precision does to it (round to nearest even, crates/mach-model/src/fp16.rs:9-60)."""
    return x.to(torch.float16).to(x.dtype)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int | None = None, rounded=same,
              scale: float | None = None) -> torch.Tensor:
    """Causal grouped-query attention over a whole sequence.

    ``q`` is ``[T, H, hd]``, ``k``/``v`` are ``[T, KV, hd]``.  Query head ``h`` reads
    key/value head ``h // (H // KV)``; the row at position ``p`` sees keys ``0..=p``
    (with ``window``: only the last ``window`` of them, ``p - window < t <= p``);
    ``scale = head_dim^-0.5``; softmax with the maximum subtracted.

    crates/mach-model/src/ref_model.rs:1130-1165 (attention_decode),
    crates/mach-model/src/config.rs:231-234 (scale).  The window is not in the reference.
    """
    T, H, hd = q.shape
    KV = k.shape[1]
    g = H // KV
    scale = hd ** -0.5 if scale is None else scale
    out = torch.zeros_like(q)
    for h in range(H):
        kv = h // g
        for p in range(T):
            lo = 0 if window is None else max(0, p - window + 1)
            scores = (k[lo:p + 1, kv, :] @ q[p, h, :]) * scale
            e = torch.exp(scores - scores.max())
            # (a reduced-precision engine rounds the probabilities that multiply the values, not those it sums)
            out[p, h, :] = (rounded(e)[:, None] * v[lo:p + 1, kv, :]).sum(dim=0) / e.sum()
    return out


def silu(x: torch.Tensor) -> torch.Tensor:
    """``x / (1 + exp(-x))``.  crates/mach-model/src/ref_model.rs:1190-1192."""
    return x / (1.0 + torch.exp(-x))


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, rounded=same) -> torch.Tensor:
    """``down( silu(gate(x)) * up(x) )``: the activation is on the gate branch.

    crates/mach-model/src/ref_model.rs:299-309, crates/mach-model/src/kernels.rs:131-140,
    tools/ref_llama.py:120-123.
    """
    return linear(rounded(silu(linear(x, w_gate)) * linear(x, w_up)), w_down)


def attention_block(x, w, prefix, positions, sizes, window=None, rounded=same):
    """q/k/v projections with optional bias, rotation of q and k, attention, output
    projection without bias.  crates/mach-model/src/batched.rs:3566-3679, 4022-4031;
    tools/ref_llama.py:100-119.
    """
    H, KV, hd = sizes["heads"], sizes["kv_heads"], sizes["head_dim"]
    T = x.shape[0]
    q = linear(x, w[prefix + "q_proj.weight"], w.get(prefix + "q_proj.bias"))
    k = linear(x, w[prefix + "k_proj.weight"], w.get(prefix + "k_proj.bias"))
    v = linear(x, w[prefix + "v_proj.weight"], w.get(prefix + "v_proj.bias"))
    yarn = yarn_of(sizes.get("rope_scaling"))
    q = rounded(rope(q.view(T, H, hd), positions, sizes["theta"], yarn))
    k = rounded(rope(k.view(T, KV, hd), positions, sizes["theta"], yarn))
    o = rounded(attention(q, k, rounded(v.view(T, KV, hd)), window, rounded, attn_scale(hd, yarn)))
    return linear(o.reshape(T, H * hd), w[prefix + "o_proj.weight"])


def layer_windows(sizes) -> list:
    """Window of each layer: none unless ``use_sliding_window``; then layers with index
    ``>= max_window_layers`` attend to the last ``sliding_window`` keys.  (Keys the
    reference does not read; meaning taken from the keys' own names and documentation.)
    """
    L = sizes["layers"]
    if not sizes.get("use_sliding_window", False):
        return [None] * L
    return [sizes["sliding_window"] if i >= sizes["max_window_layers"] else None for i in range(L)]


def forward(weights: dict, sizes: dict, tokens, compute=torch.float32, start_pos: int = 0, rounded=same,
            streams: list = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` at every position of one whole sequence.  ``rounded`` is applied wherever a
    reduced-precision run of the same formulas stores a value in its element type: the inputs of every matrix
    product (the norms' outputs, the attention output, SiLU(gate) * up), q, and the keys and values of the
    cache, and the probabilities that multiply the values; the stream, the sums, the softmax and its
    statistics stay as computed.  The default rounds nothing.  A list given as ``streams`` receives the residual
    stream after the embedding and after every layer (crates/mach-model/src/batched.rs:3040-3088).

    Pre-norm blocks ``x += attn(norm(x)); x += mlp(norm(x))``, final norm, head =
    ``lm_head.weight`` when the tensor exists, else the embedding table.
    crates/mach-model/src/batched.rs:3150-3200, 4031-4050, 4424-4453, 4580-4626;
    crates/mach-model/src/loader.rs:1025-1033 (head rule); tools/ref_llama.py:89-125.
    """
    w = {n: t.to(compute) for n, t in weights.items()}
    toks = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(start_pos, start_pos + len(toks))
    x = w["model.embed_tokens.weight"][toks]
    keep = streams.append if streams is not None else (lambda t: None)
    keep(x)
    windows = layer_windows(sizes)
    for i in range(sizes["layers"]):
        p = f"model.layers.{i}."
        xn = rounded(rms_norm(x, w[p + "input_layernorm.weight"], sizes["eps"]))
        x = x + attention_block(xn, w, p + "self_attn.", positions, sizes, windows[i], rounded)
        xn = rounded(rms_norm(x, w[p + "post_attention_layernorm.weight"], sizes["eps"]))
        x = x + swiglu(xn, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"], rounded)
        keep(x)
    xf = rounded(rms_norm(x, w["model.norm.weight"], sizes["eps"]))
    head = w["lm_head.weight"] if "lm_head.weight" in w and not sizes.get("tied", False) else w["model.embed_tokens.weight"]
    return linear(xf, head)


def sizes_from_config(cfg: dict) -> dict:
    """Sizes the plain model needs, read from config.json's own keys.
    crates/mach-server/src/startup.rs:63-98."""
    heads = cfg["num_attention_heads"]
    return {
        "layers": cfg["num_hidden_layers"],
        "hidden": cfg["hidden_size"],
        "heads": heads,
        "kv_heads": cfg.get("num_key_value_heads", heads),
        "head_dim": cfg.get("head_dim", cfg["hidden_size"] // heads),
        "intermediate": cfg["intermediate_size"],
        "vocab": cfg["vocab_size"],
        "eps": cfg.get("rms_norm_eps", 1e-6),
        "theta": cfg.get("rope_theta", 10000.0),
        "rope_scaling": cfg.get("rope_scaling"),
        "tied": cfg.get("tie_word_embeddings", False),
        "use_sliding_window": cfg.get("use_sliding_window", False),
        "sliding_window": cfg.get("sliding_window"),
        "max_window_layers": cfg.get("max_window_layers", cfg["num_hidden_layers"]),
    }


def greedy_generate(weights, sizes, prompt, max_new, eos=None, compute=torch.float32):
    """Greedy continuation by recomputing the whole sequence for every new token."""
    seq = list(prompt)
    out = []
    for _ in range(max_new):
        logits = forward(weights, sizes, seq, compute)[-1]
        tok = argmax_first(logits)
        out.append(tok)
        seq.append(tok)
        if eos is not None and tok == eos:
            break
    return out


# ---------------------------------------------------------------- sampling

MASK64 = (1 << 64) - 1
RNG_GOLDEN = 0x9E3779B97F4A7C15


def mix64(z: int) -> int:
    """SplitMix64 finalizer.  crates/mach-model/src/sampling.rs:27-31."""
    z &= MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
    return z ^ (z >> 31)


def next_uniform(state: int):
    """One draw in [0, 1): finalizer of the state *before* the increment, top 24 bits.
    Returns ``(u, new_state)``.  crates/mach-model/src/sampling.rs:34-44."""
    z = mix64(state)
    return (z >> 40) / 16777216.0, (state + RNG_GOLDEN) & MASK64


def argmax_first(logits) -> int:
    """Smallest index among the maxima.  crates/mach-model/src/sampling.rs:1153-1161."""
    best = 0
    vals = logits.tolist()
    for i, v in enumerate(vals):
        if v > vals[best]:
            best = i
    return best


def sample(logits, temperature, top_k, top_p, state, presence=0.0, frequency=0.0, counts=(), bias=()):
    """CPU mirror of the sampler; returns ``(token, new_state)``.  One draw and one
    state advance per call, also when greedy.
    crates/mach-model/src/sampling.rs:1169-1274 (sample_cpu).
    """
    import numpy as np
    x = np.asarray(logits, dtype=np.float32).copy()
    u, state = next_uniform(state)
    for t, c in counts:
        if t < len(x) and c > 0:
            x[t] -= np.float32(presence + frequency * c)
    for t, b in bias:
        if t < len(x):
            x[t] += np.float32(b)
    if temperature <= 0.0:
        return argmax_first(torch.from_numpy(x)), state
    maxv, minv = x.max(), x.min()
    inv_t = np.float32(1.0 / temperature)
    prob = np.exp((x - maxv) * inv_t).astype(np.float32)
    k_eff = top_k if 0 < top_k < len(x) else 0
    thr = -np.inf
    if k_eff:
        lo, hi = np.float32(minv), np.float32(maxv)
        for _ in range(30):
            mid = np.float32((lo + hi) * np.float32(0.5))
            if int((x > mid).sum()) >= k_eff:
                lo = mid
            else:
                hi = mid
        thr = hi
    s_tot = np.float32(prob.sum(dtype=np.float32))
    cut = np.float32(0.0)
    use_topp = top_p < 1.0
    if use_topp:
        lo, hi = np.float32(0.0), np.float32(1.0)
        for _ in range(30):
            mid = np.float32((lo + hi) * np.float32(0.5))
            acc = prob[prob >= mid].sum(dtype=np.float32)
            if acc >= np.float32(top_p) * s_tot:
                lo = mid
            else:
                hi = mid
        cut = lo
    allowed = np.ones(len(x), dtype=bool)
    if k_eff:
        allowed &= x >= thr
    if use_topp:
        allowed &= prob >= cut
    target = np.float32(u) * prob[allowed].sum(dtype=np.float32)
    acc = np.float32(0.0)
    for i in range(len(x)):
        if allowed[i]:
            acc = np.float32(acc + prob[i])
            if acc > target:
                return i, state
    return argmax_first(torch.from_numpy(x)), state


def f32_to_bf16_bits(x: float) -> int:
    """Round-to-nearest-even on the high 16 bits.  crates/mach-model/src/fp16.rs:84-94."""
    import struct
    b = struct.unpack("<I", struct.pack("<f", x))[0]
    h = b >> 16
    rem = b & 0xFFFF
    if rem > 0x8000 or (rem == 0x8000 and (h & 1) == 1):
        h = (h + 1) & 0xFFFF
    return h
