"""The one boundary between Python and the HIP libraries (role of ``mach-kernel-sys`` in the
reference, ``crates/mach-kernel-sys/src/hip.rs``): torch tensors own the memory, every
operand is checked on the host against what the kernel and its grid assume, and the raw
pointers go to the ``extern "C"`` entry points on torch's current stream.

There is no fallback: without a GPU or without the libraries, construction raises.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build

_c_float, _c_void = ctypes.c_float, ctypes.c_void_p


def _c_int(v) -> int:
    """An argument of C type int: ctypes passes a Python int as one by itself (and refuses one that does not
    fit), which spares an object per argument; pointers and floats need their wrappers."""
    return int(v)



class KernelError(RuntimeError):
    pass


def _ptr(t: Optional[torch.Tensor]):
    return _c_void(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """torch's current stream on the current device as a raw handle.  The private accessor costs a
    fraction of a microsecond; ``torch.cuda.current_stream()`` builds an object (several microseconds,
    and a step issues some two hundred launches)."""
    if _raw_stream is not None:
        return _c_void(_raw_stream(torch.cuda.current_device()))
    return _c_void(torch.cuda.current_stream().cuda_stream)


class HipOps:
    """Kernels of one element type: ``torch.bfloat16`` or ``torch.float16`` (serving; the same kernels with the
    other two-byte type, the reference's own fast precision, ``crates/mach-model/src/config.rs:3-11``) or
    ``torch.float32`` (true 32-bit)."""
    ELEMS = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}

    def __init__(self, dtype: torch.dtype, device: str = "cuda:0"):
        if dtype not in self.ELEMS:
            raise KernelError(f"no kernels for element type {dtype}; bfloat16, float16 and float32 are built")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the HIP kernels have no CPU fallback")
        self.dtype = dtype
        self.device = torch.device(device)
        self._index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self.elem = self.ELEMS[dtype]
        self._libs: list = []
        self._core = self._load(build.ensure_library("core", self.elem))
        self._attn = {}
        self._cus = torch.cuda.get_device_properties(self._index).multi_processor_count
        # what the library plans for a product depends on its sizes alone: asked once per size
        self._plans: dict = {}

    def _load(self, path: str):
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load {path}: {e}") from None
        lib.ms_last_error.restype = ctypes.c_char_p
        lib.ms_launch_count.restype = ctypes.c_long
        self._libs.append(lib)
        return lib

    def launch_count(self) -> int:
        """Kernels launched so far by the libraries this object has loaded."""
        return sum(int(lib.ms_launch_count()) for lib in self._libs)

    def _stream(self):
        """torch's current stream on this object's device as a raw handle."""
        if _raw_stream is not None:
            return _c_void(_raw_stream(self._index))
        return _c_void(torch.cuda.current_stream(self.device).cuda_stream)

    def _check(self, lib, rc: int):
        if rc != 0:
            raise KernelError(lib.ms_last_error().decode())

    def _want(self, t: torch.Tensor, dtype, name: str, *shape):
        """The operand is what the kernel assumes: on the GPU, of this type, contiguous, of this shape if one
        is given.  Runs for every operand of every launch, so the good case is a few attribute reads."""
        if not t.is_cuda or t.dtype is not dtype or not t.is_contiguous():
            raise KernelError(f"{name}: expected a contiguous {dtype} GPU tensor, got {t.dtype} on {t.device}"
                              f"{'' if t.is_contiguous() else ' (not contiguous)'}")
        if shape and t.shape != shape:
            raise KernelError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")

    def require_sizes(self, what: str, reductions=(), head_dim: Optional[int] = None, norm_width: Optional[int] = None,
                      rotated_row: Optional[int] = None) -> None:
        """Refuses, when a model is put together, sizes that the kernels do not take: a product sums over a
        multiple of 8 elements, a head has a multiple of 16 up to the largest attention tile, a normalised row
        and a row of q, k and v that is rotated and written to the cache fit a block's row buffer."""
        for name, k in reductions:
            if k <= 0 or k % 8:
                raise KernelError(f"{what}: {name} = {k} must be a positive multiple of 8 (the products sum over it in 16-byte chunks)")
        if norm_width is not None and not 0 < norm_width <= self._core.ms_max_norm_width():
            raise KernelError(f"{what}: width {norm_width} is outside what the norm kernel takes (1 to {self._core.ms_max_norm_width()})")
        if rotated_row is not None and not 0 < rotated_row <= self._core.ms_max_rope_row():
            raise KernelError(f"{what}: (heads + 2 x key/value heads) x head size = {rotated_row} is outside what the rotation "
                              f"kernel takes (1 to {self._core.ms_max_rope_row()})")
        if head_dim is not None:
            try:
                build.attention_tile_for(head_dim)
            except build.BuildError as e:
                raise KernelError(f"{what}: {e}") from None

    # ------------------------------------------------------------------ elementwise
    def embed(self, tokens: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        T, (V, d) = tokens.numel(), table.shape
        self._want(tokens, torch.int32, "embed tokens", T)
        self._want(table, self.dtype, "embed table")
        x = torch.empty((T, d), dtype=torch.float32, device=table.device)
        self._check(self._core, self._core.ms_embed(_ptr(tokens), _ptr(table), _ptr(x), _c_int(T), _c_int(d), _c_float(scale),
                                                    self._stream()))
        return x

    def feed_tokens(self, tokens: torch.Tensor, sampled: torch.Tensor, rows: torch.Tensor, src: torch.Tensor) -> None:
        """``tokens[rows[i]] = sampled[src[i]]`` where ``rows[i]`` is no negative number: the rows of a step whose
        input the step before it sampled take it on the device."""
        n = rows.numel()
        self._want(tokens, torch.int32, "feed_tokens tokens")
        self._want(sampled, torch.int32, "feed_tokens sampled")
        self._want(rows, torch.int32, "feed_tokens rows", n)
        self._want(src, torch.int32, "feed_tokens src", n)
        self._check(self._core, self._core.ms_feed_tokens(_ptr(tokens), _ptr(sampled), _ptr(rows), _ptr(src), _c_int(n),
                                                          _c_int(tokens.numel()), _c_int(sampled.numel()), self._stream()))

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, rows: Optional[torch.Tensor] = None,
                out_f32: bool = False, partials: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Norm of ``x + sum(partials)`` (of its ``rows`` if given).  With ``partials [P, T, d]`` and
        no ``rows`` the sum is also written back into ``x``."""
        T, d = x.shape
        self._want(x, torch.float32, "rmsnorm input")
        self._want(weight, torch.float32, "rmsnorm weight", d)
        n, P = T, 0
        if rows is not None:
            self._want(rows, torch.int32, "rmsnorm rows")
            n = rows.numel()
        if partials is not None:
            P = partials.shape[0]
            self._want(partials, torch.float32, "rmsnorm partial sums", P, T, d)
        out = torch.empty((n, d), dtype=torch.float32 if out_f32 else self.dtype, device=x.device)
        self._check(self._core, self._core.ms_rmsnorm(_ptr(x), _ptr(partials), _c_int(P), _c_int(T), _ptr(rows),
                                                      _ptr(weight), _ptr(out), _c_int(int(out_f32)), _c_int(n), _c_int(d),
                                                      _c_float(eps), self._stream()))
        return out

    def add_partials(self, x: torch.Tensor, partials: torch.Tensor) -> None:
        """``x += sum(partials)`` in order."""
        T, d = x.shape
        self._want(x, torch.float32, "stream")
        self._want(partials, torch.float32, "partial sums", partials.shape[0], T, d)
        self._check(self._core, self._core.ms_add_partials(_ptr(x), _ptr(partials), _c_int(partials.shape[0]), _c_int(T),
                                                           _c_int(d), self._stream()))

    def rope_kv_write(self, qkv: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor,
                      inv_freq: Optional[torch.Tensor], slot_map: Optional[torch.Tensor], kpool: Optional[torch.Tensor],
                      vpool: Optional[torch.Tensor], H: int, KV: int, hd: int, page_size: int) -> torch.Tensor:
        """``qkv [P, T, stride]`` are partial sums of the q/k/v projection (see :meth:`linear_split`);
        their sum plus ``bias`` is rotated (q and k) and written (k and v) into the pages.  Returns
        q ``[T, H * hd]`` in the element type."""
        if qkv.dim() == 2:
            qkv = qkv.unsqueeze(0)
        P, T, stride = qkv.shape
        self._want(qkv, torch.float32, "rope qkv")
        self._want(positions, torch.int32, "rope positions", T)
        if bias is not None:
            self._want(bias, torch.float32, "rope bias", stride)
        if inv_freq is not None:
            self._want(inv_freq, torch.float32, "rope inv_freq", hd // 2)
        if slot_map is not None:
            self._want(slot_map, torch.int32, "rope slot_map", T)
            pages = kpool.shape[0]
            self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
            self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        q = torch.empty((T, H * hd), dtype=self.dtype, device=qkv.device)
        self._check(self._core, self._core.ms_rope_kv_write(
            _ptr(qkv), _c_int(P), _ptr(bias), _c_int(stride), _ptr(positions), _ptr(inv_freq), _ptr(slot_map), _ptr(q),
            _ptr(kpool), _ptr(vpool), _c_int(T), _c_int(H), _c_int(KV), _c_int(hd), _c_int(page_size), self._stream()))
        return q

    def rope_table(self, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
        """Float32 ``[T, hd / 2, 2]``: cosine and sine of ``positions[t] * inv_freq[j]``, as the rotation kernels
        compute them; for :meth:`linear_qkv_rope`."""
        T, half = positions.numel(), inv_freq.numel()
        self._want(positions, torch.int32, "rope table positions", T)
        self._want(inv_freq, torch.float32, "rope table inv_freq", half)
        cs = torch.empty((T, half, 2), dtype=torch.float32, device=inv_freq.device)
        self._check(self._core, self._core.ms_rope_table(_ptr(positions), _ptr(inv_freq), _ptr(cs), _c_int(T), _c_int(half), self._stream()))
        return cs

    def qkv_rope_takes(self, M: int, H: int, KV: int, hd: int, K: int) -> bool:
        """Whether :meth:`linear_qkv_rope` takes this shape (else: :meth:`linear_split` and :meth:`rope_kv_write`)."""
        return bool(self._plan("ms_qkv_rope_takes", M, H, KV, hd, K))

    def linear_qkv_rope(self, a: torch.Tensor, w_qkv: torch.Tensor, bias: Optional[torch.Tensor], rope_cs: torch.Tensor,
                        slot_map: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, H: int, KV: int, hd: int,
                        page_size: int) -> torch.Tensor:
        """The q/k/v projection ``a @ w_qkv.T + bias`` of a step of many rows with the rotation of queries and keys
        (by ``rope_cs`` of :meth:`rope_table`) and the write of keys and values into their pages in the product's own
        epilogue.  Returns q ``[T, H * hd]`` in the element type."""
        M, N, K = self._mm_operands(a, w_qkv, "linear_qkv_rope")
        if N != (H + 2 * KV) * hd:
            raise KernelError(f"linear_qkv_rope: weight of {N} rows for {H} + 2 x {KV} heads of {hd}")
        if bias is not None:
            self._want(bias, torch.float32, "linear_qkv_rope bias", N)
        self._want(rope_cs, torch.float32, "linear_qkv_rope angles", M, hd // 2, 2)
        self._want(slot_map, torch.int32, "linear_qkv_rope slot_map", M)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
        self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        q = torch.empty((M, H * hd), dtype=self.dtype, device=a.device)
        self._check(self._core, self._core.ms_linear_qkv_rope(
            _ptr(a), _ptr(w_qkv), _ptr(bias), _ptr(rope_cs), _ptr(slot_map), _ptr(q), _ptr(kpool), _ptr(vpool), _c_int(M), _c_int(H),
            _c_int(KV), _c_int(hd), _c_int(page_size), _c_int(K), self._stream()))
        return q

    # ------------------------------------------------------------------ matrix products
    def _mm_operands(self, a: torch.Tensor, w: torch.Tensor, what: str):
        self._want(a, self.dtype, f"{what} input")
        self._want(w, self.dtype, f"{what} weight")
        M, K = a.shape
        if w.shape[1] != K:
            raise KernelError(f"{what}: input has {K} columns, weight has {w.shape[1]}")
        return M, w.shape[0], K

    SKINNY_ROWS = 64  # at most this many rows: the weight-streaming kernels

    def _plan(self, what: str, *sizes: int, lib=None) -> int:
        key = (what, sizes)
        v = self._plans.get(key)
        if v is None:
            v = self._plans[key] = int(getattr(lib or self._core, what)(*[_c_int(x) for x in sizes]))
        return v

    def _tiled(self, M: int, N: int, K: int) -> bool:
        """Whether the tiled kernel takes this product: always above SKINNY_ROWS rows; below, where it was
        measured faster (in bfloat16 every large weight from one row on, because its blocks stream the
        weight with several K steps in flight, and smaller ones from 8 to 32 rows on; never in 32-bit)."""
        return M > self.SKINNY_ROWS or bool(self._plan("ms_prefers_tiled", M, N, K))

    def linear_split(self, a: torch.Tensor, w: torch.Tensor, allow_partials: bool = True) -> torch.Tensor:
        """Float32 ``[P, M, N]`` whose sum over P is ``a @ w.T``.  Within one kernel family the cut
        of K depends on N and K only, so the consumer that adds the parts sees the same sums for a row
        whatever else is in the batch; which family runs depends on the number of rows (see
        :meth:`_tiled`), and the two differ in rounding."""
        M, N, K = self._mm_operands(a, w, "linear_split")
        if self._tiled(M, N, K):
            P = self._plan("ms_tiled_partials", M, N, K) if allow_partials else 1
            if P == 1:
                return self.linear(a, w, None, out_f32=True).unsqueeze(0)
            out = torch.empty((P, M, N), dtype=torch.float32, device=a.device)
            self._check(self._core, self._core.ms_linear_split_tiled(_ptr(a), _ptr(w), _ptr(out), _c_int(M), _c_int(N),
                                                                     _c_int(K), self._stream()))
            return out
        P = self._plan("ms_skinny_partials", M, N, K, int(allow_partials))
        out = torch.empty((P, M, N), dtype=torch.float32, device=a.device)
        self._check(self._core, self._core.ms_linear_skinny(_ptr(a), _ptr(w), _ptr(out), _c_int(M), _c_int(N), _c_int(K),
                                                            _c_int(int(allow_partials)), self._stream()))
        return out

    def linear(self, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
               out_f32: bool = False) -> torch.Tensor:
        """``a @ w.T (+ bias)``; 32-bit output on request (logits)."""
        M, N, K = self._mm_operands(a, w, "linear")
        if not self._tiled(M, N, K) and out_f32 and bias is None:
            return self.linear_split(a, w, allow_partials=False)[0]
        if bias is not None:
            self._want(bias, torch.float32, "linear bias", N)
        out = torch.empty((M, N), dtype=torch.float32 if out_f32 else self.dtype, device=a.device)
        self._check(self._core, self._core.ms_linear(_ptr(a), _ptr(w), _ptr(bias), _ptr(out), _c_int(int(out_f32)),
                                                     _c_int(M), _c_int(N), _c_int(K), self._stream()))
        return out

    def linear_residual(self, a: torch.Tensor, w: torch.Tensor, x: torch.Tensor) -> Optional[torch.Tensor]:
        """``x += a @ w.T`` in the 32-bit residual stream.  When the product is cut along K over several
        blocks (a long K under few rows, or too few tiles to fill the chip) the sum is not added here:
        the float32 partial sums ``[P, M, N]`` are returned for the consumer (the next norm) to fold
        in; otherwise None."""
        M, N, K = self._mm_operands(a, w, "linear_residual")
        self._want(x, torch.float32, "residual stream", M, N)
        if not self._tiled(M, N, K):
            if M > 32 or self._plan("ms_skinny_partials", M, N, K, 1) > 1:
                return self.linear_split(a, w)
            # all of K inside one block: one writer an element, added in the epilogue (up to 32 rows the
            # kernel has registers to ask for the stream's values ahead; beyond, the next norm adds the sum)
            self._check(self._core, self._core.ms_linear_residual_skinny(_ptr(a), _ptr(w), _ptr(x), _c_int(M), _c_int(N),
                                                                         _c_int(K), self._stream()))
            return None
        if self._plan("ms_tiled_partials", M, N, K) > 1:
            return self.linear_split(a, w)
        self._check(self._core, self._core.ms_linear_residual(_ptr(a), _ptr(w), _ptr(x), _c_int(M), _c_int(N), _c_int(K),
                                                              self._stream()))
        return None

    def prenorm_swiglu_takes(self, M: int, N: int, K: int, n_gate_up: int) -> bool:
        """Whether ``x += a @ w.T`` (``w [N, K]``) followed by the gated product of ``rmsnorm(x)`` with an
        interleaved weight of ``n_gate_up`` rows can run as two kernels without a norm between them: the
        first leaves ``x * norm_w`` and the rows' sums of squares beside the sum, the second divides its
        finished sums by the root mean square (:meth:`linear_residual_prenorm`, :meth:`linear_swiglu_scaled`)."""
        return (not self._tiled(M, N, K) and self._plan("ms_skinny_prenorm_parts", M, N, K) > 0
                and bool(self._plan("ms_swiglu_scaled_takes", M, n_gate_up // 2, N)
                         or self._plan("ms_swiglu_scaled_skinny_takes", M, n_gate_up // 2, N)))

    def linear_residual_prenorm(self, a: torch.Tensor, w: torch.Tensor, x: torch.Tensor, norm_w: torch.Tensor):
        """``x += a @ w.T`` in place; returns ``(x * norm_w`` in the element type, float32 ``[parts, M]`` whose sum
        over parts is the rows' sums of squares of ``x``)``."""
        M, N, K = self._mm_operands(a, w, "linear_residual_prenorm")
        self._want(x, torch.float32, "residual stream", M, N)
        self._want(norm_w, torch.float32, "norm weight", N)
        parts = self._plan("ms_skinny_prenorm_parts", M, N, K)
        if parts < 1:
            raise KernelError(f"linear_residual_prenorm: M={M} N={N} K={K} is not taken")
        hn = torch.empty((M, N), dtype=self.dtype, device=a.device)
        ss = torch.empty((parts, M), dtype=torch.float32, device=a.device)
        self._check(self._core, self._core.ms_linear_residual_prenorm_skinny(
            _ptr(a), _ptr(w), _ptr(x), _ptr(norm_w), _ptr(hn), _ptr(ss), _c_int(M), _c_int(N), _c_int(K), self._stream()))
        return hn, ss

    def linear_swiglu_scaled(self, hn: torch.Tensor, row_ss: torch.Tensor, eps: float, w_gate_up: torch.Tensor,
                             intermediate: int, activation: str = "silu") -> torch.Tensor:
        """:meth:`linear_swiglu` of rows ``hn`` that lack their norm's division: both products of a row are
        divided by ``sqrt(sum(row_ss[:, row]) / K + eps)`` before the activation."""
        act = gate_activation_code(activation)
        M, N, K = self._mm_operands(hn, w_gate_up, "linear_swiglu_scaled")
        if N != 2 * ((intermediate + 15) // 16) * 16:
            raise KernelError(f"linear_swiglu_scaled: interleaved weight has {N} rows for intermediate size {intermediate}")
        self._want(row_ss, torch.float32, "linear_swiglu_scaled sums of squares", row_ss.shape[0], M)
        out = torch.empty((M, intermediate), dtype=self.dtype, device=hn.device)
        few_rows = bool(self._plan("ms_swiglu_scaled_skinny_takes", M, intermediate, K))
        fn = self._core.ms_linear_swiglu_scaled_skinny if few_rows else self._core.ms_linear_swiglu_scaled
        self._check(self._core, fn(_ptr(hn), _ptr(row_ss), _c_int(row_ss.shape[0]), _c_float(eps), _ptr(w_gate_up), _ptr(out),
                                   _c_int(M), _c_int(intermediate), _c_int(K), _c_int(act), self._stream()))
        return out

    def linear_swiglu(self, a: torch.Tensor, w_gate_up: torch.Tensor, intermediate: int, activation: str = "silu") -> torch.Tensor:
        """``act(a @ gate.T) * (a @ up.T)`` with gate and up rows interleaved in blocks of 16
        (see :func:`interleave_gate_up`); ``activation`` is one of :data:`GATE_ACTIVATIONS` (SiLU gives the
        method its name)."""
        act = gate_activation_code(activation)
        M, N, K = self._mm_operands(a, w_gate_up, "linear_swiglu")
        if N != 2 * ((intermediate + 15) // 16) * 16:
            raise KernelError(f"linear_swiglu: interleaved weight has {N} rows for intermediate size {intermediate}")
        out = torch.empty((M, intermediate), dtype=self.dtype, device=a.device)
        fn = self._core.ms_linear_swiglu if self._tiled(M, N, K) else self._core.ms_linear_swiglu_skinny
        self._check(self._core, fn(_ptr(a), _ptr(w_gate_up), _ptr(out), _c_int(M), _c_int(intermediate), _c_int(K),
                                   _c_int(act), self._stream()))
        return out

    # ------------------------------------------------------------------ products with the norm folded in
    def norm_folds_into(self, M: int, N: int, K: int, n_partials: int) -> bool:
        """Whether a few-rows product over the stream can apply the stream's RMS norm itself (at most
        16 rows, and a shape the few-rows kernel would take anyway)."""
        return (not self._tiled(M, N, K)
                and bool(self._plan("ms_skinny_norm_takes", M, N, K, n_partials)))

    def _normed_operands(self, x, partials, norm_w, w, what):
        M, K = x.shape
        self._want(x, torch.float32, f"{what} stream", M, K)
        self._want(norm_w, torch.float32, f"{what} norm weight", K)
        self._want(w, self.dtype, f"{what} weight")
        if w.dim() != 2 or w.shape[1] != K:
            raise KernelError(f"{what}: weight {tuple(w.shape)} for a stream of width {K}")
        P = 0
        if partials is not None:
            P = partials.shape[0]
            self._want(partials, torch.float32, f"{what} pending sums", P, M, K)
        x_new = torch.empty_like(x) if P else None
        return M, w.shape[0], K, P, x_new

    def linear_split_normed(self, x: torch.Tensor, partials: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                            w: torch.Tensor):
        """``rmsnorm(x + sum(partials)) @ w.T`` as float32 ``[1, M, N]``, and the stream with the
        pending sums added (a new tensor; None if nothing was pending)."""
        M, N, K, P, x_new = self._normed_operands(x, partials, norm_w, w, "linear_split_normed")
        out = torch.empty((1, M, N), dtype=torch.float32, device=x.device)
        self._check(self._core, self._core.ms_linear_norm_skinny(
            _ptr(x), _ptr(partials), _c_int(P), _c_int(M), _ptr(norm_w), _c_float(eps), _ptr(x_new), _ptr(w), _ptr(out),
            _c_int(M), _c_int(N), _c_int(K), self._stream()))
        return out, x_new

    def linear_swiglu_normed(self, x: torch.Tensor, partials: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float,
                             w_gate_up: torch.Tensor, intermediate: int, activation: str = "silu"):
        """``act(h @ gate.T) * (h @ up.T)`` for ``h = rmsnorm(x + sum(partials))`` (see
        :meth:`linear_swiglu`), and the stream with the pending sums added (or None)."""
        act = gate_activation_code(activation)
        M, N, K, P, x_new = self._normed_operands(x, partials, norm_w, w_gate_up, "linear_swiglu_normed")
        if N != 2 * ((intermediate + 15) // 16) * 16:
            raise KernelError(f"linear_swiglu_normed: interleaved weight has {N} rows for intermediate size {intermediate}")
        out = torch.empty((M, intermediate), dtype=self.dtype, device=x.device)
        self._check(self._core, self._core.ms_linear_swiglu_norm_skinny(
            _ptr(x), _ptr(partials), _c_int(P), _c_int(M), _ptr(norm_w), _c_float(eps), _ptr(x_new), _ptr(w_gate_up), _ptr(out),
            _c_int(M), _c_int(intermediate), _c_int(K), _c_int(act), self._stream()))
        return out, x_new

    # ------------------------------------------------------------------ attention
    def _attention_lib(self, hd: int):
        nd = build.attention_tile_for(hd)
        if nd not in self._attn:
            lib = self._load(build.ensure_library("attention", self.elem, nd))
            self._attn[nd] = (lib, getattr(lib, f"ms_paged_attention_nd{nd}"),
                              getattr(lib, f"ms_attention_rows_per_block_nd{nd}")(),
                              getattr(lib, f"ms_decode_attention_nd{nd}"), getattr(lib, f"ms_attention_key_tile_nd{nd}")(),
                              getattr(lib, f"ms_decode_attention_fused_nd{nd}"))
        return self._attn[nd]

    def attention_rows_per_block(self, hd: int) -> int:
        return self._attention_lib(hd)[2]

    def paged_attention(self, q: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_table: torch.Tensor,
                        seq_q_start: torch.Tensor, seq_q_len: torch.Tensor, seq_pos0: torch.Tensor,
                        work: torch.Tensor, H: int, KV: int, hd: int, page_size: int, window: Optional[int],
                        scale: float, max_key_groups: int = 0, key_splits: int = 0) -> torch.Tensor:
        """``max_key_groups`` asks for that many groups of waves sharing a block's keys (0: the kernel's
        choice); ``key_splits`` for that many blocks sharing them (0: the library's choice by the number of blocks
        of rows, the step's rows and the width of the block tables), merged by a second kernel."""
        lib, fn = self._attention_lib(hd)[:2]
        T = q.shape[0]
        self._want(q, self.dtype, "attention q", T, H * hd)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
        self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        S = seq_q_start.numel()
        self._want(block_table, torch.int32, "block table")
        if block_table.dim() != 2 or block_table.shape[0] != S:
            raise KernelError(f"attention: block table {tuple(block_table.shape)} for {S} requests")
        for t, n in ((seq_q_start, "seq_q_start"), (seq_q_len, "seq_q_len"), (seq_pos0, "seq_pos0")):
            self._want(t, torch.int32, n, S)
        self._want(work, torch.int32, "attention work")
        if work.dim() != 2 or work.shape[1] != 2 or work.shape[0] == 0:
            raise KernelError(f"attention: work list of shape {tuple(work.shape)}")
        out = torch.empty((T, H * hd), dtype=self.dtype, device=q.device)
        nsplit = key_splits or self._plan(f"ms_attention_splits_nd{build.attention_tile_for(hd)}", work.shape[0], KV, T, hd, page_size,
                                          block_table.shape[1], window or 0, lib=lib)
        part_o = part_ml = None
        if nsplit > 1:
            part_o = torch.empty((T, H, nsplit, hd), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((T, H, nsplit, 2), dtype=torch.float32, device=q.device)
        self._check(lib, fn(_ptr(q), _ptr(kpool), _ptr(vpool), _ptr(out), _ptr(block_table), _c_int(block_table.shape[1]),
                            _ptr(seq_q_start), _ptr(seq_q_len), _ptr(seq_pos0), _ptr(work), _c_int(work.shape[0]),
                            _c_int(H), _c_int(KV), _c_int(hd), _c_int(page_size), _c_int(pages), _c_int(window or 0),
                            _c_float(scale), _c_int(max_key_groups), _c_int(T), _c_int(nsplit), _ptr(part_o), _ptr(part_ml),
                            self._stream()))
        return out

    DECODE_MAX_GROUP = 16  # query heads per key/value head the decode kernel takes

    def _decode_splits(self, S: int, KV: int, table_width: int, page_size: int, window: Optional[int], key_tile: int,
                       hd: int = 64) -> int:
        """Blocks sharing a request's keys: as many as stay within one round of the chip, which holds two blocks a CU
        with small heads and one with heads above 64 (measured at head sizes 64 and 128, 1 to 200 requests: a split more
        than that starts a second round of blocks, and every round has the kernel's whole chain of latencies in it: 7B
        heads, 48 requests of 512 keys, 22 us uncut, 31 in two; 0.5B heads, 200 requests, 19 against 25), at least
        four key tiles each."""
        span = table_width * page_size if not window else min(table_width * page_size, window + key_tile)
        tiles = max(1, -(-span // key_tile))
        blocks = self._cus * (2 if hd <= 64 else 1)
        return max(1, min(blocks // (S * KV), -(-tiles // 4), 64))

    def decode_attention_fused(self, qkv: torch.Tensor, bias: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor],
                               slot_map: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor,
                               block_table: torch.Tensor, seq_pos0: torch.Tensor, H: int, KV: int, hd: int,
                               page_size: int, window: Optional[int], scale: float) -> torch.Tensor:
        """Decode attention from the partial sums ``qkv [P, S, stride]`` of the q/k/v projection: bias,
        rotation, cache write and attention over the pages in one launch, the merge of the
        splits in a second."""
        lib, key_tile, fn = self._attention_lib(hd)[0], self._attention_lib(hd)[4], self._attention_lib(hd)[5]
        if qkv.dim() == 2:
            qkv = qkv.unsqueeze(0)
        P, S, stride = qkv.shape
        self._want(qkv, torch.float32, "attention qkv")
        if bias is not None:
            self._want(bias, torch.float32, "attention bias", stride)
        if inv_freq is not None:
            self._want(inv_freq, torch.float32, "attention inv_freq", hd // 2)
        self._want(slot_map, torch.int32, "attention slot_map", S)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
        self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        self._want(block_table, torch.int32, "block table")
        if block_table.dim() != 2 or block_table.shape[0] != S:
            raise KernelError(f"attention: block table {tuple(block_table.shape)} for {S} requests")
        self._want(seq_pos0, torch.int32, "seq_pos0", S)
        if H // KV > self.DECODE_MAX_GROUP:
            raise KernelError(f"decode attention: {H // KV} heads per key/value head, at most {self.DECODE_MAX_GROUP}")
        nsplit = self._decode_splits(S, KV, block_table.shape[1], page_size, window, key_tile, hd)
        out = torch.empty((S, H * hd), dtype=self.dtype, device=qkv.device)
        part_o = part_ml = None
        if nsplit > 1:
            part_o = torch.empty((S, H, nsplit, hd), dtype=torch.float32, device=qkv.device)
            part_ml = torch.empty((S, H, nsplit, 2), dtype=torch.float32, device=qkv.device)
        self._check(lib, fn(_ptr(qkv), _c_int(P), _c_int(stride), _ptr(bias), _ptr(inv_freq), _ptr(slot_map), _ptr(kpool),
                            _ptr(vpool), _ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(block_table),
                            _c_int(block_table.shape[1]), _ptr(seq_pos0), _c_int(S), _c_int(H), _c_int(KV), _c_int(hd),
                            _c_int(page_size), _c_int(window or 0), _c_int(nsplit), _c_float(scale), self._stream()))
        return out

    def decode_attention(self, q: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_table: torch.Tensor,
                         seq_pos0: torch.Tensor, H: int, KV: int, hd: int, page_size: int, window: Optional[int],
                         scale: float) -> torch.Tensor:
        """Attention of a step in which request ``s`` has the single row ``s``.  The keys are cut
        into splits so that the grid fills the chip; how many follows from the number of
        requests and the width of the block table only."""
        lib, _, _, fn, key_tile = self._attention_lib(hd)[:5]
        S = q.shape[0]
        self._want(q, self.dtype, "attention q", S, H * hd)
        pages = kpool.shape[0]
        self._want(kpool, self.dtype, "key pool", pages, KV, page_size, hd)
        self._want(vpool, self.dtype, "value pool", pages, KV, hd, page_size)
        self._want(block_table, torch.int32, "block table")
        if block_table.dim() != 2 or block_table.shape[0] != S:
            raise KernelError(f"attention: block table {tuple(block_table.shape)} for {S} requests")
        self._want(seq_pos0, torch.int32, "seq_pos0", S)
        if H // KV > self.DECODE_MAX_GROUP:
            raise KernelError(f"decode attention: {H // KV} heads per key/value head, at most {self.DECODE_MAX_GROUP}")
        nsplit = self._decode_splits(S, KV, block_table.shape[1], page_size, window, key_tile, hd)
        out = torch.empty((S, H * hd), dtype=self.dtype, device=q.device)
        part_o = part_ml = None
        if nsplit > 1:
            part_o = torch.empty((S, H, nsplit, hd), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((S, H, nsplit, 2), dtype=torch.float32, device=q.device)
        self._check(lib, fn(_ptr(q), _ptr(kpool), _ptr(vpool), _ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(block_table),
                            _c_int(block_table.shape[1]), _ptr(seq_pos0), _c_int(S), _c_int(H), _c_int(KV), _c_int(hd),
                            _c_int(page_size), _c_int(window or 0), _c_int(nsplit), _c_float(scale), self._stream()))
        return out

    # ------------------------------------------------------------------ sampling
    def sample(self, logits, temperature, top_k, top_p, state, any_greedy: bool = True):
        """One token per row; ``state`` (int64 SplitMix64 states) advances in place.
        Returns ``(tokens int32, logprobs float32)``."""
        both = self.sample_packed(logits, temperature, top_k, top_p, state, any_greedy)
        return both[0], both[1].view(torch.float32)

    def sample_packed(self, logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                      state: torch.Tensor, any_greedy: bool = True, also_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """:meth:`sample` with both results in one int32 tensor ``[2, W]`` (tokens, then the bits of
        the logprobs) so that one copy brings them to the host.  With ``any_greedy`` a first
        launch finds the maxima of 64 chunks of every row, so that a greedy row is not one
        block's serial scan.  ``also_tokens`` (int32 ``[W]``) receives the tokens as well: the
        place where a following step reads its input."""
        W, V = logits.shape
        self._want(logits, torch.float32, "sample logits")
        self._want(temperature, torch.float32, "sample temperature", W)
        self._want(top_k, torch.int32, "sample top_k", W)
        self._want(top_p, torch.float32, "sample top_p", W)
        self._want(state, torch.int64, "sample state", W)
        if also_tokens is not None:
            self._want(also_tokens, torch.int32, "sample also_tokens", W)
        both = torch.empty((2, W), dtype=torch.int32, device=logits.device)  # tokens, then logprob bits
        tok, lp = both[0], both[1].view(torch.float32)
        pv = pi = None
        if any_greedy:
            chunks = self._core.ms_sample_chunks()
            pv = torch.empty((W, chunks), dtype=torch.float32, device=logits.device)
            pi = torch.empty((W, chunks), dtype=torch.int32, device=logits.device)
        self._check(self._core, self._core.ms_sample(_ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                                     _ptr(state), _ptr(tok), _ptr(lp), _ptr(pv), _ptr(pi),
                                                     _ptr(also_tokens), _c_int(W), _c_int(V), self._stream()))
        return both

    def top_logprobs(self, logits: torch.Tensor, inv_t: torch.Tensor, k: int):
        """The ``k`` most probable tokens of every row and their log-probabilities at the row's
        temperature (``inv_t``), ties to the smaller id.  Returns ``(tokens [W, k], logprobs [W, k])``."""
        W, V = logits.shape
        self._want(logits, torch.float32, "top_logprobs logits")
        self._want(inv_t, torch.float32, "top_logprobs inv_t", W)
        width = self._core.ms_top_logprobs_max()
        tok = torch.empty((W, width), dtype=torch.int32, device=logits.device)
        lp = torch.empty((W, width), dtype=torch.float32, device=logits.device)
        self._check(self._core, self._core.ms_top_logprobs(_ptr(logits), _ptr(inv_t), _ptr(tok), _ptr(lp), _c_int(W),
                                                           _c_int(V), _c_int(k), self._stream()))
        return tok[:, :k], lp[:, :k]

    def logit_edit(self, logits: torch.Tensor, row_of: torch.Tensor, token: torch.Tensor, delta: torch.Tensor) -> None:
        """``logits[row_of[e], token[e]] += delta[e]`` (penalties and biases merged on the host)."""
        n = row_of.numel()
        self._want(logits, torch.float32, "logit_edit logits")
        self._want(row_of, torch.int32, "logit_edit rows", n)
        self._want(token, torch.int32, "logit_edit tokens", n)
        self._want(delta, torch.float32, "logit_edit deltas", n)
        self._check(self._core, self._core.ms_logit_edit(_ptr(logits), _c_int(logits.shape[1]), _ptr(row_of), _ptr(token),
                                                         _ptr(delta), _c_int(n), self._stream()))


# The activations a gated product applies to its gate branch, by the name a specification gives them, and the
# number the kernels know them by.
GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def gate_activation_code(name: str) -> int:
    try:
        return GATE_ACTIVATIONS[name]
    except KeyError:
        raise KernelError(f"gated product: activation {name!r} is not built (built: {', '.join(sorted(GATE_ACTIVATIONS))})") from None


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``[2 * ceil16(I), d]``: blocks of 16 gate rows and the same 16 up rows alternate, zero
    rows pad the last block; the layout :meth:`HipOps.linear_swiglu` multiplies by."""
    I, d = gate.shape
    Ip = (I + 15) // 16 * 16
    g = torch.zeros((Ip, d), dtype=gate.dtype, device=gate.device)
    u = torch.zeros((Ip, d), dtype=gate.dtype, device=gate.device)
    g[:I] = gate
    u[:I] = up
    return torch.stack([g.view(Ip // 16, 16, d), u.view(Ip // 16, 16, d)], dim=1).reshape(2 * Ip, d).contiguous()


_OPS = {}


def get_ops(dtype: torch.dtype, device: str = "cuda:0") -> HipOps:
    key = (dtype, device)
    if key not in _OPS:
        _OPS[key] = HipOps(dtype, device)
    return _OPS[key]
