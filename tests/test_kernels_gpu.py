"""Each HIP kernel alone against its plain reference, at sizes other than the engine's:
head sizes in steps of 16, odd numbers of heads and groups, widths and vocabularies that
are no power of two, page sizes 16 to 128, single rows beside long portions."""
import math

import pytest
import torch

from emulated_ops import EmulatedOps
from gpu_util import DEV, assert_close
from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def ops_for(dtype):
    from machserve_amd.kernels import get_ops
    return get_ops(dtype, DEV)


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,V,d", [(1, 50, 24), (37, 1000, 200), (300, 777, 896)])
def test_embed(dtype, T, V, d):
    ops = ops_for(dtype)
    table = rnd((V, d), dtype, 1)
    toks = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(2), dtype=torch.int32)
    got = ops.embed(toks.to(DEV), table.to(DEV))
    assert torch.equal(got.cpu(), table[toks.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,d,eps", [(1, 8, 1e-6), (5, 200, 1e-5), (130, 896, 1e-6), (3, 5000, 1e-2), (7, 1536, 1e-6), (6, 4100, 1e-6)])
def test_rmsnorm(dtype, T, d, eps):
    ops = ops_for(dtype)
    x = rnd((T, d), torch.float32, 3, 3.0)
    w = 1 + rnd((d,), torch.float32, 4, 0.1)
    ref = P.rms_norm(x, w, eps)
    assert_close(ops.rmsnorm(x.to(DEV), w.to(DEV), eps), ref, dtype, "rmsnorm")
    rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32)
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, rows.to(DEV), out_f32=True)
    assert_close(got, ref[rows.long()], torch.float32, "rmsnorm of gathered rows")
    # pending sums are folded in, and written back when no rows are gathered
    parts = rnd((3, T, d), torch.float32, 5)
    total = x + parts.sum(0)
    xd = x.to(DEV).clone()
    assert_close(ops.rmsnorm(xd, w.to(DEV), eps, partials=parts.to(DEV)), P.rms_norm(total, w, eps), dtype, "norm of sums")
    assert_close(xd, total, torch.float32, "sums written back")
    xd = x.to(DEV).clone()
    got = ops.rmsnorm(xd, w.to(DEV), eps, rows.to(DEV), True, parts.to(DEV))
    assert_close(got, P.rms_norm(total, w, eps)[rows.long()], torch.float32, "gathered norm of sums")
    assert torch.equal(xd.cpu(), x), "gathered rows leave the stream alone"
    ops.add_partials(xd, parts.to(DEV))
    assert_close(xd, total, torch.float32, "add_partials")
    # eight, nine, twelve and sixteen pending sums (more than eight come in a second round of loads), each
    # plane with a value of its own scale so that a plane left out or taken twice shows
    for n in (8, 9, 12, 16, 17):
        parts = torch.stack([rnd((T, d), torch.float32, 20 + k, 0.5 + 0.25 * k) for k in range(n)])
        total = x + parts.sum(0)
        xd = x.to(DEV).clone()
        assert_close(ops.rmsnorm(xd, w.to(DEV), eps, partials=parts.to(DEV)), P.rms_norm(total, w, eps), dtype, f"norm of {n} sums")
        assert_close(xd, total, torch.float32, f"{n} sums written back")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 16, 8), (7, 1000, 200), (64, 130, 896), (65, 257, 72), (300, 896, 4864),
                                   (129, 9728 + 16, 64),
                                   # the tiled kernel's K steps: one partial step, one whole, two whole, whole + partial
                                   (70, 100, 40), (130, 64, 64), (100, 96, 128), (513, 1200, 136), (2048, 1152, 904),
                                   # few tiles, whole K steps: four LDS buffers in turn, with four, five, seven and nineteen steps
                                   (64, 200, 256), (48, 264, 320), (40, 130, 448), (100, 72, 1216),
                                   # so many tiles that tiles of 128x160 save a round: whole tiles, and ragged rows and columns
                                   (1024, 9728, 136), (1000, 9700, 264),
                                   # tiles of 256x256 under eight waves, taken where they fill their rounds of a block a CU: whole
                                   # tiles with two whole K steps; ragged rows and columns with a partial last step; a long K
                                   (4096, 4096, 128), (4000, 4090, 136), (3840, 3584, 1600)])
def test_linear(dtype, M, N, K):
    ops = ops_for(dtype)
    a, w = rnd((M, K), dtype, 5), rnd((N, K), dtype, 6, K ** -0.5)
    b = rnd((N,), torch.float32, 7)
    ref = P.linear(a.double(), w.double(), b.double())
    assert_close(ops.linear(a.to(DEV), w.to(DEV), b.to(DEV), out_f32=True), ref, torch.float32 if dtype == torch.float32 else dtype, "linear f32 out")
    assert_close(ops.linear(a.to(DEV), w.to(DEV), None), P.linear(a.double(), w.double()), dtype, "linear")
    x = rnd((M, N), torch.float32, 8)
    xd = x.to(DEV).clone()
    # K cut over several blocks (a long K under few rows, or few tiles): partial sums; else added in the epilogue
    pending = ops.linear_residual(a.to(DEV), w.to(DEV), xd)
    if pending is not None:
        ops.add_partials(xd, pending)
    assert_close(xd, x.double() + P.linear(a.double(), w.double()), torch.float32 if dtype == torch.float32 else dtype, "linear_residual")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(65, 896, 4864), (300, 130, 1096), (2048, 896, 4864), (200, 200, 520), (100, 1536, 8960),
                                   (100, 1536, 1536), (130, 136, 264),
                                   # a very long K under few tiles of 256x256: K cut so that the slices fill the chip's round
                                   (1000, 3584, 16448)])
def test_linear_many_rows_cut_along_k(dtype, M, N, K):
    """A product with too few tiles to fill the chip is cut along K into ordered partial sums."""
    ops = ops_for(dtype)
    a, w = rnd((M, K), dtype, 41), rnd((N, K), dtype, 42, K ** -0.5)
    parts = ops.linear_split(a.to(DEV), w.to(DEV))
    if K >= 16384:
        assert parts.shape[0] == (1 if dtype == torch.float32 else 4), "56 tiles of 256x256 in four slices are a round of the chip"
    assert parts.shape[1:] == (M, N) and (dtype != torch.float32 or parts.shape[0] == 1)
    assert_close(parts.sum(0), P.linear(a.double(), w.double()), torch.float32 if dtype == torch.float32 else dtype)
    assert ops.linear_split(a.to(DEV), w.to(DEV), allow_partials=False).shape[0] == 1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 16, 8), (3, 1000, 200), (8, 896, 4864), (17, 1152, 896), (17, 896, 904), (33, 130, 72),
                                   (64, 9728, 896), (5, 40000, 136), (48, 896, 896), (7, 1536, 1536), (3, 12000, 896)])
def test_linear_few_rows(dtype, M, N, K):
    """The weight-streaming kernels: partial sums that add up to the product, cut the same way
    for every number of rows, and a row's sums do not depend on the other rows."""
    ops = ops_for(dtype)
    a, w = rnd((M, K), dtype, 21), rnd((N, K), dtype, 22, K ** -0.5)
    ref = P.linear(a.double(), w.double())
    parts = ops.linear_split(a.to(DEV), w.to(DEV))
    assert parts.shape[1:] == (M, N)
    assert_close(parts.sum(0), ref, torch.float32 if dtype == torch.float32 else dtype, "sum of partial sums")
    whole = ops.linear_split(a.to(DEV), w.to(DEV), allow_partials=False)
    assert whole.shape == (1, M, N)
    assert_close(whole[0], ref, torch.float32 if dtype == torch.float32 else dtype, "one sum")
    assert_close(ops.linear(a.to(DEV), w.to(DEV), None, out_f32=True), ref, torch.float32 if dtype == torch.float32 else dtype)
    if M <= 32 and ops._tiled(M, N, K) == ops._tiled(1, N, K):
        # within one kernel family K is cut by N and K alone up to 32 rows: a row by itself gives the same bits
        alone = ops.linear_split(a[M - 1:].to(DEV).contiguous(), w.to(DEV))
        assert alone.shape[0] == parts.shape[0] and torch.equal(alone[:, 0], parts[:, M - 1])
    x0 = rnd((M, N), torch.float32, 23)
    x = x0.to(DEV)
    pend = ops.linear_residual(a.to(DEV), w.to(DEV), x)
    if pend is None:  # K inside one block, or a large weight under many rows (tiled kernel): added in the epilogue
        assert (parts.shape[0] == 1 and M <= 32) or ops._tiled(M, N, K)
        assert_close(x.cpu() - x0, ref, torch.float32 if dtype == torch.float32 else dtype, "added in place")
    else:
        assert torch.equal(pend, parts) and torch.equal(x.cpu(), x0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K,NP", [(1, 1152, 896, 0), (8, 1152, 896, 5), (16, 300, 264, 1), (3, 2048, 1536, 2),
                                      (5, 130, 1000, 3), (16, 4608, 3584, 6), (2, 64, 4864, 4)])
def test_products_with_the_norm_folded_in(dtype, M, N, K, NP):
    """rmsnorm(x + pending sums) times a weight in one kernel: the norm's factor applied to the
    finished sums, the stream with the sums added written to another buffer (the same bits as adding
    them in order), and the same with the gated activation."""
    from machserve_amd.kernels import interleave_gate_up
    ops = ops_for(dtype)
    # the engine folds the norm in only while there is little to read; the kernels take up to six pending sums
    # (never in half precision: the folded forms round x * weight before the division, which its range does not bear)
    assert ops.norm_folds_into(M, N, K, NP) == (dtype != torch.float16 and (NP == 0 or (NP == 1 and M <= 4)))
    assert not ops.norm_folds_into(17, N, K, 0)
    eps = 1e-5
    x = rnd((M, K), torch.float32, 31, 2.0)
    parts = rnd((NP, M, K), torch.float32, 32) if NP else None
    nw = 1 + rnd((K,), torch.float32, 33, 0.1)
    w = rnd((N, K), dtype, 34, K ** -0.5)
    total = x.clone()
    for p in range(NP):
        total += parts[p]
    h = P.rms_norm(total, nw, eps)
    ref = P.linear(h.double(), w.double())
    dev = lambda t: None if t is None else t.to(DEV)
    out, x_new = ops.linear_split_normed(dev(x), dev(parts), dev(nw), eps, dev(w))
    assert out.shape == (1, M, N) and (x_new is None) == (NP == 0)
    assert_close(out[0], ref, torch.float32 if dtype == torch.float32 else dtype, "product of the normed stream")
    if NP:
        assert torch.equal(x_new.cpu(), total), "the stream with its pending sums, added in order"
    I = N // 2 - 3
    g, u = rnd((I, K), dtype, 35, K ** -0.5 * 3), rnd((I, K), dtype, 36, K ** -0.5)
    ref = P.silu(P.linear(h.double(), g.double())) * P.linear(h.double(), u.double())
    got, x_new = ops.linear_swiglu_normed(dev(x), dev(parts), dev(nw), eps, interleave_gate_up(g, u).to(DEV), I)
    assert_close(got, ref, dtype, "gated product of the normed stream")
    if NP:
        assert torch.equal(x_new.cpu(), total)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K,I", [(8, 896, 896, 4864), (1, 896, 896, 4864), (20, 320, 264, 203), (32, 256, 128, 100),
                                     (5, 1000, 200, 50), (16, 1536, 904, 120), (3, 64, 72, 65536), (13, 2048, 136, 40),
                                     (17, 896, 896, 4864)])
def test_residual_product_prepares_the_norm_for_the_gated_product(dtype, M, N, K, I):
    """x += a w^T leaves x * norm_w and the rows' sums of squares beside the sum; the gated product of those rows
    divides its finished sums by the root mean square: together rmsnorm(x + a w^T) through gate and up."""
    from machserve_amd.kernels import interleave_gate_up
    ops = ops_for(dtype)
    if ops._plan("ms_skinny_prenorm_parts", M, N, K) < 1:
        pytest.skip("K is cut over several blocks for this shape, or the build is half precision (which rounds after the division)")
    eps = 1e-5
    a, w = rnd((M, K), dtype, 51), rnd((N, K), dtype, 52, K ** -0.5)
    x, nw = rnd((M, N), torch.float32, 53, 2.0), 1 + rnd((N,), torch.float32, 54, 0.1)
    x_new = x.double() + P.linear(a.double(), w.double())
    xd = x.to(DEV).clone()
    hn, ss = ops.linear_residual_prenorm(a.to(DEV), w.to(DEV), xd, nw.to(DEV))
    plain = torch.float32 if dtype == torch.float32 else dtype
    assert_close(xd, x_new, plain, "stream")
    assert_close(hn, xd.cpu().double() * nw.double(), dtype, "stream times the norm's weight")
    assert_close(ss.sum(0), (xd.cpu().double() ** 2).sum(1), torch.float32, "sums of squares")
    g, u = rnd((I, N), dtype, 55, N ** -0.5 * 3), rnd((I, N), dtype, 56, N ** -0.5)
    takes = ops.prenorm_swiglu_takes(M, N, K, 2 * ((I + 15) // 16) * 16)
    # the tiled form wants whole K steps of 64; at most 16 rows go to the few-rows form, which takes any K
    assert takes == (dtype == torch.bfloat16 and ((N % 64 == 0 and N >= 256) or M <= 16) and not ops._tiled(M, N, K))
    if takes:
        h = P.rms_norm(x_new.float(), nw, eps)
        ref = P.silu(P.linear(h.double(), g.double())) * P.linear(h.double(), u.double())
        got = ops.linear_swiglu_scaled(hn, ss, eps, interleave_gate_up(g, u).to(DEV), I)
        assert_close(got, ref, dtype, "gated product of the normed stream")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("scale,weight", [(1e4, 16.0), (1e-4, 0.02), (1.0, 1.0)])
@pytest.mark.parametrize("M", [1, 8, 16, 24])
def test_a_large_or_tiny_stream_goes_through_the_norm_and_its_reader(dtype, scale, weight, M):
    """The stream of a real checkpoint may be large (times a norm's weight: beyond half precision's 65,504) or tiny
    (among its subnormals): the norm's reader, whichever way it is run (the norm folded into the product, left to
    the product before it, or on its own), gives what the plain norm followed by the plain product gives, rounding
    after the division as the reference's f16 path does (crates/mach-model/src/kernels.rs:63-80)."""
    from machserve_amd.config import NormSpec
    from machserve_amd.kernels import interleave_gate_up
    from machserve_amd.parts import NORMS, ResidualStream, Runtime
    ops = ops_for(dtype)
    rt = Runtime(torch.device(DEV), dtype, ops)
    K, N, I, Ka, eps = 896, 1152, 4864, 896, 1e-13
    norm = NORMS.build(NormSpec("rmsnorm", K, eps), rt)
    nw = (1 + rnd((K,), torch.float32, 71, 0.1)) * weight
    norm.load({"weight": nw.to(DEV)})
    x = rnd((M, K), torch.float32, 72, scale)
    w = rnd((N, K), dtype, 73, K ** -0.5)
    g, u = rnd((I, K), dtype, 74, K ** -0.5 * 3 / weight), rnd((I, K), dtype, 75, K ** -0.5 / weight)
    a, wo = rnd((M, Ka), dtype, 76), rnd((K, Ka), dtype, 77, Ka ** -0.5 * scale)

    def rounded(h):
        return h.to(dtype).double()
    # 1. the norm's reader is a product that is summed later (q/k/v)
    stream = ResidualStream(x.to(DEV).clone(), ops)
    got = norm.pending(stream).linear_split(w.to(DEV)).sum(0)
    assert_close(got, P.linear(rounded(P.rms_norm(x, nw, eps)), w.double()), dtype, "q/k/v-like product of the normed stream")
    # 2. the reader is the gated product, and a product is still to be added to the stream before the norm
    stream = ResidualStream(x.to(DEV).clone(), ops)
    stream.add_linear(a.to(DEV), wo.to(DEV))
    got = norm.pending(stream).linear_swiglu(interleave_gate_up(g, u).to(DEV), I)
    x2 = (x.double() + P.linear(a.double(), wo.double())).float()
    h = rounded(P.rms_norm(x2, nw, eps))
    assert torch.isfinite(got.float()).all()
    assert_close(got, P.silu(P.linear(h, g.double())) * P.linear(h, u.double()), dtype, "gated product of the normed stream")
    assert_close(stream.value(), x2, torch.float32 if dtype == torch.float32 else dtype, "the stream itself")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I,K", [(1, 4864, 896), (9, 168, 64), (16, 4864, 896), (200, 328, 192), (40, 1000, 576)])
def test_gated_products_with_another_activation(dtype, M, I, K):
    """The activation on the gate is an argument: the tanh form of GELU (crates/mach-model/src/kernels.rs:199-208)
    against the library's own, through every kernel that applies an activation: the tiled and the few-rows gated
    product, the one that applies the stream's norm itself, and the one that divides its finished sums."""
    import torch.nn.functional as F
    from machserve_amd.kernels import KernelError, interleave_gate_up
    ops = ops_for(dtype)
    gelu = lambda t: F.gelu(t, approximate="tanh")
    a, g, u = rnd((M, K), dtype, 9), rnd((I, K), dtype, 10, K ** -0.5), rnd((I, K), dtype, 11, K ** -0.5)
    gate, up = P.linear(a.double(), g.double()), P.linear(a.double(), u.double())
    ref = gelu(gate) * up
    assert (ref - P.silu(gate) * up).abs().max() > 0.03 * ref.abs().max(), "the test must tell the activations apart"
    w = interleave_gate_up(g, u).to(DEV)
    assert_close(ops.linear_swiglu(a.to(DEV), w, I, "gelu_tanh"), ref, dtype, "gated product, GELU")
    assert_close(ops.linear_swiglu(a.to(DEV), w, I, "silu"), P.silu(gate) * up, dtype, "gated product, SiLU by name")
    with pytest.raises(KernelError, match="gelu_erf"):
        ops.linear_swiglu(a.to(DEV), w, I, "gelu_erf")
    eps = 1e-5
    x, nw = rnd((M, K), torch.float32, 12, 2.0), 1 + rnd((K,), torch.float32, 13, 0.1)
    h = P.rms_norm(x, nw, eps).double()
    ref = gelu(P.linear(h, g.double())) * P.linear(h, u.double())
    if ops.norm_folds_into(M, w.shape[0], K, 0):
        got, _ = ops.linear_swiglu_normed(x.to(DEV), None, nw.to(DEV), eps, w, I, "gelu_tanh")
        assert_close(got, ref, dtype, "gated product of the normed stream, GELU")
    Ka = 72
    if ops.prenorm_swiglu_takes(M, K, Ka, w.shape[0]):
        b, wo = rnd((M, Ka), dtype, 14), rnd((K, Ka), dtype, 15, Ka ** -0.5)
        xd = x.to(DEV).clone()
        hn, ss = ops.linear_residual_prenorm(b.to(DEV), wo.to(DEV), xd, nw.to(DEV))
        h = P.rms_norm(xd.cpu(), nw, eps).double()
        ref = gelu(P.linear(h, g.double())) * P.linear(h, u.double())
        assert_close(ops.linear_swiglu_scaled(hn, ss, eps, w, I, "gelu_tanh"), ref, dtype, "gated product with row factors, GELU")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,I,K", [(1, 16, 8), (9, 160, 64), (70, 328, 192), (200, 4864, 896), (64, 4864, 896), (33, 264, 136),
                                   (64, 328, 256), (50, 1000, 576),
                                   # tiles of 128x160 (five pairs of gate and up tiles): whole, and ragged at both edges
                                   (2048, 4864, 896), (1000, 4850, 200),
                                   # tiles of 256x256 (two pairs of gate and up tiles a wave): whole, and ragged at both edges
                                   (4096, 2048, 128), (4000, 2040, 200),
                                   # the same tiles where they fill 0.89 of the chip under a short K
                                   (1536, 4864, 896)])
def test_linear_swiglu(dtype, M, I, K):
    from machserve_amd.kernels import interleave_gate_up
    ops = ops_for(dtype)
    a, g, u = rnd((M, K), dtype, 9), rnd((I, K), dtype, 10, K ** -0.5 * 3), rnd((I, K), dtype, 11, K ** -0.5)
    ref = P.silu(P.linear(a.double(), g.double())) * P.linear(a.double(), u.double())
    got = ops.linear_swiglu(a.to(DEV), interleave_gate_up(g, u).to(DEV), I)
    assert_close(got, ref, dtype, "swiglu")
    swapped = P.silu(P.linear(a.double(), u.double())) * P.linear(a.double(), g.double())
    assert (ref - swapped).abs().max() > 0.05 * ref.abs().max(), "the test must tell gate from up"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,hd,ps,theta", [(4, 2, 16, 16, 1e4), (6, 1, 32, 32, 1e6), (5, 5, 48, 64, 5e4),
                                              (14, 2, 64, 64, 1e6), (3, 3, 128, 128, 1e6)])
def test_rope_kv_write(dtype, H, KV, hd, ps, theta):
    ops, emu = ops_for(dtype), EmulatedOps(dtype)
    T, pages = 45, 12
    qkv = rnd((T, (H + 2 * KV) * hd), torch.float32, 12)
    pos = torch.randint(0, 3000, (T,), generator=torch.Generator().manual_seed(13), dtype=torch.int32)
    perm = torch.randperm(pages * ps, generator=torch.Generator().manual_seed(14))[:T].to(torch.int32)
    j = torch.arange(hd // 2, dtype=torch.float32)
    inv = 1.0 / torch.pow(torch.tensor(theta, dtype=torch.float32), 2.0 * j / hd)
    kp, vp = torch.zeros(pages, KV, ps, hd, dtype=dtype), torch.zeros(pages, KV, hd, ps, dtype=dtype)
    q_ref = emu.rope_kv_write(qkv, None, pos, inv, perm, kp, vp, H, KV, hd, ps)
    # the emulation's rotation against the plain model's
    q_plain = P.rope(qkv[:, :H * hd].view(T, H, hd), pos, theta).reshape(T, H * hd)
    assert_close(q_ref, q_plain, dtype, "emulated rotation")
    kd, vd = torch.zeros_like(kp).to(DEV), torch.zeros_like(vp).to(DEV)
    q = ops.rope_kv_write(qkv.to(DEV), None, pos.to(DEV), inv.to(DEV), perm.to(DEV), kd, vd, H, KV, hd, ps)
    assert_close(q, q_plain, dtype, "q rotation")
    assert_close(kd, kp, dtype, "key pages")
    assert_close(vd, vp, dtype, "value pages")
    # without a table of frequencies nothing rotates
    q0 = ops.rope_kv_write(qkv.to(DEV), None, pos.to(DEV), None, None, None, None, H, KV, hd, ps)
    assert_close(q0, qkv[:, :H * hd], dtype, "no rotation")
    # three partial sums and a bias: the kernel adds them before it rotates
    parts = torch.stack([qkv * 0.5, qkv * 0.25 - 1.0, qkv * 0.25 + 1.0])
    bias = rnd(((H + 2 * KV) * hd,), torch.float32, 15)
    kp2, vp2 = torch.zeros_like(kp), torch.zeros_like(vp)
    q_ref2 = emu.rope_kv_write(qkv + bias, None, pos, inv, perm, kp2, vp2, H, KV, hd, ps)
    kd.zero_(), vd.zero_()
    q2 = ops.rope_kv_write(parts.to(DEV), bias.to(DEV), pos.to(DEV), inv.to(DEV), perm.to(DEV), kd, vd, H, KV, hd, ps)
    assert_close(q2, q_ref2, dtype, "q from partial sums")
    assert_close(kd, kp2, dtype, "key pages from partial sums")
    assert_close(vd, vp2, dtype, "value pages from partial sums")
    # seven and eleven partial sums (a portion of about a hundred rows cuts the projection's K seven times)
    for n in (7, 11):
        g = torch.Generator().manual_seed(16 + n)
        cut = torch.randn((n - 1, *qkv.shape), generator=g)
        parts = torch.cat([cut, (qkv - cut.sum(0)).unsqueeze(0)])
        kd.zero_(), vd.zero_()
        qn = ops.rope_kv_write(parts.to(DEV), bias.to(DEV), pos.to(DEV), inv.to(DEV), perm.to(DEV), kd, vd, H, KV, hd, ps)
        assert_close(qn, emu.rope_kv_write(parts.sum(0) + bias, None, pos, inv, perm, kp2.zero_(), vp2.zero_(), H, KV, hd, ps), dtype,
                     f"q from {n} partial sums")
        assert_close(kd, kp2, dtype, f"key pages from {n} partial sums")
        assert_close(vd, vp2, dtype, f"value pages from {n} partial sums")


def _dead_pages_removed(table, seqs, ps, window):
    """The block table as the cache manager hands it over once pages behind the window have been given
    back: a logical page that ends at or before ``cached - window + 1`` (no row of the step sees it) is -1."""
    table = table.clone()
    for i, (c, n) in enumerate(seqs):
        table[i, :max(0, c - window + 1) // ps] = -1
    return table


def _attention_case(dtype, H, KV, hd, ps, window, seqs, seed, peak=False, groups=0, splits=0, dead_pages=False):
    """seqs: list of (cached length, rows in this step).  Builds scattered pages holding random
    keys and values for positions < cached + rows and queries for the step's rows.  With
    ``dead_pages`` the kernel's block table has -1 where the pages lie wholly behind the window."""
    ops, emu = ops_for(dtype), EmulatedOps(dtype)
    g = H // KV
    gen = torch.Generator().manual_seed(seed)
    n_pages = sum(-(-(c + n) // ps) for c, n in seqs) + 3
    order = torch.randperm(n_pages, generator=gen).tolist()
    kp = rnd((n_pages, KV, ps, hd), dtype, seed + 1)
    vp = rnd((n_pages, KV, hd, ps), dtype, seed + 2)
    width = max(-(-(c + n) // ps) for c, n in seqs)
    table = torch.full((len(seqs), width), -1, dtype=torch.int32)
    q_start, q_len, pos0, work = [], [], [], []
    T = 0
    for i, (c, n) in enumerate(seqs):
        for p in range(-(-(c + n) // ps)):
            table[i, p] = order.pop()
        q_start.append(T), q_len.append(n), pos0.append(c)
        work += [(i, r0) for r0 in range(0, n * g, ops.attention_rows_per_block(hd))]
        T += n
    q = rnd((T, H * hd), dtype, seed + 3)
    if peak:
        # one far key stands out for one query row: scale that key and query so that the score
        # towers over the rest and a missed key shows in the output
        i, (c, n) = max(enumerate(seqs), key=lambda t: t[1][0])
        row, head, far = q_start[i] + n - 1, H - 1, (1 if not window else c + n - window)
        kvh = head // g
        page, off = int(table[i, far // ps]), far % ps
        qv = q[row, head * hd:(head + 1) * hd].float()
        kp[page, kvh, off, :] = (qv / qv.norm() * 8.0).to(dtype)
        q[row, head * hd:(head + 1) * hd] = (qv / qv.norm() * 8.0 * math.sqrt(hd) / 4).to(dtype)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    args = (i32(q_start), i32(q_len), i32(pos0), i32(work).view(-1, 2))
    if groups or splits:
        emu = EmulatedOps(torch.float32)  # the reference unrounded: the tolerance allows the output's one rounding
    emu.rows_per_block = ops.attention_rows_per_block(hd)
    ref = emu.paged_attention(q, kp, vp, table, *args, H, KV, hd, ps, window, hd ** -0.5)
    if dead_pages:
        table = _dead_pages_removed(table, seqs, ps, window)
        assert (table < 0).sum() > (table.shape[1] - torch.tensor([-(-(c + n) // ps) for c, n in seqs])).sum(), "no page is dead"
    got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV), table.to(DEV), *[a.to(DEV) for a in args], H, KV, hd,
                              ps, window, hd ** -0.5, groups, splits)
    return got, ref


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,hd,ps", [(4, 2, 16, 16), (6, 1, 32, 32), (5, 5, 48, 16), (14, 2, 64, 64), (7, 7, 80, 32),
                                        (12, 2, 128, 64), (20, 1, 64, 128), (2, 1, 256, 16)])
def test_attention_mixed_batch(dtype, H, KV, hd, ps):
    seqs = [(0, 1), (0, 70), (130, 1), (37, 45), (ps - 1, 2), (ps, 1), (2 * ps - 1, 1)]
    got, ref = _attention_case(dtype, H, KV, hd, ps, None, seqs, 100 + hd)
    assert_close(got, ref, dtype, "attention")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("groups", [1, 2, 4])
@pytest.mark.parametrize("H,KV,hd,ps,window", [(4, 2, 16, 16, None), (14, 2, 64, 64, None), (6, 3, 128, 32, None),
                                               (2, 1, 256, 16, None), (6, 2, 64, 16, 100), (3, 1, 48, 32, 333)])
def test_attention_key_groups(dtype, groups, H, KV, hd, ps, window):
    """The keys of a block shared by 1, 2 or 4 groups of waves: short and long requests in one
    launch, lengths that end inside a round of tiles, and a far key that must not be missed."""
    seqs = [(0, 1), (0, 300), (517, 1), (700, 37), (3, 2), (1023, 1), (64 * groups, 1), (64 * groups - 1, 2)]
    got, ref = _attention_case(dtype, H, KV, hd, ps, window, seqs, 300 + hd + groups, peak=True, groups=groups)
    assert_close(got, ref, dtype, f"attention with {groups} key groups")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits,dead_pages", [(0, False), (3, False), (0, True)])
@pytest.mark.parametrize("H,KV,hd,ps,window", [(14, 2, 64, 64, None), (6, 2, 64, 16, 100), (20, 1, 64, 128, None), (8, 8, 64, 32, 333),
                                               (3, 1, 64, 16, 31)])
def test_attention_in_tiles_of_32_rows(dtype, splits, dead_pages, H, KV, hd, ps, window):
    """The kernel of 32-row tiles that the two-byte libraries have for a head size of 64 (blocks of 128 flat rows, four
    key groups, tiles loaded straight into four LDS stages, the block table in LDS, a reference maximum that follows
    lazily), asked for by name: requests that end inside a tile, inside a round of four tiles and inside a block of
    rows, contexts of a few thousand keys, a window with the pages behind it given back, the keys cut over blocks, and
    a far key that must not be missed.  (The 32-bit library has no such kernel and answers with its general one.)"""
    if dead_pages and window is None:
        pytest.skip("pages are given back behind a window only")
    seqs = [(0, 1), (0, 300), (517, 1), (3000, 37), (3, 2), (1023, 1), (128, 1), (127, 2), (31, 2), (95, 130), (2040, 19)]
    got, ref = _attention_case(dtype, H, KV, hd, ps, window, seqs, 600 + ps + splits, peak=True, groups=32, splits=splits,
                               dead_pages=dead_pages)
    assert_close(got, ref, dtype, "attention in tiles of 32 rows")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits", [2, 5, 64])
@pytest.mark.parametrize("H,KV,hd,ps,window", [(4, 2, 16, 16, None), (14, 2, 64, 64, None), (6, 3, 128, 32, None),
                                               (6, 2, 64, 16, 100), (3, 1, 48, 32, 333)])
def test_attention_key_splits(dtype, splits, H, KV, hd, ps, window):
    """The keys of a block of rows cut over several blocks and merged: short and long requests in
    one launch (most splits of the short ones are empty), and a far key that must not be missed."""
    seqs = [(0, 1), (0, 300), (517, 1), (1500, 37), (3, 2), (1023, 1), (128, 1), (127, 2)]
    got, ref = _attention_case(dtype, H, KV, hd, ps, window, seqs, 400 + hd + splits, peak=True, splits=splits)
    assert_close(got, ref, dtype, f"attention with the keys cut over {splits} blocks")


def test_the_library_s_choice_of_key_splits():
    """How many blocks share the keys of a block of rows when the caller leaves it to the library: none for block
    tables that may belong to prompts running whole (no wider than twice the step's rows) and for a full chip; few rows
    behind a long context are cut, in the kernel of 32-row tiles (head size 64, two-byte elements) so that blocks times
    splits stay within the chip's CUs, at least 1,024 keys a split; a window bounds the keys that count."""
    ops = ops_for(torch.bfloat16)
    lib = ops._attention_lib(64)[0]
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    plan = lambda n_work, KV, T, hd, ps, width, window: lib.ms_attention_splits_nd4(n_work, KV, T, hd, ps, width, window)
    assert plan(56, 2, 1024, 64, 64, 32, 0) == 1                     # a prompt of 1,024 tokens whole
    assert plan(84, 2, 1536, 64, 64, 32, 0) == 1
    assert plan(14, 2, 256, 64, 64, 256, 0) == min(cus // 28, 16)    # 256 rows behind thousands of keys
    assert plan(28, 2, 512, 64, 64, 128, 0) == min(cus // 56, 8)
    assert plan(56, 2, 1024, 64, 64, 64, 0) == min(cus // 112, 4)
    assert plan(200, 2, 3600, 64, 64, 256, 0) == 1                   # the chip is full
    assert plan(1, 2, 1, 64, 64, 4096, 0) == 64                      # never more than the kernels take
    assert plan(14, 2, 256, 64, 64, 256, 500) == 1                   # a window of 500 keys: nothing to cut
    assert plan(4, 2, 64, 64, 16, 64, 0) == min(-(-384 // 8), 1024 // 512)   # a short table: the general kernel's rule
    lib128 = ops._attention_lib(128)[0]
    assert lib128.ms_attention_splits_nd8(7, 4, 256, 128, 64, 128, 0) == min(-(-384 // 28), 8192 // 512)
    f32 = ops_for(torch.float32)._attention_lib(64)[0]
    assert f32.ms_attention_splits_nd4(14, 2, 256, 64, 64, 256, 0) == min(-(-384 // 28), 16384 // 512)   # no 32-row kernel in 32-bit


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 17, 64, 100])
def test_attention_window(dtype, window):
    seqs = [(0, 150), (200, 1), (63, 3), (0, 1)]
    got, ref = _attention_case(dtype, 6, 2, 32, 16, window, seqs, 200 + window)
    assert_close(got, ref, dtype, f"attention with window {window}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,splits", [(17, 0), (100, 0), (100, 3), (333, 0)])
def test_attention_window_with_pages_given_back(dtype, window, splits):
    """The pages behind the window are gone (-1 in the block table), as the cache manager leaves them:
    the kernel never looks a dead page up, whichever key tile, group of waves or split would hold it; the far
    key at the window's edge still counts."""
    seqs = [(0, 150), (200, 1), (63, 3), (0, 1), (700, 30), (1023, 1)]
    got, ref = _attention_case(dtype, 6, 2, 32, 16, window, seqs, 500 + window, peak=True, splits=splits, dead_pages=True)
    assert_close(got, ref, dtype, f"attention with window {window} and dead pages")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 300])
def test_attention_far_key_stands_out(dtype, window):
    seqs = [(700, 1), (0, 5), (400, 40)]
    got, ref = _attention_case(dtype, 8, 2, 64, 64, window, seqs, 300, peak=True)
    assert_close(got, ref, dtype, "attention with a far key that dominates")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,hd,ps,window", [(4, 2, 16, 16, None), (6, 1, 32, 32, None), (5, 5, 48, 16, 40),
                                               (14, 2, 64, 64, None), (16, 1, 80, 32, 100), (12, 2, 128, 64, None),
                                               (2, 1, 256, 16, None), (14, 2, 64, 64, 1)])
def test_decode_attention(dtype, H, KV, hd, ps, window):
    """One row per request, contexts from 0 to a few thousand keys, scattered pages; against the
    plain attention of the same rows, and against the general kernel."""
    ops, emu = ops_for(dtype), EmulatedOps(dtype)
    lens = [0, 1, ps - 1, ps, 130, 700, 2049] if hd < 256 else [0, 5, 300]
    gen = torch.Generator().manual_seed(500 + hd)
    n_pages = sum(-(-(c + 1) // ps) for c in lens) + 2
    order = torch.randperm(n_pages, generator=gen).tolist()
    kp, vp = rnd((n_pages, KV, ps, hd), dtype, 501), rnd((n_pages, KV, hd, ps), dtype, 502)
    width = max(-(-(c + 1) // ps) for c in lens)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    for i, c in enumerate(lens):
        for p in range(-(-(c + 1) // ps)):
            table[i, p] = order.pop()
    S = len(lens)
    q = rnd((S, H * hd), dtype, 503)
    # one far key towers over the rest for the longest request's last head
    c = lens[-1]
    far = 3 if not window else max(0, c - window + 1)
    qv = q[S - 1, (H - 1) * hd:].float()
    kp[int(table[S - 1, far // ps]), KV - 1, far % ps, :] = (qv / qv.norm() * 8.0).to(dtype)
    q[S - 1, (H - 1) * hd:] = (qv / qv.norm() * 8.0 * math.sqrt(hd) / 4).to(dtype)
    pos0 = torch.tensor(lens, dtype=torch.int32)
    ref = emu.decode_attention(q, kp, vp, table, pos0, H, KV, hd, ps, window, hd ** -0.5)
    got = ops.decode_attention(q.to(DEV), kp.to(DEV), vp.to(DEV), table.to(DEV), pos0.to(DEV), H, KV, hd, ps, window, hd ** -0.5)
    assert_close(got, ref, dtype, "decode attention")
    ar = torch.arange(S, dtype=torch.int32)
    work = torch.stack([ar, torch.zeros_like(ar)], 1).contiguous()
    gen_out = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV), table.to(DEV), ar.to(DEV), torch.ones_like(ar).to(DEV),
                                  pos0.to(DEV), work.to(DEV), H, KV, hd, ps, window, hd ** -0.5)
    assert_close(got, gen_out.float().cpu(), dtype, "decode kernel against the general kernel")
    # a request alone (other split count) agrees within rounding
    one = ops.decode_attention(q[S - 1:].to(DEV).contiguous(), kp.to(DEV), vp.to(DEV), table[S - 1:].to(DEV).contiguous(),
                               pos0[S - 1:].to(DEV), H, KV, hd, ps, window, hd ** -0.5)
    assert_close(one, ref[S - 1:], dtype, "decode attention of one request")
    if window:
        # the pages behind the window given back, as the cache manager leaves the table
        dead = _dead_pages_removed(table, [(c, 1) for c in lens], ps, window)
        assert (dead[S - 1] < 0).sum() > 0
        got = ops.decode_attention(q.to(DEV), kp.to(DEV), vp.to(DEV), dead.to(DEV), pos0.to(DEV), H, KV, hd, ps, window, hd ** -0.5)
        assert_close(got, ref, dtype, "decode attention with dead pages")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,hd,ps,window,P_", [(4, 2, 16, 16, None, 1), (6, 1, 32, 32, None, 3), (5, 5, 48, 16, 40, 1),
                                                  (14, 2, 64, 64, None, 2), (12, 2, 128, 64, None, 1), (16, 1, 80, 32, 100, 1)])
def test_decode_attention_fused(dtype, H, KV, hd, ps, window, P_):
    """Bias, rotation, cache write and attention from partial sums of the projection; twice in a
    row with the same pages, the second time one position on, as decoding does."""
    ops, emu = ops_for(dtype), EmulatedOps(dtype)
    lens = [0, 1, ps - 1, ps, 130, 700, 2049, 63, 64]
    S = len(lens)
    gen = torch.Generator().manual_seed(600 + hd)
    n_pages = sum(-(-(c + 2) // ps) for c in lens) + 2
    order = torch.randperm(n_pages, generator=gen).tolist()
    kp, vp = rnd((n_pages, KV, ps, hd), dtype, 601), rnd((n_pages, KV, hd, ps), dtype, 602)
    width = max(-(-(c + 2) // ps) for c in lens)
    table = torch.full((S, width), -1, dtype=torch.int32)
    for i, c in enumerate(lens):
        for p in range(-(-(c + 2) // ps)):
            table[i, p] = order.pop()
    stride = (H + 2 * KV) * hd
    bias = rnd((stride,), torch.float32, 603)
    j = torch.arange(hd // 2, dtype=torch.float32)
    inv = 1.0 / torch.pow(torch.tensor(1e4), 2.0 * j / hd)
    kd, vd = kp.to(DEV), vp.to(DEV)
    for step in range(2):
        pos0 = torch.tensor([c + step for c in lens], dtype=torch.int32)
        slot_map = torch.tensor([int(table[i, (c + step) // ps]) * ps + (c + step) % ps for i, c in enumerate(lens)], dtype=torch.int32)
        qkv = rnd((S, stride), torch.float32, 604 + step)
        parts = torch.stack([qkv / P_ + (k - (P_ - 1) / 2) for k in range(P_)])  # P_ parts that sum to qkv
        ref = emu.decode_attention_fused(parts, bias, inv, slot_map, kp, vp, table, pos0, H, KV, hd, ps, window, hd ** -0.5)
        got = ops.decode_attention_fused(parts.to(DEV), bias.to(DEV), inv.to(DEV), slot_map.to(DEV), kd, vd, table.to(DEV),
                                         pos0.to(DEV), H, KV, hd, ps, window, hd ** -0.5)
        assert_close(got, ref, dtype, f"fused decode attention, step {step}")
        assert_close(kd, kp, dtype, "key pages")
        assert_close(vd, vp, dtype, "value pages")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,hd,ps,window", [(14, 2, 64, 64, None), (4, 1, 128, 16, None), (6, 2, 64, 32, 4000)])
def test_attention_long_contexts(dtype, H, KV, hd, ps, window):
    """Contexts of nine and twenty thousand keys: a decoded row (many splits, merged in batches) and
    a portion of a prompt far into its request, with a key near the start (or at the window's
    edge) that towers over the rest, so that a range of keys that went missing would show."""
    ops, emu = ops_for(dtype), EmulatedOps(dtype)
    lens = [20011, 9000, 5]
    S = len(lens)
    gen = torch.Generator().manual_seed(700 + hd)
    n_pages = sum(-(-(c + 1) // ps) for c in lens) + 2
    order = torch.randperm(n_pages, generator=gen).tolist()
    kp, vp = rnd((n_pages, KV, ps, hd), dtype, 701), rnd((n_pages, KV, hd, ps), dtype, 702)
    width = max(-(-(c + 1) // ps) for c in lens)
    table = torch.full((S, width), -1, dtype=torch.int32)
    for i, c in enumerate(lens):
        for p in range(-(-(c + 1) // ps)):
            table[i, p] = order.pop()
    q = rnd((S, H * hd), dtype, 703)
    for i in (0, 1):
        far = 2 if not window else lens[i] - window + 1
        qv = q[i, (H - 1) * hd:].float()
        kp[int(table[i, far // ps]), KV - 1, far % ps, :] = (qv / qv.norm() * 8.0).to(dtype)
        q[i, (H - 1) * hd:] = (qv / qv.norm() * 8.0 * math.sqrt(hd) / 4).to(dtype)
    pos0 = torch.tensor(lens, dtype=torch.int32)
    ref = emu.decode_attention(q, kp, vp, table, pos0, H, KV, hd, ps, window, hd ** -0.5)
    got = ops.decode_attention(q.to(DEV), kp.to(DEV), vp.to(DEV), table.to(DEV), pos0.to(DEV), H, KV, hd, ps, window, hd ** -0.5)
    assert_close(got, ref, dtype, "decode attention over long contexts")
    # the last 150 positions of the 9,000-key request as one portion
    n, c = 150, lens[1] + 1 - 150
    g = H // KV
    qq = rnd((n, H * hd), dtype, 704)
    qq[n - 1] = q[1]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    emu.rows_per_block = ops.attention_rows_per_block(hd)
    args = (i32([0]), i32([n]), i32([c]), i32([(0, r0) for r0 in range(0, n * g, emu.rows_per_block)]).view(-1, 2))
    tab = table[1:2].contiguous()
    ref2 = emu.paged_attention(qq, kp, vp, tab, *args, H, KV, hd, ps, window, hd ** -0.5)
    got2 = ops.paged_attention(qq.to(DEV), kp.to(DEV), vp.to(DEV), tab.to(DEV), *[a.to(DEV) for a in args], H, KV, hd, ps,
                               window, hd ** -0.5)
    assert_close(got2, ref2, dtype, "a portion far into a long request")
    assert_close(got2[n - 1:].float().cpu(), got[1:2].float().cpu(), dtype, "its last row against the decode kernel")


@pytest.mark.parametrize("H,KV,hd,ps,T", [(4, 4, 32, 16, 50), (6, 2, 64, 32, 131), (3, 1, 48, 16, 70)])
def test_attention_equals_library_attention_without_rotation_or_paging(H, KV, hd, ps, T):
    """One request, its whole prompt in one step, pages in order: the kernel is plain causal attention,
    ``torch.nn.functional.scaled_dot_product_attention`` with the key/value heads repeated for their
    groups (head h reads key/value head h // g).  Then the last row again through the decode kernel."""
    import torch.nn.functional as F
    dtype, g = torch.float32, H // KV
    ops = ops_for(dtype)
    q, k, v = rnd((T, H, hd), dtype, 1), rnd((T, KV, hd), dtype, 2), rnd((T, KV, hd), dtype, 3)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None].double(),
                                          k.transpose(0, 1).repeat_interleave(g, 0)[None].double(),
                                          v.transpose(0, 1).repeat_interleave(g, 0)[None].double(), is_causal=True)
    want = want[0].transpose(0, 1).reshape(T, H * hd).float()
    n_pages = -(-T // ps)
    kp, vp = torch.zeros(n_pages, KV, ps, hd), torch.zeros(n_pages, KV, hd, ps)
    for t in range(T):
        kp[t // ps, :, t % ps, :] = k[t]
        vp[t // ps, :, :, t % ps] = v[t]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    table = i32(list(range(n_pages))).view(1, -1)
    work = i32([(0, r0) for r0 in range(0, T * g, ops.attention_rows_per_block(hd))]).view(-1, 2)
    got = ops.paged_attention(q.reshape(T, H * hd).to(DEV), kp.to(DEV), vp.to(DEV), table, i32([0]), i32([T]), i32([0]), work,
                              H, KV, hd, ps, None, hd ** -0.5)
    assert_close(got, want, dtype, "kernel against library attention")
    last = ops.decode_attention(q[T - 1:].reshape(1, H * hd).to(DEV), kp.to(DEV), vp.to(DEV), table, i32([T - 1]), H, KV, hd, ps,
                                None, hd ** -0.5)
    assert_close(last, want[T - 1:], dtype, "decode kernel against library attention")


@pytest.mark.parametrize("dtype", DTYPES)
def test_refusals(dtype):
    from machserve_amd.kernels import KernelError
    ops = ops_for(dtype)
    a, w = torch.zeros(4, 12, dtype=dtype, device=DEV), torch.zeros(16, 12, dtype=dtype, device=DEV)
    with pytest.raises(KernelError, match="multiple of 8"):
        ops.linear(a, w)
    with pytest.raises(Exception, match="multiple of 16"):
        ops.attention_rows_per_block(40)
    with pytest.raises(KernelError, match="GPU tensor"):
        ops.linear(a.cpu(), w)


def test_sampler_matches_cpu_mirror():
    """Peaked logits as in crates/mach-model/src/sampling.rs:1711-1752: the boundary tiers and
    the draw land far from any edge, so the orders of summation cannot change the outcome."""
    ops = ops_for(torch.float32)
    V, n = 2048, 12
    logits = torch.zeros(n, V)
    for s in range(n):
        logits[s] = 0.5 - 1.2 * torch.arange(V) * 0.25
        logits[s, ::37] += 0.05
        logits[s] = logits[s].roll(s * 97)
    temps = torch.tensor([[0.8, 1.0, 1.2, 0.0][i % 4] for i in range(n)])
    ks = torch.tensor([[0, 0, 40, 10][i % 4] for i in range(n)], dtype=torch.int32)
    ps_ = torch.tensor([[0.95, 1.0, 0.9, 0.8][i % 4] for i in range(n)])
    seeds = torch.tensor([7000 + i for i in range(n)], dtype=torch.int64)
    state = seeds.clone().to(DEV)
    for rep in range(3):
        got, _ = ops.sample(logits.to(DEV), temps.to(DEV), ks.to(DEV), ps_.to(DEV), state, any_greedy=rep != 1)
        for i in range(n):
            st = int(seeds[i]) + rep * P.RNG_GOLDEN
            want, new = P.sample(logits[i].numpy(), float(temps[i]), int(ks[i]), float(ps_[i]), st & P.MASK64)
            assert int(got[i]) == want, f"row {i} rep {rep}"
    want_state = [(int(s) + 3 * P.RNG_GOLDEN) & P.MASK64 for s in seeds]
    assert [int(v) & P.MASK64 for v in state.cpu().tolist()] == want_state


def test_sampler_draw_at_the_top_of_the_mass_falls_back_to_the_first_allowed_token():
    """A draw of u = 1 - 2^-24 (state 4375518: the finalizer's top 24 bits are all ones) on a row whose
    last segment is 64 tokens of probability 2^-26 behind a mass of one: each of them is lost when added
    to the running sum, so no walk passes the target, and the rule for that case decides: the first
    allowed token, then the maximum (crates/mach-model/src/sampling.rs:385-400).  In the second row the
    first allowed token is not the maximum: the kernel's rule gives token 0 where the reference's CPU
    mirror, which falls back to the maximum (sampling.rs:1270-1273), would give token 5."""
    ops = ops_for(torch.float32)
    assert P.next_uniform(4375518)[0] == 1.0 - 2.0 ** -24
    V = 1024 * 64
    tiny = -26.0 * 0.6931471805599453
    logits = torch.full((2, V), -200.0)
    logits[:, -64:] = tiny
    logits[0, 0] = 0.0                    # the maximum is also the first allowed token
    logits[1, 0], logits[1, 5] = tiny, 0.0
    state = torch.tensor([4375518, 4375518], dtype=torch.int64, device=DEV)
    got, _ = ops.sample(logits.to(DEV), torch.ones(2, device=DEV), torch.zeros(2, dtype=torch.int32, device=DEV),
                        torch.ones(2, device=DEV), state, any_greedy=False)
    assert got.cpu().tolist() == [0, 0]
    assert P.sample(logits[0].numpy(), 1.0, 0, 1.0, 4375518)[0] == 0     # the mirror agrees where the two rules do
    # a draw far from the top of the same rows walks as usual
    state = torch.tensor([5, 5], dtype=torch.int64, device=DEV)
    got, _ = ops.sample(logits.to(DEV), torch.ones(2, device=DEV), torch.zeros(2, dtype=torch.int32, device=DEV),
                        torch.ones(2, device=DEV), state, any_greedy=False)
    assert got.cpu().tolist() == [0, 5]


def test_sampler_greedy_ties_and_spread():
    ops = ops_for(torch.float32)
    V = 1000
    logits = torch.zeros(3, V)
    logits[0, [5, 700, 999]] = 2.0           # ties: the smallest index wins
    logits[1, 999] = 1.0
    logits[2] = torch.randn(V, generator=torch.Generator().manual_seed(1))
    z = torch.zeros(3)
    tok, lp = ops.sample(logits.to(DEV), z.to(DEV), torch.zeros(3, dtype=torch.int32, device=DEV), torch.ones(3).to(DEV),
                         torch.zeros(3, dtype=torch.int64, device=DEV))
    assert tok.cpu().tolist() == [5, 999, int(logits[2].argmax())]
    tok, lp = ops.sample(logits.to(DEV), z.to(DEV), torch.zeros(3, dtype=torch.int32, device=DEV), torch.ones(3).to(DEV),
                         torch.zeros(3, dtype=torch.int64, device=DEV), any_greedy=False)  # the one-block scan agrees
    assert tok.cpu().tolist() == [5, 999, int(logits[2].argmax())]
    big = torch.randn(5, 151936, generator=torch.Generator().manual_seed(2))
    big[3, [77, 150000]] = 9.0
    tok, _ = ops.sample(big.to(DEV), torch.zeros(5).to(DEV), torch.zeros(5, dtype=torch.int32, device=DEV), torch.ones(5).to(DEV),
                        torch.zeros(5, dtype=torch.int64, device=DEV))
    assert tok.cpu().tolist() == [int(big[i].argmax()) if i != 3 else 77 for i in range(5)]
    # the maximum at the borders of the chunks that the first stage cuts a row into, with rows that are 16-byte aligned
    # (a thread reads four entries at a time) and rows that are not
    for V2 in (1000, 1001, 777, 4096, 6002):
        chunk = -(-(-(-V2 // 64)) // 4) * 4
        places = sorted({0, 1, 3, 4, chunk - 1, chunk, chunk + 1, 2 * chunk - 1, 5 * chunk, V2 - 5, V2 - 4, V2 - 1} & set(range(V2)))
        rows = torch.randn(len(places), V2, generator=torch.Generator().manual_seed(V2))
        for i, at in enumerate(places):
            rows[i, at] = 30.0
            if at + 2 < V2:
                rows[i, at + 2] = 30.0           # a tie further on loses
        n = len(places)
        tok, _ = ops.sample(rows.to(DEV), torch.zeros(n).to(DEV), torch.zeros(n, dtype=torch.int32, device=DEV), torch.ones(n).to(DEV),
                            torch.zeros(n, dtype=torch.int64, device=DEV))
        assert tok.cpu().tolist() == places, f"vocabulary of {V2}"
    # a flat distribution is covered by different seeds
    flat = torch.zeros(64, V)
    st = torch.arange(1, 65, dtype=torch.int64).to(DEV)
    tok, _ = ops.sample(flat.to(DEV), torch.ones(64).to(DEV), torch.zeros(64, dtype=torch.int32, device=DEV),
                        torch.ones(64).to(DEV), st)
    assert len(set(tok.cpu().tolist())) > 40


def test_top_logprobs():
    """Ranked by probability, ties to the smaller id, logprob = log softmax at the row's temperature
    (crates/mach-model/src/sampling.rs:405-410)."""
    ops = ops_for(torch.float32)
    V = 5000
    logits = torch.randn(4, V, generator=torch.Generator().manual_seed(3)) * 3
    logits[1, [10, 4000, 77]] = 20.0     # a three-way tie at the top: ids ascending
    logits[2] = 0.0                      # all equal: the first ids
    inv_t = torch.tensor([1.0, 0.5, 2.0, 1.25])
    tok, lp = ops.top_logprobs(logits.to(DEV), inv_t.to(DEV), 20)
    tok, lp = tok.cpu(), lp.cpu()
    assert tok.shape == (4, 20)
    assert tok[1, :3].tolist() == [10, 77, 4000] and tok[2].tolist() == list(range(20))
    ref = torch.log_softmax(logits.double() * inv_t.double()[:, None], -1)
    for r in range(4):
        order = sorted(range(V), key=lambda i: (-logits[r, i].item(), i))[:20]
        assert tok[r].tolist() == order
        assert (lp[r].double() - ref[r, order]).abs().max() < 1e-4
    tok3, _ = ops.top_logprobs(logits.to(DEV), inv_t.to(DEV), 3)
    assert tok3.shape == (4, 3) and torch.equal(tok3.cpu(), tok[:, :3])


def test_feed_tokens():
    """The rows of a step whose input the step before it sampled take it on the device: listed rows only, entries of
    row -1 (the list is filled up to a fixed length) and anything outside either buffer change nothing."""
    ops = ops_for(torch.float32)
    tokens = torch.arange(100, 120, dtype=torch.int32, device=DEV)
    sampled = torch.tensor([7, 8, 9, 10, 11], dtype=torch.int32, device=DEV)
    rows = torch.tensor([3, 0, 19, -1, -1, 25, 4, -1], dtype=torch.int32, device=DEV)
    src = torch.tensor([4, 0, 2, 1, 0, 1, 9, 0], dtype=torch.int32, device=DEV)
    ops.feed_tokens(tokens, sampled, rows, src)
    want = list(range(100, 120))
    want[3], want[0], want[19] = 11, 7, 9       # row 25 is beyond the tokens, sample 9 beyond the samples
    assert tokens.cpu().tolist() == want


def test_logit_edit():
    ops = ops_for(torch.float32)
    x = torch.zeros(2, 10, device=DEV)
    ops.logit_edit(x, torch.tensor([0, 1, 1], dtype=torch.int32, device=DEV),
                   torch.tensor([3, 0, 9], dtype=torch.int32, device=DEV), torch.tensor([1.5, -2.0, 4.0], device=DEV))
    ref = torch.zeros(2, 10)
    ref[0, 3], ref[1, 0], ref[1, 9] = 1.5, -2.0, 4.0
    assert torch.equal(x.cpu(), ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,H,KV,hd,K,ps", [(260, 3, 1, 64, 136, 16), (300, 14, 2, 64, 896, 64), (530, 4, 4, 64, 264, 32),
                                            (2048, 14, 2, 64, 896, 64), (1100, 12, 3, 64, 200, 64), (3000, 14, 2, 64, 896, 64)])
def test_qkv_product_that_rotates_and_writes_the_cache(dtype, M, H, KV, hd, K, ps):
    """The q/k/v projection of a step of many rows with bias, rotation and cache write in its epilogue: the same queries
    and the same pages as the plain product (32-bit sums) followed by the rotation kernel, and as the plain formulas
    (crates/mach-model/src/batched.rs:3566-3679); rows with a negative slot leave the pages alone; positions that are
    not the rows' indices."""
    ops = ops_for(dtype)
    assert ops.qkv_rope_takes(M, H, KV, hd, K) and not ops.qkv_rope_takes(256, H, KV, hd, K)
    assert not ops.qkv_rope_takes(M, H, KV, 80, K) and not ops.qkv_rope_takes(M, H, KV, 128, K)   # other heads: the two kernels
    N = (H + 2 * KV) * hd
    a, w, bias = rnd((M, K), dtype, 1), rnd((N, K), dtype, 2, K ** -0.5), rnd((N,), torch.float32, 3)
    gen = torch.Generator().manual_seed(4)
    positions = torch.randint(0, 5000, (M,), generator=gen, dtype=torch.int32)
    pages = -(-M // ps) + 2
    slots = torch.randperm(pages * ps, generator=gen)[:M].to(torch.int32)
    slots[5] = -1                                    # a row that writes nothing
    inv_freq = (1.0 / (10000.0 ** (torch.arange(hd // 2, dtype=torch.float32) * 2 / hd)))
    dev = lambda t: t.to(DEV)
    kp0, vp0 = rnd((pages, KV, ps, hd), dtype, 5), rnd((pages, KV, hd, ps), dtype, 6)
    # the two kernels it replaces
    kp1, vp1 = dev(kp0).clone(), dev(vp0).clone()
    sums = ops.linear(dev(a), dev(w), None, out_f32=True)
    q1 = ops.rope_kv_write(sums, dev(bias), dev(positions), dev(inv_freq), dev(slots), kp1, vp1, H, KV, hd, ps)
    # the one kernel
    kp2, vp2 = dev(kp0).clone(), dev(vp0).clone()
    table = ops.rope_table(dev(positions), dev(inv_freq))
    ang = positions.double()[:, None] * inv_freq.double()[None, :]
    assert (table[..., 0].cpu().double() - torch.cos(ang)).abs().max() < 1e-3 and (table[..., 1].cpu().double() - torch.sin(ang)).abs().max() < 1e-3
    q2 = ops.linear_qkv_rope(dev(a), dev(w), dev(bias), table, dev(slots), kp2, vp2, H, KV, hd, ps)
    assert_close(q2, q1.double(), dtype, "queries against the two kernels")
    assert_close(kp2, kp1.double(), dtype, "key pages against the two kernels")
    assert_close(vp2, vp1.double(), dtype, "value pages against the two kernels")
    # the plain formulas
    x = P.linear(a.double(), w.double(), bias.double())
    qr = P.rope(x[:, :H * hd].view(M, H, hd).float(), positions.long(), 10000.0).reshape(M, H * hd)
    assert_close(q2, qr.double(), dtype, "queries against the plain rotation")
    kr = P.rope(x[:, H * hd:(H + KV) * hd].view(M, KV, hd).float(), positions.long(), 10000.0)
    t = 17
    page, off = int(slots[t]) // ps, int(slots[t]) % ps
    assert_close(kp2[page, :, off, :], kr[t].double(), dtype, "a key in its page")
    assert_close(vp2[page, :, :, off], x[t, (H + KV) * hd:].view(KV, hd), dtype, "a value in its page")
    # what no row writes stays as it was (the row with the negative slot, and the slots nobody has)
    written = torch.zeros(pages * ps, dtype=torch.bool)
    written[slots[slots >= 0].long()] = True
    keep = (~written).view(pages, ps)
    assert torch.equal(kp2.cpu().permute(0, 2, 1, 3)[keep], kp0.permute(0, 2, 1, 3)[keep])
    assert torch.equal(vp2.cpu().permute(0, 3, 1, 2)[keep], vp0.permute(0, 3, 1, 2)[keep])
