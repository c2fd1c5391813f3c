"""The decode attention entry point that allocates nothing (``csrc/no_alloc.h``), called through ctypes
as a caller without torch's allocator would, against the existing entry point with workspaces of the
caller's: twice in a row on the same GPU, the second time with a smaller step, whose results must not
be touched by what the first call left in the scratch."""
import ctypes

import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _case(lib, nd, dtype, lens, H, KV, hd, ps, nsplit, seed):
    gen = torch.Generator().manual_seed(seed)
    S = len(lens)
    pages_of = [-(-(c + 1) // ps) for c in lens]
    n_pages = sum(pages_of) + 2
    order = torch.randperm(n_pages, generator=gen).tolist()
    width = max(pages_of)
    table = torch.full((S, width), -1, dtype=torch.int32)
    for i, n in enumerate(pages_of):
        for p in range(n):
            table[i, p] = order.pop()
    rnd = lambda *shape: (torch.randn(*shape, generator=gen) * 0.5).to(dtype).to(DEV)
    q, kp, vp = rnd(S, H * hd), rnd(n_pages, KV, ps, hd), rnd(n_pages, KV, hd, ps)
    table, pos0 = table.to(DEV), torch.tensor(lens, dtype=torch.int32, device=DEV)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    scale = ctypes.c_float(hd ** -0.5)
    # the existing entry point: the caller brings the workspaces
    want = torch.full((S, H * hd), float("nan"), dtype=dtype, device=DEV)
    part_o = torch.empty((S, H, nsplit, hd), dtype=torch.float32, device=DEV)
    part_ml = torch.empty((S, H, nsplit, 2), dtype=torch.float32, device=DEV)
    rc = getattr(lib, f"ms_decode_attention_nd{nd}")(ptr(q), ptr(kp), ptr(vp), ptr(want), ptr(part_o), ptr(part_ml), ptr(table),
                                                     width, ptr(pos0), S, H, KV, hd, ps, 0, nsplit, scale, stream)
    assert rc == 0, lib.ms_last_error().decode()
    # the new one: inputs and output only
    got = torch.full((S, H * hd), float("nan"), dtype=dtype, device=DEV)
    # what the device itself says is free (hipMemGetInfo): it sees an allocation made by the library or the runtime,
    # which torch's own counters would not
    torch.cuda.synchronize()
    before = torch.cuda.mem_get_info()[0]
    rc = getattr(lib, f"ms_decode_attention_noalloc_nd{nd}")(ptr(q), ptr(kp), ptr(vp), ptr(got), ptr(table), width, ptr(pos0),
                                                             S, H, KV, hd, ps, 0, nsplit, scale, stream)
    assert rc == 0, lib.ms_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == before, "the device's free memory changed across the call"
    assert not torch.isnan(got.float()).any()
    assert torch.equal(got, want), f"largest difference {(got.float() - want.float()).abs().max().item()}"


@pytest.mark.parametrize("dtype,elem", [(torch.bfloat16, "bf16"), (torch.float16, "f16"), (torch.float32, "f32")])
def test_decode_attention_that_allocates_nothing(dtype, elem):
    from machserve_amd.kernels import build
    hd = 64
    nd = build.attention_tile_for(hd)
    lib = ctypes.CDLL(build.ensure_library("attention", elem, nd))
    lib.ms_last_error.restype = ctypes.c_char_p
    getattr(lib, f"ms_decode_attention_noalloc_max_floats_nd{nd}").restype = ctypes.c_long
    most = getattr(lib, f"ms_decode_attention_noalloc_max_floats_nd{nd}")()
    assert most == 1 << 20
    # a step of seven requests with up to 2,049 keys, sixteen splits; then a smaller one (three requests, four
    # splits) that reuses the head of the same scratch
    _case(lib, nd, dtype, [0, 1, 63, 64, 130, 700, 2049], 14, 2, hd, 64, 16, seed=1)
    _case(lib, nd, dtype, [5, 300, 77], 14, 2, hd, 64, 4, seed=2)
    _case(lib, nd, dtype, [9], 4, 4, hd, 16, 1, seed=3)   # no splits: the scratch is not used
    # beyond the scratch: refused with the sizes, and nothing is launched
    S, H, nsplit = 64, 64, 64
    assert S * H * nsplit * (hd + 2) > most
    z = ctypes.c_void_p(0)
    rc = getattr(lib, f"ms_decode_attention_noalloc_nd{nd}")(z, z, z, z, z, 1, z, S, H, 8, hd, 64, 0, nsplit, ctypes.c_float(0.125), z)
    assert rc != 0 and "exceed the scratch" in lib.ms_last_error().decode()
