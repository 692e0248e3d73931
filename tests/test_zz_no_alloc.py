"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes: decode attention
with the keys shared out over workgroups, the partial results in the library's own static buffer
instead of a workspace argument.  Its output must equal, bit for bit, what the entry point with a
workspace gives (the kernels are the same), on two calls in a row, the second with a smaller input;
and a size beyond the buffer is refused."""
import ctypes
import math

import pytest
import torch

pytestmark = [pytest.mark.gpu, pytest.mark.needs_device]
DEV = "cuda:0"

_VP, _I, _F, _L = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_long
COMMON = [_VP, _I, _VP, _VP, _I, _VP, _I, _I, _I, _I, _I, _F, _I, _VP, _I, _I]      # q .. n_splits


def library():
    from deliverance_amd.kernels import build
    lib = build.load()
    lib.da_attn_decode_split.argtypes = COMMON + [_VP, _L, _VP]
    lib.da_attn_decode_split_static.argtypes = COMMON + [_VP]
    lib.da_attn_decode_split_bytes.argtypes = [_I, _I, _I, _I]
    lib.da_attn_decode_split_bytes.restype = _L
    for f in (lib.da_attn_decode_split, lib.da_attn_decode_split_static):
        f.restype = _I
    return lib


def case(S, Hq, Hkv, D, page, max_len, seed):
    """Sequences of random lengths with random keys and values in pages that lie anywhere in the pool."""
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(1, max_len + 1, (S,), generator=g)
    lens[0] = max_len
    max_blocks = -(-max_len // page)
    n_pages = S * max_blocks + 3
    perm = torch.randperm(n_pages, generator=g)
    bt = torch.full((S, max_blocks), -1, dtype=torch.int32)
    k = 0
    for s in range(S):
        for j in range(-(-int(lens[s]) // page)):
            bt[s, j] = perm[k]; k += 1
    cache = (torch.randn(n_pages, 2, Hkv, page, D, generator=g)).to(torch.bfloat16)
    q = torch.randn(S, Hq * D, generator=g).to(torch.bfloat16)
    return q.to(DEV), cache.to(DEV), bt.to(DEV), lens.to(torch.int32).to(DEV), max_blocks


def run_both(lib, S, Hq, Hkv, D, page, max_len, n_splits, seed):
    q, cache, bt, lens, max_blocks = case(S, Hq, Hkv, D, page, max_len, seed)
    stream = torch.cuda.current_stream().cuda_stream
    scale = 1.0 / math.sqrt(D)
    args = [q.data_ptr(), q.stride(0), cache.data_ptr(), bt.data_ptr(), max_blocks, lens.data_ptr(), S, Hq, Hkv, D, page,
            scale, 0]
    nbytes = lib.da_attn_decode_split_bytes(S, Hq, D, n_splits)
    ws = torch.full((nbytes // 4,), float("nan"), device=DEV)
    want = torch.full((S, Hq * D), float("nan"), dtype=torch.bfloat16, device=DEV)
    rc = lib.da_attn_decode_split(*args, want.data_ptr(), want.stride(0), n_splits, ws.data_ptr(), nbytes, stream)
    assert rc == 0, lib.da_last_error().decode()
    got = torch.full_like(want, float("nan"))
    torch.cuda.synchronize()
    # free device memory as the runtime itself reports it (torch's own counters would not see an
    # allocation made inside the library)
    before = torch.cuda.mem_get_info()[0]
    rc = lib.da_attn_decode_split_static(*args, got.data_ptr(), got.stride(0), n_splits, stream)
    assert rc == 0, lib.da_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= before, "the entry point took device memory"
    assert torch.isfinite(want.float()).all()
    assert torch.equal(got, want), f"S={S} Hq={Hq} D={D} splits={n_splits}: {(got.float() - want.float()).abs().max()}"
    return got


def test_the_static_scratch_entry_point_gives_what_the_workspace_one_gives():
    lib = library()
    # two calls in a row on one stream; the second is smaller and finds the first one's partial results in the buffer
    a = run_both(lib, S=5, Hq=4, Hkv=2, D=64, page=16, max_len=3000, n_splits=6, seed=1)
    b = run_both(lib, S=2, Hq=2, Hkv=2, D=32, page=32, max_len=1300, n_splits=2, seed=2)
    assert a.shape == (5, 256) and b.shape == (2, 64)
    # and a larger one again, other head size and page
    run_both(lib, S=3, Hq=6, Hkv=3, D=128, page=64, max_len=2100, n_splits=3, seed=3)


def test_the_static_scratch_entry_point_refuses_what_its_buffer_cannot_hold():
    lib = library()
    S, Hq, D, n_splits = 64, 32, 256, 8                       # 64 * 32 * 8 * 258 * 4 bytes = 16.9 MB > 8 MiB
    assert lib.da_attn_decode_split_bytes(S, Hq, D, n_splits) > (8 << 20)
    q = torch.zeros(S, Hq * D, dtype=torch.bfloat16, device=DEV)
    cache = torch.zeros(4, 2, Hq, 16, D, dtype=torch.bfloat16, device=DEV)
    bt = torch.zeros(S, 200, dtype=torch.int32, device=DEV)
    lens = torch.ones(S, dtype=torch.int32, device=DEV)
    out = torch.zeros_like(q)
    rc = lib.da_attn_decode_split_static(q.data_ptr(), q.stride(0), cache.data_ptr(), bt.data_ptr(), 200, lens.data_ptr(),
                                         S, Hq, Hq, D, 16, 0.1, 0, out.data_ptr(), out.stride(0), n_splits,
                                         torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and "bytes of scratch" in lib.da_last_error().decode()
    rc = lib.da_attn_decode_split_static(q.data_ptr(), q.stride(0), cache.data_ptr(), bt.data_ptr(), 200, lens.data_ptr(),
                                         S, Hq, Hq, D, 16, 0.1, 0, out.data_ptr(), out.stride(0), 1,
                                         torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and "shares" in lib.da_last_error().decode()
