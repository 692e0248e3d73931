"""Each kernel alone against a plain reference, at other sizes than the engine's tiny models
use: sizes that are no power of two, head sizes in steps of 16, grouped heads, windows, pages
scattered over the pool, and a pool that is NaN wherever nothing was written."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import helpers
import plain_gpt2 as P

pytestmark = pytest.mark.gpu
DEV = helpers.DEVICE


@pytest.fixture(scope="module")
def ops():
    from deliverance_amd.kernels import ops as o
    return o


def bf(x):
    return x.to(torch.bfloat16)


# ----------------------------------------------------------------------------- embedding, norm
@pytest.mark.simt_quick
@pytest.mark.parametrize("table_dtype", [torch.float32, torch.bfloat16])
def test_embed(ops, table_dtype):
    g = torch.Generator().manual_seed(0)
    V, Pn, E, N = 1000, 77, 200, 37
    wte = torch.randn(V, E, generator=g).to(table_dtype).to(DEV)
    wpe = torch.randn(Pn, E, generator=g).to(table_dtype).to(DEV)
    tok = torch.randint(0, V, (N,), generator=g, dtype=torch.int32).to(DEV)
    pos = torch.randint(0, Pn, (N,), generator=g, dtype=torch.int32).to(DEV)
    out = torch.empty(N, E, device=DEV)
    ops.embed(tok, pos, wte, wpe, out)
    want = wte.float()[tok.long()] + wpe.float()[pos.long()]
    assert torch.equal(out, want)
    ops.embed(tok, pos, wte, None, out)
    assert torch.equal(out, wte.float()[tok.long()])


@pytest.mark.simt_quick
def test_embed_scale_and_row_copies(ops):
    g = torch.Generator().manual_seed(2)
    V, Pn, E, N = 300, 50, 72, 21
    wte, wpe = bf(torch.randn(V, E, generator=g)).to(DEV), bf(torch.randn(Pn, E, generator=g)).to(DEV)
    tok = torch.randint(0, V, (N,), generator=g, dtype=torch.int32).to(DEV)
    pos = torch.randint(0, Pn, (N,), generator=g, dtype=torch.int32).to(DEV)
    out = torch.empty(N, E, device=DEV)
    ops.embed(tok, pos, wte, wpe, out, scale=8.5)
    assert torch.equal(out, wte.float()[tok.long()] * 8.5 + wpe.float()[pos.long()])
    # rows gathered and converted; rows added into the 32-bit stream
    rows = torch.tensor([20, 0, 7, 7, 3], dtype=torch.int32, device=DEV)
    for dt in (torch.float32, torch.bfloat16):
        dst = torch.empty(5, E, device=DEV, dtype=dt)
        ops.copy_rows(out, dst, rows=rows)
        assert torch.equal(dst, out[rows.long()].to(dt))
        dst = torch.empty(N, E, device=DEV, dtype=dt)
        ops.copy_rows(out, dst)
        assert torch.equal(dst, out.to(dt))
    acc = torch.randn(N, E, generator=g).to(DEV)
    want = acc + bf(out).float()
    ops.copy_rows(bf(out), acc, accumulate=True)
    assert torch.equal(acc, want)
    with pytest.raises(ops.KernelError, match="float32 destination"):
        ops.copy_rows(out, bf(out), accumulate=True)


@pytest.mark.simt_quick
@pytest.mark.parametrize("E,eps", [(7, 1e-5), (200, 1e-6), (1600, 1e-5), (64, 1e-1)])
def test_layernorm(ops, E, eps):
    g = torch.Generator().manual_seed(1)
    N = 19
    x = (torch.randn(N, E, generator=g) * 3 + 5).to(DEV)       # a large mean: E[x^2]-mean^2 would lose digits
    w, b = torch.randn(E, generator=g).to(DEV), torch.randn(E, generator=g).to(DEV)
    out = torch.empty(N, E, device=DEV)
    ops.layernorm(x, w, b, eps, out)
    want = F.layer_norm(x.double(), (E,), w.double(), b.double(), eps)
    assert (out.double() - want).abs().max() < 2e-5
    # bfloat16 parameters and output, gathered rows
    rows = torch.tensor([5, 0, 18, 5], dtype=torch.int32, device=DEV)
    o2 = torch.empty(4, E, device=DEV, dtype=torch.bfloat16)
    ops.layernorm(x, bf(w), bf(b), eps, o2, rows)
    want2 = F.layer_norm(x.double(), (E,), bf(w).double(), bf(b).double(), eps)[rows.long()]
    assert (o2.double() - want2).abs().max() < 4e-2
    assert torch.equal(o2[0], o2[3])
    if E == 7:   # the reference's own vector (LayerNormTest.java:40,51,77,88)
        xv = torch.tensor([[-1.1151, 0.1490, -1.0923, -1.4551, 1.3358, 0.3075, 0.6278]], device=DEV)
        o3 = torch.empty(1, 7, device=DEV)
        ops.layernorm(xv, torch.ones(7, device=DEV), torch.zeros(7, device=DEV), 1e-5, o3)
        want3 = torch.tensor([-0.9635, 0.3355, -0.9401, -1.3129, 1.5551, 0.4984, 0.8275], device=DEV)
        assert (o3[0] - want3).abs().max() < 1e-4


# ----------------------------------------------------------------------------- products
def _gemm_case(ops, fn, M, N, K, dtype, act, accumulate, bias, out_dtype, g):
    a = (torch.randn(M, K, generator=g) * 0.5).to(dtype).to(DEV)
    w = (torch.randn(N, K, generator=g) * 0.2).to(dtype).to(DEV)
    b = torch.randn(N, generator=g).to(dtype).to(DEV) if bias else None
    base = torch.randn(M, N, generator=g).to(DEV)
    out = base.clone() if accumulate else torch.empty(M, N, device=DEV, dtype=out_dtype)
    fn(a, w, b, out, act, accumulate)
    ref = a.double() @ w.double().t()
    if bias:
        ref = ref + b.double()
    if act == "gelu_new":
        ref = F.gelu(ref, approximate="tanh")
    elif act == "gelu":
        ref = F.gelu(ref)
    elif act == "relu":
        ref = F.relu(ref)
    elif act == "silu":
        ref = F.silu(ref)
    if accumulate:
        ref = ref + base.double()
    return out.double(), ref


@pytest.mark.simt_quick
@pytest.mark.parametrize("M,N,K", [(1, 50, 24), (5, 1000, 96), (70, 200, 96), (130, 77, 200), (64, 64, 64)])
def test_gemm_plain_32bit(ops, M, N, K):
    g = torch.Generator().manual_seed(M * 1000 + N)
    for act, acc, bias in ((None, False, True), ("gelu_new", False, True), ("gelu", False, False),
                           (None, True, True), ("silu", False, True), ("relu", False, True)):
        out, ref = _gemm_case(ops, ops.linear_ref, M, N, K, torch.float32, act, acc, bias, torch.float32, g)
        assert (out - ref).abs().max() < 2e-5 * max(1.0, ref.abs().max().item())


@pytest.mark.parametrize("M", [1, helpers.quick(3, mark="simt_a"), 5, 8, 12, 16, helpers.quick(17, mark="simt_a"), 40, 64,
                               helpers.quick(65, mark="simt_a"), 128, helpers.quick(200, mark="simt_a"), 513, 1100, 2048])
@pytest.mark.parametrize("N,K", [helpers.quick(96, 200, mark="simt_b"), helpers.quick(1000, 96, mark="simt_b"), (2304, 768),
                                 helpers.quick(50, 24, mark="simt_b"), helpers.quick(300, 2056, mark="simt_b"), (1030, 1160),
                                 (4200, 200), helpers.quick(4096, 8, mark="simt_b")])
def test_gemm_matrix_cores(ops, M, N, K):
    """Every kernel form behind ``linear_mfma`` (up to 4 rows and 2,048 columns: 4x4x4 products, 4 to 16
    wavefronts; up to 64 rows: 16x16x32 products fed through LDS, 1 to 4 row tiles, 8 or 12 wavefronts;
    else block tiles of 64x64, 128x64 and 128x128, chosen by the number of tiles: 1,100 and 2,048 rows
    reach the larger ones), each with a last step that K cuts or a K below one slab."""
    helpers.skip_in_simulation_if(M * N * K > 1.2e8)
    g = torch.Generator().manual_seed(M * 7 + N)
    for act, acc, bias, od in ((None, False, True, torch.bfloat16), ("gelu_new", False, True, torch.bfloat16),
                               (None, True, True, torch.float32), (None, False, False, torch.float32),
                               ("gelu", False, True, torch.bfloat16)):
        out, ref = _gemm_case(ops, ops.linear_mfma, M, N, K, torch.bfloat16, act, acc, bias, od, g)
        tol = (1e-2 if od == torch.bfloat16 else 1e-4) * max(1.0, ref.abs().max().item())
        assert (out - ref).abs().max() < tol, (act, acc, bias, od)


@pytest.mark.parametrize("M,N,K", [(1600, 2000, 200), (1555, 1999, 320), (2048, 1600, 1600), (1536, 2304, 768), (2048, 2304, 768),
                                   (4096, 768, 3072), (2500, 1600, 2112), (2048, 1600, 6400)])
def test_gemm_tiles_alone_on_their_compute_units(ops, M, N, K):
    """The library's own choice where 128 x 128 tiles would be 140 to 512: a K that a slab cuts and a long K with
    192 to 256 tiles (operands through registers, four slabs in flight: GPT-2 1.5B's proj), whole slabs (operands
    straight into LDS: 128 x 128 tiles for 208 and 216 tiles, GPT-2 1.5B's out-proj among them, and for 260
    tiles with a K above 2,048; 256 x 128 for 288 tiles, GPT-2 124M's q|k|v; 128 x 128 for 192 tiles and a K of 3,072)."""
    helpers.skip_in_simulation_if(True)
    g = torch.Generator().manual_seed(M + N + K)
    for act, acc, bias, od in ((None, False, True, torch.bfloat16), ("gelu_new", False, True, torch.bfloat16),
                               (None, True, True, torch.float32), (None, False, False, torch.float32)):
        out, ref = _gemm_case(ops, ops.linear_mfma, M, N, K, torch.bfloat16, act, acc, bias, od, g)
        tol = (1e-2 if od == torch.bfloat16 else 1e-4) * max(1.0, ref.abs().max().item())
        assert (out - ref).abs().max() < tol, (act, acc, bias, od)


@pytest.mark.parametrize("form", ["wide", "wide_256x128", "wide_128x128"])
@pytest.mark.parametrize("M,N,K", [helpers.quick(300, 200, 128), (257, 520, 64), (2048, 1600, 320), (700, 4800, 192)])
def test_gemm_wide_tiles(ops, M, N, K, form):
    """The tiles whose operands go from memory straight into LDS (two stages of a, three of w), in their
    three shapes (256 x 256, 256 x 128, 128 x 128): every epilogue against 64-bit arithmetic, and bit for
    bit what the other tile forms give (all sum over k in ascending steps of 16); edges in M and N, one to
    five slabs."""
    g = torch.Generator().manual_seed(M + N + K)
    wide = lambda *a_, **k_: ops.linear_mfma(*a_, form=form, **k_)
    for act, acc, bias, od in ((None, False, True, torch.bfloat16), ("gelu_new", False, True, torch.bfloat16),
                               ("gelu", False, False, torch.bfloat16), (None, True, True, torch.float32),
                               (None, False, False, torch.float32), ("silu", False, True, torch.bfloat16)):
        out, ref = _gemm_case(ops, wide, M, N, K, torch.bfloat16, act, acc, bias, od, g)
        tol = (1e-2 if od == torch.bfloat16 else 1e-4) * max(1.0, ref.abs().max().item())
        assert (out - ref).abs().max() < tol, (act, acc, bias, od)
    a = bf(torch.randn(M, K, generator=g) * 0.5).to(DEV)
    w = bf(torch.randn(N, K, generator=g) * 0.2).to(DEV)
    b = bf(torch.randn(N, generator=g)).to(DEV)
    for od, acc in ((torch.bfloat16, False), (torch.float32, True)):
        o1 = torch.full((M, N), 0.25, device=DEV, dtype=od)
        o2 = o1.clone()
        ops.linear_mfma(a, w, b, o1, None, acc, form=form)
        ops.linear_mfma(a, w, b, o2, None, acc)
        assert torch.equal(o1, o2), (od, acc)
    with pytest.raises(ops.KernelError, match="multiple of 64"):
        ops.linear_mfma(a[:, :K - 8].contiguous(), w[:, :K - 8].contiguous(), b, o1, form=form)


@pytest.mark.parametrize("form", ["wide", "wide_256x128", "wide_128x128"])
@pytest.mark.parametrize("M", [helpers.quick(300), 1000])
def test_gemm_wide_tiles_write_keys_and_values(ops, M, form):
    g = torch.Generator().manual_seed(M)
    Hq, Hkv, D, page, K = 5, 3, 48, 16, 128
    N = (Hq + 2 * Hkv) * D
    n_pages = (M + page - 1) // page + 2
    a = bf(torch.randn(M, K, generator=g)).to(DEV)
    w = bf(torch.randn(N, K, generator=g) * 0.1).to(DEV)
    bias = bf(torch.randn(N, generator=g)).to(DEV)
    perm = torch.randperm(n_pages * page, generator=g)[:M].to(torch.int32)
    perm[M // 2] = -1
    runs = torch.cat([torch.arange(16, 16 + M // 2), torch.arange(16 + M // 2 + 19, 16 + M // 2 + 19 + M - M // 2)]).to(torch.int32)
    runs[M // 4] = -1
    for order in (perm, runs):
        slots = order.to(DEV)
        c1 = torch.zeros(n_pages + 2, 2, Hkv, page, D, dtype=torch.bfloat16, device=DEV)
        c2 = torch.zeros_like(c1)
        out1 = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
        out2 = torch.empty_like(out1)
        ops.linear_mfma(a, w, bias, out1, kv_cache=c1, slot_map=slots, q_cols=Hq * D, form=form)
        ops.linear_mfma(a, w, bias, out2)
        ops.kv_write(out2, Hq * D, (Hq + Hkv) * D, c2, slots, Hkv, D)
        assert torch.equal(out1, out2)
        assert torch.equal(c1, c2) and c1.abs().sum() > 0


@pytest.mark.simt_quick
@pytest.mark.parametrize("M", [20, 200])
def test_gemm_into_rows_longer_than_the_result(ops, M):
    """The output's rows are longer than N (a view of a wider matrix): the tile kernel stores whole
    16-byte pieces up to the last one that N cuts, which goes out entry by entry; what lies behind
    column N is not touched, with a store, a 32-bit store and +=."""
    g = torch.Generator().manual_seed(M)
    N, K, LD = 1030, 96, 1040
    a = bf(torch.randn(M, K, generator=g) * 0.5).to(DEV)
    w = bf(torch.randn(N, K, generator=g) * 0.2).to(DEV)
    b = bf(torch.randn(N, generator=g)).to(DEV)
    ref = a.double() @ w.double().t() + b.double()
    for od, acc in ((torch.bfloat16, False), (torch.float32, False), (torch.float32, True)):
        big = torch.full((M, LD), 7.0, device=DEV, dtype=od)
        out = big[:, :N]
        ops.linear_mfma(a, w, b, out, None, acc)
        want = ref + (7.0 if acc else 0.0)
        tol = (1e-2 if od == torch.bfloat16 else 1e-4) * max(1.0, want.abs().max().item())
        assert (out.double() - want).abs().max() < tol, (od, acc)
        assert torch.equal(big[:, N:], torch.full((M, LD - N), 7.0, device=DEV, dtype=od)), (od, acc)


@pytest.mark.simt_quick
def test_gemm_rows_do_not_depend_on_the_batch(ops):
    """A row's result is the same, bit for bit, whatever other rows share the call, as long as the call
    takes the same kernel form (block tiles; 16x16x32 products up to 64 rows; 4x4x4 products up to 4
    rows and 2,048 columns); between forms it differs by the rounding of 32-bit sums at most."""
    g = torch.Generator().manual_seed(3)
    K, N = 768, 300
    a = bf(torch.randn(200, K, generator=g)).to(DEV)
    w = bf(torch.randn(N, K, generator=g) * 0.1).to(DEV)

    def rows(lo, hi, dtype=torch.bfloat16):
        out = torch.empty(hi - lo, N, device=DEV, dtype=dtype)
        ops.linear_mfma(a[lo:hi].contiguous(), w, None, out)
        return out

    full = rows(0, 200)
    assert torch.equal(rows(60, 150), full[60:150])                 # block tiles
    small = rows(0, 64)
    assert torch.equal(rows(3, 23)[7], small[10])                   # 16x16x32: 20 rows, 64 rows
    assert torch.equal(rows(4, 12)[6], small[10])                   # ... 8 rows
    assert torch.equal(rows(10, 11)[0], rows(8, 12)[2])             # 4x4x4: 1 row, 4 rows
    assert torch.equal(rows(10, 13)[0], rows(10, 11)[0])            # ... 3 rows
    exact = a[10].double() @ w.double().t()
    scale = exact.abs().max().item()
    forms = [rows(10, 11, torch.float32)[0], rows(0, 64, torch.float32)[10], rows(0, 200, torch.float32)[10]]
    for f in forms:
        assert (f.double() - exact).abs().max() < 2e-6 * scale


@pytest.mark.simt_quick
def test_gemm_refuses_what_it_cannot_take(ops):
    a = torch.zeros(4, 12, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(8, 12, device=DEV, dtype=torch.bfloat16)
    out = torch.zeros(4, 8, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(ops.KernelError, match="multiples of 8"):
        ops.linear_mfma(a, w, None, out)
    ops.linear(a, w, None, out)                     # the dispatcher sends it to the plain kernel
    with pytest.raises(ops.KernelError):
        ops.linear_ref(a, w, None, torch.zeros(4, 9, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(ops.KernelError, match="float32 output"):
        ops.linear_ref(a, w, None, out, None, True)


# ----------------------------------------------------------------------------- paged attention
class PagedCase:
    """Sequences with their keys and values scattered over a NaN-filled pool."""

    def __init__(self, lens, new, Hq, Hkv, D, page, dtype, seed, scale_boost=None):
        g = torch.Generator().manual_seed(seed)
        self.lens, self.new, self.Hq, self.Hkv, self.D, self.page = lens, new, Hq, Hkv, D, page
        S = len(lens)
        n_pages = sum(-(-n // page) for n in lens) + 5
        perm = torch.randperm(n_pages, generator=g).tolist()
        self.cache = torch.full((n_pages, 2, Hkv, page, D), float("nan"), dtype=dtype, device=DEV)
        max_blocks = max(-(-n // page) for n in lens)
        bt = torch.full((S, max_blocks), -1, dtype=torch.int32)
        self.k, self.v, self.q = [], [], []
        for s, n in enumerate(lens):
            k = torch.randn(n, Hkv * D, generator=g).to(dtype)
            v = torch.randn(n, Hkv * D, generator=g).to(dtype)
            q = torch.randn(new[s], Hq * D, generator=g).to(dtype)
            if scale_boost is not None:      # one far key stands out for the last query
                far, boost = scale_boost
                q[-1] *= boost
                qv = q[-1].float().view(Hq, D)[:: Hq // Hkv]
                k[far] = (qv / qv.norm(dim=1, keepdim=True) * 8.0).reshape(-1).to(dtype)
            self.k.append(k); self.v.append(v); self.q.append(q)
            for j in range(-(-n // page)):
                bt[s, j] = perm.pop()
        self.bt = bt.to(DEV)
        # fill through the engine's own write kernel
        from deliverance_amd.kernels import ops as o
        for s, n in enumerate(lens):
            qkv = torch.cat([torch.zeros(n, Hq * D, dtype=dtype), self.k[s], self.v[s]], dim=1).to(DEV)
            slots = torch.tensor([int(bt[s, pos // page]) * page + pos % page for pos in range(n)], dtype=torch.int32, device=DEV)
            o.kv_write(qkv, Hq * D, Hq * D + Hkv * D, self.cache, slots, Hkv, D)
        self.qcat = torch.cat(self.q).to(DEV)
        starts = np.cumsum([0] + list(new))
        self.q_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
        self.seq_lens = torch.tensor(lens, dtype=torch.int32, device=DEV)
        self.seq_of = torch.tensor([s for s, n in enumerate(new) for _ in range(n)], dtype=torch.int32, device=DEV)
        self.pos = torch.tensor([lens[s] - new[s] + i for s in range(S) for i in range(new[s])], dtype=torch.int32, device=DEV)

    def plain(self, scale, window):
        outs = []
        for s in range(len(self.lens)):
            o = P.causal_attention(self.q[s].double().numpy(), self.k[s].double().numpy(), self.v[s].double().numpy(),
                                   self.Hq, scale, window=window, n_kv_head=self.Hkv, past=self.lens[s] - self.new[s])
            outs.append(o)
        return np.concatenate(outs)


ATT_TOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,D,page,window", [helpers.quick(4, 4, 16, 16, None), (6, 2, 48, 16, None), helpers.quick(2, 1, 80, 32, 37),
                                                  (3, 3, 128, 64, None), (5, 5, 64, 16, 100)])
def test_attention_plain_kernel(ops, dtype, Hq, Hkv, D, page, window):
    case = PagedCase(lens=[70, 5, 131, 64], new=[70, 1, 9, 2], Hq=Hq, Hkv=Hkv, D=D, page=page, dtype=dtype, seed=D)
    out = torch.empty_like(case.qcat)
    scale = 0.7 / math.sqrt(D)
    ops.attention_ref(case.qcat, case.cache, case.bt, case.seq_of, case.pos, Hq, scale, window, out)
    assert np.abs(out.double().cpu().numpy() - case.plain(scale, window)).max() < ATT_TOL[dtype]


@pytest.mark.parametrize("Hq,Hkv,D,page,window", [helpers.quick(4, 4, 16, 16, None), (6, 2, 48, 16, None), helpers.quick(2, 1, 80, 32, 37),
                                                  (3, 3, 128, 64, None), (12, 12, 64, 16, None), (5, 5, 64, 16, 100),
                                                  helpers.quick(2, 2, 256, 16, None), (25, 25, 64, 32, 70)])
def test_attention_decode_kernel(ops, Hq, Hkv, D, page, window):
    lens = [1, 2, 63, 64, 65, 300, 129, 17, 1000]
    case = PagedCase(lens=lens, new=[1] * len(lens), Hq=Hq, Hkv=Hkv, D=D, page=page, dtype=torch.bfloat16, seed=D + 1)
    out = torch.empty_like(case.qcat)
    scale = 0.7 / math.sqrt(D)
    ops.attention_decode(case.qcat, case.cache, case.bt, case.seq_lens, len(lens), Hq, scale, window, out)
    got = out.double().cpu().numpy()
    assert np.isfinite(got).all()
    assert np.abs(got - case.plain(scale, window)).max() < ATT_TOL[torch.bfloat16]


@pytest.mark.parametrize("n_splits", [2, helpers.quick(3, mark="simt_a"), 7, 16])
@pytest.mark.parametrize("Hq,Hkv,D,page,window", [helpers.quick(2, 2, 64, 16, None, mark="simt_b"), (4, 2, 48, 32, None),
                                                  helpers.quick(1, 1, 128, 64, 700, mark="simt_b"), (3, 3, 16, 16, 90)])
def test_attention_decode_with_keys_split_over_workgroups(ops, Hq, Hkv, D, page, window, n_splits):
    """Every (sequence, head) pair's keys in ``n_splits`` shares with a merge in a fixed order: shares
    that hold nothing (short sequences, a window that has passed them), one key, a share's first and
    last key, sequences that end at a share's edge."""
    width = 2100                                                   # keys the block table spans
    span = -(-(-(-width // page) * page) // n_splits // 64) * 64    # what the kernel gives a share
    lens = [1, 2, 63, span, span + 1, 2 * span - 1 if 2 * span - 1 <= width else width, 1030, width, 700]
    case = PagedCase(lens=lens, new=[1] * len(lens), Hq=Hq, Hkv=Hkv, D=D, page=page, dtype=torch.bfloat16, seed=D + n_splits)
    assert case.bt.shape[1] == -(-width // page)
    scale = 0.7 / math.sqrt(D)
    out = torch.full_like(case.qcat, float("nan"))
    ws = torch.full((ops.decode_workspace_floats(len(lens), Hq, D, n_splits),), float("nan"), device=DEV)
    ops.attention_decode(case.qcat, case.cache, case.bt, case.seq_lens, len(lens), Hq, scale, window, out, n_splits, ws)
    got = out.double().cpu().numpy()
    assert np.isfinite(got).all()
    assert np.abs(got - case.plain(scale, window)).max() < ATT_TOL[torch.bfloat16]
    one = torch.empty_like(case.qcat)
    ops.attention_decode(case.qcat, case.cache, case.bt, case.seq_lens, len(lens), Hq, scale, window, one)
    assert (out.float() - one.float()).abs().max() < 2e-2          # the two kernels differ by rounding only
    with pytest.raises(ops.KernelError, match="workspace"):
        ops.attention_decode(case.qcat, case.cache, case.bt, case.seq_lens, len(lens), Hq, scale, window, out, n_splits, ws[:10])


@pytest.mark.parametrize("where", ["first", "share_end", helpers.quick("share_start"), "second_share_end", "last", "window_edge"])
@pytest.mark.parametrize("D,page,window,n_splits", [helpers.quick(64, 16, None, 3), (144, 32, None, 2), (64, 16, 700, 4), (32, 64, 1500, 16)])
def test_attention_decode_split_sees_one_far_key(ops, D, page, window, n_splits, where):
    """One key among 2,100 carries nearly all the weight of the last query: a share's first or last key,
    the sequence's first or last, or the oldest key that the window still holds.  Random keys alone give
    near-uniform weights, under which a lost key moves the result by a thousandth."""
    n = 2100
    span = -(-(-(-n // page) * page) // n_splits // 64) * 64
    far = {"first": 0, "share_end": span - 1, "share_start": span, "second_share_end": min(2 * span, n) - 1, "last": n - 1,
           "window_edge": n - (window or n)}[where]
    Hq, Hkv = 2, 1
    case = PagedCase(lens=[n], new=[1], Hq=Hq, Hkv=Hkv, D=D, page=page, dtype=torch.bfloat16, seed=D + far, scale_boost=(far, 3.0))
    scale = 0.7 / math.sqrt(D)
    want = case.plain(scale, window)
    seen = window is None or far >= n - window
    if seen:      # the far key's value is the answer, nearly
        assert np.abs(want[0, :D] - case.v[0][far].double().numpy()[:D]).max() < 0.1
    out = torch.full_like(case.qcat, float("nan"))
    ws = torch.full((ops.decode_workspace_floats(1, Hq, D, n_splits),), float("nan"), device=DEV)
    ops.attention_decode(case.qcat, case.cache, case.bt, case.seq_lens, 1, Hq, scale, window, out, n_splits, ws)
    assert np.abs(out.double().cpu().numpy() - want).max() < ATT_TOL[torch.bfloat16], (where, far)


@pytest.mark.simt_quick
def test_when_decode_attention_splits_its_keys(ops):
    assert ops.decode_splits(1, 12, 64, 16) == 1                   # 1,024 keys: one share
    assert ops.decode_splits(1, 12, 256, 16) == 4                  # 4,096 keys, 12 pairs: shares of 1,024
    assert ops.decode_splits(8, 25, 256, 16) == 2                  # 200 pairs: two shares fill the chip
    assert ops.decode_splits(64, 12, 256, 16) == 1                 # 768 pairs fill it alone
    assert ops.decode_splits(1, 1, 4096, 16) == 32                 # never more than 32


@pytest.mark.parametrize("Hq,Hkv,D,page,window", [(4, 4, 16, 16, None), helpers.quick(6, 2, 48, 16, None), helpers.quick(2, 1, 80, 32, 37),
                                                  (3, 3, 128, 64, None), (12, 12, 64, 16, None), (5, 5, 64, 16, 100),
                                                  (2, 2, 256, 16, None), (2, 2, 240, 16, None), helpers.quick(3, 1, 64, 32, 200)])
def test_attention_prefill_kernel(ops, Hq, Hkv, D, page, window):
    lens = [70, 200, 131, 64, 2, 300, 513]
    new = [70, 9, 131, 2, 2, 129, 260]            # whole prompts, short portions after a long past, tiles' edges
    case = PagedCase(lens=lens, new=new, Hq=Hq, Hkv=Hkv, D=D, page=page, dtype=torch.bfloat16, seed=D + 2)
    scale = 0.7 / math.sqrt(D)
    want = case.plain(scale, window)
    # a workgroup's form, row blocks x wavefronts that share out a row block's keys; 0: the kernel's own choice
    for form in [0, 41] + ([22] if D <= 128 else []) + ([42, 14] if D <= 64 else []):
        out = torch.full_like(case.qcat, float("nan"))
        ops.attention_prefill(case.qcat, case.cache, case.bt, case.q_start, case.seq_lens, 0, len(lens), max(new), Hq,
                              scale, window, out, form=form)
        got = out.double().cpu().numpy()
        assert np.isfinite(got).all(), form
        assert np.abs(got - want).max() < ATT_TOL[torch.bfloat16], form
    if D > 64:
        with pytest.raises(ops.KernelError, match="form 14"):
            ops.attention_prefill(case.qcat, case.cache, case.bt, case.q_start, case.seq_lens, 0, len(lens), max(new), Hq,
                                  scale, window, out, form=14)


@pytest.mark.simt_quick
@pytest.mark.parametrize("form", [41, 42, 22, 14])
def test_attention_prefill_finds_a_far_key_in_every_phase(ops, form):
    """One key among 700 is made to stand out for one query row (key and query scaled up along one
    direction): the row's output is then that key's value, whichever wavefront's share the key lies in
    (with 2 or 4 wavefronts to a row block a share is every 2nd or 4th tile of 64 keys) and wherever
    in its tile."""
    Hq, Hkv, D, page, n = 2, 2, 64, 16, 700
    case = PagedCase(lens=[n], new=[n], Hq=Hq, Hkv=Hkv, D=D, page=page, dtype=torch.bfloat16, seed=31)
    scale = 1.0 / math.sqrt(D)
    row = n - 1
    for far in (0, 63, 64, 129, 200, 300, 447, 640, 699):
        q = case.qcat.clone()
        cache = case.cache.clone()
        pg, r = int(case.bt[0, far // page]), far % page
        direction = torch.zeros(D); direction[far % D] = 30.0
        for h in range(Hq):
            q[row, h * D:(h + 1) * D] = direction.to(torch.bfloat16)
            cache[pg, 0, h, r, :] = direction.to(torch.bfloat16)
        out = torch.empty_like(q)
        ops.attention_prefill(q, cache, case.bt, case.q_start, case.seq_lens, 0, 1, n, Hq, scale, None, out, form=form)
        for h in range(Hq):
            value = cache[pg, 1, h].reshape(D, page)[:, r].float()          # values lie dimension-major in a page
            assert (out[row, h * D:(h + 1) * D].float() - value).abs().max() < 2e-2, (far, h)


@pytest.mark.simt_quick
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_row_that_sees_no_key_gives_zeros(ops, dtype):
    """The padding rows of a fixed-shape decode step: length 0, a block table of -1.  Zeros, never NaN
    (NaN would spread through the row's residual into its logits and into the sampling kernel)."""
    Hq, Hkv, D, page = 4, 2, 32, 16
    case = PagedCase(lens=[20, 7], new=[1, 1], Hq=Hq, Hkv=Hkv, D=D, page=page, dtype=dtype, seed=8)
    q = torch.cat([case.qcat, torch.randn(2, Hq * D).to(dtype).to(DEV)])
    bt = torch.cat([case.bt, torch.full((2, case.bt.shape[1]), -1, dtype=torch.int32, device=DEV)])
    seq_of = torch.tensor([0, 1, 2, 3], dtype=torch.int32, device=DEV)
    pos = torch.tensor([19, 6, 0, 0], dtype=torch.int32, device=DEV)
    out = torch.full_like(q, float("nan"))
    ops.attention_ref(q, case.cache, bt, seq_of, pos, Hq, 0.2, None, out)
    want = case.plain(0.2, None)
    assert np.abs(out[:2].double().cpu().numpy() - want).max() < ATT_TOL[dtype]
    assert torch.equal(out[2:], torch.zeros_like(out[2:]))
    if dtype == torch.bfloat16:
        out2 = torch.full_like(q, float("nan"))
        lens = torch.tensor([20, 7, 0, 0], dtype=torch.int32, device=DEV)
        ops.attention_decode(q, case.cache, bt, lens, 4, Hq, 0.2, None, out2)
        assert torch.equal(out2[2:], torch.zeros_like(out2[2:]))
        assert np.abs(out2[:2].double().cpu().numpy() - want).max() < ATT_TOL[dtype]


@pytest.mark.simt_quick
def test_attention_reference_vector_shape(ops):
    """The shape of the reference's own paged-attention test: 4 query heads on 2 key heads, head 8
    there (16 here: head sizes come in steps of 16), pages of 3 rows there (16 here), 5 visible rows,
    scale 0.25, inputs by its closed formula (tensor/src/test/java/io/teknek/deliverance/tensor/
    operations/TensorOperationsDecodePagedAttentionTest.java:18-47,92-99)."""
    Hq, Hkv, D, page, rows = 4, 2, 16, 16, 5

    def tensor(r, c, seed):
        return torch.tensor([[(((i * 19 + j * 23 + seed) % 43) - 21) / 21.0 for j in range(c)] for i in range(r)])
    q = tensor(1, Hq * D, 3)
    k = torch.cat([tensor(3, Hkv * D, 7), tensor(3, Hkv * D, 11)])[:rows]
    v = torch.cat([tensor(3, Hkv * D, 13), tensor(3, Hkv * D, 17)])[:rows]
    want = P.causal_attention(q.double().numpy(), k.double().numpy(), v.double().numpy(), Hq, 0.25, n_kv_head=Hkv, past=rows - 1)
    for dtype in (torch.float32, torch.bfloat16):
        cache = torch.full((2, 2, Hkv, page, D), float("nan"), dtype=dtype, device=DEV)
        qkv = torch.cat([torch.zeros(rows, Hq * D), k, v], dim=1).to(dtype).to(DEV)
        slots = torch.tensor([16 + i for i in range(rows)], dtype=torch.int32, device=DEV)     # page 1
        ops.kv_write(qkv, Hq * D, Hq * D + Hkv * D, cache, slots, Hkv, D)
        bt = torch.tensor([[1]], dtype=torch.int32, device=DEV)
        qd = q.to(dtype).to(DEV)
        out = torch.empty_like(qd)
        ops.attention_ref(qd, cache, bt, torch.zeros(1, dtype=torch.int32, device=DEV),
                          torch.tensor([rows - 1], dtype=torch.int32, device=DEV), Hq, 0.25, None, out)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert np.abs(out.double().cpu().numpy() - want).max() < tol
        if dtype == torch.bfloat16:
            out2 = torch.empty_like(qd)
            ops.attention_decode(qd, cache, bt, torch.tensor([rows], dtype=torch.int32, device=DEV), 1, Hq, 0.25, None, out2)
            assert np.abs(out2.double().cpu().numpy() - want).max() < tol


@pytest.mark.simt_quick
@pytest.mark.parametrize("page", [16, 32, 64])
@pytest.mark.parametrize("N", [40, 600])
def test_cache_write_puts_every_key_and_value_in_its_row(ops, N, page):
    """Both write kernels (a token a workgroup; 16 tokens a workgroup from 256 tokens on) against
    direct placement: whole aligned pages in order, runs that start inside a page, single rows
    all over, and tokens whose keys are not kept (-1)."""
    Hq, Hkv, D = 3, 2, 48
    g = torch.Generator().manual_seed(N + page)
    n_pages = 4 * (N // page + 2)
    free = torch.randperm(n_pages, generator=g).tolist()
    slots = []
    while len(slots) < N:
        kind = len(slots) // 16 % 4
        pg = free.pop()
        if kind == 0:      # a whole page in order
            slots += [pg * page + i for i in range(page)]
        elif kind == 1:    # a run that starts inside the page
            slots += [pg * page + i for i in range(5, page)]
        elif kind == 2:    # rows of a page in any order
            slots += [pg * page + int(i) for i in torch.randperm(page, generator=g)[:11]]
        else:              # not kept
            slots += [-1] * 7
    slots = slots[:N]
    qkv = bf(torch.randn(N, (Hq + 2 * Hkv) * D, generator=g)).to(DEV)
    st = torch.tensor(slots, dtype=torch.int32, device=DEV)
    for dtype in (torch.bfloat16, torch.float32):
        x = qkv.to(dtype)
        cache = torch.zeros(n_pages, 2, Hkv, page, D, dtype=dtype, device=DEV)
        ops.kv_write(x, Hq * D, (Hq + Hkv) * D, cache, st, Hkv, D)
        want = torch.zeros(n_pages, 2, Hkv, page, D, dtype=dtype)
        want_v = torch.zeros(n_pages, Hkv, D, page, dtype=dtype)          # values lie dimension-major in a page
        xc = x.cpu()
        for n, sl in enumerate(slots):
            if sl < 0:
                continue
            pg, row = divmod(sl, page)
            want[pg, 0, :, row, :] = xc[n, Hq * D:(Hq + Hkv) * D].view(Hkv, D)
            want_v[pg, :, :, row] = xc[n, (Hq + Hkv) * D:].view(Hkv, D)
        got = cache.cpu()
        assert torch.equal(got[:, 0], want[:, 0])
        assert torch.equal(got[:, 1].reshape(n_pages, Hkv, D, page), want_v)


def test_a_far_key_among_hundreds_is_found(ops):
    """Random keys give near-uniform weights, which would hide a lost key: here one key far back
    carries almost all the weight of the last query."""
    for far, n in ((3, 700), (255, 700), (256, 700), (639, 700)):
        case = PagedCase(lens=[n], new=[1], Hq=2, Hkv=2, D=64, page=16, dtype=torch.bfloat16, seed=far, scale_boost=(far, 3.0))
        scale = 1 / 8
        want = case.plain(scale, None)
        # the weight of the far key dominates: the result is close to that key's value
        assert np.abs(want[0, :64] - case.v[0][far, :64].double().numpy()).max() < 0.2
        out = torch.empty_like(case.qcat)
        ops.attention_decode(case.qcat, case.cache, case.bt, case.seq_lens, 1, 2, scale, None, out)
        assert np.abs(out.double().cpu().numpy() - want).max() < 2e-2
        case2 = PagedCase(lens=[n], new=[130], Hq=2, Hkv=2, D=64, page=16, dtype=torch.bfloat16, seed=far, scale_boost=(far, 3.0))
        out2 = torch.empty_like(case2.qcat)
        ops.attention_prefill(case2.qcat, case2.cache, case2.bt, case2.q_start, case2.seq_lens, 0, 1, 130, 2, scale, None, out2)
        assert np.abs(out2.double().cpu().numpy() - case2.plain(scale, None)).max() < 2e-2


# ----------------------------------------------------------------------------- sampling
def _records(params_list, V, seeds):
    import struct
    from deliverance_amd.sampling import JavaRandom, device_record
    words, us = [], []
    for p, seed in zip(params_list, seeds):
        rng = JavaRandom(seed)
        rec = device_record(p, rng, V)
        words += struct.unpack("<8i", rec)
        us.append(struct.unpack("<fififfii", rec)[4])
    return torch.tensor(words, dtype=torch.int32, device=DEV), us


def test_sampling_kernel_against_the_plain_sampler(ops):
    from deliverance_amd.sampling import GeneratorParameters as GP
    g = torch.Generator().manual_seed(5)
    V = 50257
    combos = [GP(), GP(temperature=0.8), GP(temperature=1.3, top_k=50), GP(temperature=0.7, top_p=0.9),
              GP(temperature=1.0, top_k=40, top_p=0.95), GP(temperature=1.0, top_k=0.999), GP(temperature=2.0, top_p=0.3),
              GP(temperature=0.9, top_k=5, top_p=0.5, uniform_top_p=1.0), GP(temperature=1.0, top_p=1.0)]
    rows, plist, seeds = [], [], []
    for i in range(4):
        for c in combos:
            rows.append(torch.randn(V, generator=g) * 3.0)
            plist.append(c); seeds.append(100 + i)
    logits = torch.stack(rows).to(DEV)
    rec, us = _records(plist, V, seeds)
    out = torch.empty(len(rows), dtype=torch.int32, device=DEV)
    ops.sample(logits, rec, out)
    got = out.cpu().tolist()
    for r, (p, u) in enumerate(zip(plist, us)):
        lg = rows[r].numpy()
        want = int(np.argmax(lg)) if p.temperature == 0 else \
            P.sample_top_k_top_p(lg, p.temperature, p.top_k, p.top_p, p.uniform_top_p, u)
        assert got[r] == want, (r, p)


@pytest.mark.simt_quick
def test_sampling_vectors_of_the_reference(ops):
    """core/src/test/java/io/teknek/deliverance/model/TopKSamplerTest.java:23-54, with the draws given."""
    import struct
    logits = torch.tensor([[5.0, 4.0, 3.0, 2.0, 1.0]] * 5 + [[1.0, 1.0, 1.0, 0.0, 1.0]] * 2, device=DEV)

    def rec(T, k, p, uni, u):
        return struct.unpack("<8i", struct.pack("<fififfii", T, k, p, uni, u, 0.0, 0, 0))
    words = (rec(1.0, 2, 0.95, 0, 0.99) + rec(1.0, 2, 0.95, 0, 0.60) + rec(1.0, 2, 0.95, 1, 0.60) + rec(0.0, 0, 0.0, 0, 0.0)
             + rec(1.0, 0, 0.0, 0, 0.999999) + rec(0.0, 0, 0.0, 0, 0.0) + rec(1.0, 3, 0.0, 0, 0.70))
    out = torch.empty(7, dtype=torch.int32, device=DEV)
    ops.sample(logits, torch.tensor(words, dtype=torch.int32, device=DEV), out)
    # weighted 0.99 -> 1, weighted 0.60 -> 0, uniform in nucleus 0.60 -> 1, greedy -> 0, u ~ 1 -> last token,
    # greedy ties -> lowest index, top-3 of equal logits keeps indices 0,1,2 and 0.70 lands on the third
    assert out.cpu().tolist() == [1, 0, 1, 0, 4, 0, 2]


@pytest.mark.simt_quick
def test_xtc_and_logprobs(ops):
    import struct
    V = 1000
    g = torch.Generator().manual_seed(9)
    lg = torch.randn(V, generator=g)
    lg[10], lg[20], lg[30] = 9.0, 8.5, 8.0          # three tokens above a 10% threshold
    logits = torch.stack([lg, lg, lg]).to(DEV)

    def rec(T, thr, active):
        return struct.unpack("<8i", struct.pack("<fififfii", T, 0, 0.0, 0, 0.0, thr, active, 0))
    words = rec(0.0, 0.1, 1) + rec(0.0, 0.1, 0) + rec(1.0, 0.1, 1)
    out = torch.empty(3, dtype=torch.int32, device=DEV)
    params = torch.tensor(words, dtype=torch.int32, device=DEV)
    ops.sample(logits, params, out)
    # active: the least likely of the tokens above the threshold; inactive: the maximum
    assert out.cpu().tolist() == [30, 10, 30]
    idx = torch.empty(3, 4, dtype=torch.int32, device=DEV)
    lp = torch.empty(3, 4, dtype=torch.float32, device=DEV)
    ops.top_logprobs(logits, params, 4, idx, lp)
    want = torch.log_softmax(lg.double(), 0)
    top = torch.topk(want, 4)
    assert idx[0].cpu().tolist() == top.indices.tolist()
    assert (lp[0].cpu().double() - top.values).abs().max() < 1e-4


# ----------------------------------------------------------------------------- fused norm + product
@pytest.mark.parametrize("M,N,K", [helpers.quick(1, 96, 64), (8, 2304, 768), helpers.quick(17, 1000, 96), (32, 200, 1600), (5, 50257, 768),
                                   (16, 520, 1024), helpers.quick(12, 72, 1000), helpers.quick(9, 40, 520), (3, 1000, 1600), (16, 300, 2048),
                                   helpers.quick(5, 64, 1304), helpers.quick(2, 48, 8), (11, 200, 1992), (8, 200, 1280),
                                   helpers.quick(7, 48, 2040)])
@pytest.mark.parametrize("pdtype", [torch.bfloat16, torch.float32])
def test_fused_norm_product(ops, M, N, K, pdtype):
    helpers.skip_in_simulation_if(M * N * K > 1.2e8)
    g = torch.Generator().manual_seed(M + N)
    x = (torch.randn(M + 3, K, generator=g) * 2 + 1).to(DEV)
    gw, gb = torch.randn(K, generator=g).to(pdtype).to(DEV), torch.randn(K, generator=g).to(pdtype).to(DEV)
    w = bf(torch.randn(N, K, generator=g) * 0.1).to(DEV)
    # the product's bias in the norm's dtype (the kernels for parameters of one dtype) or, with 32-bit norm
    # parameters and an even M, in bfloat16 (the general kernel)
    bias = bf(torch.randn(N, generator=g)).to(pdtype if M % 2 else torch.bfloat16).to(DEV)
    rows = torch.tensor([(i * 7) % (M + 3) for i in range(M)], dtype=torch.int32, device=DEV)
    a = F.layer_norm(x.double(), (K,), gw.double(), gb.double(), 1e-5)[rows.long()].to(torch.bfloat16).double()
    for act, od in ((None, torch.float32), ("gelu_new", torch.bfloat16)):
        out = torch.empty(M, N, device=DEV, dtype=od)
        ops.linear_ln(x, rows, M, gw, gb, 1e-5, w, bias, out, act=act)
        ref = a @ w.double().t() + bias.double()
        if act:
            ref = F.gelu(ref, approximate="tanh")
        tol = (2e-2 if od == torch.bfloat16 else 2e-3) * max(1.0, ref.abs().max().item())
        assert (out.double() - ref).abs().max() < tol


@pytest.mark.parametrize("M", [helpers.quick(5), helpers.quick(40), helpers.quick(300), 1000, 2100])
def test_product_writes_keys_and_values(ops, M):
    """The skinny (M <= 64) and tile kernels scatter the k | v columns in their epilogue."""
    g = torch.Generator().manual_seed(M)
    Hq, Hkv, D, page, K = 5, 3, 48, 16, (128 if M >= 2000 else 104)      # a K that no slab cuts, too
    N = (Hq + 2 * Hkv) * D
    n_pages = (M + page - 1) // page + 2
    a = bf(torch.randn(M, K, generator=g)).to(DEV)
    w = bf(torch.randn(N, K, generator=g) * 0.1).to(DEV)
    bias = bf(torch.randn(N, generator=g)).to(DEV)
    perm = torch.randperm(n_pages * page, generator=g)[:M].to(torch.int32)
    perm[M // 2] = -1
    # the places in any order; and as a prompt portion has them: runs of consecutive rows, one from a
    # multiple of 8 on (values go over in 16-byte runs), one from 3 on, with a token that is not kept
    runs = torch.cat([torch.arange(16, 16 + M // 2), torch.arange(16 + M // 2 + 19, 16 + M // 2 + 19 + M - M // 2)]).to(torch.int32)
    runs[M // 4] = -1
    for order in (perm, runs):
        slots = order.to(DEV)
        c1 = torch.zeros(n_pages + 2, 2, Hkv, page, D, dtype=torch.bfloat16, device=DEV)
        c2 = torch.zeros_like(c1)
        out1 = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
        out2 = torch.empty_like(out1)
        ops.linear_mfma(a, w, bias, out1, kv_cache=c1, slot_map=slots, q_cols=Hq * D)
        ops.linear_mfma(a, w, bias, out2)
        ops.kv_write(out2, Hq * D, (Hq + Hkv) * D, c2, slots, Hkv, D)
        assert torch.equal(out1, out2)
        assert torch.equal(c1, c2) and c1.abs().sum() > 0


@pytest.mark.simt_quick
@pytest.mark.parametrize("M,K", [(9, 96), (7, 1312)])
def test_fused_norm_product_writes_keys_and_values(ops, M, K):
    """(7 rows and a wide K: two groups of 16 columns a workgroup)"""
    g = torch.Generator().manual_seed(11)
    Hq, Hkv, D, page = 6, 2, 48, 16
    N = (Hq + 2 * Hkv) * D
    x = torch.randn(M, K, generator=g).to(DEV)
    gw, gb = bf(torch.randn(K, generator=g)).to(DEV), bf(torch.randn(K, generator=g)).to(DEV)
    w = bf(torch.randn(N, K, generator=g) * 0.1).to(DEV)
    bias = bf(torch.randn(N, generator=g)).to(DEV)
    slots = torch.tensor([3 * page + 5, -1, 0, 17, 40, 41, 42, 95, 64][:M], dtype=torch.int32, device=DEV)
    c1 = torch.zeros(6, 2, Hkv, page, D, dtype=torch.bfloat16, device=DEV)
    c2 = torch.zeros_like(c1)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    ops.linear_ln(x, None, M, gw, gb, 1e-5, w, bias, out, kv_cache=c1, slot_map=slots, q_cols=Hq * D)
    ops.kv_write(out, Hq * D, (Hq + Hkv) * D, c2, slots, Hkv, D)      # the separate kernel on the same rows
    assert torch.equal(c1, c2) and c1.abs().sum() > 0
