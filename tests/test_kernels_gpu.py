"""Each HIP kernel alone against its plain PyTorch reference (kernel_refs.py), at sizes other
than the engine's tiny models: widths and vocabularies that are no power of two, head sizes
from 16 to 256, grouped key heads, several page sizes."""
import math

import pytest
import torch

import kernel_refs as R
from plain import sampler_plain as SP

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def ops():
    from denno_beta_amd.kernels import ops as o
    return o


def rnd(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


TOL = {torch.float32: dict(atol=2e-5, rtol=2e-5), torch.bfloat16: dict(atol=2e-2, rtol=2e-2)}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E", [40, 1600])
def test_embed(dtype, E):
    wte, wpe = rnd(777, E, seed=1, dtype=dtype), rnd(50, E, seed=2, dtype=dtype)
    tok, pos = i32([0, 776, 5, 5, 300]), i32([0, 49, 7, 8, 1])
    out = torch.empty(5, E, device=DEV)
    ops().embed(tok, pos, wte, wpe, out)
    assert torch.equal(out, R.embed(tok, pos, wte, wpe, torch.empty_like(out)))
    ops().embed(tok, pos, wte, None, out)
    assert torch.equal(out, wte[tok.long()].float())


@pytest.mark.parametrize("E", [40, 100, 1600, 3000, 9000])
def test_layernorm(E):
    x = rnd(9, E, seed=3, scale=3.0) + 1.5
    g, b = rnd(E, seed=4), rnd(E, seed=5)
    for out_dtype in (torch.float32, torch.bfloat16):
        for rows in (None, i32([8, 0, 3])):
            n = 9 if rows is None else 3
            out = torch.empty(n, E, dtype=out_dtype, device=DEV)
            ops().layernorm(x, g, b, 1e-6, out, rows)
            want = R.layernorm(x, g, b, 1e-6, torch.empty(n, E, device=DEV), rows)
            assert torch.allclose(out.float(), want, **TOL[out_dtype])
    out = torch.empty(9, E, device=DEV)
    ops().layernorm(x, g, None, 1e-2, out)
    assert torch.allclose(out, R.layernorm(x, g, None, 1e-2, torch.empty_like(out)), atol=2e-5)
    # the reference's vector (crates/denno-engine/src/tensor.rs:1706-1718), widened to a kernel-sized row
    x2 = torch.tensor([[0.0, 2.0] * 8], device=DEV)
    ops().layernorm(x2, torch.full((16,), 2.0, device=DEV), torch.ones(16, device=DEV), 0.0, out16 := torch.empty(1, 16, device=DEV))
    assert torch.allclose(out16, torch.tensor([[-1.0, 3.0] * 8], device=DEV), atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kv_write(dtype):
    hkv, dh, ps, n_pages = 3, 32, 8, 6
    src = rnd(7, 5 * hkv * dh, seed=6, dtype=dtype)
    slots = i32([0, 9, 47, -1, 10, 23, 40])
    k = torch.zeros(n_pages, hkv, ps, dh, dtype=dtype, device=DEV)
    v = torch.zeros(n_pages, hkv, dh, ps, dtype=dtype, device=DEV)
    k2, v2 = torch.zeros_like(k), torch.zeros_like(v)
    ops().kv_write(src, hkv * dh, 3 * hkv * dh, slots, k, v)
    R.kv_write(src, hkv * dh, 3 * hkv * dh, slots, k2, v2)
    assert torch.equal(k, k2) and torch.equal(v, v2) and k.abs().sum() > 0


@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 1001, 72), (5, 64, 8), (130, 200, 320), (64, 1600, 1600), (33, 50257, 96),
                                   (200, 333, 72), (300, 1600, 1600), (257, 129, 200), (2048, 256, 6400),
                                   (48, 4800, 1600), (17, 4104, 72), (40, 33000, 40),
                                   # on both sides of the borders between the bfloat16 kernels: columns (2,560; 4,096),
                                   # rows (104 / 105, 208 / 209), a long inner size into the stream (65 .. 512 rows)
                                   (48, 2552, 256), (64, 2568, 1280), (104, 4104, 1024), (105, 4104, 1024),
                                   (208, 2304, 768), (209, 2304, 768), (65, 1032, 4128), (512, 1000, 4096)])
def test_linear(in_dtype, M, N, K):
    a, w, bias = rnd(M, K, seed=7, dtype=in_dtype), rnd(N, K, seed=8, dtype=in_dtype, scale=0.2), rnd(N, seed=9)
    if in_dtype == torch.bfloat16:      # the MFMA kernels take the packed matrix; rows go to the plain kernel
        rows, w = w, ops().pack_matrix(w)
        assert torch.equal(w.rows(), rows)
        w_ref = rows
    else:
        w_ref = w
    # the reference sums in 64-bit; a 32-bit sum of K terms is off by about sqrt(K) roundings
    tol = dict(TOL[in_dtype])
    tol["atol"] = max(tol["atol"], 4e-6 * math.sqrt(K))
    exact = lambda epi: R.linear(a.double(), w_ref.double(), bias.double(), out=torch.empty(M, N, dtype=torch.float64, device=DEV),   # noqa: E731
                                 epilogue=epi).float()
    for out_dtype in (torch.float32, in_dtype):
        for epi in ("none", "gelu_tanh", "gelu_erf"):
            out = torch.empty(M, N, dtype=out_dtype, device=DEV)
            ops().linear(a, w, bias, out=out, epilogue=epi)
            assert torch.allclose(out.float(), exact(epi), **(tol if out_dtype == in_dtype else dict(tol, rtol=TOL[in_dtype]["rtol"]))), (out_dtype, epi)
    res = rnd(M, N, seed=10)
    want = (res.double() + a.double() @ w_ref.double().t()).float()
    ops().linear(a, w, None, residual=res)
    assert torch.allclose(res, want, **tol)
    # rows taken out of a wider matrix (a leading dimension larger than K)
    wide = rnd(M, K + 24, seed=11, dtype=in_dtype)
    out = torch.empty(M, N, device=DEV)
    ops().linear(wide[:, 8:8 + K], w, bias, out=out)
    assert torch.allclose(out, R.linear(wide[:, 8:8 + K], w_ref, bias, out=torch.empty_like(out)), **tol)
    if in_dtype == torch.bfloat16 and M * N * K < 10 ** 8:
        # bfloat16 rows, not packed: the plain kernel
        ops().linear(a, w_ref, bias, out=out)
        assert torch.allclose(out, exact("none"), **tol)


def test_linear_with_every_tile_of_the_many_rows_kernel():
    """Beyond 256 rows the tile is chosen per product from a list: every tile on the list, on sizes
    that are no multiple of it, with a short K (fewer slabs than the kernel keeps in flight) and
    longer ones (each picks another arrangement of waves and stages), for each kind of output."""
    o = ops()
    tile = o._lib("gemm").dn_gemm_tile
    cases = {}
    # per tile and K the smallest product that gets it.  K = 64: one stage; 416: no multiple of 64, so a slab a
    # stage; 448: two slabs a stage; 4,160: a long K, which takes more stages in flight
    for K in (64, 416, 448, 4160):
        for M in range(260, 4200, 140):
            for N in range(136, 10000, 232):
                t = tile(M, N, K)
                if (t, K) not in cases or M * N < cases[(t, K)][0] * cases[(t, K)][1]:
                    cases[(t, K)] = (M, N, K)
    assert len({t for t, _ in cases}) == 9, sorted(cases)
    tol = dict(TOL[torch.bfloat16])
    for M, N, K in cases.values():
        a, w, bias = rnd(M, K, seed=1, dtype=torch.bfloat16), rnd(N, K, seed=2, dtype=torch.bfloat16, scale=0.2), rnd(N, seed=3)
        wp = o.pack_matrix(w)
        exact = (a.double() @ w.double().t() + bias.double()).float()
        for out_dtype in (torch.float32, torch.bfloat16):
            out = torch.empty(M, N, dtype=out_dtype, device=DEV)
            o.linear(a, wp, bias, out=out)
            assert torch.allclose(out.float(), exact, **tol), (M, N, K, out_dtype)
        out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        o.linear(a, wp, bias, out=out, epilogue="gelu_tanh")
        assert torch.allclose(out.float(), torch.nn.functional.gelu(exact, approximate="tanh"), **tol), (M, N, K)
        res = rnd(M, N, seed=4)
        want = res + exact
        o.linear(a, wp, bias, residual=res)
        assert torch.allclose(res, want, **tol), (M, N, K)


@pytest.mark.parametrize("M", [1, 8, 20, 64, 70, 300, 1000])
@pytest.mark.parametrize("slots_in", ["any order", "runs"])
@pytest.mark.parametrize("queries_only", [False, True])
def test_linear_qkv_writes_the_cache(M, slots_in, queries_only):
    """The fused projection with the cache write in its epilogue (of the few-rows kernel or of the
    tiled one) against the product followed by the separate write.  Slots in any order, or as a
    prompt's portion has them: runs of consecutive slots (the tiled kernel then stores a dim's
    values of four tokens at once), starting anywhere.  The output holds all columns, or the
    queries alone."""
    H, Hkv, dh, ps, n_pages, K = 6, 2, 32, 16, max(40, (M + 101) // 16 + 1), 96
    N = (H + 2 * Hkv) * dh
    a, w, bias = rnd(M, K, seed=1, dtype=torch.bfloat16), rnd(N, K, seed=2, dtype=torch.bfloat16, scale=0.2), rnd(N, seed=3)
    g = torch.Generator().manual_seed(M)
    if slots_in == "runs":
        starts, slots = [8, 10, 40, 101], []     # the first and third run start 4-aligned
        for i in range(M):
            slots.append(starts[i * 4 // max(M, 1)] + i)       # four runs
        slots = torch.tensor(slots, dtype=torch.int32)
    else:
        slots = torch.randperm(n_pages * ps, generator=g)[:M].to(torch.int32)
    if M > 2:
        slots[2] = -1
    slots = slots.to(DEV)
    pools = [torch.zeros(n_pages, Hkv, ps, dh, dtype=torch.bfloat16, device=DEV),
             torch.zeros(n_pages, Hkv, dh, ps, dtype=torch.bfloat16, device=DEV)]
    want_pools = [torch.zeros_like(p) for p in pools]
    w = ops().pack_matrix(w)
    out = torch.full((M, H * dh if queries_only else N), 7.0, dtype=torch.bfloat16, device=DEV)
    queries = ops().linear_qkv(a, w, bias, out, slots, pools[0], pools[1], H * dh)
    want = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops().linear(a, w, bias, out=want)
    R.kv_write(want, H * dh, (H + Hkv) * dh, slots, want_pools[0], want_pools[1])
    assert torch.equal(queries, want[:, :H * dh]) and (queries_only or torch.equal(out, want))
    assert torch.equal(pools[0], want_pools[0]) and torch.equal(pools[1], want_pools[1])
    assert pools[0].abs().sum() > 0 and pools[1].abs().sum() > 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,K,ps", [(1, 256, 16), (8, 1600, 16), (7, 264, 12), (33, 512, 8), (64, 384, 16), (65, 256, 16), (5, 96, 16)])
def test_linear_qkv_in_the_plain_kernels(dtype, M, K, ps):
    """The fused projection with weights in rows (the 32-bit engine's): with few rows and a K of several segments
    the kernel that adds the segments' sums writes the cache too; with more rows, or one segment, a kernel of its
    own does.  Either way against the product followed by the reference's write, bit for bit, a row without a slot
    among them and a page size that is no power of two."""
    H, Hkv, dh, n_pages = 5, 3, 16, 30
    N = (H + 2 * Hkv) * dh
    a, w, bias = rnd(M, K, seed=1, dtype=dtype), rnd(N, K, seed=2, dtype=dtype, scale=0.2), rnd(N, seed=3)
    slots = torch.randperm(n_pages * ps, generator=torch.Generator().manual_seed(M))[:M].to(torch.int32)
    if M > 2:
        slots[2] = -1
    slots = slots.to(DEV)
    pools = [torch.zeros(n_pages, Hkv, ps, dh, dtype=dtype, device=DEV), torch.zeros(n_pages, Hkv, dh, ps, dtype=dtype, device=DEV)]
    want_pools = [torch.zeros_like(p) for p in pools]
    out = torch.full((M, N), 7.0, dtype=dtype, device=DEV)
    before = ops().launches
    queries = ops().linear_qkv(a, w, bias, out, slots, pools[0], pools[1], H * dh)
    fused = M <= 64 and K > 128
    assert ops().launches - before == (1 if fused else 2), (M, K)
    want = torch.empty(M, N, dtype=dtype, device=DEV)
    ops().linear(a, w, bias, out=want)
    R.kv_write(want, H * dh, (H + Hkv) * dh, slots, want_pools[0], want_pools[1])
    assert torch.equal(out, want) and torch.equal(queries, want[:, :H * dh])
    assert torch.equal(pools[0], want_pools[0]) and torch.equal(pools[1], want_pools[1])
    assert pools[0].abs().sum() > 0 and pools[1].abs().sum() > 0


@pytest.mark.parametrize("M,E,I,epilogue", [(1, 64, 256, "gelu_tanh"), (8, 1600, 6400, "gelu_tanh"), (5, 96, 320, "gelu_erf"),
                                            (16, 1600, 4800, "none"), (13, 2560, 1024, "none"), (3, 4096, 4112, "gelu_tanh"),
                                            (9, 16, 16, "none"), (2, 336, 1000, "none")])
def test_a_norm_inside_the_products_on_both_sides_of_it(M, E, I, epilogue):
    """x += a W1^T + b1 leaves the rows times gamma in bfloat16 and their statistics by blocks of 16
    columns; the next product runs on those rows and applies the norm to its sums: against the plain
    references of both, against the three kernels one after the other (product into the stream,
    LayerNorm, product), and a row alone."""
    a = rnd(M, I, seed=1, dtype=torch.bfloat16)
    x0 = rnd(M, E, seed=2, scale=3.0) + 1.5                   # rows whose mean is half their spread
    w1, b1 = rnd(E, I, seed=3, dtype=torch.bfloat16, scale=0.05), rnd(E, seed=4)
    w2, b2 = rnd(I, E, seed=5, dtype=torch.bfloat16, scale=0.1), rnd(I, seed=6)
    gamma, beta = 1 + rnd(E, seed=7, scale=0.1), rnd(E, seed=8, scale=0.1)
    p1, p2 = ops().pack_matrix(w1), ops().pack_matrix(w2)
    assert ops().norm_stream_takes(M, E, p1)
    for b in (beta, None):
        x = x0.clone()
        copy, stats = ops().norm_stream_buffers(M, E, DEV)
        copy.fill_(7.0), stats.fill_(7.0)
        ops().linear_norm_out(a, p1, b1, x, gamma, copy, stats)
        x_ref, copy_ref, stats_ref = x0.clone(), torch.empty_like(copy), torch.empty_like(stats)
        R.linear_norm_out(a, w1, b1, x_ref, gamma, copy_ref, stats_ref)
        x_two = ops().linear(a, p1, b1, residual=x0.clone())
        assert torch.equal(x, x_two)                                # the same sums as the kernel that leaves nothing
        assert torch.allclose(x, x_ref, atol=2e-2, rtol=2e-2)
        assert torch.equal(copy, (x * gamma).to(torch.bfloat16))
        assert torch.allclose(stats[:, :, 0], stats_ref[:, :, 0], atol=1e-3, rtol=1e-3)
        assert torch.allclose(stats[:, :, 1], stats_ref[:, :, 1], atol=1e-2, rtol=1e-2)
        c1, c2 = ops().norm_folded(p2.rows(), b2, gamma, b)
        c1r, c2r = R.norm_folded(w2, b2, gamma, b)
        assert torch.allclose(c1, c1r, atol=1e-4, rtol=1e-4) and torch.allclose(c2, c2r, atol=1e-4, rtol=1e-4)
        out = torch.full((M, I), 7.0, dtype=torch.bfloat16, device=DEV)
        ops().linear_norm_in(copy, stats, c1, c2, 1e-5, p2, out, epilogue=epilogue)
        plain = R.linear_norm_in(copy, stats, c1, c2, 1e-5, w2, torch.empty_like(out), epilogue=epilogue)
        assert torch.allclose(out.float(), plain.float(), atol=3e-2, rtol=2e-2), (M, E, I)
        # against the norm as a kernel of its own on the 32-bit rows: here the rows are rounded to
        # bfloat16 before the mean is taken off, there after; the two differ by roundings only
        h = ops().layernorm(x, gamma, b, 1e-5, torch.empty(M, E, dtype=torch.bfloat16, device=DEV))
        three = ops().linear(h, p2, b2, out=torch.empty_like(out), epilogue=epilogue)
        assert (out.float() - three.float()).norm() <= 1e-2 * three.float().norm(), (M, E, I)
    alone = torch.empty(1, I, dtype=torch.bfloat16, device=DEV)
    ops().linear_norm_in(copy[M - 1:M].contiguous(), stats[M - 1:M].contiguous(), c1, c2, 1e-5, p2, alone, epilogue=epilogue)
    assert torch.equal(alone[0], out[M - 1])


@pytest.mark.parametrize("M,E,I,epilogue", [(17, 1600, 6400, "gelu_tanh"), (40, 1408, 5632, "none"), (64, 1600, 4800, "gelu_tanh"),
                                            (33, 1024, 1040, "none"), (50, 2048, 4096, "gelu_erf")])
@pytest.mark.parametrize("layout", ["packed", "rows"])
def test_a_norm_inside_products_of_17_to_64_rows(M, E, I, epilogue, layout):
    """The same with the rows travelling packed, as they do from 17 rows on, or in rows: the product
    into the stream reads packed rows and leaves a packed copy, the product after it reads that and
    writes packed rows."""
    pk = layout == "packed"
    a = rnd(M, I, seed=1, dtype=torch.bfloat16)
    x0 = rnd(M, E, seed=2, scale=3.0) + 1.5
    w1, b1 = rnd(E, I, seed=3, dtype=torch.bfloat16, scale=0.05), rnd(E, seed=4)
    w2, b2 = rnd(I, E, seed=5, dtype=torch.bfloat16, scale=0.1), rnd(I, seed=6)
    gamma, beta = 1 + rnd(E, seed=7, scale=0.1), rnd(E, seed=8, scale=0.1)
    p1, p2 = ops().pack_matrix(w1), ops().pack_matrix(w2)
    assert ops().norm_stream_takes(M, E, p1) and ops().norm_stream_takes(M, E, p2)
    x = x0.clone()
    copy, stats = ops().norm_stream_buffers(M, E, DEV)
    assert isinstance(copy, ops().PackedMatrix)
    if not pk:
        copy = torch.empty(M, E, dtype=torch.bfloat16, device=DEV)
    ops().linear_norm_out(ops().pack_matrix(a) if pk and I % 32 == 0 else a, p1, b1, x, gamma, copy, stats)
    x_two = ops().linear(a, p1, b1, residual=x0.clone())
    assert torch.allclose(x, x_two, atol=1e-4, rtol=1e-5)          # the same product from rows and from packed rows
    copy_rows = copy.rows() if pk else copy
    assert torch.equal(copy_rows, (x * gamma).to(torch.bfloat16))
    stats_ref = torch.empty_like(stats)
    R.linear_norm_out(a, w1, b1, x0.clone(), gamma, torch.empty(M, E, dtype=torch.bfloat16, device=DEV), stats_ref)
    assert torch.allclose(stats[:, :, 0], stats_ref[:, :, 0], atol=1e-3, rtol=1e-3)
    assert torch.allclose(stats[:, :, 1], stats_ref[:, :, 1], atol=1e-2, rtol=1e-2)
    c1, c2 = ops().norm_folded(p2.rows(), b2, gamma, beta)
    out = ops().packed_rows(M, I, DEV) if pk and I % 32 == 0 else torch.full((M, I), 7.0, dtype=torch.bfloat16, device=DEV)
    ops().linear_norm_in(copy, stats, c1, c2, 1e-5, p2, out, epilogue=epilogue)
    out_rows = out.rows() if isinstance(out, ops().PackedMatrix) else out
    plain = R.linear_norm_in(copy_rows, stats, c1, c2, 1e-5, w2, torch.empty(M, I, dtype=torch.bfloat16, device=DEV), epilogue=epilogue)
    assert torch.allclose(out_rows.float(), plain.float(), atol=3e-2, rtol=2e-2), (M, E, I)
    h = ops().layernorm(x, gamma, beta, 1e-5, torch.empty(M, E, dtype=torch.bfloat16, device=DEV))
    three = ops().linear(h, p2, b2, out=torch.empty(M, I, dtype=torch.bfloat16, device=DEV), epilogue=epilogue)
    assert (out_rows.float() - three.float()).norm() <= 1e-2 * three.float().norm(), (M, E, I)
    # the same rows among 16 give the same as among M (another kernel: to rounding)
    few_copy, few_stats = copy_rows[:16].contiguous(), stats[:16].contiguous()
    few = ops().linear_norm_in(few_copy, few_stats, c1, c2, 1e-5, p2, torch.empty(16, I, dtype=torch.bfloat16, device=DEV), epilogue=epilogue)
    assert torch.allclose(few.float(), out_rows[:16].float(), atol=3e-2, rtol=2e-2)


@pytest.mark.parametrize("M,E,I", [(5, 96, 320), (16, 1600, 4800), (33, 1024, 4096), (64, 1600, 6400)])
def test_a_norm_without_a_mean_inside_the_products(M, E, I):
    """The same two kernels run a norm that takes no mean off, x / sqrt(mean(x^2) + eps) * gamma: the product after it
    takes the squares about 0 and uses no c1.  Against that norm in 64-bit followed by the product, on rows whose mean
    is as large as their spread (a mean taken off by mistake would show)."""
    a = rnd(M, I, seed=1, dtype=torch.bfloat16)
    x0 = rnd(M, E, seed=2, scale=2.0) + 2.0
    w1, b1 = rnd(E, I, seed=3, dtype=torch.bfloat16, scale=0.05), rnd(E, seed=4)
    w2, b2 = rnd(I, E, seed=5, dtype=torch.bfloat16, scale=0.1), rnd(I, seed=6)
    gamma = 1 + rnd(E, seed=7, scale=0.1)
    p1, p2 = ops().pack_matrix(w1), ops().pack_matrix(w2)
    x = x0.clone()
    copy, stats = ops().norm_stream_buffers(M, E, DEV)
    ops().linear_norm_out(a, p1, b1, x, gamma, copy, stats)
    c1, c2 = ops().norm_folded(p2.rows(), b2, gamma, None, no_mean=True)
    assert not c1.any() and torch.allclose(c2, b2)
    packed_out = M > 16
    out = ops().packed_rows(M, I, DEV) if packed_out else torch.empty(M, I, dtype=torch.bfloat16, device=DEV)
    ops().linear_norm_in(copy, stats, c1, c2, 1e-6, p2, out, epilogue="gelu_tanh", no_mean=True)
    got = (out.rows() if packed_out else out).float()
    xd = x.double()
    y = xd / torch.sqrt((xd * xd).mean(dim=1, keepdim=True) + 1e-6) * gamma.double()
    want = torch.nn.functional.gelu(y @ w2.double().t() + b2.double(), approximate="tanh").float()
    assert (got - want).norm() <= 1e-2 * want.norm(), (M, E, I, ((got - want).norm() / want.norm()).item())
    # with the mean taken off the result is another one
    wrong = torch.nn.functional.layer_norm(xd, (E,), gamma.double(), None, 1e-6)
    wrong = torch.nn.functional.gelu(wrong @ w2.double().t() + b2.double(), approximate="tanh").float()
    assert (got - wrong).norm() > 0.1 * want.norm()
    plain = R.linear_norm_in(copy if not packed_out else copy.rows(), stats, c1, c2, 1e-6, w2, torch.empty(M, I, dtype=torch.bfloat16, device=DEV),
                             epilogue="gelu_tanh", no_mean=True)
    assert torch.allclose(got, plain.float(), atol=3e-2, rtol=2e-2)


def test_a_norm_inside_a_fused_projection_writes_the_cache():
    H, Hkv, dh, ps, n_pages, E, M = 6, 2, 48, 16, 12, 160, 7
    N = (H + 2 * Hkv) * dh
    x = rnd(M, E, seed=1, scale=2.0) + 0.7
    gamma, beta = 1 + rnd(E, seed=2, scale=0.1), rnd(E, seed=3, scale=0.1)
    copy = (x * gamma).to(torch.bfloat16)
    stats = torch.empty(M, E // 16, 2, device=DEV)
    blocks = x.view(M, -1, 16)
    stats[:, :, 0] = blocks.mean(-1)
    stats[:, :, 1] = ((blocks - blocks.mean(-1, keepdim=True)) ** 2).sum(-1)
    w, bias = rnd(N, E, seed=4, dtype=torch.bfloat16, scale=0.2), rnd(N, seed=5)
    wp = ops().pack_matrix(w)
    c1, c2 = ops().norm_folded(wp.rows(), bias, gamma, beta)
    slots = torch.randperm(n_pages * ps, generator=torch.Generator().manual_seed(M))[:M].to(torch.int32)
    slots[2] = -1
    slots = slots.to(DEV)
    for queries_only in (False, True):
        pools = [torch.zeros(n_pages, Hkv, ps, dh, dtype=torch.bfloat16, device=DEV),
                 torch.zeros(n_pages, Hkv, dh, ps, dtype=torch.bfloat16, device=DEV)]
        want_pools = [torch.zeros_like(p) for p in pools]
        out = torch.full((M, H * dh if queries_only else N), 7.0, dtype=torch.bfloat16, device=DEV)
        queries = ops().linear_norm_in(copy, stats, c1, c2, 1e-5, wp, out, kv=(slots, pools[0], pools[1], H * dh))
        want = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        ops().linear_norm_in(copy, stats, c1, c2, 1e-5, wp, want)
        R.kv_write(want, H * dh, (H + Hkv) * dh, slots, want_pools[0], want_pools[1])
        assert torch.equal(queries, want[:, :H * dh]) and (queries_only or torch.equal(out, want))
        assert torch.equal(pools[0], want_pools[0]) and torch.equal(pools[1], want_pools[1])
        assert pools[0].abs().sum() > 0 and pools[1].abs().sum() > 0
    h = ops().layernorm(x, gamma, beta, 1e-5, torch.empty(M, E, dtype=torch.bfloat16, device=DEV))
    two = ops().linear(h, wp, bias, out=torch.empty(M, N, dtype=torch.bfloat16, device=DEV))
    assert (want.float() - two.float()).norm() <= 1e-2 * two.float().norm()


def test_the_norm_inside_products_refuses_what_it_cannot_take():
    wp = ops().pack_matrix(rnd(32, 64, seed=2, dtype=torch.bfloat16))
    assert not ops().norm_stream_takes(17, 64, wp) and not ops().norm_stream_takes(4, 40, wp) and not ops().norm_stream_takes(65, 1600, wp)
    assert not ops().norm_stream_takes(4, 8192, wp) and not ops().norm_stream_takes(4, 64, rnd(32, 64, dtype=torch.bfloat16))
    copy, stats = ops().norm_stream_buffers(17, 64, DEV)
    c = rnd(32, seed=3)
    with pytest.raises(ops().KernelError):
        ops().linear_norm_in(copy, stats, c, c, 1e-5, wp, torch.empty(17, 32, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ops().KernelError):
        ops().linear_norm_out(rnd(17, 64, dtype=torch.bfloat16), wp, None, rnd(17, 32), c, *ops().norm_stream_buffers(17, 32, DEV))


@pytest.mark.parametrize("M", [100, 129, 200, 256, 300, 1000, 2100, 4200])
@pytest.mark.parametrize("rows_in", ["packed", "rows"])
@pytest.mark.parametrize("K", [160, 192, 4160])
def test_linear_qkv_with_many_columns(M, rows_in, K):
    """The fused projection where its columns are many (the many-rows kernel takes it from 129 rows on,
    with packed rows too): heads of 48, a grouped cache, pages of 32, slots in runs that start anywhere.
    An inner size that is a multiple of 64 goes two slabs a stage, a long one keeps more stages in flight,
    and the rows decide the tile."""
    if rows_in == "packed" and M > 256:
        pytest.skip("packed rows end at 256")
    o = ops()
    H, Hkv, dh, ps = 64, 16, 48, 32
    N = (H + 2 * Hkv) * dh
    assert N >= 4096
    n_pages = (M + 40) // ps + 2
    a, w, bias = rnd(M, K, seed=1, dtype=torch.bfloat16), rnd(N, K, seed=2, dtype=torch.bfloat16, scale=0.2), rnd(N, seed=3)
    slots = torch.tensor([(5 if i < M // 3 else 12 if i < 2 * M // 3 else 33) + i for i in range(M)], dtype=torch.int32)
    slots[7] = -1
    slots = slots.to(DEV)
    pools = [torch.zeros(n_pages, Hkv, ps, dh, dtype=torch.bfloat16, device=DEV),
             torch.zeros(n_pages, Hkv, dh, ps, dtype=torch.bfloat16, device=DEV)]
    want_pools = [torch.zeros_like(p) for p in pools]
    wp = o.pack_matrix(w)
    out = torch.full((M, H * dh), 7.0, dtype=torch.bfloat16, device=DEV)
    queries = o.linear_qkv(o.pack_matrix(a) if rows_in == "packed" else a, wp, bias, out, slots, pools[0], pools[1], H * dh)
    want = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    o.linear(a, wp, bias, out=want)
    R.kv_write(want, H * dh, (H + Hkv) * dh, slots, want_pools[0], want_pools[1])
    assert torch.equal(queries, want[:, :H * dh])
    assert torch.equal(pools[0], want_pools[0]) and torch.equal(pools[1], want_pools[1])
    assert pools[0].abs().sum() > 0 and pools[1].abs().sum() > 0
    exact = (a.double() @ w.double().t() + bias.double()).float()
    assert torch.allclose(want.float(), exact, **TOL[torch.bfloat16])


@pytest.mark.parametrize("M", [1, 8, 16, 17, 40, 64, 65, 100, 130, 200, 256])
@pytest.mark.parametrize("N,K", [(1600, 1600), (4800, 1600), (96, 6400), (33024, 64)])
def test_linear_with_packed_rows(M, N, K):
    """The few-rows product reading packed rows and writing them gives, bit for bit, what it gives
    with rows in the ordinary layout; so does LayerNorm."""
    o = ops()
    a, w, bias = rnd(M, K, seed=M, dtype=torch.bfloat16), o.pack_matrix(rnd(N, K, seed=N, dtype=torch.bfloat16, scale=0.05)), rnd(N, seed=3)
    ap = o.pack_matrix(a)
    assert torch.equal(ap.rows(), a)
    want = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    for epi in ("none", "gelu_tanh"):
        o.linear(a, w, bias, out=want, epilogue=epi)
        got = o.packed_rows(M, N, DEV)
        o.linear(ap, w, bias, out=got, epilogue=epi)
        assert torch.equal(got.rows(), want)
        mixed = torch.empty_like(want)
        o.linear(ap, w, bias, out=mixed, epilogue=epi)
        assert torch.equal(mixed, want)
    res, res2 = rnd(M, N, seed=4), rnd(M, N, seed=4)
    o.linear(a, w, bias, residual=res)
    o.linear(ap, w, bias, residual=res2)
    assert torch.equal(res, res2)
    x, g, b = rnd(M, K, seed=5), rnd(K, seed=6), rnd(K, seed=7)
    rows = o.layernorm(x, g, b, 1e-5, torch.empty(M, K, dtype=torch.bfloat16, device=DEV))
    assert torch.equal(o.layernorm(x, g, b, 1e-5, o.packed_rows(M, K, DEV)).rows(), rows)
    pick = i32(list(range(M - 1, -1, -1)))
    assert torch.equal(o.layernorm(x, g, b, 1e-5, o.packed_rows(M, K, DEV), pick).rows(), rows.flip(0))


@pytest.mark.parametrize("M", [65, 96, 100, 129, 256, 300, 512, 513])
@pytest.mark.parametrize("N,K", [(1600, 6400), (1032, 4128), (96, 4096)])
def test_linear_into_the_stream_with_a_long_inner_size(M, N, K):
    """65 to 512 rows, fewer than 4,096 columns, K from 4,096 on, added into the residual stream: K is shared
    out among workgroups and a second kernel adds the shares in order.  Against 64-bit sums; from rows and from
    packed rows alike; the same bits on a second call."""
    o = ops()
    a, w, bias = rnd(M, K, seed=M, dtype=torch.bfloat16), rnd(N, K, seed=N, dtype=torch.bfloat16, scale=0.05), rnd(N, seed=3)
    wp = o.pack_matrix(w)
    x0 = rnd(M, N, seed=4)
    want = (x0.double() + a.double() @ w.double().t() + bias.double()).float()
    got = o.linear(a, wp, bias, residual=x0.clone())
    assert torch.allclose(got, want, atol=2e-3, rtol=1e-4), (got - want).abs().max().item()
    assert torch.equal(o.linear(a, wp, bias, residual=x0.clone()), got)
    if M <= 256:
        assert torch.equal(o.linear(o.pack_matrix(a), wp, bias, residual=x0.clone()), got)
    # one request's rows do not depend on the rows beside them (other kernels below 65 rows: not the same bits)
    if M >= 130:
        part = o.linear(a[:M - 30].contiguous(), wp, bias, residual=x0[:M - 30].clone())
        assert torch.allclose(part, got[:M - 30], atol=2e-3, rtol=1e-4)


def test_packed_rows_are_refused_where_no_kernel_takes_them():
    o = ops()
    w = o.pack_matrix(rnd(64, 64, dtype=torch.bfloat16))
    with pytest.raises(o.KernelError, match="at most 256 rows"):
        o.packed_rows(257, 64, DEV)
    with pytest.raises(o.KernelError, match="multiple of 32"):
        o.packed_rows(4, 48, DEV)
    with pytest.raises(o.KernelError, match="need a packed matrix"):
        o.linear(o.packed_rows(4, 64, DEV), rnd(64, 64, dtype=torch.bfloat16), None, out=torch.empty(4, 64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(o.KernelError, match="packed rows as out"):
        o.linear(rnd(270, 64, dtype=torch.bfloat16), w, None, out=o.PackedMatrix(torch.empty(17 * 2 * 512, dtype=torch.bfloat16, device=DEV), (270, 64)))
    with pytest.raises(o.KernelError, match="bfloat16 rows"):
        o.linear(rnd(4, 64), w, None, out=torch.empty(4, 64, device=DEV))


def test_linear_rows_do_not_depend_on_the_batch():
    a, w = rnd(150, 96, seed=1), rnd(333, 96, seed=2)
    full = torch.empty(150, 333, device=DEV)
    ops().linear(a, w, None, out=full)
    for rows in ([0], [149], [3, 77, 78]):
        sub = torch.empty(len(rows), 333, device=DEV)
        ops().linear(a[rows].contiguous(), w, None, out=sub)
        assert torch.equal(sub, full[rows])


@pytest.mark.parametrize("N,K", [(1600, 1600), (1600, 6400), (50257, 320), (100, 96), (333, 200), (4800, 1608)])
def test_plain_linear_has_one_order_of_summation_whatever_the_rows(N, K):
    """The 32-bit product has two kernels (up to 64 rows, where K's segments may be workgroups of their
    own with a second kernel that adds their sums; more rows) and four row tiles: a row's result is the
    same bits in all of them, alone or among 200 rows, with bias, GELU or the residual sum."""
    a, w, bias = rnd(200, K, seed=1), rnd(N, K, seed=2, scale=0.1), rnd(N, seed=3)
    full = {}
    for epi in ("none", "gelu_erf"):
        full[epi] = ops().linear(a, w, bias, out=torch.empty(200, N, device=DEV), epilogue=epi)
    res0 = rnd(200, N, seed=4)
    full["residual"] = ops().linear(a, w, bias, residual=res0.clone())
    want = R.linear(a.double(), w.double(), bias.double(), out=torch.empty(200, N, dtype=torch.float64, device=DEV)).float()
    assert torch.allclose(full["none"], want, atol=4e-6 * math.sqrt(K), rtol=2e-5)
    for rows in ([0], [199], [5, 6], list(range(3, 11)), list(range(40, 49)), list(range(16)), list(range(100, 133)),
                 list(range(64)), list(range(65))):
        sub = a[rows].contiguous()
        for epi in ("none", "gelu_erf"):
            got = ops().linear(sub, w, bias, out=torch.empty(len(rows), N, device=DEV), epilogue=epi)
            assert torch.equal(got, full[epi][rows]), (len(rows), epi)
        got = ops().linear(sub, w, bias, residual=res0[rows].contiguous())
        assert torch.equal(got, full["residual"][rows]), (len(rows), "residual")


def test_linear_refuses_what_it_cannot_take():
    o = ops()
    with pytest.raises(o.KernelError, match="multiple of 8"):
        o.pack_matrix(rnd(4, 12, dtype=torch.bfloat16))
    with pytest.raises(o.KernelError, match="does not fit"):
        o.linear(rnd(2, 16), rnd(4, 24), None, out=torch.empty(2, 4, device=DEV))
    with pytest.raises(o.KernelError):
        o.linear(rnd(2, 16), rnd(4, 16, dtype=torch.bfloat16), None, out=torch.empty(2, 4, device=DEV))
    with pytest.raises(o.KernelError, match="GPU"):
        o.linear(torch.zeros(2, 16), rnd(4, 16), None, out=torch.empty(2, 4, device=DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(2, 4, 12), (5, 33, 7), (70, 50, 101), (64, 130, 1601), (300, 66, 30), (1, 9, 1)])
def test_plain_linear_takes_any_inner_size(dtype, M, N, K):
    """The plain product (all of 32-bit, and bfloat16 operands that the matrix-core kernels do not take) runs any
    inner size, with every epilogue, against 64-bit sums; rows of a width that is no multiple of 4 included."""
    o = ops()
    a, w, bias = rnd(M, K, seed=1, dtype=dtype), rnd(N, K, seed=2, dtype=dtype, scale=0.3), rnd(N, seed=3)
    exact = a.double() @ w.double().t() + bias.double()
    tol = TOL[dtype]
    for epi, f in (("none", lambda t: t), ("gelu_tanh", lambda t: torch.nn.functional.gelu(t, approximate="tanh")),
                   ("gelu_erf", torch.nn.functional.gelu)):
        out = torch.empty(M, N, dtype=dtype, device=DEV)
        o.linear(a, w, bias, out=out, epilogue=epi)
        assert torch.allclose(out.float(), f(exact).float(), **tol), (M, N, K, epi)
    res = rnd(M, N, seed=4)
    want = (res.double() + exact).float()
    o.linear(a, w, bias, residual=res)
    assert torch.allclose(res, want, **tol)
    # a row's result does not depend on the rows beside it (one order of summation)
    if dtype == torch.float32 and M > 1:
        alone = torch.empty(1, N, device=DEV)
        o.linear(a[M - 1:M].contiguous(), w, bias, out=alone)
        both = torch.empty(M, N, device=DEV)
        o.linear(a, w, bias, out=both)
        assert torch.equal(alone[0], both[M - 1])


def paged_case(seq_lens, new_rows, H, Hkv, dh, ps, dtype, seed=0, q_scale=1.0):
    """A cache filled with random keys and values for requests of the given lengths, scattered
    over shuffled pages, and the tables of a step in which request s brings new_rows[s] rows."""
    g = torch.Generator().manual_seed(seed)
    blocks = [-(-n // ps) for n in seq_lens]
    n_pages = sum(blocks) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    k = (torch.randn(n_pages, Hkv, ps, dh, generator=g)).to(dtype).to(DEV)
    v = (torch.randn(n_pages, Hkv, dh, ps, generator=g)).to(dtype).to(DEV)
    bt = torch.full((len(seq_lens), max(blocks)), -1, dtype=torch.int32)
    tiles, wide, row = [], [], 0
    for s, (n, new) in enumerate(zip(seq_lens, new_rows)):
        for b in range(blocks[s]):
            bt[s, b] = perm.pop()
        for i in range(0, new, 16):
            tiles.append((s, row + i, min(16, new - i), n - new + i))
        for i in range(0, new, 128):
            wide.append((s, row + i, min(128, new - i), n - new + i))
        row += new
    q = (torch.randn(row, 3 * H * dh, generator=g) * q_scale).to(dtype).to(DEV)
    paged_case.wide = i32(wide).t().contiguous()
    return q, k, v, bt.to(DEV), i32(tiles).t().contiguous(), row


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,Hkv,dh,ps,window", [(4, 4, 16, 16, 0), (25, 25, 64, 16, 0), (6, 2, 48, 8, 0),
                                                (2, 1, 128, 64, 0), (3, 3, 256, 16, 0), (4, 2, 32, 16, 20),
                                                (5, 5, 80, 32, 7), (4, 2, 15, 16, 0), (3, 3, 100, 8, 9), (2, 1, 250, 16, 0),
                                                (5, 5, 1, 16, 0)])
def test_attention(dtype, H, Hkv, dh, ps, window):
    # four requests: a decoded token far into a long context, a whole prompt, a portion, a first token
    seq_lens, new_rows = [300, 70, 133, 1], [1, 70, 21, 1]
    q, k, v, bt, tiles, T = paged_case(seq_lens, new_rows, H, Hkv, dh, ps, dtype, seed=H + dh)
    scale = 1 / math.sqrt(dh)
    out = torch.zeros(T, H * dh, dtype=dtype, device=DEV)
    ops().attention(q[:, H * dh:2 * H * dh], out, k, v, bt, tiles, H, scale, window)
    want = R.attention(q[:, H * dh:2 * H * dh], torch.zeros(T, H * dh, device=DEV), k, v, bt, tiles, H, scale, window)
    assert torch.allclose(out.float(), want, **TOL[dtype])


@pytest.mark.parametrize("H,Hkv,dh,ps,window", [(4, 4, 16, 16, 0), (25, 25, 64, 16, 0), (6, 2, 48, 32, 0),
                                                (2, 1, 128, 64, 0), (3, 3, 96, 16, 0), (4, 2, 32, 16, 20),
                                                (5, 5, 64, 32, 7), (2, 2, 64, 16, 150), (4, 2, 64, 48, 0),
                                                (3, 3, 32, 80, 30), (5, 5, 80, 16, 0), (2, 1, 112, 16, 25),
                                                (2, 2, 144, 16, 0), (2, 1, 160, 32, 0), (3, 3, 176, 16, 0),
                                                (2, 2, 192, 16, 90), (1, 1, 208, 16, 0), (2, 1, 224, 48, 0),
                                                (1, 1, 240, 16, 0), (2, 2, 256, 16, 40)])
def test_attention_mfma_kernel_for_portions(H, Hkv, dh, ps, window):
    """The bfloat16 kernel for portions of prompts (tiles of up to 128 rows): a long portion deep
    in a context, a whole prompt, a short portion, single rows."""
    seq_lens, new_rows = [430, 70, 133, 1, 200], [300, 70, 21, 1, 1]
    q, k, v, bt, tiles, T = paged_case(seq_lens, new_rows, H, Hkv, dh, ps, torch.bfloat16, seed=H + dh)
    scale = 1 / math.sqrt(dh)
    out = torch.zeros(T, H * dh, dtype=torch.bfloat16, device=DEV)
    ops().attention(q[:, :H * dh], out, k, v, bt, tiles, H, scale, window, tiles_wide=paged_case.wide)
    want = R.attention(q[:, :H * dh], torch.zeros(T, H * dh, device=DEV), k, v, bt, tiles, H, scale, window)
    assert torch.allclose(out.float(), want, **TOL[torch.bfloat16])
    if (H * dh) % 32 == 0:
        # the first 200 rows as packed rows (the same requests, the long portion cut short)
        new_rows[0] = 107
        q2, k2, v2, bt2, tiles2, T2 = paged_case(seq_lens, new_rows, H, Hkv, dh, ps, torch.bfloat16, seed=H + dh)
        rows = torch.zeros(T2, H * dh, dtype=torch.bfloat16, device=DEV)
        ops().attention(q2[:, :H * dh], rows, k2, v2, bt2, tiles2, H, scale, window, tiles_wide=paged_case.wide)
        packed = ops().packed_rows(T2, H * dh, DEV)
        ops().attention(q2[:, :H * dh], packed, k2, v2, bt2, tiles2, H, scale, window, tiles_wide=paged_case.wide)
        assert T2 == 200 and torch.equal(packed.rows(), rows)


@pytest.mark.parametrize("H,Hkv,dh,ps,window", [(8, 8, 64, 16, 0), (8, 2, 32, 32, 40), (8, 4, 64, 48, 0),
                                                (8, 8, 96, 16, 0), (8, 2, 128, 32, 60), (8, 8, 80, 16, 0),
                                                (8, 4, 160, 16, 30), (8, 8, 256, 16, 0)])
def test_attention_mfma_kernel_with_many_workgroups(H, Hkv, dh, ps, window):
    """More workgroups than CUs, so that they follow one another on a CU: two groups of waves a workgroup up to
    heads of 64, one group beyond (two tiles of keys a step for heads of 96, one for 128)."""
    g = torch.Generator().manual_seed(3)
    new_rows = [int(n) for n in torch.randint(1, 200, (36,), generator=g)]
    seq_lens = [n + int(x) for n, x in zip(new_rows, torch.randint(0, 150, (36,), generator=g))]
    q, k, v, bt, tiles, T = paged_case(seq_lens, new_rows, H, Hkv, dh, ps, torch.bfloat16, seed=H + dh)
    assert paged_case.wide.shape[1] * H > 256
    scale = 1 / math.sqrt(dh)
    out = torch.zeros(T, H * dh, dtype=torch.bfloat16, device=DEV)
    ops().attention(q[:, :H * dh], out, k, v, bt, tiles, H, scale, window, tiles_wide=paged_case.wide)
    want = R.attention(q[:, :H * dh], torch.zeros(T, H * dh, device=DEV), k, v, bt, tiles, H, scale, window)
    assert torch.allclose(out.float(), want, **TOL[torch.bfloat16])


@pytest.mark.parametrize("H,Hkv,dh,ps,window", [(4, 4, 16, 16, 0), (25, 25, 64, 16, 0), (6, 2, 32, 32, 0),
                                                (2, 1, 128, 64, 0), (3, 3, 256, 16, 0), (5, 5, 64, 16, 100),
                                                (2, 2, 64, 32, 300), (4, 2, 64, 48, 0), (3, 3, 32, 80, 90),
                                                (6, 2, 48, 16, 0), (5, 5, 80, 32, 0), (3, 3, 96, 16, 0),
                                                (2, 1, 112, 16, 50), (2, 2, 144, 16, 0), (2, 1, 160, 16, 0),
                                                (1, 1, 176, 32, 0), (2, 2, 192, 16, 0), (1, 1, 208, 16, 70),
                                                (2, 1, 224, 16, 0), (2, 2, 240, 16, 0)])
def test_attention_split_kernel_for_decoding(H, Hkv, dh, ps, window):
    """The bfloat16 kernel for steps in which every request brings one row: contexts on both sides
    of a split's edge (256 keys) and of a page's."""
    seq_lens = [1, 17, 256, 257, 700, 1024, 512, 64]
    q, k, v, bt, tiles, T = paged_case(seq_lens, [1] * len(seq_lens), H, Hkv, dh, ps, torch.bfloat16, seed=dh)
    scale = 1 / math.sqrt(dh)
    want = R.attention(q[:, :H * dh], torch.zeros(T, H * dh, device=DEV), k, v, bt, tiles, H, scale, window)
    for max_context in (1024, 1040):         # the second: a launch sized for a longer context than any request's
        if max_context > bt.shape[1] * ps:
            continue
        out = torch.zeros(T, H * dh, dtype=torch.bfloat16, device=DEV)
        ops().attention(q[:, :H * dh], out, k, v, bt, tiles, H, scale, window, tiles_wide=paged_case.wide,
                        single_rows=True, max_context=max_context)
        assert torch.allclose(out.float(), want, **TOL[torch.bfloat16])
        # every size of workgroup that the head size allows, not only the one that `attention` picks here
        for waves in (4, 8, 16):
            if waves <= (16 if dh <= 64 else 8 if dh <= 128 else 4):
                other = torch.zeros(T, H * dh, dtype=torch.bfloat16, device=DEV)
                ops().attention(q[:, :H * dh], other, k, v, bt, tiles, H, scale, window, single_rows=True,
                                max_context=max_context, decode_waves=waves)
                assert torch.allclose(other.float(), want, **TOL[torch.bfloat16]), waves
        if (H * dh) % 32 == 0:               # the same rows, packed for the product that follows
            packed = ops().packed_rows(T, H * dh, DEV)
            ops().attention(q[:, :H * dh], packed, k, v, bt, tiles, H, scale, window, single_rows=True,
                            max_context=max_context)
            assert torch.equal(packed.rows(), out)
    # one short request alone: a single split, written without the join
    out = torch.zeros(1, H * dh, dtype=torch.bfloat16, device=DEV)
    one = (q[1:2, :H * dh], k, v, bt[1:2].contiguous(), i32([[0], [0], [1], [16]]), H, scale, window)
    ops().attention(one[0], out, *one[1:], single_rows=True, max_context=17)
    assert torch.allclose(out.float(), want[1:2], **TOL[torch.bfloat16])
    if (H * dh) % 32 == 0:
        packed = ops().packed_rows(1, H * dh, DEV)
        ops().attention(one[0], packed, *one[1:], single_rows=True, max_context=17)
        assert torch.equal(packed.rows(), out)
        with pytest.raises(ops().KernelError, match="bfloat16 kernels only"):
            ops().attention(one[0], packed, *one[1:])


@pytest.mark.parametrize("dh", [64, 48, 96, 208])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_finds_a_far_key(dtype, dh):
    """One key among hundreds matches the query strongly: the output must be its value, whichever
    page and tile it lies in (the first key, a page's edge, the last key of a tile, the newest).  Head sizes
    that are a power of two and others (whose keys leave lanes of the decode kernel empty)."""
    H, ps, n = 2, 16, 700
    for far in (0, 15, 16, 63, 64, 383, 699):
        q, k, v, bt, tiles, T = paged_case([n], [1], H, H, dh, ps, dtype, seed=far)
        page, off = int(bt[0, far // ps]), far % ps
        qh = q[0, :dh].float()
        k[page, 0, off] = (qh / qh.norm() * 40).to(dtype)       # score 40 |q| against about |q| for the others
        tol = 1e-2 if dtype == torch.bfloat16 else 1e-4
        for kw in (dict(), dict(tiles_wide=paged_case.wide), dict(single_rows=True, max_context=n)):
            out = torch.zeros(1, H * dh, dtype=dtype, device=DEV)
            ops().attention(q[:, :H * dh], out, k, v, bt, tiles, H, 1.0, **kw)
            assert torch.allclose(out[0, :dh].float(), v[page, 0, :, off].float(), atol=tol), (far, kw.keys())


def test_attention_window_edges():
    """With values that encode their position, the window's first and last key are seen exactly."""
    H, dh, ps, n, window = 1, 16, 16, 200, 37
    q, k, v, bt, tiles, T = paged_case([n], [n], H, H, dh, ps, torch.float32, seed=1)
    k.zero_()                       # all scores equal: the output is the mean of the values in the window
    for pos in range(n):
        v[int(bt[0, pos // ps]), 0, :, pos % ps] = float(pos)
    out = torch.zeros(T, dh, device=DEV)
    ops().attention(q[:, :dh], out, k, v, bt, tiles, H, 1.0, window)
    for pos in (0, 1, 36, 37, 38, 100, 199):
        lo = max(0, pos - window + 1)
        assert abs(out[pos, 0].item() - (lo + pos) / 2) < 1e-3, pos


@pytest.mark.parametrize("H,dh,window,n", [(2, 64, 37, 700), (2, 64, 100, 700), (1, 128, 100, 1000), (3, 32, 300, 520)])
def test_attention_window_edges_in_every_kernel(H, dh, window, n):
    """All scores equal and values that name their position (dim p % dh is 1 at position p): the output is,
    per dim, the share of the window's positions with that remainder, so one key too many or too few at
    either edge of the window changes a dim by 1 / window, which is far above what bfloat16 rounds.
    The 32-bit kernel, the bfloat16 kernel for portions and the bfloat16 kernel for single rows (with the
    context split over workgroups where the head size makes chunks of 512 keys, so that a split lies
    wholly before the window)."""
    ps = 16
    for dtype in (torch.float32, torch.bfloat16):
        q, k, v, bt, tiles, T = paged_case([n], [n], H, H, dh, ps, dtype, seed=window)
        k.zero_(), v.zero_()
        pos = torch.arange(n, device=DEV)
        pages, offs = bt[0, pos // ps].long(), pos % ps
        for h in range(H):
            v[pages, h, pos % dh, offs] = 1.0
        # want[p, d]: how many positions of [lo, p] have remainder d, over the window's length
        onehot = torch.zeros(n, dh, device=DEV)
        onehot[pos, pos % dh] = 1.0
        cum = torch.cat([torch.zeros(1, dh, device=DEV), onehot.cumsum(0)])
        lo = (pos - window + 1).clamp(min=0)
        want = ((cum[pos + 1] - cum[lo]) / (pos - lo + 1).unsqueeze(1)).repeat(1, H)
        kinds = [dict()] if dtype == torch.float32 else [dict(tiles_wide=paged_case.wide)]
        for kw in kinds:
            out = torch.zeros(T, H * dh, dtype=dtype, device=DEV)
            ops().attention(q[:, :H * dh], out, k, v, bt, tiles, H, 1.0, window, **kw)
            worst = (out.float() - want).abs().max(dim=1).values
            assert worst.max().item() < 0.2 / window, (dtype, int(worst.argmax()), worst.max().item())
        if dtype == torch.bfloat16:
            for p in sorted({0, 1, window - 2, window - 1, window, window + 1, 255, 256, 257, 511, 512, 513, n - 1}):
                if p >= n:
                    continue
                out = torch.zeros(1, H * dh, dtype=dtype, device=DEV)
                ops().attention(q[p:p + 1, :H * dh], out, k, v, bt, i32([[0], [0], [1], [p]]), H, 1.0, window,
                                single_rows=True, max_context=min(-(-(p + 1) // 256) * 256, bt.shape[1] * ps))
                assert (out[0].float() - want[p]).abs().max().item() < 0.2 / window, ("single row", p)


@pytest.mark.parametrize("dh,ps", [(32, 16), (64, 16), (64, 4), (64, 6), (64, 64)])
def test_attention_rows_do_not_depend_on_the_batch(dh, ps):
    # (heads of 64 on pages of a multiple of 4 keys have a kernel of their own for steps of single rows; a page of
    # 6 keys and heads of 32 take the general one)
    H = 4
    q, k, v, bt, tiles, T = paged_case([200, 90], [50, 90], H, H, dh, ps, torch.float32, seed=2)
    out = torch.zeros(T, H * dh, device=DEV)
    ops().attention(q[:, :H * dh], out, k, v, bt, tiles, H, 0.2)
    # request 0's last row alone, as a decoded token: in the kernel for portions, and in the kernels for steps of
    # single rows, where every tile of keys is a workgroup of its own (launched for its context and for a longer one)
    one = torch.zeros(1, H * dh, device=DEV)
    ops().attention(q[49:50, :H * dh], one, k, v, bt, i32([[0], [0], [1], [199]]), H, 0.2)
    assert torch.equal(one[0], out[49])
    for max_context in (200, min(264, bt.shape[1] * ps)):
        one = torch.zeros(1, H * dh, device=DEV)
        ops().attention(q[49:50, :H * dh], one, k, v, bt, i32([[0], [0], [1], [199]]), H, 0.2, single_rows=True,
                        max_context=max_context)
        assert torch.equal(one[0], out[49])
    # both requests' last rows as one step of single rows, with a window
    win = torch.zeros(T, H * dh, device=DEV)
    ops().attention(q[:, :H * dh], win, k, v, bt, tiles, H, 0.2, 70)
    two = torch.zeros(2, H * dh, device=DEV)
    rows = torch.stack([q[49, :H * dh], q[139, :H * dh]]).contiguous()
    ops().attention(rows, two, k, v, bt, i32([[0, 1], [0, 1], [1, 1], [199, 89]]), H, 0.2, 70, single_rows=True,
                    max_context=200)
    assert torch.equal(two[0], win[49]) and torch.equal(two[1], win[139])


def test_sample_greedy_and_walk():
    V = 50257
    logits = rnd(6, V, seed=3, scale=2.0)
    logits[0, 100] = logits[0, 40000] = 50.0            # two maxima: the first wins (sampler.rs:569-582)
    logits[1, 7] = float("nan")                         # NaN is ignored (sampler.rs:1222-1224)
    logits[2, :] = float("-inf")                        # nothing is greater than -inf: index 0
    temp = torch.tensor([0.0, 0.0, 0.0, 0.8, 1.0, 2.5], device=DEV)
    u = torch.tensor([0.0, 0.0, 0.0, 0.3, 0.999999, 0.5], device=DEV)
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    ops().sample(logits, temp, u, out)
    got = out.tolist()
    assert got[0] == 100 and got[1] == int(torch.nan_to_num(logits[1], nan=-1e30).argmax()) and got[2] == 0
    for r in (3, 4, 5):
        want = SP.temperature_walk(logits[r].tolist(), float(temp[r]), float(u[r]))
        assert abs(got[r] - want) <= 1 or abs(float(logits[r, got[r]]) - float(logits[r, want])) < 1e-3, r
    # u = 0 picks the first token
    ops().sample(logits[3:4], temp[3:4], torch.zeros(1, device=DEV), out[:1])
    assert out[0].item() == 0


@pytest.mark.parametrize("V", [1, 17, 64, 65, 1000, 4097, 50257, 300001])
def test_temperature_walk_at_other_vocabulary_sizes(V):
    """The walk's place against the running sums in 64-bit: for every row and its uniform number u the token
    picked is the first whose running share of the probability reaches u, to within what 32-bit sums can tell
    (the share before the token is at most u, the share with it at least u, both with a margin of 1e-5).  Sizes
    below, at and above a wave's 64 tokens, a block's worth, and one that needs blocks of more than 64 tokens."""
    from denno_beta_amd.sampling import uniform
    n = 16
    logits = rnd(n, V, seed=V % 1000, scale=3.0)
    temp = torch.tensor([0.3, 0.7, 1.0, 1.9] * 4, device=DEV)
    u = torch.tensor([uniform(11, i) for i in range(n - 2)] + [0.0, 0.9999999], device=DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ops().sample(logits, temp, u, out)
    z = logits.double().cpu() / temp.double().cpu()[:, None]
    cum = torch.softmax(z, dim=1).cumsum(dim=1)
    for r, tok in enumerate(out.tolist()):
        assert 0 <= tok < V
        before = float(cum[r, tok - 1]) if tok > 0 else 0.0
        assert before <= float(u[r]) + 1e-5 and float(cum[r, tok]) >= float(u[r]) - 1e-5, (r, tok, before, float(cum[r, tok]), float(u[r]))
    assert out[n - 2].item() == 0


def test_sample_frequencies():
    # [0, 4] at T = 1: index 1 with probability 0.982 (sampler.rs:686-704), here over a row padded with -inf
    from denno_beta_amd.sampling import uniform
    n, V = 4000, 333
    logits = torch.full((n, V), float("-inf"), device=DEV)
    logits[:, 17], logits[:, 200] = 0.0, 4.0
    u = torch.tensor([uniform(5, i) for i in range(n)], device=DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ops().sample(logits, torch.ones(n, device=DEV), u, out)
    assert set(out.tolist()) == {17, 200}
    assert abs((out == 200).float().mean().item() - 0.982) < 0.02


def test_sample_top_and_penalties():
    from denno_beta_amd.sampling import uniform
    V = 1003
    logits = rnd(8, V, seed=4, scale=3.0)
    logits[2, 10] = logits[2, 900] = logits[2].max() + 1      # a tie at the top
    rows = i32([1, 2, 5, 6, 7])
    ks, ps = i32([5, 1, 0, 40, 2048]), torch.tensor([1.0, 1.0, 0.7, 0.9, 0.3], device=DEV)
    temp = torch.full((8,), 0.7, device=DEV)
    for trial in range(5):
        u = torch.tensor([uniform(trial, i) for i in range(8)], device=DEV)
        out = torch.full((8,), -1, dtype=torch.int32, device=DEV)
        undecided = torch.full((5,), -1, dtype=torch.int32, device=DEV)
        ops().sample_top(logits, rows, temp, u, ks, ps, out, undecided)
        want = R.sample_top(logits.cpu(), rows.cpu(), temp.cpu(), u.cpu(), ks.cpu(), ps.cpu(),
                            torch.full((8,), -1, dtype=torch.int32), torch.zeros(5, dtype=torch.int32))
        assert out.tolist() == want.tolist(), trial
        assert undecided.tolist() == [0] * 5          # a vocabulary within the 2,048 candidates is always decided
    assert out[2].item() == 10
    # contexts as rows of a table of histories, with other tokens behind each row's length that must not count
    ctx = i32([3, 4, 3, 9, 4, 3, 1, 1] + [5, 5, 5, 5, 5, 5, 5, 5] + [7, 8, 7, 8, 7, 2, 2, 2])
    begin, length = i32([0, 8, 16]), i32([6, 0, 5])
    l = rnd(3, V, seed=5)
    want = R.penalties(l.clone().cpu(), ctx.cpu(), begin.cpu(), length.cpu(), torch.tensor([1.5, 1.0, 1.0]),
                       torch.tensor([0.3, 0.0, 0.0]), torch.tensor([0.2, 0.0, 0.5]), torch.tensor([0, 0, 2], dtype=torch.int32))
    before = l.clone()
    ops().penalties(l, ctx, begin, length, torch.tensor([1.5, 1.0, 1.0], device=DEV), torch.tensor([0.3, 0.0, 0.0], device=DEV),
                    torch.tensor([0.2, 0.0, 0.5], device=DEV), i32([0, 0, 2]), bounds=21)
    assert torch.allclose(l.cpu(), want, atol=1e-6) and l[2, 8].item() == float("-inf")
    assert torch.equal(l[1], before[1]) and l[0, 1] == before[0, 1] and l[2, 2] == before[2, 2]
    with pytest.raises(Exception):
        ops().penalties(l, ctx, begin, length, torch.ones(3, device=DEV), torch.zeros(3, device=DEV),
                        torch.zeros(3, device=DEV), i32([0, 0, 0]), bounds=25)


def test_penalties_over_long_contexts():
    """Contexts from nothing to more tokens than the kernel keeps in the workgroup's memory (8,192), few distinct
    tokens so that each is counted often, every row with its own options; tokens outside the vocabulary count for
    nothing."""
    V = 517
    lens = [0, 1, 2, 700, 1025, 8192, 8193, 9001]
    g = torch.Generator().manual_seed(12)
    width = 9100
    table = torch.randint(0, V, (len(lens), width), generator=g, dtype=torch.int32)
    table[3, 5] = V + 3
    table[4, 0] = -1
    for r, n in enumerate(lens):                    # what lies behind a context must not count: a token that
        table[r, n:] = 77                           # would show at once
    ctx = table.to(DEV).view(-1)
    begin, length = i32([r * width for r in range(len(lens))]), i32(lens)
    rep = torch.tensor([1.3, 1.3, 1.0, 1.2, 1.0, 1.5, 1.1, 1.0])
    fq = torch.tensor([0.1, 0.0, 0.2, 0.05, 0.0, 0.01, 0.02, 0.0])
    pr = torch.tensor([0.0, 0.4, 0.0, 0.3, 0.0, 0.2, 0.0, 0.0])
    ng = torch.tensor([2, 2, 2, 3, 2, 0, 4, 2], dtype=torch.int32)
    l = rnd(len(lens), V, seed=6, scale=2.0)
    want = R.penalties(l.clone().cpu(), ctx.cpu(), begin.cpu(), length.cpu(), rep, fq, pr, ng)
    ops().penalties(l, ctx, begin, length, rep.to(DEV), fq.to(DEV), pr.to(DEV), ng.to(DEV), bounds=7 * width + 9001)
    assert torch.equal(torch.isinf(l.cpu()), torch.isinf(want))
    fin = ~torch.isinf(want)
    assert torch.allclose(l.cpu()[fin], want[fin], atol=1e-5, rtol=1e-6)
    assert torch.equal(l[0].cpu(), want[0]) and (l[7].cpu() != rnd(len(lens), V, seed=6, scale=2.0)[7].cpu()).sum() > 0


def test_history_append():
    """Sampled tokens go behind their requests' histories, each at its own place, and nothing else changes."""
    history = torch.arange(100, 140, dtype=torch.int32, device=DEV)        # 4 histories of 10 places
    tokens = i32([11, 22, 33, 44, 55, -1, -1])                            # a step's tokens, and flags behind them
    begin, length, rows = i32([30, 0, 10]), i32([9, 0, 4]), i32([4, 0, 2])
    want = R.history_append(history.clone().cpu(), begin.cpu(), length.cpu(), rows.cpu(), tokens.cpu())
    ops().history_append(history, begin, length, rows, tokens, bounds=(39, 4))
    assert history.tolist() == want.tolist()
    assert history[39].item() == 55 and history[0].item() == 11 and history[14].item() == 33
    changed = (history.cpu() != torch.arange(100, 140, dtype=torch.int32)).nonzero().flatten().tolist()
    assert changed == [0, 14, 39]
    with pytest.raises(Exception):
        ops().history_append(history, begin, length, rows, tokens, bounds=(40, 4))
    with pytest.raises(Exception):
        ops().history_append(history, begin, length, rows, tokens, bounds=(39, 7))


@pytest.mark.parametrize("V,levels", [(6000, 3), (6000, 40), (50257, 7), (3000, 1), (2100, 2)])
def test_sample_top_with_many_equal_logits(V, levels):
    """Logits that take few different values, so that many keys are equal to the one at the cut: of these the
    ones with the lowest indices belong to the candidates, as the plain sampler sorts (value descending, then
    index ascending).  With 3 levels over 6,000 tokens some 2,000 tie at the cut, with 1 or 2 levels more than the
    2,048 that the kernel lists before it ranks them (it then walks the row in stretches)."""
    from denno_beta_amd.sampling import uniform
    g = torch.Generator().manual_seed(V + levels)
    logits = (torch.randint(0, levels, (6, V), generator=g).float() * 0.5).to(DEV).contiguous()
    rows = i32([0, 1, 2, 3, 4, 5])
    ks, ps = i32([1, 7, 300, 2048, 0, 0]), torch.tensor([1.0, 0.9, 1.0, 0.95, 0.5, 0.02], device=DEV)
    temp = torch.full((6,), 0.9, device=DEV)
    for trial in range(3):
        u = torch.tensor([uniform(trial, i) for i in range(6)], device=DEV)
        out = torch.full((6,), -1, dtype=torch.int32, device=DEV)
        undecided = torch.full((6,), -1, dtype=torch.int32, device=DEV)
        ops().sample_top(logits, rows, temp, u, ks, ps, out, undecided)
        want_und = torch.zeros(6, dtype=torch.int32)
        want = R.sample_top(logits.cpu(), rows.cpu(), temp.cpu(), u.cpu(), ks.cpu(), ps.cpu(),
                            torch.full((6,), -1, dtype=torch.int32), want_und)
        assert undecided.tolist() == want_und.tolist(), trial
        for i in range(6):
            if want_und[i] or out[i].item() == want[i].item():
                continue
            # The walk over hundreds of equal numbers in 32-bit may end one place from where the plain sampler's
            # (in 64-bit) ends: a neighbour in the sorted list is right too, anything else is not
            order = sorted(range(V), key=lambda j: (-float(logits[i, j]), j))
            at = order.index(want[i].item())
            assert out[i].item() in order[max(0, at - 1):at + 2], (trial, i, out[i].item(), want[i].item())
    assert out[0].item() == int(logits[0].argmax())      # top_k 1: the first of the largest
    # top_k 7 of a row whose largest value is taken by hundreds of tokens: one of the seven with the lowest indices
    if levels <= 7:
        first7 = [j for j in range(V) if float(logits[1, j]) == float(logits[1].max())][:7]
        assert out[1].item() in first7


def test_top_p_beyond_the_2048_largest_takes_the_whole_vocabulary():
    """Flat logits over a vocabulary of 50,257 with top-p 0.9999: among the 2,048 largest the cut falls on
    the last, so the subset kernel must leave the row undecided and the kernel over the whole sorted
    vocabulary decide it, as the reference falls back to its full path (sampler.rs:387-435).  Tokens
    outside the 2,048 largest are drawn, and each draw is the plain sampler's."""
    from denno_beta_amd.sampling import Sampler, SamplingParams, uniform
    V, n = 50257, 24
    g = torch.Generator().manual_seed(8)
    row = torch.randn(V, generator=g) * 0.05
    row[777] = 0.5                                      # one clear head of the list
    logits = row.repeat(n, 1).to(DEV).contiguous()
    rows = i32(list(range(n)))
    ps = torch.full((n,), 0.9999, device=DEV)
    ps[n - 1] = 1e-6                                    # so small a p that the head alone is kept: decided in the subset
    temp = torch.full((n,), 1.0, device=DEV)
    u = torch.tensor([uniform(3, i) for i in range(n)], device=DEV)
    out = torch.full((n,), -1, dtype=torch.int32, device=DEV)
    undecided = torch.full((n,), -1, dtype=torch.int32, device=DEV)
    ops().sample_top(logits, rows, temp, u, i32([0] * n), ps, out, undecided)
    assert undecided.tolist() == [1] * (n - 1) + [0] and out[n - 1].item() == 777
    ops().sample_full(logits, rows[:n - 1].contiguous(), temp, u, ps[:n - 1].contiguous(), out)
    top = set(row.topk(2048).indices.tolist())
    got = out.tolist()
    assert sum(1 for t in got[:n - 1] if t not in top) > n // 2, "draws never left the 2,048 largest"
    for i in range(0, n - 1, 4):
        tok, whole = SP.top_p_alone(row.tolist(), 1.0, 0.9999, float(u[i]))
        assert whole and tok == got[i], i
    # the second kernel launched behind the first with the first's own flags: the rows left undecided get the
    # same tokens, and the row that was decided keeps its token (it is not even looked at)
    again = torch.full((n,), -1, dtype=torch.int32, device=DEV)
    flags = torch.full((n,), -1, dtype=torch.int32, device=DEV)
    ops().sample_top(logits, rows, temp, u, i32([0] * n), ps, again, flags)
    ops().sample_full(logits, rows, temp, u, ps, again, only=flags)
    assert again.tolist() == got
    # the sampler does both steps, and with top_p = 1 takes the plain walk
    sp = SamplingParams(temperature=1.0, top_p=0.9999, seed=3)
    toks = Sampler(torch.device(DEV)).sample(logits[:4].clone(), [sp] * 4, [3] * 4, [0, 1, 2, 3], [[]] * 4)
    assert toks == got[:4]
    one = SamplingParams(temperature=1.0, top_p=1.0, seed=3)
    toks = Sampler(torch.device(DEV)).sample(logits[:4].clone(), [one] * 4, [3] * 4, [0, 1, 2, 3], [[]] * 4)
    assert toks == [SP.temperature_walk(row.tolist(), 1.0, uniform(3, i)) for i in range(4)]


@pytest.mark.parametrize("M,N,K", [(65, 1600, 1600), (128, 1600, 6400), (200, 1280, 5120), (256, 1024, 1024), (100, 96, 4096)])
@pytest.mark.parametrize("rows_in", ["packed", "rows"])
def test_a_product_whose_sum_the_next_norm_adds(M, N, K, rows_in):
    """A product into the stream may leave its shares' sums for the norm that reads the stream next: that norm's kernel
    adds them (shares in order, then the bias) and norms the updated rows.  The stream and the normed rows are, bit
    for bit, what the kernel that only adds the shares followed by the norm's own kernel give; the sum is right
    against 64 bits; where the product that adds into the stream itself shares K out the same way, its bits too."""
    o = ops()
    a, w, bias = rnd(M, K, seed=1, dtype=torch.bfloat16), rnd(N, K, seed=2, dtype=torch.bfloat16, scale=0.05), rnd(N, seed=3)
    gamma, beta = 1 + rnd(N, seed=4, scale=0.1), rnd(N, seed=5, scale=0.1)
    x0 = rnd(M, N, seed=6)
    wp = o.pack_matrix(w)
    ain = o.pack_matrix(a) if rows_in == "packed" else a
    assert o.linear_deferred_shares(M, wp) in (2, 4)
    part = o.linear_deferred(ain, wp)
    assert part.shape == (o.linear_deferred_shares(M, wp), M, N)
    for b in (bias, None):
        for packed_out in (False, True):
            if packed_out and N % 32 != 0:
                continue
            x = x0.clone()
            out = o.packed_rows(M, N, DEV) if packed_out else torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            o.layernorm_join(x, part, b, gamma, beta, 1e-5, out)
            x2 = o.join(part, b, x0.clone())
            out2 = o.layernorm(x2, gamma, beta, 1e-5, o.packed_rows(M, N, DEV) if packed_out else torch.empty(M, N, dtype=torch.bfloat16, device=DEV))
            assert torch.equal(x, x2)
            assert torch.equal(out.rows() if packed_out else out, out2.rows() if packed_out else out2)
    exact = (x0.double() + a.double() @ w.double().t() + bias.double()).float()
    x = o.join(part, bias, x0.clone())
    assert torch.allclose(x, exact, **TOL[torch.bfloat16])
    if K >= 4096:       # the product that adds into the stream itself cuts K into the same shares
        assert torch.equal(o.linear(ain, wp, bias, residual=x0.clone()), x)
    # 32-bit out of the norm, and what is not deferred
    out32 = torch.empty(M, N, device=DEV)
    x = x0.clone()
    o.layernorm_join(x, part, bias, gamma, None, 1e-5, out32)
    assert torch.equal(out32, o.layernorm(x, gamma, None, 1e-5, torch.empty(M, N, device=DEV)))
    assert o.linear_deferred_shares(64, wp) == 0 and o.linear_deferred_shares(300, wp) == 0
    assert o.linear_deferred_shares(M, o.pack_matrix(rnd(4800, K, seed=7, dtype=torch.bfloat16))) == 0


@pytest.mark.parametrize("M", [1, 5, 16, 40, 100])
@pytest.mark.parametrize("K", [8, 16, 24, 32, 40, 56])
def test_few_rows_product_with_an_inner_size_below_64(M, K):
    """The few-rows kernels load A in pieces of 16 bytes at fixed places of a row (a row's share of a pair of steps
    is 128 bytes); with an inner size below 64 some of those places lie beyond the row.  Such a piece is not loaded
    (its load goes to the start of the row, which is inside A) and counts as zeros."""
    o = ops()
    for N in (16, 96):
        a, w, bias = rnd(M, K, seed=1, dtype=torch.bfloat16), rnd(N, K, seed=2, dtype=torch.bfloat16, scale=0.3), rnd(N, seed=3)
        wp = o.pack_matrix(w)
        exact = (a.double() @ w.double().t() + bias.double()).float()
        out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        o.linear(a, wp, bias, out=out)
        assert torch.allclose(out.float(), exact, **TOL[torch.bfloat16]), (M, N, K)
        res = rnd(M, N, seed=4)
        want = res + exact
        o.linear(a, wp, bias, residual=res)
        assert torch.allclose(res, want, **TOL[torch.bfloat16]), (M, N, K)
