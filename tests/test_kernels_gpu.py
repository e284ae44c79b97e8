"""Each HIP kernel alone against a plain torch reference of the same operation, at
sizes other than the engine's (tails, widths that are no power of two)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def vslot(s):
    """Where the cache keeps slot s of a value column: bits 2 and 3 exchanged."""
    return (s & ~12) | ((s & 4) << 1) | ((s & 8) >> 1)


def kslot(keys, ps, hd, s):
    """Where the cache keeps the key of slot s of one (page, head): `keys` is that head's
    ps * hd elements; chunks of 16 dims lie together ([hd / 16][slot][16]) where hd is a
    multiple of 16, else a key's dims in a row.  A view of shape [hd / chunk, chunk]: assign
    `k.view(-1, chunk)` to it, or read it with `.reshape(hd)`."""
    kc = 16 if hd % 16 == 0 else hd
    return keys.view(hd // kc, ps, kc)[:, s, :]


def close(a, b, tol):
    """|a - b| <= tol * (1 + |b|), the reference's form (/root/reference/internal/ggml/q8_test.go:24-26)."""
    a, b = a.double().cpu(), b.double().cpu()
    bad = (a - b).abs() > tol * (1 + b.abs())
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} differ; worst {float((a - b).abs().max()):.3e}"


@pytest.mark.parametrize("n,d", [(1, 7), (5, 64), (3, 1027), (17, 4096)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(n, d, out_dtype):
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(n * 1000 + d)
    x = torch.randn(n, d, generator=g) * 3
    w = 1 + 0.1 * torch.randn(d, generator=g)
    eps = 1e-5
    ref = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps) * w.double()
    out = torch.empty(n, d, dtype=out_dtype, device=DEV)
    ops.rmsnorm(out, x.to(DEV), w.to(DEV), eps)
    close(out, ref, 1e-5 if out_dtype == torch.float32 else 1e-2)
    # gathered rows, bfloat16 weight
    rows = torch.tensor([n - 1, 0], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, d, dtype=out_dtype, device=DEV)
    wb = w.to(torch.bfloat16)
    ops.rmsnorm(out2, x.to(DEV), wb.to(DEV), eps, rows)
    ref2 = (x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps) * wb.double())[[n - 1, 0]]
    close(out2, ref2, 1e-5 if out_dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("n,d", [(1, 7), (5, 1027), (300, 72)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_rows_as_they_are(n, d, out_dtype):
    """What stands where a model has no norm: the rows, all or gathered, rounded once."""
    from hfee_amd.kernels import ops
    x = torch.randn(n, d, generator=torch.Generator().manual_seed(n + d)) * 3
    out = torch.empty(n, d, dtype=out_dtype, device=DEV)
    ops.cast_rows(out, x.to(DEV))
    assert torch.equal(out.cpu(), x.to(out_dtype))
    rows = torch.tensor([n - 1, 0, n // 2], dtype=torch.int32, device=DEV)
    out2 = torch.full((3, d), 7.0, dtype=out_dtype, device=DEV)
    ops.cast_rows(out2, x.to(DEV), rows)
    assert torch.equal(out2.cpu(), x[[n - 1, 0, n // 2]].to(out_dtype))


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (7, 33, 100), (64, 64, 16), (65, 130, 1027), (3, 172, 64), (200, 96, 172)])
@pytest.mark.parametrize("accumulate", [False, True])
def test_gemm_f32(M, N, K, accumulate):
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(M + 7 * N + 13 * K)
    x, w = torch.randn(M, K, generator=g), torch.randn(N, K, generator=g)
    c0 = torch.randn(M, N, generator=g)
    ref = x.double() @ w.double().t() + (c0.double() if accumulate else 0)
    out = c0.clone().to(DEV)
    ops.linear(out, x.to(DEV), w.to(DEV), accumulate=accumulate)
    mag = (x.abs().double() @ w.abs().double().t())        # error relative to the terms' size
    err = (out.double().cpu() - ref).abs()
    assert (err <= 1e-6 * (1 + mag)).all(), float((err / (1 + mag)).max())


def test_gemm_f32_rows_do_not_depend_on_the_batch():
    """Bit-equal results for a row whether it runs alone or among others."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    x, w = torch.randn(77, 300, generator=g).to(DEV), torch.randn(130, 300, generator=g).to(DEV)
    full = torch.empty(77, 130, device=DEV)
    ops.linear(full, x, w)
    for r in (0, 63, 64, 76):
        one = torch.empty(1, 130, device=DEV)
        ops.linear(one, x[r:r + 1].contiguous(), w)
        assert torch.equal(one[0], full[r])


@pytest.mark.parametrize("M,N,K", [(1, 16, 32), (1, 4096, 4096), (8, 100, 256), (16, 33, 1000), (17, 64, 128),
                                   (64, 172, 96), (5, 96, 172), (33, 320, 96), (3, 50, 20)])
@pytest.mark.parametrize("kernel", [1, 2])
@pytest.mark.parametrize("mode", ["bf16", "f32", "add"])
def test_gemm_bf16(M, N, K, kernel, mode):
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(M + 7 * N + 13 * K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    ref = x.double() @ w.double().t()
    if mode == "bf16":
        out = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
        ops.linear(out, x.to(DEV), w.to(DEV), kernel=kernel)
        tol = 1e-2
    elif mode == "f32":
        out = torch.zeros(M, N, dtype=torch.float32, device=DEV)
        ops.linear(out, x.to(DEV), w.to(DEV), kernel=kernel)
        tol = 1e-5
    else:
        c0 = torch.randn(M, N, generator=g)
        out = c0.clone().to(DEV)
        ops.linear(out, x.to(DEV), w.to(DEV), accumulate=True, kernel=kernel)
        ref = ref + c0.double()
        tol = 1e-5
    mag = x.abs().double() @ w.abs().double().t()
    err = (out.double().cpu() - ref).abs()
    assert (err <= tol * (1 + mag)).all(), float((err / (1 + mag)).max())


@pytest.mark.parametrize("M,N,K", [(65, 512, 2048), (128, 1024, 4096), (200, 520, 3000), (130, 256, 14336), (384, 640, 2112),
                                   (100, 2048, 2048), (512, 4096, 8192), (1000, 2048, 8256), (2048, 2048, 8192),
                                   (1024, 4096, 4096), (768, 4096, 4096), (512, 6144, 4096), (1024, 4096, 7680), (300, 4100, 8192), (200, 3080, 14336),
                                   (17, 4096, 4096), (40, 6144, 4096), (64, 4096, 14336), (33, 8192, 2112)])
@pytest.mark.parametrize("mode", ["bf16", "f32", "add"])
def test_gemm_bf16_with_k_cut_over_workgroups(M, N, K, mode):
    """Products with too few 128 x 128 tiles for the chip: given scratch, K is cut over up to
    eight times as many workgroups and a second kernel adds the partial products (K that is
    no multiple of the cut, M and N that are no multiples of a tile; the last three sizes: the
    cuts made by the kernel of 256 x 128 tiles, whole tiles of rows and not, a last cut that is
    shorter; then more by that kernel: two cuts of K = 4,096 and of 7,680, half a round of its tiles each; rows padded
    by a third to its tiles of 256 and weight rows that are no multiple of a tile, in three and in eight cuts;
    the last four: 17 to 64 rows over a large weight that lies as rows only, which the tiled kernel takes with its cuts);
    the same numbers as without scratch up to the order of the sums."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(M + 3 * N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    ref = x.double() @ w.double().t()
    mag = x.abs().double() @ w.abs().double().t()
    words = ops.linear_scratch(M, N, K)
    assert words >= 2 * M * N and words % (M * N) == 0
    scratch = torch.full((words,), float("nan"), dtype=torch.float32, device=DEV)
    c0 = torch.randn(M, N, generator=g)
    outs = []
    for kw in (dict(scratch=scratch), dict()):
        if mode == "add":
            out = c0.clone().to(DEV)
            ops.linear(out, x.to(DEV), w.to(DEV), accumulate=True, **kw)
            want, tol = ref + c0.double(), 1e-5
        else:
            out = torch.zeros(M, N, dtype=torch.bfloat16 if mode == "bf16" else torch.float32, device=DEV)
            ops.linear(out, x.to(DEV), w.to(DEV), **kw)
            want, tol = ref, 1e-2 if mode == "bf16" else 1e-5
        err = (out.double().cpu() - want).abs()
        assert (err <= tol * (1 + mag + want.abs())).all(), float((err / (1 + mag)).max())
        outs.append(out.double().cpu())
    # with and without the cut: the same sums in another order
    cut_err = (outs[0] - outs[1]).abs()
    order_tol = 1e-2 if mode == "bf16" else 2e-6
    assert (cut_err <= order_tol * (1 + mag + outs[1].abs())).all(), float((cut_err / (1 + mag)).max())
    assert ops.linear_scratch(16, N, K) == 0 and ops.linear_scratch(2048, 4096, K) == 0


@pytest.mark.parametrize("M,N,K", [(65, 512, 2048), (128, 1024, 4096), (200, 520, 3000), (130, 256, 14336), (384, 4096, 2112),
                                   (100, 2052, 2048), (100, 512, 1024), (70, 1001, 2048), (2048, 512, 1024), (40, 512, 2048),
                                   (90, 260, 2050), (512, 4096, 8192), (1000, 2048, 8256), (1024, 4096, 4096), (1024, 4096, 7680), (300, 4100, 8192), (160, 4096, 14336), (33, 4096, 4096), (64, 4096, 14336)])
@pytest.mark.parametrize("weight_dtype", [torch.float32, torch.bfloat16])
def test_product_that_adds_into_the_stream_and_goes_on_with_the_norm(M, N, K, weight_dtype):
    """The product that adds into the residual stream together with the norm of the new rows:
    where K is cut over workgroups one kernel adds the partial products and norms the row; in
    every other case (too few or too many rows, a short K, a width that the kernel does not
    take, unaligned operands, no scratch) it is the two launches.  Bit-equal to the product
    followed by the norm either way, and right against float64."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(M + 3 * N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(DEV)
    c0 = torch.randn(M, N, generator=g).to(DEV)
    nw = (1.0 + 0.2 * torch.randn(N, generator=g)).to(weight_dtype).to(DEV)
    eps = 1e-5
    words = ops.linear_scratch(M, N, K)
    for with_scratch in (True, False):
        kw = dict(scratch=torch.full((words,), float("nan"), dtype=torch.float32, device=DEV)) if words and with_scratch else {}
        two, normed_two = c0.clone(), torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
        ops.linear(two, x, w, accumulate=True, **kw)
        ops.rmsnorm(normed_two, two, nw, eps)
        one, normed_one = c0.clone(), torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.linear_add_norm(one, x, w, normed_one, nw, eps, **kw)
        assert torch.equal(one, two)
        assert torch.equal(normed_one, normed_two)
    ref = c0.double().cpu() + x.double().cpu() @ w.double().cpu().t()
    ref_normed = ref / torch.sqrt((ref * ref).mean(dim=1, keepdim=True) + eps) * nw.double().cpu()
    assert (normed_one.double().cpu() - ref_normed).abs().max() <= 1e-2 * (1 + ref_normed.abs().max())


@pytest.mark.parametrize("M,N,K", [(128, 128, 32), (300, 200, 520), (2048, 512, 1024), (129, 258, 72), (65, 130, 200),
                                   (257, 384, 64), (1000, 96, 4096), (600, 520, 192), (256, 512, 64),
                                   (513, 258, 320)])
@pytest.mark.parametrize("kernel", [0, 2, 3, 4, 5, 6, 7, 8])
def test_gemm_bf16_tiled_large(M, N, K, kernel):
    """The tiled kernels each alone (2: 128x128 tiles, 3: the simple one, 4: 256x256, 5:
    256x128, 6: 256x192, 7: 128x128 and 8: 128x192 loaded straight into LDS; 4 to 8 hand a K that is no multiple of 64 to 2) and the automatic
    choice, with every epilogue."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    ref = x.double() @ w.double().t()
    mag = x.abs().double() @ w.abs().double().t()
    out = torch.zeros(M, N, dtype=torch.float32, device=DEV)
    ops.linear(out, x.to(DEV), w.to(DEV), kernel=kernel)
    err = (out.double().cpu() - ref).abs()
    assert (err <= 1e-5 * (1 + mag)).all(), float((err / (1 + mag)).max())
    c0 = torch.randn(M, N, generator=g)
    acc = c0.clone().to(DEV)
    ops.linear(acc, x.to(DEV), w.to(DEV), accumulate=True, kernel=kernel)
    err = (acc.double().cpu() - ref - c0.double()).abs()
    assert (err <= 1e-5 * (1 + mag)).all()
    if kernel != 3:
        gated = torch.zeros(M, N // 2, dtype=torch.bfloat16, device=DEV)
        ops.linear(gated, x.to(DEV), w.to(DEV), gate=True, kernel=kernel)
        want = torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2]
        err = (gated.double().cpu() - want).abs()
        assert (err <= 2e-2 * (1 + mag[:, 0::2]) * (1 + mag[:, 1::2])).all()


def test_gemm_bf16_over_two_launches():
    """A product whose last round of large tiles would fill a part of the chip only goes
    to two kernels, split along the weight rows: every epilogue, the seam included."""
    from hfee_amd.kernels import ops
    M, N, K = 1024, 24704, 1024
    first, n1, second = ops.tiled_plan(M, N, K)
    assert second != 0 and 0 < n1 < N and n1 % 2 == 0, "this shape is meant to be split"
    g = torch.Generator().manual_seed(11)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    ref = x.float() @ w.float().t()                    # (the operands are exact in float32)
    mag = x.abs().float() @ w.abs().float().t()
    xd, wd = x.to(DEV), w.to(DEV)
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
    ops.linear(out, xd, wd)
    assert ((out.cpu() - ref).abs() <= 2e-5 * (1 + mag)).all()
    half = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear(half, xd, wd)
    assert ((half.float().cpu() - ref).abs() <= 1e-2 * (1 + mag)).all()
    c0 = torch.randn(M, N, generator=g)
    acc = c0.clone().to(DEV)
    ops.linear(acc, xd, wd, accumulate=True)
    assert ((acc.cpu() - ref - c0).abs() <= 2e-5 * (1 + mag)).all()
    gated = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.linear(gated, xd, wd, gate=True)
    want = torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2]
    assert ((gated.float().cpu() - want).abs() <= 2e-2 * (1 + mag[:, 0::2]) * (1 + mag[:, 1::2])).all()
    # the shapes of the benchmark's model: gate/up is split, the others are not
    assert ops.tiled_plan(2048, 28672, 4096)[2] != 0
    assert ops.tiled_plan(2048, 4096, 4096)[2] == 0 and ops.tiled_plan(2048, 4096, 14336)[2] == 0


def test_weights_in_tiles():
    """tile_weight lays [n, k] out in kilobytes of 16 rows x 32 columns, each in the order
    [column group of 8][row][8 columns], the tiles of 16 rows one after the other along k; n
    and k are filled up with zeros; rows() gives the weight back."""
    from hfee_amd.kernels import ops
    for n, k in ((16, 32), (48, 96), (50, 40), (7, 8), (33, 200)):
        w = torch.arange(n * k, dtype=torch.float32).reshape(n, k).to(torch.bfloat16).to(DEV)
        t = ops.tile_weight(w)
        nt, kt = (n + 15) // 16, (k + 31) // 32
        assert t.tiles.shape == (nt, kt, 512) and t.shape == (n, k) and t.row_stride == kt * 512
        assert torch.equal(t.rows(), w)
        flat = t.tiles.cpu()
        for row, col in ((0, 0), (n - 1, k - 1), (n // 2, k // 3), (min(17, n - 1), min(33, k - 1))):
            lane = 16 * ((col % 32) // 8) + row % 16              # the lane that holds it, and where in its 16 bytes
            assert flat[row // 16, col // 32, lane * 8 + col % 8] == w[row, col].cpu()
        assert float(flat.float().abs().sum()) == float(w.float().abs().sum())      # the filling is zeros


@pytest.mark.parametrize("M,N,K", [(1, 48, 64), (8, 344, 96), (16, 100, 256), (3, 16400, 1024), (16, 16500, 2048),
                                   (5, 17000, 4096), (2, 16390, 3072), (33, 200, 128), (64, 52, 1024),
                                   (7, 50, 40), (12, 107, 200), (4, 20, 8), (9, 6144, 512),
                                   (16, 5130, 1280), (3, 8000, 200),      # more workgroups than CUs, at most twice as many
                                   (5, 8300, 5120), (7, 8200, 8192)])      # the persistent kernel at K = 5,120 and 8,192
@pytest.mark.parametrize("epilogue", ["bf16", "f32", "add", "swiglu"])
@pytest.mark.parametrize("norm", [False, True])
def test_fused_decode_products(M, N, K, epilogue, norm):
    """The streaming and the persistent kernel with every epilogue, with and without
    the norm in front, against the unfused formulas."""
    from hfee_amd.kernels import ops
    if norm and M > 16:
        pytest.skip("the fused norm takes at most 16 rows")
    if epilogue == "swiglu" and N % 2:
        N += 1
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    if norm:
        xs = torch.randn(M + 3, K, generator=g) * 2
        nw = (1 + 0.1 * torch.randn(K, generator=g)).to(torch.bfloat16 if K % 64 else torch.float32)
        rows = torch.randperm(M + 3, generator=g)[:M].to(torch.int32)
        x = xs[rows.long()]
        h = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5) * nw.double()
    else:
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        h = x.double()
    ref = h @ w.double().t()
    mag = h.abs() @ w.double().abs().t()
    c0 = torch.randn(M, N, generator=g)
    if epilogue == "swiglu":
        ref = torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2]
        mag = (mag[:, 0::2] + 1) * (mag[:, 1::2] + 1)
        out = torch.zeros(M, N // 2, dtype=torch.bfloat16, device=DEV)
    elif epilogue == "add":
        ref = ref + c0.double()
        out = c0.clone().to(DEV)
    else:
        out = torch.zeros(M, N, dtype=torch.bfloat16 if epilogue == "bf16" else torch.float32, device=DEV)
    if norm:
        ops.linear_fused(out, xs.to(DEV), ops.tile_weight(w.to(DEV)), epilogue, norm_weight=nw.to(DEV), eps=1e-5, rows=rows.to(DEV), m=M)
    else:
        ops.linear_fused(out, x.to(DEV), ops.tile_weight(w.to(DEV)), epilogue)
    tol = 2e-2 if epilogue in ("bf16", "swiglu") or norm else 1e-5
    err = (out.double().cpu() - ref).abs()
    assert (err <= tol * (1 + mag)).all(), float((err / (1 + mag)).max())


@pytest.mark.parametrize("M,N,K", [(17, 48, 1024), (33, 200, 2048), (64, 344, 3072), (40, 6150, 4096), (64, 100, 1024),
                                   (48, 30, 2048), (64, 200, 512), (33, 520, 1536), (50, 344, 3584),
                                   (64, 136, 2304), (40, 72, 1280), (33, 200, 11008), (20, 136, 2304), (32, 72, 11008)])     # last slices of 256 and of 768 columns
@pytest.mark.parametrize("epilogue", ["bf16", "f32", "add", "swiglu", "emit", "scaled"])
def test_products_of_17_to_64_rows(M, N, K, epilogue):
    """The kernel that keeps the batch in LDS and cuts K over workgroups (17 to 64 rows,
    K a multiple of 256: slices of 1,024 and a last, shorter one) and the kernel that adds its
    slices up, with every epilogue, twice in a row on the same scratch, against the unfused formulas."""
    _products_of_17_to_64_rows(M, N, K, epilogue, 1)


@pytest.mark.parametrize("M,N,K", [(17, 48, 512), (33, 200, 1536), (64, 4100, 2048), (40, 6150, 4096), (64, 100, 1024),
                                   (50, 33000, 512), (24, 130, 2560)])
@pytest.mark.parametrize("epilogue", ["bf16", "f32", "add", "swiglu", "emit", "scaled"])
def test_products_of_17_to_64_rows_and_many_weight_rows(M, N, K, epilogue):
    """The kernel whose waves own 16 weight rows each over the whole of K (a multiple of 512),
    the batch passing through LDS 512 columns at a time: one round of a workgroup, several, and
    fewer row groups than a workgroup has waves; every epilogue; against the unfused formulas."""
    _products_of_17_to_64_rows(M, N, K, epilogue, 2)


def _products_of_17_to_64_rows(M, N, K, epilogue, kernel):
    from hfee_amd.kernels import ops
    if epilogue == "swiglu" and N % 2:
        N += 1
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    ref = x.double() @ w.double().t()
    mag = x.double().abs() @ w.double().abs().t()
    words = ops.mid_rows_scratch(M, N, K) if kernel == 1 else 0
    assert kernel == 2 or (words > 0) == (K > 1024)
    scratch = torch.full((max(words, 1),), float("nan"), dtype=torch.float32, device=DEV)
    kw = dict(scratch=scratch, force_mid_rows=kernel)
    c0 = torch.randn(M, N, generator=g)
    for _ in range(2):
        if epilogue == "swiglu":
            want = torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2]
            bound = 2e-2 * (mag[:, 0::2] + 1) * (mag[:, 1::2] + 1)
            out = torch.zeros(M, N // 2, dtype=torch.bfloat16, device=DEV)
            ops.linear_fused(out, x.to(DEV), ops.tile_weight(w.to(DEV)), "swiglu", **kw)
        elif epilogue in ("add", "emit"):
            want, bound = ref + c0.double(), 1e-5 * (1 + mag + c0.abs().double())
            out = c0.clone().to(DEV)
            emit = None
            if epilogue == "emit":
                nw = (1 + 0.1 * torch.randn(N, generator=g)).float()
                emitted = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
                shares = torch.zeros(((N + 15) // 16) * 64, dtype=torch.float32, device=DEV)
                emit = dict(weight=nw.to(DEV), out=emitted, shares=shares)
            ops.linear_fused(out, x.to(DEV), ops.tile_weight(w.to(DEV)), "add", emit=emit, **kw)
            if emit:
                close(emitted, want * nw.double(), 1e-2)
                got = shares.view(-1, 64)[:, :M].double().sum(0).cpu()
                assert torch.allclose(got, (want ** 2).sum(-1), rtol=1e-5)
        elif epilogue == "scaled":
            # x stands for an emitted tensor; the shares are made up so that every row has its own scale
            blocks = 5
            shares = torch.rand(blocks * 64, generator=g) + 0.5
            scale = 1 / torch.sqrt(shares.view(blocks, 64)[:, :M].double().sum(0) / K + 1e-5)
            want, bound = ref * scale[:, None], 2e-2 * (1 + mag * scale[:, None])
            out = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
            ops.linear_fused(out, x.to(DEV), ops.tile_weight(w.to(DEV)), "bf16", row_scale=dict(shares=shares.to(DEV), blocks=blocks, eps=1e-5), **kw)
        else:
            want, bound = ref, (2e-2 if epilogue == "bf16" else 1e-5) * (1 + mag)
            out = torch.zeros(M, N, dtype=torch.bfloat16 if epilogue == "bf16" else torch.float32, device=DEV)
            ops.linear_fused(out, x.to(DEV), ops.tile_weight(w.to(DEV)), epilogue, **kw)
        err = (out.double().cpu() - want).abs()
        assert (err <= bound).all(), float((err / bound).max())


@pytest.mark.parametrize("M,N,K,N2", [(1, 64, 96, 48), (8, 200, 256, 344), (16, 4096, 1024, 16400), (33, 104, 64, 72),
                                       (64, 520, 128, 100), (40, 200, 64, 16400), (64, 2048, 128, 17000), (17, 96, 64, 16384),
                                       (9, 5120, 320, 6000)])     # both products: more workgroups than CUs, at most twice as many
@pytest.mark.parametrize("epilogue2", ["bf16", "swiglu", "add"])
def test_norm_in_two_halves(M, N, K, N2, epilogue2):
    """A norm between two products, without a launch of its own: the product that adds
    into the residual stream also writes bfloat16(x_new * w_norm) and its shares of the
    rows' sums of squares; the next product reads that and scales its finished sums.
    Against residual add, RMSNorm and product done apart."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(M + 3 * N + 7 * K + N2)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    x0 = torch.randn(M, N, generator=g) * 2
    nw = (1 + 0.1 * torch.randn(N, generator=g)).to(torch.float32 if N % 64 else torch.bfloat16)
    w2 = (torch.randn(N2, N, generator=g) / math.sqrt(N)).to(torch.bfloat16)
    eps = 1e-5
    x1 = x0.double() + a.double() @ w1.double().t()
    h = x1 / torch.sqrt((x1 ** 2).mean(-1, keepdim=True) + eps) * nw.double()
    ref = h @ w2.double().t()
    mag = h.abs() @ w2.double().abs().t()
    # first product
    x = x0.clone().to(DEV)
    emitted = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    blocks = (N + 15) // 16
    shares = torch.full((blocks * 64,), float("nan"), dtype=torch.float32, device=DEV)
    ops.linear_fused(x, a.to(DEV), ops.tile_weight(w1.to(DEV)), "add", emit=dict(weight=nw.to(DEV), out=emitted, shares=shares))
    err = (x.double().cpu() - x1).abs()
    assert (err <= 1e-5 * (1 + x0.abs().double() + a.abs().double() @ w1.abs().double().t())).all()
    got_ss = shares.view(blocks, 64)[:, :M].double().sum(0).cpu()
    assert torch.allclose(got_ss, (x1 ** 2).sum(-1), rtol=1e-5)
    close(emitted, x1 * nw.double(), 1e-2)
    # second product
    scale = dict(shares=shares, blocks=blocks, eps=eps)
    if epilogue2 == "swiglu":
        out = torch.zeros(M, N2 // 2, dtype=torch.bfloat16, device=DEV)
        ref = torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2]
        mag = (mag[:, 0::2] + 1) * (mag[:, 1::2] + 1)
    elif epilogue2 == "add":
        c0 = torch.randn(M, N2, generator=g)
        out = c0.clone().to(DEV)
        ref = ref + c0.double()
    else:
        out = torch.zeros(M, N2, dtype=torch.bfloat16, device=DEV)
    ops.linear_fused(out, emitted, ops.tile_weight(w2.to(DEV)), epilogue2, row_scale=scale)
    err = (out.double().cpu() - ref).abs()
    assert (err <= 2e-2 * (1 + mag)).all(), float((err / (1 + mag)).max())


@pytest.mark.parametrize("H,K,hd,half,M", [(4, 2, 16, 8, 5), (3, 1, 32, 16, 16), (6, 3, 48, 8, 1), (2, 2, 128, 64, 9),
                                           (4, 2, 16, 8, 100), (6, 3, 48, 8, 130), (2, 2, 128, 64, 300), (5, 1, 64, 32, 65),
                                           (40, 8, 128, 64, 9)])      # 7,168 weight rows: more workgroups than CUs
@pytest.mark.parametrize("norm", [False, True])
def test_fused_qkv_rotation_and_cache_write(H, K, hd, half, M, norm):
    """Projection + rotation (pairs 2i, 2i+1) + cache write in one launch against the
    separate steps: the streaming kernels (up to 64 rows) and the tiled ones."""
    if norm and M > 16:
        pytest.skip("the fused norm takes at most 16 rows")
    _check_fused_qkv(H, K, hd, half, M, norm, 96)


@pytest.mark.parametrize("H,K,hd,half,M,d", [(4, 2, 16, 8, 100, 128), (2, 2, 128, 64, 300, 256), (6, 3, 48, 8, 130, 192),
                                             (16, 8, 128, 64, 1100, 512)])
def test_fused_qkv_through_the_tiled_kernels_with_whole_steps_of_k(H, K, hd, half, M, d):
    """The same epilogue behind the tiled kernels that take a K of whole steps of 64: one round of
    128 x 128 tiles loaded straight into LDS (the first three), the large tiles (the last)."""
    _check_fused_qkv(H, K, hd, half, M, False, d)


@pytest.mark.parametrize("kernel", [1, 2])
@pytest.mark.parametrize("H,K,hd,half,M,d", [(4, 2, 16, 8, 17, 2048), (5, 1, 64, 32, 64, 1024), (6, 3, 48, 8, 40, 3072)])
def test_fused_qkv_with_the_batch_in_lds(H, K, hd, half, M, d, kernel):
    """The same through the kernels for 17 to 64 rows: the one that cuts K over workgroups and
    the one for many weight rows."""
    from hfee_amd.kernels import ops
    N = (H + 2 * K) * hd
    scratch = torch.full((max(ops.mid_rows_scratch(M, N, d), 1),), float("nan"), dtype=torch.float32, device=DEV)
    _check_fused_qkv(H, K, hd, half, M, False, d, scratch=scratch, force_mid_rows=kernel)


def _check_fused_qkv(H, K, hd, half, M, norm, d, **kw):
    from plain_llama import plain_rope
    from hfee_amd.kernels import ops
    ps = 16
    g = torch.Generator().manual_seed(H + hd + M)
    N = (H + 2 * K) * hd
    w = (torch.randn(N, d, generator=g) / math.sqrt(d)).to(torch.bfloat16)
    pos = torch.randint(0, 60, (M,), generator=g).to(torch.int32)
    seg = torch.arange(M, dtype=torch.int32)
    tables = torch.stack([torch.randperm(M * 4, generator=g)[:4] for _ in range(M)]).to(torch.int32)   # each row its own pages
    tables = (tables // 4 * 0 + torch.arange(M * 4).reshape(M, 4)[:, torch.randperm(4, generator=g)]).to(torch.int32)
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) * 2 / (2 * half)))
    ang = torch.arange(64, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    if norm:
        x = torch.randn(M, d, generator=g) * 2
        nw = 1 + 0.1 * torch.randn(d, generator=g)
        h = x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-6) * nw.double()
    else:
        x = torch.randn(M, d, generator=g).to(torch.bfloat16)
        h = x.double()
    y = h @ w.double().t()
    q_ref = y[:, :H * hd].reshape(M, H, hd).clone()
    k_ref = y[:, H * hd:(H + K) * hd].reshape(M, K, hd).clone()
    v_ref = y[:, (H + K) * hd:].reshape(M, K, hd)
    q_ref[..., :2 * half] = plain_rope(q_ref[..., :2 * half], pos.tolist(), inv, "interleaved")
    k_ref[..., :2 * half] = plain_rope(k_ref[..., :2 * half], pos.tolist(), inv, "interleaved")
    layer = torch.zeros(M * 4, 2, K, ps * hd, dtype=torch.bfloat16, device=DEV)
    q_out = torch.zeros(M, H * hd, dtype=torch.bfloat16, device=DEV)
    ops.linear_fused(q_out, x.to(DEV), ops.tile_weight(w.to(DEV)) if M <= 64 else w.to(DEV), "qkv", norm_weight=nw.to(DEV) if norm else None, eps=1e-6,
                     qkv=dict(positions=pos.to(DEV), token_segment=seg.to(DEV), block_tables=tables.to(DEV), cos=cos, sin=sin,
                              cache_layer=layer, num_heads=H, kv_heads=K, head_dim=hd, page_size=ps), **kw)
    close(q_out, q_ref.reshape(M, H * hd), 2e-2)
    lay = layer.cpu()
    for m in range(M):
        p = int(pos[m])
        page, slot = int(tables[m, p // ps]), p % ps
        for kh in range(K):
            close(kslot(lay[page, 0, kh], ps, hd, slot).reshape(hd), k_ref[m, kh], 2e-2)
            close(lay[page, 1, kh].view(hd, ps)[:, vslot(slot)], v_ref[m, kh], 2e-2)
    assert int((lay != 0).sum()) <= M * 2 * K * hd, "nothing but the tokens' own slots is written"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_and_add(dtype):
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    gu = (torch.randn(9, 2 * 173, generator=g) * 4).to(dtype)
    out = torch.empty(9, 173, dtype=dtype, device=DEV)
    gud = gu.to(DEV)
    ops.swiglu(out, gud[:, :173], gud[:, 173:])
    ref = torch.nn.functional.silu(gu[:, :173].double()) * gu[:, 173:].double()
    close(out, ref, 1e-6 if dtype == torch.float32 else 1e-2)
    out2 = torch.empty(9, 173, dtype=dtype, device=DEV)          # gate and up in alternating columns
    ops.swiglu(out2, gud[:, 0::2], gud[:, 1::2])
    close(out2, torch.nn.functional.silu(gu[:, 0::2].double()) * gu[:, 1::2].double(), 1e-6 if dtype == torch.float32 else 1e-2)
    x = torch.randn(9, 173, generator=g)
    xd = x.clone().to(DEV)
    ops.residual_add(xd, out)
    close(xd, x.double() + out.double().cpu(), 1e-6)


def _activation(name, g):
    f = torch.nn.functional
    return {"silu": f.silu, "gelu": f.gelu, "gelu_tanh": lambda t: f.gelu(t, approximate="tanh"), "relu": f.relu}[name](g)


@pytest.mark.parametrize("activation", ["silu", "gelu_tanh", "gelu", "relu"])
def test_every_gate_kernel_with_every_activation(activation):
    """The gate's activation is an argument of every kernel that gates: the kernel of its own
    (both dtypes), the epilogue of each tiled kernel (128 x 128, 256 x 256, 256 x 128, 256 x 192 and
    the automatic choice), against the library's function in float64.  (The kernels for at most
    64 rows gate with the reference's activation alone; the feed-forward part sends another one
    through the kernel of its own.)  An unknown name is refused."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(11)
    for dtype in (torch.float32, torch.bfloat16):
        gu = (torch.randn(9, 2 * 173, generator=g) * 3).to(dtype)
        out = torch.empty(9, 173, dtype=dtype, device=DEV)
        ops.swiglu(out, gu.to(DEV)[:, 0::2], gu.to(DEV)[:, 1::2], activation=activation)
        close(out, _activation(activation, gu[:, 0::2].double()) * gu[:, 1::2].double(), 1e-6 if dtype == torch.float32 else 1e-2)

    def check(out, x, w, tol=2e-2):
        ref = x.double() @ w.double().t()
        mag = x.abs().double() @ w.abs().double().t()
        want = _activation(activation, ref[:, 0::2]) * ref[:, 1::2]
        err = (out.double().cpu() - want).abs()
        assert (err <= tol * (1 + mag[:, 0::2]) * (1 + mag[:, 1::2])).all(), float(err.max())
        # (a kernel that took another activation would be far off: the four differ by tenths around 1)
        assert activation == "silu" or not torch.allclose(want, torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2], atol=1e-2)

    for M, N, K in ((300, 520, 320), (513, 258, 64)):
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        w = (torch.randn(N, K, generator=g) * 2 / math.sqrt(K)).to(torch.bfloat16)
        for kernel in (0, 2, 4, 5, 6):
            out = torch.zeros(M, N // 2, dtype=torch.bfloat16, device=DEV)
            ops.linear(out, x.to(DEV), w.to(DEV), gate=True, kernel=kernel, activation=activation)
            check(out, x, w)
    with pytest.raises(ops.KernelError, match="unknown gate activation"):
        ops.swiglu(out, out, out, activation="swoosh")


@pytest.mark.parametrize("d", [97, 104, 2048 + 8, 4096])      # odd; a multiple of 8 (eight elements a thread); several workgroups a row
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(dtype, d):
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    table = torch.randn(321, d, generator=g).to(dtype)
    ids = torch.tensor([0, 320, 5, 5, 17], dtype=torch.int32)
    out = torch.empty(5, d, dtype=torch.float32, device=DEV)
    ops.embed(out, table.to(DEV), ids.to(DEV))
    assert torch.equal(out.cpu(), table[ids.long()].float())


@pytest.mark.parametrize("d,n,wdtype", [(4096, 8, torch.bfloat16), (2048, 1, torch.float32), (5128, 64, torch.bfloat16),
                                        (40, 3, torch.float32)])
def test_embed_with_the_first_half_of_the_norm_that_follows(d, n, wdtype):
    """The rows as float32, bfloat16(row * weight), and the rows' sums of squares in shares
    that a product with `row_scale` turns into the norm: the two halves together against the
    norm in one piece (the shares against a float64 sum)."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(d + n)
    table = torch.randn(97, d, generator=g).to(torch.bfloat16)
    weight = (1 + 0.2 * torch.randn(d, generator=g)).to(wdtype)
    ids = torch.randint(0, 97, (n,), generator=g, dtype=torch.int32)
    blocks = ops.embed_emit_blocks(d)
    out = torch.empty(n, d, dtype=torch.float32, device=DEV)
    emitted = torch.full((n, d), 7.0, dtype=torch.bfloat16, device=DEV)
    shares = torch.full((blocks * 64,), 7.0, dtype=torch.float32, device=DEV)
    assert ops.can_embed_emit(table, n) and not ops.can_embed_emit(table, 65) and not ops.can_embed_emit(table.float(), n)
    ops.embed(out, table.to(DEV), ids.to(DEV), emit=dict(weight=weight.to(DEV), out=emitted, shares=shares))
    rows = table[ids.long()].float()
    assert torch.equal(out.cpu(), rows)
    assert torch.equal(emitted.cpu(), (rows * weight.float()).to(torch.bfloat16))
    sums = shares.cpu().view(blocks, 64)[:, :n].double().sum(0)
    assert torch.allclose(sums, rows.double().pow(2).sum(1), rtol=1e-5)
    with pytest.raises(Exception, match="64 rows"):
        ops.embed(torch.empty(65, d, dtype=torch.float32, device=DEV), table.to(DEV),
                  torch.zeros(65, dtype=torch.int32, device=DEV),
                  emit=dict(weight=weight.to(DEV), out=torch.empty(65, d, dtype=torch.bfloat16, device=DEV), shares=shares))


def _paged(kv, page_size, pages_order):
    """kv: [T, K, hd] -> cache layer tensor with the pages in the given order, and the table."""
    T, K, hd = kv[0].shape
    nblocks = (T + page_size - 1) // page_size
    num_pages = max(pages_order) + 1
    layer = torch.zeros(num_pages, 2, K, page_size * hd, dtype=kv[0].dtype)
    layer += 7.0   # stale contents that must never show
    for b in range(nblocks):
        p = pages_order[b]
        for s in range(min(page_size, T - b * page_size)):
            t = b * page_size + s
            for h in range(K):
                kslot(layer[p, 0, h], page_size, hd, s)[:] = kv[0][t, h].view(-1, 16 if hd % 16 == 0 else hd)
                layer[p, 1, h].view(hd, page_size)[:, vslot(s)] = kv[1][t, h]
    return layer, torch.tensor([pages_order[:nblocks]], dtype=torch.int32)


@pytest.mark.parametrize("H,K,hd,T,window", [(4, 2, 16, 37, 0), (3, 1, 32, 100, 0), (6, 3, 48, 70, 0),
                                             (2, 2, 64, 33, 0), (4, 1, 128, 130, 0), (4, 2, 16, 90, 20),
                                             (5, 5, 80, 40, 0), (1, 1, 256, 35, 0), (12, 2, 64, 200, 0),
                                             (8, 1, 256, 70, 33),
                                             (3, 3, 128, 300, 0), (5, 5, 64, 200, 70), (2, 2, 48, 129, 0)])     # no two heads share keys
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_kernels(H, K, hd, T, window, dtype):
    """Plain kernel (both dtypes) and the matrix-core kernels (bfloat16) against
    the reference formula, on pages in scrambled order."""
    _check_attention(H, K, hd, T, window, dtype, 16)


@pytest.mark.parametrize("H,K,hd,T,window,ps", [(4, 1, 128, 130, 0, 32), (8, 2, 64, 150, 40, 64), (4, 1, 48, 300, 0, 128),
                                                (16, 2, 32, 97, 50, 32)])
def test_attention_kernels_with_larger_pages(H, K, hd, T, window, ps):
    """The same with pages of 32, 64 and 128 slots (a tile of 32 keys then lies in one page)."""
    _check_attention(H, K, hd, T, window, torch.bfloat16, ps)


def _check_attention(H, K, hd, T, window, dtype, ps):
    from plain_llama import plain_attention
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(H * 100 + hd + T)
    q = torch.randn(T, H, hd, generator=g).to(dtype)
    k = torch.randn(T, K, hd, generator=g).to(dtype)
    v = torch.randn(T, K, hd, generator=g).to(dtype)
    scale = 1 / math.sqrt(hd)
    ref = plain_attention(q, k, v, scale, window=window).reshape(T, H * hd)
    nblocks = (T + ps - 1) // ps
    order = torch.randperm(nblocks + 5, generator=g)[:nblocks].tolist()
    layer, table = _paged((k, v), ps, order)
    layer, table = layer.to(DEV), table.to(DEV)
    positions = torch.arange(T, dtype=torch.int32, device=DEV)
    seg = torch.zeros(T, dtype=torch.int32, device=DEV)
    qd = q.reshape(T, H * hd).to(DEV)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    out = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
    ops.attention_plain(out, qd, layer, positions, seg, table, H, K, hd, ps, scale, window)
    close(out, ref, tol)
    if dtype == torch.bfloat16:
        tiles = torch.tensor([(o, min(32, T - o), o, 0) for o in range(0, T, 32)], dtype=torch.int32, device=DEV)
        # the automatic choice, one wave per (tile, head), tiles shared in LDS, and (four heads or a
        # multiple to a KV head, head sizes up to 128) a row tile's keys in two halves
        for kernel in (0, 1, 2) + ((3,) if ops.attention_halves_fit(hd, H // K) else ()):
            out2 = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
            ops.attention_bf16_prefill(out2, qd, layer, tiles, table, H, K, hd, ps, scale, window, kernel=kernel)
            close(out2, ref, tol)
        # runs of up to four row tiles of a head that share its key tiles (taken where no two heads share keys)
        n_tiles = tiles.shape[0]
        runs = torch.tensor([(t, min(4, n_tiles - t)) for t in range(0, n_tiles, 4)], dtype=torch.int32, device=DEV)
        out2 = torch.full((T, H * hd), float("nan"), dtype=dtype, device=DEV)
        ops.attention_bf16_prefill(out2, qd, layer, tiles, table, H, K, hd, ps, scale, window, runs=runs)
        close(out2, ref, tol)
        # decode kernel: the last rows as single queries, with and without split keys
        # (joined by a second launch, and by the workgroup that finishes last: twice, the
        # second time on the counters that the first call left)
        counters = torch.zeros(3 * K, dtype=torch.int32, device=DEV)
        for splits, cnt in ((1, None), (3, None), (3, counters), (4, counters)):
            rows = torch.tensor([T - 1, T // 2, 0], dtype=torch.int32, device=DEV)
            out3 = torch.zeros(T, H * hd, dtype=dtype, device=DEV)
            partial = torch.zeros(3 * H * splits * (hd + 2), dtype=torch.float32, device=DEV)
            ops.attention_bf16_decode(out3, qd, layer, rows, rows.clone(), torch.zeros(3, dtype=torch.int32, device=DEV),
                                      table, H, K, hd, ps, scale, window, partial, splits, counters=cnt)
            close(out3[[T - 1, T // 2, 0]], ref[[T - 1, T // 2, 0]], tol)
            assert int(counters.abs().sum()) == 0


@pytest.mark.parametrize("H,K,hd,window", [(8, 2, 128, 0), (4, 1, 64, 0), (16, 2, 32, 300), (8, 1, 96, 0)])
def test_prefill_attention_with_a_row_tiles_keys_in_two_halves(H, K, hd, window):
    """One launch over portions of several sequences: a prompt of 1,500 tokens from its start (row
    tiles with 1 to 47 key tiles, odd and even counts, the odd tile with the first half), a
    portion of 70 rows deep in a context of 900, portions of 33, 2 and 1 rows; against the plain
    formula for every row, with one key far back scaled up in every sequence so that a half that
    is skipped, joined with a wrong weight or read from the other ring would show.  The host's
    choice for these row tiles is this kernel; for the row tiles of a portion deep in a long
    context, which are all alike, it is the other."""
    from plain_llama import plain_attention
    from hfee_amd.kernels import ops
    ps = 16
    g = torch.Generator().manual_seed(hd + H)
    lengths = [1500, 900, 33, 2, 1]            # keys of each sequence
    portions = [(0, 1500), (830, 70), (0, 33), (0, 2), (0, 1)]      # (first position, rows) that this step runs
    scale = 1 / math.sqrt(hd)
    blocks = [(n + ps - 1) // ps for n in lengths]
    order = torch.randperm(sum(blocks) + 3, generator=g).tolist()
    layer = torch.full((sum(blocks) + 3, 2, K, ps * hd), 7.0, dtype=torch.bfloat16)
    table = torch.zeros(len(lengths), max(blocks), dtype=torch.int32)
    qs, refs, tiles, row = [], [], [], 0
    for s, (n, (first, rows)) in enumerate(zip(lengths, portions)):
        q = torch.randn(n, H, hd, generator=g).to(torch.bfloat16)
        k = (torch.randn(n, K, hd, generator=g) * 0.7).to(torch.bfloat16)
        v = torch.randn(n, K, hd, generator=g).to(torch.bfloat16)
        far = n // 3
        k[far] = (q[first:first + rows].float().mean(0).view(K, H // K, hd).mean(1) * 6).to(torch.bfloat16)
        pages = order[:blocks[s]]
        order = order[blocks[s]:]
        one, _ = _paged((k, v), ps, pages)
        for p in pages:
            layer[p] = one[p]
        table[s, :blocks[s]] = torch.tensor(pages, dtype=torch.int32)
        refs.append(plain_attention(q, k, v, scale, window=window)[first:first + rows].reshape(rows, H * hd))
        qs.append(q[first:first + rows].reshape(rows, H * hd))
        for off in range(0, rows, 32):
            tiles.append((row + off, min(32, rows - off), first + off, s))
        row += rows
    q_all, ref = torch.cat(qs).to(DEV), torch.cat(refs)
    tiles = torch.tensor(tiles, dtype=torch.int32, device=DEV)
    outs = {}
    for kernel in (3, 0, 2):
        out = torch.full((row, H * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.attention_bf16_prefill(out, q_all, layer.to(DEV), tiles, table.to(DEV), H, K, hd, ps, scale, window, kernel=kernel)
        close(out, ref, 2e-2)
    assert ops.attention_halves_fit(hd, H // K)
    assert ops.prefill_attention_kernel(tiles.tolist(), window, K, H // K, hd) == 3
    deep = [(32 * i, 32, 30000 + 32 * i, 0) for i in range(64)]
    assert ops.prefill_attention_kernel(deep, 0, 8, 4, hd) == 0
    assert ops.prefill_attention_kernel([(0, 32, 0, 0)], 0, 8, 4, hd) == 0 and ops.prefill_attention_kernel([], 0, 8, 4, hd) == 0
    with pytest.raises(Exception, match="two halves"):
        ops.attention_bf16_prefill(out[:, :K * hd].contiguous(), q_all[:, :K * hd].contiguous(), layer.to(DEV), tiles, table.to(DEV), K, K, hd, ps,
                                   scale, window, kernel=3)           # (no two heads share keys: not this kernel's case)


@pytest.mark.parametrize("seed", range(12))
def test_prefill_attention_kernels_on_drawn_steps(seed):
    """Steps drawn at random: head sizes, heads to a KV head, page sizes, windows, and a mix of
    portions (some from a sequence's start, some deep in a context, some of a few rows) over
    pages in scrambled order with stale contents elsewhere.  Every matrix-core prefill kernel
    that takes the shape (the choice of the host among them) against the plain kernel, which is
    checked against the formula at small sizes."""
    import random
    from hfee_amd.kernels import ops
    rng = random.Random(900 + seed)
    hd = rng.choice([16, 32, 64, 64, 96, 128, 128, 48, 160])
    K = rng.choice([1, 2, 3])
    group = rng.choice([4, 4, 8, 1, 2, 12])
    H = K * group
    ps = rng.choice([16, 16, 32, 64])
    window = rng.choice([0, 0, 0, 40, 257])
    g = torch.Generator(device=DEV).manual_seed(seed)
    portions = []          # (keys before the portion, rows)
    for _ in range(rng.randint(1, 5)):
        kind = rng.random()
        before = 0 if kind < 0.4 else rng.randint(1, 3000)
        rows = rng.choice([1, 2, 31, 32, 33, rng.randint(2, 700)])
        portions.append((before, rows))
    blocks = [(b + r + ps - 1) // ps for b, r in portions]
    total_pages = sum(blocks) + 4
    cache = (torch.randn(total_pages, 2, K, ps * hd, generator=g, device=DEV) * 0.6).to(torch.bfloat16)
    order = torch.randperm(total_pages, generator=g, device=DEV).to(torch.int32)
    table = torch.zeros(len(portions), max(blocks), dtype=torch.int32, device=DEV)
    tiles, positions, seg, at = [], [], [], 0
    row = 0
    for s, ((before, rows), nb) in enumerate(zip(portions, blocks)):
        table[s, :nb] = order[at:at + nb]
        at += nb
        for off in range(0, rows, 32):
            tiles.append((row + off, min(32, rows - off), before + off, s))
        positions += list(range(before, before + rows))
        seg += [s] * rows
        row += rows
    q = (torch.randn(row, H * hd, generator=g, device=DEV) * 0.8).to(torch.bfloat16)
    positions = torch.tensor(positions, dtype=torch.int32, device=DEV)
    seg = torch.tensor(seg, dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(hd)
    ref = torch.zeros(row, H * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention_plain(ref, q, cache, positions, seg, table, H, K, hd, ps, scale, window)
    dev_tiles = torch.tensor(tiles, dtype=torch.int32, device=DEV)
    choice = ops.prefill_attention_kernel(tiles, window, K, group, hd)
    kernels = [1, 2] + ([3] if ops.attention_halves_fit(hd, group) else [])
    assert choice in (0, 3) and (choice == 0 or 3 in kernels)
    what = dict(hd=hd, K=K, group=group, ps=ps, window=window, portions=portions)
    for kernel in kernels:
        out = torch.full((row, H * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.attention_bf16_prefill(out, q, cache, dev_tiles, table, H, K, hd, ps, scale, window, kernel=kernel)
        worst = float((out.float() - ref.float()).abs().max())
        assert worst <= 2e-2 * (1 + float(ref.float().abs().max())), (kernel, worst, what)
    if group == 1:
        runs = torch.tensor(ops.attention_runs(tiles, hd), dtype=torch.int32, device=DEV)
        out = torch.full((row, H * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.attention_bf16_prefill(out, q, cache, dev_tiles, table, H, K, hd, ps, scale, window, runs=runs)
        assert float((out.float() - ref.float()).abs().max()) <= 2e-2 * (1 + float(ref.float().abs().max())), what


@pytest.mark.parametrize("B,splits", [(40, 1), (70, 2), (12, 3)])
def test_decode_attention_with_more_workgroups_than_cus(B, splits):
    """With more (segment, KV head, split) workgroups than the chip has CUs the decode kernel
    runs in the form that holds one tile's operands, two workgroups a CU; with fewer, in the
    form that loads one tile ahead.  Both against the plain attention kernel."""
    from hfee_amd.kernels import ops
    H, K, hd, ps, blocks = 16, 8, 64, 16, 20
    g = torch.Generator().manual_seed(B)
    cache = (torch.randn(B * blocks, 2, K, ps * hd, generator=g) * 0.5).to(torch.bfloat16).to(DEV)
    tables = torch.randperm(B * blocks, generator=g).to(torch.int32).reshape(B, blocks).to(DEV)
    q = torch.randn(B, H * hd, generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.randint(0, blocks * ps, (B,), generator=g).to(torch.int32)
    pos[0], pos[1] = 0, blocks * ps - 1
    pos = pos.to(DEV)
    order = torch.arange(B, dtype=torch.int32, device=DEV)
    want = torch.zeros(B, H * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention_plain(want, q, cache, pos, order, tables, H, K, hd, ps, 0.125, 0)
    out = torch.zeros(B, H * hd, dtype=torch.bfloat16, device=DEV)
    partial = torch.zeros(B * H * splits * (hd + 2), dtype=torch.float32, device=DEV)
    counters = torch.zeros(B * K, dtype=torch.int32, device=DEV)
    ops.attention_bf16_decode(out, q, cache, order, pos, order, tables, H, K, hd, ps, 0.125, 0, partial, splits,
                              counters=counters if splits > 1 else None)
    close(out, want, 2e-2)
    assert int(counters.abs().sum()) == 0


@pytest.mark.parametrize("splits", [1, 5])
def test_decode_attention_with_segments_in_order(splits):
    """Without the segments' rows and block-table rows (segment i is row i, has block table i)
    the decode kernel gives bit for bit what it gives with them spelled out."""
    from hfee_amd.kernels import ops
    H, K, hd, ps, B, blocks = 6, 2, 64, 16, 5, 12
    g = torch.Generator().manual_seed(splits)
    cache = torch.randn(B * blocks, 2, K, ps * hd, generator=g).to(torch.bfloat16).to(DEV)
    tables = torch.randperm(B * blocks, generator=g).to(torch.int32).reshape(B, blocks).to(DEV)
    q = torch.randn(B, H * hd, generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.tensor([0, 17, 100, 191, 64], dtype=torch.int32, device=DEV)
    order = torch.arange(B, dtype=torch.int32, device=DEV)
    outs = []
    for rows, tabs in ((order, order), (None, None), (None, order), (order, None)):
        out = torch.zeros(B, H * hd, dtype=torch.bfloat16, device=DEV)
        partial = torch.zeros(B * H * splits * (hd + 2), dtype=torch.float32, device=DEV)
        counters = torch.zeros(B * K, dtype=torch.int32, device=DEV)
        ops.attention_bf16_decode(out, q, cache, rows, pos, tabs, tables, H, K, hd, ps, 0.125, 0, partial, splits,
                                  counters=counters if splits > 1 else None)
        outs.append(out)
    assert float(outs[0].float().abs().sum()) > 0
    for o in outs[1:]:
        assert torch.equal(o, outs[0])


@pytest.mark.parametrize("pairing", ["half", "interleaved"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_cache_write(pairing, dtype):
    from plain_llama import plain_rope, plain_rope_frequencies
    from hfee_amd.kernels import ops
    from hfee_amd.parts.rotary import Rotary
    from hfee_amd.config.specs import PositionSpec, params
    H, K, hd, T, ps = 3, 2, 32, 21, 16
    rot = Rotary(PositionSpec("rope", params(head_dim=hd, rotary_dim=hd, theta=10000.0, scaling=None, pairing=pairing)))
    rot.prepare(64, DEV)
    g = torch.Generator().manual_seed(8)
    q = torch.randn(T, H * hd, generator=g).to(dtype)
    k = torch.randn(T, K * hd, generator=g).to(dtype)
    v = torch.randn(T, K * hd, generator=g).to(dtype)
    pos = torch.arange(5, 5 + T, dtype=torch.int32)
    inv = plain_rope_frequencies(hd, 10000.0)
    q_ref = plain_rope(q.reshape(T, H, hd), pos.tolist(), inv, pairing).reshape(T, H * hd)
    k_ref = plain_rope(k.reshape(T, K, hd), pos.tolist(), inv, pairing)
    layer = torch.zeros(4, 2, K, ps * hd, dtype=dtype, device=DEV)
    table = torch.tensor([[2, 0, 3, 1]], dtype=torch.int32, device=DEV)
    qd = q.to(DEV)
    ops.rope_cache_write(qd, k.to(DEV), v.to(DEV), pos.to(DEV), torch.zeros(T, dtype=torch.int32, device=DEV),
                         table, rot.cos, rot.sin, rot.pairing, layer, H, K, hd, ps, int(pos.max()))
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    close(qd, q_ref, tol)
    lay = layer.cpu()
    for t in range(T):
        p = int(pos[t])
        page, slot = [2, 0, 3, 1][p // ps], p % ps
        for h in range(K):
            close(kslot(lay[page, 0, h], ps, hd, slot).reshape(hd), k_ref[t, h], tol)
            assert torch.equal(lay[page, 1, h].view(hd, ps)[:, vslot(slot)], v[t].view(K, hd)[h])


@pytest.mark.parametrize("H,K,hd,rotary,d,n,portions", [(8, 2, 64, 64, 2048, 100, True), (4, 4, 128, 128, 4096, 65, False),
                                                        (6, 2, 48, 32, 2304, 130, True), (8, 2, 64, 0, 2048, 70, True),
                                                        (8, 2, 64, 64, 1024, 100, True), (8, 2, 64, 64, 2048, 40, True),
                                                        (32, 8, 128, 128, 4096, 512, True), (32, 8, 64, 64, 2048, 512, True),     # (two cuts by 256 x 128 tiles; one round of tiles, whole)
                                                        (32, 8, 128, 128, 4096, 40, False), (32, 8, 128, 128, 4096, 24, True)])   # (17 to 64 rows over a large weight as rows)
def test_rotation_that_adds_up_a_cut_product(H, K, hd, rotary, d, n, portions):
    """The q/k/v product of a portion cut along K, its partial products added up by the
    rotation kernel on its way to q and to the cache: bit-equal to the product (with the kernel
    that adds the cuts) followed by the rotation.  Part of the head rotated, nothing rotated;
    portions of prompts (values through groups of 16 tokens) and single tokens of many
    sequences; and the cases that are not cut (a short K, few rows): no cuts, nothing launched."""
    from hfee_amd.kernels import ops
    from hfee_amd.parts.rotary import Rotary
    from hfee_amd.config.specs import PositionSpec, params
    ps = 16
    g = torch.Generator().manual_seed(n + d + hd)
    width = (H + 2 * K) * hd
    x = torch.randn(n, d, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(width, d, generator=g) / math.sqrt(d)).to(torch.bfloat16).to(DEV)
    cos = sin = None
    if rotary:
        rot = Rotary(PositionSpec("rope", params(head_dim=hd, rotary_dim=rotary, theta=10000.0, scaling=None, pairing="interleaved")))
        rot.prepare(512, DEV)
        cos, sin = rot.cos, rot.sin
    if portions:      # two requests, portions of consecutive positions
        first = n // 2
        pos = torch.cat([torch.arange(32, 32 + first), torch.arange(5, 5 + n - first)]).to(torch.int32)
        seg = torch.cat([torch.zeros(first), torch.ones(n - first)]).to(torch.int32)
        per = max(16, (32 + first + ps - 1) // ps)
        tables = torch.stack([torch.randperm(per + 8, generator=g)[:per],
                              per + 8 + torch.randperm(per + 8, generator=g)[:per]]).to(torch.int32)
    else:             # one token each of n sequences
        pos = torch.randint(0, 200, (n,), generator=g).to(torch.int32)
        seg = torch.arange(n, dtype=torch.int32)
        tables = torch.stack([i * 13 + torch.randperm(13, generator=g) for i in range(n)]).to(torch.int32)
    pages = int(tables.max()) + 1
    pos, seg, tables = pos.to(DEV), seg.to(DEV), tables.to(DEV)
    words = ops.linear_scratch(n, width, d)
    scratch = torch.full((max(words, 1),), float("nan"), dtype=torch.float32, device=DEV)
    cuts = ops.linear_cuts(x, w, scratch if words else None)
    assert (cuts > 1) == (words > 0) and (cuts == 0 or words == cuts * n * width)
    if d <= 1024 or (n <= 64 and width * d < 16 << 20) or (d, n) == (2048, 512):
        assert cuts == 0
        return
    assert cuts > 1
    got_q = torch.full((n, width), float("nan"), dtype=torch.bfloat16, device=DEV)[:, :H * hd]
    got_cache = torch.zeros(pages, 2, K, ps * hd, dtype=torch.bfloat16, device=DEV)
    ops.rope_cache_write_cuts(got_q, scratch, cuts, pos, seg, tables, cos, sin, got_cache, H, K, hd, ps, int(pos.max()),
                              portions=portions)
    qkv = torch.zeros(n, width, dtype=torch.bfloat16, device=DEV)
    ops.linear(qkv, x, w, scratch=scratch)
    want_cache = torch.zeros_like(got_cache)
    ops.rope_cache_write(qkv[:, :H * hd], qkv[:, H * hd:(H + K) * hd], qkv[:, (H + K) * hd:], pos, seg, tables, cos, sin, 1,
                         want_cache, H, K, hd, ps, int(pos.max()), portions=portions)
    assert torch.equal(got_q, qkv[:, :H * hd])
    assert torch.equal(got_cache, want_cache)
    assert got_cache.abs().sum() > 0


@pytest.mark.parametrize("ps,H,K,hd", [(16, 3, 2, 32), (32, 3, 2, 32), (16, 13, 13, 128), (16, 5, 5, 256), (32, 20, 20, 80)])
def test_rope_cache_write_of_long_portions(ps, H, K, hd):
    """From 32 tokens on the values of 16 consecutive tokens are written together: whole
    32-byte runs of the transposed value layout where the 16 tokens fill 16 slots in a row of
    one page, element by element where they do not (a portion that starts inside a page, a
    group that spans two requests, the last, partial group).  Two requests with their own
    block tables; every key and value is found where the layout says.  With many KV heads
    (13 of 128, 5 of 256, 20 of 80) a group's heads are dealt over two or three workgroups,
    the last of them with fewer heads."""
    from hfee_amd.kernels import ops
    from hfee_amd.parts.rotary import Rotary
    from hfee_amd.config.specs import PositionSpec, params
    rot = Rotary(PositionSpec("rope", params(head_dim=hd, rotary_dim=hd, theta=10000.0, scaling=None, pairing="interleaved")))
    rot.prepare(256, DEV)
    # request 0: positions 32 .. 84 (starts on a page's edge); request 1: positions 5 .. 58 (does not)
    pos = torch.tensor(list(range(32, 85)) + list(range(5, 59)), dtype=torch.int32)
    seg = torch.tensor([0] * 53 + [1] * 54, dtype=torch.int32)
    T = pos.numel()
    g = torch.Generator().manual_seed(ps)
    q = torch.randn(T, H * hd, generator=g).to(torch.bfloat16)
    k = torch.randn(T, K * hd, generator=g).to(torch.bfloat16)
    v = torch.randn(T, K * hd, generator=g).to(torch.bfloat16)
    blocks = 96 // ps
    tables = torch.randperm(2 * blocks, generator=g).to(torch.int32).reshape(2, blocks)
    layer = torch.zeros(2 * blocks, 2, K, ps * hd, dtype=torch.bfloat16, device=DEV)
    one_by_one = torch.zeros_like(layer)
    args = (rot.cos, rot.sin, rot.pairing)
    ops.rope_cache_write(q.clone().to(DEV), k.to(DEV), v.to(DEV), pos.to(DEV), seg.to(DEV), tables.to(DEV), *args,
                         layer, H, K, hd, ps, int(pos.max()))
    for t in range(T):          # the same, a token a call: the path for short batches
        ops.rope_cache_write(q[t:t + 1].clone().to(DEV), k[t:t + 1].to(DEV), v[t:t + 1].to(DEV), pos[t:t + 1].to(DEV),
                             torch.zeros(1, dtype=torch.int32, device=DEV), tables[int(seg[t]):int(seg[t]) + 1].to(DEV),
                             *args, one_by_one, H, K, hd, ps, int(pos.max()))
    assert torch.equal(layer, one_by_one)
    # and told that the tokens are no portions (single tokens of many sequences): every token's own
    # workgroup writes its values; the same cache
    alone = torch.zeros_like(layer)
    ops.rope_cache_write(q.clone().to(DEV), k.to(DEV), v.to(DEV), pos.to(DEV), seg.to(DEV), tables.to(DEV), *args,
                         alone, H, K, hd, ps, int(pos.max()), portions=False)
    assert torch.equal(layer, alone)
    lay = layer.cpu()
    for t in range(T):
        p = int(pos[t])
        page, slot = int(tables[int(seg[t]), p // ps]), p % ps
        for h in range(K):
            assert torch.equal(lay[page, 1, h].view(hd, ps)[:, vslot(slot)], v[t].view(K, hd)[h])


def test_argmax_first_maximum_wins():
    from hfee_amd.kernels import ops
    logits = torch.zeros(3, 5000)
    logits[0, 4000] = 2.0
    logits[0, 17] = 2.0          # equal maxima: the first one
    logits[1] = -1.0
    logits[1, 4999] = -0.5
    logits[2, 0] = 1.0
    out = torch.zeros(3, dtype=torch.int32, device=DEV)
    ops.argmax(out, logits.to(DEV))
    assert out.tolist() == [17, 4999, 0]


@pytest.mark.parametrize("rows,V", [(1, 128256), (8, 128256), (3, 5000), (64, 33000), (5, 2048 * 3 + 5), (200, 9000)])
def test_argmax_over_several_workgroups_a_row(rows, V):
    """With partial results and counters the kernel spreads a row over workgroups and the last
    one to arrive takes the best: the first maximum still wins, across the stretches too;
    twice on the same counters; rows of -inf and NaN give id 0 as with one workgroup."""
    from hfee_amd.kernels import ops
    g = torch.Generator().manual_seed(rows + V)
    logits = torch.randn(rows, V, generator=g)
    top = logits.max().item() + 1
    for r in range(rows):
        a, b = sorted(torch.randint(0, V, (2,), generator=g).tolist())
        logits[r, a] = top
        logits[r, b] = top               # equal maxima, mostly in different stretches: the first one
    if rows > 2:
        logits[1] = float("-inf")
        logits[2] = float("nan")
    want = [int(torch.nonzero(row == row.max())[0]) if torch.isfinite(row.max()) else 0 for row in logits]
    dev = logits.to(DEV)
    partial = torch.full((rows * ops.ARGMAX_PARTS * 2,), float("nan"), device=DEV)
    counters = torch.zeros(rows, dtype=torch.int32, device=DEV)
    single = torch.zeros(rows, dtype=torch.int32, device=DEV)
    ops.argmax(single, dev)
    assert single.tolist() == want
    for _ in range(2):
        out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        ops.argmax(out, dev, partial, counters)
        assert out.tolist() == want
        assert int(counters.abs().sum()) == 0


@pytest.mark.parametrize("H,K,hd,ps,ctx", [(8, 2, 128, 16, 9000), (4, 1, 64, 16, 5000), (8, 2, 128, 32, 6000)])
def test_attention_over_long_contexts(H, K, hd, ps, ctx):
    """Thousands of keys: the block table no longer fits the 64 entries that a wave holds at
    a time, so the window moves several times per request.  One key far back is made to
    stand out for every query, so that a region that is skipped or read twice shows.  The
    matrix-core kernels (decode with several splits, prefill for the last rows) against the
    plain kernel, which is itself checked against the formula at small sizes."""
    from hfee_amd.kernels import ops
    B = 2
    g = torch.Generator(device=DEV).manual_seed(ctx + hd)
    blocks = (ctx + ps - 1) // ps
    cache = (torch.randn(B * blocks, 2, K, ps * hd, generator=g, device=DEV) * 0.5).to(torch.bfloat16)
    table = torch.randperm(B * blocks, generator=g, device=DEV).to(torch.int32).reshape(B, blocks)
    scale = 1 / math.sqrt(hd)
    # queries: the last 40 rows of request 0 (a prefill portion deep in the context) and one decode row of each request
    T = 40
    q = torch.randn(T + B, H * hd, generator=g, device=DEV).to(torch.bfloat16)
    far = [ctx // 3 + 5, ctx // 2 + 11]
    for b in range(B):      # key `far[b]` of every kv head points along the queries' mean direction, scaled up
        page, slot = int(table[b, far[b] // ps]), far[b] % ps
        for kh in range(K):
            rows = q[:T] if b == 0 else q[T + b:T + b + 1]
            mean = rows.float().view(-1, H, hd)[:, kh * (H // K)].mean(0)
            kslot(cache[page, 0, kh], ps, hd, slot)[:] = (mean / mean.norm() * 30).to(torch.bfloat16).view(-1, 16)
    positions = torch.cat([torch.arange(ctx - T, ctx), torch.tensor([ctx - 1, ctx - 8])]).to(torch.int32).to(DEV)
    seg = torch.tensor([0] * T + [0, 1], dtype=torch.int32, device=DEV)
    ref = torch.zeros(T + B, H * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention_plain(ref, q, cache, positions, seg, table, H, K, hd, ps, scale, 0)
    out = torch.zeros_like(ref)
    tiles = torch.tensor([(0, 32, ctx - T, 0), (32, T - 32, ctx - T + 32, 0)], dtype=torch.int32, device=DEV)
    for kernel in (1, 2) + ((3,) if ops.attention_halves_fit(hd, H // K) else ()):
        out.zero_()
        ops.attention_bf16_prefill(out, q, cache, tiles, table, H, K, hd, ps, scale, 0, kernel=kernel)
        assert (out[:T].float() - ref[:T].float()).abs().max() <= 2e-2 * (1 + ref[:T].float().abs().max())
    rows = torch.tensor([T, T + 1], dtype=torch.int32, device=DEV)
    for splits in (1, 5, 16):
        out.zero_()
        partial = torch.zeros(B * H * splits * (hd + 2), dtype=torch.float32, device=DEV)
        counters = torch.zeros(B * K, dtype=torch.int32, device=DEV)
        ops.attention_bf16_decode(out, q, cache, rows, positions[T:].contiguous(), torch.arange(B, dtype=torch.int32, device=DEV),
                                  table, H, K, hd, ps, scale, 0, partial, splits, counters=counters if splits > 1 else None)
        assert (out[T:].float() - ref[T:].float()).abs().max() <= 2e-2 * (1 + ref[T:].float().abs().max())
        assert int(counters.abs().sum()) == 0
    # the far key carries weight: without it the result would be another
    assert ref.float().abs().max() > 0.2


@pytest.mark.parametrize("H,K,hd", [(32, 8, 128), (32, 8, 64), (6, 1, 48)])
def test_split_key_join_on_buffers_that_are_used_again(H, K, hd):
    """The engine hands every layer and every step the same buffer for the splits' partial
    results and the same counters.  Three hundred calls in a row on one such pair, each with
    new queries, positions, page tables, batch sizes and split counts (both forms of the
    kernel: a tile ahead with up to one workgroup a CU, tile by tile beyond; splits that find
    no key at all), none waited for before the next is queued: every call's output is bit for
    bit the output of the same call with the splits joined by a second launch on buffers of
    its own, and the counters are zero after every batch of calls."""
    import random
    from hfee_amd.kernels import ops
    ps, blocks, b_max, s_max = 16, 80, 40, 8
    rng = random.Random(hd + K)
    g = torch.Generator(device=DEV).manual_seed(hd)
    cache = (torch.randn(b_max * blocks, 2, K, ps * hd, generator=g, device=DEV) * 0.5).to(torch.bfloat16)
    shared_partial = torch.full((b_max * H * s_max * (hd + 2),), 3.0e30, dtype=torch.float32, device=DEV)
    shared_counters = torch.zeros(b_max * K, dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(hd)
    done = 0
    while done < 300:
        group = []
        for _ in range(10):
            B = rng.choice([1, 1, 2, 3, 8, 8, 20, 40])
            splits = rng.randint(2, s_max)
            tables = torch.randperm(b_max * blocks, generator=g, device=DEV)[:B * blocks].to(torch.int32).reshape(B, blocks)
            q = torch.randn(B, H * hd, generator=g, device=DEV).to(torch.bfloat16)
            pos = torch.tensor([rng.choice([0, 5, 31, 32, 100, rng.randrange(blocks * ps), blocks * ps - 1])
                                for _ in range(B)], dtype=torch.int32, device=DEV)
            out = torch.zeros(B, H * hd, dtype=torch.bfloat16, device=DEV)
            ops.attention_bf16_decode(out, q, cache, None, pos, None, tables, H, K, hd, ps, scale, 0,
                                      shared_partial[:B * H * splits * (hd + 2)], splits,
                                      counters=shared_counters[:B * K])
            group.append((B, splits, tables, q, pos, out))
        assert int(shared_counters.abs().sum()) == 0, f"the counters are not back at zero after call {done + 10}"
        for B, splits, tables, q, pos, out in group:
            want = torch.zeros(B, H * hd, dtype=torch.bfloat16, device=DEV)
            partial = torch.zeros(B * H * splits * (hd + 2), dtype=torch.float32, device=DEV)
            ops.attention_bf16_decode(want, q, cache, None, pos, None, tables, H, K, hd, ps, scale, 0, partial, splits,
                                      counters=None)
            assert torch.equal(out, want), f"call {done}: batch {B}, {splits} splits, positions {pos.tolist()}"
            done += 1
    # and the join is the right one: against the plain kernel
    B, splits, tables, q, pos, out = group[-1]
    ref = torch.zeros_like(out)
    ops.attention_plain(ref, q, cache, pos, torch.arange(B, dtype=torch.int32, device=DEV), tables, H, K, hd, ps, scale, 0)
    close(out, ref, 2e-2)


def _poison():
    """Numbers that overflow: rows of 1e38 against weights of +-10."""
    return 1.0e38


@pytest.mark.parametrize("M", [1, 9, 40, 100, 300])
def test_only_finite_numbers_reach_the_cache(M):
    """Keys and values that overflow to infinity or NaN (here: projections of rows of 1e38) are
    written to the cache as finite numbers, by every kernel that writes there: the products
    with the q/k/v epilogue (streaming, batch in LDS, tiled) and the rotation kernels (a token
    a workgroup; values of 16 tokens together).  The attention kernels multiply keys that a
    query must not see by zero, and zero times infinity would be NaN for the page's next owner."""
    from hfee_amd.kernels import ops
    H, K, hd, half, d, ps = 4, 2, 32, 16, 1024, 16
    g = torch.Generator().manual_seed(M)
    N = (H + 2 * K) * hd
    w = (torch.randn(N, d, generator=g) * 10).to(torch.bfloat16).to(DEV)
    x = torch.randn(M, d, generator=g)
    x[::2] = _poison()
    x = x.to(torch.bfloat16).to(DEV)
    pos = torch.arange(M, dtype=torch.int32, device=DEV)
    seg = torch.zeros(M, dtype=torch.int32, device=DEV)
    nblocks = (M + ps - 1) // ps
    tables = torch.arange(nblocks, dtype=torch.int32, device=DEV).reshape(1, nblocks)
    ang = torch.arange(M + 1, dtype=torch.float64)[:, None] * (1.0 / 10000.0 ** (torch.arange(half) / half))[None, :]
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    plain_y = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
    ops.linear(plain_y, x, w)
    assert not torch.isfinite(plain_y.float()).all(), "the test's inputs must overflow"

    def fresh():
        return torch.zeros(nblocks, 2, K, ps * hd, dtype=torch.bfloat16, device=DEV)

    def check(layer, what):
        assert torch.isfinite(layer.float()).all(), f"{what}: a number that is not finite reached the cache"
        assert float(layer.float().abs().max()) > 1e37, f"{what}: the overflowing rows were not written at all"
    qkv = dict(positions=pos, token_segment=seg, block_tables=tables, cos=cos, sin=sin, num_heads=H, kv_heads=K,
               head_dim=hd, page_size=ps)
    q_out = torch.zeros(M, H * hd, dtype=torch.bfloat16, device=DEV)
    layer = fresh()
    ops.linear_fused(q_out, x, ops.tile_weight(w) if M <= 64 else w, "qkv", qkv=dict(qkv, cache_layer=layer))      # streaming up to 64 rows, tiled beyond
    check(layer, "q/k/v epilogue")
    if 16 < M <= 64:
        layer = fresh()
        scratch = torch.zeros(ops.mid_rows_scratch(M, N, d), dtype=torch.float32, device=DEV)
        ops.linear_fused(q_out, x, ops.tile_weight(w), "qkv", qkv=dict(qkv, cache_layer=layer), scratch=scratch, force_mid_rows=True)
        check(layer, "q/k/v epilogue with the batch in LDS")
    y = plain_y.clone()
    for pairing in (1, 0):          # the kernel for adjacent pairs (values of 16 tokens together from 32 rows on); the general one
        layer = fresh()
        ops.rope_cache_write(y[:, :H * hd], y[:, H * hd:(H + K) * hd], y[:, (H + K) * hd:], pos, seg, tables, cos, sin,
                             pairing, layer, H, K, hd, ps, M - 1)
        check(layer, f"rotation kernel, pairing {pairing}")
    y32 = plain_y.float()
    layer = torch.zeros(nblocks, 2, K, ps * hd, dtype=torch.float32, device=DEV)
    ops.rope_cache_write(y32[:, :H * hd], y32[:, H * hd:(H + K) * hd], y32[:, (H + K) * hd:], pos, seg, tables, cos, sin,
                         0, layer, H, K, hd, ps, M - 1)
    check(layer, "rotation kernel, 32-bit")


def test_a_cache_layer_of_more_than_four_gigabytes():
    """A pool that the free memory of this GPU suggests makes a cache layer of several gigabytes
    (128 requests of 8,192 tokens at the 8B sizes: 4.3 GB a layer).  Here a layer of 70,000 pages
    of 64 KiB (4.6 GB): sequences whose pages lie beyond the 2 GiB and 4 GiB marks, among low
    ones, in scrambled order.  Keys and values get there through the rotation kernel (portions)
    and through the decode product's epilogue (the sequences' last tokens); the prefill kernels
    that take a layer of this size (the ones that address the whole layer through one 32-bit
    offset are not chosen and refuse it when forced), the decode kernel with and without key
    splits and the plain kernel read them; all against the formula on the numbers themselves,
    with a far key scaled up so that a page read from the wrong place shows."""
    from plain_llama import plain_attention
    from hfee_amd.kernels import ops
    H, K, hd, ps, d = 32, 8, 128, 16, 256
    pages = 70_000
    free, _ = torch.cuda.mem_get_info()
    if free < 12 << 30:
        pytest.skip("needs 12 GB of free device memory")
    layer = torch.zeros(pages, 2, K, ps * hd, dtype=torch.bfloat16, device=DEV)
    assert layer.numel() * 2 > 1 << 32
    g = torch.Generator().manual_seed(70)
    scale = 1 / math.sqrt(hd)
    lengths = [701, 301, 91, 34]                 # the last token of each comes through the decode product
    portions = [(0, 700), (260, 40), (0, 90), (32, 1)]       # (first position, rows) of the prefill kernels' step
    blocks = [(n + ps - 1) // ps for n in lengths]
    # pages beyond 4 GiB (from 65,536 on), beyond 2 GiB (from 32,768 on), and low ones
    pool = torch.cat([65_540 + torch.randperm(4_400, generator=g)[:40], 32_770 + torch.randperm(1_000, generator=g)[:20],
                      torch.randperm(500, generator=g)[:16]])
    pool = pool[torch.randperm(pool.numel(), generator=g)].tolist()
    table = torch.zeros(len(lengths), max(blocks), dtype=torch.int32)
    w = (torch.randn((H + 2 * K) * hd, d, generator=g) / math.sqrt(d)).to(torch.bfloat16)
    w_tiles = ops.tile_weight(w.to(DEV))
    qs, ks, vs, xs = [], [], [], []
    for s, n in enumerate(lengths):
        mine, pool = pool[:blocks[s]], pool[blocks[s]:]
        table[s, :blocks[s]] = torch.tensor(mine, dtype=torch.int32)
        x_last = torch.randn(1, d, generator=g).to(torch.bfloat16)
        last = (x_last.double() @ w.double().t()).to(torch.bfloat16)        # what the product makes of the last token
        q = torch.cat([torch.randn(n - 1, H * hd, generator=g).to(torch.bfloat16), last[:, :H * hd]])
        k = torch.cat([(torch.randn(n - 1, K * hd, generator=g) * 0.7).to(torch.bfloat16), last[:, H * hd:(H + K) * hd]])
        v = torch.cat([torch.randn(n - 1, K * hd, generator=g).to(torch.bfloat16), last[:, (H + K) * hd:]])
        first, rows = portions[s]
        k[n // 3] = (q[first:first + rows].float().mean(0).view(K, H // K, hd).mean(1) * 5).reshape(K * hd).to(torch.bfloat16)
        qs.append(q), ks.append(k), vs.append(v), xs.append(x_last)
    assert int(table.max()) > 65_536
    table = table.to(DEV)
    # every token but the last: the rotation kernel without a rotation, one portion a launch and all in one
    k_all = torch.cat([k[:-1] for k in ks]).to(DEV)
    v_all = torch.cat([v[:-1] for v in vs]).to(DEV)
    pos_all = torch.cat([torch.arange(n - 1) for n in lengths]).to(torch.int32).to(DEV)
    seg_all = torch.cat([torch.full((n - 1,), s) for s, n in enumerate(lengths)]).to(torch.int32).to(DEV)
    ops.rope_cache_write(None, k_all, v_all, pos_all, seg_all, table, None, None, 1, layer, H, K, hd, ps, max(lengths))
    # the last tokens: the product of few rows with the cache write in its epilogue
    q_last = torch.full((len(lengths), H * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    last_pos = torch.tensor([n - 1 for n in lengths], dtype=torch.int32, device=DEV)
    order = torch.arange(len(lengths), dtype=torch.int32, device=DEV)
    ops.linear_fused(q_last, torch.cat(xs).to(DEV), w_tiles, "qkv",
                     qkv=dict(positions=last_pos, token_segment=order, block_tables=table, cos=None, sin=None,
                              cache_layer=layer, num_heads=H, kv_heads=K, head_dim=hd, page_size=ps))
    close(q_last, torch.stack([q[-1] for q in qs]), 2e-2)
    # what the formula says for every row of the step and for the last tokens
    full = [plain_attention(q.view(-1, H, hd), k.view(-1, K, hd), v.view(-1, K, hd), scale) for q, k, v in zip(qs, ks, vs)]
    ref_step = torch.cat([f[first:first + rows].reshape(rows, H * hd) for f, (first, rows) in zip(full, portions)])
    ref_last = torch.stack([f[-1].reshape(H * hd) for f in full])
    q_step = torch.cat([q[first:first + rows] for q, (first, rows) in zip(qs, portions)]).to(DEV)
    tiles, positions, seg, row = [], [], [], 0
    for s, (first, rows) in enumerate(portions):
        for off in range(0, rows, 32):
            tiles.append((row + off, min(32, rows - off), first + off, s))
        positions += list(range(first, first + rows))
        seg += [s] * rows
        row += rows
    dev_tiles = torch.tensor(tiles, dtype=torch.int32, device=DEV)
    for kernel in (0, 1, 2):
        out = torch.full((row, H * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.attention_bf16_prefill(out, q_step, layer, dev_tiles, table, H, K, hd, ps, scale, 0, kernel=kernel)
        close(out, ref_step, 2e-2)
    with pytest.raises(Exception, match="two halves"):
        ops.attention_bf16_prefill(out, q_step, layer, dev_tiles, table, H, K, hd, ps, scale, 0, kernel=3)
    out = torch.full((row, H * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.attention_plain(out, q_step, layer, torch.tensor(positions, dtype=torch.int32, device=DEV),
                        torch.tensor(seg, dtype=torch.int32, device=DEV), table, H, K, hd, ps, scale, 0)
    close(out, ref_step, 2e-2)
    counters = torch.zeros(len(lengths) * K, dtype=torch.int32, device=DEV)
    for splits in (1, 3):
        out = torch.full((len(lengths), H * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        partial = torch.zeros(len(lengths) * H * splits * (hd + 2), dtype=torch.float32, device=DEV)
        ops.attention_bf16_decode(out, q_last, layer, None, last_pos, None, table, H, K, hd, ps, scale, 0, partial, splits,
                                  counters=counters if splits > 1 else None)
        close(out, ref_last, 2e-2)
    del layer
    torch.cuda.empty_cache()
