"""Each kernel alone against a plain float64 reference of the same operation, at sizes
other than the models' (tails, widths that are no power of two)."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _ops():
    from dlgo_amd.kernels import ops
    return ops


def close(got, want, rel, what=""):
    got = got.double().cpu()
    want = want.double().cpu()
    scale = want.abs().max().item() + 1e-30
    err = (got - want).abs().max().item()
    assert err <= rel * scale, f"{what}: max error {err:.3e} against scale {scale:.3e} (allowed {rel:.1e} of it)"


DT = [(torch.float32, 2e-6, 1e-5), (torch.bfloat16, 1.0, 1.2e-2)]   # dtype, -, relative tolerance


@pytest.mark.parametrize("dtype,_,rel", DT)
def test_embed(dtype, _, rel):
    ops = _ops()
    g = torch.Generator().manual_seed(1)
    table = torch.randn(37, 24, generator=g).to(dtype).to(DEV)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 24, dtype=torch.float32, device=DEV)
    ops.embed(table, ids, out)
    assert torch.equal(out.cpu(), table.float().cpu()[ids.cpu().long()])


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("d", [4, 7, 96, 1024, 1500, 4096])
def test_rmsnorm(dtype, _, rel, d):
    ops = _ops()
    g = torch.Generator().manual_seed(d)
    x = (torch.randn(9, d, generator=g) * 3).to(DEV)
    w = (1 + 0.3 * torch.randn(d, generator=g)).to(DEV)
    eps = 1e-3
    out = torch.empty(9, d, dtype=dtype, device=DEV)
    ops.rmsnorm(x, w, eps, out)
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps) * w.double()
    close(out, want, rel, f"rmsnorm d={d}")
    rows = torch.tensor([8, 0, 3], dtype=torch.int32, device=DEV)
    out2 = torch.empty(3, d, dtype=dtype, device=DEV)
    ops.rmsnorm(x, w, eps, out2, rows)
    assert torch.equal(out2, out[rows.long()])


def test_rmsnorm_reference_vectors():
    """The reference's own vectors (ops/norm_test.go:8-52)."""
    ops = _ops()
    x = torch.tensor([[1., 2., 3., 4.]], device=DEV)
    out = torch.empty_like(x)
    ops.rmsnorm(x, torch.ones(4, device=DEV), 1e-5, out)
    close(out, x.double() / math.sqrt(7.5 + 1e-5), 1e-6)
    ones = torch.ones(1, 4, device=DEV)
    w = torch.tensor([2., 3., 4., 5.], device=DEV)
    ops.rmsnorm(ones, w, 1e-5, out)
    close(out, w.double()[None] / math.sqrt(1 + 1e-5), 1e-6)


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("rows,cols", [(1, 5), (9, 300), (3, 1030)])
def test_bias_add(dtype, _, rel, rows, cols):
    """y += b on rows in the run dtype and on float32 rows, also where the rows are a slice of wider ones
    (ops.AddBias, ops/ops.go; used by models/llm/forward.go:227-235)."""
    ops = _ops()
    g = torch.Generator().manual_seed(rows * cols)
    wide = torch.randn(rows, cols + 7, generator=g).to(dtype).to(DEV)
    b = torch.randn(cols, generator=g).to(DEV)
    y = wide[:, 3:3 + cols]
    before = wide.clone()
    ops.bias_add(y, b)
    close(y, before[:, 3:3 + cols].double() + b.double(), rel, "bias")
    assert torch.equal(wide[:, :3], before[:, :3]) and torch.equal(wide[:, 3 + cols:], before[:, 3 + cols:])
    res = torch.randn(rows, cols, generator=g).to(DEV)
    want = res.double() + b.double()
    ops.bias_add(res, b)
    close(res, want, 1e-6, "bias on float32 rows")
    with pytest.raises(ops.KernelError, match="does not fit"):
        ops.bias_add(res, b[:-1].contiguous())


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("heads,kv,hd", [(3, 1, 16), (5, 5, 80), (2, 1, 200)])
def test_head_rmsnorm(dtype, _, rel, heads, kv, hd):
    """Every q head and every k head normalised over its own elements with one weight vector of the head's size
    (models/llm/forward.go:236-244); the value heads behind them stay as they are."""
    ops = _ops()
    g = torch.Generator().manual_seed(heads * hd)
    t = 6
    qkv = (2 * torch.randn(t, (heads + 2 * kv) * hd, generator=g)).to(dtype).to(DEV)
    wq, wk = (1 + 0.3 * torch.randn(hd, generator=g)).to(DEV), (1 + 0.3 * torch.randn(hd, generator=g)).to(DEV)
    before = qkv.clone()
    eps = 1e-3
    ops.head_rmsnorm(qkv, 0, heads, hd, wq, eps)
    ops.head_rmsnorm(qkv, heads * hd, kv, hd, wk, eps)

    def plain_heads(x, n, w):
        x = x.double().reshape(t, n, hd)
        return (x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.double()).reshape(t, n * hd)
    close(qkv[:, :heads * hd], plain_heads(before[:, :heads * hd], heads, wq), rel, "q heads")
    close(qkv[:, heads * hd:(heads + kv) * hd], plain_heads(before[:, heads * hd:(heads + kv) * hd], kv, wk), rel, "k heads")
    assert torch.equal(qkv[:, (heads + kv) * hd:], before[:, (heads + kv) * hd:])
    with pytest.raises(ops.KernelError, match="do not fit"):
        ops.head_rmsnorm(qkv, hd, heads + 2 * kv, hd, wq, eps)


GEMM_SHAPES = [(200, 37, 96), (130, 5, 40), (64, 1, 64), (388, 130, 352), (34, 8, 160), (512, 257, 128), (6, 3, 8),
               (32790, 20, 2048),      # wide enough for the kernel that gives a block four groups of rows
               # few tokens and weight rows of whole kilobytes (2, 3, 6 and 16 KB in bfloat16): these go through LDS
               (100, 11, 1024), (8200, 16, 1536), (40, 3, 3072), (72, 1, 8192), (50, 8, 512),
               # rows of 5, 7 and 28 KB: a wave takes several kilobytes in turn
               (40, 9, 2560), (24, 16, 3584), (100, 4, 14336)]


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("kind", [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 14, 15, 16, 17, 18, 19])
@pytest.mark.parametrize("n,t,k", GEMM_SHAPES)
def test_gemm_store_and_accumulate(dtype, _, rel, kind, n, t, k):
    ops = _ops()
    if (kind == 1 and t > 8) or ((5 <= kind <= 11 or kind >= 15) and t > 64):
        pytest.skip("the streaming kernels take a few rows only")
    if dtype == torch.bfloat16 and k % 8:
        pytest.skip("bfloat16 rows come in 16-byte pieces")
    g = torch.Generator().manual_seed(n * 1000 + t)
    w = torch.randn(n, k, generator=g).to(dtype).to(DEV)
    x = torch.randn(t, k, generator=g).to(dtype).to(DEV)
    want = x.double() @ w.double().T
    out = torch.empty(t, n, dtype=dtype, device=DEV)
    ops.gemm(w, x, out, ops.EPI_STORE, kind)
    close(out, want, rel, f"gemm store kind={kind}")
    out32 = torch.empty(t, n, dtype=torch.float32, device=DEV)
    ops.gemm(w, x, out32, ops.EPI_STORE_F32, kind)
    close(out32, want, 1e-5 if dtype == torch.float32 else 1e-5, f"gemm store f32 kind={kind}")
    res = torch.randn(t, n, generator=g).to(DEV)
    res0 = res.clone()
    ops.gemm(w, x, res, ops.EPI_ACCUM_F32, kind)
    close(res, res0.double() + want, 1e-5, f"gemm accumulate kind={kind}")


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("kind", [20, 21, 22, 23])
@pytest.mark.parametrize("n,t,k", [(300, 130, 64), (517, 259, 128), (128, 128, 192), (1030, 77, 1024), (250, 700, 2048)])
def test_gemm_direct_to_lds(dtype, _, rel, kind, n, t, k):
    """The kernels that load tiles straight into LDS: one k tile, fewer tiles than stages, many; edges in n and t;
    every epilogue.  Row i of the weights is marked so that a row landing in another row's place shows."""
    ops = _ops()
    g = torch.Generator().manual_seed(n + 7 * t + k)
    w = torch.randn(n, k, generator=g)
    w[:, 0] += torch.arange(n) % 7
    w = w.to(dtype).to(DEV)
    x = torch.randn(t, k, generator=g)
    x[:, 0] += 1
    x = x.to(dtype).to(DEV)
    want = x.double() @ w.double().T
    out = torch.empty(t, n, dtype=dtype, device=DEV)
    ops.gemm(w, x, out, ops.EPI_STORE, kind)
    close(out, want, rel, f"gemm store kind={kind}")
    res = torch.randn(t, n, generator=g).to(DEV)
    res0 = res.clone()
    ops.gemm(w, x, res, ops.EPI_ACCUM_F32, kind)
    close(res, res0.double() + want, 1e-5, f"gemm accumulate kind={kind}")
    if n % 2 == 0:
        sw = torch.empty(t, n // 2, dtype=dtype, device=DEV)
        ops.gemm(w, x, sw, ops.EPI_SWIGLU, kind)
        gd, ud = want[:, 0::2], want[:, 1::2]
        close(sw, gd / (1 + torch.exp(-gd)) * ud, rel, f"swiglu kind={kind}")
    with pytest.raises(ops.KernelError):
        ops.gemm(w[:, :k - 8].contiguous(), x[:, :k - 8].contiguous(), out, ops.EPI_STORE, kind)


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("n,t,k,splits", [(130, 20, 512, 2), (64, 64, 2048, 5), (257, 33, 1024, 8), (2048, 64, 8192, 0), (300, 17, 4096, 0),
                                          (96, 40, 640, 3),
                                          # 96 and 80 tiles of output: between a half and a whole round of the chip, where
                                          # the number of runs is chosen by rounds times tiles of k (four and three here)
                                          (6144, 32, 4096, 0), (5120, 17, 3072, 0)])
def test_gemm_with_split_inner_size(dtype, _, rel, n, t, k, splits):
    """The inner size shared out over blocks whose sums are added in a fixed order: every epilogue, runs that do not
    divide the tiles evenly, and twice the same bits."""
    ops = _ops()
    if dtype == torch.float32:
        k //= 2         # the same number of 128-byte pieces
    g = torch.Generator().manual_seed(n + 7 * t + k)
    w = torch.randn(n, k, generator=g)
    w[:, 0] += torch.arange(n) % 7
    w = w.to(dtype).to(DEV)
    x = torch.randn(t, k, generator=g).to(dtype).to(DEV)
    want = x.double() @ w.double().T
    scratch = torch.full((ops.GEMM_SPLIT_FLOATS,), float("nan"), device=DEV)
    out = torch.empty(t, n, dtype=dtype, device=DEV)
    ops.gemm(w, x, out, ops.EPI_STORE, scratch=scratch, splits=splits)
    close(out, want, rel, "split store")
    again = torch.empty_like(out)
    ops.gemm(w, x, again, ops.EPI_STORE, scratch=scratch, splits=splits)
    assert torch.equal(out, again)
    res = torch.randn(t, n, generator=g).to(DEV)
    res0 = res.clone()
    ops.gemm(w, x, res, ops.EPI_ACCUM_F32, scratch=scratch, splits=splits)
    close(res, res0.double() + want, 1e-5, "split accumulate")
    out32 = torch.empty(t, n, dtype=torch.float32, device=DEV)
    ops.gemm(w, x, out32, ops.EPI_STORE_F32, scratch=scratch, splits=splits)
    close(out32, want, 1e-5, "split store f32")
    if n % 2 == 0:
        sw = torch.empty(t, n // 2, dtype=dtype, device=DEV)
        ops.gemm(w, x, sw, ops.EPI_SWIGLU, scratch=scratch, splits=splits)
        gd, ud = want[:, 0::2], want[:, 1::2]
        close(sw, gd / (1 + torch.exp(-gd)) * ud, rel, "split swiglu")
    if splits > 1:
        with pytest.raises(ops.KernelError):
            ops.gemm(w, x, out, ops.EPI_STORE, scratch=scratch[:splits * t * n - 1], splits=splits)
        with pytest.raises(ops.KernelError):
            ops.gemm(w, x, out, ops.EPI_STORE, splits=splits)


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("n,t,k,fused", [(2048, 8, 8192, True), (1024, 64, 4096, True), (4096, 33, 8192, True), (3072, 30, 2048, True),
                                         (2052, 8, 8192, True), (2048, 8, 512, False), (2050, 8, 8192, False), (2048, 200, 8192, True),
                                         (2048, 200, 2048, False), (2048, 600, 8192, False)])
def test_gemm_into_the_residual_that_leaves_the_next_norm(dtype, _, rel, n, t, k, fused):
    """A product whose inner size is shared out adds into the residual rows and leaves their RMSNorm beside them; where
    the product would not be split (or N does not suit) it does nothing and says so."""
    ops = _ops()
    if dtype == torch.float32:
        k //= 2
    g = torch.Generator().manual_seed(n + t)
    w = (0.05 * torch.randn(n, k, generator=g)).to(dtype).to(DEV)
    x = torch.randn(t, k, generator=g).to(dtype).to(DEV)
    res = (torch.randn(t, n, generator=g) * (1 + torch.arange(t)[:, None] % 3)).to(DEV)
    nw = (1 + 0.3 * torch.randn(n, generator=g)).to(DEV)
    eps = 1e-3
    scratch = torch.full((ops.GEMM_SPLIT_FLOATS,), float("nan"), device=DEV)
    normed = torch.full((t, n), float("nan"), dtype=dtype, device=DEV)
    res0 = res.clone()
    did = ops.gemm_accum_then_norm(w, x, res, scratch, nw, eps, normed)
    assert did == fused
    if not did:
        assert torch.equal(res, res0) and torch.isnan(normed.float()).all()
        return
    want = res0.double() + x.double() @ w.double().T
    close(res, want, 1e-5, "residual")
    rd = res.double()                                  # the norm of the rows as the kernel left them
    close(normed, rd / torch.sqrt((rd * rd).mean(-1, keepdim=True) + eps) * nw.double(), 1e-5 if dtype == torch.float32 else 8e-3, "norm")
    # the same bits as the separate way: split product, then the norm kernel
    res2 = res0.clone()
    ops.gemm(w, x, res2, ops.EPI_ACCUM_F32, scratch=scratch)
    assert torch.equal(res2, res)
    normed2 = torch.empty_like(normed)
    ops.rmsnorm(res2, nw, eps, normed2)
    close(normed2, normed.double(), 1e-6 if dtype == torch.float32 else 8e-3, "norm kernel")


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("kind", [0, 1, 2, 3, 4, 5])
@pytest.mark.parametrize("f,t,k", [(160, 5, 64), (352, 70, 128), (9, 2, 16), (1030, 200, 72), (40, 33, 2056), (8200, 64, 256), (16401, 9, 2048), (20, 6, 5120)])
def test_gemm_swiglu(dtype, _, rel, kind, f, t, k):
    ops = _ops()
    if (kind == 1 and t > 8) or (kind == 5 and t > 64):
        pytest.skip("the streaming kernels take a few rows only")
    g = torch.Generator().manual_seed(f + t)
    gate = torch.randn(f, k, generator=g).to(dtype)
    up = torch.randn(f, k, generator=g).to(dtype)
    x = (torch.randn(t, k, generator=g) * 0.5).to(dtype).to(DEV)
    w = torch.stack([gate, up], dim=1).reshape(2 * f, k).contiguous().to(DEV)
    out = torch.empty(t, f, dtype=dtype, device=DEV)
    ops.gemm(w, x, out, ops.EPI_SWIGLU, kind)
    gd, ud = x.double().cpu() @ gate.double().T, x.double().cpu() @ up.double().T
    want = gd / (1 + torch.exp(-gd)) * ud
    close(out, want, rel, f"swiglu kind={kind}")


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("kind", [0, 10, 11])
@pytest.mark.parametrize("n,t,k", [(200, 8, 96), (130, 1, 40), (96, 17, 2048), (388, 64, 352), (34, 48, 160), (32780, 3, 2048),
                                   (8204, 9, 1024), (72, 16, 1536), (100, 1, 4096), (50, 7, 3072), (40, 5, 512)])
def test_gemm_with_fused_rmsnorm(dtype, _, rel, n, t, k, kind):
    """The product with the normed rows that are never written, in every epilogue, by both kernels (the weights read
    straight into registers; the weights going through LDS in whole 1 KB runs, for the shapes that kernel takes)."""
    ops = _ops()
    g = torch.Generator().manual_seed(n + t)
    w = (0.5 * torch.randn(n, k, generator=g)).to(dtype).to(DEV)
    x = (2 * torch.randn(t, k, generator=g)).to(DEV)
    nw = (1 + 0.3 * torch.randn(k, generator=g)).to(DEV)
    eps = 1e-2
    xd = x.double()
    xn = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps) * nw.double()
    want = xn @ w.double().T
    tol = 1e-5 if dtype == torch.float32 else 1.5e-2
    out = torch.empty(t, n, dtype=dtype, device=DEV)
    ops.gemm_rmsnorm(w, x, nw, eps, out, kind=kind)
    close(out, want, tol, "store")
    out32 = torch.empty(t, n, device=DEV)
    ops.gemm_rmsnorm(w, x, nw, eps, out32, ops.EPI_STORE_F32, kind=kind)
    close(out32, want, tol, "store f32")
    res = torch.randn(t, n, generator=g).to(DEV)
    res0 = res.clone()
    ops.gemm_rmsnorm(w, x, nw, eps, res, ops.EPI_ACCUM_F32, kind=kind)
    close(res, res0.double() + want, tol, "accumulate")
    hid = torch.empty(t, n // 2, dtype=dtype, device=DEV)
    ops.gemm_rmsnorm(w, x, nw, eps, hid, ops.EPI_SWIGLU, kind=kind)
    gd, ud = want[:, 0::2], want[:, 1::2]
    close(hid, gd / (1 + torch.exp(-gd)) * ud, tol * 2, "swiglu")


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("n1,k1,n2,t", [(1024, 1024, 200, 8), (1536, 2048, 132, 1), (2048, 1536, 96, 16), (3072, 1024, 64, 5), (4096, 4096, 40, 3),
                                        (1024, 8192, 64, 8), (1024, 5120, 32, 3), (2048, 14336, 48, 16), (1024, 2560, 32, 2), (1024, 3584, 32, 9)])
def test_norm_left_in_parts_and_applied_by_the_next_product(dtype, _, rel, n1, k1, n2, t):
    """A product that adds into the residual rows leaves the rows times the norm's weights and the sums of squares in
    shares; the next product multiplies its sums by the factor.  Together: residual += x W1^T; out = rmsnorm(residual) W2^T.
    The widths are chosen so that both weights have rows of whole KB in both dtypes (n1 is the second one's inner size);
    the first one's rows go up to 28 KB, which a wave takes in several turns."""
    ops = _ops()
    es = torch.tensor([], dtype=dtype).element_size()
    n1, k1 = n1 * 2 // es, k1 * 2 // es          # the sizes are given for 2-byte elements
    g = torch.Generator().manual_seed(n1 + t)
    w1 = (0.3 * torch.randn(n1, k1, generator=g)).to(dtype).to(DEV)
    w2 = (0.5 * torch.randn(n2, n1, generator=g)).to(dtype).to(DEV)
    x = torch.randn(t, k1, generator=g).to(dtype).to(DEV)
    res = (3 * torch.randn(t, n1, generator=g)).to(DEV)
    nw = (1 + 0.3 * torch.randn(n1, generator=g)).to(DEV)
    eps = 1e-2
    assert ops.streams_few_rows(w1, t, ops.ROLE_LEAVES_NORM) and ops.streams_few_rows(w2, t, ops.ROLE_APPLIES_NORM)
    assert not ops.streams_few_rows(w2[:, :n1 - 8], t) and not ops.streams_few_rows(w1, 17)
    new_res = res.double() + x.double() @ w1.double().T
    xn = new_res / torch.sqrt((new_res * new_res).mean(-1, keepdim=True) + eps) * nw.double()
    want = xn @ w2.double().T
    tol = 1e-5 if dtype == torch.float32 else 1.5e-2
    unscaled = torch.empty(t, n1, dtype=dtype, device=DEV)
    parts = torch.full((16 * ((n1 + 7) // 8) + 7,), float("nan"), device=DEV)
    left = ops.gemm_accum_leave_norm(w1, x, res, nw, eps, unscaled, parts)
    close(res, new_res, 1e-5, "residual")
    # a share for every 16 columns, or for every 8 where blocks of 16 weight rows would leave compute units idle
    assert left.n_parts in ((n1 + 15) // 16, (n1 + 7) // 8) and left.width == n1
    close(left.parts[:t * left.n_parts].view(t, -1).sum(-1), (new_res * new_res).sum(-1), 1e-5, "sum of squares")
    close(unscaled, new_res * nw.double(), 1e-6 if dtype == torch.float32 else 8e-3, "unscaled rows")
    for epi, shape, odt in ((ops.EPI_STORE, (t, n2), dtype), (ops.EPI_STORE_F32, (t, n2), torch.float32)):
        out = torch.empty(shape, dtype=odt, device=DEV)
        ops.gemm_scaled(w2, left, out, epi)
        close(out, want, tol, f"epilogue {epi}")
    acc = torch.randn(t, n2, generator=g).to(DEV)
    acc0 = acc.clone()
    ops.gemm_scaled(w2, left, acc, ops.EPI_ACCUM_F32)
    close(acc, acc0.double() + want, tol, "accumulate")
    hid = torch.empty(t, n2 // 2, dtype=dtype, device=DEV)
    ops.gemm_scaled(w2, left, hid, ops.EPI_SWIGLU)
    gd, ud = want[:, 0::2], want[:, 1::2]
    close(hid, gd / (1 + torch.exp(-gd)) * ud, tol * 2, "swiglu")
    with pytest.raises(ops.KernelError, match="whole KB"):
        ops.gemm_scaled(w2[:, :n1 - 8].contiguous(), ops.UnscaledNorm(unscaled[:, :n1 - 8].contiguous(), parts, left.n_parts, n1 - 8, eps),
                        torch.empty(t, n2, dtype=dtype, device=DEV))


@pytest.mark.parametrize("n1", [5120, 8192])
def test_norm_hand_off_refuses_widths_beyond_its_shares(n1):
    """The streamed products keep at most 256 shares of a row's sum of squares, one for every 16 columns: a normed width
    beyond 4,096 is not theirs, as the product that leaves the norm or as the one that applies it, and the predicates
    that the parts ask say so, so that such a model takes the norm kernel instead of an error in its first decode step."""
    ops = _ops()
    w1 = torch.zeros(n1, 1024, dtype=torch.bfloat16, device=DEV)        # leaves a norm over n1 columns
    w2 = torch.zeros(64, n1, dtype=torch.bfloat16, device=DEV)          # would apply it
    for t in (1, 8, 16):
        assert ops.streams_few_rows(w1, t) and ops.streams_few_rows(w2, t)             # the plain products are streamed
        assert not ops.streams_few_rows(w1, t, ops.ROLE_LEAVES_NORM) and not ops.can_leave_unscaled(w1, t)
        assert not ops.streams_few_rows(w2, t, ops.ROLE_APPLIES_NORM) and not ops.can_take_unscaled(w2, t)
    narrow = torch.zeros(4096, 1024, dtype=torch.bfloat16, device=DEV)
    assert ops.can_leave_unscaled(narrow, 8) and ops.can_take_unscaled(torch.zeros(64, 4096, dtype=torch.bfloat16, device=DEV), 8)
    t = 4
    with pytest.raises(ops.KernelError, match="width of up to 4096"):
        ops.gemm_accum_leave_norm(w1, torch.zeros(t, 1024, dtype=torch.bfloat16, device=DEV), torch.zeros(t, n1, device=DEV),
                                  torch.ones(n1, device=DEV), 1e-5, torch.empty(t, n1, dtype=torch.bfloat16, device=DEV),
                                  torch.empty(t * (n1 // 16), device=DEV))


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("n1,k1,n2,t", [(256, 128, 136, 17), (2048, 512, 384, 300), (1024, 2048, 1030, 130), (96, 64, 64, 64),
                                        (4096, 256, 264, 257), (512, 8192, 128, 520)])
def test_norm_left_and_applied_by_tiled_products(dtype, _, rel, n1, k1, n2, t):
    """The same hand-off for steps of many rows: the tiled product that adds into the residual leaves the rows times
    the norm's weights and a share of the sums of squares for every 32 columns; the next tiled product multiplies its
    sums by each row's factor.  residual += x W1^T; out = rmsnorm(residual) W2^T, plain and through SwiGLU."""
    ops = _ops()
    g = torch.Generator().manual_seed(n1 + t)
    w1 = (0.3 * torch.randn(n1, k1, generator=g)).to(dtype).to(DEV)
    w2 = (0.5 * torch.randn(n2, n1, generator=g)).to(dtype).to(DEV)
    x = torch.randn(t, k1, generator=g).to(dtype).to(DEV)
    res = (3 * torch.randn(t, n1, generator=g)).to(DEV)
    nw = (1 + 0.3 * torch.randn(n1, generator=g)).to(DEV)
    eps = 1e-2
    if not (ops.can_leave_unscaled(w1, t) and ops.can_take_unscaled(w2, t)):
        pytest.skip("a product of this shape has its k shared out: its ordered sum writes the norm itself")
    assert not ops.can_leave_unscaled(w1[:n1 - 8], t) and not ops.can_take_unscaled(w2[:, :n1 - 8], t)
    new_res = res.double() + x.double() @ w1.double().T
    xn = new_res / torch.sqrt((new_res * new_res).mean(-1, keepdim=True) + eps) * nw.double()
    want = xn @ w2.double().T
    tol = 1e-5 if dtype == torch.float32 else 1.5e-2
    unscaled = torch.empty(t, n1, dtype=dtype, device=DEV)
    parts = torch.full((t * ((n1 + 15) // 16) + 7,), float("nan"), device=DEV)
    left = ops.gemm_accum_leave_norm(w1, x, res, nw, eps, unscaled, parts)
    close(res, new_res, 1e-5, "residual")
    assert left.n_parts == n1 // 32 and left.width == n1
    close(left.parts[:t * left.n_parts].view(t, -1).sum(-1), (new_res * new_res).sum(-1), 1e-5, "sum of squares")
    close(unscaled, new_res * nw.double(), 1e-5 if dtype == torch.float32 else 8e-3, "unscaled rows")
    out = torch.empty(t, n2, dtype=dtype, device=DEV)
    ops.gemm_scaled(w2, left, out)
    close(out, want, tol, "store")
    hid = torch.empty(t, n2 // 2, dtype=dtype, device=DEV)
    ops.gemm_scaled(w2, left, hid, ops.EPI_SWIGLU)
    gd, ud = want[:, 0::2], want[:, 1::2]
    close(hid, gd / (1 + torch.exp(-gd)) * ud, tol * 2, "swiglu")
    # into a part of wider rows, from a part of the weight's rows (as the attention's QKV product does)
    wide = torch.full((t, n2 + 16), 7.0, dtype=dtype, device=DEV)
    ops.gemm_scaled(w2[:n2 - 8], left, wide[:, :n2 - 8])
    close(wide[:, :n2 - 8], want[:, :n2 - 8], tol, "store into a part of the rows")
    assert (wide[:, n2 - 8:] == 7.0).all()
    with pytest.raises(ops.KernelError):
        ops.gemm_scaled(w2, left, torch.empty(t, n2, device=DEV), ops.EPI_STORE_F32)


# the products of decoders with hidden sizes of 2,048 (a vocabulary of 128,256), 2,560 and 5,120, the latter two being
# widths the kernels were not tuned on: rows of 5 KB (five waves a block), 10, 20 and 40 KB (several turns a wave)
CHOICES = [
    # n, k, rows of x, streamed?
    (3072, 2048, 8, True), (2048, 2048, 16, True), (16384, 2048, 16, True),
    (2048, 8192, 8, False),            # few blocks and 16 KB rows: k is shared out over the split tiles
    (128256, 2048, 8, True), (128256, 2048, 9, False),
    (3840, 2560, 8, True), (2560, 2560, 16, True), (20480, 2560, 8, True),
    (2560, 10240, 1, False),           # few blocks, 20 KB rows
    (128256, 2560, 1, False),          # a vocabulary streams only with a wave per kilobyte of a row
    (7680, 5120, 4, True), (7680, 5120, 8, False), (5120, 5120, 16, False),     # 10 KB rows: from 8 rows of x on, tiles
    (5120, 20480, 1, False),           # 40 KB rows: tiles for any number of rows
    (40960, 5120, 8, False), (40960, 5120, 1, True),
    (128256, 5120, 1, False),
    (3072, 2048, 32, False), (2056, 1032, 32, True),      # 17 to 64 rows: tiles, unless they cannot load the rows
]


@pytest.mark.parametrize("n,k,t,streamed", CHOICES)
def test_the_choice_of_product_kernel_follows_bytes_and_blocks(n, k, t, streamed):
    """gemm()'s own choice between streaming W and tiles, stated for the products of three decoders, two of them of
    widths no kernel was tuned on; and whatever it chooses is the product."""
    ops = _ops()
    g = torch.Generator().manual_seed(n + k + t)
    w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    x = torch.randn(t, k, generator=g).to(torch.bfloat16).to(DEV)
    assert ops.compute_units(DEV) == 256, "the table above is for 256 compute units"
    assert ops.gemm_streams(w, t) is streamed
    scratch = torch.empty(ops.GEMM_SPLIT_FLOATS, device=DEV)
    out = torch.empty(t, n, device=DEV)
    ops.gemm(w, x, out, ops.EPI_STORE_F32, scratch=scratch)
    want = x.double() @ w.double().T
    close(out, want, 2e-3, "the chosen kernel")
    acc = torch.ones(t, n, device=DEV)
    ops.gemm(w, x, acc, ops.EPI_ACCUM_F32, scratch=scratch)
    close(acc, want + 1.0, 2e-3, "the chosen kernel, adding")


def test_gemm_reference_vectors():
    """blas/blas_test.go:21-64: identity, [[1,2],[3,4]]·[1,1] = [3,7], batch layout out[p*rows + r]."""
    ops = _ops()
    w = torch.zeros(4, 4, device=DEV)
    w[:2, :2] = torch.tensor([[1., 2.], [3., 4.]])
    x = torch.zeros(2, 4, device=DEV)
    x[0, :2] = 1.0
    x[1, 0] = 2.0
    out = torch.empty(2, 4, device=DEV)
    for kind in (1, 4):
        ops.gemm(w, x, out, ops.EPI_STORE, kind)
        assert out.cpu()[:, :2].tolist() == [[3.0, 7.0], [2.0, 6.0]]


def test_gemm_refuses_what_it_cannot_do():
    ops = _ops()
    w = torch.zeros(8, 6, device=DEV)
    x = torch.zeros(2, 6, device=DEV)
    with pytest.raises(ops.KernelError, match="multiple of 4"):
        ops.gemm(w, x, torch.empty(2, 8, device=DEV))
    with pytest.raises(ops.KernelError):
        ops.gemm(torch.zeros(8, 8, device=DEV), torch.zeros(2, 8, device=DEV), torch.empty(2, 9, device=DEV))


# ---------------------------------------------------------------------------
# rotation + cache write, attention over the paged cache
# ---------------------------------------------------------------------------
def _paged_setup(dtype, n_seq_lens, kv_heads, hd, n_units=2, unit=1, seed=0, shuffle=True):
    """A page pool with pages handed out in a scrambled order, poisoned with NaN where nothing was written."""
    from dlgo_amd.cache import PAGE
    g = torch.Generator().manual_seed(seed)
    pages_per = [(n + PAGE - 1) // PAGE for n in n_seq_lens]
    n_pages = sum(pages_per) + 3
    order = torch.randperm(n_pages, generator=g).tolist() if shuffle else list(range(n_pages))
    max_pages = max(pages_per) + 1
    table = torch.full((len(n_seq_lens) + 2, max_pages), -1, dtype=torch.int32)
    it = iter(order)
    slots = list(range(len(n_seq_lens), 0, -1))      # not the identity
    for slot, npg in zip(slots, pages_per):
        for j in range(npg):
            table[slot, j] = next(it)
    unit_elems = 2 * kv_heads * PAGE * hd
    page_stride = unit_elems * n_units
    storage = torch.full((n_pages * page_stride,), float("nan"), dtype=dtype)
    return table, slots, storage, page_stride, unit * unit_elems, kv_heads * PAGE * hd


def _rope_ref(v, pos, freqs, interleaved):
    half = len(freqs)
    ang = pos * freqs
    c, s = np.cos(ang), np.sin(ang)
    out = v.copy()
    if interleaved:
        x0, x1 = v[..., 0:2 * half:2], v[..., 1:2 * half:2]
        out[..., 0:2 * half:2] = x0 * c - x1 * s
        out[..., 1:2 * half:2] = x0 * s + x1 * c
    else:
        x0, x1 = v[..., :half], v[..., half:2 * half]
        out[..., :half] = x0 * c - x1 * s
        out[..., half:2 * half] = x0 * s + x1 * c
    return out


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("H,KV,hd,rot,inter", [(4, 2, 16, 16, False), (6, 3, 48, 48, True), (8, 1, 128, 64, False),
                                               (2, 2, 32, 32, True), (4, 2, 16, 8, False), (3, 1, 32, 12, True)])
def test_rope_kv_write(dtype, _, rel, H, KV, hd, rot, inter):
    ops = _ops()
    from dlgo_amd.cache import PAGE
    from dlgo_amd.parts import rotary_frequencies
    lens = [70, 3, 129]
    starts = [5, 0, 64]                      # the rows continue sequences that already hold tokens
    q_lens = [l - s for l, s in zip(lens, starts)]
    table, slots, storage, page_stride, unit_off, v_off = _paged_setup(dtype, lens, KV, hd)
    T = sum(q_lens)
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn(T, (H + 2 * KV) * hd, generator=g).to(dtype)
    positions = torch.tensor([p for s, n in zip(starts, q_lens) for p in range(s, s + n)], dtype=torch.int32)
    tok_seq = torch.tensor([i for i, n in enumerate(q_lens) for _ in range(n)], dtype=torch.int32)
    freqs = rotary_frequencies(rot, 10000.0)
    ang = np.arange(200)[:, None] * freqs[None]
    cos, sin = torch.from_numpy(np.cos(ang).astype(np.float32)), torch.from_numpy(np.sin(ang).astype(np.float32))
    dq = qkv.clone().to(DEV)
    store = storage.clone().to(DEV)
    ops.rope_kv(dq, H, KV, hd, rot, inter, cos.to(DEV), sin.to(DEV), positions.to(DEV), tok_seq.to(DEV),
                torch.tensor(slots, dtype=torch.int32, device=DEV), table.to(DEV), store[unit_off:], page_stride, v_off)
    dq, store = dq.cpu(), store.cpu()
    src = qkv.double().numpy().reshape(T, H + 2 * KV, hd)
    for t in range(T):
        pos = int(positions[t])
        want_q = _rope_ref(src[t, :H], pos, freqs, inter)
        close(dq[t, :H * hd].reshape(H, hd), torch.from_numpy(want_q), rel, "rotated q")
        page = int(table[slots[int(tok_seq[t])], pos // PAGE])
        base = page * page_stride + unit_off
        kpage = store[base: base + KV * PAGE * hd].reshape(KV, PAGE, hd)
        vpage = store[base + v_off: base + v_off + KV * hd * PAGE].reshape(KV, hd, PAGE)
        close(kpage[:, pos % PAGE], torch.from_numpy(_rope_ref(src[t, H:H + KV], pos, freqs, inter)), rel, "stored k")
        assert torch.equal(vpage[:, :, pos % PAGE], qkv[t].reshape(H + 2 * KV, hd)[H + KV:]), "stored v"
    # nothing else was written: the other unit of each page and unused rows are still NaN
    written = (~torch.isnan(store.float())).sum().item()
    assert written == T * 2 * KV * hd


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("H,KV,hd,rot,inter,write", [(4, 2, 16, 16, False, True), (6, 3, 48, 48, True, True),
                                                     (8, 1, 128, 64, False, True), (5, 1, 80, 32, False, False)])
def test_rope_kv_from_unsummed_runs(dtype, _, rel, H, KV, hd, rot, inter, write):
    """The rows as three unsummed planes (values whose sums are exact in every dtype) give what the summed rows give, bit
    for bit: rotated queries in qkv, keys and values in the pages."""
    ops = _ops()
    from dlgo_amd.parts import rotary_frequencies
    lens, starts = [70, 3, 129], [5, 0, 64]
    q_lens = [l - s for l, s in zip(lens, starts)]
    table, slots, storage, page_stride, unit_off, v_off = _paged_setup(dtype, lens, KV, hd)
    T = sum(q_lens)
    cols = (H + (2 * KV if write else 0)) * hd
    g = torch.Generator().manual_seed(5)
    planes = torch.randint(-8, 9, (3, T, cols), generator=g).float() / 8      # sums: multiples of 1/8 below 4
    rows = torch.zeros(T, (H + 2 * KV) * hd)
    rows[:, :cols] = planes[0] + planes[1] + planes[2]
    positions = torch.tensor([p for s, n in zip(starts, q_lens) for p in range(s, s + n)], dtype=torch.int32).to(DEV)
    tok_seq = torch.tensor([i for i, n in enumerate(q_lens) for _ in range(n)], dtype=torch.int32).to(DEV)
    freqs = rotary_frequencies(rot, 10000.0)
    ang = np.arange(200)[:, None] * freqs[None]
    cos, sin = torch.from_numpy(np.cos(ang).astype(np.float32)).to(DEV), torch.from_numpy(np.sin(ang).astype(np.float32)).to(DEV)
    slot_t = torch.tensor(slots, dtype=torch.int32, device=DEV)
    got = []
    # the third way stores the values thread by thread (the arrangement for steps of single tokens): the same pages
    for unsummed, single in ((None, False), (ops.UnsummedRows(planes.reshape(-1).to(DEV), 3, T, cols), False),
                             (ops.UnsummedRows(planes.reshape(-1).to(DEV), 3, T, cols), True), (None, True)):
        dq = rows.to(dtype).to(DEV) if unsummed is None else torch.full_like(rows, float("nan")).to(dtype).to(DEV)
        store = storage.clone().to(DEV)
        ops.rope_kv(dq, H, KV if write else 0, hd, rot, inter, cos, sin, positions, tok_seq, slot_t, table.to(DEV),
                    store[unit_off:], page_stride, v_off, write_kv=write, unsummed=unsummed, single_tokens=single)
        got.append((dq[:, :H * hd].cpu(), store.cpu()))
    for other in got[1:]:
        assert torch.equal(got[0][0], other[0]), "rotated queries"
        assert torch.equal(torch.nan_to_num(got[0][1].float(), nan=-77.0), torch.nan_to_num(other[1].float(), nan=-77.0)), "pages"


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("H,KV,hd,rot,inter", [(4, 2, 16, 16, False), (6, 3, 48, 32, True), (8, 1, 128, 128, False), (3, 1, 6, 6, False)])
def test_rope_kv_of_single_tokens_finds_the_pages_by_row(dtype, _, rel, H, KV, hd, rot, inter):
    """A step of single tokens with the sequences' page-table rows given in the order of the rows writes the pages that
    the way through sequence and slot writes, bit for bit.  The table by slot is then not read: it holds holes only."""
    ops = _ops()
    from dlgo_amd.parts import rotary_frequencies
    lens = [70, 3, 129, 64, 65]
    table, slots, storage, page_stride, unit_off, v_off = _paged_setup(dtype, lens, KV, hd)
    T = len(lens)
    g = torch.Generator().manual_seed(11)
    rows = torch.randn(T, (H + 2 * KV) * hd, generator=g)
    positions = torch.tensor([l - 1 for l in lens], dtype=torch.int32).to(DEV)
    order = [3, 0, 4, 1, 2]                                    # the rows' sequences, not in the order of the rows
    tok_seq = torch.tensor(order, dtype=torch.int32).to(DEV)
    positions = positions[tok_seq.long()]
    freqs = rotary_frequencies(rot, 10000.0)
    ang = np.arange(200)[:, None] * freqs[None]
    cos, sin = torch.from_numpy(np.cos(ang).astype(np.float32)).to(DEV), torch.from_numpy(np.sin(ang).astype(np.float32)).to(DEV)
    slot_t = torch.tensor(slots, dtype=torch.int32, device=DEV)
    by_row = torch.full((T + 3, table.shape[1]), -1, dtype=torch.int32)
    by_row[:T] = table[torch.tensor(slots)[torch.tensor(order)]]
    got = []
    for pages, by_slot in ((None, table), (by_row.to(DEV), torch.full_like(table, -1))):
        dq = rows.to(dtype).to(DEV)
        store = storage.clone().to(DEV)
        ops.rope_kv(dq, H, KV, hd, rot, inter, cos, sin, positions, tok_seq, slot_t, by_slot.to(DEV), store[unit_off:], page_stride,
                    v_off, single_tokens=True, seq_pages=pages)
        got.append((dq[:, :H * hd].cpu(), store.cpu()))
    assert (~torch.isnan(got[0][1].float())).sum().item() == T * 2 * KV * hd
    assert torch.equal(got[0][0], got[1][0]), "rotated queries"
    assert torch.equal(torch.nan_to_num(got[0][1].float(), nan=-77.0), torch.nan_to_num(got[1][1].float(), nan=-77.0)), "pages"
    with pytest.raises(ops.KernelError, match="pages by sequence"):
        ops.rope_kv(rows.to(dtype).to(DEV), H, KV, hd, rot, inter, cos, sin, positions, tok_seq, slot_t, table.to(DEV),
                    storage.clone().to(DEV)[unit_off:], page_stride, v_off, single_tokens=True, seq_pages=by_row[:T - 1].to(DEV))


def _attention_ref(q, k, v, H, KV, hd, pos_of_q, lo_of_q):
    """q [n, H*hd]; k, v [len, KV*hd] for one sequence; row i attends keys lo..pos."""
    g = H // KV
    out = np.zeros_like(q)
    for i in range(q.shape[0]):
        for h in range(H):
            kvh = h // g
            ks = k[lo_of_q[i]:pos_of_q[i] + 1, kvh * hd:(kvh + 1) * hd]
            vs = v[lo_of_q[i]:pos_of_q[i] + 1, kvh * hd:(kvh + 1) * hd]
            s = ks @ q[i, h * hd:(h + 1) * hd] / math.sqrt(hd)
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, h * hd:(h + 1) * hd] = p @ vs
    return out


def _fill_cache(storage, table, slot, k, v, KV, hd, page_stride, unit_off, v_off):
    from dlgo_amd.cache import PAGE
    for pos in range(k.shape[0]):
        page = int(table[slot, pos // PAGE])
        base = page * page_stride + unit_off
        for kvh in range(KV):
            o = base + (kvh * PAGE + pos % PAGE) * hd
            storage[o:o + hd] = k[pos, kvh * hd:(kvh + 1) * hd]
            ov = base + v_off + kvh * hd * PAGE + pos % PAGE
            storage[ov: ov + hd * PAGE: PAGE] = v[pos, kvh * hd:(kvh + 1) * hd]


ATT_CASES = [  # H, KV, hd, window, [(cached length, rows of this step)]
    (4, 2, 16, 0, [(70, 70), (3, 1), (129, 5)]),
    (6, 3, 48, 0, [(200, 200), (65, 1)]),
    (4, 1, 32, 0, [(1, 1), (64, 64), (300, 1), (130, 66)]),
    (8, 8, 64, 0, [(150, 150)]),
    (4, 2, 16, 20, [(100, 100), (90, 1)]),
    (2, 1, 128, 70, [(260, 3), (260, 260)]),
    # one row per sequence (the split kernel in bfloat16)
    (4, 2, 16, 0, [(70, 1), (3, 1), (129, 1), (64, 1), (65, 1)]),
    (32, 8, 64, 0, [(700, 1), (1, 1), (333, 1)]),
    (40, 2, 32, 0, [(200, 1), (77, 1)]),
    (6, 2, 48, 50, [(300, 1), (20, 1), (128, 1)]),
    (8, 8, 128, 0, [(150, 1)]),
    # long sequences: the pages of one sequence are split over several blocks and merged by a second kernel
    (4, 2, 16, 0, [(9000, 1), (70, 1)]),
    (32, 2, 128, 0, [(2700, 1), (100, 1), (2049, 1)]),
    (8, 8, 64, 300, [(9000, 1), (8500, 1)]),
    # groups that do not divide a tile
    (6, 2, 48, 0, [(100, 100), (31, 7)]),
    (40, 2, 32, 0, [(90, 90)]),
    (4, 4, 80, 0, [(130, 130), (5, 5)]),
    # rows of tiles (one sequence, one kv head) that do not divide the 256 blocks of a round of the chip
    (32, 4, 32, 0, [(63, 45), (300, 215), (2, 1), (300, 214), (2, 1)]),
    (32, 4, 128, 0, [(63, 45), (300, 215), (2, 1), (300, 214), (2, 1)]),
    (6, 3, 16, 0, [(700, 700), (650, 650), (90, 90), (300, 300), (641, 641), (64, 64), (200, 77), (690, 690)]),
]


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("H,KV,hd,window,seqs", ATT_CASES)
@pytest.mark.parametrize("kernel", ["rows", "auto", "registers"])
def test_attention_over_pages(dtype, _, rel, H, KV, hd, window, seqs, kernel):
    ops = _ops()
    if kernel == "registers" and (dtype != torch.bfloat16 or any(r != 1 for _, r in seqs)):
        pytest.skip("the variant is the bfloat16 split kernel's: one row per sequence")
    lens = [l for l, _ in seqs]
    table, slots, storage, page_stride, unit_off, v_off = _paged_setup(dtype, lens, KV, hd, seed=hd)
    g = torch.Generator().manual_seed(H * 100 + hd)
    qs, pos, tok_seq, want = [], [], [], []
    for i, (length, rows) in enumerate(seqs):
        k = (torch.randn(length, KV * hd, generator=g) * 1.5).to(dtype)
        v = torch.randn(length, KV * hd, generator=g).to(dtype)
        q = (torch.randn(rows, H * hd, generator=g) * 1.5).to(dtype)
        _fill_cache(storage, table, slots[i], k, v, KV, hd, page_stride, unit_off, v_off)
        p = list(range(length - rows, length))
        lo = [max(0, x - window + 1) if window else 0 for x in p]
        want.append(_attention_ref(q.double().numpy(), k.double().numpy(), v.double().numpy(), H, KV, hd, p, lo))
        qs.append(q)
        pos += p
        tok_seq += [i] * rows
    q = torch.cat(qs).to(DEV)
    out = torch.full((q.shape[0], H * hd), float("nan"), dtype=dtype, device=DEV)
    args = (q, out, H, KV, hd, torch.tensor(pos, dtype=torch.int32, device=DEV),
            torch.tensor(tok_seq, dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
            table.to(DEV), storage.to(DEV)[unit_off:], page_stride, v_off)
    if kernel == "rows":
        ops.attention_rows(*args, window=window)
    else:
        q_lens = [r for _, r in seqs]
        starts = [l - r for l, r in seqs]
        # "registers": the split kernel that reads pages straight into its operands (the default sends them through LDS)
        ops.attention(*args, q_lens=q_lens, start_pos=starts, window=window, split_variant=1 if kernel == "registers" else 0)
    close(out, torch.from_numpy(np.concatenate(want)), rel if dtype == torch.float32 else 2e-2, "attention")


@pytest.mark.parametrize("dtype,_,rel", DT)
@pytest.mark.parametrize("kernel", ["rows", "auto", "registers"])
def test_attention_finds_a_far_key_and_respects_the_window_edge(dtype, _, rel, kernel):
    """Random scores hide a key that is skipped or read twice.  Here one key among hundreds matches the query
    so strongly that the output is that key's value: the first key, one in the middle of a page, the last key
    of a page, the first of the next, the token itself; with a window, the key at its edge counts and the one just
    outside does not."""
    ops = _ops()
    if kernel == "registers" and dtype != torch.bfloat16:
        pytest.skip("the variant is the bfloat16 split kernel's")
    H, KV, hd = 4, 2, 32
    length = 450
    g = torch.Generator().manual_seed(9)
    table, slots, storage, page_stride, unit_off, v_off = _paged_setup(dtype, [length], KV, hd, seed=4)
    k = (0.05 * torch.randn(length, KV * hd, generator=g)).to(dtype)
    v = torch.randn(length, KV * hd, generator=g).to(dtype)
    probe = torch.zeros(hd)
    probe[3] = 1.0
    marks = [0, 37, 63, 64, 300, 449]
    for i, t in enumerate(marks):
        k[t, :hd] = 0
        k[t, i] = 60.0                       # kv head 0: key t answers to a query along axis i
    _fill_cache(storage, table, slots[0], k, v, KV, hd, page_stride, unit_off, v_off)
    dev = lambda x, dt=torch.int32: torch.tensor(x, dtype=dt, device=DEV)

    def run(queries, positions, window):
        q = torch.zeros(len(queries), H * hd)
        for r, axis in enumerate(queries):
            q[r, axis] = 60.0                # head 0 (kv head 0)
            q[r, hd + axis] = 60.0           # head 1 (kv head 0 too)
        q = q.to(dtype).to(DEV)
        out = torch.empty(len(queries), H * hd, dtype=dtype, device=DEV)
        args = (q, out, H, KV, hd, dev(positions), dev([0] * len(queries)), dev(slots), table.to(DEV),
                storage.to(DEV)[unit_off:], page_stride, v_off)
        if kernel == "rows" or len(queries) > 1:
            ops.attention_rows(*args, window=window)
        else:
            ops.attention(*args, q_lens=[1], start_pos=positions, window=window, split_variant=1 if kernel == "registers" else 0)
        return out.float().cpu()
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for i, t in enumerate(marks):            # a single row at the last position sees every marked key
        out = run([i], [length - 1], 0)
        assert torch.allclose(out[0, :hd], v[t, :hd].float(), atol=tol), (i, t)
        assert torch.allclose(out[0, hd:2 * hd], v[t, :hd].float(), atol=tol)
    # causality: a row before the marked key does not see it (its output is an average of many values)
    out = run([4], [299], 0)
    assert not torch.allclose(out[0, :hd], v[300, :hd].float(), atol=0.2)
    # the window: at position 449 with window 150 the key at 300 is the oldest one seen; with 149 it is gone
    assert torch.allclose(run([4], [449], 150)[0, :hd], v[300, :hd].float(), atol=tol)
    assert not torch.allclose(run([4], [449], 149)[0, :hd], v[300, :hd].float(), atol=0.2)


def _wider(table, bound):
    """The page table with room for sequences of `bound` pages (a recorded step's launch is sized for the longest
    sequence the cache allows, whatever the sequences hold)."""
    if bound is None:
        return table
    wide = torch.full((table.shape[0], bound), -1, dtype=table.dtype)
    wide[:, :table.shape[1]] = table
    return wide


@pytest.mark.parametrize("bound", [None, 3000])
@pytest.mark.parametrize("variant", [0, 1, "pages by sequence"])
@pytest.mark.parametrize("H,KV,hd,rot,inter,window", [(4, 2, 16, 16, False, 0), (32, 8, 64, 64, False, 0), (6, 3, 48, 32, True, 0),
                                                       (40, 2, 32, 32, False, 0), (8, 8, 128, 128, True, 50), (4, 1, 80, 0, False, 0),
                                                       (6, 2, 80, 48, False, 0), (2, 1, 256, 256, False, 0)])
def test_decode_attention_that_rotates_and_stores_by_itself(H, KV, hd, rot, inter, window, variant, bound):
    """One row per sequence: the split kernel given unrotated [q | k | v] rows against the two-kernel way
    (rotate and store, then attend): the same output, the same cache afterwards.  Also with a launch sized for
    sequences of 3,000 pages, of whose blocks a short sequence uses a few; and with the sequences' page numbers given
    by their place in the step, where the fused kernel must not look at the table by slot (which then holds nonsense)."""
    ops = _ops()
    from dlgo_amd.parts import rotary_frequencies
    dtype = torch.bfloat16
    lens = [70, 3, 129, 64, 65, 1, 2000]
    table, slots, storage, page_stride, unit_off, v_off = _paged_setup(dtype, lens, KV, hd, seed=rot + hd)
    table = _wider(table, bound)
    g = torch.Generator().manual_seed(H + hd)
    for i, n in enumerate(lens):                       # what the sequences hold before this step
        if n > 1:
            k = torch.randn(n - 1, KV * hd, generator=g).to(dtype)
            v = torch.randn(n - 1, KV * hd, generator=g).to(dtype)
            _fill_cache(storage, table, slots[i], k, v, KV, hd, page_stride, unit_off, v_off)
    storage = torch.nan_to_num(storage.float(), nan=7.0).to(dtype)      # so that the caches can be compared
    qkv = torch.randn(len(lens), (H + 2 * KV) * hd, generator=g).to(dtype)
    cos = sin = None
    if rot:
        ang = np.arange(2048)[:, None] * rotary_frequencies(rot, 10000.0)[None]
        cos, sin = (torch.from_numpy(f(ang).astype(np.float32)).to(DEV) for f in (np.cos, np.sin))
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    positions, tok_seq, dslots = dev([n - 1 for n in lens]), dev(list(range(len(lens)))), dev(slots)
    outs, caches = [], []
    for fused in (False, True):
        store = storage.clone().to(DEV)
        rows = qkv.clone().to(DEV)
        out = torch.empty(len(lens), H * hd, dtype=dtype, device=DEV)
        by_seq = variant == "pages by sequence"
        common = dict(q_lens=[1] * len(lens), start_pos=[n - 1 for n in lens], window=window, kernel="split",
                      split_variant=0 if by_seq else variant)
        if fused:
            extra, by_slot = {}, table.to(DEV)
            if by_seq:
                extra = dict(seq_pages=table[torch.tensor(slots, dtype=torch.long)].contiguous().to(DEV))
                by_slot = torch.zeros_like(by_slot)          # every entry names page 0: of no use to anyone
            ops.attention(rows, out, H, KV, hd, positions, tok_seq, dslots, by_slot, store[unit_off:], page_stride, v_off,
                          rotation=(cos, sin, rot, inter) if rot else None, new_kv=True, **common, **extra)
        else:
            ops.rope_kv(rows, H, KV, hd, rot, inter, cos, sin, positions, tok_seq, dslots, table.to(DEV), store[unit_off:],
                        page_stride, v_off)
            ops.attention(rows, out, H, KV, hd, positions, tok_seq, dslots, table.to(DEV), store[unit_off:], page_stride, v_off,
                          **common)
        outs.append(out.float().cpu())
        caches.append(store.cpu())
    assert torch.equal(caches[0], caches[1])
    assert torch.allclose(outs[0], outs[1], atol=1e-6, rtol=0)


def _fill_pages(storage, table, slot, k, v, KV, hd, page_stride, unit_off, v_off):
    """_fill_cache a page at a time."""
    from dlgo_amd.cache import PAGE
    for pg in range((k.shape[0] + PAGE - 1) // PAGE):
        p0, p1 = pg * PAGE, min(k.shape[0], (pg + 1) * PAGE)
        base = int(table[slot, pg]) * page_stride + unit_off
        for kvh in range(KV):
            o = base + kvh * PAGE * hd
            storage[o:o + (p1 - p0) * hd] = k[p0:p1, kvh * hd:(kvh + 1) * hd].reshape(-1)
            ov = base + v_off + kvh * hd * PAGE
            storage[ov:ov + hd * PAGE].view(hd, PAGE)[:, :p1 - p0] = v[p0:p1, kvh * hd:(kvh + 1) * hd].T


@pytest.mark.parametrize("kernel", ["bfloat16", "bfloat16 registers", "bfloat16 pages by sequence", "float32"])
@pytest.mark.parametrize("H,KV,hd,bound,lens", [
    # 288 (sequence, kv head) pairs fill the chip by themselves: a sequence gets a second block from about 12,000 tokens
    (8, 8, 64, 400, [12500, 8200, 4097, 64, 65, 1] + [3 + 7 * i for i in range(30)]),
    # ten pairs: every sequence is dealt to 26 blocks, the longest to more of the 47 the launch holds
    (4, 2, 128, 3000, [9000, 300, 1, 2049, 130]),
    # 64 pairs: four blocks each, ten for the sequence of 40,000 tokens
    (4, 2, 128, 3000, [40000, 77, 9000] + [5 + 11 * i for i in range(29)]),
])
def test_decode_attention_of_short_sequences_in_a_launch_sized_for_long_ones(H, KV, hd, bound, lens, kernel):
    """A recorded decode step is launched with blocks for the longest sequence the cache allows; a sequence uses as many
    of them as its own pages call for.  A page that falls between two blocks' shares, or is read by both, would be lost
    among thousands of random keys, so each sequence holds marked keys (the first and last of its pages, of the first
    and last page, of the pages where a share may end), each answering to a query along one axis so strongly that the
    output is that key's value."""
    ops = _ops()
    from dlgo_amd.cache import PAGE
    dtype = torch.float32 if kernel == "float32" else torch.bfloat16
    table, slots, storage, page_stride, unit_off, v_off = _paged_setup(dtype, lens, KV, hd, seed=hd + len(lens))
    table = _wider(table, bound)
    g = torch.Generator().manual_seed(bound)
    n_marks = 16
    marks, values = [], []
    for i, length in enumerate(lens):
        pages = (length + PAGE - 1) // PAGE
        cand = [0, PAGE - 1, PAGE, length - 1, length - 2, (pages - 1) * PAGE, (pages - 1) * PAGE - 1]
        for used in (2, 3, 4, 5, 6, 7, 8, 26, 27, 30):
            span = (pages + used - 1) // used
            cand += [span * PAGE - 1, span * PAGE, 2 * span * PAGE - 1, 2 * span * PAGE, (used - 1) * span * PAGE]
        mine = []
        for c in cand:
            if 0 <= c < length and c not in mine:
                mine.append(c)
        mine = (mine * n_marks)[:n_marks] if len(mine) < n_marks else mine[:n_marks]
        k = (0.05 * torch.randn(length, KV * hd, generator=g)).to(dtype)
        v = torch.randn(length, KV * hd, generator=g).to(dtype)
        for axis, t in enumerate(mine):
            if mine.index(t) == axis:               # a position marked twice answers to its first axis
                for kvh in range(KV):
                    k[t, kvh * hd:(kvh + 1) * hd] = 0
                    k[t, kvh * hd + axis] = 60.0
        _fill_pages(storage, table, slots[i], k, v, KV, hd, page_stride, unit_off, v_off)
        marks.append(mine)
        values.append(v.float())
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    n = len(lens)
    store = storage.to(DEV)
    positions, tok_seq, dslots, dtable = dev([x - 1 for x in lens]), dev(list(range(n))), dev(slots), table.to(DEV)
    g_heads = H // KV
    for axis in range(n_marks):
        q = torch.zeros(n, H, hd)
        q[:, :, axis] = 60.0
        q = q.reshape(n, H * hd).to(dtype).to(DEV)
        out = torch.full((n, H * hd), float("nan"), dtype=dtype, device=DEV)
        extra, by_slot = {}, dtable
        if kernel == "bfloat16 pages by sequence":      # the pages' numbers by place in the step; the table by slot is not to be read
            extra = dict(seq_pages=dtable[dslots.long()].contiguous())
            by_slot = torch.zeros_like(dtable)
        ops.attention(q, out, H, KV, hd, positions, tok_seq, dslots, by_slot, store[unit_off:], page_stride, v_off,
                      q_lens=[1] * n, start_pos=[x - 1 for x in lens], kernel="split", max_pages_used=bound,
                      split_variant=1 if kernel == "bfloat16 registers" else 0, **extra)
        got = out.float().cpu().view(n, H, hd)
        for i in range(n):
            t = marks[i][axis]
            if marks[i].index(t) != axis:           # a short sequence has fewer marks than axes
                continue
            for h in range(H):
                kvh = h // g_heads
                assert torch.allclose(got[i, h], values[i][t, kvh * hd:(kvh + 1) * hd], atol=2e-2), \
                    f"sequence {i} of {lens[i]} tokens, key {t}, head {h}"


def test_attention_reference_vectors():
    """layers/gqa_test.go: one cached position gives V for every head of the group (:8-43);
    equal keys give the plain mean, with a window of 2 at position 3 of v = 0,1,2,3 that is 2.5 (:110-136)."""
    ops = _ops()
    H, KV, hd = 4, 2, 16
    table, slots, storage, page_stride, unit_off, v_off = _paged_setup(torch.float32, [1, 4], KV, hd)
    v0 = torch.arange(KV * hd, dtype=torch.float32)[None]
    _fill_cache(storage, table, slots[0], torch.randn(1, KV * hd), v0, KV, hd, page_stride, unit_off, v_off)
    kk = torch.ones(4, KV * hd)
    vv = torch.arange(4, dtype=torch.float32)[:, None].repeat(1, KV * hd)
    _fill_cache(storage, table, slots[1], kk, vv, KV, hd, page_stride, unit_off, v_off)
    q = torch.randn(2, H * hd).to(DEV)
    out = torch.empty(2, H * hd, device=DEV)
    ops.attention_rows(q, out, H, KV, hd, torch.tensor([0, 3], dtype=torch.int32, device=DEV),
                       torch.tensor([0, 1], dtype=torch.int32, device=DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                       table.to(DEV), storage.to(DEV)[unit_off:], page_stride, v_off, window=2)
    got = out.cpu()
    assert torch.equal(got[0].reshape(H, hd), v0.reshape(KV, hd).repeat_interleave(2, 0))
    assert torch.allclose(got[1], torch.full((H * hd,), 2.5), atol=1e-6)


# ---------------------------------------------------------------------------
# sampling
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,width", [(torch.float32, 128256), (torch.float32, 5), (torch.int32, 1), (torch.bfloat16, 6),
                                         (torch.bfloat16, 2 * 8 * 64 * 80 * 3), (torch.int32, 37)])
def test_copy_rows_gathers_and_scatters(dtype, width):
    """dst[dst_rows[i]] = src[src_rows[i]]: rows picked out (the loop's logits and ids), rows put in place (page-table
    rows), both at once within one tensor (pages copied), for rows of whole 16 bytes and of odd sizes."""
    ops = _ops()
    g = torch.Generator().manual_seed(width)
    n = 9
    src = (torch.randn(n, width, generator=g) * 100).to(dtype).to(DEV)
    pick = torch.tensor([7, 0, 0, 3], dtype=torch.int32, device=DEV)
    out = ops.copy_rows(src, torch.zeros(4, width, dtype=dtype, device=DEV), src_rows=pick)
    assert torch.equal(out, src[pick.long()])
    place = torch.tensor([5, 1, 8], dtype=torch.int32, device=DEV)
    dst = torch.full((n, width), 3, dtype=dtype, device=DEV)
    ops.copy_rows(src, dst, dst_rows=place)
    want = torch.full((n, width), 3, dtype=dtype, device=DEV)
    want[place.long()] = src[:3]
    assert torch.equal(dst, want)
    both = src.clone()
    ops.copy_rows(both, both, src_rows=torch.tensor([0, 4], dtype=torch.int32, device=DEV),
                  dst_rows=torch.tensor([6, 2], dtype=torch.int32, device=DEV))
    want = src.clone()
    want[[6, 2]] = src[[0, 4]]
    assert torch.equal(both, want)
    # a strided view (rows of a wider tensor), a 1-d tensor as rows of one element, fewer rows than the lists hold
    if width >= 4 and dtype != torch.bfloat16:
        view = src[:, :width // 2 * 2][:, :2]
        assert torch.equal(ops.copy_rows(view, torch.zeros(2, 2, dtype=dtype, device=DEV), src_rows=pick, n=2), view[pick[:2].long()])
    if width == 1:
        flat = src[:, 0].contiguous()
        assert torch.equal(ops.copy_rows(flat, torch.zeros(4, dtype=dtype, device=DEV), src_rows=pick), flat[pick.long()])
    with pytest.raises(ops.KernelError):
        ops.copy_rows(src, torch.zeros(2, width, dtype=dtype, device=DEV), src_rows=pick)             # four rows into two
    if dtype == torch.bfloat16:
        with pytest.raises(ops.KernelError):
            ops.copy_rows(src[:, :3].contiguous(), torch.zeros(4, 3, dtype=dtype, device=DEV), src_rows=pick)   # 6-byte rows


def test_argmax_first_maximum():
    ops = _ops()
    x = torch.zeros(3, 70001, device=DEV)
    x[0, 5] = 2.0
    x[0, 69000] = 2.0
    x[1, 70000] = 1.0
    x[2, :] = -1.0
    out = torch.empty(3, dtype=torch.int32, device=DEV)
    ops.argmax(x, out)
    assert out.tolist() == [5, 70000, 0]
    v = torch.tensor([[1., 5., 2., 3.]], device=DEV)            # ops/sampling_test.go:9-16
    ops.argmax(v, out[:1])
    assert out[:1].tolist() == [1]


def _sample(logits, temp, top_k=0, top_p=1.0, min_p=0.0, pen=1.0, recent=None, u=0.5):
    ops = _ops()
    n, v = logits.shape
    lg = logits.float().to(DEV)
    f = lambda val: torch.full((n,), val, dtype=torch.float32, device=DEV)
    rec = None
    if recent is not None:
        rec = torch.tensor(recent, dtype=torch.int32, device=DEV)
    uu = torch.tensor(u if isinstance(u, list) else [u] * n, dtype=torch.float32, device=DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ops.sample(lg, torch.empty(n, v, device=DEV), f(temp),
               torch.full((n,), top_k, dtype=torch.int32, device=DEV), f(top_p), f(min_p), f(pen), rec, uu, out)
    return out.tolist()


@pytest.mark.parametrize("v", [11, 384, 5000, 128256])
def test_sample_matches_plain(v):
    import plain_llama as plain
    g = torch.Generator().manual_seed(v)
    logits = torch.randn(6, v, generator=g) * 2.0
    us = [0.03, 0.37, 0.5, 0.81, 0.999, 0.61]
    cases = [dict(temp=0.8), dict(temp=1.0, top_k=5), dict(temp=0.7, top_p=0.6), dict(temp=1.3, min_p=0.2),
             dict(temp=0.9, top_k=40, top_p=0.9, pen=1.1), dict(temp=0.0)]
    recent = [[int(logits[i].argmax()), 3, 3, -1] for i in range(6)]
    for c in cases:
        got = _sample(logits, c.get("temp"), c.get("top_k", 0), c.get("top_p", 1.0), c.get("min_p", 0.0), c.get("pen", 1.0),
                      recent, us)
        for i in range(6):
            want = plain.sample_token(logits[i].double().numpy(), us[i], c["temp"], c.get("top_k", 0), c.get("top_p", 1.0),
                                      c.get("min_p", 0.0), c.get("pen", 1.0), [t for t in recent[i] if t >= 0])
            assert got[i] == want, (c, i)


def test_sample_top_k_in_awkward_rows():
    """Rows that the quick way of top-k cannot take, or only just: many equal values at the cut, a k-th value far below
    the maximum, a k beyond what it keeps, a row of negative values: the same token as the plain implementation."""
    import plain_llama as plain
    g = torch.Generator().manual_seed(5)
    v = 6000
    rows = []
    r = torch.randn(v, generator=g) * 2
    r[100:1400] = 9.0                         # 1300 equal values at the top: more than the quick way keeps
    rows.append((r, dict(temp=1.0, top_k=50)))
    r = torch.randn(v, generator=g) * 0.01 - 40.0
    r[7] = 30.0                               # everything else far below the maximum
    rows.append((r, dict(temp=1.0, top_k=5)))
    r = torch.randn(v, generator=g) * 3
    rows.append((r, dict(temp=1.5, top_k=2000, top_p=0.95)))          # k beyond the candidates kept
    r = -torch.rand(v, generator=g) * 5 - 1                           # all negative
    rows.append((r, dict(temp=0.6, top_k=40, top_p=0.9, min_p=0.05)))
    r = torch.randn(v, generator=g)
    r[5::7] = 2.5                             # ties inside the kept set and at its edge
    rows.append((r, dict(temp=0.9, top_k=300, top_p=0.8)))
    r = torch.tensor([-0., -0., 0.1, -0., -0.25, -0.25, -0., 0., -0.25, 0., 0.])     # -0 and +0 are one value, tied at the cut
    rows.append((r, dict(temp=0.3, top_k=40, top_p=0.5, min_p=0.2)))
    rows.append((torch.cat([r, torch.full((3000,), -5.0)]), dict(temp=0.3, top_p=0.5)))
    for logits, c in rows:
        for u in (0.00137, 0.2031, 0.5531, 0.8973, 0.99951):       # no multiples of 1/1300: the equal values' edges
            got = _sample(logits[None], c["temp"], c.get("top_k", 0), c.get("top_p", 1.0), c.get("min_p", 0.0), u=u)[0]
            want = plain.sample_token(logits.double().numpy(), u, c["temp"], c.get("top_k", 0), c.get("top_p", 1.0),
                                      c.get("min_p", 0.0), 1.0, [])
            assert got == want, (c, u)


def test_sample_wide_rows_dealt_to_several_blocks():
    """A wide vocabulary with a small top-k: a row's parts go to blocks of their own first, and whatever they cannot
    finish falls to the one-block kernel.  Rows of every kind in one call, each with its own options: a plain one, one
    whose kept values are tied beyond what a part may keep (200 equal values in one part), one whose k-th value lies
    far below the maximum, ties across parts at the cut, a row without top-k, a greedy row, k at and beyond the limit
    of this way, a penalised maximum."""
    import plain_llama as plain
    ops = _ops()
    g = torch.Generator().manual_seed(11)
    v = 128256
    rows, opts, recents = [], [], []

    def add(r, recent=(), **c):
        rows.append(r)
        opts.append(c)
        recents.append(list(recent))
    add(torch.randn(v, generator=g) * 2, temp=0.7, top_k=40, top_p=0.9, pen=1.1, recent=[5, 77, 5])
    r = torch.randn(v, generator=g) * 2
    r[9000:9200] = 11.0
    add(r, temp=1.0, top_k=50)
    r = torch.randn(v, generator=g) * 0.01 - 40.0
    r[70007] = 30.0
    add(r, temp=1.0, top_k=5)
    r = torch.randn(v, generator=g)
    r[3::4001] = 6.5                         # 33 equal values, one in every part, straddling the cut at k = 20
    add(r, temp=0.9, top_k=20, top_p=0.95)
    add(torch.randn(v, generator=g) * 3, temp=0.8)
    add(torch.randn(v, generator=g) * 3, temp=0.0, top_k=40)
    add(torch.randn(v, generator=g) * 3, temp=1.2, top_k=128, min_p=0.01)
    add(torch.randn(v, generator=g) * 3, temp=1.2, top_k=129, top_p=0.99)
    # a top-k beyond what a part may offer: the parts offer their largest 128 and the last block checks that the row's
    # largest k are among them; they are not where one part holds 300 of the largest 400, and not beyond 1,024
    add(torch.randn(v, generator=g) * 3, temp=0.9, top_k=500)
    add(torch.randn(v, generator=g) * 3, temp=1.0, top_k=1000, min_p=0.001)
    add(torch.randn(v, generator=g) * 3, temp=1.0, top_k=1025)
    r = torch.randn(v, generator=g)
    r[4008 * 7 + 5: 4008 * 7 + 305] += 8.0
    add(r, temp=1.5, top_k=400)
    r = torch.randn(v, generator=g) * 2
    top = int(r.argmax())
    add(r, temp=0.5, top_k=3, pen=4.0, recent=[top, int(r.topk(2).indices[1])])
    n = len(rows)
    width = max(len(x) for x in recents) or 1
    rec = torch.full((n, width), -1, dtype=torch.int32)
    for i, x in enumerate(recents):
        rec[i, :len(x)] = torch.tensor(x, dtype=torch.int32)
    lg = torch.stack(rows).to(DEV)
    col = lambda name, default, dt: torch.tensor([c.get(name, default) for c in opts], dtype=dt, device=DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    work = torch.empty(n, v, device=DEV)
    for u in (0.00137, 0.2031, 0.5531, 0.8973, 0.99951):
        ops.sample(lg, work, col("temp", 1.0, torch.float32), col("top_k", 0, torch.int32), col("top_p", 1.0, torch.float32),
                   col("min_p", 0.0, torch.float32), col("pen", 1.0, torch.float32), rec.to(DEV),
                   torch.full((n,), u, dtype=torch.float32, device=DEV), out)
        got = out.tolist()
        for i, c in enumerate(opts):
            want = plain.sample_token(rows[i].double().numpy(), u, c["temp"], c.get("top_k", 0), c.get("top_p", 1.0),
                                      c.get("min_p", 0.0), c.get("pen", 1.0), recents[i])
            assert got[i] == want, (i, c, u)
        # a caller that knows no row has a small top-k may say so, and two kernels are not launched: the same tokens
        # (said of rows that do have one, it costs time only: the one-block kernel takes them)
        again = torch.empty_like(out)
        ops.sample(lg, work, col("temp", 1.0, torch.float32), col("top_k", 0, torch.int32), col("top_p", 1.0, torch.float32),
                   col("min_p", 0.0, torch.float32), col("pen", 1.0, torch.float32), rec.to(DEV),
                   torch.full((n,), u, dtype=torch.float32, device=DEV), again, dealt_rows=False)
        assert again.tolist() == got, u


@pytest.mark.parametrize("v", [20011, 128256])
def test_sample_whole_rows_from_the_masses_of_their_parts(v):
    """A wide row that no top-k, top-p or min-p cuts is drawn from by the parts' sums: each part's mass from its own
    maximum, scaled to the row's, then the piece of 256 that reaches the target, then its elements.  Random rows are
    compared with the plain pipeline; rows whose mass sits in three far-apart tokens say exactly which token a draw
    must give: by position in the row (first, middle and last part, the last element of a part, the very last element),
    with one of them penalised away, and with half the row masked."""
    import plain_llama as plain
    ops = _ops()
    g = torch.Generator().manual_seed(v)
    per = ((v + 31) // 32 + 3) & ~3                      # a part's elements
    rows, opts, recents, expect = [], [], [], []

    def add(r, recent=(), expect_by_u=None, **c):
        rows.append(r)
        opts.append(c)
        recents.append(list(recent))
        expect.append(expect_by_u)
    add(torch.randn(v, generator=g) * 2, temp=0.8)
    add(torch.randn(v, generator=g) * 3, temp=1.3, pen=1.5, recent=[7, 7, 100, v - 1])
    add(torch.randn(v, generator=g) * 2, temp=1.0, top_k=v + 3)            # a top-k that cuts nothing
    spikes = [5, 17 * per - 1, v - 1]                    # first part; the last element of a part; the last of the row
    r = torch.randn(v, generator=g) * 0.01 - 30.0
    r[spikes] = 20.0
    add(r, temp=1.0, expect_by_u={0.2: spikes[0], 0.5: spikes[1], 0.9: spikes[2], 0.999: spikes[2], 0.001: spikes[0]})
    add(r.clone(), temp=2.0, pen=4.0, recent=[spikes[1], 3],              # the middle one penalised: 20 -> 5, e^-7.5 of the others
        expect_by_u={0.2: spikes[0], 0.45: spikes[0], 0.55: spikes[2], 0.9: spikes[2]})
    r = torch.randn(v, generator=g)
    r[torch.randperm(v, generator=g)[: v // 2]] = float("-inf")
    r[per * 9: per * 10] = float("-inf")                 # and a whole part
    add(r, temp=0.7)
    # two tokens hold the mass, neighbours in one piece of 256, and the first of them is penalised away: the walk
    # through the piece has to know that too, or every draw would stop at the first
    r = torch.randn(v, generator=g) * 0.01 - 30.0
    near = 5 * per + 300
    r[[near, near + 3]] = 20.0
    add(r, temp=2.0, pen=4.0, recent=[11, near], expect_by_u={u: near + 3 for u in (0.001, 0.2, 0.45, 0.5, 0.55, 0.9, 0.999)})
    n = len(rows)
    width = max(len(x) for x in recents) or 1
    rec = torch.full((n, width), -1, dtype=torch.int32)
    for i, x in enumerate(recents):
        rec[i, :len(x)] = torch.tensor(x, dtype=torch.int32)
    lg = torch.stack(rows).to(DEV)
    col = lambda name, default, dt: torch.tensor([c.get(name, default) for c in opts], dtype=dt, device=DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    work = torch.empty(n, v, device=DEV)
    for u in (0.001, 0.2, 0.45, 0.5, 0.55, 0.9, 0.999):
        ops.sample(lg, work, col("temp", 1.0, torch.float32), col("top_k", 0, torch.int32), col("top_p", 1.0, torch.float32),
                   col("min_p", 0.0, torch.float32), col("pen", 1.0, torch.float32), rec.to(DEV),
                   torch.full((n,), u, dtype=torch.float32, device=DEV), out)
        got = out.tolist()
        for i, c in enumerate(opts):
            if expect[i] is not None:
                if u in expect[i]:
                    assert got[i] == expect[i][u], (i, c, u)
                continue
            want = plain.sample_token(rows[i].double().numpy(), u, c["temp"], c.get("top_k", 0), 1.0, 0.0, c.get("pen", 1.0), recents[i])
            assert got[i] == want, (i, c, u)
            assert rows[i][got[i]] > float("-inf")


@pytest.mark.parametrize("v", [20011, 128256])
def test_sample_rows_cut_by_min_p_alone(v):
    """A wide row whose only cut is min-p: each part offers what lies within log(min_p) of its own maximum, which
    holds everything within that of the row's.  Against the plain pipeline: random rows with loose and tight cuts, a
    row with so loose a cut that the parts give up (the one-block kernel takes it), the survivors all in one part,
    the largest element penalised below the cut, a masked part; and a row whose survivors are known, one in the first
    part and one in the last, so that a draw says which."""
    import plain_llama as plain
    ops = _ops()
    g = torch.Generator().manual_seed(v + 1)
    per = ((v + 31) // 32 + 3) & ~3
    rows, opts, recents, expect = [], [], [], []

    def add(r, recent=(), expect_by_u=None, **c):
        rows.append(r)
        opts.append(c)
        recents.append(list(recent))
        expect.append(expect_by_u)
    add(torch.randn(v, generator=g) * 2, temp=0.8, min_p=0.05)
    add(torch.randn(v, generator=g) * 2, temp=1.0, min_p=0.5)
    add(torch.randn(v, generator=g) * 2, temp=1.5, min_p=1e-6)                 # nearly everything stays: too much to offer
    r = torch.randn(v, generator=g) * 0.5
    r[3 * per + 10: 3 * per + 90] += 9.0                                       # 80 survivors, all in one part
    add(r, temp=1.0, min_p=0.01)
    r = torch.randn(v, generator=g) * 0.5
    r[6 * per + 10: 6 * per + 310] += 9.0                                      # 300 in one part: more than a part may offer,
    add(r, temp=1.0, min_p=0.01)                                               # and the row must not be drawn from the 128
    r = torch.randn(v, generator=g) * 2
    top = int(r.argmax())
    add(r, temp=0.7, min_p=0.2, pen=8.0, recent=[top])                         # the maximum falls, the cut with it
    r = torch.randn(v, generator=g) * 2
    r[per * 20: per * 21] = float("-inf")
    add(r, temp=0.9, min_p=0.1, top_k=v)
    r = torch.randn(v, generator=g) * 0.01 - 30.0
    r[7] = 20.0
    r[v - 2] = 20.0 + math.log(3.0)                                            # three times the weight of the other
    add(r, temp=1.0, min_p=0.1, expect_by_u={0.1: 7, 0.24: 7, 0.26: v - 2, 0.9: v - 2})
    n = len(rows)
    width = max(len(x) for x in recents) or 1
    rec = torch.full((n, width), -1, dtype=torch.int32)
    for i, x in enumerate(recents):
        rec[i, :len(x)] = torch.tensor(x, dtype=torch.int32)
    lg = torch.stack(rows).to(DEV)
    col = lambda name, default, dt: torch.tensor([c.get(name, default) for c in opts], dtype=dt, device=DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    work = torch.empty(n, v, device=DEV)
    for u in (0.003, 0.1, 0.24, 0.26, 0.61, 0.9, 0.997):
        ops.sample(lg, work, col("temp", 1.0, torch.float32), col("top_k", 0, torch.int32), col("top_p", 1.0, torch.float32),
                   col("min_p", 0.0, torch.float32), col("pen", 1.0, torch.float32), rec.to(DEV),
                   torch.full((n,), u, dtype=torch.float32, device=DEV), out)
        got = out.tolist()
        for i, c in enumerate(opts):
            if expect[i] is not None:
                if u in expect[i]:
                    assert got[i] == expect[i][u], (i, c, u)
                continue
            want = plain.sample_token(rows[i].double().numpy(), u, c["temp"], c.get("top_k", 0), 1.0, c["min_p"], c.get("pen", 1.0), recents[i])
            assert got[i] == want, (i, c, u)


def test_sample_reference_behaviour():
    """ops/sampling_test.go: a dominant logit is always drawn (:18-30); temperature 2 halves the logits (:48-57)."""
    logits = torch.zeros(1, 50)
    logits[0, 17] = 100.0
    for u in (1e-6, 0.3, 0.999):
        assert _sample(logits, 1.0, u=u) == [17]
    lg = torch.tensor([[2., 4., 6.]])          # temperature 2 -> [1,2,3]: p = softmax([1,2,3])
    p = torch.softmax(torch.tensor([1., 2., 3.]), 0).cumsum(0)
    assert _sample(lg, 2.0, u=float(p[0]) - 1e-3) == [0]
    assert _sample(lg, 2.0, u=float(p[0]) + 1e-3) == [1]
    assert _sample(lg, 2.0, u=float(p[1]) + 1e-3) == [2]
    # top-k 2 on [1,4,2,5,3] keeps ids 1 and 3 (:59-70)
    lg = torch.tensor([[1., 4., 2., 5., 3.]])
    seen = {_sample(lg, 1.0, top_k=2, u=u / 20)[0] for u in range(20)}
    assert seen == {1, 3}
    # penalty 2 on [2,-1,3,0] for ids {0,1} -> [1,-2,3,0] (:32-46): id 0 drops below id 2 by more
    lg = torch.tensor([[2., -1., 3., 0.]])
    p = torch.softmax(torch.tensor([1., -2., 3., 0.]), 0)
    assert _sample(lg, 1.0, pen=2.0, recent=[[0, 1]], u=float(p[0]) - 1e-3) == [0]
    assert _sample(lg, 1.0, pen=2.0, recent=[[0, 1]], u=float(p[0] + p[1]) + 1e-3) == [2]
