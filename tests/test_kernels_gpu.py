"""Each HIP kernel alone against a plain float64/float32 PyTorch reference of the same
operation, at sizes other than the engine's test models."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"
F16S = [torch.bfloat16, torch.float16]


@pytest.fixture(scope="module")
def ops():
    import llm_infer_amd  # noqa: F401
    from llm_infer_amd.kernels import ops as o
    return o


def _tol(dtype):
    return {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]


def test_embed(ops):
    g = torch.Generator().manual_seed(0)
    for dt in [torch.float32] + F16S:
        table = torch.randn(331, 80, generator=g).to(dt).to(DEV)
        toks = torch.tensor([0, 330, 17, 17, 5], dtype=torch.int32, device=DEV)
        out = ops.embed(table, toks)
        assert out.dtype == torch.float32
        assert torch.equal(out, table[toks.long()].float())


@pytest.mark.parametrize("d", [30, 64, 96, 100, 1000, 1022, 4096, 8192, 10000])
def test_rmsnorm(ops, d):
    g = torch.Generator().manual_seed(d)
    x = (torch.randn(7, d, generator=g) * 3).to(DEV)
    w = (1 + 0.1 * torch.randn(d, generator=g)).to(DEV)
    for eps in (1e-5, 1e-2):
        ref = (x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps) * w.double())
        for dt in [torch.float32] + F16S:
            out = ops.rmsnorm(x, w, eps, dt)
            assert out.dtype == dt
            assert torch.allclose(out.double(), ref, rtol=_tol(dt), atol=_tol(dt))
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    out = ops.rmsnorm(x, w, 1e-5, torch.float32, rows)
    assert torch.equal(out, ops.rmsnorm(x, w, 1e-5, torch.float32)[rows.long()])
    # eps inside the root: tiny inputs are scaled by 1/sqrt(eps), not blown up
    tiny = torch.full((1, d), 1e-4, device=DEV)
    out = ops.rmsnorm(tiny, torch.ones(d, device=DEV), 1e-2, torch.float32)
    assert torch.allclose(out, torch.full_like(out, 1e-4 / math.sqrt(1e-8 + 1e-2)), rtol=1e-5)


def _linear_ref(x, w, mode, res=None):
    y = x.double() @ w.double().t()
    if mode == 1:
        return res.double() + y
    if mode == 2:
        g, u = y[:, 0::2], y[:, 1::2]
        return g / (1 + torch.exp(-g)) * u
    if mode == 4:                                   # the gate's other activation: gelu in its tanh form
        g, u = y[:, 0::2], y[:, 1::2]
        return torch.nn.functional.gelu(g, approximate="tanh") * u
    return y


LIN_CASES = [  # M, N, K
    (1, 64, 64), (2, 16400, 4096), (16, 1000, 2056), (9, 40, 4104), (3, 172, 96), (8, 100, 256), (5, 6, 8), (13, 344, 64), (33, 130, 136),
    (64, 256, 512), (70, 200, 1024), (129, 384, 320), (200, 136, 72), (256, 512, 2048), (384, 256, 192),
    (927, 96, 16), (140, 40, 24),                   # K shorter than any tile's depth: the chunks past K are masked, not read
]


@pytest.mark.parametrize("M,N,K", LIN_CASES)
@pytest.mark.parametrize("dt", [torch.float32] + F16S)
def test_linear_all_kernels_and_epilogues(ops, M, N, K, dt):
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    x = torch.randn(M, K, generator=g).to(dt).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dt).to(DEV)
    res = torch.randn(M, N, generator=g).to(DEV)
    kinds = ["fma"]
    if dt != torch.float32:
        if M <= 16:
            kinds.append("gemv_mfma")
        kinds += ["mfma:0:1", "mfma:1:1", "mfma:2:1", "mfma:2:3", "mfma:0:2", "big:0", "big:1", "big:0:3", None]
    for kind in kinds:
        for mode in (0, 1, 2, 4):
            if mode in (2, 4) and N % 2:
                continue
            ref = _linear_ref(x, w, mode, res)
            if mode == 1:
                out = res.clone()
                ops.linear(x, w, mode, out=out, force=kind)
                tol = 1e-5 if dt == torch.float32 else 2e-4
            elif mode in (2, 4):
                out = ops.linear(x, w, mode, out_dtype=torch.float32, force=kind)
                tol = 1e-5 if dt == torch.float32 else 2e-4
            else:
                out = ops.linear(x, w, mode, out_dtype=torch.float32, force=kind)
                tol = 1e-5 if dt == torch.float32 else 2e-4
            err = (out.double() - ref).abs().max().item()
            assert err < tol * (1 + ref.abs().max().item()), (kind, mode, err)
            if dt != torch.float32 and mode != 1:
                out16 = ops.linear(x, w, mode, out_dtype=dt, force=kind)
                assert out16.dtype == dt
                assert torch.allclose(out16.double(), ref, rtol=_tol(dt), atol=_tol(dt))


TILED_CASES = [(1, 64, 64), (3, 172, 96), (16, 40, 4096), (9, 16400, 256), (17, 100, 64), (64, 256, 512),
               (33, 4100, 2048), (48, 72, 8192), (50, 6144, 4096), (65, 48, 32), (97, 200, 14336), (30, 520, 96), (128, 16, 160),
               (70, 200, 1024), (96, 1000, 416), (128, 136, 2048), (129, 384, 320), (256, 520, 2048), (384, 512, 192), (300, 1000, 96)]


@pytest.mark.parametrize("M,N,K", TILED_CASES)
@pytest.mark.parametrize("dt", F16S)
def test_linear_tiled_weights(ops, M, N, K, dt):
    """The same products with W kept in matrix-core order: every kernel that reads it, every epilogue."""
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    x = torch.randn(M, K, generator=g).to(dt).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dt).to(DEV)
    res = torch.randn(M, N, generator=g).to(DEV)
    wt = ops.tile_weight(w)
    assert ops.is_tiled(wt) and wt.logical == (N, K) and wt.numel() == (N + 15) // 16 * 16 * K and wt.owner == "device"
    assert torch.equal(ops.untile(wt), w.to(DEV))
    kinds = [None, "mfma:0:1", "mfma:1:2", "mfma:2:1", "big:0", "big:1", "big:0:2", "big:1:5"] + (["gemv_mfma"] if M <= 16 else [])
    # W into registers (tiles of 256, 192, 128 rows of W): the planner's choice and every tile, K whole and split
    kinds += ["wreg", "wreg:0", "wreg:1", "wreg:2", "wreg:0:2", "wreg:1:5", "wreg:2:3"]
    # the narrowest tile with W four steps ahead, with 64 rows of X (:1) and with 128 (:2), K whole and split
    kinds += ["wreg:2:1:1", "wreg:2:3:1", "wreg:2:1:2", "wreg:2:4:2", "wreg:2:1:3", "wreg:2:4:3"]        # (:3: three steps ahead)
    # workgroups that take fewer blocks of 16 rows of W than their tile has (the last field), for every tile
    kinds += ["wreg:2:1:1:7", "wreg:2:3:1:5", "wreg:2:1:2:6", "wreg:0:2:0:13", "wreg:1:1:0:9", "wreg:2:1:0:1"]
    # all of K in one workgroup, the rows of X through LDS of each wave's own (up to 128 rows): one and two tiles of W
    kinds += ["rows", "rows:1", "rows:2"] if M <= 128 else []
    for kind in kinds:
        for mode in (0, 1, 2, 4):
            if mode in (2, 4) and N % 2:
                continue
            ref = _linear_ref(x, w, mode, res)
            if mode == 1:
                out = res.clone()
                ops.linear(x, wt, mode, out=out, force=kind)
            else:
                out = ops.linear(x, wt, mode, out_dtype=torch.float32, force=kind)
            err = (out.double() - ref).abs().max().item()
            assert err < 2e-4 * (1 + ref.abs().max().item()), (kind, mode, err)
    if M <= 64:
        for nt, kw in ((1, 4), (1, 8), (2, 4), (2, 8)):
            if M > 32 and nt == 1:            # three or four tiles of rows of X go with two tiles of W
                continue
            out = ops.gemv_tiled(x, wt, out_dtype=torch.float32, nt=nt, kw=kw)
            assert (out.double() - _linear_ref(x, w, 0)).abs().max().item() < 2e-4 * 4
    if N % 32 == 0:
        head = ops.linear(x, wt.prefix(N // 2), out_dtype=torch.float32)
        assert (head.double() - _linear_ref(x, w[:N // 2], 0)).abs().max().item() < 2e-4 * 4
    with pytest.raises(ops.KernelError):
        ops.linear(x, wt, force="fma")
    with pytest.raises(ops.KernelError):
        ops.tile_weight(w[:, :K - 8].contiguous())


@pytest.mark.parametrize("dt", F16S)
@pytest.mark.parametrize("M,d,K2,N2", [(1, 4096, 4096, 6144), (8, 4096, 14336, 28672), (16, 96, 160, 200), (5, 2048, 64, 128256),
                                       (12, 4096, 14336, 28672), (16, 4096, 4096, 22016), (14, 4096, 4096, 6144)])
def test_norm_split_over_two_products(ops, M, d, K2, N2, dt):
    """A decode step's product that adds into the residual stream prepares the norm that reads the rows
    next (x * weight in 16 bits, sums of squares), and the product behind the norm finishes it: the same
    result as norm kernel + product, without the kernel.  The preparation is void as soon as anything
    else writes to the rows, and for any other norm.  (From 9 rows on, gate and up against a wide matrix finish
    the norm in the tiled GEMM's epilogue instead of gemv_tiled's: the last two cases.)"""
    g = torch.Generator().manual_seed(M + d)
    x0 = torch.randn(M, d, generator=g) * 3
    a = (torch.randn(M, K2, generator=g) * 0.5).to(dt)
    wo = (torch.randn(d, K2, generator=g) * 0.05).to(dt)
    wn = (1 + 0.1 * torch.randn(d, generator=g)).to(DEV)
    w2 = (torch.randn(N2, d, generator=g) * 0.05).to(dt)
    eps = 1e-5
    wot = ops.tile_weight(wo.to(DEV))
    x = x0.to(DEV)
    ops.linear(a.to(DEV), wot, ops.EPI_ADD, out=x)
    assert ops.lazy_rmsnorm(x, wn, eps, dt) is None                         # nobody said which norm comes next
    x = x0.to(DEV)
    ops.expect_norm(x, wn)
    ops.linear(a.to(DEV), wot, ops.EPI_ADD, out=x)
    x_ref = x0.double() + a.double() @ wo.double().t()
    assert (x.double().cpu() - x_ref).abs().max().item() < 1e-3 * (1 + x_ref.abs().max().item())
    ln = ops.lazy_rmsnorm(x, wn, eps, dt)
    assert isinstance(ln, ops.LazyNorm) and ln.dtype == dt and tuple(ln.shape) == (M, d)
    assert torch.allclose(ln.ss.double().sum(0).cpu()[:M], (x.double().cpu() ** 2).sum(1), rtol=1e-5)
    assert torch.allclose(ln.xw.double().cpu(), x.double().cpu() * wn.double().cpu() * ln.scale, rtol=2.0 ** -8)
    w2t = ops.tile_weight(w2.to(DEV))
    fused = ops.linear(ln, w2t, out_dtype=torch.float32)
    h = ops.rmsnorm(x, wn, eps, dt)
    assert torch.equal(ln.tensor(), h)
    plain = ops.linear(h, w2t, out_dtype=torch.float32)
    xd = x.double().cpu()
    ref = (xd / torch.sqrt((xd ** 2).mean(1, keepdim=True) + eps) * wn.double().cpu()) @ w2.double().t()
    own = (plain.double().cpu() - ref).abs().max().item()                   # what rounding the normed rows to 16 bits costs
    assert (fused.double().cpu() - ref).abs().max().item() < 1.5 * own + 1e-6
    # the gated epilogue, and a weight that is not tiled (the norm is then taken by its kernel)
    if N2 % 2 == 0:
        gated = ops.linear(ln, w2t, ops.EPI_SWIGLU, out_dtype=torch.float32)
        g_ref = torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2]
        g_own = (ops.linear(h, w2t, ops.EPI_SWIGLU, out_dtype=torch.float32).double().cpu() - g_ref).abs().max().item()
        assert (gated.double().cpu() - g_ref).abs().max().item() < 1.5 * g_own + 1e-6
    assert torch.equal(ops.linear(ln, w2.to(DEV)[:64].contiguous(), out_dtype=torch.float32),
                       ops.linear(h, w2.to(DEV)[:64].contiguous(), out_dtype=torch.float32))
    # anything else that writes to the rows voids the preparation; so does another norm's weight
    assert ops.lazy_rmsnorm(x, wn.clone(), eps, dt) is None
    assert ops.lazy_rmsnorm(x, wn, eps, torch.float32) is None              # a 32-bit norm is never deferred
    x += 1.0
    assert ops.lazy_rmsnorm(x, wn, eps, dt) is None
    ops.linear(a.to(DEV), wot, ops.EPI_ADD, out=x)
    assert ops.lazy_rmsnorm(x, wn, eps, dt) is not None
    ops.linear(a.to(DEV), wo.to(DEV), ops.EPI_ADD, out=x)                   # a kernel that prepares nothing
    assert ops.lazy_rmsnorm(x, wn, eps, dt) is None
    ops.linear(a.to(DEV), wot, ops.EPI_ADD, out=x)
    assert ops.lazy_rmsnorm(x.view(M, d), wn, eps, dt) is None              # another tensor object, no record
    if M < 16:
        big = torch.zeros(17, d, device=DEV)
        ops.expect_norm(big, wn)
        ops.linear(torch.zeros(17, K2, device=DEV, dtype=dt), wot, ops.EPI_ADD, out=big)
        assert ops.lazy_rmsnorm(big, wn, eps, dt) is None                   # more than 16 rows: the norm kernel


@pytest.mark.parametrize("dt", F16S)
@pytest.mark.parametrize("M,N2", [(7, 768), (12, 65536)])
@pytest.mark.parametrize("rms,wscale", [(1e-2, 0.02), (1e3, 0.02), (1e3, 4.0), (3.0, 1.0)])
def test_norm_split_over_two_products_at_a_models_own_scale(ops, rms, wscale, M, N2, dt):
    """The rows that travel in 16 bits between the two products are x * weight; a checkpoint's residual stream
    may be of the order of 0.01 or of 1000 and its norm weights of 0.02.  In float16 each row is scaled by a
    power of two taken from the norm before (left by the norm kernel, then by each product that finishes a
    norm), so the split norm is as exact as norm kernel + product at every scale, down a chain of layers in
    which the rows grow; a view of the rows that a kernel writes through voids the preparation too.  The second
    shape is gate and up of 12 rows against a wide matrix, where the tiled GEMM finishes the norm and leaves the
    scales."""
    d, K2 = 1024, 512
    gated = N2 > 768
    assert not gated or ops._wreg_plan(M, N2, d) == (2, 1)
    mode = ops.EPI_SWIGLU if gated else ops.EPI_STORE
    g = torch.Generator().manual_seed(3)
    x0 = torch.randn(M, d, generator=g) * rms
    x0[2, 5] = 40 * rms                                            # a row with one large element
    wn = (wscale * (1 + 0.3 * torch.randn(d, generator=g))).to(DEV)
    # (the product's own operands stay of moderate size in 16 bits: what it adds is of the order of rms 3^layer)
    wo = (torch.randn(d, K2, generator=g) * 0.05 * rms / 34).to(dt)
    w2 = (torch.randn(N2, d, generator=g) * 0.05).to(dt)
    wot, w2t = ops.tile_weight(wo.to(DEV)), ops.tile_weight(w2.to(DEV))
    eps = 1e-6
    x = x0.to(DEV)
    ops.rmsnorm(x, wn, eps, dt)                                    # the norm before: in float16 it leaves the rows' scales
    assert (getattr(x, "_li_row_scale", None) is not None) == (dt == torch.float16)
    for layer in range(3):                                         # the rows grow by a factor of about 3 a layer
        a = (torch.randn(M, K2, generator=g) * 30 * 3 ** layer).to(dt)
        ops.expect_norm(x, wn)
        ops.linear(a.to(DEV), wot, ops.EPI_ADD, out=x)
        ln = ops.lazy_rmsnorm(x, wn, eps, dt)
        assert ln is not None and (ln.row_scales is not None) == (dt == torch.float16)
        assert torch.isfinite(ln.xw.float()).all()
        fused = ops.linear(ln, w2t, mode, out_dtype=torch.float32)
        assert (getattr(x, "_li_row_scale", None) is not None) == (dt == torch.float16)
        xd = x.double().cpu()
        ref = (xd / torch.sqrt((xd ** 2).mean(1, keepdim=True) + eps) * wn.double().cpu()) @ w2.double().t()
        if gated:
            ref = torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2]
        plain = ops.linear(ops.rmsnorm(x.clone(), wn, eps, dt), w2t, mode, out_dtype=torch.float32)
        # (a gated product's largest errors sit at its few largest outputs, and the largest of them differs by a
        # factor of two between two roundings of the same quality: there the root mean square is compared)
        size = (lambda e: e.pow(2).mean().sqrt().item()) if gated else (lambda e: e.abs().max().item())
        own = size(plain.double().cpu() - ref)
        err = size(fused.double().cpu() - ref)
        assert err < 1.5 * own + 1e-6 * size(ref), (layer, err, own)
    # a kernel that writes through a view of the rows voids what was prepared for the rows themselves
    ops.expect_norm(x, wn)
    ops.linear(a.to(DEV), wot, ops.EPI_ADD, out=x)
    assert ops.lazy_rmsnorm(x, wn, eps, dt) is not None
    ops.linear(a.to(DEV)[:4].contiguous(), wot, ops.EPI_ADD, out=x[:4])
    assert ops.lazy_rmsnorm(x, wn, eps, dt) is None


def test_gate_activation_alone(ops):
    """act(gate) * up on interleaved columns, for a product that was stored unactivated."""
    g = torch.Generator().manual_seed(3)
    gu = (torch.randn(5, 2 * 173, generator=g) * 3).to(DEV)
    gate, up = gu[:, 0::2].double(), gu[:, 1::2].double()
    for gelu, ref in ((False, gate / (1 + torch.exp(-gate)) * up),
                      (True, torch.nn.functional.gelu(gate, approximate="tanh") * up)):
        out = ops.swiglu(gu, torch.float32, gelu=gelu)
        assert out.shape == (5, 173) and (out.double() - ref).abs().max() < 1e-5 * (1 + ref.abs().max())
        assert ops.swiglu(gu, torch.bfloat16, gelu=gelu).dtype == torch.bfloat16


@pytest.mark.parametrize("dt", F16S)
@pytest.mark.parametrize("M,d,K2", [(17, 256, 2048), (64, 4096, 4096), (200, 1000, 8192), (300, 96, 2080)])
def test_norm_taken_by_the_sum_of_split_products(ops, M, d, K2, dt):
    """With K split, the kernel that adds the partial sums into the residual rows also takes the norm that
    reads them next: bit for bit what the reduction and the norm kernel give, one kernel less.  Void as soon
    as anything else writes to the rows, for another weight or eps, and never made when K is not split."""
    g = torch.Generator().manual_seed(M + d)
    x0 = torch.randn(M, d, generator=g) * 3
    a = (torch.randn(M, K2, generator=g) * 0.5).to(dt).to(DEV)
    wot = ops.tile_weight((torch.randn(d, K2, generator=g) * 0.05).to(dt).to(DEV))
    wn = (1 + 0.1 * torch.randn(d, generator=g)).to(DEV)
    eps = 1e-5
    plain = x0.to(DEV)
    ops.linear(a, wot, ops.EPI_ADD, out=plain, force="wreg:2:2")
    assert ops.prepared_rmsnorm(plain, wn, eps, dt) is None                 # nobody said which norm comes next
    x = x0.to(DEV)
    ops.expect_norm(x, wn, eps)
    ops.linear(a, wot, ops.EPI_ADD, out=x, force="wreg:2:2")
    assert torch.equal(x, plain)
    ready = ops.prepared_rmsnorm(x, wn, eps, dt)
    assert ready is not None and ready.dtype == dt and torch.equal(ready, ops.rmsnorm(x, wn, eps, dt))
    assert ops.prepared_rmsnorm(x, wn.clone(), eps, dt) is None and ops.prepared_rmsnorm(x, wn, 2 * eps, dt) is None
    assert ops.prepared_rmsnorm(x, wn, eps, torch.float32) is None
    x += 1.0
    assert ops.prepared_rmsnorm(x, wn, eps, dt) is None                     # torch wrote to the rows
    y = x0.to(DEV)
    ops.expect_norm(y, wn, eps)
    ops.linear(a, wot, ops.EPI_ADD, out=y, force="wreg:2:2")
    ops.linear(a, wot, ops.EPI_ADD, out=y, force="wreg:2:1")                # a product without a split wrote to them
    assert ops.prepared_rmsnorm(y, wn, eps, dt) is None
    # the planner's own choice at these sizes
    z = x0.to(DEV)
    ops.expect_norm(z, wn, eps)
    ops.linear(a, wot, ops.EPI_ADD, out=z)
    ready = ops.prepared_rmsnorm(z, wn, eps, dt)
    assert ready is None or torch.equal(ready, ops.rmsnorm(z, wn, eps, dt))
    # (where the product runs as gemm_rows, all of K in a workgroup, there is no second kernel to take the norm)
    assert M < 64 or ops._wreg_plan(M, d, K2)[1] == 1 or ops._rows_plan(M, d, K2, True) or ready is not None


@pytest.mark.parametrize("M,N,K", [(2048, 8560, 736), (5000, 4048, 736), (1300, 12288, 4096)])
def test_large_products(ops, M, N, K):
    """Products of many tiles as the planner runs them: a K that is 32 more than a multiple of 64, widths and
    heights that end inside a tile."""
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).to(torch.float16).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.float16).to(DEV)
    out = ops.linear(x, ops.tile_weight(w), out_dtype=torch.float32)
    for r0 in range(0, M, 4096):                       # the reference in slices: it is float64
        ref = x[r0:r0 + 4096].double() @ w.double().t()
        assert (out[r0:r0 + 4096].double() - ref).abs().max().item() < 2e-4 * (1 + ref.abs().max().item())


def test_linear_rows_do_not_depend_on_the_batch_in_float32(ops):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(70, 136, generator=g).to(DEV)
    w = torch.randn(100, 136, generator=g).to(DEV)
    whole = ops.linear(x, w, out_dtype=torch.float32)
    for r in (0, 63, 64, 69):
        assert torch.equal(ops.linear(x[r:r + 1].contiguous(), w, out_dtype=torch.float32)[0], whole[r])


def test_linear_mixed_precision_weights_stay_32_bit(ops):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 64, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randn(32, 64, generator=g).to(DEV)                     # float32 weight, bfloat16 activations
    out = ops.linear(x, w, out_dtype=torch.float32)
    assert torch.allclose(out.double(), x.double() @ w.double().t(), atol=1e-4)


def test_linear_refuses_what_it_cannot_do(ops):
    x = torch.randn(4, 12).to(torch.bfloat16).to(DEV)
    w = torch.randn(6, 12).to(torch.bfloat16).to(DEV)
    with pytest.raises(ops.KernelError):
        ops.linear(x, w, force="gemv_mfma")                           # K = 12 is no multiple of 8
    with pytest.raises(ops.KernelError):
        ops.linear(x, w, force="mfma:0:1")
    out = ops.linear(x, w, out_dtype=torch.float32)                  # the general kernel takes it
    assert torch.allclose(out.double(), x.double() @ w.double().t(), atol=1e-4)
    with pytest.raises(ops.KernelError):
        ops.linear(x, w[:5].contiguous(), 2)                          # SwiGLU needs gate/up pairs


# ---------------------------------------------------------------------------
# attention over the paged cache
# ---------------------------------------------------------------------------
def _fill_cache(ops, dtype, K, hd, seqs, n_slots=8, window=None):
    """Writes k, v (no rotation) for sequences given as (slot, k [n, K, hd], v) into a fresh cache."""
    from llm_infer_amd.cache import Cache, KVSpec
    total = sum(k.shape[0] for _, k, _ in seqs)
    cache = Cache([KVSpec(K, hd, window)], max_tokens=total + 64 * len(seqs) + 64, max_positions=4096,
                  dtype=dtype, device=DEV, n_slots=n_slots)
    view = None
    for slot_hint, k, v in seqs:
        slot = cache.alloc_slot()
        assert slot == slot_hint
        n = k.shape[0]
        cache.grow([slot], [n])
        view = cache.view(0)
        qkv = torch.cat([torch.zeros(n, 1 * hd), k.reshape(n, K * hd).float(), v.reshape(n, K * hd).float()], 1).to(DEV)
        pos = torch.arange(n, dtype=torch.int32, device=DEV)
        ts = torch.full((n,), slot, dtype=torch.int32, device=DEV)
        ops.rope_store(qkv.contiguous(), None, 0, False, pos, ts, view.page_table, view.page_stride, view.k, view.v,
                       1, K, hd, dtype)
    return cache, view


def _attn_ref(q, k, v, window=None):
    import plain_llama as P
    return P.attention(q.double(), k.double(), v.double(), window)


ATTN_CASES = [  # H, K, hd, lengths
    (4, 2, 16, [7, 1, 13]), (3, 1, 32, [1, 4, 9, 16, 31]), (5, 5, 48, [70, 64, 65]),
    (8, 2, 64, [200, 3]), (8, 1, 128, [130, 257]), (2, 2, 80, [66]), (40, 1, 16, [5, 90]),
]


@pytest.mark.parametrize("H,K,hd,lens", ATTN_CASES)
@pytest.mark.parametrize("dt", [torch.float32] + F16S)
def test_attention_whole_prompts_and_decode(ops, H, K, hd, lens, dt):
    g = torch.Generator().manual_seed(H * 100 + hd)
    seqs, qs = [], []
    for i, n in enumerate(lens):
        k = torch.randn(n, K, hd, generator=g).to(dt)
        v = torch.randn(n, K, hd, generator=g).to(dt)
        q = (torch.randn(n, H, hd, generator=g) * 1.5).to(dt)
        seqs.append((i, k, v))
        qs.append(q)
    cache, view = _fill_cache(ops, dt, K, hd, seqs)
    scale = hd ** -0.5
    refs = [_attn_ref(q.float(), k.float(), v.float()) for q, (_, k, v) in zip(qs, seqs)]
    tol = {torch.float32: 2e-5, torch.float16: 3e-3, torch.bfloat16: 2.5e-2}[dt]
    # all sequences whole, in one step
    from llm_infer_amd.engine.step import StepContext
    ctx = StepContext(DEV, list(range(len(lens))), [[0] * n for n in lens], [0] * len(lens), [[] for _ in lens])
    q_all = torch.cat(qs).to(DEV).contiguous()
    if dt == torch.float32:
        out = ops.attention_f32(q_all, view.as_tuple(), ctx.pos, ctx.tok_slot, H, K, hd, scale, None)
    else:
        out = ops.attention_prefill(q_all, view.as_tuple(), ops.prefill_meta(ctx), H, K, hd, scale, None)
    ref_all = torch.cat(refs)
    err = (out.double().cpu() - ref_all).abs().max().item()
    assert err < tol, err
    # the last token of every sequence as a decode step, with every split count
    q_last = torch.stack([q[-1] for q in qs]).to(DEV).contiguous()
    ref_last = torch.stack([r[-1] for r in refs])
    seq_slot = torch.arange(len(lens), dtype=torch.int32, device=DEV)
    seq_ctx = torch.tensor(lens, dtype=torch.int32, device=DEV)
    if dt == torch.float32:
        pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=DEV)
        out = ops.attention_f32(q_last, view.as_tuple(), pos, seq_slot, H, K, hd, scale, None)
        assert (out.double().cpu() - ref_last).abs().max().item() < tol
    else:
        for splits in (1, 2, 3, 4, 8, 16, 24):               # merged inside a workgroup, by the merge kernel, or both
            out = ops.attention_decode(q_last, view.as_tuple(), seq_slot, seq_ctx, len(lens), H, K, hd, scale,
                                       None, splits)
            err = (out.double().cpu() - ref_last).abs().max().item()
            assert err < tol, (splits, err)


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_attention_window_and_far_key(ops, dt):
    """One far key among hundreds stands out by its score; the window cuts it off exactly at its edge."""
    H, K, hd, n = 2, 1, 32, 300
    g = torch.Generator().manual_seed(5)
    k = (torch.randn(n, K, hd, generator=g) * 0.1)
    v = torch.randn(n, K, hd, generator=g)
    q = torch.randn(n, H, hd, generator=g) * 0.1
    far = 37
    k[far, 0, :] = 0
    k[far, 0, 3] = 12.0
    q[:, :, 3] = 6.0                      # every query looks hard at key `far`
    k, v, q = k.to(dt), v.to(dt), q.to(dt)
    cache, view = _fill_cache(ops, dt, K, hd, [(0, k, v)])
    from llm_infer_amd.engine.step import StepContext
    ctx = StepContext(DEV, [0], [[0] * n], [0], [[]])
    scale = hd ** -0.5
    tol = 2e-5 if dt == torch.float32 else 2.5e-2
    for window in (None, 100, 64, 1):
        ref = _attn_ref(q.float(), k.float(), v.float(), window)
        qd = q.to(DEV).contiguous()
        if dt == torch.float32:
            out = ops.attention_f32(qd, view.as_tuple(), ctx.pos, ctx.tok_slot, H, K, hd, scale, window)
        else:
            out = ops.attention_prefill(qd, view.as_tuple(), ops.prefill_meta(ctx), H, K, hd, scale, window)
        assert (out.double().cpu() - ref).abs().max().item() < tol, window
        if window == 100:
            # position far+99 still sees the far key, far+100 does not
            o = out.float().cpu()
            assert (o[far + 99, 0] - v[far, 0].float()).abs().max() < 0.05
            assert (o[far + 100, 0] - v[far, 0].float()).abs().max() > 0.2
        if dt != torch.float32:
            last = qd[-1:].contiguous()
            out1 = ops.attention_decode(last, view.as_tuple(), torch.zeros(1, dtype=torch.int32, device=DEV),
                                        torch.tensor([n], dtype=torch.int32, device=DEV), 1, H, K, hd, scale,
                                        window, 2)
            assert (out1.double().cpu()[0] - ref[-1]).abs().max().item() < tol


@pytest.mark.parametrize("dt", F16S)
@pytest.mark.parametrize("window", [100, 64])
def test_decode_attention_at_the_window_edge(ops, dt, window):
    """The 16-bit decode kernel cuts the window exactly: a far key that outweighs all others is seen by
    the last position that may see it and not by the next, with every count of splits; and with the
    pages below the window given back and everything free filled with NaN."""
    H, K, hd, n = 2, 1, 32, 300
    scale = hd ** -0.5
    tol = 3e-3 if dt == torch.float16 else 2.5e-2

    def make(far):
        g = torch.Generator().manual_seed(far)
        k = torch.randn(n, K, hd, generator=g) * 0.1
        v = torch.randn(n, K, hd, generator=g)
        q = torch.randn(n, H, hd, generator=g) * 0.1
        k[far, 0, :] = 0
        k[far, 0, 3] = 12.0
        q[:, :, 3] = 6.0
        return k.to(dt), v.to(dt), q.to(dt)

    def decode(view, q_row, ctx_len, splits):
        return ops.attention_decode(q_row.to(DEV).contiguous(), view.as_tuple(), torch.zeros(1, dtype=torch.int32, device=DEV),
                                    torch.tensor([ctx_len], dtype=torch.int32, device=DEV), 1, H, K, hd, scale,
                                    window, splits).float().cpu()[0]

    # a cache that keeps everything; the context length moves over the edge
    far = 37
    k, v, q = make(far)
    cache, view = _fill_cache(ops, dt, K, hd, [(0, k, v)])
    ref = _attn_ref(q.float(), k.float(), v.float(), window)
    for splits in (1, 2, 8):
        for ctx_len, sees in ((far + window, True), (far + window + 1, False)):
            out = decode(view, q[ctx_len - 1:ctx_len], ctx_len, splits)
            assert (out.double() - ref[ctx_len - 1]).abs().max().item() < tol, (splits, ctx_len)
            assert ((out[0] - v[far, 0].float()).abs().max() < 0.05) == sees, (splits, ctx_len)
    # a cache of a window group: pages that lie wholly below the window are given back, and whatever is
    # free (the page that free table entries point at included) holds NaN
    for far, sees in ((n - window, True), (n - window - 1, False)):
        k, v, q = make(far)
        cache, view = _fill_cache(ops, dt, K, hd, [(0, k, v)], window=window)
        cache.trim_windows([0])
        group = cache.groups[0]
        first = group.first_needed_page(n)
        assert first >= 3 and sorted(group.pages_of[0]) == list(range(first, (n + 63) // 64))
        free = [p for p in range(group.n_pages) if p not in group.pool.held()]
        group.storage[torch.tensor(free, device=DEV)] = float("nan")
        ref = _attn_ref(q.float(), k.float(), v.float(), window)[-1]
        for splits in (1, 2, 8):
            out = decode(view, q[-1:], n, splits)
            assert torch.isfinite(out).all(), (far, splits)
            assert (out.double() - ref).abs().max().item() < tol, (far, splits)
            assert ((out[0] - v[far, 0].float()).abs().max() < 0.05) == sees, (far, splits)


def test_rope_store_rotation_and_cache_layout(ops):
    """Rotation against the plain formula, both pairings, partial rotary dim; keys read back
    through attention with a one-hot query."""
    import plain_llama as P
    H, K, hd, rot, n = 2, 2, 32, 16, 70
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn(n, (H + 2 * K) * hd, generator=g)
    from llm_infer_amd.cache import Cache, KVSpec
    cache = Cache([KVSpec(K, hd)], 256, 1024, torch.float32, DEV, 2)
    slot = cache.alloc_slot()
    cache.grow([slot], [n])
    view = cache.view(0)
    pos = torch.arange(n, dtype=torch.int32, device=DEV)
    ts = torch.zeros(n, dtype=torch.int32, device=DEV)
    i = torch.arange(0, rot, 2, dtype=torch.float32)
    inv = (1.0 / torch.pow(torch.tensor(10000.0), i / rot)).to(DEV)
    q = ops.rope_store(qkv.to(DEV), inv, rot, False, pos, ts, view.page_table, view.page_stride, view.k, view.v,
                       H, K, hd, torch.float32)
    ref_q = P.rope(qkv[:, :H * hd].view(n, H, hd).double(), torch.arange(n), 10000.0, rot)
    assert torch.allclose(q.double().cpu(), ref_q, atol=2e-5)
    ref_k = P.rope(qkv[:, H * hd:(H + K) * hd].view(n, K, hd).double(), torch.arange(n), 10000.0, rot)
    ref_v = qkv[:, (H + K) * hd:].view(n, K, hd).double()
    # read keys back: a one-hot query at dim j gives scores k[t, j]; check through decode attention
    # on the values instead: attention with all-equal scores averages v
    zero_q = torch.zeros(1, H, hd, device=DEV)
    out = ops.attention_f32(zero_q, view.as_tuple(), torch.tensor([n - 1], dtype=torch.int32, device=DEV),
                            torch.zeros(1, dtype=torch.int32, device=DEV), H, K, hd, 1.0, None)
    assert torch.allclose(out[0].double().cpu(), ref_v.mean(0), atol=1e-5)
    # keys: q = e_j * big picks the token with the largest k[:, j]
    for j in (0, 5, 17, 31):
        qq = torch.zeros(1, H, hd, device=DEV)
        qq[0, :, j] = 200.0
        out = ops.attention_f32(qq, view.as_tuple(), torch.tensor([n - 1], dtype=torch.int32, device=DEV),
                                torch.zeros(1, dtype=torch.int32, device=DEV), H, K, hd, 1.0, None)
        for h in range(H):
            best = ref_k[:, h, j].argmax().item()
            assert torch.allclose(out[0, h].double().cpu(), ref_v[best, h], atol=1e-3), (j, h)
    # half pairing equals the plain rotation applied to de-interleaved heads
    q2 = ops.rope_store(qkv.to(DEV), inv, rot, True, pos, ts, None, None, None, None, H, 0, hd, torch.float32)
    x = qkv[:, :H * hd].view(n, H, hd).double()
    perm = torch.cat([torch.stack([torch.arange(rot // 2), torch.arange(rot // 2) + rot // 2], 1).reshape(-1),
                      torch.arange(rot, hd)])
    ref_half = torch.empty_like(x)
    ref_half[..., perm] = P.rope(x[..., perm], torch.arange(n), 10000.0, rot)
    assert torch.allclose(q2.double().cpu(), ref_half, atol=2e-5)


@pytest.mark.parametrize("dt", F16S)
@pytest.mark.parametrize("T,H,K,hd,rot,d", [(1, 4, 2, 16, 16, 64), (9, 3, 1, 32, 16, 96), (70, 5, 5, 48, 24, 160),
                                           (200, 8, 2, 64, 64, 256), (3, 2, 0, 32, 32, 64)])
def test_rotation_fused_into_the_projection(ops, dt, T, H, K, hd, rot, d):
    """The product whose epilogue rotates and stores equals the product followed by rope_store:
    q and the cache pages within one rounding of the stored dtype when both use the same sums."""
    from llm_infer_amd.cache import Cache, KVSpec
    g = torch.Generator().manual_seed(T + hd)
    x = torch.randn(T, d, generator=g).to(dt).to(DEV)
    w = (torch.randn((H + 2 * K) * hd, d, generator=g) / math.sqrt(d)).to(dt).to(DEV)
    inv = (1.0 / torch.pow(torch.tensor(500.0), torch.arange(0, rot, 2, dtype=torch.float32) / rot)).to(DEV)
    pos = (torch.arange(T, dtype=torch.int32) + 60).to(DEV)
    ts = torch.zeros(T, dtype=torch.int32, device=DEV)

    def fresh():
        c = Cache([KVSpec(max(K, 1), hd)], 512, 1024, dt, DEV, 2)
        s_ = c.alloc_slot()
        c.grow([s_], [60 + T])
        return c, c.view(0)

    c0, v0 = fresh()
    qkv = ops.linear(x, w, out_dtype=torch.float32, force="fma")
    args0 = (v0.page_table, v0.page_stride, v0.k, v0.v) if K else (None, None, None, None)
    q0 = ops.rope_store(qkv, inv, rot, False, pos, ts, *args0, H, K, hd, dt)
    kinds = ["fma", None] + (["gemv_mfma"] if T <= 16 else []) + ["mfma:0:1", "mfma:2:2"]
    for tiled in (False, True):
        if tiled and d % 32:
            continue
        ww = ops.tile_weight(w) if tiled else w
        for kind in kinds + (["wreg:0", "wreg:1:2", "wreg:2"] if tiled else []):
            if tiled and kind == "fma":
                continue
            c1, v1 = fresh()
            args1 = (v1.page_table, v1.page_stride, v1.k, v1.v) if K else (None, None, None, None)
            table = ops.rope_table(inv, pos, T) if kind != "fma" else None     # with and without the table
            q1 = ops.linear_rope_store(x, ww, inv, rot, pos, ts, *args1, H, K, hd, dt, force=kind, cos_sin=table)
            # the same float32 sums on the "fma" path: at most one rounding of the stored dtype apart
            tol = (2.0 ** -9 if dt == torch.float16 else 2.0 ** -7) if kind == "fma" else 2e-2
            assert (q1.float() - q0.float()).abs().max().item() <= tol * (1 + q0.float().abs().max().item()), kind
            if K:
                a, b = c0.groups[0].storage.float(), c1.groups[0].storage.float()
                assert (a - b).abs().max().item() <= tol * (1 + a.abs().max().item()), kind
                assert (b != 0).sum().item() >= 0.9 * T * 2 * K * hd


def test_token_probability(ops):
    import plain_llama as P
    g = torch.Generator().manual_seed(5)
    for V in (7, 65, 331, 5000, 128256, 300007):
        logits = torch.randn(5, V, generator=g) * 4
        logits[0, V // 2] = 40.0                                   # nearly all the mass on one token
        tokens = [V // 2, 0, V - 1, V, -1]                         # the last two lie outside the vocabulary
        got = ops.token_prob(logits.to(DEV), torch.tensor(tokens, dtype=torch.int32, device=DEV)).cpu()
        want = torch.tensor([P.token_prob(logits[i].double(), t) for i, t in enumerate(tokens)])
        assert got[3] == 0 and got[4] == 0
        torch.testing.assert_close(got, want.float(), rtol=2e-5, atol=1e-12)
        assert got[0] > 0.999
        # all tokens of a row add up to one
        row = logits[1:2].expand(V, V).contiguous().to(DEV) if V <= 331 else None
        if row is not None:
            every = ops.token_prob(row, torch.arange(V, dtype=torch.int32, device=DEV))
            assert abs(every.double().sum().item() - 1.0) < 1e-5


def test_sampling_kernels(ops):
    import plain_llama as P
    g = torch.Generator().manual_seed(0)
    for V in (7, 64, 65, 256, 331, 5000, 128256, 300007):      # one chunk, 32 chunks, chunks longer than 4,096
        logits = torch.randn(6, V, generator=g) * 3
        logits[1, 3] = logits[1, V - 2] = 50.0                    # a tie: the first wins
        logits[2, V - 1] = 60.0
        d = logits.to(DEV)
        got = ops.argmax(d).tolist()
        assert got == [P.sample_greedy(r) for r in logits]
        assert got[1] == 3 and got[2] == V - 1
        for T in (0.01, 0.8, 2.0, 1e6):             # from nearly only the maximum to nearly equal chances
            rs = [0.0, 0.25, 0.5, 0.75, 0.999, 0.9999999]
            r = torch.tensor(rs, dtype=torch.float32, device=DEV)
            got = ops.sample(d, T, forced_r=r).tolist()
            for b in range(6):
                p = P.probabilities(logits[b].double(), T)
                c = torch.cumsum(p, 0)
                lo = c[got[b] - 1].item() if got[b] > 0 else 0.0
                hi = c[got[b]].item()
                assert lo - 1e-5 <= rs[b] < hi + 1e-5, (V, T, b, got[b])
        assert ops.sample(d, 0.0).tolist() == ops.argmax(d).tolist()
    # the generator: host twin equals the device, streams differ by key, counter advances
    state = torch.tensor([[11, 0], [12, 0]], dtype=torch.int64, device=DEV)
    slots = torch.tensor([1, 0], dtype=torch.int32, device=DEV)
    logits = torch.zeros(2, 64, device=DEV)                     # uniform distribution: token = floor(r * 64)
    t1 = ops.sample(logits, 1.0, slots, state).tolist()
    t2 = ops.sample(logits, 1.0, slots, state).tolist()
    assert state[:, 1].tolist() == [2, 2]
    assert t1 == [int(ops.uniform01(12, 0) * 64), int(ops.uniform01(11, 0) * 64)]
    assert t2 == [int(ops.uniform01(12, 1) * 64), int(ops.uniform01(11, 1) * 64)]
    us = [ops.uniform01(5, i) for i in range(2000)]
    assert 0.45 < sum(us) / len(us) < 0.55 and min(us) >= 0.0 and max(us) < 1.0
    # drawn tokens follow the probabilities: 8192 sequences with generators of their own, one draw each
    n, V = 8192, 7
    row = torch.tensor([2.0, 0.5, -1.0, 1.5, 0.0, -3.0, 1.0])
    p = P.probabilities(row.double(), 0.7)
    state = torch.stack([torch.arange(n, dtype=torch.int64) + 1000, torch.zeros(n, dtype=torch.int64)], 1).to(DEV)
    drawn = ops.sample(row.repeat(n, 1).to(DEV), 0.7, torch.arange(n, dtype=torch.int32, device=DEV), state)
    freq = torch.bincount(drawn.cpu().long(), minlength=V).double() / n
    sigma = torch.sqrt(p * (1 - p) / n)
    assert ((freq - p).abs() < 5 * sigma + 1e-9).all(), (freq.tolist(), p.tolist())
