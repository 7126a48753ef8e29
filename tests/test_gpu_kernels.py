"""Each kernel alone against its plain reference, at sizes other than the engine's."""
import math

import pytest
import torch

import plain_llama as P
from gpu_tools import DEV, PagedKV, attention_ctx

pytestmark = pytest.mark.gpu

F32, BF16 = torch.float32, torch.bfloat16


@pytest.fixture(autouse=True)
def _ops():
    from photon_infer_amd import ops
    prev = ops.use_fast_kernels(True)
    yield ops
    ops.use_fast_kernels(prev)


def gen(seed):
    return torch.Generator().manual_seed(seed)


def close(got, want, rel, what=""):
    scale = max(1e-6, want.abs().max().item())
    err = (got.float().cpu() - want.float()).abs().max().item()
    assert err <= rel * scale, f"{what}: max error {err:.3e} exceeds {rel:.1e} x scale {scale:.3e}"


# ------------------------------------------------------------------ embedding
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_embedding(_ops, dtype):
    table = torch.randn(1001, 72, generator=gen(0)).to(dtype)
    ids = torch.tensor([0, 1000, 5, 5, 77], dtype=torch.int32)
    out = torch.empty(5, 72, dtype=F32, device=DEV)
    _ops.embedding(out, table.to(DEV), ids.to(DEV))
    assert torch.equal(out.cpu(), P.embedding(table.float(), ids.tolist()))
    bad = torch.tensor([3, 1001, -1], dtype=torch.int32, device=DEV)   # outside the table: NaN rows, no fault
    out = torch.zeros(3, 72, dtype=F32, device=DEV)
    _ops.embedding(out, table.to(DEV), bad)
    assert not out[0].isnan().any() and out[1:].isnan().all()


# ------------------------------------------------------------------ RMS norm
@pytest.mark.parametrize("D", [24, 100, 1000, 2048, 4100])
@pytest.mark.parametrize("out_dtype,w_dtype", [(F32, F32), (BF16, BF16), (BF16, F32)])
def test_rmsnorm(_ops, D, out_dtype, w_dtype):
    x = torch.randn(7, D, generator=gen(D)) * 3 + 0.5
    w = (torch.rand(D, generator=gen(1)) + 0.5).to(w_dtype)
    out = torch.empty(7, D, dtype=out_dtype, device=DEV)
    _ops.rmsnorm(out, x.to(DEV), w.to(DEV), 1e-6)
    want = P.rmsnorm(x, w.float(), 1e-6)
    close(out, want, 2e-6 if out_dtype == F32 else 2 ** -8, f"rmsnorm D={D}")
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    out2 = torch.empty(3, D, dtype=out_dtype, device=DEV)
    _ops.rmsnorm(out2, x.to(DEV), w.to(DEV), 1e-6, rows)
    assert torch.equal(out2, out[[6, 0, 3]])


@pytest.mark.parametrize("D", [24, 1001, 2048, 4100])
@pytest.mark.parametrize("splits", [1, 3, 4, 9])
@pytest.mark.parametrize("out_dtype", [F32, BF16])
def test_rmsnorm_adds_the_pieces_of_a_pending_update_first(_ops, D, splits, out_dtype):
    """A product into the stream that was split over k waits in the workspace; the norm adds its
    pieces (in split order), writes the sum back into the stream and normalises it, in one pass:
    all rows, or only the rows it is asked for.  D = 1001 takes the general kernel, the others
    the kernel with 16-byte accesses (one, one and two groups per thread)."""
    from photon_infer_amd.ops.workspace import Partials, PendingUpdate
    M = 7
    x0 = torch.randn(M, D, generator=gen(D)) * 2 + 0.25
    pieces = torch.randn(splits, M, D, generator=gen(D + splits))
    w = (torch.rand(D, generator=gen(1)) + 0.5).to(out_dtype)
    total = x0.double() + pieces.double().sum(0)
    want = P.rmsnorm(total, w.double(), 1e-5)
    tol = 3e-6 if out_dtype == F32 else 2 ** -8
    for rows in (None, [5, 0, 3]):
        ws = _ops.KernelWorkspace(DEV)
        x = x0.clone().to(DEV)
        ws.pending = PendingUpdate(x, Partials(pieces.to(DEV), splits, M, D))
        sel = list(range(M)) if rows is None else rows
        out = torch.full((len(sel), D), float("nan"), dtype=out_dtype, device=DEV)
        _ops.rmsnorm(out, x, w.to(DEV), 1e-5, None if rows is None else torch.tensor(rows, dtype=torch.int32, device=DEV), ws=ws)
        assert ws.pending is None and ws.counts["added_by_norm"] == 1
        close(out, want[sel], tol, f"norm of stream + pieces, D={D} splits={splits} rows={rows}")
        close(x[sel], total[sel], 1e-6, "the stream holds the sum afterwards")
        others = [m for m in range(M) if m not in sel]
        assert torch.equal(x[others].cpu(), x0[others])            # rows not asked for are left alone
        # a second norm of the same stream finds nothing pending and the same values
        again = torch.empty_like(out)
        _ops.rmsnorm(again, x, w.to(DEV), 1e-5, None if rows is None else torch.tensor(rows, dtype=torch.int32, device=DEV), ws=ws)
        assert torch.equal(again, out)
    # a pending update of another stream is not this norm's to add
    ws = _ops.KernelWorkspace(DEV)
    other = torch.zeros(M, D, device=DEV)
    ws.pending = PendingUpdate(other, Partials(pieces.to(DEV), splits, M, D))
    x = x0.clone().to(DEV)
    out = torch.empty(M, D, dtype=out_dtype, device=DEV)
    _ops.rmsnorm(out, x, w.to(DEV), 1e-5, ws=ws)
    assert ws.pending is not None and torch.equal(x.cpu(), x0)
    close(out, P.rmsnorm(x0.double(), w.double(), 1e-5), tol, "norm beside another stream's pending update")


def test_a_second_split_product_applies_the_first_ones_pieces(_ops):
    """The workspace holds one product's pieces: a product that needs it applies the pending
    update of the other stream before it overwrites them."""
    M, N, K = 4, 512, 2048
    a = (torch.randn(M, K, generator=gen(1)) * 0.25).to(BF16).to(DEV)
    w1 = (torch.randn(N, K, generator=gen(2)) * 0.25).to(BF16).to(DEV)
    w2 = (torch.randn(N, K, generator=gen(3)) * 0.25).to(BF16).to(DEV)
    ws = _ops.KernelWorkspace(DEV)
    x, y = torch.ones(M, N, device=DEV), torch.full((M, N), 2.0, device=DEV)
    _ops.gemm(x, a, w1, accumulate=True, may_defer=True, ws=ws)
    assert ws.pending is not None and ws.pending.is_for(x) and ws.counts["split_products"] == 1
    _ops.gemm(y, a, w2, accumulate=True, may_defer=True, ws=ws)
    assert ws.pending.is_for(y) and ws.counts["flushed"] == 1
    _ops.materialize(y, ws)
    close(x, 1.0 + a.double().cpu() @ w1.double().cpu().t(), 2e-6, "first stream")
    close(y, 2.0 + a.double().cpu() @ w2.double().cpu().t(), 2e-6, "second stream")
    # two workspaces never see each other's pieces
    ws1, ws2 = _ops.KernelWorkspace(DEV), _ops.KernelWorkspace(DEV)
    x, y = torch.ones(M, N, device=DEV), torch.full((M, N), 2.0, device=DEV)
    _ops.gemm(x, a, w1, accumulate=True, may_defer=True, ws=ws1)
    _ops.gemm(y, a, w2, accumulate=True, may_defer=True, ws=ws2)
    assert ws1.pending.is_for(x) and ws2.pending.is_for(y) and ws1.counts["flushed"] == 0
    _ops.materialize(x, ws1), _ops.materialize(y, ws2)
    close(x, 1.0 + a.double().cpu() @ w1.double().cpu().t(), 2e-6, "first workspace")
    close(y, 2.0 + a.double().cpu() @ w2.double().cpu().t(), 2e-6, "second workspace")


def test_rmsnorm_reference_vectors(_ops):
    # tests/ops/test_rmsnorm.cpp:102-181
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [2.0, 4.0, 6.0, 8.0]], device=DEV)
    out = torch.empty(2, 4, device=DEV)
    _ops.rmsnorm(out, x, torch.tensor([0.5, 1.0, 1.5, 2.0], device=DEV), 1e-5)
    w = torch.tensor([0.5, 1.0, 1.5, 2.0])
    assert torch.allclose(out[0].cpu(), w * x[0].cpu() / math.sqrt(7.5 + 1e-5), atol=1e-6)
    assert torch.allclose(out[1].cpu(), w * x[1].cpu() / math.sqrt(30 + 1e-5), atol=1e-6)


# ------------------------------------------------------------------ SwiGLU
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_swiglu(_ops, dtype):
    T, I = 5, 176
    gu = (torch.randn(T, 2 * I, generator=gen(2)) * 4).to(dtype)
    gu[0, :4] = torch.tensor([1.0, 2.0, 3.0, 4.0]).to(dtype)          # tests/ops/test_swiglu.cpp:159-216
    gu[0, I:I + 4] = torch.tensor([0.5, 1.0, 1.5, 2.0]).to(dtype)
    gu[1, :3] = torch.tensor([90.0, -90.0, 0.0]).to(dtype)
    out = torch.empty(T, I, dtype=dtype, device=DEV)
    _ops.swiglu(out, gu.to(DEV))
    want = P.swiglu(gu[:, :I].float(), gu[:, I:].float())
    close(out, want, 1e-6 if dtype == F32 else 2 ** -8, "swiglu")
    assert not out.isnan().any() and out[1, 1].item() == 0 and out[1, 2].item() == 0


# ------------------------------------------------------------------ matrix products
GEMM_SHAPES = [(1, 14, 3), (2, 2, 3), (5, 176, 64), (33, 100, 72), (64, 384, 128), (70, 1001, 96), (1, 256, 64),
               (130, 64, 200), (257, 320, 136), (8, 2048, 512), (300, 520, 264),
               (40, 200, 1032), (64, 72, 520), (48, 1001, 96), (35, 130, 2048),
               # few rows and a k of which some wave holds less than one step of 64
               (4, 50, 160), (16, 33, 8), (3, 64, 200), (9, 40, 344), (12, 776, 272)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("a_dtype,w_dtype,c_dtype", [(F32, F32, F32), (BF16, BF16, BF16), (BF16, BF16, F32), (BF16, F32, BF16)])
@pytest.mark.parametrize("fast", [False, True])
def test_gemm(_ops, M, N, K, a_dtype, w_dtype, c_dtype, fast):
    if fast and not (a_dtype == BF16 and w_dtype == BF16):
        pytest.skip("the matrix-core kernels take bfloat16 operands only")
    _ops.use_fast_kernels(fast)
    a = torch.randn(M, K, generator=gen(M + N)).to(a_dtype)
    w = torch.randn(N, K, generator=gen(K)).to(w_dtype)
    want = a.double() @ w.double().t()
    out = torch.empty(M, N, dtype=c_dtype, device=DEV)
    _ops.gemm(out, a.to(DEV), w.to(DEV))
    close(out, want, 2e-6 if c_dtype == F32 else 2 ** -8, f"gemm {M}x{N}x{K}")
    if c_dtype == F32:
        base = torch.randn(M, N, generator=gen(9))
        acc = base.clone().to(DEV)
        _ops.gemm(acc, a.to(DEV), w.to(DEV), accumulate=True)
        close(acc, want + base.double(), 2e-6, "gemm accumulate")


@pytest.mark.parametrize("M", [1, 3, 16, 17, 64, 65, 200])
@pytest.mark.parametrize("I,K", [(176, 64), (272, 128), (8192 // 8, 2048 // 8)])
def test_gemm_with_swiglu_in_the_epilogue(_ops, M, I, K):
    """Gate and up rows interleaved by 16: product and activation in one kernel."""
    a = torch.randn(M, K, generator=gen(M)).to(BF16)
    g = (torch.randn(I, K, generator=gen(I)) * 0.3).to(BF16)
    u = (torch.randn(I, K, generator=gen(K)) * 0.3).to(BF16)
    w_il = torch.stack([g.view(I // 16, 16, K), u.view(I // 16, 16, K)], dim=1).reshape(2 * I, K).contiguous()
    want = P.swiglu(a.double() @ g.double().t(), a.double() @ u.double().t())
    for fast in (True, False):
        _ops.use_fast_kernels(fast)
        out = torch.empty(M, I, dtype=BF16, device=DEV)
        _ops.gemm_swiglu(out, a.to(DEV), w_il.to(DEV), 16)
        close(out, want, 2 ** -7, f"fused swiglu fast={fast}")
    halves = torch.cat([g, u]).to(DEV)
    out = torch.empty(M, I, dtype=BF16, device=DEV)
    _ops.gemm_swiglu(out, a.to(DEV), halves, 0)
    close(out, want, 2 ** -7, "swiglu on halves")


@pytest.mark.parametrize("M,N,K", [(1024, 12288, 192), (1000, 12300, 256), (1000, 12300, 264), (2048, 6200, 72)])
def test_gemm_on_large_tiles(_ops, M, N, K):
    """Enough 256 x 256 tiles to fill the chip: the one-wave-per-SIMD kernel, with ragged edges
    in every dimension and a k that is no multiple of its slab."""
    _ops.use_fast_kernels(True)
    a = torch.randn(M, K, generator=gen(M)).to(BF16)
    w = torch.randn(N, K, generator=gen(N)).to(BF16)
    want = a.double() @ w.double().t()
    for c_dtype, rel in ((BF16, 2 ** -8), (F32, 2e-6)):
        out = torch.empty(M, N, dtype=c_dtype, device=DEV)
        _ops.gemm(out, a.to(DEV), w.to(DEV))
        close(out, want, rel, f"large gemm {M}x{N}x{K} {c_dtype}")
    base = torch.randn(M, N, generator=gen(9))
    acc = base.clone().to(DEV)
    _ops.gemm(acc, a.to(DEV), w.to(DEV), accumulate=True)
    close(acc, want + base.double(), 2e-6, "large gemm accumulate")


@pytest.mark.parametrize("M,N,K", [(2048, 2040, 6208),      # 64 tiles of 256 x 256, a long k: four pieces on the large-tile kernel
                                   (1024, 2040, 4104)])     # 128 tiles of 128 x 128, k no multiple of the slab: pieces on the small tiles
def test_gemm_on_large_tiles_split_over_k(_ops, M, N, K):
    """Few output tiles and a long k: pieces over k from the tile kernels, summed by materialize."""
    _ops.use_fast_kernels(True)
    a = (torch.randn(M, K, generator=gen(1)) * 0.25).to(BF16)
    w = (torch.randn(N, K, generator=gen(2)) * 0.25).to(BF16)
    base = torch.randn(M, N, generator=gen(3))
    want = a.double() @ w.double().t() + base.double()
    x = base.clone().to(DEV)
    ws = _ops.KernelWorkspace(DEV)
    _ops.gemm(x, a.to(DEV), w.to(DEV), accumulate=True, may_defer=True, ws=ws)
    assert ws.pending is not None and ws.pending.pieces.splits > 1 and torch.equal(x.cpu(), base)   # nothing added yet
    _ops.materialize(x, ws)
    assert ws.pending is None and ws.counts["applied"] == 1
    close(x, want, 2e-6, "k-split large gemm")
    # without a workspace nothing is ever left pending: the same product is finished by the call
    y = base.clone().to(DEV)
    _ops.gemm(y, a.to(DEV), w.to(DEV), accumulate=True, may_defer=True)
    close(y, want, 2e-6, "large gemm without a workspace")


@pytest.mark.parametrize("M,I,K", [(1000, 6160, 200), (1000, 6160, 192), (2048, 8192, 64)])
def test_gemm_with_swiglu_on_large_tiles(_ops, M, I, K):
    _ops.use_fast_kernels(True)
    a = torch.randn(M, K, generator=gen(M)).to(BF16)
    g = (torch.randn(I, K, generator=gen(I)) * 0.3).to(BF16)
    u = (torch.randn(I, K, generator=gen(K)) * 0.3).to(BF16)
    w_il = torch.stack([g.view(I // 16, 16, K), u.view(I // 16, 16, K)], dim=1).reshape(2 * I, K).contiguous()
    want = P.swiglu(a.double() @ g.double().t(), a.double() @ u.double().t())
    out = torch.empty(M, I, dtype=BF16, device=DEV)
    _ops.gemm_swiglu(out, a.to(DEV), w_il.to(DEV), 16)
    close(out, want, 2 ** -7, "fused swiglu on large tiles")


def test_gemm_reference_vectors(_ops):
    # tests/ops/test_matmul.cpp:90-204
    W = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]], device=DEV)
    X = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]], device=DEV)
    out = torch.empty(2, 2, device=DEV)
    _ops.gemm(out, X, W)
    assert out.cpu().tolist() == [[14.0, 32.0], [32.0, 77.0]]


@pytest.mark.parametrize("N,K", [(16, 64), (48, 192), (80, 2048), (1024, 320), (2064, 1088)])
def test_products_read_a_weight_matrix_or_its_streaming_copy_to_the_same_bits(_ops, N, K):
    """A workspace may hold a second copy of a weight matrix in the order the weight-streaming
    kernels load it (16 rows x 64 columns per 2 KB); products of up to 128 tokens then read the
    copy.  Same arithmetic in the same order, so every bit agrees with the product from the
    matrix itself: single tokens and the shared-activation kernel, stored, added and left in
    pieces, the activation in the epilogue, and key ranges merged on the way in."""
    _ops.use_fast_kernels(True)
    g = gen(N + K)
    w = (torch.randn(N, K, generator=g) * 0.1).to(BF16).to(DEV)
    layout = _ops.stream_layout(w)
    # the layout itself: lane group lg of a wave holds columns 16 lg + 8 h .. + 7 of row lr in fragment h
    t = layout.cpu().view(N // 16, K // 64, 2, 4, 16, 8)
    for rb, kb, h, lg, lr in [(0, 0, 0, 0, 0), (N // 16 - 1, K // 64 - 1, 1, 3, 15), (0, K // 64 - 1, 1, 2, 7)]:
        k0 = kb * 64 + lg * 16 + h * 8
        assert torch.equal(t[rb, kb, h, lg, lr], w.cpu()[rb * 16 + lr, k0:k0 + 8])
    with_copy, without = _ops.KernelWorkspace(DEV), _ops.KernelWorkspace(DEV)
    assert with_copy.add_stream_copy(w) and not with_copy.add_stream_copy(w[:, :K - 8])
    for M in (1, 5, 16, 17, 32, 33, 64, 100, 128, 200):
        a = torch.randn(M, K, generator=g).to(BF16).to(DEV)
        for c_dtype in (BF16, F32):
            got, want = torch.empty(M, N, dtype=c_dtype, device=DEV), torch.empty(M, N, dtype=c_dtype, device=DEV)
            _ops.gemm(got, a, w, ws=with_copy)
            _ops.gemm(want, a, w, ws=without)
            assert torch.equal(got, want), f"stored, {M} tokens, {c_dtype}"
        base = torch.randn(M, N, generator=g).to(DEV)
        got, want = base.clone(), base.clone()
        _ops.gemm(got, a, w, accumulate=True, may_defer=True, ws=with_copy)
        _ops.gemm(want, a, w, accumulate=True, may_defer=True, ws=without)
        _ops.materialize(got, with_copy)
        _ops.materialize(want, without)
        assert torch.equal(got, want), f"added, {M} tokens"
        close(want, a.double().cpu() @ w.double().cpu().t() + base.double().cpu(), 2e-5, f"against float64, {M} tokens")
        if N % 32 == 0:
            got, want = torch.empty(M, N // 2, dtype=BF16, device=DEV), torch.empty(M, N // 2, dtype=BF16, device=DEV)
            _ops.gemm_swiglu(got, a, w, 16, ws=with_copy)
            _ops.gemm_swiglu(want, a, w, 16, ws=without)
            assert torch.equal(got, want), f"activation in the epilogue, {M} tokens"
    # a slice of the matrix is not the matrix the copy was made of
    part = torch.empty(4, 16, dtype=F32, device=DEV)
    _ops.gemm(part, a[:4], w[:16], ws=with_copy)
    want = torch.empty(4, 16, dtype=F32, device=DEV)
    _ops.gemm(want, a[:4], w[:16], ws=without)
    assert torch.equal(part, want)


@pytest.mark.parametrize("fast", [False, True])
def test_gemm_rows_do_not_depend_on_the_batch(_ops, fast):
    """A row's result is the same whatever other rows share the launch."""
    _ops.use_fast_kernels(fast)
    a = torch.randn(150, 264, generator=gen(3)).to(BF16).to(DEV)
    w = torch.randn(520, 264, generator=gen(4)).to(BF16).to(DEV)
    whole = torch.empty(150, 520, dtype=F32, device=DEV)
    _ops.gemm(whole, a, w)
    for lo, hi in [(0, 1), (7, 9), (64, 150), (149, 150), (3, 70)]:
        part = torch.empty(hi - lo, 520, dtype=F32, device=DEV)
        _ops.gemm(part, a[lo:hi], w)
        close(part, whole[lo:hi].cpu(), 2e-6, f"rows {lo}:{hi}")


def test_gemm_takes_strided_views(_ops):
    a_full = torch.randn(9, 300, generator=gen(5)).to(BF16).to(DEV)
    w = torch.randn(40, 128, generator=gen(6)).to(BF16).to(DEV)
    a = a_full[:, 64:192]                       # dense rows, row stride 300
    out_full = torch.zeros(9, 100, dtype=BF16, device=DEV)
    _ops.gemm(out_full[:, 8:48], a, w)
    close(out_full[:, 8:48], a.double().cpu() @ w.double().cpu().t(), 2 ** -8, "strided gemm")
    assert out_full[:, :8].abs().max() == 0 and out_full[:, 48:].abs().max() == 0


def test_ops_refuse_what_they_do_not_take(_ops):
    from photon_infer_amd import KernelError
    with pytest.raises(KernelError, match="GPU only"):
        _ops.gemm(torch.empty(2, 2), torch.empty(2, 3), torch.empty(2, 3))
    with pytest.raises(KernelError, match="shapes"):
        _ops.gemm(torch.empty(2, 2, device=DEV), torch.empty(2, 3, device=DEV), torch.empty(2, 4, device=DEV))
    with pytest.raises(KernelError, match="head_dim"):
        _ops.check_attention_sizes(4, 2, 40)
    with pytest.raises(KernelError, match="head_dim"):
        _ops.check_attention_sizes(4, 2, 272)
    with pytest.raises(KernelError, match="multiple"):
        _ops.check_attention_sizes(6, 4, 64)
    with pytest.raises(KernelError, match="float32 or bfloat16"):
        _ops.swiglu(torch.empty(2, 4, dtype=torch.float16, device=DEV), torch.empty(2, 8, dtype=torch.float16, device=DEV))


# ------------------------------------------------------------------ rotation + cache write
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("hd,rot,inter", [(16, 16, False), (48, 48, True), (64, 32, False), (128, 128, False), (256, 256, True)])
def test_rope_kv_write(_ops, dtype, hd, rot, inter):
    nh, nkv, page = 3, 3 if hd == 48 else 1, 4
    q_lens, kv_lens = [5, 1, 9], [5, 30, 14]          # a whole prompt, a decode at position 29, a later portion
    T = sum(q_lens)
    ctx = attention_ctx(q_lens, kv_lens, dtype)
    freqs = P.rope_frequencies(rot, 500000.0, dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                                                    high_freq_factor=4.0, original_max_position_embeddings=16))
    inv = torch.tensor(freqs, dtype=torch.float64).to(F32).to(DEV)
    qkv = torch.randn(T, (nh + 2 * nkv) * hd, generator=gen(hd)).to(dtype)
    dev = qkv.to(DEV)
    q, k, v = dev[:, :nh * hd], dev[:, nh * hd:(nh + nkv) * hd], dev[:, (nh + nkv) * hd:]
    pages = 12
    table = torch.full((3, 8), -1, dtype=torch.int32)
    order = torch.randperm(pages * 2, generator=gen(7))[: 2 + 8 + 4].tolist()
    table[0, :2], table[1, :8], table[2, :4] = torch.tensor(order[:2]), torch.tensor(order[2:10]), torch.tensor(order[10:14])
    kc = torch.zeros(pages * 2, nkv, page, hd, dtype=dtype, device=DEV)
    vc = torch.zeros(pages * 2, nkv, hd, page, dtype=dtype, device=DEV)
    _ops.rope_kv_write(q, k, v, ctx.positions, ctx.req_of_token, (inv, rot, inter), nh, nkv, hd, kc, vc, table.to(DEV), page)
    pos = ctx.positions.cpu().tolist()
    rel = 1e-6 if dtype == F32 else 2 ** -8
    q_want = P.rope(qkv[:, :nh * hd].float().reshape(T, nh, hd), pos, freqs, inter)
    k_want = P.rope(qkv[:, nh * hd:(nh + nkv) * hd].float().reshape(T, nkv, hd), pos, freqs, inter)
    v_want = qkv[:, (nh + nkv) * hd:].float().reshape(T, nkv, hd)
    close(q.reshape(T, nh, hd), q_want, rel, "q")
    req = ctx.req_of_token.cpu().tolist()
    written = torch.zeros(pages * 2, page, dtype=torch.bool)
    for t in range(T):
        pg, sl = table[req[t], pos[t] // page].item(), pos[t] % page
        written[pg, sl] = True
        close(kc[pg, :, sl], k_want[t], rel, f"k of token {t}")
        assert torch.equal(vc[pg, :, :, sl].cpu().float(), v_want[t])
    # nothing else in the pool was touched
    assert kc.cpu()[~written.unsqueeze(1).expand(-1, nkv, -1)].abs().max() == 0
    assert vc.cpu().permute(0, 1, 3, 2)[~written.unsqueeze(1).expand(-1, nkv, -1)].abs().max() == 0


@pytest.mark.parametrize("hd,page,rotate", [(64, 16, True), (128, 4, True), (64, 8, False), (16, 4, True)])
@pytest.mark.parametrize("pieces", [0, 3, 6])
def test_rope_kv_write_many_tokens(_ops, hd, page, rotate, pieces):
    """Prompts take the kernel with wide accesses: portions that start at any row of the batch
    and at any position, single tokens among them, pages of several sizes; q, k and v as a
    bfloat16 tensor or as float32 pieces of a product split over k (summed in float32, rounded
    once after the rotation)."""
    nh, nkv, dtype = 4, 2, BF16
    q_lens, kv_lens = [40, 1, 23, 7, 16], [40, 30, 55, 19, 48]    # whole, decode, later portions (rows 41.., 64.., 71..)
    R, T = len(q_lens), sum(q_lens)
    ctx = attention_ctx(q_lens, kv_lens, dtype)
    freqs = P.rope_frequencies(hd, 10000.0, None)
    inv = torch.tensor(freqs, dtype=torch.float64).to(F32).to(DEV)
    if pieces:
        from photon_infer_amd.ops import fast
        part = torch.randn(pieces, T, (nh + 2 * nkv) * hd, generator=gen(hd + page)) * 0.5
        qkv = part[0].clone()
        for s_ in range(1, pieces):       # the kernel's order of adding
            qkv += part[s_]
        source = fast.Partials(part.to(DEV), pieces, T, (nh + 2 * nkv) * hd)
        q = torch.empty(T, nh * hd, dtype=dtype, device=DEV)
    else:
        qkv = torch.randn(T, (nh + 2 * nkv) * hd, generator=gen(hd + page)).to(dtype)
        dev = qkv.to(DEV)
        q, k, v = dev[:, :nh * hd], dev[:, nh * hd:(nh + nkv) * hd], dev[:, (nh + nkv) * hd:]
    blocks = [-(-kv // page) for kv in kv_lens]
    pages = sum(blocks) + 3
    order = torch.randperm(pages, generator=gen(11)).tolist()
    table = torch.full((R, max(blocks)), -1, dtype=torch.int32)
    it = iter(order)
    for r in range(R):
        for b in range(blocks[r]):
            table[r, b] = next(it)
    kc = torch.zeros(pages, nkv, page, hd, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, nkv, hd, page, dtype=dtype, device=DEV)
    if pieces:
        _ops.rope_kv_write(q, None, None, ctx.positions, ctx.req_of_token, (inv, hd, False) if rotate else None, nh, nkv, hd,
                           kc, vc, table.to(DEV), page, pieces=source, write_kv=True)
    else:
        _ops.rope_kv_write(q, k, v, ctx.positions, ctx.req_of_token, (inv, hd, False) if rotate else None, nh, nkv, hd, kc, vc,
                           table.to(DEV), page)
    pos = ctx.positions.cpu().tolist()
    req = ctx.req_of_token.cpu().tolist()
    turn = (lambda x: P.rope(x, pos, freqs, False)) if rotate else (lambda x: x)
    q_want = turn(qkv[:, :nh * hd].float().reshape(T, nh, hd))
    k_want = turn(qkv[:, nh * hd:(nh + nkv) * hd].float().reshape(T, nkv, hd))
    v_want = qkv[:, (nh + nkv) * hd:].float().reshape(T, nkv, hd)
    close(q.reshape(T, nh, hd), q_want, 2 ** -8, "q")
    written = torch.zeros(pages, page, dtype=torch.bool)
    kc_h, vc_h = kc.cpu().float(), vc.cpu().float()
    for t in range(T):
        pg, sl = table[req[t], pos[t] // page].item(), pos[t] % page
        written[pg, sl] = True
        close(kc_h[pg, :, sl], k_want[t], 2 ** -8, f"k of token {t}")
        assert torch.equal(vc_h[pg, :, :, sl], v_want[t].to(dtype).float()), f"v of token {t}"
    assert kc_h[~written.unsqueeze(1).expand(-1, nkv, -1)].abs().max() == 0
    assert vc_h.permute(0, 1, 3, 2)[~written.unsqueeze(1).expand(-1, nkv, -1)].abs().max() == 0


@pytest.mark.parametrize("hd,nh,nkv,page,window,rotate", [(64, 8, 2, 16, 0, True), (128, 4, 4, 32, 40, True), (64, 6, 2, 16, 24, False),
                                                          (128, 16, 1, 16, 0, True)])
@pytest.mark.parametrize("pieces", [False, True])
def test_decode_attention_from_projection(_ops, hd, nh, nkv, page, window, rotate, pieces):
    """A step of single tokens through the kernel that rotates, writes the cache and attends at
    once: the cache it leaves and its outputs are, bit for bit, those of the separate kernels
    (a token's logits must not depend on what else the step held), and the outputs agree with
    plain attention over that cache.  The new token at a page's first and
    last slot, a context of one token, few and many keys, the projection as a tensor and as
    float32 pieces.  The slot of the new token holds large numbers beforehand: a kernel that
    read it before it was written, or counted the token twice, or not at all, would show."""
    from photon_infer_amd.ops import fast
    kv_lens = [1, page, page + 1, 2 * page + 1, 300, 1000, 65]
    R = len(kv_lens)
    ctx = attention_ctx([1] * R, kv_lens, BF16)
    g = gen(hd + nh + page)
    seqs = [(torch.randn(kv, nkv, hd, generator=g) * 0.5, torch.randn(kv, nkv, hd, generator=g)) for kv in kv_lens]
    kv = PagedKV(seqs, page, BF16, seed=3)
    table = kv.table.cpu()
    for r, n in enumerate(kv_lens):
        pg, sl = table[r, (n - 1) // page].item(), (n - 1) % page
        kv.k[pg, :, sl] = 1e4
        kv.v[pg, :, :, sl] = -1e4
    N = (nh + 2 * nkv) * hd
    if pieces:
        part = (torch.randn(3, R, N, generator=g) * 0.4).to(DEV)
        qkv = fast.Partials(part, 3, R, N)
    else:
        qkv = (torch.randn(R, N, generator=g) * 0.6).to(BF16).to(DEV)
    freqs = P.rope_frequencies(hd, 10000.0, None)
    inv = torch.tensor(freqs, dtype=torch.float64).to(F32).to(DEV)
    rotary = (inv, hd, False) if rotate else None
    scale = hd ** -0.5

    # the separate kernels, on a copy of the cache
    k1, v1 = kv.k.clone(), kv.v.clone()
    if pieces:
        q = torch.empty(R, nh * hd, dtype=BF16, device=DEV)
        _ops.rope_kv_write(q, None, None, ctx.positions, ctx.req_of_token, rotary, nh, nkv, hd, k1, v1, kv.table, page,
                           pieces=qkv, write_kv=True)
    else:
        own = qkv.clone()
        q = own[:, :nh * hd]
        _ops.rope_kv_write(q, own[:, nh * hd:(nh + nkv) * hd], own[:, (nh + nkv) * hd:], ctx.positions, ctx.req_of_token,
                           rotary, nh, nkv, hd, k1, v1, kv.table, page)
    apart = torch.empty(R, nh * hd, dtype=BF16, device=DEV)
    _ops.paged_attention(apart, q, k1, v1, kv.table, ctx, nh, nkv, hd, page, scale, window)
    # plain attention over the cache they left
    k_h, v_h = k1.cpu().float(), v1.cpu().float()
    dense = []
    for r, n in enumerate(kv_lens):
        pages = [table[r, b].item() for b in range(-(-n // page))]
        dense.append((torch.cat([k_h[pg].transpose(0, 1) for pg in pages])[:n], torch.cat([v_h[pg].permute(2, 0, 1) for pg in pages])[:n]))
    qs = [q[r].float().cpu().reshape(1, nh, hd) for r in range(R)]
    want = dense_attention(qs, dense, [1] * R, kv_lens, scale, window or None).reshape(R, nh * hd)
    close(apart, want, 2 ** -7, "the separate kernels")

    k2, v2 = kv.k.clone(), kv.v.clone()
    got = torch.full((R, nh * hd), 7.0, dtype=BF16, device=DEV)
    assert _ops.decode_attention_from_projection(got, qkv, ctx, rotary, nh, nkv, hd, k2, v2, kv.table, page, scale, window, True)
    assert torch.equal(k2, k1) and torch.equal(v2, v1), "the cache differs"
    assert not torch.equal(k2, kv.k), "nothing was written"
    close(got, want, 2 ** -7, "one kernel")
    assert torch.equal(got, apart), "a step of single tokens must not depend on which kernels ran it"
    # without the cache write (a layer that reads another layer's cache): queries only, keys from the cache
    got2 = torch.full((R, nh * hd), 7.0, dtype=BF16, device=DEV)
    k3 = k2.clone()
    assert _ops.decode_attention_from_projection(got2, qkv, ctx, rotary, nh, nkv, hd, k3, v2, kv.table, page, scale, window, False)
    assert torch.equal(got2, apart) and torch.equal(k3, k2)
    # the key ranges left unmerged for the product that reads the output next: the o projection
    # merges them as it stages its activations, to the same bits as the merging kernel
    ws = _ops.KernelWorkspace(DEV)
    k4, v4 = kv.k.clone(), kv.v.clone()
    untouched = torch.full((R, nh * hd), 7.0, dtype=BF16, device=DEV)
    ranges = _ops.decode_attention_from_projection(untouched, qkv, ctx, rotary, nh, nkv, hd, k4, v4, kv.table, page, scale, window,
                                                   True, ws, leave_ranges=True)
    assert isinstance(ranges, _ops.KeyRanges) and ranges.count > 1 and torch.equal(k4, k1) and torch.equal(v4, v1)
    assert (untouched == 7.0).all()
    for n_out, w_dtype in ((96, BF16), (40, BF16), (200, F32)):
        w_o = (torch.randn(n_out, nh * hd, generator=g) * 0.05).to(w_dtype).to(DEV)
        x0 = torch.randn(R, n_out, generator=g).to(DEV)
        want_x, got_x = x0.clone(), x0.clone()
        _ops.gemm(want_x, apart, w_o, accumulate=True)
        _ops.gemm(got_x, ranges, w_o, accumulate=True, ws=ws)
        assert torch.equal(got_x, want_x), f"o projection from key ranges, {n_out} x {w_dtype}"
        want_b, got_b = torch.empty(R, n_out, dtype=BF16, device=DEV), torch.empty(R, n_out, dtype=BF16, device=DEV)
        _ops.gemm(want_b, apart, w_o)
        _ops.gemm(got_b, ranges, w_o, ws=ws)
        assert torch.equal(got_b, want_b)
    assert ws.counts["ranges_merged_by_product"] == 4              # the float32 weights went through the merging kernel
    # the same from the matrix's copy in the streaming kernels' order
    w_o = (torch.randn(96, nh * hd, generator=g) * 0.05).to(BF16).to(DEV)
    copies = _ops.KernelWorkspace(DEV)
    assert copies.add_stream_copy(w_o)
    want_x, got_x = torch.empty(R, 96, dtype=F32, device=DEV), torch.empty(R, 96, dtype=F32, device=DEV)
    _ops.gemm(want_x, ranges, w_o, ws=ws)
    _ops.gemm(got_x, ranges, w_o, ws=copies)
    assert torch.equal(got_x, want_x) and copies.counts["ranges_merged_by_product"] == 1
    # and left in pieces for the stream's next norm, as the model's o projection is
    w_o = (torch.randn(96, nh * hd, generator=g) * 0.05).to(BF16).to(DEV)
    x0 = torch.randn(R, 96, generator=g).to(DEV)
    want_x, got_x = x0.clone(), x0.clone()
    _ops.gemm(want_x, apart, w_o, accumulate=True)
    _ops.gemm(got_x, ranges, w_o, accumulate=True, may_defer=True, ws=ws)
    _ops.materialize(got_x, ws)
    assert torch.equal(got_x, want_x)


def test_decode_attention_from_projection_declines_what_it_does_not_serve(_ops):
    hd, nh, nkv, page = 64, 4, 2, 16
    seqs = [(torch.randn(20, nkv, hd), torch.randn(20, nkv, hd))] * 2
    kv = PagedKV(seqs, page, BF16)
    qkv = torch.randn(2, (nh + 2 * nkv) * hd).to(BF16).to(DEV)
    out = torch.empty(2, nh * hd, dtype=BF16, device=DEV)
    inv = torch.ones(16, dtype=F32, device=DEV)
    # rotation over a part of the head
    ctx = attention_ctx([1, 1], [20, 20], BF16)
    assert not _ops.decode_attention_from_projection(out, qkv, ctx, (inv, 32, False), nh, nkv, hd, kv.k, kv.v, kv.table, page, 0.1, 0, True)
    # a step with a prompt portion
    ctx = attention_ctx([2, 1], [20, 20], BF16)
    qkv3 = torch.randn(3, (nh + 2 * nkv) * hd).to(BF16).to(DEV)
    out3 = torch.empty(3, nh * hd, dtype=BF16, device=DEV)
    assert not _ops.decode_attention_from_projection(out3, qkv3, ctx, None, nh, nkv, hd, kv.k, kv.v, kv.table, page, 0.1, 0, True)


# ------------------------------------------------------------------ attention over pages
def dense_attention(qs, kvs, q_lens, kv_lens, scale, window):
    """Plain attention per request: the queries are the last q_len positions of kv_len keys."""
    outs = []
    for q, (k, v), n, kv in zip(qs, kvs, q_lens, kv_lens):
        full_q = torch.zeros(kv, q.shape[1], q.shape[2], dtype=torch.float64)   # in double: only the kernel's rounding counts
        full_q[kv - n:] = q.double()
        outs.append(P.attention(full_q, k.double(), v.double(), scale, window=window)[kv - n:])
    return torch.cat(outs)


ATTN_CASES = [
    # nh, nkv, hd, page, q_lens, kv_lens, window
    (4, 2, 16, 4, [5, 9, 17], [5, 9, 17], None),                 # whole prompts
    (4, 1, 32, 8, [1, 1, 1, 1], [1, 7, 33, 100], None),          # decodes, page edges: 1, 7, 33 = 4 pages + 1
    (6, 3, 48, 16, [2, 16, 1, 3], [40, 16, 65, 130], None),      # mixed, portions down to two tokens
    (8, 8, 64, 16, [70], [300], None),                           # a late portion of a long prompt
    (32, 8, 64, 16, [1, 1], [513, 1200], None),                  # the bench's head layout
    (2, 1, 128, 16, [33, 1], [33, 200], None),
    (3, 1, 256, 8, [4, 1], [20, 9], None),
    (4, 2, 16, 4, [6, 1, 20], [6, 23, 40], 7),                   # a window: edge inside and across portions
    (4, 4, 80, 16, [1, 5], [90, 37], 16),
    # sizes the matrix-core kernels take
    (4, 2, 64, 16, [1, 1, 1, 1, 1], [1, 16, 17, 200, 1000], None),   # decodes: first token, page edges, long
    (6, 2, 64, 16, [40, 1, 2, 100], [40, 77, 300, 100], None),       # three heads per kv head, mixed batch
    (4, 1, 128, 32, [65, 1], [200, 31], None),                       # one kv head, pages of 32
    (8, 2, 64, 16, [1, 1, 1], [50, 333, 64], 40),                    # decodes with a window
    (8, 2, 64, 64, [130, 3, 1], [130, 250, 99], 33),                 # portions with a window, pages of 64
    (16, 1, 64, 16, [1, 1], [129, 2], None),                         # sixteen heads on one kv head
    (32, 1, 64, 16, [1, 70], [75, 70], None),                        # more heads per kv head than a wave's columns
    # the other head sizes of the matrix-core kernels: every multiple of 16 up to 256; sizes that are
    # no multiple of 32 end in half a fragment
    (4, 2, 16, 16, [1, 20, 1], [40, 20, 300], None),
    (3, 1, 48, 16, [33, 1, 2], [33, 90, 130], None),
    (4, 4, 80, 16, [1, 5, 1], [90, 37, 600], 16),
    (5, 5, 80, 32, [64, 1], [200, 257], None),
    (2, 1, 112, 16, [1, 1, 17], [15, 129, 50], None),
    (2, 2, 144, 16, [1, 1], [100, 31], None),
    (4, 2, 176, 16, [1], [260], None),
    (3, 1, 240, 16, [1, 1], [64, 65], 30),
    (4, 2, 32, 16, [1, 1, 1], [5, 100, 333], None),
    (4, 2, 32, 16, [70, 1, 3], [300, 20, 64], None),
    (6, 2, 96, 16, [40, 1, 2, 100], [40, 77, 300, 100], None),
    (3, 3, 96, 32, [1, 1, 1, 1], [1, 32, 33, 500], 48),
    (4, 2, 160, 32, [1, 1], [129, 64], None),
    (4, 1, 192, 16, [1, 1], [50, 700], None),
    (8, 2, 224, 16, [1], [300], 100),
    (2, 2, 256, 16, [1, 1, 1], [1, 33, 400], None),
    # portions at head sizes above 128: the tile kernel in rounds of 64 keys, 16 columns per wave
    (4, 1, 192, 16, [5, 1], [50, 700], None),
    (2, 2, 144, 16, [70, 1, 3], [300, 20, 64], None),
    (6, 2, 160, 32, [40, 1, 2, 100], [40, 77, 300, 100], None),
    (3, 1, 176, 16, [33, 17], [33, 90], 48),
    (4, 4, 208, 16, [65, 2], [200, 130], None),
    (8, 2, 224, 16, [20, 1], [150, 300], 100),
    (2, 1, 240, 16, [64], [64], None),
    (8, 2, 256, 16, [130, 3, 1], [130, 250, 99], 33),
    (4, 1, 256, 16, [37, 1], [2600, 900], None),                     # few tiles, many keys: cut and merged at head size 256
    (8, 2, 128, 16, [1, 70, 1, 1, 2], [900, 300, 33, 1, 50], None),  # single tokens beside portions: two kernels share the step
    (4, 2, 64, 16, [1, 3, 1], [700, 40, 18], 25),                    # the same with a window
    (8, 2, 64, 16, [70, 5], [2100, 40], None),                       # few tiles, many keys: their key ranges are cut and merged
    (4, 1, 128, 16, [33, 1, 40], [1500, 900, 2100], None),           # the same at head size 128, beside a single token
    (8, 2, 64, 32, [50], [2300], 700),                               # cut tiles with a window
]


@pytest.mark.parametrize("case", ATTN_CASES, ids=[f"case{i}" for i in range(len(ATTN_CASES))])
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("fast", [False, True])
def test_paged_attention(_ops, case, dtype, fast):
    nh, nkv, hd, page, q_lens, kv_lens, window = case
    if fast and dtype == F32:
        pytest.skip("the matrix-core kernels take bfloat16 only")
    _ops.use_fast_kernels(fast)
    g = gen(nh * 1000 + hd)
    scale = 1.0 / math.sqrt(hd)
    kvs = [(torch.randn(kv, nkv, hd, generator=g).to(dtype).float(), torch.randn(kv, nkv, hd, generator=g).to(dtype).float())
           for kv in kv_lens]
    qs = [(torch.randn(n, nh, hd, generator=g) * 2).to(dtype).float() for n in q_lens]
    paged = PagedKV(kvs, page, dtype, seed=hd)
    ctx = attention_ctx(q_lens, kv_lens, dtype)
    q = torch.cat(qs).reshape(-1, nh * hd).to(dtype).to(DEV)
    out = torch.empty_like(q)
    _ops.paged_attention(out, q, paged.k, paged.v, paged.table, ctx, nh, nkv, hd, page, scale, window or 0)
    want = dense_attention(qs, kvs, q_lens, kv_lens, scale, window).reshape(-1, nh * hd)
    close(out, want, 3e-6 if dtype == F32 else 2 ** -7, "attention")


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("fast", [False, True])
def test_attention_finds_one_far_key_among_hundreds(_ops, dtype, fast):
    """One key far back matches the query strongly: the output must be (nearly) its value.
    A kernel that drops a page, a split or the first / last key of a range fails this."""
    if fast and dtype == F32:
        pytest.skip("the matrix-core kernels take bfloat16 only")
    _ops.use_fast_kernels(fast)
    nh, nkv, hd, page = 4, 2, 64, 16
    g = gen(11)
    for kv_len, q_len, hot in [(777, 1, 3), (777, 1, 776), (640, 1, 639), (777, 1, 512), (500, 37, 15), (500, 37, 463),
                               (129, 2, 127),
                               # one long request: the decode kernel cuts it into its largest number of key ranges
                               (9000, 1, 5), (9000, 1, 4417), (9000, 1, 8999),
                               # a portion at the end of a long context: its tiles' key ranges are cut
                               (2600, 37, 3), (2600, 37, 1290), (2600, 37, 2580)]:
        k = torch.randn(kv_len, nkv, hd, generator=g) * 0.1
        v = torch.randn(kv_len, nkv, hd, generator=g)
        q = torch.randn(q_len, nh, hd, generator=g) * 0.1
        direction = torch.randn(hd, generator=g)
        direction = direction / direction.norm() * 8.0
        k[hot] = direction                                     # |k| = 8
        q += direction * 2.0                                   # score of the hot key: 16 * 8 / 8 = 16 above the rest
        paged = PagedKV([(k.to(dtype).float(), v.to(dtype).float())], page, dtype, seed=kv_len)
        ctx = attention_ctx([q_len], [kv_len], dtype)
        qd = q.reshape(q_len, nh * hd).to(dtype).to(DEV)
        out = torch.empty_like(qd)
        _ops.paged_attention(out, qd, paged.k, paged.v, paged.table, ctx, nh, nkv, hd, page, 1.0 / 8.0, 0)
        out = out.float().cpu().reshape(q_len, nh, hd)
        for t in range(q_len):
            p = kv_len - q_len + t
            if hot <= p:                                       # visible: its value dominates
                for h in range(nh):
                    assert (out[t, h] - v[hot, h // 2].to(dtype).float()).abs().max() < 0.05, (kv_len, q_len, hot, t)
            else:                                              # not yet visible: it must not leak in
                want = P.attention(torch.cat([torch.zeros(p, nh, hd), q[t:t + 1].to(dtype).float()]),
                                   k[:p + 1].to(dtype).float(), v[:p + 1].to(dtype).float(), 1.0 / 8.0)[p]
                assert (out[t] - want).abs().max() < 0.05


def test_pages_beyond_four_gibibytes_of_a_pool(_ops):
    """A pool of keys (and one of values) larger than 2^32 bytes, the requests' pages at its far
    end and a few at its start: the rotation's cache write, both prompt kernels, the decode
    kernel and the one that starts from the projection address them right.  A page id times a
    page's bytes that was formed in 32 bits would read the fill (1e4) or write somewhere else,
    which the count of changed cells shows."""
    nh, nkv, hd, page, dtype = 16, 8, 128, 16, BF16
    page_bytes = nkv * page * hd * 2
    pages = (1 << 32) // page_bytes + 3000
    q_lens, kv_lens = [40, 1, 1, 23], [40, 700, 33, 300]
    R, T = len(q_lens), sum(q_lens)
    g = gen(5)
    seqs = [((torch.randn(kv, nkv, hd, generator=g) * 0.5).to(dtype), torch.randn(kv, nkv, hd, generator=g).to(dtype)) for kv in kv_lens]
    blocks = [-(-kv // page) for kv in kv_lens]
    ids = torch.randperm(2900, generator=g)[:sum(blocks)] + (pages - 2900)          # beyond 4 GiB
    ids[::7] = torch.randperm(1000, generator=g)[:len(ids[::7])]                   # and some at the start
    table = torch.full((R, max(blocks)), -1, dtype=torch.int32)
    kc = torch.full((pages, nkv, page, hd), 1e4, dtype=dtype, device=DEV)
    vc = torch.full((pages, nkv, hd, page), -1e4, dtype=dtype, device=DEV)
    assert kc.numel() * 2 > 1 << 32
    it = iter(ids.tolist())
    old_cells = 0
    for r, (k, v) in enumerate(seqs):
        old = kv_lens[r] - q_lens[r]                       # what earlier steps left; this step's tokens come through the kernels
        for b in range(blocks[r]):
            pg = next(it)
            table[r, b] = pg
            n = max(0, min(page, old - b * page))
            if n:
                kc[pg, :, :n] = k[b * page: b * page + n].transpose(0, 1).to(DEV)
                vc[pg, :, :, :n] = v[b * page: b * page + n].permute(1, 2, 0).to(DEV)
            old_cells += n
    table_d = table.to(DEV)
    ctx = attention_ctx(q_lens, kv_lens, dtype)
    freqs = P.rope_frequencies(hd, 10000.0, None)
    inv = torch.tensor(freqs, dtype=torch.float64).to(F32).to(DEV)
    pos = ctx.positions.cpu().tolist()
    # this step's tokens: q, k, v before the rotation, such that the rotated keys are the sequences' own
    new_k = torch.cat([k[kv - n:] for (k, _), n, kv in zip(seqs, q_lens, kv_lens)]).float()
    new_v = torch.cat([v[kv - n:] for (_, v), n, kv in zip(seqs, q_lens, kv_lens)]).float()
    q_raw = (torch.randn(T, nh, hd, generator=g) * 2).to(dtype)
    qkv = torch.cat([q_raw.reshape(T, -1), new_k.to(dtype).reshape(T, -1), new_v.to(dtype).reshape(T, -1)], dim=1).to(DEV)
    q = qkv[:, :nh * hd]
    _ops.rope_kv_write(q, qkv[:, nh * hd:(nh + nkv) * hd], qkv[:, (nh + nkv) * hd:], ctx.positions, ctx.req_of_token, (inv, hd, False),
                       nh, nkv, hd, kc, vc, table_d, page)
    fill = torch.tensor(1e4, dtype=dtype).item()          # the fill as bfloat16 holds it
    changed_k = int((kc != fill).sum().item())
    changed_v = int((vc != -fill).sum().item())
    assert changed_k == changed_v == (old_cells + T) * nkv * hd, "cells were written elsewhere, or not at all"
    k_rot = P.rope(new_k, pos, freqs, False)
    req = ctx.req_of_token.cpu().tolist()
    for t in (0, 39, 40, 41, 42, T - 1):
        pg, sl = table[req[t], pos[t] // page].item(), pos[t] % page
        close(kc[pg, :, sl], k_rot[t], 2 ** -8, f"k of token {t}")
        assert torch.equal(vc[pg, :, :, sl].cpu().float(), new_v[t].to(dtype).float())
    # attention over what the cache now holds, by every kernel
    dense, row = [], 0
    for r, kv in enumerate(kv_lens):
        pgs = table[r, :blocks[r]].tolist()
        dense.append((torch.cat([kc[pg].transpose(0, 1) for pg in pgs])[:kv].cpu().float(),
                      torch.cat([vc[pg].permute(2, 0, 1) for pg in pgs])[:kv].cpu().float()))
    qs, row = [], 0
    for n in q_lens:
        qs.append(q[row:row + n].cpu().float().reshape(n, nh, hd))
        row += n
    scale = hd ** -0.5
    want = dense_attention(qs, dense, q_lens, kv_lens, scale, None).reshape(T, nh * hd)
    for fast in (True, False):
        _ops.use_fast_kernels(fast)
        out = torch.empty(T, nh * hd, dtype=dtype, device=DEV)
        _ops.paged_attention(out, q.contiguous(), kc, vc, table_d, ctx, nh, nkv, hd, page, scale, 0)
        close(out, want, 2 ** -7, f"attention, matrix-core kernels {fast}")
    _ops.use_fast_kernels(True)
    # a step of single tokens through the kernel that starts from the projection
    ctx1 = attention_ctx([1] * R, [kv + 1 for kv in kv_lens], dtype)
    assert all(kv % page for kv in kv_lens)       # every request's last page has room for one more token
    step = (torch.randn(R, (nh + 2 * nkv) * hd, generator=g) * 0.6).to(dtype).to(DEV)
    got = torch.empty(R, nh * hd, dtype=dtype, device=DEV)
    assert _ops.decode_attention_from_projection(got, step, ctx1, (inv, hd, False), nh, nkv, hd, kc, vc, table_d, page, scale, 0, True)
    assert int((kc != fill).sum().item()) == changed_k + R * nkv * hd
    dense1, q1 = [], []
    pos1 = ctx1.positions.cpu().tolist()
    q_rot = P.rope(step[:, :nh * hd].cpu().float().reshape(R, nh, hd), pos1, freqs, False).to(dtype).float()
    for r, kv in enumerate(kv_lens):
        pgs = table[r, :-(-(kv + 1) // page)].tolist()
        dense1.append((torch.cat([kc[pg].transpose(0, 1) for pg in pgs])[:kv + 1].cpu().float(),
                       torch.cat([vc[pg].permute(2, 0, 1) for pg in pgs])[:kv + 1].cpu().float()))
        q1.append(q_rot[r:r + 1])
    want1 = dense_attention(q1, dense1, [1] * R, [kv + 1 for kv in kv_lens], scale, None).reshape(R, nh * hd)
    close(got, want1, 2 ** -7, "from the projection")


# ------------------------------------------------------------------ sampling
def test_greedy_takes_the_lowest_index_among_equals(_ops):
    V = 128256
    l = torch.randn(6, V, generator=gen(12))
    l[0, 7] = 100.0                                            # tests/model/test_llama_model.cpp:236-249
    l[1, [70000, 99, 120000]] = 50.0
    l[2] = 0.0
    l[3, V - 1] = 60.0
    l[4, :] = float("-inf"); l[4, 4321] = -5.0
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    _ops.sample(out, l.to(DEV))
    assert out.cpu().tolist()[:5] == [7, 99, 0, V - 1, 4321]
    assert out[5].item() == P.argmax(l[5])


def test_temperature_sampling_matches_the_inverse_cdf(_ops):
    V = 1001
    g = gen(13)
    l = torch.randn(64, V, generator=g) * 3
    temps = torch.full((64,), 0.8)
    temps[::7] = 0.0                                           # greedy rows beside sampled rows
    u = torch.rand(64, generator=g)
    out = torch.empty(64, dtype=torch.int32, device=DEV)
    _ops.sample(out, l.to(DEV), temps.to(DEV), u.to(DEV))
    got = out.cpu().tolist()
    for r in range(64):
        if temps[r] == 0:
            assert got[r] == P.argmax(l[r])
            continue
        p = torch.softmax(l[r].double() / 0.8, 0)
        c = torch.cumsum(p, 0)
        lo = c[got[r] - 1].item() if got[r] > 0 else 0.0
        assert lo - 1e-5 <= u[r].item() <= c[got[r]].item() + 1e-5, r


def test_temperature_sampling_frequencies_and_limits(_ops):
    from photon_infer_amd.sampling import uniform_draw
    l = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]]).expand(4000, 5).contiguous()
    u = torch.tensor([uniform_draw(123, i) for i in range(4000)])
    assert 0 < u.min() and u.max() < 1 and abs(u.mean().item() - 0.5) < 0.02
    out = torch.empty(4000, dtype=torch.int32, device=DEV)
    _ops.sample(out, l.to(DEV), torch.full((4000,), 0.8, device=DEV), u.to(DEV))
    freq = torch.bincount(out.cpu().long(), minlength=5).float() / 4000
    assert (freq - torch.softmax(l[0] / 0.8, 0)).abs().max() < 0.025
    # a tiny temperature is the argmax; u near 1 still lands on a token with p > 0
    _ops.sample(out[:2], l[:2].to(DEV), torch.full((2,), 1e-4, device=DEV), torch.tensor([0.3, 0.9999999], device=DEV))
    assert out[:2].cpu().tolist() == [2, 2]


# ------------------------------------------------------------------ sampling from large vocabularies (two kernels)
def _sample_chunk(V):
    """Length of the chunks a row of V logits is cut into (0: rows this short take one kernel)."""
    from photon_infer_amd.ops import _lib
    chunks = _lib.load("core").pi_sample_chunks(V)
    return -(-V // chunks) if chunks else 0


@pytest.mark.parametrize("V", [16385, 50021, 128256])
def test_temperature_sampling_of_large_vocabularies_matches_the_inverse_cdf(_ops, V):
    assert _sample_chunk(V) > 0 and _sample_chunk(16384) == 0
    g = gen(V)
    M = 24
    l = torch.randn(M, V, generator=g) * 3
    temps = torch.full((M,), 0.7)
    temps[::5] = 0.0                                            # greedy rows beside sampled rows
    temps[1::5] = 1.9
    u = torch.rand(M, generator=g)
    u[2], u[3], u[7] = 0.0, 0.99999994, 1e-7
    out = torch.empty(M, dtype=torch.int32, device=DEV)
    _ops.sample(out, l.to(DEV), temps.to(DEV), u.to(DEV))
    got = out.cpu().tolist()
    for r in range(M):
        if temps[r] == 0:
            assert got[r] == int(l[r].argmax())
            continue
        c = torch.cumsum(torch.softmax(l[r].double() / temps[r].item(), 0), 0)
        lo = c[got[r] - 1].item() if got[r] > 0 else 0.0
        assert lo - 2e-5 <= u[r].item() <= c[got[r]].item() + 2e-5, (r, got[r], lo, u[r].item(), c[got[r]].item())


@pytest.mark.parametrize("V", [16385, 50021, 128256])
def test_temperature_sampling_at_the_edges_of_chunks(_ops, V):
    """Rows whose probability sits on a few tokens at chunk edges, so that the draw names its token
    without doubt: the last token of a chunk and the first of the next, chunks without any weight
    before, between and after them, the first and the last token of the row."""
    chunk = _sample_chunk(V)
    chunks = -(-V // chunk)
    NEG = float("-inf")
    rows, draws, want = [], [], []

    def case(weights: dict, u: float, token: int, floor=NEG):
        row = torch.full((V,), floor)
        for i, w in weights.items():
            row[i] = math.log(w)
        rows.append(row)
        draws.append(u)
        want.append(token)

    k = chunks // 2
    a, b = k * chunk - 1, k * chunk                      # last token of chunk k-1, first of chunk k
    for u, tok in ((0.25, a), (0.4999, a), (0.5001, b), (0.75, b), (1e-9, a), (0.99999994, b)):
        case({a: 0.5, b: 0.5}, u, tok)                   # every other chunk holds -inf only
    # the same with a little weight everywhere (1e-12 in all of the rest together)
    for u, tok in ((0.25, a), (0.4999, a), (0.5001, b), (0.75, b)):
        case({a: 0.5, b: 0.5}, u, tok, floor=math.log(1e-12 / V))
    # first and last token of the row; the last chunk is the short one
    case({0: 0.3, V - 1: 0.7}, 0.29, 0)
    case({0: 0.3, V - 1: 0.7}, 0.31, V - 1)
    case({0: 0.3, V - 1: 0.7}, 0.99999994, V - 1)
    # three tokens in three different chunks with empty chunks between them
    x, y, z = 5, (chunks // 3) * chunk + 17, (chunks - 1) * chunk + 1
    for u, tok in ((0.1, x), (0.21, y), (0.69, y), (0.71, z), (0.95, z)):
        case({x: 0.2, y: 0.5, z: 0.3}, u, tok)
    # all the weight in one chunk, spread over the chunk's last 100 tokens
    lo_tok = 2 * chunk - 100
    for u in (0.005, 0.505, 0.995):
        case({lo_tok + i: 0.01 for i in range(100)}, u, lo_tok + int(u * 100))
    l = torch.stack(rows)
    for tau in (1.0, 0.5):
        # at temperature tau the weights are p^(1/tau): feed tau * log p to keep the intended weights
        out = torch.empty(len(rows), dtype=torch.int32, device=DEV)
        _ops.sample(out, (l * tau).to(DEV), torch.full((len(rows),), tau, device=DEV), torch.tensor(draws, device=DEV))
        assert out.cpu().tolist() == want, tau
    # the plain implementation agrees on the crafted rows (a few of them: it walks the row in Python)
    for r in (1, 2, 11, 14):
        assert P.sample_temperature(l[r].double(), 1.0, draws[r]) == want[r]
