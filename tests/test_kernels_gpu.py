"""Each kernel alone against its plain reference, at other sizes than the tiny models'."""

import math

import numpy as np
import pytest
import torch

import plain_qwen2 as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def rnd(shape, seed, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def tol(dtype, ref, f32=1e-5, bf16=2.0 ** -7):
    return f32 * max(1.0, ref.abs().max().item()) if dtype == torch.float32 else bf16 * ref.abs().max().item()


@pytest.fixture(scope="module")
def ops():
    from from_scratch_inference_engine_amd import ops as o

    o.load(build_if_missing=False)
    return o


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(ops, dtype):
    table = rnd((1000, 896), 0, dtype)
    ids = torch.tensor([999, 0, 17, 17, 500], dtype=torch.int32)
    out = ops.embedding(table.cuda(), ids.cuda()).cpu()
    assert out.dtype == torch.float32 and torch.equal(out, plain.embedding(table.float(), ids.tolist()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, eps", [(896, 1e-6), (100, 1e-5), (4099, 0.5)])
def test_rmsnorm_alone_fused_and_rows(ops, dtype, hidden, eps):
    x, d, w = rnd((7, hidden), 1), rnd((7, hidden), 2, dtype), rnd((hidden,), 3) + 1.0
    ref = plain.rms_norm(x, w, eps)
    out = ops.rmsnorm(x.cuda(), w.cuda(), eps, dtype).float().cpu()
    assert (out - ref).abs().max() <= tol(dtype, ref)
    # fused with the residual sum: the stream is updated in float32, the norm sees the sum
    res = x.clone().cuda()
    out = ops.rmsnorm(res, w.cuda(), eps, dtype, delta=d.cuda(), write_back=True).float().cpu()
    summed = x + d.float()
    assert torch.equal(res.cpu(), summed)
    ref = plain.rms_norm(summed, w, eps)
    assert (out - ref).abs().max() <= tol(dtype, ref)
    # chosen rows, pending delta not written back
    rows = torch.tensor([6, 0, 3, 3], dtype=torch.int32)
    res = x.clone().cuda()
    out = ops.rmsnorm(res, w.cuda(), eps, dtype, delta=d.cuda(), rows=rows.cuda()).float().cpu()
    assert torch.equal(res.cpu(), x) and (out - ref[rows.long()]).abs().max() <= tol(dtype, ref)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_and_adds(ops, dtype):
    for inter in (4864, 333):  # gate and up interleaved: (g0, u0, g1, u1, ...)
        x = rnd((5, 2 * inter), 4, dtype, 3.0)
        ref = plain.silu_mul(x.float()[:, 0::2], x.float()[:, 1::2])
        out = ops.swiglu(x.cuda()).float().cpu()
        assert (out - ref).abs().max() <= tol(dtype, ref)
    res, d = rnd((3, 333), 5), rnd((3, 333), 6, dtype)
    assert torch.equal(ops.residual_add(res.clone().cuda(), d.cuda()).cpu(), res + d.float())
    y, b = rnd((4, 77), 7, dtype), rnd((77,), 8)
    assert (ops.bias_add(y.clone().cuda(), b.cuda()).float().cpu() - (y.float() + b)).abs().max() <= tol(dtype, y.float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("from_table", [False, True])  # the angles computed by the kernel, or read from the step's table
@pytest.mark.parametrize("heads, kv, hd, theta", [(14, 2, 64, 1e6), (3, 3, 48, 1e4), (5, 1, 256, 5e5), (7, 2, 24, 3e4)])
def test_rope_and_cache_write(ops, dtype, from_table, heads, kv, hd, theta):
    t, page, pages = 9, 4, 11
    width = (heads + 2 * kv) * hd
    qkv, bias = rnd((t, width), 9, dtype), rnd((width,), 10)
    pos = torch.tensor([3, 4, 5, 0, 1, 4000, 17, 18, 19], dtype=torch.int32)
    slots = torch.tensor([12, 13, 14, 40, 41, -1, 5, 6, 7], dtype=torch.int32)
    inv = torch.tensor([theta ** (-2.0 * i / hd) for i in range(hd // 2)], dtype=torch.float64)
    k_pool = torch.zeros((pages, kv, page, hd), dtype=dtype)
    v_pool = torch.zeros((pages, kv, hd, page), dtype=dtype)
    dq, dk, dv = qkv.clone().cuda(), k_pool.cuda(), v_pool.cuda()
    table = ops.rope_table(pos.cuda(), inv.cuda()) if from_table else None
    ops.rope_kv_write(dq, pos.cuda(), heads, kv, hd, inv.cuda(), slots=slots.cuda(), k_pool=dk, v_pool=dv,
                      page_size=page, bias=bias.cuda(), cos_sin=table)
    if from_table:  # without a bias and without a cache as well
        alone = qkv.clone().cuda()
        ops.rope_kv_write(alone, pos.cuda(), heads, kv, hd, inv.cuda(), cos_sin=table)
        want = plain.rope(qkv.float()[:, :heads * hd], heads, hd, theta, pos.tolist())
        assert (alone.float().cpu()[:, :heads * hd] - want).abs().max() <= tol(dtype, want, f32=2e-6)
        assert torch.equal(alone.cpu()[:, (heads + kv) * hd:], qkv[:, (heads + kv) * hd:])
    full = qkv.float() + bias
    q_ref = plain.rope(full[:, :heads * hd], heads, hd, theta, pos.tolist())
    k_ref = plain.rope(full[:, heads * hd:(heads + kv) * hd], kv, hd, theta, pos.tolist())
    v_ref = full[:, (heads + kv) * hd:]
    got = dq.float().cpu()
    assert (got[:, :heads * hd] - q_ref).abs().max() <= tol(dtype, q_ref, f32=2e-6)
    assert (got[:, heads * hd:(heads + kv) * hd] - k_ref).abs().max() <= tol(dtype, k_ref, f32=2e-6)
    kp, vp = dk.float().cpu(), dv.float().cpu()
    written = torch.zeros(pages * page, dtype=torch.bool)
    for i, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        written[s] = True
        assert (kp[s // page, :, s % page, :].reshape(-1) - k_ref[i]).abs().max() <= tol(dtype, k_ref, f32=2e-6)
        assert (vp[s // page, :, :, s % page].reshape(-1) - v_ref[i]).abs().max() <= tol(dtype, v_ref, f32=2e-6)
    untouched = ~written.reshape(pages, 1, page, 1).expand_as(kp)
    assert kp[untouched].abs().max() == 0 and vp.transpose(2, 3)[untouched].abs().max() == 0
    if from_table:
        # the projection as three partial sums (what a product cut along its inner dimension leaves):
        # the same q heads and pools; the k and v columns of the result are not written
        g = torch.Generator().manual_seed(5)
        p1, p2 = torch.randn(t, width, generator=g), torch.randn(t, width, generator=g)
        parts = torch.stack([p1, p2, qkv.float() - p1 - p2]).cuda()
        out = torch.full((t, width), 7.0, dtype=dtype).cuda()
        dk2, dv2 = k_pool.cuda(), v_pool.cuda()
        ops.rope_kv_write(out, pos.cuda(), heads, kv, hd, inv.cuda(), slots=slots.cuda(), k_pool=dk2, v_pool=dv2,
                          page_size=page, bias=bias.cuda(), cos_sin=table, parts=parts)
        out = out.float().cpu()
        assert (out[:, :heads * hd] - q_ref).abs().max() <= tol(dtype, q_ref, f32=4e-6)
        assert (out[:, heads * hd:] == 7.0).all()
        assert (dk2.float().cpu() - kp).abs().max() <= tol(dtype, k_ref, f32=4e-6)
        assert (dv2.float().cpu() - vp).abs().max() <= tol(dtype, v_ref, f32=4e-6)
        with pytest.raises(Exception, match="partial sums"):
            ops.rope_kv_write(out.to(dtype).cuda(), pos.cuda(), heads, kv, hd, inv.cuda(), parts=parts)
    # no rotation, no cache: only the bias on q and k
    dq = qkv.clone().cuda()
    ops.rope_kv_write(dq, pos.cuda(), heads, kv, hd, None, bias=bias.cuda())
    assert (dq.float().cpu()[:, :(heads + kv) * hd] - full[:, :(heads + kv) * hd]).abs().max() <= tol(dtype, full)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [16, 8, 4])
def test_rope_from_table_on_a_long_batch(ops, dtype, page):
    """From 1,024 tokens on a block takes eight tokens and writes the values of eight consecutive
    slots that start at a multiple of 8 with one store per dimension.  A batch of 1,029 tokens:
    portions whose slots run on (aligned and not), single tokens anywhere, tokens that are not
    stored, a tail of five; every slot of the pools is compared."""
    heads, kv, hd, theta = 4, 2, 32, 1e4
    t = 1029
    pages = 2 * t // page + 8
    g = torch.Generator().manual_seed(77 + page)
    slots = torch.full((t,), -1, dtype=torch.int32)
    free = torch.randperm(pages, generator=g).tolist()
    i = 0
    while i < t:
        kind = int(torch.randint(0, 4, (1,), generator=g))
        if kind == 0:                      # a portion: consecutive slots over whole pages, from a random offset
            n = min(int(torch.randint(5, 90, (1,), generator=g)), t - i)
            off = int(torch.randint(0, page, (1,), generator=g))
            need = -(-(off + n) // page)
            mine = [free.pop() for _ in range(need)]
            for j in range(n):
                slots[i + j] = mine[(off + j) // page] * page + (off + j) % page
            i += n
        elif kind == 1:                    # a decoded token
            slots[i] = free.pop() * page + int(torch.randint(0, page, (1,), generator=g))
            i += 1
        elif kind == 2:                    # not stored
            i += 1
        else:                              # eight aligned ones
            n = min(8, t - i)
            p0 = free.pop() if page >= 8 else None
            for j in range(n):
                slots[i + j] = (p0 * page + j) if p0 is not None else free.pop() * page
            i += n
    width = (heads + 2 * kv) * hd
    qkv, bias = rnd((t, width), 90, dtype), rnd((width,), 91)
    pos = torch.randint(0, 5000, (t,), generator=g, dtype=torch.int32)
    inv = torch.tensor([theta ** (-2.0 * k / hd) for k in range(hd // 2)], dtype=torch.float64)
    dq = qkv.clone().cuda()
    dk = torch.zeros((pages, kv, page, hd), dtype=dtype).cuda()
    dv = torch.zeros((pages, kv, hd, page), dtype=dtype).cuda()
    table = ops.rope_table(pos.cuda(), inv.cuda())
    ops.rope_kv_write(dq, pos.cuda(), heads, kv, hd, inv.cuda(), slots=slots.cuda(), k_pool=dk, v_pool=dv,
                      page_size=page, bias=bias.cuda(), cos_sin=table)
    full = qkv.float() + bias
    q_ref = plain.rope(full[:, :heads * hd], heads, hd, theta, pos.tolist())
    k_ref = plain.rope(full[:, heads * hd:(heads + kv) * hd], kv, hd, theta, pos.tolist())
    v_ref = full[:, (heads + kv) * hd:]
    got = dq.float().cpu()
    assert (got[:, :heads * hd] - q_ref).abs().max() <= tol(dtype, q_ref, f32=2e-6)
    assert (got[:, heads * hd:(heads + kv) * hd] - k_ref).abs().max() <= tol(dtype, k_ref, f32=2e-6)
    want_k = torch.zeros(pages * page, kv * hd)
    want_v = torch.zeros(pages * page, kv * hd)
    stored = slots >= 0
    want_k[slots[stored].long()] = k_ref[stored]
    want_v[slots[stored].long()] = v_ref[stored]
    kp = dk.float().cpu().permute(0, 2, 1, 3).reshape(pages * page, kv * hd)   # [slot][kv head][dim]
    vp = dv.float().cpu().permute(0, 3, 1, 2).reshape(pages * page, kv * hd)
    assert (kp - want_k).abs().max() <= tol(dtype, k_ref, f32=2e-6)
    assert (vp - want_v).abs().max() <= tol(dtype, v_ref, f32=2e-6)


@pytest.mark.parametrize("m, n, k", [(1, 4864, 896), (5, 151, 100), (8, 1000, 4864), (37, 300, 129), (130, 896, 1000)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm(ops, dtype, m, n, k):
    x, w, b = rnd((m, k), 11, dtype), rnd((n, k), 12, dtype, 0.05), rnd((n,), 13)
    ref = plain.linear(x.float(), w.float(), b)
    for kind in (1, 2) if m <= 8 else (1,):
        out = ops.gemm(x.cuda(), w.cuda(), b.cuda(), kind=kind).float().cpu()
        assert (out - ref).abs().max() <= tol(dtype, ref, f32=2e-6), f"kind {kind}"
    out32 = ops.gemm(x.cuda(), w.cuda(), None, out_dtype=torch.float32).cpu()
    assert out32.dtype == torch.float32 and (out32 - plain.linear(x.float(), w.float())).abs().max() <= 2e-5 * ref.abs().max() + 1e-6


@pytest.mark.parametrize("m, n, k, waves", [(1, 4864, 896, 0), (8, 1000, 4864, 0), (16, 48, 64, 1), (17, 151, 104, 2),
                                             (33, 896, 1000, 4), (64, 3584, 2048, 16), (50, 16, 8, 8), (7, 4608, 3584, 0)])
def test_gemm_mfma_skinny(ops, m, n, k, waves):
    x, w, b = rnd((m, k), 14, torch.bfloat16), rnd((n, k), 15, torch.bfloat16, 0.05), rnd((n,), 16)
    ref = plain.linear(x.float(), w.float(), b)
    out = ops.gemm_mfma_skinny(x.cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32, waves=waves).cpu()
    assert (out - ref).abs().max() <= 2e-5 * ref.abs().max()  # float32 sums of exact bfloat16 products
    if m > 16:  # bfloat16 results are offered for decoding's few rows only
        with pytest.raises(ops.KernelError, match="bfloat16 results for at most 16 rows"):
            ops.gemm_mfma_skinny(x.cuda(), w.cuda(), None, waves=waves)
        return
    out = ops.gemm_mfma_skinny(x.cuda(), w.cuda(), None, waves=waves).float().cpu()
    ref = plain.linear(x.float(), w.float())
    assert (out - ref).abs().max() <= tol(torch.bfloat16, ref)


@pytest.mark.parametrize("m, n, k, splits, waves", [(1, 896, 4864, 2, 0), (8, 3584, 18944, 8, 0), (16, 100, 1032, 4, 2),
                                                     (5, 48, 136, 2, 1), (13, 1000, 1000, 8, 4)])
def test_gemm_mfma_skinny_partial_sums_feed_the_norm(ops, m, n, k, splits, waves):
    """K cut into slices: the partial sums add up to the product, and the norm that takes them
    as its delta gives what it gives for the whole product."""
    x, w = rnd((m, k), 24, torch.bfloat16), rnd((n, k), 25, torch.bfloat16, 0.05)
    ref = plain.linear(x.float(), w.float())
    parts = ops.gemm_mfma_skinny(x.cuda(), w.cuda(), splits=splits, waves=waves)
    assert parts.shape == (splits, m, n) and parts.dtype == torch.float32
    total = parts.cpu().double().sum(0).float()
    assert (total - ref).abs().max() <= 2e-5 * ref.abs().max()
    # a slice holds only its own part of K (a slice that read beyond its end would not)
    k_slice = -(-(-(-k // splits)) // 64) * 64
    first = plain.linear(x[:, :k_slice].float(), w[:, :k_slice].float())
    assert (parts[0].cpu() - first).abs().max() <= 2e-5 * ref.abs().max()
    if n % 4:
        return
    res0, g, eps = rnd((m, n), 26), rnd((n,), 27) + 1.0, 1e-6
    for dtype in DTYPES:
        res = res0.clone().cuda()
        out = ops.rmsnorm(res, g.cuda(), eps, dtype, delta=parts, write_back=True).float().cpu()
        summed = res0 + total
        assert (res.cpu() - summed).abs().max() <= 1e-5 * summed.abs().max()
        want = plain.rms_norm(summed, g, eps)
        assert (out - want).abs().max() <= tol(dtype, want)
        rows = torch.tensor([m - 1, 0], dtype=torch.int32)
        res = res0.clone().cuda()
        out = ops.rmsnorm(res, g.cuda(), eps, dtype, delta=parts, rows=rows.cuda()).float().cpu()
        assert torch.equal(res.cpu(), res0) and (out - want[rows.long()]).abs().max() <= tol(dtype, want)


@pytest.mark.parametrize("m, n, k, splits, waves", [(17, 151, 256, 1, 0), (64, 272, 1024, 4, 8), (33, 100, 384, 2, 4),
                                                     (50, 16, 128, 1, 8), (64, 3584, 2048, 8, 0), (40, 1000, 1152, 1, 4),
                                                     (5, 130, 640, 2, 0)])
def test_gemm_mfma_wide(ops, m, n, k, splits, waves):
    """The product that shares the rows of x through LDS: whole, and cut into slices whose partial
    sums add up; a slice holds its own part of K only; sizes it does not take are refused."""
    x, w = rnd((m, k), 44, torch.bfloat16), rnd((n, k), 45, torch.bfloat16, 0.05)
    ref = plain.linear(x.float(), w.float())
    out = ops.gemm_mfma_wide(x.cuda(), w.cuda(), splits=splits, waves=waves)
    assert out.dtype == torch.float32 and out.shape == ((m, n) if splits == 1 else (splits, m, n))
    total = out.cpu() if splits == 1 else out.cpu().double().sum(0).float()
    assert (total - ref).abs().max() <= 2e-5 * ref.abs().max()  # float32 sums of exact bfloat16 products
    if splits > 1:
        k_slice = -(-(-(-k // splits)) // 128) * 128
        first = plain.linear(x[:, :k_slice].float(), w[:, :k_slice].float())
        assert (out[0].cpu() - first).abs().max() <= 2e-5 * ref.abs().max()
        last = plain.linear(x[:, k_slice * (splits - 1):].float(), w[:, k_slice * (splits - 1):].float())
        assert (out[-1].cpu() - last).abs().max() <= 2e-5 * ref.abs().max()
    # the same rows give the same sums whatever else is in the batch
    if m > 3:
        fewer = ops.gemm_mfma_wide(x[2:m - 1].contiguous().cuda(), w.cuda(), splits=splits, waves=waves)
        assert torch.equal(fewer.cpu(), out.cpu()[..., 2:m - 1, :])
    # and whatever the launch shape: one or two blocks of W a wave, 2, 4 or 8 waves a workgroup
    for blocks, wv in [(1, 2), (2, 4), (2, 8), (1, 8), (2, 2)]:
        other = ops.gemm_mfma_wide(x.cuda(), w.cuda(), splits=splits, waves=wv, blocks=blocks)
        assert torch.equal(other.cpu(), out.cpu()), (blocks, wv)


def _exact(x, w):
    """x . w^T in float64 on the device: the exact sums of the bfloat16 products, to float32's last bits."""
    return (x.cuda().double() @ w.cuda().double().t()).float().cpu()


@pytest.mark.parametrize("n, k", [(3584, 18944), (5120, 13824), (5120, 27648), (3584, 3584), (152064, 3584)])
def test_gemm_mfma_wide_at_the_large_models_shapes(ops, n, k):
    """The residual projections and the logits at the layer sizes of the 7B, 14B and 32B shapes,
    with the slices the engine's Linear picks there for 8, 17 and 64 rows (K = 18944 on 256 compute
    units: eight slices, seven of 2,432 and one of 1,920, at 8 rows; nine at 64), and with 3, 7 and
    16 slices where K gives them."""
    from from_scratch_inference_engine_amd.parts.linear import Linear

    w = rnd((n, k), 51, torch.bfloat16, 0.05)
    picked = {}
    for m in (8, 17, 64):
        x = rnd((m, k), 50 + m, torch.bfloat16)
        ref = _exact(x, w)
        picked[m] = 1 if n == 152064 else Linear(k, n).wide_splits(m)
        for splits in {picked[m]} | ({3, 7, 16} if n != 152064 and m == 17 else set()):
            if not ops.gemm_mfma_wide_splits_ok(k, splits):
                continue
            out = ops.gemm_mfma_wide(x.cuda(), w.cuda(), splits=splits).cpu()
            total = out if splits == 1 else out.double().sum(0).float()
            assert (total - ref).abs().max() <= 2e-5 * ref.abs().max(), (m, n, k, splits)
    if n != 152064:
        assert picked[8] == (7 if k == 3584 else 8), picked           # as many slices of 512 or more as K gives, up to 8
        if ops.compute_units() == 256:
            assert picked[64] == {(3584, 18944): 9, (5120, 13824): 6, (5120, 27648): 6, (3584, 3584): 4}[(n, k)], picked


def test_gemm_mfma_skinny_at_the_large_models_shapes(ops):
    """Logits of 1 and 7 rows at a vocabulary of 152,064; SiLU(gate) * up at the 32B shape's
    2 x 27,648 rows of 5,120; the output projection's partial sums at hidden 5,120."""
    w = rnd((152064, 3584), 52, torch.bfloat16, 0.05)
    for m in (1, 7):
        x = rnd((m, 3584), 53 + m, torch.bfloat16)
        ref = _exact(x, w)
        out = ops.gemm_mfma_skinny(x.cuda(), w.cuda(), out_dtype=torch.float32).cpu()
        assert (out - ref).abs().max() <= 2e-5 * ref.abs().max(), m
    w = rnd((2 * 27648, 5120), 54, torch.bfloat16, 0.03)
    for m in (1, 16):
        x = rnd((m, 5120), 55 + m, torch.bfloat16)
        full = _exact(x, w)
        ref = plain.silu_mul(full[:, 0::2], full[:, 1::2])
        out = ops.gemm_mfma_skinny(x.cuda(), w.cuda(), epilogue="swiglu").float().cpu()
        assert (out - ref).abs().max() <= tol(torch.bfloat16, ref), m
    w = rnd((5120, 5120), 56, torch.bfloat16, 0.05)
    x = rnd((8, 5120), 57, torch.bfloat16)
    from from_scratch_inference_engine_amd.parts.linear import Linear
    splits = Linear(5120, 5120).residual_splits(8)
    assert splits > 1
    out = ops.gemm_mfma_skinny(x.cuda(), w.cuda(), splits=splits).cpu().double().sum(0).float()
    assert (out - _exact(x, w)).abs().max() <= 2e-5 * out.abs().max()


def test_gemm_mfma_wide_refuses_what_it_does_not_take(ops):
    x, w = rnd((20, 200), 46, torch.bfloat16), rnd((32, 200), 47, torch.bfloat16)
    with pytest.raises(ops.KernelError, match="whole stages of 128"):
        ops.gemm_mfma_wide(x.cuda(), w.cuda())
    x, w = rnd((20, 384), 46, torch.bfloat16), rnd((32, 384), 47, torch.bfloat16)
    assert not ops.gemm_mfma_wide_splits_ok(384, 4) and ops.gemm_mfma_wide_splits_ok(384, 2)
    with pytest.raises(ops.KernelError, match="whole stages of 128"):
        ops.gemm_mfma_wide(x.cuda(), w.cuda(), splits=4)
    x = rnd((65, 384), 46, torch.bfloat16)
    with pytest.raises(ops.KernelError, match="at most 64 rows"):
        ops.gemm_mfma_wide(x.cuda(), w.cuda())


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_at_every_row_length_class(ops, dtype):
    """A thread of the vector kernel holds one to eight quads of the row (1,024 values a quad):
    row lengths in every class, at its upper edge and just inside it, with eight partial sums (one of
    the counts the kernel is made for, as all from 2 to 9 are) or with 10, 12 or 16 (its loop over any count)."""
    for i, hidden in enumerate((1024, 1028, 2560, 3072, 3584, 5120, 5124, 6144, 7000, 8192)):
        x, g = rnd((2, hidden), 40), rnd((hidden,), 41) + 1.0
        parts = rnd(((8, 3, 5, 6, 9, 7, 16, 12, 10, 2)[i], 2, hidden), 42)
        summed = x + parts.double().sum(0).float()
        want = plain.rms_norm(summed, g, 1e-6)
        res = x.clone().cuda()
        out = ops.rmsnorm(res, g.cuda(), 1e-6, dtype, delta=parts.cuda(), write_back=True).float().cpu()
        assert (res.cpu() - summed).abs().max() <= 1e-5 * summed.abs().max(), hidden
        assert (out - want).abs().max() <= tol(dtype, want), hidden


def test_rmsnorm_adds_partial_sums_at_odd_sizes(ops):
    """Sizes the vector kernel does not take: hidden not a multiple of 4 and larger than its registers hold."""
    for hidden, n_parts in [(102, 2), (9001 * 4, 4), (4099, 8), (4099, 9), (102, 5)]:
        x, g = rnd((3, hidden), 28), rnd((hidden,), 29) + 1.0
        parts = rnd((n_parts, 3, hidden), 30)
        summed = x + parts.double().sum(0).float()
        want = plain.rms_norm(summed, g, 1e-5)
        res = x.clone().cuda()
        out = ops.rmsnorm(res, g.cuda(), 1e-5, torch.float32, delta=parts.cuda(), write_back=True).cpu()
        assert (res.cpu() - summed).abs().max() <= 1e-5 * summed.abs().max()
        assert (out - want).abs().max() <= tol(torch.float32, want)


@pytest.mark.parametrize("m, heads, kv, hd, k, theta, use_bias", [
    (1, 14, 2, 64, 896, 1e6, True), (9, 3, 3, 48, 72, 1e4, True), (16, 5, 1, 256, 320, 5e5, False),
    (7, 28, 4, 128, 3584, 1e6, True), (33, 2, 1, 16, 64, 1e4, True),
    # on 256 compute units these deal 10 and 14 rotary pairs a workgroup; with a head size of 160 a block's pairs span two heads
    (8, 24, 4, 160, 256, 1e4, True), (16, 40, 8, 128, 128, 1e6, False),
    # the q/k/v projection of the 14B and 32B shapes (7,168 rows of 5,120)
    (1, 40, 8, 128, 5120, 1e6, True), (8, 40, 8, 128, 5120, 1e6, True), (16, 40, 8, 128, 5120, 1e6, True),
    # up to 6 rows of a large projection: two workgroups a compute unit, 5 pairs each on 256 units (the last
    # one has 4; with a head size of 160 a workgroup's pairs span two heads), 7 pairs at 7,168 rows
    (1, 28, 4, 128, 3584, 1e6, True), (4, 28, 4, 128, 3584, 1e6, True), (6, 28, 4, 128, 3584, 1e6, False),
    (3, 24, 4, 160, 256, 1e4, True), (5, 40, 8, 128, 5120, 1e6, True)])
def test_projection_with_rotary_epilogue(ops, m, heads, kv, hd, k, theta, use_bias):
    """q/k/v projection, bias, rotation and cache write in one kernel, against the plain formulas
    on the float32 product (one rounding to bfloat16, after the rotation)."""
    page, pages = 4, 24
    n = (heads + 2 * kv) * hd
    x, w = rnd((m, k), 40, torch.bfloat16), rnd((n, k), 41, torch.bfloat16, 0.05)
    bias = rnd((n,), 42) if use_bias else None
    g = torch.Generator().manual_seed(43)
    pos = torch.randint(0, 5000, (m,), generator=g, dtype=torch.int32)
    slots = torch.randperm(pages * page, generator=g)[:m].to(torch.int32)
    slots[m // 2] = -1  # this token is not stored
    inv = torch.tensor([theta ** (-2.0 * i / hd) for i in range(hd // 2)], dtype=torch.float64)
    dk = torch.zeros((pages, kv, page, hd), dtype=torch.bfloat16).cuda()
    dv = torch.zeros((pages, kv, hd, page), dtype=torch.bfloat16).cuda()
    got = ops.gemm_mfma_skinny_rope(x.cuda(), w.cuda(), None if bias is None else bias.cuda(), pos.cuda(), heads, kv,
                                    hd, inv.cuda(), slots=slots.cuda(), k_pool=dk, v_pool=dv, page_size=page)
    full = plain.linear(x.float(), w.float(), bias)
    q_ref = plain.rope(full[:, :heads * hd], heads, hd, theta, pos.tolist())
    k_ref = plain.rope(full[:, heads * hd:(heads + kv) * hd], kv, hd, theta, pos.tolist())
    v_ref = full[:, (heads + kv) * hd:]
    bf = torch.bfloat16
    assert (got.float().cpu()[:, :heads * hd] - q_ref).abs().max() <= tol(bf, q_ref)
    kp, vp = dk.float().cpu(), dv.float().cpu()
    written = torch.zeros(pages * page, dtype=torch.bool)
    for i, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        written[s] = True
        assert (kp[s // page, :, s % page, :].reshape(-1) - k_ref[i]).abs().max() <= tol(bf, k_ref), f"k of token {i}"
        assert (vp[s // page, :, :, s % page].reshape(-1) - v_ref[i]).abs().max() <= tol(bf, v_ref), f"v of token {i}"
    untouched = ~written.reshape(pages, 1, page, 1).expand_as(kp)
    assert kp[untouched].abs().max() == 0 and vp.transpose(2, 3)[untouched].abs().max() == 0
    # with the cosines and sines from the step's table instead of the kernel's own: the same bits
    table = ops.rope_table(pos.cuda(), inv.cuda())
    ang = pos.double().unsqueeze(1) * inv.unsqueeze(0)
    assert (table[..., 0].cpu() - torch.cos(ang).float()).abs().max() <= 5e-7
    assert (table[..., 1].cpu() - torch.sin(ang).float()).abs().max() <= 5e-7
    dk2, dv2 = torch.zeros_like(dk), torch.zeros_like(dv)
    got2 = ops.gemm_mfma_skinny_rope(x.cuda(), w.cuda(), None if bias is None else bias.cuda(), pos.cuda(), heads, kv,
                                     hd, inv.cuda(), slots=slots.cuda(), k_pool=dk2, v_pool=dv2, page_size=page,
                                     cos_sin=table)
    assert torch.equal(got2[:, :heads * hd], got[:, :heads * hd]) and torch.equal(dk2, dk) and torch.equal(dv2, dv)
    # the same without a cache and without rotation: q is the product plus bias
    got = ops.gemm_mfma_skinny_rope(x.cuda(), w.cuda(), None if bias is None else bias.cuda(), pos.cuda(), heads, kv,
                                    hd, None)
    assert (got.float().cpu()[:, :heads * hd] - full[:, :heads * hd]).abs().max() <= tol(bf, full)


@pytest.mark.parametrize("m, n, k", [(1, 9728, 896), (8, 352, 64), (13, 640, 192), (16, 37888, 3584)])
def test_gemm_mfma_skinny_with_swiglu_epilogue(ops, m, n, k):
    x, w = rnd((m, k), 17, torch.bfloat16), rnd((n, k), 18, torch.bfloat16, 0.05)
    full = plain.linear(x.float(), w.float())
    ref = plain.silu_mul(full[:, 0::2], full[:, 1::2])
    out = ops.gemm_mfma_skinny(x.cuda(), w.cuda(), epilogue="swiglu")
    assert out.shape == (m, n // 2)
    assert (out.float().cpu() - ref).abs().max() <= tol(torch.bfloat16, ref)


@pytest.mark.parametrize("m, n, k", [(3, 9728, 896), (8, 356, 128), (13, 644, 384), (16, 37888, 3584), (40, 1028, 256),
                                     (64, 27648, 5120), (9, 55296, 5120)])
def test_gemm_mfma_wide_with_swiglu_epilogue(ops, m, n, k):
    """The kernel that shares x through LDS with silu(gate) * up from its accumulators: every number of
    16-row tiles, an N that ends inside a block of rows, one and two blocks a wave, and the gate/up
    shapes of the large models."""
    from from_scratch_inference_engine_amd.ops import KernelError

    x, w = rnd((m, k), 17, torch.bfloat16), rnd((n, k), 18, torch.bfloat16, 0.05)
    full = (x.cuda().double() @ w.cuda().double().t()).float().cpu()
    ref = plain.silu_mul(full[:, 0::2], full[:, 1::2])
    for waves, blocks in ((0, 0), (2, 2), (8, 1)):
        out = ops.gemm_mfma_wide_swiglu(x.cuda(), w.cuda(), waves=waves, blocks=blocks)
        assert out.shape == (m, n // 2) and out.dtype == torch.bfloat16
        assert (out.float().cpu() - ref).abs().max() <= tol(torch.bfloat16, ref), (waves, blocks)
    with pytest.raises(KernelError, match="multiple of 4"):
        ops.gemm_mfma_wide_swiglu(x.cuda(), w[:n - 2].contiguous().cuda())


@pytest.mark.parametrize("n,k", [(331, 1024), (3072, 1024), (1000, 1536), (48, 128), (17, 256), (18944 * 2, 3584),
                                 (3584, 18944), (5120, 13824), (152064, 3584)])
def test_products_on_fragment_ordered_weights(ops, n, k):
    """The copy of a weight in the order of the matrix instruction's fragments: the layout itself
    (against the same permutation written with tensor views), and the products on it, which add the
    same numbers in the same order as on rows and so give the same bits: every number of 16-row tiles,
    an N that ends inside a block of 16 rows (the copy's last block is filled up with zeros), slices
    of K, both epilogues, every launch shape."""
    from from_scratch_inference_engine_amd.ops import KernelError

    w = rnd((n, k), 31, torch.bfloat16, 0.05).cuda()
    f = ops.fragment_order(w)
    assert f.shape == (n, k) and f.data.numel() == -(-n // 16) * 16 * k
    n16 = -(-n // 16) * 16
    padded = torch.zeros(n16, k, dtype=torch.bfloat16, device="cuda")
    padded[:n] = w
    # [block, row, step, k group, 8] -> [block, step, k group, row, 8]: lane = 16 * k group + row
    want = padded.view(n16 // 16, 16, k // 32, 4, 8).permute(0, 2, 3, 1, 4).reshape(-1)
    assert torch.equal(f.data, want)
    big = n * k > 1 << 24
    for m in ((8, 64) if big else (1, 2, 5, 16, 17, 33, 48, 64)):
        x = rnd((m, k), 32 + m, torch.bfloat16).cuda()
        shapes = ((0, 0),) if big else ((0, 0), (2, 1), (2, 2), (4, 1), (4, 2), (8, 1), (8, 2))
        for splits in (1, 2, 3, 8, 16):
            if not ops.gemm_mfma_wide_splits_ok(k, splits):
                continue
            for waves, blocks in shapes:
                a = ops.gemm_mfma_wide(x, w, splits=splits, waves=waves, blocks=blocks)
                b = ops.gemm_mfma_wide(x, f, splits=splits, waves=waves, blocks=blocks)
                assert torch.equal(a, b), (m, splits, waves, blocks)
        if n % 4 == 0:
            a = ops.gemm_mfma_wide_swiglu(x, w)
            for waves, blocks in shapes + (() if big else ((3, 2), (5, 2), (6, 2), (7, 2))):  # odd numbers of waves: this copy only
                b = ops.gemm_mfma_wide_swiglu(x, f, waves=waves, blocks=blocks)
                assert torch.equal(a, b), (m, waves, blocks)
            with pytest.raises(KernelError, match="waves must be"):
                ops.gemm_mfma_wide_swiglu(x, w, waves=5, blocks=2)
    # 65 to 128 rows (five to eight tiles of x, the eighth with LDS that the launch asks for): only on this copy and only where the launch shape has two
    # row blocks a wave and four waves or more, which the real gate/up and down shapes have; a row's sums
    # are those of the same row in a product of 64 rows
    for m in (65, 80, 112, 128):
        x = rnd((m, k), 77 + m, torch.bfloat16).cuda()
        splits = ops.gemm_mfma_wide_best_splits(m, n, k)
        takes = ops.gemm_mfma_wide_takes(m, f, splits)
        assert takes or (n, k) not in ((3584, 18944), (5120, 13824), (152064, 3584)), (m, splits)
        assert not takes or n >= 2048, (m, splits)  # (few rows of W leave no launch shape with two blocks a wave)
        assert not ops.gemm_mfma_wide_takes(m, w, splits) and not ops.gemm_mfma_wide_takes(129, f, splits)
        if takes:
            got = ops.gemm_mfma_wide(x, f, splits=splits)
            assert torch.equal(got[..., :64, :], ops.gemm_mfma_wide(x[:64].contiguous(), f, splits=splits))
            assert torch.equal(got[..., 64:, :], ops.gemm_mfma_wide(x[64:].contiguous(), f, splits=splits))
        else:
            with pytest.raises(KernelError, match="rows only on a fragment-ordered weight|at most 64 rows"):
                ops.gemm_mfma_wide(x, f, splits=splits)
        if n % 4 == 0:
            takes = ops.gemm_mfma_wide_takes(m, f, 1, gate_up=True)
            assert takes == (n >= 24577), m  # four waves of two blocks a workgroup, one workgroup a unit, from there on
            if takes:
                got = ops.gemm_mfma_wide_swiglu(x, f)
                assert torch.equal(got[:64], ops.gemm_mfma_wide_swiglu(x[:64].contiguous(), f))
                assert torch.equal(got[64:], ops.gemm_mfma_wide_swiglu(x[64:].contiguous(), f))
        with pytest.raises(KernelError, match="at most 64 rows"):
            ops.gemm_mfma_wide(x, w, splits=splits)
    x = rnd((64, k), 32 + 64, torch.bfloat16).cuda()
    if not big:
        full = (x.double() @ w.double().t()).float()  # 64 rows
        assert (ops.gemm_mfma_wide(x, f) - full).abs().max() <= tol(torch.float32, full.cpu()) * 4
    with pytest.raises(KernelError, match="multiple of 32"):
        ops.fragment_order(w[:, :k - 16].contiguous())
    with pytest.raises(KernelError, match="inner size"):
        ops.gemm_mfma_wide(x[:, :k // 2].contiguous(), f)


def test_refusals(ops):
    from from_scratch_inference_engine_amd.ops import KernelError

    x, w = torch.zeros(65, 64, dtype=torch.bfloat16).cuda(), torch.zeros(32, 64, dtype=torch.bfloat16).cuda()
    with pytest.raises(KernelError, match="at most 64 rows"):
        ops.gemm_mfma_skinny(x, w)
    with pytest.raises(KernelError, match="multiple of 8"):
        ops.gemm_mfma_skinny(x[:4, :60].contiguous(), w[:, :60].contiguous())
    with pytest.raises(KernelError, match="too short for 2 slices"):
        ops.gemm_mfma_skinny(x[:4], w, splits=2)
    with pytest.raises(KernelError, match="partial sums come in"):
        ops.gemm_mfma_skinny(x[:4], w, splits=3)
    with pytest.raises(KernelError, match="inner size"):
        ops.gemm(x, w[:, :32].contiguous())
    with pytest.raises(KernelError, match="contiguous"):
        ops.gemm(x[:, ::2], w[:, ::2])
    with pytest.raises(KernelError, match="GPU"):
        ops.swiglu(torch.zeros(2, 4))
    with pytest.raises(KernelError, match="float32 or bfloat16"):
        ops.swiglu(torch.zeros(2, 4, dtype=torch.float16).cuda())
    with pytest.raises(KernelError, match="head_dim"):
        q = torch.zeros(1, 3 * 300).cuda()
        ops.attention_scalar(q, 900, torch.zeros(1, 1, 4, 300).cuda(), torch.zeros(1, 1, 300, 4).cuda(),
                             torch.zeros(1, 1, dtype=torch.int32).cuda(), torch.zeros(1, 8, dtype=torch.int32).cuda(), 1,
                             torch.zeros(1, 300).cuda(), None, 1, 1, 300, None, 1.0, 1)


# ------------------------------------------------------------------------------ attention
def paged_case(seqs, heads, kv, hd, page, dtype, seed, window=None, shuffle=True, edit=None, scalar=False):
    """seqs: list of (past, n_new).  Returns device inputs for the kernel and per-seq q/k/v.
    ``edit(qs, ks, vs)`` may change the random tensors in place before the pages are filled."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner
    from from_scratch_inference_engine_amd import ops

    g = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-(p + n) // page) for p, n in seqs) + 3
    order = (torch.randperm(total_pages, generator=torch.Generator().manual_seed(seed + 1)).tolist()
             if shuffle else list(range(total_pages)))
    k_pool = torch.full((total_pages, kv, page, hd), 7.0)  # stale content in unused slots
    v_pool = torch.full((total_pages, kv, hd, page), -9.0)
    max_pages = max(-(-(p + n) // page) for p, n in seqs)
    tables = torch.full((len(seqs), max_pages), -1, dtype=torch.int32)
    qs, ks, vs = [], [], []
    for p, n in seqs:
        qs.append(torch.randn(n, heads * hd, generator=g).to(dtype).float())
        ks.append(torch.randn(p + n, kv * hd, generator=g).to(dtype).float())
        vs.append(torch.randn(p + n, kv * hd, generator=g).to(dtype).float())
    if edit is not None:
        edit(qs, ks, vs)
    for s, (p, n) in enumerate(seqs):
        total = p + n
        held = -(-total // page)
        for i in range(held):
            tables[s, i] = order.pop()
        mine = tables[s, :held].long()
        k_all = torch.full((held * page, kv, hd), 7.0)  # the tail of the last page keeps stale content
        v_all = torch.full((held * page, kv, hd), -9.0)
        k_all[:total], v_all[:total] = ks[s].reshape(total, kv, hd), vs[s].reshape(total, kv, hd)
        k_pool[mine] = k_all.reshape(held, page, kv, hd).permute(0, 2, 1, 3)
        v_pool[mine] = v_all.reshape(held, page, kv, hd).permute(0, 2, 3, 1)

    class Host:
        n_seqs = len(seqs)
        q_lens = [n for _, n in seqs]
        past_lens = [p for p, _ in seqs]
        q_starts = [0]
        page_size = page
        compute_dtype = torch.float32 if scalar else dtype  # scalar: the float32-arithmetic kernel on this storage
    for _, n in seqs:
        Host.q_starts.append(Host.q_starts[-1] + n)
    plan = AttentionPlanner(heads, kv, hd, window).plan(Host)
    return dict(q=torch.cat(qs).to(dtype), k_pool=k_pool.to(dtype), v_pool=v_pool.to(dtype), tables=tables, plan=plan,
                qs=qs, ks=ks, vs=vs)


def run_attention(ops, case, heads, kv, hd, window=None, share_keys=True):
    """``share_keys``: long portions go to the kernel that stages keys in LDS for four tiles,
    where it takes the geometry."""
    q = case["q"].cuda()
    t = q.shape[0]
    plan = case["plan"]
    out = torch.zeros((t, heads * hd), dtype=q.dtype).cuda()
    partials = torch.empty(max(plan["n_partial"], 1) * heads * (hd + 2), dtype=torch.float32).cuda()
    items = torch.from_numpy(plan["items"]).cuda()
    common = (out, partials, heads, kv, hd, window, 1.0 / math.sqrt(hd), t)
    pools = (case["k_pool"].cuda(), case["v_pool"].cuda(), case["tables"].cuda())
    if plan["mfma"]:
        if plan["n_small"]:
            ops.attention_mfma(q, heads * hd, *pools, items, plan["n_small"], *common, large=False, waves=plan["waves"])
        page = case["k_pool"].shape[2]
        if plan["n_large"] and not plan["n_long"] and share_keys and ops.attention_mfma_lds_ok(hd, page):
            ops.attention_mfma_lds(q, heads * hd, *pools, items[plan["n_small"]:],
                                   torch.from_numpy(plan["groups"]).cuda(), plan["n_groups"], out, heads, kv, hd,
                                   window, 1.0 / math.sqrt(hd), t)
        elif plan["n_large"]:
            ops.attention_mfma(q, heads * hd, *pools, items[plan["n_small"]:], plan["n_large"], *common, large=True)
        if plan["n_long"]:
            ops.attention_mfma(q, heads * hd, *pools, items[plan["n_small"] + plan["n_large"]:], plan["n_long"], *common,
                               large=True, waves=4)
    else:
        ops.attention_scalar(q, heads * hd, *pools, items, plan["n_small"] + plan["n_large"], *common)
    if plan["n_merges"]:
        ops.attention_merge(partials, torch.from_numpy(plan["merges"]).cuda(), plan["n_merges"], out, heads, hd)
    return out.float().cpu()


@pytest.mark.parametrize("dtype, scalar", [(torch.float32, True), (torch.bfloat16, True), (torch.bfloat16, False)])
@pytest.mark.parametrize("heads, kv, hd, page, window", [
    (14, 2, 64, 16, None),   # the reference's kernel test sizes (tests/cpp/test_cuda_kernels.cpp:126-164)
    (4, 4, 48, 4, None),     # plain multi-head, head size no power of two
    (20, 1, 32, 8, None),    # more heads per kv head than rows of a block
    (6, 2, 128, 16, 37),     # a window
    (3, 1, 256, 64, None),
    (28, 4, 128, 16, None),  # a large model's geometry: 7 heads per kv head
    (2, 1, 80, 12, 300),     # head size an odd multiple of 16, page size no power of two
    (6, 3, 64, 16, None),    # three kv heads: they do not divide the device's eight dies
    (40, 8, 128, 16, None),  # the 14B and 32B geometry: 5 heads per kv head, one kv head a die
    (5, 1, 128, 32, 200),    # head size 128 with a page size other than 16, and a window
])
def test_attention_over_pages(ops, dtype, scalar, heads, kv, hd, page, window):
    # (past, new): the reference's (7, 5) and (19, 1), a long decode that is split, whole prompts,
    # portions starting mid-page, a two-token portion
    seqs = [(7, 5), (19, 1), (600, 1), (0, 33), (300, 2), (123, 70), (0, 1), (40, 200), (2500, 1), (900, 130)]
    case = paged_case(seqs, heads, kv, hd, page, dtype, seed=hd + heads, window=window, scalar=scalar)
    assert case["plan"]["mfma"] == (not scalar)
    out = run_attention(ops, case, heads, kv, hd, window)
    row = 0
    for (p, n), q, k, v in zip(seqs, case["qs"], case["ks"], case["vs"]):
        ref = plain.attention(q, k, v, heads, kv, hd, query_offset=p, window=window)
        err = (out[row:row + n] - ref).abs().max().item()
        assert err <= (2e-6 if dtype == torch.float32 else 2.0 ** -7 * ref.abs().max().item()), f"seq past {p} new {n}: {err}"
        row += n
    if not scalar and ops.attention_mfma_lds_ok(hd, page) and case["plan"]["n_large"]:
        # the long portions went through the kernel that shares keys in LDS; the one-wave kernel
        # must give the same up to the rounding of the probabilities
        assert 0 < case["plan"]["n_groups"] < case["plan"]["n_large"]
        alone = run_attention(ops, case, heads, kv, hd, window, share_keys=False)
        assert (alone - out).abs().max() <= 2.0 ** -7 * out.abs().max()


@pytest.mark.parametrize("heads, kv, seqs", [
    (28, 4, [(0, 4096)]),                # a whole long prompt: 32 groups of four tiles a kv head on the die-mapped grid
    (28, 4, [(4096, 2048), (17000, 1)]),  # a portion behind thousands of cached keys; a decode of 67 splits and their merge
    (40, 8, [(0, 4096)]),
    (40, 8, [(4096, 2048), (12000, 1)]),
])
def test_attention_over_pages_at_the_lengths_that_are_timed(ops, heads, kv, seqs):
    """The prompt and context lengths that the measurements quote, at the head geometries of the
    large models (head size 128, page 16, bfloat16), against the plain attention."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    hd, page = 128, 16
    AttentionPlanner.compute_units = 4096  # as on a device with so many idle units: the decode is cut into items of 128 keys
    try:
        case = paged_case(seqs, heads, kv, hd, page, torch.bfloat16, seed=heads)
    finally:
        AttentionPlanner.compute_units = None
    plan = case["plan"]
    assert plan["mfma"] and (plan["n_groups"] > 100 or plan["n_merges"])
    out = run_attention(ops, case, heads, kv, hd)
    row = 0
    for (p, n), q, k, v in zip(seqs, case["qs"], case["ks"], case["vs"]):
        ref = plain.attention(q, k, v, heads, kv, hd, query_offset=p)
        err = (out[row:row + n] - ref).abs().max().item()
        assert err <= 2.0 ** -7 * ref.abs().max().item(), f"seq past {p} new {n}: {err}"
        row += n
    if len(seqs) > 1:
        assert max(m[2] for m in plan["merges"]) > (64 if heads == 28 else 40)  # splits of the long decode


@pytest.mark.parametrize("units", [4096, 8])  # items of 128 keys, one wave each, and a merge; whole requests, up to 8 waves
@pytest.mark.parametrize("heads, kv, hd, page, window, n_parts, bias", [
    (28, 4, 128, 16, None, 8, True),   # a large model's geometry
    (40, 8, 128, 16, None, 4, True),
    (12, 4, 128, 16, None, 11, True),  # more slices than the kernel reads at once
    (14, 2, 64, 8, None, 3, True),
    (20, 1, 32, 8, None, 1, False),    # more heads per kv head than rows of a block: two workgroups a kv head, one of them writes
    (6, 3, 96, 24, None, 2, True),     # head size and page size no powers of two
    (3, 1, 256, 64, None, 5, False),
    (6, 2, 128, 16, 37, 7, True),      # a window
])
def test_attention_from_the_projections_partial_sums(ops, units, heads, kv, hd, page, window, n_parts, bias):
    """A step of one token a request: the kernel that takes q/k/v as the partial sums of a product cut
    along K (adds them up, adds the bias, rotates, scores the new key from registers, writes it and the
    value into the pools) against the kernels that do these one after the other.  Positions at the
    edges of pages, of the blocks of 32 keys and of the items of 128."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    pasts = [0, 19, 31, 32, 600, 127, 128, 2500, 1023, 1024, 7, 255]
    seqs = [(p, 1) for p in pasts]
    t, width = len(seqs), (heads + 2 * kv) * hd
    AttentionPlanner.compute_units = units
    try:
        case = paged_case(seqs, heads, kv, hd, page, torch.bfloat16, seed=heads + hd, window=window)
    finally:
        AttentionPlanner.compute_units = None
    plan = case["plan"]
    assert plan["mfma"] and plan["single"] and not plan["n_large"]
    if window is None:
        assert plan["n_merges"] > 0 if units == 4096 else plan["waves"] > 1
    g = torch.Generator().manual_seed(5)
    parts = torch.randn(n_parts, t, width, generator=g).cuda()
    b = torch.randn(width, generator=g).cuda() if bias else None
    positions = torch.tensor(pasts, dtype=torch.int32).cuda()
    inv_freq = torch.pow(torch.tensor(1e4, dtype=torch.float64), -torch.arange(0, hd, 2, dtype=torch.float64) / hd).cuda()
    table = ops.rope_table(positions, inv_freq)
    tables = case["tables"]
    slots = torch.tensor([int(tables[s, p // page]) * page + p % page for s, p in enumerate(pasts)], dtype=torch.int32).cuda()
    items = torch.from_numpy(plan["items"]).cuda()
    merges = torch.from_numpy(plan["merges"]).cuda()
    scale = 1.0 / math.sqrt(hd)

    def pools():
        return case["k_pool"].cuda().clone(), case["v_pool"].cuda().clone(), tables.cuda()

    # one after the other: the sums added and rotated into q and the pools, then attention over the pools
    k1, v1, bt = pools()
    qkv = torch.empty(t, width, dtype=torch.bfloat16).cuda()
    ops.rope_kv_write(qkv, positions, heads, kv, hd, inv_freq, slots=slots, k_pool=k1, v_pool=v1, page_size=page, bias=b,
                      cos_sin=table, parts=parts)
    out1 = torch.zeros(t, heads * hd, dtype=torch.bfloat16).cuda()
    partials1 = torch.zeros(max(plan["n_partial"], 1) * heads * (hd + 2)).cuda()
    ops.attention_mfma(qkv, width, k1, v1, bt, items, plan["n_small"], out1, partials1, heads, kv, hd, window, scale, t,
                       large=False, waves=plan["waves"])
    # in one kernel
    k2, v2, bt = pools()
    out2 = torch.zeros(t, heads * hd, dtype=torch.bfloat16).cuda()
    partials2 = torch.zeros_like(partials1)
    assert ops.attention_mfma_qkv_ok(hd, page)
    ops.attention_mfma_qkv(parts, b, table, slots, k2, v2, bt, items, plan["n_small"], out2, partials2, heads, kv, hd,
                           window, scale, waves=plan["waves"])
    if plan["n_merges"]:
        ops.attention_merge(partials1, merges, plan["n_merges"], out1, heads, hd)
        ops.attention_merge(partials2, merges, plan["n_merges"], out2, heads, hd)
    torch.cuda.synchronize()
    # the pools: the new keys and values are there (the rotation's roundings may differ in the last
    # bit), and nothing else has changed
    for new, old, start in ((k2, k1, case["k_pool"].cuda()), (v2, v1, case["v_pool"].cuda())):
        assert (old != start).sum() >= t * kv * hd * 0.9
        assert (new.float() - old.float()).abs().max() <= 2.0 ** -7 * old.float().abs().max()
        assert torch.equal(new != start, old != start) or ((new != start) ^ (old != start)).sum() <= 4  # (a value that rounds to the stale one)
    ref, got = out1.float(), out2.float()
    assert ref.abs().max() > 0.1
    for row in range(t):
        err = (got[row] - ref[row]).abs().max().item()
        assert err <= 2.0 ** -6 * ref[row].abs().max().item(), f"request of {pasts[row]} past keys: {err}"
    with pytest.raises(ops.KernelError, match="multiple of 32"):
        ops.attention_mfma_qkv(torch.zeros(1, 1, 3 * 48).cuda(), None, torch.zeros(1, 24, 2).cuda(), slots[:1],
                               torch.zeros(2, 1, 8, 48, dtype=torch.bfloat16).cuda(),
                               torch.zeros(2, 1, 48, 8, dtype=torch.bfloat16).cuda(), bt[:1], items, 1,
                               torch.zeros(1, 48, dtype=torch.bfloat16).cuda(), None, 1, 1, 48, None, 1.0)


@pytest.mark.parametrize("dtype, scalar", [(torch.float32, True), (torch.bfloat16, False)])
def test_attention_finds_one_far_key_and_respects_edges(ops, dtype, scalar):
    """Inputs that random data would hide a fault behind: for every query one key far back (or
    at the far edge of its window) carries nearly the whole softmax, so the output must be that
    key's value; and louder keys sit where the query must not look: right after its own
    position and right before its window."""
    heads, kv, hd, page = 4, 2, 32, 8
    group = heads // kv
    for window in (None, 100):
        seqs = [(700, 1), (350, 3)]
        chosen = {}

        def edit(qs, ks, vs):
            for s, (p, n) in enumerate(seqs):
                for i in range(n):
                    pos = p + i
                    far = pos - window + 1 if window else 3 + 8 * i   # the window's first key / hundreds back
                    chosen[(s, i)] = far
                    q = qs[s][i].reshape(heads, hd)
                    for kvh in range(kv):
                        # the heads of one group share the key: point all of them at it
                        q[kvh * group:(kvh + 1) * group] = q[kvh * group] * 1.0
                        u = q[kvh * group] / q[kvh * group].norm()
                        ks[s][far].reshape(kv, hd)[kvh] = (40.0 * u).to(dtype).float()
                        q[kvh * group:(kvh + 1) * group] = (8.0 * u).to(dtype).float()
                        loud = (400.0 * u).to(dtype).float()
                        if pos + 1 < p + n:
                            ks[s][pos + 1].reshape(kv, hd)[kvh] = loud       # the future
                        if window and pos - window >= 0 and pos - window not in chosen.values():
                            ks[s][pos - window].reshape(kv, hd)[kvh] = loud  # just outside the window

        case = paged_case(seqs, heads, kv, hd, page, dtype, seed=3, window=window, edit=edit, scalar=scalar)
        out = run_attention(ops, case, heads, kv, hd, window)
        row = 0
        for s, ((p, n), q, k, v) in enumerate(zip(seqs, case["qs"], case["ks"], case["vs"])):
            ref = plain.attention(q, k, v, heads, kv, hd, query_offset=p, window=window)
            assert (out[row:row + n] - ref).abs().max() <= (5e-6 if dtype == torch.float32 else 2.0 ** -7 * ref.abs().max())
            for i in range(n):  # and the plain result is what the construction says: the far key's value
                want = v[chosen[(s, i)]].reshape(kv, 1, hd).expand(kv, group, hd).reshape(-1)
                if i == 0:
                    assert (ref[i] - want).abs().max() < 1e-3
            row += n


@pytest.mark.parametrize("heads, hd, dtype", [(3, 32, torch.float32), (5, 80, torch.bfloat16), (28, 128, torch.bfloat16),
                                             (2, 256, torch.float32)])
def test_attention_merge_alone(ops, heads, hd, dtype):
    """Records of 1 to 257 splits (up to 32 are one wave's work, more are dealt to four waves in runs,
    a run of more than 64 takes a wave two passes), some of them empty (maximum -inf), one token's
    records a stride apart, against the sums written out."""
    g = torch.Generator().manual_seed(hd)
    splits = [1, 2, 3, 9, 32, 33, 64, 65, 130, 257]
    stride = 2  # two tokens of a portion lie side by side in every split
    slots = sum(n * stride for n in splits)
    rec = torch.randn(slots, heads, hd + 2, generator=g)
    rec[:, :, hd] = 3.0 * torch.randn(slots, heads, generator=g)       # maxima, natural units
    rec[:, :, hd + 1] = torch.rand(slots, heads, generator=g) + 0.1    # denominators
    merges, want, first = [], [], 0
    for row, n in enumerate(splits):
        for t in range(stride):
            idx = [first + t + i * stride for i in range(n)]
            if n >= 3:  # an empty split in the middle: a window that has passed it
                rec[idx[1], :, hd] = float("-inf")
                rec[idx[1], :, hd + 1] = 0.0
            r = rec[idx].double()
            w = torch.exp(r[:, :, hd] - r[:, :, hd].max(0).values)
            want.append(((r[:, :, :hd] * w[:, :, None]).sum(0) / (r[:, :, hd + 1] * w).sum(0)[:, None]).reshape(-1))
            merges.append((row * stride + t, first + t, n, stride))
        first += n * stride
    out = torch.zeros(len(merges), heads * hd, dtype=dtype).cuda()
    ops.attention_merge(rec.reshape(-1).cuda(), torch.tensor(merges, dtype=torch.int32).cuda(), len(merges), out, heads, hd)
    want = torch.stack(want).float()
    err = (out.float().cpu() - want).abs().max().item()
    assert err <= (2e-5 if dtype == torch.float32 else 2.0 ** -8) * want.abs().max().item(), err


def test_attention_long_tiles_on_four_waves(ops, monkeypatch):
    """Large tiles may be given four waves that split the keys and merge in the workgroup."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    monkeypatch.setattr(AttentionPlanner, "long_keys", 96)
    heads, kv, hd, page = 8, 2, 64, 8
    seqs = [(500, 70), (0, 300), (37, 3)]
    case = paged_case(seqs, heads, kv, hd, page, torch.bfloat16, seed=9)
    assert case["plan"]["n_long"] > 0 and case["plan"]["n_large"] > 0
    out = run_attention(ops, case, heads, kv, hd)
    row = 0
    for (p, n), q, k, v in zip(seqs, case["qs"], case["ks"], case["vs"]):
        ref = plain.attention(q, k, v, heads, kv, hd, query_offset=p)
        assert (out[row:row + n] - ref).abs().max() <= 2.0 ** -7 * ref.abs().max()
        row += n


def test_attention_does_not_depend_on_page_ids(ops):
    heads, kv, hd, page = 8, 2, 64, 16
    seqs = [(100, 1), (0, 40)]
    for dtype in DTYPES:
        a = run_attention(ops, paged_case(seqs, heads, kv, hd, page, dtype, 5, shuffle=True), heads, kv, hd)
        b = run_attention(ops, paged_case(seqs, heads, kv, hd, page, dtype, 5, shuffle=False), heads, kv, hd)
        assert torch.equal(a, b)


# ------------------------------------------------------------------------------ sampling
def test_argmax_ties_and_large_vocab(ops):
    # tests/cpp/test_cuda_kernels.cpp:201-235: V = 151936 rows equal a host scan; ties -> smallest index
    logits = rnd((5, 151936), 20)
    logits[1, 77] = logits[1, 140000] = 50.0
    logits[2, 151935] = 60.0
    logits[3, 0] = 60.0
    out = ops.sample(logits.cuda()).cpu().tolist()
    assert out == [plain.argmax(r) for r in logits] and out[1] == 77 and out[2] == 151935 and out[3] == 0
    small = torch.tensor([[0.0, 1.0, 5.0, 1.0, 0.0, 5.0]])
    assert ops.sample(small.cuda()).item() == 2


@pytest.mark.parametrize("vocab", [509, 151936])
def test_sampling_matches_plain_given_u(ops, vocab):
    g = torch.Generator().manual_seed(21)
    rows = []
    for temp, k, p in [(0.7, 0, 1.0), (1.0, 0, 1.0), (0.3, 5, 1.0), (1.5, 50, 0.9), (1.0, 0, 0.5), (2.0, 1, 1.0),
                       (0.0, 0, 1.0), (0.9, 3, 0.2)]:
        for u in (0.0, 0.013, 0.37, 0.5, 0.81, 0.999):
            rows.append((temp, k, p, u))
    logits = torch.randn(len(rows), vocab, generator=g) * 2.0
    logits[3, 10] = logits[3, 11] = logits[3].max() + 1.0  # a tie at the top
    dev = lambda v, dt: torch.tensor(v, dtype=dt).cuda()
    out = ops.sample(logits.cuda(), dev([r[0] for r in rows], torch.float32), dev([r[1] for r in rows], torch.int32),
                     dev([r[2] for r in rows], torch.float32), dev([r[3] for r in rows], torch.float64)).cpu().tolist()
    bad = []
    for i, (temp, k, p, u) in enumerate(rows):
        want = plain.sample(logits[i], temp, k, p, u)
        if out[i] != want:
            # tolerate a draw that sits on a boundary of the cumulative sum within float rounding
            alt = {plain.sample(logits[i], temp, k, p, min(max(u + d, 0.0), 0.999999)) for d in (-1e-6, 1e-6)}
            if out[i] not in alt:
                bad.append((i, rows[i], out[i], want))
    assert not bad, bad


def test_sampling_distribution(ops):
    # tests/cpp/test_sampler.cpp:44-56: logits {0, 2, 0} pick index 1 with probability 0.787
    n = 4000
    logits = torch.tensor([[0.0, 2.0, 0.0]]).repeat(n, 1).cuda()
    u = ((torch.arange(n, dtype=torch.float64) + 0.5) / n).cuda()
    ones = torch.ones(n, dtype=torch.float32).cuda()
    out = ops.sample(logits, ones, torch.zeros(n, dtype=torch.int32).cuda(), ones, u).cpu()
    assert abs((out == 1).float().mean().item() - 0.7869) < 0.002
    assert (out[:400] == 0).all() and (out[-400:] == 2).all()  # vocabulary order of the draw


def test_random_weights_are_the_same_bits_on_the_device_and_on_the_host(ops):
    """The random-weights mode: the kernel and the host code of the counter-based generator agree
    bit for bit (weights, norm weights, integer tables; float32 and rounded to bfloat16), so a
    model made on the device is the model that the written folder holds."""
    from from_scratch_inference_engine_amd.weights import random_init as r
    from from_scratch_inference_engine_amd.weights.loader import TensorSpec

    for name, shape, init in [("model.embed_tokens.weight", (509, 192), "weight"), ("model.norm.weight", (3584,), "norm"),
                              ("a.bias", (7,), "bias"), ("ids", (33, 5), "int"), ("big", (1 << 21,), "weight")]:
        spec = TensorSpec(name, shape, init)
        for dtype in (torch.float32, torch.bfloat16):
            host = r.random_tensor(spec, 41, dtype, "cpu")
            dev = r.random_tensor(spec, 41, dtype, "cuda:0")
            assert dev.is_cuda and dev.dtype == host.dtype and torch.equal(dev.cpu(), host), (name, dtype)


@pytest.mark.parametrize("m, n, k", [(1, 4864, 896), (5, 151, 100), (8, 1000, 4864), (17, 3584, 18944), (37, 300, 132),
                                     (64, 896, 1000), (64, 37888, 3584), (3, 16, 4)])
def test_gemm_mfma_fp32(ops, m, n, k):
    """True float32 on the matrix cores: against the float64 product of the same float32 values
    (no reduced-precision mode would pass 2e-6), with and without bias; a row's sums do not depend
    on the other rows; whatever the number of waves that split K."""
    x, w, b = rnd((m, k), 70), rnd((n, k), 71, scale=0.05), rnd((n,), 72)
    ref = (x.cuda().double() @ w.cuda().double().t()).cpu()
    out = ops.gemm_mfma_fp32(x.cuda(), w.cuda(), b.cuda()).cpu()
    assert (out.double() - (ref + b.double())).abs().max() <= 2e-6 * max(1.0, ref.abs().max().item())
    plain_out = ops.gemm_mfma_fp32(x.cuda(), w.cuda()).cpu()
    assert (plain_out.double() - ref).abs().max() <= 2e-6 * max(1.0, ref.abs().max().item())
    if m > 2:
        fewer = ops.gemm_mfma_fp32(x[1:m - 1].contiguous().cuda(), w.cuda()).cpu()
        assert torch.equal(fewer, plain_out[1:m - 1])
    for waves in (1, 2, 8):
        other = ops.gemm_mfma_fp32(x.cuda(), w.cuda(), waves=waves).cpu()
        assert (other.double() - ref).abs().max() <= 2e-6 * max(1.0, ref.abs().max().item())
    with pytest.raises(ops.KernelError, match="multiple of 4"):
        ops.gemm_mfma_fp32(torch.zeros(2, 6).cuda(), torch.zeros(3, 6).cuda())
    with pytest.raises(ops.KernelError, match="at most 64 rows"):
        ops.gemm_mfma_fp32(torch.zeros(65, 8).cuda(), torch.zeros(3, 8).cuda())
