"""Each HIP kernel alone against a plain 32-bit reference of the same operation, at sizes other
than the tiny models': ragged widths, head sizes in steps of 16, every group ratio, odd
vocabularies, any page size."""

import math

import pytest
import torch

import plain_llama
from kernel_helpers import attention_reference, make_paged

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def ops():
    from llmserve.ops import library

    return library


def rnd(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def ulp(dtype, ref):
    """One rounding of the largest value for bfloat16; accumulated 32-bit rounding otherwise."""
    scale = max(1e-3, float(ref.abs().max()))
    return scale * (2.0 ** -7 if dtype == torch.bfloat16 else 2e-6)


# ------------------------------------------------------------------ row-wise kernels
@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_gather(dtype):
    table = rnd(333, 100, seed=1).to(dtype)
    ids = torch.tensor([0, 332, 7, 7, 100], dtype=torch.int32)
    out = torch.empty(5, 100, dtype=dtype, device=DEV)
    ops().embed_gather(out, table.to(DEV), ids.to(DEV))
    assert torch.equal(out.cpu(), table[ids.long()])
    bad = torch.tensor([5, 333, -1], dtype=torch.int32)
    out = torch.zeros(3, 100, dtype=dtype, device=DEV)
    ops().embed_gather(out, table.to(DEV), bad.to(DEV))
    assert torch.equal(out[0].cpu(), table[5]) and out[1:].isnan().all()  # a bad id is loud, not a stray read


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,eps", [(64, 1e-5), (100, 1e-6), (2048, 1e-5), (5000, 1e-6)])
def test_rmsnorm(dtype, hidden, eps):
    x = rnd(9, hidden, seed=2, scale=3.0).to(dtype)
    delta = rnd(9, hidden, seed=3).to(dtype)
    w = (1 + 0.1 * rnd(hidden, seed=4)).to(dtype)
    ref = plain_llama.rms_norm(x, w, eps).float()
    out = ops().rmsnorm(torch.empty_like(x, device=DEV), x.to(DEV), w.to(DEV), eps)
    assert (out.float().cpu() - ref).abs().max() <= ulp(dtype, ref)
    # residual sum in 32-bit, rounded once, written back, then normed
    summed = (x.float() + delta.float()).to(dtype)
    ref = plain_llama.rms_norm(summed, w, eps).float()
    resid = x.clone().to(DEV)
    out = ops().rmsnorm(torch.empty_like(resid), resid, w.to(DEV), eps, delta=delta.to(DEV), resid_out=resid)
    assert torch.equal(resid.cpu(), summed)
    assert (out.float().cpu() - ref).abs().max() <= ulp(dtype, ref)
    # only some rows, nothing written back
    rows = torch.tensor([8, 0, 3], dtype=torch.int32)
    resid = x.clone().to(DEV)
    out = torch.empty(3, hidden, dtype=dtype, device=DEV)
    ops().rmsnorm(out, resid, w.to(DEV), eps, delta=delta.to(DEV), rows=rows.to(DEV))
    assert (out.float().cpu() - ref[rows.long()]).abs().max() <= ulp(dtype, ref)
    assert torch.equal(resid.cpu(), x)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,parts", [(64, 2), (96, 3), (2048, 2), (333, 4), (5000, 2)])
def test_rmsnorm_takes_the_delta_as_partial_sums(dtype, hidden, parts):
    """The delta as 32-bit partial sums of a product whose K was split: the same bits as the delta they add
    up to, rounded to the model's dtype, would give."""
    x = rnd(9, hidden, seed=2, scale=3.0).to(dtype)
    p = rnd(parts * 9, hidden, seed=3).view(parts, 9, hidden)
    total = torch.zeros(9, hidden)
    for i in range(parts):
        total += p[i]  # the kernel adds in this order
    delta = total.to(dtype)
    w = (1 + 0.1 * rnd(hidden, seed=4)).to(dtype)
    want_resid = x.clone().to(DEV)
    want = ops().rmsnorm(torch.empty_like(want_resid), want_resid, w.to(DEV), 1e-5, delta=delta.to(DEV), resid_out=want_resid)
    resid = x.clone().to(DEV)
    got = ops().rmsnorm(torch.empty_like(resid), resid, w.to(DEV), 1e-5, delta=p.to(DEV), resid_out=resid)
    assert torch.equal(resid, want_resid) and torch.equal(got, want)
    rows = torch.tensor([8, 0, 3], dtype=torch.int32, device=DEV)
    got = ops().rmsnorm(torch.empty(3, hidden, dtype=dtype, device=DEV), x.to(DEV), w.to(DEV), 1e-5, delta=p.to(DEV), rows=rows)
    assert torch.equal(got, want[rows.long()])
    with pytest.raises(ValueError, match="partial sums"):
        ops().rmsnorm(torch.empty_like(resid), resid, w.to(DEV), 1e-5, delta=p[:, :8].contiguous().to(DEV))


def test_rmsnorm_tiny_inputs_feel_eps():
    x = rnd(2, 96, seed=5, scale=1e-3)
    w = torch.ones(96)
    for eps in (1e-5, 1e-6):
        out = ops().rmsnorm(torch.empty(2, 96, device=DEV), x.to(DEV), w.to(DEV), eps)
        assert torch.allclose(out.cpu(), plain_llama.rms_norm(x, w, eps), atol=1e-6)


@pytest.mark.parametrize("nh,nkv,d,bs", [(4, 2, 16, 16), (8, 8, 64, 8), (16, 2, 128, 32), (6, 3, 48, 24), (4, 4, 32, 4),
                                         (2, 20, 16, 16), (20, 20, 32, 64)])
def test_rope_store_prompt_tokens_side_by_side(nh, nkv, d, bs):
    """A prompt's tokens lie side by side in their pages: 16 of them (8 where the page size is no multiple of 16) whose
    first slot is a multiple of that are a run, whose workgroups share the KV heads out (fewer heads than tokens,
    and more) and store 16 bytes per dimension.  Runs that start off such a boundary (in the page, and in the batch),
    break in the middle (another page, a token without a slot), or end early, and a second request behind the first,
    leave as single values: every slot must hold its own token's values and nothing else may change."""
    dtype = torch.bfloat16
    pages = 16
    # request a: 29 tokens from slot 3 of page 2 on through pages 5 and 1 (pages need not follow each other)
    # request b: 16 tokens from the start of page 7, the 12th without a slot; then 5 scattered single tokens
    def run(page_list, first, count):
        out, page_i, off = [], 0, first
        for _ in range(count):
            out.append(page_list[page_i] * bs + off)
            off += 1
            if off == bs:
                page_i, off = page_i + 1, 0
        return out
    slots = run([2, 5, 1, 9, 10, 11, 0, 4], 3, 29) + run([7, 3, 6, 8], 0, 16)  # (12 of the 16 pages at most)
    slots[29 + 11] = -1
    free = sorted(set(range(pages * bs)) - set(slots))
    assert len(free) >= 8
    slots += [free[0], free[-1], free[len(free) // 2], -1, free[1]]
    n = len(slots)
    width = (nh + 2 * nkv) * d
    qkv = rnd(n, width, seed=16).to(dtype)
    positions = torch.arange(n, dtype=torch.int32)
    inv_freq = 1.0 / (1e4 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    k_pool = torch.full((pages, nkv, bs, d), 7.0, dtype=dtype, device=DEV)
    v_pool = torch.full((pages, nkv, d, bs), 7.0, dtype=dtype, device=DEV)
    dev_qkv = qkv.clone().to(DEV)
    ops().rope_store(dev_qkv, inv_freq.to(DEV), positions.to(DEV), torch.tensor(slots, dtype=torch.int32, device=DEV),
                     k_pool, v_pool, nh, nkv, d, bs)
    v = qkv[:, (nh + nkv) * d:].view(n, nkv, d)
    vp = v_pool.cpu()
    written = torch.zeros(pages, bs, dtype=torch.bool)
    for i, sl in enumerate(slots):
        if sl < 0:
            continue
        page, off = divmod(sl, bs)
        written[page, off] = True
        assert torch.equal(vp[page, :, :, off], v[i]), f"token {i} (slot {sl})"
    assert (vp.permute(0, 3, 1, 2)[~written] == 7).all()
    assert torch.equal(dev_qkv.cpu()[:, (nh + nkv) * d:], qkv[:, (nh + nkv) * d:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,bs,theta", [(4, 2, 16, 16, 1e4), (3, 1, 32, 8, 5e5), (8, 8, 64, 4, 1e4),
                                               (5, 5, 48, 1, 1e6), (16, 2, 128, 32, 1e4)])
def test_rope_store(dtype, nh, nkv, d, bs, theta):
    n = 7
    width = (nh + 2 * nkv) * d
    qkv = rnd(n, width, seed=6).to(dtype)
    positions = torch.tensor([0, 1, 2, 500, 1999, 37, 4095], dtype=torch.int32)
    pages = 6
    others = [s for s in torch.randperm(bs * pages, generator=torch.Generator().manual_seed(d)).tolist()
              if s not in (0, bs * pages - 1)]
    slots = torch.tensor([others[0], 0, bs * pages - 1, -1, others[1], others[2], others[3]], dtype=torch.int32)
    inv_freq = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    k_pool = torch.full((pages, nkv, bs, d), 7.0, dtype=dtype, device=DEV)
    v_pool = torch.full((pages, nkv, d, bs), 7.0, dtype=dtype, device=DEV)
    dev_qkv = qkv.clone().to(DEV)
    ops().rope_store(dev_qkv, inv_freq.to(DEV), positions.to(DEV), slots.to(DEV), k_pool, v_pool, nh, nkv, d, bs)
    got = dev_qkv.cpu()
    cos, sin = plain_llama.rope_cos_sin(positions, d, theta)
    q = qkv[:, : nh * d].view(n, nh, d).transpose(0, 1)
    k = qkv[:, nh * d: (nh + nkv) * d].view(n, nkv, d).transpose(0, 1)
    v = qkv[:, (nh + nkv) * d:].view(n, nkv, d)
    q_ref = plain_llama.apply_rope(q, cos, sin).transpose(0, 1).reshape(n, nh * d)
    k_ref = plain_llama.apply_rope(k, cos, sin).transpose(0, 1)  # [n, nkv, d]
    tol = ulp(dtype, q_ref.float()) if dtype == torch.bfloat16 else 2e-4 * float(q_ref.abs().max())  # sin/cos of large angles
    assert (got[:, : nh * d].float() - q_ref.float()).abs().max() <= tol
    assert torch.equal(got[:, (nh + nkv) * d:], qkv[:, (nh + nkv) * d:])  # v is left alone
    kp, vp = k_pool.cpu(), v_pool.cpu()
    written = torch.zeros(pages, bs, dtype=torch.bool)
    for i, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        page, off = divmod(s, bs)
        written[page, off] = True
        assert (kp[page, :, off].float() - k_ref[i].float()).abs().max() <= tol
        assert torch.equal(vp[page, :, :, off], v[i])
    assert (kp.transpose(1, 2)[~written] == 7).all() and (vp.permute(0, 3, 1, 2)[~written] == 7).all()
    # without frequencies nothing is rotated, keys are stored as they are
    dev_qkv = qkv.clone().to(DEV)
    ops().rope_store(dev_qkv, None, positions.to(DEV), slots.to(DEV), k_pool, v_pool, nh, nkv, d, bs)
    assert torch.equal(dev_qkv.cpu(), qkv)
    page, off = divmod(int(slots[0]), bs)
    assert torch.equal(k_pool.cpu()[page, :, off], k.transpose(0, 1)[0])



@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [176, 5632, 33])
def test_silu_mul(dtype, inter):
    gu = rnd(5, 2 * inter, seed=7, scale=4.0).to(dtype)
    ref = (plain_llama.silu(gu[:, :inter]) * gu[:, inter:]).float()
    out = ops().silu_mul(torch.empty(5, inter, dtype=dtype, device=DEV), gu.to(DEV))
    assert (out.float().cpu() - ref).abs().max() <= ulp(dtype, ref)


# ------------------------------------------------------------------ matrix products
@pytest.mark.parametrize("m,n,k", [(1, 256, 64), (5, 333, 96), (64, 100, 176), (130, 65, 17), (300, 513, 1000)])
def test_gemm_fma(m, n, k):
    a, w, b = rnd(m, k, seed=8), rnd(n, k, seed=9), rnd(n, seed=10)
    ref = a.double() @ w.double().t() + b.double()
    out = ops().gemm_fma(torch.empty(m, n, device=DEV), a.to(DEV), w.to(DEV), b.to(DEV))
    assert (out.cpu().double() - ref).abs().max() <= 2e-6 * math.sqrt(k) * float(ref.abs().max())
    ab, wb = a.bfloat16(), w.bfloat16()
    ref = ab.double() @ wb.double().t()
    out = ops().gemm_fma(torch.empty(m, n, device=DEV), ab.to(DEV), wb.to(DEV))  # bfloat16 in, 32-bit out
    assert (out.cpu().double() - ref).abs().max() <= 2e-6 * math.sqrt(k) * float(ref.abs().max())
    out = ops().gemm_fma(torch.empty(m, n, dtype=torch.bfloat16, device=DEV), ab.to(DEV), wb.to(DEV))
    assert (out.float().cpu().double() - ref).abs().max() <= 2.0 ** -8 * float(ref.abs().max())


@pytest.mark.parametrize("kernel,m", [("skinny", 1), ("skinny", 7), ("skinny", 16), ("skinny", 17), ("skinny", 33),
                                      ("skinny", 64), ("tile", 5), ("tile", 65), ("tile", 128), ("tile", 300)])
@pytest.mark.parametrize("n,k", [(16, 64), (333, 96), (100, 176), (2056, 2048), (512, 5632)])
def test_gemm_bf16(kernel, m, n, k):
    a, w, b = rnd(m, k, seed=11).bfloat16(), rnd(n, k, seed=12).bfloat16(), rnd(n, seed=13).bfloat16()
    ref = a.double() @ w.double().t() + b.double()
    out = ops().gemm_bf16(torch.empty(m, n, device=DEV), a.to(DEV), w.to(DEV), b.to(DEV), kernel=kernel)
    assert (out.cpu().double() - ref).abs().max() <= 2e-6 * math.sqrt(k) * float(ref.abs().max())
    out = ops().gemm_bf16(torch.empty(m, n, dtype=torch.bfloat16, device=DEV), a.to(DEV), w.to(DEV), kernel=kernel)
    ref = a.double() @ w.double().t()
    assert (out.float().cpu().double() - ref).abs().max() <= 2.0 ** -8 * float(ref.abs().max())


@pytest.mark.parametrize("m,n,k", [(1, 16, 64), (3, 333, 96), (16, 2056, 2048), (7, 100, 5632), (9, 48, 176),
                                   (17, 333, 96), (64, 2056, 2048), (40, 100, 5632), (33, 48, 176),
                                   (8, 1040, 8192), (3, 64, 28672)])  # (the last two: K of the Llama-2-70B layer)
def test_gemm_stream_plain(m, n, k):
    x, w, b = rnd(m, k, seed=11).bfloat16(), rnd(n, k, seed=12).bfloat16(), rnd(n, seed=13).bfloat16()
    ref = x.double() @ w.double().t() + b.double()
    out = ops().gemm_stream(torch.empty(m, n, device=DEV), x.to(DEV), w.to(DEV), b.to(DEV))
    assert (out.cpu().double() - ref).abs().max() <= 2e-6 * math.sqrt(k) * float(ref.abs().max())


@pytest.mark.parametrize("m,n,k,splits", [(1, 16, 64, 2), (8, 2048, 2048, 2), (5, 2048, 5632, 4), (16, 100, 5632 + 96, 3),
                                          (40, 320, 2048, 2), (3, 48, 1024, 16), (8, 512, 28672, 4)])
def test_gemm_stream_k_split_over_workgroups(m, n, k, splits):
    """K shared out to several workgroups per tile: partial sums whose total is the product (a share may be
    empty when there are fewer chunks of 512 than splits); the bias is in the first."""
    x, w, b = rnd(m, k, seed=11).bfloat16(), rnd(n, k, seed=12).bfloat16(), rnd(n, seed=13).bfloat16()
    ref = x.double() @ w.double().t() + b.double()
    parts = ops().gemm_stream(torch.full((splits, m, n), 9.0, device=DEV), x.to(DEV), w.to(DEV), b.to(DEV), k_splits=splits)
    assert parts.shape == (splits, m, n)
    assert (parts.cpu().double().sum(0) - ref).abs().max() <= 2e-6 * math.sqrt(k) * float(ref.abs().max())
    chunks = -(-k // 512)
    per = -(-chunks // splits)
    for s_ in range(splits):  # each share holds exactly its columns of K
        lo, hi = min(k, s_ * per * 512), min(k, (s_ + 1) * per * 512)
        want = x[:, lo:hi].double() @ w[:, lo:hi].double().t() + (b.double() if s_ == 0 else 0)
        assert (parts[s_].cpu().double() - want).abs().max() <= 2e-6 * math.sqrt(k) * float(ref.abs().max())
    with pytest.raises(ValueError, match="k_splits"):
        ops().gemm_stream(torch.empty(splits, m, n, device=DEV), x.to(DEV), w.to(DEV), k_splits=splits, swiglu=True)
    with pytest.raises(ValueError, match="float32"):
        ops().gemm_stream(torch.empty(splits, m, n, dtype=torch.bfloat16, device=DEV), x.to(DEV), w.to(DEV), k_splits=splits)


@pytest.mark.parametrize("m,n,k", [(64, 2048, 2048), (33, 2048, 5632), (17, 333, 1048), (50, 1002, 520), (24, 64, 176),
                                   (48, 96, 96), (1, 17, 8), (64, 40, 4096 + 40)])
def test_gemm_slices(m, n, k):
    """A slice of all rows in LDS, one array of partial sums per 512 of K: each array holds exactly its columns
    of K (rows and k-steps that do not exist add nothing, whatever the clamped loads brought), their sum is the
    product, and what lies around the arrays is not written."""
    x, w = rnd(m, k, seed=31).bfloat16(), rnd(n, k, seed=32).bfloat16()
    ref = x.double() @ w.double().t()
    slices = -(-k // 512)
    buf = torch.full((slices * m * n + 64,), 7.0, device=DEV)
    parts = ops().gemm_slices(buf[32:-32].view(slices, m, n), x.to(DEV), w.to(DEV))
    assert torch.all(buf[:32] == 7.0) and torch.all(buf[-32:] == 7.0)
    tol = 2e-6 * math.sqrt(k) * float(ref.abs().max())
    assert (parts.cpu().double().sum(0) - ref).abs().max() <= tol
    for s_ in range(slices):
        lo, hi = 512 * s_, min(k, 512 * (s_ + 1))
        assert (parts[s_].cpu().double() - x[:, lo:hi].double() @ w[:, lo:hi].double().t()).abs().max() <= tol
    # rows of a larger tensor: the stride of x is not K
    wide = torch.cat([x, rnd(m, 8, seed=33).bfloat16()], dim=1).to(DEV)
    again = ops().gemm_slices(torch.empty(slices, m, n, device=DEV), wide[:, :k], w.to(DEV))
    assert torch.equal(again, parts)
    with pytest.raises(ValueError, match="shape"):
        ops().gemm_slices(torch.empty(slices + 1, m, n, device=DEV), x.to(DEV), w.to(DEV))
    with pytest.raises(ValueError, match="1..64"):
        ops().gemm_slices(torch.empty(slices, 65, n, device=DEV), rnd(65, k).bfloat16().to(DEV), w.to(DEV))


@pytest.mark.parametrize("m,inter,k", [(1, 176, 64), (5, 5632, 2048), (16, 256, 96), (37, 5632, 2048), (64, 256, 1024),
                                       (8, 1792, 8192)])
def test_gemm_stream_gated_epilogue(m, inter, k):
    """gate and up of the feed-forward in one product over [gate; up], silu(gate) * up in the epilogue:
    the same bits as the product followed by the activation kernel."""
    x = rnd(m, k, seed=16).bfloat16()
    w = torch.cat([rnd(inter, k, seed=17, scale=0.2), rnd(inter, k, seed=18, scale=0.2)]).bfloat16()
    g, u = plain_llama.linear(x, w[:inter]), plain_llama.linear(x, w[inter:])
    ref = (plain_llama.silu(g) * u).float()
    out = ops().gemm_stream(torch.empty(m, inter, dtype=torch.bfloat16, device=DEV), x.to(DEV), w.to(DEV), swiglu=True)
    assert (out.float().cpu() - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max())
    gu = ops().gemm_stream(torch.empty(m, 2 * inter, dtype=torch.bfloat16, device=DEV), x.to(DEV), w.to(DEV))
    act = ops().silu_mul(torch.empty(m, inter, dtype=torch.bfloat16, device=DEV), gu)
    assert torch.equal(act, out)


@pytest.mark.parametrize("nh,nkv,d,bs,theta,bias,m", [(4, 2, 16, 16, 1e4, False, 5), (3, 1, 32, 8, 5e5, True, 5),
                                                      (8, 2, 64, 16, 1e4, False, 64), (2, 2, 48, 8, None, True, 33)])
def test_gemm_stream_rotary_epilogue(nh, nkv, d, bs, theta, bias, m):
    """q/k/v projection with the rotation and the cache store in the epilogue: the same bits as the
    projection followed by the rotation kernel."""
    k, pages = (4096 if m in (9, 12, 24) else 96), 12  # (a long K: the rows are kept in registers, not in LDS)
    n = (nh + 2 * nkv) * d
    x, w = rnd(m, k, seed=23).bfloat16().to(DEV), rnd(n, k, seed=24, scale=0.3 if k < 1000 else 0.05).bfloat16().to(DEV)
    b = rnd(n, seed=25).bfloat16().to(DEV) if bias else None
    gen = torch.Generator().manual_seed(35)
    positions = torch.randint(0, 4096, (m,), generator=gen).to(torch.int32)
    positions[0] = 0
    positions = positions.to(DEV)
    slots = torch.randperm(bs * pages, generator=gen)[:m].to(torch.int32)
    slots[m // 2] = -1
    slots = slots.to(DEV)
    inv_freq = (1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV) if theta else None
    pools = lambda: (torch.full((pages, nkv, bs, d), 7.0, dtype=torch.bfloat16, device=DEV),  # noqa: E731
                     torch.full((pages, nkv, d, bs), 7.0, dtype=torch.bfloat16, device=DEV))
    k1, v1 = pools()
    qkv = ops().gemm_stream(torch.empty(m, n, dtype=torch.bfloat16, device=DEV), x, w, b)
    ops().rope_store(qkv, inv_freq, positions, slots, k1, v1, nh, nkv, d, bs)
    k2, v2 = pools()
    q = ops().gemm_stream(torch.empty(m, nh * d, dtype=torch.bfloat16, device=DEV), x, w, b,
                          rope=dict(n_heads=nh, n_kv_heads=nkv, head_dim=d, inv_freq=inv_freq, positions=positions,
                                    slots=slots, k_pool=k2, v_pool=v2, block_size=bs))
    assert torch.equal(q, qkv[:, : nh * d]) and torch.equal(k1, k2) and torch.equal(v1, v2)
    assert (k2 != 7).any() and (v2 != 7).any()
    # without slots only q is produced
    k3, v3 = pools()
    q3 = ops().gemm_stream(torch.empty(m, nh * d, dtype=torch.bfloat16, device=DEV), x, w, b,
                           rope=dict(n_heads=nh, n_kv_heads=nkv, head_dim=d, inv_freq=inv_freq, positions=positions,
                                     slots=None, k_pool=k3, v_pool=v3, block_size=bs))
    assert torch.equal(q3, q) and (k3 == 7).all() and (v3 == 7).all()


# ------------------------------------------------------------------ gemm_decode: one workgroup per compute unit
@pytest.mark.parametrize("m,n,k", [(1, 16, 64), (3, 333, 96), (16, 2056, 2048), (7, 100, 5632), (9, 48, 176),
                                   (8, 32000, 2048), (5, 2048, 4096), (8, 24, 5888), (2, 5000, 8), (12, 40, 2944),
                                   (17, 333, 96), (64, 2056, 2048), (33, 32000, 2048), (40, 100, 1024), (48, 50, 176),
                                   (25, 3000, 1032), (16, 2048, 5632), (9, 333, 3072 - 8), (12, 4100, 4096), (16, 40, 6144),
                                   (24, 4100, 4096), (32, 100, 3072 - 8), (17, 48, 2048 + 8)])
def test_gemm_decode_plain(m, n, k):
    x, w, b = rnd(m, k, seed=11).bfloat16(), rnd(n, k, seed=12).bfloat16(), rnd(n, seed=13).bfloat16()
    ref = x.double() @ w.double().t() + b.double()
    buf = torch.full((m * n + 64,), 7.0, device=DEV)
    out = ops().gemm_decode(buf[32:-32].view(m, n), x.to(DEV), w.to(DEV), b.to(DEV))
    assert (out.cpu().double() - ref).abs().max() <= 2e-6 * math.sqrt(k) * float(ref.abs().max())
    assert torch.all(buf[:32] == 7.0) and torch.all(buf[-32:] == 7.0)
    out = ops().gemm_decode(torch.empty(m, n, dtype=torch.bfloat16, device=DEV), x.to(DEV), w.to(DEV))
    ref = x.double() @ w.double().t()
    assert (out.float().cpu().double() - ref).abs().max() <= 2.0 ** -8 * float(ref.abs().max())
    # rows of a larger tensor: the stride of x is not K
    wide = torch.cat([x, rnd(m, 8, seed=33).bfloat16()], dim=1).to(DEV)
    assert torch.equal(ops().gemm_decode(torch.empty(m, n, dtype=torch.bfloat16, device=DEV), wide[:, :k], w.to(DEV)), out)


@pytest.mark.parametrize("m,n,k,parts", [(64, 2048, 5632, 3), (17, 333, 2048 + 8, 2), (33, 4096, 11008, 6), (40, 100, 520, 5),
                                         (24, 2048, 5632, 3), (64, 48, 256, 2)])
def test_gemm_decode_shares_k_out_for_many_rows(m, n, k, parts):
    """17 to 64 rows against a weight whose K does not fit the registers: partial sums per part of K."""
    x, w = rnd(m, k, seed=61).bfloat16(), rnd(n, k, seed=62, scale=0.2).bfloat16()
    ref = x.double() @ w.double().t()
    out = ops().gemm_decode(torch.full((parts, m, n), float("nan"), device=DEV), x.to(DEV), w.to(DEV), k_parts=parts)
    assert (out.sum(0).cpu().double() - ref).abs().max() <= 1e-5 * float(ref.abs().max()) + 1e-5
    each = -(-(-(-k // 128)) // parts) * 128  # the first part alone is the product over its columns
    first = x[:, :each].double() @ w[:, :each].double().t()
    assert (out[0].cpu().double() - first).abs().max() <= 1e-5 * float(first.abs().max()) + 1e-5
    best = ops().gemm_decode_k_parts(m, k)  # the number of parts the parts of a model would ask for: it has to work too
    assert 1 <= best <= 8
    if best > 1:
        again = ops().gemm_decode(torch.empty(best, m, n, device=DEV), x.to(DEV), w.to(DEV), k_parts=best)
        assert (again.sum(0).cpu().double() - ref).abs().max() <= 1e-5 * float(ref.abs().max()) + 1e-5
    with pytest.raises(ValueError, match="shared out"):
        ops().gemm_decode(torch.empty(parts, 8, n, device=DEV), x[:8].to(DEV), w.to(DEV), k_parts=parts)


def test_gemm_decode_refuses_what_it_cannot_take():
    x, w = rnd(65, 64).bfloat16().to(DEV), rnd(32, 64).bfloat16().to(DEV)
    with pytest.raises(ValueError, match="1..64"):
        ops().gemm_decode(torch.empty(65, 32, dtype=torch.bfloat16, device=DEV), x, w)
    with pytest.raises(ValueError, match="taken as they are"):
        ops().gemm_decode(torch.empty(17, 32, dtype=torch.bfloat16, device=DEV), x[:17], w, norm=(rnd(64).bfloat16().to(DEV), 1e-5))
    for rows, big in ((2, ops().GEMM_DECODE_MAX_K + 8), (9, ops().GEMM_DECODE_MAX_K + 8), (17, 4096 + 8), (33, 2048 + 8)):
        with pytest.raises(ValueError, match="do not fit"):
            ops().gemm_decode(torch.empty(rows, 32, dtype=torch.bfloat16, device=DEV), rnd(rows, big).bfloat16().to(DEV),
                              rnd(32, big).bfloat16().to(DEV))
    with pytest.raises(ValueError, match="one epilogue"):
        ops().gemm_decode(torch.empty(2, 16, dtype=torch.bfloat16, device=DEV), x[:2], w, swiglu=True,
                          residual=torch.empty(2, 32, dtype=torch.bfloat16, device=DEV))
    assert not ops().gemm_decode_supported(x, w) and ops().gemm_decode_supported(x[:64], w)


@pytest.mark.parametrize("m,n,k,eps", [(1, 64, 64, 1e-5), (8, 2560, 2048, 1e-5), (16, 333, 96, 1e-6), (5, 100, 4096, 1e-5),
                                       (3, 48, 5888 - 8, 1e-6), (13, 200, 2560, 1e-5), (16, 11264, 2048, 1e-5),
                                       (16, 2560, 4096, 1e-5), (9, 100, 5632, 1e-6), (12, 333, 3072 + 8, 1e-6)])
def test_gemm_decode_norms_its_rows_on_the_way_in(m, n, k, eps):
    """RMSNorm in the prologue: the same as the norm kernel followed by the product (the sum of squares is added up
    in another order, so the normed rows may differ by one rounding)."""
    x = rnd(m, k, seed=41, scale=3.0).bfloat16()
    nw = (1 + 0.1 * rnd(k, seed=42)).bfloat16()
    w = rnd(n, k, seed=43, scale=0.1).bfloat16()
    normed = plain_llama.rms_norm(x, nw, eps)
    ref = normed.double() @ w.double().t()
    out = ops().gemm_decode(torch.empty(m, n, device=DEV), x.to(DEV), w.to(DEV), norm=(nw.to(DEV), eps))
    # a normed element may be rounded the other way: 2^-8 of it, times its weight, summed over K at random signs
    tol = 2.0 ** -8 * float(normed.float().abs().max()) * float(w.float().abs().max()) * math.sqrt(k)
    assert (out.cpu().double() - ref).abs().max() <= tol
    # against the norm kernel and the plain product of this library
    y = ops().rmsnorm(torch.empty(m, k, dtype=torch.bfloat16, device=DEV), x.to(DEV), nw.to(DEV), eps)
    two = ops().gemm_decode(torch.empty(m, n, device=DEV), y, w.to(DEV))
    assert (out - two).abs().max() <= tol
    assert (out != two).float().mean() < 0.5  # mostly the same bits


@pytest.mark.parametrize("m,inter,k", [(1, 176, 64), (5, 5632, 2048), (16, 256, 96), (8, 1000, 4096), (3, 22, 2048),
                                       (64, 5632, 2048), (17, 176, 64), (37, 1000, 1024), (32, 256, 2048),
                                       (16, 11008, 4096), (10, 100, 6144 - 8), (32, 11008, 4096), (20, 50, 2560)])
def test_gemm_decode_gated_epilogue(m, inter, k):
    """silu(gate) * up in the epilogue: the same bits as the product followed by the activation kernel."""
    x = rnd(m, k, seed=16).bfloat16()
    w = torch.cat([rnd(inter, k, seed=17, scale=0.2), rnd(inter, k, seed=18, scale=0.2)]).bfloat16()
    g, u = plain_llama.linear(x, w[:inter]), plain_llama.linear(x, w[inter:])
    ref = (plain_llama.silu(g) * u).float()
    out = ops().gemm_decode(torch.empty(m, inter, dtype=torch.bfloat16, device=DEV), x.to(DEV), w.to(DEV), swiglu=True)
    assert (out.float().cpu() - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max())
    gu = ops().gemm_decode(torch.empty(m, 2 * inter, dtype=torch.bfloat16, device=DEV), x.to(DEV), w.to(DEV))
    act = ops().silu_mul(torch.empty(m, inter, dtype=torch.bfloat16, device=DEV), gu)
    assert torch.equal(act, out)


@pytest.mark.parametrize("nh,nkv,d,bs,theta,bias,m", [(4, 2, 16, 16, 1e4, False, 5), (3, 1, 32, 8, 5e5, True, 5),
                                                      (32, 4, 64, 16, 1e4, False, 8), (2, 2, 48, 8, None, True, 16),
                                                      (5, 5, 128, 16, 1e4, True, 3), (6, 3, 80, 16, 1e6, False, 1),
                                                      (32, 4, 64, 16, 1e4, False, 64), (3, 1, 32, 8, 5e5, True, 33),
                                                      (8, 2, 128, 16, 1e4, True, 20), (32, 8, 128, 16, 1e4, False, 12),
                                                      (3, 3, 64, 8, 1e4, True, 9), (32, 32, 128, 16, 1e4, False, 24)])
def test_gemm_decode_rotary_epilogue(nh, nkv, d, bs, theta, bias, m):
    """q/k/v projection with the rotation and the cache store in the epilogue: the same bits as the
    projection followed by the rotation kernel."""
    k, pages = 96, 12
    n = (nh + 2 * nkv) * d
    x, w = rnd(m, k, seed=23).bfloat16().to(DEV), rnd(n, k, seed=24, scale=0.3).bfloat16().to(DEV)
    b = rnd(n, seed=25).bfloat16().to(DEV) if bias else None
    gen = torch.Generator().manual_seed(35)
    positions = torch.randint(0, 4096, (m,), generator=gen).to(torch.int32)
    positions[0] = 0
    positions = positions.to(DEV)
    slots = torch.randperm(bs * pages, generator=gen)[:m].to(torch.int32)
    slots[m // 2] = -1
    slots = slots.to(DEV)
    inv_freq = (1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).to(DEV) if theta else None
    pools = lambda: (torch.full((pages, nkv, bs, d), 7.0, dtype=torch.bfloat16, device=DEV),  # noqa: E731
                     torch.full((pages, nkv, d, bs), 7.0, dtype=torch.bfloat16, device=DEV))
    k1, v1 = pools()
    qkv = ops().gemm_decode(torch.empty(m, n, dtype=torch.bfloat16, device=DEV), x, w, b)
    ops().rope_store(qkv, inv_freq, positions, slots, k1, v1, nh, nkv, d, bs)
    k2, v2 = pools()
    rope = dict(n_heads=nh, n_kv_heads=nkv, head_dim=d, inv_freq=inv_freq, positions=positions, slots=slots,
                k_pool=k2, v_pool=v2, block_size=bs)
    q = ops().gemm_decode(torch.empty(m, nh * d, dtype=torch.bfloat16, device=DEV), x, w, b, rope=rope)
    assert torch.equal(q, qkv[:, : nh * d]) and torch.equal(k1, k2) and torch.equal(v1, v2)
    assert (k2 != 7).any() and (v2 != 7).any() or m == 1
    k3, v3 = pools()  # without slots only q is produced
    q3 = ops().gemm_decode(torch.empty(m, nh * d, dtype=torch.bfloat16, device=DEV), x, w, b, rope=dict(rope, slots=None, k_pool=k3, v_pool=v3))
    assert torch.equal(q3, q) and (k3 == 7).all() and (v3 == 7).all()
    if theta:  # the sines and cosines from a table made ahead: the same bits
        angles = ops().rotary_angles(positions, inv_freq)
        exact = positions.double().cpu()[:, None] * inv_freq.double().cpu()[None, :]
        assert (angles.cpu().double() - torch.stack([exact.sin(), exact.cos()], dim=-1)).abs().max() < 1e-3  # (32-bit angles of up to 4,096)
        k4, v4 = pools()
        q4 = ops().gemm_decode(torch.empty(m, nh * d, dtype=torch.bfloat16, device=DEV), x, w, b,
                               rope=dict(rope, k_pool=k4, v_pool=v4, angles=angles))
        assert torch.equal(q4, q) and torch.equal(k4, k2) and torch.equal(v4, v2)


@pytest.mark.parametrize("m,n,k,bias", [(1, 64, 64, False), (8, 2048, 2048, False), (8, 2048, 5632, True), (16, 333, 176, True),
                                        (5, 4096, 4096, False), (11, 90, 2900 - 4, True), (64, 2048, 2048, False),
                                        (19, 333, 176, True), (40, 4000, 1024, True), (16, 2048, 5632, False),
                                        (13, 4096, 4096, True), (9, 50, 3000, False), (30, 4096, 4096, False)])
def test_gemm_decode_residual_epilogue(m, n, k, bias):
    """residual += x w^T: the rounded product added to the row in 32-bit and rounded once, as the norm kernel adds a
    delta (same bits as product, then that kernel's residual output)."""
    x, w = rnd(m, k, seed=51).bfloat16().to(DEV), rnd(n, k, seed=52, scale=0.1).bfloat16().to(DEV)
    b = rnd(n, seed=53).bfloat16().to(DEV) if bias else None
    wide = rnd(m, n + 8, seed=54, scale=2.0).bfloat16().to(DEV)
    res = wide[:, :n]  # (a view: the row stride is not N)
    before = res.clone()
    delta = ops().gemm_decode(torch.empty(m, n, dtype=torch.bfloat16, device=DEV), x, w, b)
    want = (before.float() + delta.float()).bfloat16()
    got = ops().gemm_decode(None, x, w, b, residual=res)
    assert got is res and torch.equal(res, want)
    assert torch.equal(wide[:, n:].cpu(), rnd(m, n + 8, seed=54, scale=2.0).bfloat16()[:, n:])


def test_gemm_decode_rows_do_not_depend_on_the_batch():
    a, w = rnd(16, 2048, seed=14).bfloat16().to(DEV), rnd(320, 2048, seed=15).bfloat16().to(DEV)
    nw = (1 + 0.1 * rnd(2048, seed=4)).bfloat16().to(DEV)
    full = ops().gemm_decode(torch.empty(16, 320, device=DEV), a, w, norm=(nw, 1e-5))
    one = ops().gemm_decode(torch.empty(1, 320, device=DEV), a[9:10].contiguous(), w, norm=(nw, 1e-5))
    assert torch.equal(full[9:10], one)


def test_gemm_bf16_rows_do_not_depend_on_the_batch():
    """A row's result is the same bits whatever else is in the batch (same kernel)."""
    a, w = rnd(40, 2048, seed=14).bfloat16().to(DEV), rnd(320, 2048, seed=15).bfloat16().to(DEV)
    full = ops().gemm_bf16(torch.empty(40, 320, device=DEV), a, w, kernel="skinny")
    one = ops().gemm_bf16(torch.empty(1, 320, device=DEV), a[17:18].contiguous(), w, kernel="skinny")
    assert torch.equal(full[17], one[0])
    full = ops().gemm_stream(torch.empty(40, 320, device=DEV), a, w)
    one = ops().gemm_stream(torch.empty(1, 320, device=DEV), a[29:30].contiguous(), w)
    assert torch.equal(full[29], one[0])


def test_gemm_bf16_refuses_what_it_cannot_take():
    a, w = torch.zeros(4, 100, dtype=torch.bfloat16, device=DEV), torch.zeros(8, 100, dtype=torch.bfloat16, device=DEV)
    assert not ops().gemm_bf16_supported(a, w)
    with pytest.raises(ValueError, match="multiples of 8"):
        ops().gemm_bf16(torch.empty(4, 8, device=DEV), a, w)
    with pytest.raises(ValueError, match="at most 64"):
        ops().gemm_bf16(torch.empty(70, 8, device=DEV), torch.zeros(70, 64, dtype=torch.bfloat16, device=DEV),
                        torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV), kernel="skinny")


# ------------------------------------------------------------------ attention
def run_attention(fn, dtype, nh, nkv, d, bs, lens, new, window=0, seed=0, craft=None):
    """Requests of lengths `lens`, the last `new[b]` tokens of each are this step's queries."""
    qs = [rnd(s, nh, d, seed=seed + 3 * b) for b, s in enumerate(lens)]
    ks = [rnd(s, nkv, d, seed=seed + 3 * b + 1) for b, s in enumerate(lens)]
    vs = [rnd(s, nkv, d, seed=seed + 3 * b + 2) for b, s in enumerate(lens)]
    if craft:
        craft(qs, ks, vs)
    qs, ks, vs = ([t.to(dtype) for t in ts] for ts in (qs, ks, vs))
    k_pool, v_pool, tables = make_paged(ks, vs, bs, dtype, seed=seed)
    q_rows, token_seq, positions, refs = [], [], [], []
    for b, (s, n) in enumerate(zip(lens, new)):
        rows = list(range(s - n, s))
        q_rows.append(qs[b][rows].reshape(n, nh * d))
        token_seq += [b] * n
        positions += rows
        refs.append(attention_reference(qs[b], ks[b], vs[b], rows, window or None))
    q = torch.cat(q_rows).contiguous().to(DEV)
    out = torch.empty(q.shape[0], nh * d, dtype=dtype, device=DEV)
    fn(out, q, k_pool.to(DEV), v_pool.to(DEV), tables.to(DEV), torch.tensor(token_seq, dtype=torch.int32, device=DEV),
       torch.tensor(positions, dtype=torch.int32, device=DEV), nh, nkv, d, bs, window)
    ref = torch.cat(refs)
    got = out.float().cpu()
    assert torch.isfinite(got).all(), "read a slot that was never written"
    return got, ref


ATT_CASES = [  # nh, nkv, d, bs, lens, new, window
    (4, 2, 16, 16, [5, 17, 33], [5, 17, 33], 0),
    (3, 1, 32, 8, [1, 7, 40, 100], [1, 1, 1, 1], 0),
    (8, 1, 64, 16, [300, 64, 129], [1, 24, 2], 0),
    (6, 2, 80, 4, [70, 19], [3, 19], 0),
    (4, 4, 128, 32, [257, 31], [1, 31], 0),
    (2, 1, 256, 16, [90], [7], 0),
    (32, 4, 64, 16, [600], [1], 0),
    (4, 2, 48, 1, [37], [37], 0),
    (4, 2, 32, 8, [150, 40], [30, 1], 16),
    (3, 3, 16, 16, [100], [100], 7),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", ATT_CASES)
def test_attention_wave(dtype, case):
    nh, nkv, d, bs, lens, new, window = case
    got, ref = run_attention(ops().attention_wave, dtype, nh, nkv, d, bs, lens, new, window, seed=20)
    tol = 2.0 ** -7 * float(ref.abs().max()) if dtype == torch.bfloat16 else 2e-5
    assert (got - ref).abs().max() <= tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("needle", [0, 15, 16, 299, 300 - 17, 141])
def test_attention_wave_finds_one_far_key(dtype, needle):
    """One key among hundreds gets all the weight (query and key scaled up): the output must be
    that key's value, wherever in the pages it lies."""
    def craft(qs, ks, vs):
        qs[0][-1] = 0
        qs[0][-1, :, 0] = 12.0
        ks[0][:, :, 0] = 0
        ks[0][needle, :, 0] = 12.0

    got, ref = run_attention(ops().attention_wave, dtype, 8, 2, 64, 16, [300], [1], 0, seed=30, craft=craft)
    assert (got - ref).abs().max() <= (2.0 ** -7 * float(ref.abs().max()) if dtype == torch.bfloat16 else 2e-5)


def test_attention_wave_window_edge():
    """The key just inside the window counts, the key just outside does not."""
    for needle, inside in ((100 - 8, False), (100 - 7, True)):
        def craft(qs, ks, vs):
            qs[0][-1] = 0
            qs[0][-1, :, 1] = 10.0
            ks[0][:, :, 1] = 0
            ks[0][needle, :, 1] = 10.0
            vs[0][needle] = 5.0

        got, ref = run_attention(ops().attention_wave, torch.float32, 2, 1, 32, 8, [101], [1], 8, seed=31, craft=craft)
        assert (got - ref).abs().max() <= 2e-5
        assert (got.mean() > 4.0) == inside


# ------------------------------------------------------------------ sampling
@pytest.mark.parametrize("vocab", [5, 333, 32000, 50257])
def test_argmax_lowest_index_wins(vocab):
    logits = rnd(6, vocab, seed=40)
    logits[1, 3 % vocab] = logits[1, vocab - 1] = 50.0  # a tie: the lower index wins
    logits[2, vocab - 1] = 60.0
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    ops().sample_rows(out, logits.to(DEV))
    want = [int(torch.argmax(row)) for row in logits]
    want[1] = 3 % vocab
    assert out.tolist() == want


def test_sampler_reference_vector():
    logits = torch.tensor([[0.1, 3.0, 0.2, 2.9, -1.0]] * 40, device=DEV)
    u = torch.linspace(0, 0.999, 40, device=DEV)
    ones, out = torch.ones(40, device=DEV), torch.empty(40, dtype=torch.int32, device=DEV)
    k = lambda v: torch.full((40,), v, dtype=torch.int32, device=DEV)  # noqa: E731
    ops().sample_rows(out, logits, temperature=ones, top_k=k(1), top_p=ones, uniform=u)
    assert set(out.tolist()) == {1}
    ops().sample_rows(out, logits, temperature=ones, top_k=k(0), top_p=torch.full((40,), 1e-6, device=DEV), uniform=u)
    assert set(out.tolist()) == {1}
    ops().sample_rows(out, logits, temperature=ones, top_k=k(2), top_p=ones, uniform=u)
    assert set(out.tolist()) == {1, 3}
    ops().sample_rows(out, logits, temperature=torch.zeros(40, device=DEV), top_k=k(0), top_p=ones, uniform=u)
    assert set(out.tolist()) == {1}


@pytest.mark.parametrize("vocab,temperature,top_k,top_p", [(333, 0.8, 0, 1.0), (32000, 1.0, 50, 1.0),
                                                           (32000, 0.7, 0, 0.9), (5000, 1.3, 40, 0.5),
                                                           (50257, 1.0, 0, 1.0), (50257, 0.9, 30, 0.8),
                                                           (32768, 0.9, 64, 0.95), (32769, 1.1, 0, 0.7),
                                                           # (more survivors of top-k than the kernel gathers before top-p)
                                                           (32000, 0.9, 2000, 0.9), (50257, 1.2, 1500, 0.6)])
def test_sample_rows_inverts_the_plain_cdf(vocab, temperature, top_k, top_p):
    rows = 24
    logits = rnd(rows, vocab, seed=41, scale=3.0)
    u = torch.rand(rows, generator=torch.Generator().manual_seed(42))
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    dev = lambda t: t.to(DEV)  # noqa: E731
    ops().sample_rows(out, dev(logits), temperature=dev(torch.full((rows,), temperature)),
                      top_k=dev(torch.full((rows,), top_k, dtype=torch.int32)),
                      top_p=dev(torch.full((rows,), top_p)), uniform=dev(u))
    for r, tok in enumerate(out.tolist()):
        probs = plain_llama.filtered_probs(logits[r], temperature, top_k, top_p)
        assert probs[tok] > 0, f"row {r}: token {tok} was filtered out by the plain sampler"
        cdf = probs.cumsum(-1)
        lo = float(cdf[tok - 1]) if tok > 0 else 0.0
        assert lo - 1e-5 <= float(u[r]) <= float(cdf[tok]) + 1e-5, (r, tok, float(u[r]), lo, float(cdf[tok]))


def test_sample_rows_mixed_batch_and_frequencies():
    logits = torch.tensor([[0.0, 1.0, 2.0, 0.5]], device=DEV).repeat(4000, 1)
    u = torch.rand(4000, generator=torch.Generator().manual_seed(43)).to(DEV)
    temp = torch.full((4000,), 0.7, device=DEV)
    temp[::2] = 0.0  # greedy rows beside sampled ones
    out = torch.empty(4000, dtype=torch.int32, device=DEV)
    ops().sample_rows(out, logits, temperature=temp, uniform=u)
    got = out.cpu()
    assert (got[::2] == 2).all()
    freq = torch.bincount(got[1::2].long(), minlength=4).float() / 2000
    assert torch.allclose(freq, torch.softmax(logits[0].cpu() / 0.7, -1), atol=0.04)


@pytest.mark.parametrize("vocab", [32000, 40000])
def test_sample_rows_do_not_depend_on_the_batch_or_the_run(vocab):
    """The thresholds are found with atomic additions to shared histograms: the sums are integers (counts, masses in
    fixed point), so a row gives the same token wherever it stands in a batch and however often it is asked."""
    rows = 33
    logits = rnd(rows, vocab, seed=44, scale=4.0)
    logits[5, 100:164] = logits[5, 99]  # many keys at one value: ties at a threshold
    u = torch.rand(rows, generator=torch.Generator().manual_seed(45))
    dev = lambda t: t.to(DEV)  # noqa: E731
    temp, k, p = torch.full((rows,), 0.9), torch.full((rows,), 50, dtype=torch.int32), torch.full((rows,), 0.8)
    k[::3] = 0
    p[1::3] = 1.0
    first = ops().sample_rows(torch.empty(rows, dtype=torch.int32, device=DEV), dev(logits), temperature=dev(temp),
                              top_k=dev(k), top_p=dev(p), uniform=dev(u)).clone()
    for _ in range(10):
        again = ops().sample_rows(torch.empty(rows, dtype=torch.int32, device=DEV), dev(logits), temperature=dev(temp),
                                  top_k=dev(k), top_p=dev(p), uniform=dev(u))
        assert torch.equal(again, first)
    order = torch.randperm(rows, generator=torch.Generator().manual_seed(46))
    moved = ops().sample_rows(torch.empty(rows, dtype=torch.int32, device=DEV), dev(logits[order]), temperature=dev(temp[order]),
                              top_k=dev(k[order]), top_p=dev(p[order]), uniform=dev(u[order]))
    assert torch.equal(moved.cpu(), first.cpu()[order])
    for r in (0, 5, 17):
        one = ops().sample_rows(torch.empty(1, dtype=torch.int32, device=DEV), dev(logits[r: r + 1]), temperature=dev(temp[r: r + 1]),
                                top_k=dev(k[r: r + 1]), top_p=dev(p[r: r + 1]), uniform=dev(u[r: r + 1]))
        assert int(one[0]) == int(first[r])


# ------------------------------------------------------------------ attention on the matrix cores
def run_attention_mfma(nh, nkv, d, bs, lens, new, window=0, seed=0, craft=None, split_waves=False, num_splits=1,
                       waves=4, merge_kernel=False, repeat=1):
    """As `run_attention`, for the bfloat16 matrix-core kernel and its request-wise arguments."""
    dtype = torch.bfloat16
    qs = [rnd(s, nh, d, seed=seed + 3 * b) for b, s in enumerate(lens)]
    ks = [rnd(s, nkv, d, seed=seed + 3 * b + 1) for b, s in enumerate(lens)]
    vs = [rnd(s, nkv, d, seed=seed + 3 * b + 2) for b, s in enumerate(lens)]
    if craft:
        craft(qs, ks, vs)
    qs, ks, vs = ([t.to(dtype) for t in ts] for ts in (qs, ks, vs))
    k_pool, v_pool, tables = make_paged(ks, vs, bs, dtype, seed=seed)
    q_rows, refs, cu = [], [], [0]
    for b, (s, n) in enumerate(zip(lens, new)):
        rows = list(range(s - n, s))
        q_rows.append(qs[b][rows].reshape(n, nh * d))
        cu.append(cu[-1] + n)
        refs.append(attention_reference(qs[b], ks[b], vs[b], rows, window or None))
    # queries sit inside a wider row, as the q part of a qkv buffer does
    q = torch.cat([torch.cat(q_rows), torch.full((cu[-1], 2 * nkv * d), float("nan"), dtype=dtype)], dim=1).contiguous().to(DEV)
    out = torch.empty(cu[-1], nh * d, dtype=dtype, device=DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    operands = (q, k_pool.to(DEV), v_pool.to(DEV), tables.to(DEV), i32(cu), i32(lens))
    for _ in range(repeat):  # (launches in a row find the counters of the one before zero again)
        out.fill_(float("nan"))
        ops().attention_mfma(out, *operands, 0, len(lens), max(new), 0, cu[-1], nh, nkv, d, bs, window, None,
                             split_waves=split_waves, num_splits=num_splits, waves=waves, merge_kernel=merge_kernel)
    got = out.float().cpu()
    assert torch.isfinite(got).all(), "read a slot that was never written"
    return got, torch.cat(refs)


MFMA_CASES = [  # nh, nkv, d, bs, lens, new, window
    (4, 2, 16, 16, [5, 17, 33], [5, 17, 33], 0),
    (3, 1, 32, 8, [1, 7, 40, 100], [1, 1, 1, 1], 0),
    (3, 1, 32, 8, [1, 7, 40, 100], [1, 7, 24, 2], 0),
    (8, 1, 64, 16, [300, 64, 129], [1, 24, 2], 0),
    (6, 2, 80, 8, [70, 19], [3, 19], 0),
    (4, 4, 128, 32, [257, 31], [1, 31], 0),
    (2, 1, 256, 16, [90], [7], 0),
    (32, 4, 64, 16, [600, 31], [1, 1], 0),
    (64, 8, 128, 16, [300, 64, 129], [1, 24, 2], 0),  # 8 heads per KV head at head_dim 128: the Llama-2-70B layer
    (64, 8, 128, 16, [700, 33], [1, 1], 0),
    (32, 1, 32, 8, [45], [3], 0),
    (5, 1, 48, 8, [77], [20], 0),
    (12, 1, 16, 24, [50], [50], 0),
    (4, 2, 32, 8, [150, 40], [30, 1], 16),
    (3, 3, 16, 16, [100], [100], 7),
    (4, 1, 64, 16, [200], [64], 40),
]


# split_waves: False = the prompt kernel (tiles shared through LDS; without a window and in a large launch every wave
# has a twin that takes every other tile for the same columns; with splits, the keys of a block shared out to
# workgroups), True = the waves (4 or 8) share the keys, optionally split over workgroups
@pytest.mark.parametrize("arrangement", [(False, 1, 4), (False, 2, 4), (False, 5, 4), (True, 1, 4), (True, 2, 4), (True, 5, 4),
                                         (True, 1, 8), (True, 3, 8)])
@pytest.mark.parametrize("case", MFMA_CASES)
def test_attention_mfma(case, arrangement):
    nh, nkv, d, bs, lens, new, window = case
    split_waves, num_splits, waves = arrangement
    if window and not split_waves and num_splits > 1:
        with pytest.raises(ValueError, match="window"):
            run_attention_mfma(nh, nkv, d, bs, lens, new, window, seed=50, num_splits=num_splits)
        return
    if waves == 8 and d > 160:
        with pytest.raises(ValueError, match="8 waves"):
            run_attention_mfma(nh, nkv, d, bs, lens, new, window, seed=50, split_waves=split_waves,
                               num_splits=num_splits, waves=waves)
        return
    got, ref = run_attention_mfma(nh, nkv, d, bs, lens, new, window, seed=50, split_waves=split_waves,
                                  num_splits=num_splits, waves=waves)
    assert (got - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max())


@pytest.mark.parametrize("case", [(8, 2, 64, 16, [300, 64, 129, 1, 17, 600, 33, 90], 4, 8), (32, 4, 64, 16, [520], 8, 8),
                                  (64, 8, 128, 16, [700, 33], 2, 8), (3, 1, 32, 8, [1, 7, 40, 100], 3, 4),
                                  (6, 2, 80, 8, [70, 19, 300], 16, 4), (4, 4, 256, 16, [257, 31], 5, 4),
                                  (32, 1, 48, 8, [450, 2], 7, 8)])
def test_decode_shares_added_up_by_the_last_workgroup(case):
    """Decoding with the keys of a request shared out to workgroups: the shares are added up inside the kernel by
    the workgroup of each column group that finishes last (data handed over past the L2 of its XCD, a counter per
    group that is zero again afterwards).  The same bits as the second kernel gives, launch after launch, and when
    the launch is replayed from a graph."""
    nh, nkv, d, bs, lens, splits, waves = case
    new = [1] * len(lens)
    want, ref = run_attention_mfma(nh, nkv, d, bs, lens, new, seed=80, split_waves=True, num_splits=splits, waves=waves,
                                   merge_kernel=True)
    assert (want - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max())
    got, _ = run_attention_mfma(nh, nkv, d, bs, lens, new, seed=80, split_waves=True, num_splits=splits, waves=waves, repeat=5)
    assert torch.equal(got, want)
    from llmserve.ops import library

    assert int(library._arrival_counters(torch.device(DEV)).abs().sum()) == 0


def test_decode_shares_added_up_inside_a_replayed_graph():
    nh, nkv, d, bs, lens, splits = 8, 2, 64, 16, [300, 64, 129, 600], 4
    dtype = torch.bfloat16
    qs = [rnd(s, nh, d, seed=90 + 3 * b) for b, s in enumerate(lens)]
    ks = [rnd(s, nkv, d, seed=91 + 3 * b) for b, s in enumerate(lens)]
    vs = [rnd(s, nkv, d, seed=92 + 3 * b) for b, s in enumerate(lens)]
    qs, ks, vs = ([t.to(dtype) for t in ts] for ts in (qs, ks, vs))
    k_pool, v_pool, tables = make_paged(ks, vs, bs, dtype, seed=9)
    q = torch.cat([qs[b][-1:].reshape(1, nh * d) for b in range(len(lens))]).contiguous().to(DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    operands = (q, k_pool.to(DEV), v_pool.to(DEV), tables.to(DEV), i32(list(range(len(lens) + 1))), i32(lens))
    out = torch.empty(len(lens), nh * d, dtype=dtype, device=DEV)

    def launch(**kw):
        ops().attention_mfma(out, *operands, 0, len(lens), 1, 0, len(lens), nh, nkv, d, bs, 0, None, split_waves=True,
                             num_splits=splits, waves=8, **kw)

    launch(merge_kernel=True)
    want = out.clone()
    launch()  # (the counters exist from here on: a graph cannot make them)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
        launch()
    for _ in range(4):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
        launch()  # eager work between the replays
        assert torch.equal(out, want)


# The prompt kernel gives a wave two column groups (32 columns) up to head_dim 128, and every wave a twin for every
# other tile of keys, once the launch has a workgroup for each of the 256 CUs (two each for two column groups up to
# head_dim 64); the cases above are too small for that.
WIDE_LAUNCH_CASES = [  # nh, nkv, d, bs, lens, new, window
    (16, 16, 32, 8, [260, 200, 131, 97, 260, 33, 1, 17], [260, 200, 131, 97, 260, 33, 1, 17], 0),  # a second group without tokens
    (16, 4, 64, 16, [520, 300, 77, 515, 512, 511, 2, 64], [520, 300, 77, 100, 512, 31, 2, 64], 0),  # portions beside whole prompts
    (16, 16, 32, 8, [300, 290, 280, 31, 300, 47], [300, 290, 280, 31, 300, 16], 50),               # a window: no twins
    (16, 16, 128, 16, [300, 129, 128, 127, 33, 290, 150, 257], [300, 129, 128, 127, 33, 290, 7, 257], 0),
    (24, 8, 80, 8, [330, 190, 1, 64, 200, 326, 65, 200], [330, 190, 1, 64, 200, 3, 65, 200], 0),
    (16, 16, 160, 8, [300, 150, 17, 290, 300, 64, 300, 1], [300, 150, 17, 290, 300, 64, 300, 1], 0),  # one group, twins
]


@pytest.mark.parametrize("case", WIDE_LAUNCH_CASES)
def test_attention_mfma_launches_that_fill_the_chip(case):
    nh, nkv, d, bs, lens, new, window = case
    g = nh // nkv
    hg = min(g, 16)
    groups = -(-max(new) // (16 // hg))
    blocks = -(-groups // (8 if d <= 128 else 4))
    workgroups = blocks * nkv * -(-g // hg) * len(lens)
    assert workgroups >= 256, "this case would run without twins"
    got, ref = run_attention_mfma(nh, nkv, d, bs, lens, new, window, seed=55)
    assert (got - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max())


# One long prompt, or a long portion behind a prefix: every wave has a twin, and the blocks of tokens are handed out
# in an order of their own (the first workgroup of every CU takes one of the longest, shortest of these first).
# One or two column groups per wave, one or two workgroups per CU, pages of 8, 16, 24 and 32 (the block index is one
# multiply with a rounded-up reciprocal), a prompt that ends in the middle of a block, of a tile and of a page.
LONG_PROMPT_CASES = [  # nh, nkv, d, bs, len, new
    (32, 4, 64, 16, 2048, 2048),   # two column groups, two workgroups per CU, every CU's first workgroup in the fold
    (32, 4, 64, 16, 2093, 1500),   # the same behind a prefix, ends off every boundary
    (16, 16, 32, 8, 2100, 2100),   # one column group (too few blocks for two), 16 tokens per group
    (16, 16, 128, 32, 1100, 1100), # head_dim 128: one workgroup per CU
    (24, 8, 48, 24, 1571, 1571),   # pages of 24 keys, 3 heads per KV head
    (8, 8, 64, 16, 4111, 4111),    # more workgroups than run at once
]


@pytest.mark.parametrize("case", LONG_PROMPT_CASES)
def test_attention_mfma_one_long_prompt(case):
    nh, nkv, d, bs, length, new = case
    got, ref = run_attention_mfma(nh, nkv, d, bs, [length], [new], 0, seed=57)
    assert (got - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max())


def test_attention_mfma_long_prompt_finds_one_far_key_per_token():
    """Every query of a long prompt looks for one key of its own, far back or near, among two thousand: a block of
    tokens that took the wrong keys, a tile that its twin skipped or a page read twice would miss some."""
    length, nh, nkv, d = 2048, 32, 4, 64
    gen = torch.Generator().manual_seed(58)
    wanted = [int(torch.randint(0, t + 1, (1,), generator=gen)) for t in range(length)]  # key of token t, <= t

    def craft(qs, ks, vs):
        # dimension 0..10 of a key spell its index in +-1; a query spells the index it wants, scaled up, so that
        # the wanted key scores 11 * 40 and every other at most 9 * 40 (55 against 45 after the scaling by 1/8)
        bits = lambda i: torch.tensor([1.0 if (i >> b) & 1 else -1.0 for b in range(11)])  # noqa: E731
        for t in range(length):
            ks[0][t, :, :11] = bits(t)
            qs[0][t, :, :11] = 40.0 * bits(wanted[t])
            vs[0][t] = 0.0
            vs[0][t, :, 0] = float(t % 128)
        ks[0][:, :, 11:] *= 0.1

    got, ref = run_attention_mfma(nh, nkv, d, 16, [length], [length], 0, seed=59, craft=craft)
    value = got.view(length, nh, d)[:, :, 0]
    want = torch.tensor([float(w % 128) for w in wanted]).unsqueeze(1).expand(length, nh)
    assert (value - want).abs().max() <= 0.51, "a token did not find its key"
    assert (got - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max())


@pytest.mark.parametrize("arrangement", [(False, 1, 4), (False, 3, 4), (True, 1, 4), (True, 3, 4), (True, 1, 8)])
@pytest.mark.parametrize("needle", [0, 15, 16, 31, 32, 299, 300 - 17, 141])
def test_attention_mfma_finds_one_far_key(needle, arrangement):
    def craft(qs, ks, vs):
        qs[0][-1] = 0
        qs[0][-1, :, 0] = 12.0
        ks[0][:, :, 0] = 0
        ks[0][needle, :, 0] = 12.0
        vs[0][needle] = 3.0

    got, ref = run_attention_mfma(8, 2, 64, 16, [300], [1], 0, seed=60, craft=craft, split_waves=arrangement[0],
                                  num_splits=arrangement[1], waves=arrangement[2])
    assert (got - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max()) and got.mean() > 2.9


# The kernels keep 64 page ids of a request in registers and fetch the next 64 when a tile leaves them: contexts
# of more than 64 pages (once and twice over), where random weights would hide a wrong page among hundreds.
LONG_CASES = [  # nh, nkv, d, bs, lens, new
    (8, 2, 64, 8, [700], [1]),           # 88 pages: decoding across one refill
    (4, 1, 32, 8, [1100], [1]),          # 138 pages: two refills
    (8, 2, 64, 16, [2300], [1]),         # 144 pages of 16
    (4, 2, 64, 8, [900], [300]),         # a portion of a long prompt: early and late blocks, refills on the way
    (4, 4, 128, 8, [640, 530], [640, 2]),  # a whole prompt of 80 pages beside the end of another
]


@pytest.mark.parametrize("arrangement", [(False, 1, 4), (False, 4, 4), (True, 1, 4), (True, 1, 8), (True, 4, 8), (True, 7, 4)])
@pytest.mark.parametrize("case", LONG_CASES)
def test_attention_mfma_long_contexts(case, arrangement):
    nh, nkv, d, bs, lens, new = case
    split_waves, num_splits, waves = arrangement
    got, ref = run_attention_mfma(nh, nkv, d, bs, lens, new, 0, seed=70, split_waves=split_waves,
                                  num_splits=num_splits, waves=waves)
    assert (got - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max())


@pytest.mark.parametrize("arrangement", [(False, 1, 4), (False, 3, 4), (True, 1, 8), (True, 3, 8)])
@pytest.mark.parametrize("needle", [0, 511, 512, 519, 520, 1023, 1024, 1090])
def test_attention_mfma_finds_one_key_beyond_the_first_pages(needle, arrangement):
    """1,100 keys in pages of 8: the one key that matters lies before, at and after the places where the
    page ids in registers are exchanged (keys 512 and 1024)."""
    def craft(qs, ks, vs):
        qs[0][-1] = 0
        qs[0][-1, :, 0] = 12.0
        ks[0][:, :, 0] = 0
        ks[0][needle, :, 0] = 12.0
        vs[0][needle] = 3.0

    got, ref = run_attention_mfma(4, 1, 32, 8, [1100], [1], 0, seed=71, craft=craft, split_waves=arrangement[0],
                                  num_splits=arrangement[1], waves=arrangement[2])
    assert (got - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max()) and got.mean() > 2.9


def test_attention_mfma_window_edge():
    for needle, inside in ((100 - 8, False), (100 - 7, True)):
        def craft(qs, ks, vs):
            qs[0][-1] = 0
            qs[0][-1, :, 1] = 10.0
            ks[0][:, :, 1] = 0
            ks[0][needle, :, 1] = 10.0
            vs[0][needle] = 5.0

        for split_waves in (False, True):
            got, ref = run_attention_mfma(2, 1, 32, 8, [101], [1], 8, seed=61, craft=craft, split_waves=split_waves)
            assert (got - ref).abs().max() <= 2.0 ** -7 * float(ref.abs().max())
            assert (got.mean() > 4.0) == inside


def test_attention_mfma_refuses_what_it_cannot_take():
    assert not ops().attention_mfma_supported(torch.bfloat16, 64, 4)
    assert not ops().attention_mfma_supported(torch.bfloat16, 40, 16)
    assert not ops().attention_mfma_supported(torch.float32, 64, 16)
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)  # noqa: E731
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    with pytest.raises(ValueError, match="multiple of 8"):
        ops().attention_mfma(z(1, 64), z(1, 64), z(2, 1, 4, 64), z(2, 1, 64, 4), i32([[0]]), i32([0, 1]), i32([1]),
                             0, 1, 1, 0, 1, 1, 1, 64, 4)
