"""Each kernel alone against a plain torch float32 reference of the same operation, at sizes
other than the engine tests' (odd widths, tails that do not fill a tile, many heads)."""

from __future__ import annotations

import math

import numpy as np
import pytest
import torch

from prefixserve_amd.engine.batch import GroupMeta, StepItem, StepPacker

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from prefixserve_amd.kernels.ops import HipOps
    from prefixserve_amd.parts.base import Workspace

    return HipOps(torch.device(DEV), Workspace(torch.device(DEV)))


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype).to(DEV)


def rel(got, want):
    return float((got.float() - want.float()).abs().max() / want.float().abs().max())


# ------------------------------------------------------------------ elementwise

@pytest.mark.parametrize("table_dtype", [torch.float32, torch.bfloat16])
def test_embed(ops, table_dtype):
    table = rnd(301, 72, dtype=table_dtype)
    ids = torch.tensor([0, 300, 5, 5, 17], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 72, device=DEV)
    ops.embed(ids, table, out)
    assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [72, 2048, 1000])
def test_add_rmsnorm(ops, act, wdt, hidden):
    t, eps = 7, 1e-5
    res = rnd(t, hidden, seed=1)
    delta = rnd(t, hidden, dtype=act, seed=2)
    w = (1 + 0.1 * rnd(hidden, seed=3)).to(wdt)
    want_res = res + delta.float()
    want = w.float() * want_res * torch.rsqrt((want_res ** 2).mean(-1, keepdim=True) + eps)
    out = torch.empty(t, hidden, dtype=act, device=DEV)
    r = res.clone()
    ops.add_rmsnorm(r, delta, w, eps, out)
    assert torch.equal(r, want_res)                                 # the residual sum is 32-bit
    assert rel(out, want) < (1e-6 if act == torch.float32 else 5e-3)
    r2 = res.clone()
    ops.add_rmsnorm(r2, None, w, eps, out)                          # first layer: nothing to add
    assert torch.equal(r2, res)
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    out3 = torch.empty(3, hidden, dtype=act, device=DEV)
    r3 = res.clone()
    ops.add_rmsnorm_rows(r3, delta, rows, w, eps, out3)
    assert torch.equal(r3, res) and rel(out3, want[rows.long()]) < (1e-6 if act == torch.float32 else 5e-3)


@pytest.mark.parametrize("hidden", [96, 2048, 5000])
def test_add_rmsnorm_sums_partial_slices(ops, hidden):
    t, eps = 5, 1e-6
    res = rnd(t, hidden, seed=1)
    parts = rnd(3, t, hidden, seed=2)
    w = (1 + 0.1 * rnd(hidden, seed=3)).to(torch.bfloat16)
    want_res = res + parts[0] + parts[1] + parts[2]
    want = w.float() * want_res * torch.rsqrt((want_res ** 2).mean(-1, keepdim=True) + eps)
    out = torch.empty(t, hidden, dtype=torch.bfloat16, device=DEV)
    r = res.clone()
    ops.add_rmsnorm(r, parts, w, eps, out)
    assert torch.equal(r, want_res) and rel(out, want) < 5e-3
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, hidden, dtype=torch.bfloat16, device=DEV)
    r2 = res.clone()
    ops.add_rmsnorm_rows(r2, parts, rows, w, eps, out2)
    assert torch.equal(r2, res) and rel(out2, want[rows.long()]) < 5e-3


def test_rmsnorm_zero_row_and_eps(ops):
    res = torch.zeros(2, 64, device=DEV)
    res[1] = 1e-4
    out = torch.empty(2, 64, device=DEV)
    ops.add_rmsnorm(res, None, torch.ones(64, device=DEV), 1e-6, out)
    assert torch.all(out[0] == 0) and torch.isfinite(out).all()
    assert abs(float(out[1, 0]) - 1e-4 / math.sqrt(1e-8 + 1e-6)) < 1e-7


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_swiglu(ops, act):
    gu = rnd(9, 2 * 344, dtype=act, scale=2.0)
    out = torch.empty(9, 344, dtype=act, device=DEV)
    ops.swiglu(gu, out)
    want = torch.nn.functional.silu(gu[:, :344].float()) * gu[:, 344:].float()
    assert rel(out, want) < (1e-6 if act == torch.float32 else 5e-3)


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,d", [(6, 3, 48), (5, 5, 16), (16, 2, 128)])
def test_rope_kv_append(ops, act, hq, hkv, d):
    from prefixserve_amd.parts.rope import rope_inv_freq

    t, blocks = 11, 6
    qkv = rnd(t, (hq + 2 * hkv) * d, dtype=act)
    pos = torch.tensor([0, 1, 2, 15, 16, 17, 40, 41, 70, 5, 33], dtype=torch.int32, device=DEV)
    inv = rope_inv_freq(d, 10000.0, None)
    ang = torch.outer(torch.arange(96, dtype=torch.float32), inv).double()
    table = torch.stack((ang.cos(), ang.sin()), -1).float().to(DEV).contiguous()
    slots = torch.tensor([p % 16 + 16 * ((p // 16 * 5 + 1) % blocks) for p in pos.tolist()], dtype=torch.int32, device=DEV)
    kv = torch.full((blocks, 2, hkv, 16 * d), 7.0, dtype=act, device=DEV)
    src = qkv.clone().float()
    ops.rope_kv_append(qkv, hq, hkv, d, pos, table, kv, slots)
    x = src[:, : (hq + hkv) * d].view(t, hq + hkv, d)
    cs = table[pos.long()]
    cos, sin = cs[..., 0][:, None], cs[..., 1][:, None]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    want = torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), -1)
    got = qkv[:, : (hq + hkv) * d].view(t, hq + hkv, d)
    assert rel(got, want) < (1e-6 if act == torch.float32 else 5e-3)
    assert torch.equal(qkv[:, (hq + hkv) * d:].float(), src[:, (hq + hkv) * d:])            # v untouched
    kp = kv[:, 0].view(blocks, hkv, 16, d)
    vp = kv[:, 1].view(blocks, hkv, d, 16)
    page, off = (slots // 16).long(), (slots % 16).long()
    assert torch.equal(kp[page, :, off, :], got[:, hq:])            # pages hold exactly what was rotated
    assert torch.equal(vp[page, :, :, off].float(), src[:, (hq + hkv) * d:].view(t, hkv, d))
    untouched = torch.ones(blocks, 16, dtype=torch.bool)
    untouched[page.cpu(), off.cpu()] = False
    assert torch.all(kp.permute(0, 2, 1, 3)[untouched.to(DEV)] == 7.0)                      # nothing else written
    q2 = src.clone().to(act)
    ops.rope_kv_append(q2, hq, hkv, d, pos, None, None, slots)     # no table, no cache: a no-op
    assert torch.equal(q2.float(), src.to(act).float())


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 64), (6, 3, 48), (24, 8, 128), (2, 1, 16)])
def test_rope_kv_append_of_whole_pages(ops, hq, hkv, d):
    """The tokens of prompts as a step brings them: one of 53 tokens over pages 4, 1, 5, 2 (three
    whole pages in order and five tokens), one of 30 tokens that starts three slots into page 3
    and so lies across the groups of 16 tokens the kernel works in, 13 tokens, then a whole page
    again; every slot nobody wrote keeps what it held."""
    from prefixserve_amd.parts.rope import rope_inv_freq

    blocks = 9
    slots = [16 * [4, 1, 5, 2][p // 16] + p % 16 for p in range(53)] + \
            [16 * [3, 6, 7][(p + 3) // 16] + (p + 3) % 16 for p in range(30)] + [16 * 8 + p for p in range(16)]
    pos = list(range(53)) + list(range(3, 33)) + list(range(16))
    # 13 more tokens in front of the last page, so that it starts a group of 16 of the step's tokens
    slots = slots[:83] + [16 * 0 + p for p in range(13)] + slots[83:]
    pos = pos[:83] + list(range(13)) + pos[83:]
    t = len(slots)
    assert t == 112 and len(set(slots)) == t
    qkv = rnd(t, (hq + 2 * hkv) * d, dtype=torch.bfloat16, seed=3)
    src = qkv.clone().float()
    inv = rope_inv_freq(d, 10000.0, None)
    ang = torch.outer(torch.arange(64, dtype=torch.float32), inv).double()
    table = torch.stack((ang.cos(), ang.sin()), -1).float().to(DEV).contiguous()
    kv = torch.full((blocks, 2, hkv, 16 * d), 7.0, dtype=torch.bfloat16, device=DEV)
    pos_t = torch.tensor(pos, dtype=torch.int32, device=DEV)
    slots_t = torch.tensor(slots, dtype=torch.int32, device=DEV)
    ops.rope_kv_append(qkv, hq, hkv, d, pos_t, table, kv, slots_t)
    got = qkv[:, : (hq + hkv) * d].view(t, hq + hkv, d)
    kp = kv[:, 0].view(blocks, hkv, 16, d)
    vp = kv[:, 1].view(blocks, hkv, d, 16)
    page, off = (slots_t // 16).long(), (slots_t % 16).long()
    assert torch.equal(kp[page, :, off, :], got[:, hq:])
    assert torch.equal(vp[page, :, :, off].float(), src[:, (hq + hkv) * d:].view(t, hkv, d))
    untouched = torch.ones(blocks, 16, dtype=torch.bool)
    untouched[page.cpu(), off.cpu()] = False
    assert untouched.sum() == blocks * 16 - t
    assert torch.all(kp.permute(0, 2, 1, 3)[untouched.to(DEV)] == 7.0) and torch.all(vp.permute(0, 3, 1, 2)[untouched.to(DEV)] == 7.0)


@pytest.mark.parametrize("m", [1, 8, 17, 40, 64])
@pytest.mark.parametrize("hq,hkv,d,k", [(6, 3, 48, 72), (4, 2, 16, 64), (32, 8, 64, 2048), (3, 1, 32, 96), (2, 2, 128, 200),
                                        (32, 8, 128, 264), (50, 1, 128, 72)])   # enough tiles for two per workgroup
def test_fused_qkv_rope_append_equals_the_separate_kernels(ops, m, hq, hkv, d, k):
    """One kernel for projection + rotation + cache write (small steps) against the product
    followed by rope_kv_append, and against float64."""
    from prefixserve_amd.parts.rope import rope_inv_freq

    blocks = 12
    x = rnd(m, k, dtype=torch.bfloat16, seed=1)
    w = rnd((hq + 2 * hkv) * d, k, dtype=torch.bfloat16, seed=2, scale=0.1)
    pos = torch.tensor([(7 * i + 3) % 150 for i in range(m)], dtype=torch.int32, device=DEV)
    slots = torch.tensor(np.random.default_rng(m).permutation(blocks * 16)[:m].tolist(), dtype=torch.int32, device=DEV)
    ang = torch.outer(torch.arange(150, dtype=torch.float32), rope_inv_freq(d, 10000.0, None)).double()
    table = torch.stack((ang.cos(), ang.sin()), -1).float().to(DEV).contiguous()
    n = (hq + 2 * hkv) * d
    kv_a = torch.full((blocks, 2, hkv, 16 * d), 3.0, dtype=torch.bfloat16, device=DEV)
    kv_b = kv_a.clone()
    fused = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops.qkv_rope_append(x, w, fused, hq, hkv, d, pos, table, kv_a, slots)
    plain = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops.linear(x, w, plain)
    ops.rope_kv_append(plain, hq, hkv, d, pos, table, kv_b, slots)
    # float64 truth
    y = (x.double() @ w.double().T)
    z = y[:, : (hq + hkv) * d].view(m, hq + hkv, d)
    cs = table[pos.long()].double()
    cos, sin = cs[..., 0][:, None], cs[..., 1][:, None]
    z1, z2 = z[..., : d // 2], z[..., d // 2:]
    want = torch.cat((torch.cat((z1 * cos - z2 * sin, z2 * cos + z1 * sin), -1).reshape(m, -1), y[:, (hq + hkv) * d:]), 1)
    assert rel(fused, want) < 5e-3 and rel(plain, want) < 1e-2
    page, off = (slots // 16).long(), (slots % 16).long()
    kp = kv_a[:, 0].view(blocks, hkv, 16, d)
    vp = kv_a[:, 1].view(blocks, hkv, d, 16)
    assert torch.equal(kp[page, :, off, :].reshape(m, -1), fused[:, hq * d:(hq + hkv) * d])      # pages hold what q/k/v hold
    assert torch.equal(vp[page, :, :, off].reshape(m, -1), fused[:, (hq + hkv) * d:])
    assert rel(kv_a.float(), kv_b.float()) < 1e-2
    touched = torch.zeros(blocks, 16, dtype=torch.bool, device=DEV)
    touched[page, off] = True
    assert torch.all(kp.permute(0, 2, 1, 3)[~touched] == 3.0) and torch.all(vp.permute(0, 3, 1, 2)[~touched] == 3.0)


# --------------------------------------------------------------------- products

@pytest.mark.parametrize("m,n,k", [(1, 100, 72), (3, 64, 16), (17, 257, 96), (130, 70, 200), (64, 128, 64),
                                   (2, 7, 2048), (8, 1001, 1000), (9, 1001, 1000), (5, 33, 70), (8, 3, 4)])
def test_linear_float32_is_exact_fp32(ops, m, n, k):
    x, w = rnd(m, k, seed=1), rnd(n, k, seed=2)
    out = torch.empty(m, n, device=DEV)
    ops.linear(x, w, out)
    want = (x.double() @ w.double().T)
    # One rounding per term, summed in order: the error grows like sqrt(k) * 2^-24. A
    # reduced-precision mode would give ~1e-3.
    assert rel(out, want) < max(2e-6, 1.2e-7 * k ** 0.5)


@pytest.mark.parametrize("n,k", [(100, 72), (257, 2048), (33, 4), (3072, 200)])
def test_linear_float32_does_not_depend_on_the_row_count(ops, n, k):
    """The kernel for a few rows and the tiled kernel sum in one order: bit for bit the same."""
    x, w = rnd(40, k, seed=1), rnd(n, k, seed=2)
    big = torch.empty(40, n, device=DEV)
    ops.linear(x, w, big)
    for m in (1, 3, 16, 17):
        small = torch.full((m + 1, n), 7.0, device=DEV)
        ops.linear(x[:m], w, small[:m])
        assert torch.equal(small[:m], big[:m]) and torch.all(small[m] == 7.0), f"{m} rows"


@pytest.mark.parametrize("m", [1, 2, 7, 16, 17, 33, 64])
@pytest.mark.parametrize("n,k", [(48, 64), (1000, 96), (129, 2048), (16, 8), (250, 72)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_linear_bf16_small_m(ops, m, n, k, out_dtype):
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.1)
    out = torch.empty(m, n, dtype=out_dtype, device=DEV)
    ops.linear(x, w, out)
    want = x.double() @ w.double().T
    assert rel(out, want) < (1e-5 if out_dtype == torch.float32 else 5e-3)


@pytest.mark.parametrize("m", [1, 3, 5, 8, 9, 16, 31, 48, 64])
@pytest.mark.parametrize("n,k", [(65536 + 40, 72), (32768 + 24, 2048), (32768 + 200, 96), (32768 + 16, 1024), (32768 + 32, 4096)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_linear_bf16_very_many_columns(ops, m, n, k, out_dtype):
    """The forms the output matrix takes: up to 8 tokens one or two row tiles per workgroup of
    eight waves that split K, from 9 tokens on more row tiles per wave; where K is a multiple of
    32, from 2 or 4 to 16 tokens, workgroups that keep the tokens in LDS (8 or 16 rows, one or
    two row tiles per group, a K so small that some waves have no step, a K of two rounds of
    steps per wave). Row counts that are no multiple of the largest group of tiles (an odd
    number of tiles among them), a K with a partial last step and a K that gives every wave
    eight steps."""
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.1)
    out = torch.full((m + 1, n), 7.0, dtype=out_dtype, device=DEV)
    ops.linear(x, w, out[:m])
    assert rel(out[:m], x.double() @ w.double().T) < (1e-5 if out_dtype == torch.float32 else 5e-3)
    assert torch.all(out[m] == 7.0)


@pytest.mark.parametrize("m", [1, 8, 33, 64])
@pytest.mark.parametrize("n,k", [(2048, 2048), (200, 8192), (72, 2056), (256, 2744), (72, 520), (256, 688)])
def test_linear_to_residual_splits_k(ops, m, n, k):
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    out = ops.linear_to_residual(x, w, "test.delta")
    split = ops.lib.psamd_linear_skinny_ksplit(m, n, k)
    assert split > 1 or k < 1024                      # these shapes do split, but for a short K (a wave wants about eight k-steps)
    if split > 1:
        assert out.dim() == 3 and out.dtype == torch.float32 and out.shape[0] == split
        assert rel(out.sum(0), x.double() @ w.double().T) < 1e-5
    else:
        assert out.dim() == 2 and rel(out, x.double() @ w.double().T) < 5e-3
    small = ops.linear_to_residual(x[:, :64].contiguous(), w[:, :64].contiguous(), "test.delta2")
    assert small.dim() == 2 and small.dtype == torch.bfloat16                      # too little K to split


@pytest.mark.parametrize("m", [3, 4, 5, 8, 9, 13, 16, 17])
@pytest.mark.parametrize("n,k", [(2048, 8192), (2064, 4128), (3080, 8192), (4096, 4096), (1024 + 8, 9024)])
def test_linear_to_residual_by_workgroups_that_stay(ops, m, n, k):
    """From 4 to 16 tokens, a K-split product with two or more groups of row tiles per workgroup
    goes to workgroups that keep their slice of the tokens in LDS (8 or 16 rows) and walk through
    their groups: K-slices of unequal length, a row count that is no multiple of 16, and token
    counts on either side of that form's range."""
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=3), rnd(n, k, dtype=torch.bfloat16, seed=4, scale=0.05)
    out = ops.linear_to_residual(x, w, "test.delta3")
    assert out.dim() == 3 and out.dtype == torch.float32
    assert torch.isfinite(out).all()
    assert rel(out.sum(0), x.double() @ w.double().T) < 1e-5


# ---- small steps without norm kernels: products that add into the residual stream, and products
# ---- that normalize the rows they read

def _rms_rows(resid, weight, eps):
    x = resid.double()
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * weight.double()


@pytest.mark.parametrize("m", [1, 3, 4, 8, 9, 16])
@pytest.mark.parametrize("n,k", [(2048, 2048), (2048, 8192), (200, 96), (2064, 4128), (4096, 14336), (72, 520), (3072, 8192)])
def test_linear_to_residual_adds_into_the_stream(ops, m, n, k):
    """Up to 16 tokens: every K-slice adds its partial sums into the float32 residual itself
    (float atomics), whatever was there before; twice in a row adds twice. Rows after the last
    token are not touched."""
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    start = rnd(m + 1, n, seed=3)
    resid = start.clone()
    if not ops.fuses_norm(m, n, torch.bfloat16):
        # a width the kernels that normalize their rows do not take (no whole 32-wide k-steps, or rows
        # that do not fit LDS): the product is handed back and the stream left alone
        out = ops.linear_to_residual(x, w, "test.add", resid[:m])
        assert out is not None and torch.equal(resid, start)
        assert rel(out.sum(0) if out.dim() == 3 else out, x.double() @ w.double().T) < 5e-3
        return
    assert ops.linear_to_residual(x, w, "test.add", resid[:m]) is None
    prod = x.double() @ w.double().T
    assert rel(resid[:m].double() - start[:m].double(), prod) < 1e-5
    assert ops.linear_to_residual(x, w, "test.add", resid[:m]) is None
    assert rel(resid[:m].double() - start[:m].double(), 2 * prod) < 1e-5
    assert torch.equal(resid[m], start[m])
    # a step too large for it hands back what is to be added, as before
    big = rnd(17, k, dtype=torch.bfloat16, seed=4)
    out = ops.linear_to_residual(big, w, "test.add2", torch.zeros(17, n, device=DEV))
    assert out is not None and rel(out.sum(0) if out.dim() == 3 else out, big.double() @ w.double().T) < 5e-3


@pytest.mark.parametrize("m,n,k", [(1024, 2048, 2048), (2100, 2048, 8192), (1030, 200, 96), (1500, 3072, 8192)])
def test_linear_to_residual_of_a_large_step_adds_in_the_library(ops, m, n, k):
    """From 1,024 tokens on the library's product adds into the float32 residual itself (its sums
    reach the stream unrounded); twice in a row adds twice, rows behind the step stay as they
    were, and without the stream, or without the library, the product is handed back."""
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.05)
    start = rnd(m + 1, n, seed=3)
    resid = start.clone()
    prod = x.double() @ w.double().T
    assert ops.linear_to_residual(x, w, "test.big", resid[:m]) is None
    assert rel(resid[:m].double() - start[:m].double(), prod) < 2e-6
    assert ops.linear_to_residual(x, w, "test.big", resid[:m]) is None
    assert rel(resid[:m].double() - start[:m].double(), 2 * prod) < 2e-6
    assert torch.equal(resid[m], start[m])
    out = ops.linear_to_residual(x, w, "test.big", None)
    assert out is not None and out.dtype == torch.bfloat16 and rel(out, prod) < 5e-3
    ops._direct_library = False
    try:
        out = ops.linear_to_residual(x, w, "test.big", resid[:m])
    finally:
        ops._direct_library = True
    assert out is not None and rel(out, prod) < 5e-3


@pytest.mark.parametrize("m", [1, 2, 5, 8, 9, 16])
@pytest.mark.parametrize("n,k,epilogue,out_dtype,wdt", [
    (8192, 2048, 1, torch.bfloat16, torch.bfloat16),      # gate/up of the 1B shape: 512 pairs of tiles
    (14336, 4096, 1, torch.bfloat16, torch.bfloat16),     # of the 8B shape: 896 pairs, workgroups that stay for several
    (344, 96, 1, torch.bfloat16, torch.float32),          # a pair count that is no multiple of anything, 32-bit norm weight
    (66000, 2048, 0, torch.float32, torch.bfloat16),      # the output matrix: two row tiles per group
    (33000, 4096, 0, torch.float32, torch.float32),       # one row tile per group
    (1001, 160, 0, torch.bfloat16, torch.bfloat16),       # bfloat16 output, a partial last tile
    (257, 64, 0, torch.float32, torch.bfloat16),
])
def test_products_that_normalize_the_rows_they_read(ops, m, n, k, epilogue, out_dtype, wdt):
    """x is handed over as rows of the float32 residual stream with their RMS norm still to be
    applied; the kernel applies it while it stages the rows. Against float64, with rows picked
    by an index list (as the logits' rows are) and in order, a norm weight in either dtype, an
    eps that matters (one row is tiny) and a row of zeros."""
    from prefixserve_amd.parts.base import NormedRows

    t = m + 5
    resid = rnd(t, k, seed=5, scale=3.0)
    resid[1] *= 1e-4                                   # eps decides this row's scale
    resid[2] = 0.0
    weight = (1.0 + 0.1 * torch.randn(k, generator=torch.Generator().manual_seed(6))).to(wdt).to(DEV)
    eps = 1e-5
    rows_list = [int(i) for i in np.random.default_rng(m).permutation(t)[:m]]
    if m >= 3:
        rows_list[0], rows_list[1] = 1, 2
    rows = torch.tensor(rows_list, dtype=torch.int32, device=DEV)
    w = rnd((2 if epilogue else 1) * n, k, dtype=torch.bfloat16, seed=7, scale=0.05)
    for idx in (rows, None):
        src = resid if idx is not None else resid[:m].contiguous()
        x = NormedRows(src, weight, eps, torch.bfloat16, idx)
        out = torch.full((m + 1, n), 7.0, dtype=out_dtype, device=DEV)
        normed = _rms_rows(src[idx.long()] if idx is not None else src, weight, eps)
        y = normed @ w.double().T
        if epilogue:
            ops.linear_swiglu(x, w, out[:m])
            y = torch.nn.functional.silu(y[:, :n]) * y[:, n:]
        else:
            ops.linear(x, w, out[:m])
        assert torch.all(out[m] == 7.0)
        # the tokens are rounded to bfloat16 once, as the norm kernel's output is
        for i in range(m):
            scale = float(y[i].abs().max())
            if scale == 0.0:
                assert float(out[i].abs().max()) == 0.0
            else:
                assert float((out[i].double() - y[i]).abs().max()) < 1e-2 * scale, f"row {i}"
    # and the same through the norm kernel, for a step the fused form does not take
    x = NormedRows(resid, weight, eps, torch.bfloat16, None)
    assert ops.normed(x).shape == (t, k) and rel(ops.normed(x), _rms_rows(resid, weight, eps)) < 5e-3


@pytest.mark.parametrize("m", [1, 5, 8, 9, 16])
@pytest.mark.parametrize("hq,hkv,d,k", [(32, 8, 64, 2048), (4, 2, 16, 64), (3, 1, 32, 96), (32, 8, 128, 4096), (50, 1, 128, 64),
                                        (6, 3, 48, 160)])
def test_qkv_rope_append_that_normalizes_its_rows(ops, m, hq, hkv, d, k):
    """q/k/v + rotation + cache write reading the residual stream and normalizing it itself,
    against float64 and against the norm kernel followed by the kernel that takes tokens."""
    from prefixserve_amd.parts.base import NormedRows
    from prefixserve_amd.parts.rope import rope_inv_freq

    blocks = 12
    resid = rnd(m, k, seed=1, scale=2.0)
    weight = (1.0 + 0.1 * torch.randn(k, generator=torch.Generator().manual_seed(2))).to(torch.bfloat16).to(DEV)
    eps = 1e-6
    w = rnd((hq + 2 * hkv) * d, k, dtype=torch.bfloat16, seed=2, scale=0.1)
    pos = torch.tensor([(7 * i + 3) % 150 for i in range(m)], dtype=torch.int32, device=DEV)
    slots = torch.tensor(np.random.default_rng(m).permutation(blocks * 16)[:m].tolist(), dtype=torch.int32, device=DEV)
    ang = torch.outer(torch.arange(150, dtype=torch.float32), rope_inv_freq(d, 10000.0, None)).double()
    table = torch.stack((ang.cos(), ang.sin()), -1).float().to(DEV).contiguous()
    n = (hq + 2 * hkv) * d
    kv_a = torch.full((blocks, 2, hkv, 16 * d), 3.0, dtype=torch.bfloat16, device=DEV)
    kv_b = kv_a.clone()
    fused = torch.full((m + 1, n), 7.0, dtype=torch.bfloat16, device=DEV)
    assert ops.fuses_norm(m, k, torch.bfloat16)
    ops.qkv_rope_append(NormedRows(resid, weight, eps, torch.bfloat16), w, fused[:m], hq, hkv, d, pos, table, kv_a, slots)
    xn = torch.empty(m, k, dtype=torch.bfloat16, device=DEV)
    ops.add_rmsnorm(resid.clone(), None, weight, eps, xn)
    plain = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    ops.qkv_rope_append(xn, w, plain, hq, hkv, d, pos, table, kv_b, slots)
    y = _rms_rows(resid, weight, eps) @ w.double().T
    z = y[:, : (hq + hkv) * d].view(m, hq + hkv, d)
    cs = table[pos.long()].double()
    cos, sin = cs[..., 0][:, None], cs[..., 1][:, None]
    z1, z2 = z[..., : d // 2], z[..., d // 2:]
    want = torch.cat((torch.cat((z1 * cos - z2 * sin, z2 * cos + z1 * sin), -1).reshape(m, -1), y[:, (hq + hkv) * d:]), 1)
    assert rel(fused[:m], want) < 1e-2 and rel(plain, want) < 1e-2 and torch.all(fused[m] == 7.0)
    page, off = (slots // 16).long(), (slots % 16).long()
    kp = kv_a[:, 0].view(blocks, hkv, 16, d)
    vp = kv_a[:, 1].view(blocks, hkv, d, 16)
    assert torch.equal(kp[page, :, off, :].reshape(m, -1), fused[:m, hq * d:(hq + hkv) * d])
    assert torch.equal(vp[page, :, :, off].reshape(m, -1), fused[:m, (hq + hkv) * d:])
    assert rel(kv_a.float(), kv_b.float()) < 2e-2
    touched = torch.zeros(blocks, 16, dtype=torch.bool, device=DEV)
    touched[page, off] = True
    assert torch.all(kp.permute(0, 2, 1, 3)[~touched] == 3.0) and torch.all(vp.permute(0, 3, 1, 2)[~touched] == 3.0)


@pytest.mark.parametrize("m", [3, 4, 7, 8, 9])
@pytest.mark.parametrize("inter,k", [(12288 + 40, 4096), (12288, 4128)])
def test_linear_swiglu_by_workgroups_that_stay(ops, m, inter, k):
    """Gate/up with K from 4,096 on and 768 or more pairs of tiles, 4 to 8 tokens."""
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(2 * inter, k, dtype=torch.bfloat16, seed=2, scale=0.03)
    out = torch.full((m + 1, inter), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.linear_swiglu(x, w, out[:m])
    gu = x.double() @ w.double().T
    want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    assert rel(out[:m], want) < 1e-2 and torch.all(out[m] == 7.0)


@pytest.mark.parametrize("m,n,k", [(65, 300, 96), (200, 64, 2048), (3, 50, 70)])
def test_linear_bf16_other_paths(ops, m, n, k):
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.1)
    for out_dtype in (torch.bfloat16, torch.float32):
        out = torch.empty(m, n, dtype=out_dtype, device=DEV)
        ops.linear(x, w, out)
        assert rel(out, x.double() @ w.double().T) < (2e-5 if out_dtype == torch.float32 else 5e-3)


def test_library_product_called_directly_and_through_torch(ops):
    """Large bfloat16 products go to hipBLASLt through the kernel library's own call (plans kept
    per shape); torch.mm is what remains if the library cannot be found. Both against float64,
    and a shape seen twice (the second call takes the kept plan)."""
    assert ops._direct_library, "hipBLASLt was not found in the process"
    for m, n, k in [(65, 300, 96), (512, 2048, 2048), (200, 64, 2048), (65, 300, 96)]:
        x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(n, k, dtype=torch.bfloat16, seed=2, scale=0.1)
        want = x.double() @ w.double().T
        direct = torch.full((m + 1, n), 7.0, dtype=torch.bfloat16, device=DEV)
        ops.linear(x, w, direct[:m])
        assert rel(direct[:m], want) < 5e-3 and torch.all(direct[m] == 7.0)
        ops._direct_library = False
        try:
            through_torch = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
            ops.linear(x, w, through_torch)
        finally:
            ops._direct_library = True
        assert rel(through_torch, want) < 5e-3
        for through_library in (True, False):                         # float32 out: more than 64 rows of logits
            ops._direct_library = through_library
            try:
                logits = torch.full((m + 1, n), 7.0, dtype=torch.float32, device=DEV)
                ops.linear(x, w, logits[:m])
            finally:
                ops._direct_library = True
            assert rel(logits[:m], want) < 2e-5 and torch.all(logits[m] == 7.0)


@pytest.mark.parametrize("m", [1, 5, 64, 100])
@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_linear_swiglu(ops, m, act):
    k, inter = 96, 344
    x, w = rnd(m, k, dtype=act, seed=1), rnd(2 * inter, k, dtype=act, seed=2, scale=0.2)
    out = torch.empty(m, inter, dtype=act, device=DEV)
    ops.linear_swiglu(x, w, out)
    gu = x.double() @ w.double().T
    want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    assert rel(out, want) < (2e-6 if act == torch.float32 else 1e-2)


@pytest.mark.parametrize("m", [8, 9, 16, 31, 48, 64])
@pytest.mark.parametrize("inter", [12800 + 40, 6400 + 40])
def test_linear_swiglu_wide(ops, m, inter):
    """An intermediate size with 800 or more tiles of gate/up pairs takes four pairs per wave from
    9 tokens on, one with 400 or more two pairs at 9 to 16 tokens; sizes that are no multiple of
    the rows of such a group, a K with a partial last step."""
    k = 72
    x, w = rnd(m, k, dtype=torch.bfloat16, seed=1), rnd(2 * inter, k, dtype=torch.bfloat16, seed=2, scale=0.2)
    gu = x.double() @ w.double().T
    want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    # above 32 tokens the library's product and the activation kernel stand in where the library
    # is found; the fused form is what remains without it, so both are run
    for through_library in ((True, False) if m > ops.FUSED_SWIGLU_MAX_ROWS else (True,)):
        ops._direct_library = through_library
        try:
            out = torch.full((m + 1, inter), 7.0, dtype=torch.bfloat16, device=DEV)
            ops.linear_swiglu(x, w, out[:m])
        finally:
            ops._direct_library = True
        assert rel(out[:m], want) < 1e-2 and torch.all(out[m] == 7.0)


# -------------------------------------------------------------------- attention

def paged_case(ops, act, hq, hkv, d, lens_new, lens_old, window=None, seed=0, num_blocks=64, poison=1e30, give_back=False):
    """Random q/k/v for items with ``old`` cached and ``new`` fresh tokens each, pages from a
    random permutation; returns (kernel output, reference output). Every slot no item writes
    holds ``poison``. ``give_back``: pages wholly in front of the window of an item's first new
    token are not in its table any more (-1, as the cache manager leaves them), and page 0,
    which stands in for them in the packed table, belongs to nobody and holds ``poison`` too."""
    rng = np.random.default_rng(seed)
    perm = [b for b in rng.permutation(num_blocks).tolist() if not (give_back and b == 0)]
    pk = StepPacker(torch.device(DEV), [GroupMeta(num_blocks, window)], 10, 100000, 8, ops.PREFILL_TILE_Q,
                    skew_rule=ops.decode_is_skewed)
    kv = torch.full((num_blocks, 2, hkv, 16 * d), poison, dtype=act, device=DEV)
    items, full = [], []
    for i, (n, old) in enumerate(zip(lens_new, lens_old)):
        pages = -(-(n + old) // 16)
        table = [perm.pop() for _ in range(pages)]
        k = rnd(n + old, hkv, d, dtype=act, seed=seed * 100 + 2 * i)
        v = rnd(n + old, hkv, d, dtype=act, seed=seed * 100 + 2 * i + 1)
        full.append((k, v))
        kp = kv[:, 0].view(num_blocks, hkv, 16, d)
        vp = kv[:, 1].view(num_blocks, hkv, d, 16)
        pos = torch.arange(n + old)
        pg = torch.tensor(table)[pos // 16].to(DEV)
        kp[pg, :, (pos % 16).to(DEV), :] = k
        vp[pg, :, :, (pos % 16).to(DEV)] = v
        if give_back:
            gone = max(0, old - window + 1) // 16
            kp[torch.tensor(table[:gone], dtype=torch.long, device=DEV)] = poison
            vp[torch.tensor(table[:gone], dtype=torch.long, device=DEV)] = poison
            table = [-1] * gone + table[gone:]
        items.append(StepItem(i, [1] * n, old, [table], slot=i % 8))
    ctx = pk.pack(items)
    t = sum(lens_new)
    qkv = rnd(t, (hq + 2 * hkv) * d, dtype=act, seed=seed + 999)
    out = torch.empty(t, hq * d, dtype=act, device=DEV)
    scale = 1.0 / math.sqrt(d)
    ops.paged_attention(qkv, out, kv, ctx, 0, hq, hkv, d, scale, window)
    want = torch.empty(t, hq, d, dtype=torch.float64, device=DEV)
    t0 = 0
    for (k, v), n, old in zip(full, lens_new, lens_old):
        q = qkv[t0:t0 + n, : hq * d].view(n, hq, d).double()
        kk = k.double().repeat_interleave(hq // hkv, 1)
        vv = v.double().repeat_interleave(hq // hkv, 1)
        s = torch.einsum("nhd,mhd->hnm", q, kk) * scale
        qpos = torch.arange(old, old + n, device=DEV)[:, None]
        kpos = torch.arange(old + n, device=DEV)[None, :]
        hide = kpos > qpos
        if window is not None:
            hide = hide | (qpos - kpos >= window)
        p = torch.softmax(s.masked_fill(hide, float("-inf")), -1)
        want[t0:t0 + n] = torch.einsum("hnm,mhd->nhd", p, vv)
        t0 += n
    return out.view(t, hq, d), want


SHAPES = [(4, 2, 16), (3, 1, 32), (8, 2, 64), (32, 8, 64), (6, 6, 96), (8, 1, 128), (40, 2, 64), (2, 2, 256), (6, 3, 48), (2, 1, 80),
          (6, 2, 256), (12, 4, 128), (5, 1, 32), (9, 3, 96),
          # head sizes that are no multiple of 32 (the last step of 32 half used) and the sizes above 128
          (8, 2, 48), (10, 2, 80), (8, 2, 112), (4, 1, 160), (6, 2, 192),
          (4, 2, 144)]      # one the matrix-core kernels do not take: the generic kernel


@pytest.mark.parametrize("hq,hkv,d", SHAPES)
@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_paged_attention_mixed_batch(ops, act, hq, hkv, d):
    """Fresh prompts, portions on top of a cached prefix, decodes with one slot left in the
    last page and with a last page exactly full: one batch."""
    new = [37, 1, 130, 1, 2, 16, 1, 1]
    old = [0, 15, 50, 31, 94, 16, 0, 200]
    got, want = paged_case(ops, act, hq, hkv, d, new, old, seed=hq + d)
    assert rel(got, want) < (2e-5 if act == torch.float32 else 2e-2)


@pytest.mark.parametrize("hq,hkv,d,longest,window", [
    (32, 8, 64, 700, None),        # 40 requests x 8 kv heads: keys not split over workgroups
    (32, 8, 64, 700, 150),         # the same with a window whose first pages were given back
    (16, 8, 128, 3300, None),      # head size 128, long contexts
    (16, 8, 128, 700, None),       # and short ones
    (6, 3, 48, 300, None),         # a head size that is no multiple of 32
    (10, 2, 80, 700, None),        # the same with five heads per kv head
    (4, 2, 144, 300, None),        # a head size the matrix-core kernels do not take: the generic kernel
])
def test_decode_attention_of_many_requests(ops, hq, hkv, d, longest, window):
    """Forty requests decode together, their contexts from 0 to ``longest`` tokens (empty, one
    token, a page's edge, a tile's edge among them): with 256 (request, kv head) pairs or more
    the keys are not split over workgroups and a wave runs through many tiles."""
    rng = np.random.default_rng(longest + d)
    old = [0, 1, 15, 16, 31, 32, 33, 63, 64, 127, 128, longest] + rng.integers(0, longest, 28).tolist()
    new = [1] * len(old)
    pages = sum(-(-(o + 1) // 16) for o in old) + 8
    got, want = paged_case(ops, torch.bfloat16, hq, hkv, d, new, old, window=window, seed=7, num_blocks=pages,
                           poison=float("nan"), give_back=window is not None)
    assert rel(got, want) < 2e-2


@pytest.mark.parametrize("hq,hkv,d,short,longest", [
    (32, 8, 64, 31, 9000),         # many workgroups already: the long request alone gets more runs
    (16, 8, 128, 7, 12500),        # few requests: runs of 1,024 keys instead of the usual short ones
    (4, 1, 64, 15, 12000),         # one kv head
    (6, 3, 96, 40, 11000),         # three kv heads, head size 96
])
def test_decode_attention_with_one_long_context_among_short_ones(ops, hq, hkv, d, short, longest):
    """One request's context is far longer than the others': the step counts as skewed and every
    request's keys are cut into runs of 1,024 or more, nine or more for the long request, one for
    the short ones, whose other runs are empty. Slots nobody wrote hold NaN. Every request is
    judged by its own rows: the long request's output, an average over thousands of random
    values, is a hundred times smaller than the short ones', and a common scale would hide it."""
    rng = np.random.default_rng(longest)
    old = rng.integers(0, 600, short).tolist()
    old.insert(short // 2, longest)
    new = [1] * len(old)
    pages = sum(-(-(o + 1) // 16) for o in old) + 8
    seen = {}
    packed = StepPacker.pack

    def spy(self, items, **kw):
        ctx = packed(self, items, **kw)
        seen["skewed"] = ctx.decode_skewed
        return ctx

    StepPacker.pack = spy
    try:
        got, want = paged_case(ops, torch.bfloat16, hq, hkv, d, new, old, seed=11, num_blocks=pages, poison=float("nan"))
    finally:
        StepPacker.pack = packed
    assert seen["skewed"]
    assert torch.isfinite(got.float()).all()
    for i in range(len(old)):
        assert rel(got[i], want[i]) < 2e-2, f"request {i} of {old[i]} keys"


@pytest.mark.parametrize("hq,hkv,d,short,longest", [
    (32, 8, 64, 31, 9000),
    (16, 8, 128, 7, 12500),
    (4, 1, 64, 15, 12000),
])
def test_skewed_decode_attention_finds_one_planted_key(ops, hq, hkv, d, short, longest):
    """The long request of a skewed step, with one key made to match its query so strongly that
    the output is that key's value: at the first and last key of the runs of 1,024 (or more)
    that different workgroups take, at the very first and the very last key. A run that is
    dropped, read twice or merged with the wrong weight cannot pass; the short requests, whose
    later runs are empty, are compared one by one with their references."""
    act = torch.bfloat16
    group = hq // hkv
    rng = np.random.default_rng(longest + 1)
    old = rng.integers(0, 600, short).tolist()
    long_at = short // 2
    old.insert(long_at, longest)
    n_req = len(old)
    num_blocks = sum(-(-(o + 1) // 16) for o in old) + 8
    perm = rng.permutation(num_blocks).tolist()
    tables = [[perm.pop() for _ in range(-(-(o + 1) // 16))] for o in old]
    ks = [rnd(o + 1, hkv, d, dtype=act, seed=100 + i, scale=0.05) for i, o in enumerate(old)]
    vs = [rnd(o + 1, hkv, d, dtype=act, seed=200 + i) for i, o in enumerate(old)]
    qkv = rnd(n_req, (hq + 2 * hkv) * d, dtype=act, seed=3, scale=0.05)
    pk = StepPacker(torch.device(DEV), [GroupMeta(num_blocks)], 10, 100000, 64, ops.PREFILL_TILE_Q,
                    skew_rule=ops.decode_is_skewed)
    items = [StepItem(i, [1], o, [t], slot=i) for i, (o, t) in enumerate(zip(old, tables))]
    nsplit, min_run = ops.decode_plan(n_req, longest + 1, True, hkv, 0)
    assert min_run == 1024 and nsplit >= 9
    run = -(-(-(-(longest + 1) // 32)) // nsplit) * 32            # keys per run: whole 32-key tiles
    run = max(run, min_run)
    plants = sorted({0, 1023, 1024, 2047, 2048, longest, longest - 1} |
                    {p + e for p in range(run, longest, run) for e in (-1, 0)})
    kv = torch.full((num_blocks, 2, hkv, 16 * d), float("nan"), dtype=act, device=DEV)
    kp, vp = kv[:, 0].view(num_blocks, hkv, 16, d), kv[:, 1].view(num_blocks, hkv, d, 16)
    for i, (o, t) in enumerate(zip(old, tables)):
        pos = torch.arange(o + 1)
        pg = torch.tensor(t)[pos // 16].to(DEV)
        kp[pg, :, (pos % 16).to(DEV), :] = ks[i]
        vp[pg, :, :, (pos % 16).to(DEV)] = vs[i]
    scale = 50.0
    want_short = {}
    for i in range(n_req):
        if i == long_at:
            continue
        q = qkv[i, : hq * d].view(hq, d).double()
        sc = torch.einsum("hd,mhd->hm", q, ks[i].double().repeat_interleave(group, 1)) * scale
        want_short[i] = torch.einsum("hm,mhd->hd", torch.softmax(sc, -1), vs[i].double().repeat_interleave(group, 1))
    for far in plants:
        page, off = tables[long_at][far // 16], far % 16
        kept = kp[page, :, off, :].clone()
        for h in range(hkv):
            q = qkv[long_at, h * group * d: h * group * d + d]
            kp[page, h, off, :] = 40.0 * q / q.float().norm()
        ctx = pk.pack(items)
        assert ctx.decode_skewed
        out = torch.empty(n_req, hq * d, dtype=act, device=DEV)
        ops.paged_attention(qkv, out, kv, ctx, 0, hq, hkv, d, scale, None)
        kp[page, :, off, :] = kept
        got = out.view(n_req, hq, d)
        assert torch.isfinite(got.float()).all()
        for h in range(hkv):
            assert rel(got[long_at, h * group], vs[long_at][far, h]) < 2e-2, f"planted key {far} of {longest}, kv head {h}: not found"
        for i, want in want_short.items():
            assert rel(got[i], want) < 2e-2, f"short request {i} ({old[i]} keys) beside planted key {far}"


@pytest.mark.parametrize("hq,hkv,d,new,old,window", [
    (32, 8, 64, [2048], [0], None),              # 512 workgroups, nothing cached: grouped, a kv head's tiles on one die
    (24, 8, 128, [2100], [0], None),             # three heads per kv head, an odd number of tiles, a last tile of 20
    (16, 8, 128, [1100], [0], None),             # two heads per kv head at head size 128: grouped, half its waves spare
    (16, 8, 128, [500], [600], None),            # the same with few workgroups: the per-head kernel
    (16, 4, 64, [2048, 2100], [0, 0], None),     # two prompts from position 0 in one step, 4 workgroups per tile
    (32, 8, 64, [512], [1536], None),            # 128 workgroups on 2,048 keys: grouped, two runs
    (16, 4, 48, [2048], [0], None),              # head size 48: grouped, the second 32 dimensions half used
    (24, 8, 80, [2100], [0], None),              # head size 80, three heads per kv head
    (8, 8, 112, [700], [500], None),             # head size 112: the per-head kernel
    (12, 4, 192, [600], [500], None),            # head size 192: grouped, one workgroup per compute unit
    (32, 8, 64, [512], [1000], None),            # 128 workgroups on fewer keys: the per-head kernel at this head size
    (32, 8, 64, [512], [7680], None),            # a portion of a long prompt: each tile's keys in four runs
    (32, 8, 128, [40], [16000], None),           # a short tail behind a long context: sixteen workgroups, fifteen runs each
    (24, 8, 128, [20, 300], [9000, 100], None),  # runs that a short request leaves empty, beside a long one; a spare wave
    (16, 4, 64, [64], [5000], 1500),             # split runs inside a window
    (40, 2, 64, [33], [6000], None),             # five workgroups per kv head, each tile's keys in five runs
    (32, 8, 128, [512], [3584], None),           # 128 workgroups at head size 128: two runs
    (8, 8, 128, [100, 40], [5000, 300], None),   # one query head per kv head: the per-head kernel, eight runs, some empty
    (16, 8, 64, [200], [3000], 2500),            # two query heads per kv head, a window: the per-head kernel, two runs
    (32, 8, 64, [768], [1536], None),            # 192 workgroups on a long prefix: grouped
    (32, 8, 128, [512], [1536], None),           # 128 workgroups at head size 128: grouped
    (32, 8, 128, [4100], [0], None),             # 1,032 workgroups at head size 128: grouped, one wave per head
    (32, 8, 64, [2048, 3], [2048, 7], None),     # 512 workgroups, much cached, beside a short portion
    (40, 2, 64, [500, 77], [100, 0], None),      # twenty heads per kv head: five workgroups per kv head
    (6, 2, 256, [1500, 1000], [0, 200], None),   # head size 256
    (16, 4, 64, [700, 300], [50, 0], 100),       # grouped, with a window
    (32, 8, 64, [2048], [0], 300),               # a long prompt with a window
    (32, 8, 64, [100], [1948], None),            # few tiles: grouped, four runs of 512 keys
    (32, 8, 64, [100], [600], None),             # few tiles on few keys: the per-head kernel
    # One or two query heads per kv head: a workgroup of the grouped kernel takes four or two
    # consecutive tiles of an item; items that end inside such a run, beside single tokens
    (32, 32, 64, [300, 70, 1, 2, 129], [0, 500, 77, 40, 1000], None),
    (32, 16, 128, [300, 70, 1, 2, 129], [0, 500, 77, 40, 1000], None),
    (16, 16, 128, [2100], [0], None),            # a last run of two tiles, the second of 20 queries
    (16, 8, 64, [2048 + 33], [0], None),         # a last run of one tile
    (32, 32, 48, [1000, 600], [24, 0], None),
    (32, 32, 64, [700, 300, 1], [150, 0, 900], 100),     # with a window
    (32, 16, 64, [2048], [300], 300),
    (8, 8, 128, [700], [500], None),             # too few workgroups for that: the per-head kernel
    (32, 32, 128, [512], [7680], None),          # four tiles per workgroup, each run of tiles' keys in two runs
    (32, 32, 64, [500], [7680], None),           # the same in four runs, a last run of tiles that ends early
    (32, 16, 128, [20, 300], [9000, 100], None), # two tiles per workgroup, runs of keys that a short request leaves empty
    (16, 16, 64, [64], [5000], 1500),            # runs of keys inside a window
    (16, 8, 64, [90], [4100], None),             # few workgroups: the per-head kernel, with its own runs
])
def test_prefill_attention_in_each_form(ops, hq, hkv, d, new, old, window):
    """The portions of a step go to the per-head or to the grouped kernel by their number of tiles
    and the head size; each at sizes that select it, with grids that are and are not multiples of
    the eight dies in their fast index."""
    pages = sum(-(-(n + o) // 16) for n, o in zip(new, old)) + 8
    got, want = paged_case(ops, torch.bfloat16, hq, hkv, d, new, old, window=window, seed=len(new) + d, num_blocks=pages)
    assert rel(got, want) < 2e-2


@pytest.mark.parametrize("hq,hkv,d,new,old,window", [
    (8, 2, 64, [37, 1, 130, 1, 2, 16, 1, 1], [0, 15, 50, 31, 94, 16, 0, 200], None),   # decode and the per-head prefill kernel
    (32, 8, 64, [2040], [0], None),                 # grouped; the last page has 8 slots nobody wrote
    (32, 8, 64, [500], [1530], None),               # the per-head kernel on a cached prefix
    (32, 8, 64, [700], [1330], None),               # grouped on a cached prefix
    (32, 8, 64, [300], [5000], None),               # grouped, the keys of a tile in five runs
    (24, 8, 128, [20, 300], [9000, 100], None),     # runs left empty
    (24, 8, 112, [20, 300], [9000, 100], None),     # the same at head size 112
    (32, 8, 48, [300], [5000], None),               # head size 48 in runs
    (8, 2, 160, [100, 40], [5000, 300], None),      # head size 160 in runs
    (8, 8, 128, [100, 40], [5000, 300], None),      # the per-head kernel with runs
    (24, 8, 128, [2100, 1], [0, 77], None),
    (32, 32, 64, [300, 70, 1, 2, 129], [0, 500, 77, 40, 1000], None),     # grouped, four tiles per workgroup
    (32, 16, 128, [700, 300, 1], [150, 0, 900], 100),                      # two tiles per workgroup, a window
    (32, 32, 64, [500], [7690], None),                                     # four tiles per workgroup, keys in runs
    (8, 2, 64, [70, 1, 1, 9], [0, 40, 130, 64], 33),        # windows whose first pages were given back
    (16, 4, 64, [700, 300, 1], [150, 0, 900], 100),
    (32, 8, 64, [2040], [300], 300),
])
@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_attention_ignores_what_lies_in_slots_nobody_wrote(ops, act, hq, hkv, d, new, old, window):
    """The rest of a request's last page, and pages a window has given back, may hold what an
    earlier owner left there, NaN and infinities included. Their keys are masked; their values
    must not reach the output either (0 x NaN is NaN)."""
    pages = sum(-(-(n + o) // 16) for n, o in zip(new, old)) + 8
    for poison in (float("nan"), float("inf")):
        got, want = paged_case(ops, act, hq, hkv, d, new, old, window=window, seed=7 + d, num_blocks=pages, poison=poison,
                               give_back=window is not None)
        assert torch.isfinite(got.float()).all(), f"poison {poison} reached the output"
        assert rel(got, want) < (2e-5 if act == torch.float32 else 2e-2)


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 16, 33, 100])
def test_paged_attention_window(ops, act, window):
    got, want = paged_case(ops, act, 8, 2, 64, [70, 1, 1, 9], [0, 40, 130, 64], window=window, seed=window)
    assert rel(got, want) < (2e-5 if act == torch.float32 else 2e-2)


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_paged_attention_long_contexts(ops, act):
    """Tens of thousands of cached positions: the decode kernel at its widest split, a portion
    on top of a long prefix, and short requests beside them in the same batch."""
    got, want = paged_case(ops, act, 8, 2, 64, [1, 300, 1, 1, 5], [20000, 9000, 3, 33000, 0], seed=5, num_blocks=4096)
    assert rel(got, want) < (2e-5 if act == torch.float32 else 2e-2)
    got, want = paged_case(ops, act, 4, 4, 128, [1, 40], [16383, 16384], seed=6, num_blocks=2100)
    assert rel(got, want) < (2e-5 if act == torch.float32 else 2e-2)


@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_attention_finds_one_far_key_among_hundreds(ops, act):
    """One old key is made to match the query strongly; the output must be that key's value,
    wherever its page lies. A kernel that skips or misplaces a page cannot pass."""
    hq, hkv, d, n_old = 8, 2, 64, 700
    for far in (0, 15, 16, 333, 511, 512, 699):
        rng = np.random.default_rng(far)
        num_blocks = 64
        perm = rng.permutation(num_blocks).tolist()
        table = [perm.pop() for _ in range(-(-(n_old + 1) // 16))]
        kv = torch.zeros((num_blocks, 2, hkv, 16 * d), dtype=act, device=DEV)
        k = rnd(n_old + 1, hkv, d, dtype=act, seed=1, scale=0.05)
        v = rnd(n_old + 1, hkv, d, dtype=act, seed=2)
        qkv = rnd(1, (hq + 2 * hkv) * d, dtype=act, seed=3, scale=0.05)
        q = qkv[0, : hq * d].view(hq, d)
        k[far] = 0
        for h in range(hkv):
            k[far, h] = 40.0 * q[h * (hq // hkv)] / q[h * (hq // hkv)].float().norm()     # aligned with the group's first head
        pos = torch.arange(n_old + 1)
        pg = torch.tensor(table)[pos // 16].to(DEV)
        kv[:, 0].view(num_blocks, hkv, 16, d)[pg, :, (pos % 16).to(DEV), :] = k
        kv[:, 1].view(num_blocks, hkv, d, 16)[pg, :, :, (pos % 16).to(DEV)] = v
        pk = StepPacker(torch.device(DEV), [GroupMeta(num_blocks)], 10, 4096, 8, ops.PREFILL_TILE_Q)
        ctx = pk.pack([StepItem("a", [1], n_old, [table])])
        out = torch.empty(1, hq * d, dtype=act, device=DEV)
        # a large scale makes the softmax one-hot on the planted key for the aligned heads
        ops.paged_attention(qkv, out, kv, ctx, 0, hq, hkv, d, 50.0, None)
        for h in range(hkv):
            head = h * (hq // hkv)
            assert rel(out.view(hq, d)[head], v[far, h]) < 2e-2, f"far key at {far}, head {head}"


@pytest.mark.parametrize("hq,hkv,d,new,old,window", [
    (32, 8, 64, 100, 1948, None),       # few tiles: grouped, four runs of 512 keys
    (32, 8, 64, 100, 600, None),        # few tiles on few keys: the per-head kernel, keys split over its four waves
    (32, 8, 64, 512, 1536, None),       # grouped on a cached prefix, two runs of 1,024 keys
    (32, 8, 64, 512, 1000, None),       # the per-head kernel on a cached prefix, 128 workgroups' worth
    (32, 8, 64, 512, 7680, None),       # four runs of 2,048 keys
    (32, 8, 128, 40, 8000, None),       # head size 128, seven runs of 1,152 keys
    (16, 4, 64, 64, 5000, 1500),        # runs inside a window
    (4, 4, 128, 70, 6000, None),        # the per-head kernel, five runs
    (16, 8, 64, 90, 4100, None),        # two query heads per kv head: the per-head kernel, four runs
    (32, 8, 64, 800, 1248, None),       # grouped, on a cached prefix
    (32, 8, 64, 2048, 0, None),         # grouped, a whole prompt
    (24, 8, 128, 700, 500, None),       # head size 128, three heads per kv head
    (16, 8, 128, 1100, 100, None),      # head size 128, two heads per kv head: grouped with spare waves
    (32, 8, 128, 4100, 0, None),        # head size 128, a long prompt: one wave per head
    (32, 8, 64, 2048, 0, 300),          # a whole prompt with a window
    (16, 4, 64, 600, 200, 100),         # grouped with a window
])
def test_prefill_attention_finds_one_planted_key(ops, hq, hkv, d, new, old, window):
    """With random keys a 32-key tile that is dropped or read twice far from the diagonal moves
    the output by a percent or two, which a tolerance hides. Here one key is made to match one
    query so strongly that the query's output is that key's value: planted at the edges of
    pages, of 32-key tiles and of the 64-key iterations, in the first and the last tile a query
    sees, in the cached prefix and among the new tokens; and with a window, on its first key
    inside (found) and on the key just outside (must not be seen at all)."""
    act = torch.bfloat16
    total = old + new
    num_blocks = -(-total // 16) + 4
    rng = np.random.default_rng(d + new)
    table = rng.permutation(num_blocks).tolist()[: -(-total // 16)]
    group = hq // hkv
    k = rnd(total, hkv, d, dtype=act, seed=1, scale=0.05)
    v = rnd(total, hkv, d, dtype=act, seed=2)
    qkv = rnd(new, (hq + 2 * hkv) * d, dtype=act, seed=3, scale=0.05)
    pk = StepPacker(torch.device(DEV), [GroupMeta(num_blocks, window)], 10, 100000, 8, ops.PREFILL_TILE_Q)
    pos = torch.arange(total)
    pg = torch.tensor(table)[pos // 16].to(DEV)
    last = total - 1
    # (query position, key position, must the key be seen)
    plants = [(last, 0, True), (last, 15, True), (last, 16, True), (last, 31, True), (last, 32, True), (last, 63, True),
              (last, 64, True), (last, old - 1 if old else 95, True), (last, old, True), (last, last - 32, True),
              (last, last, True), (old + 33, 32, True), (old + 33, old + 33, True), (old + new // 2, 127, True),
              (old + new // 2, 128, True), (old + 1, 0, True)]
    # where runs of keys that different workgroups take may begin and end
    plants += [(last, p + e, True) for p in range(512, total, 128) for e in (-1, 0)]
    if window is not None:
        plants = [(q, max(q - window + 1, 0), True) for q, _, _ in plants[:4]] + \
                 [(last, last - window + 1, True), (last, last - window, False), (old + new // 2, old + new // 2 - window, False),
                  (old + 40, max(old + 40 - window + 1, 0), True), (last, last - 5, True)] + \
                 [(last, p + e, True) for p in range((last - window + 512) & ~127, last, 128) for e in (-1, 0)]
    for q_pos, far, seen in plants:
        if not 0 <= far <= q_pos:
            continue
        kk = k.clone()
        qi = q_pos - old
        for h in range(hkv):
            q = qkv[qi, h * group * d: h * group * d + d]                         # the group's first head
            kk[far, h] = 40.0 * q / q.float().norm()
        kv = torch.zeros((num_blocks, 2, hkv, 16 * d), dtype=act, device=DEV)
        kv[:, 0].view(num_blocks, hkv, 16, d)[pg, :, (pos % 16).to(DEV), :] = kk
        kv[:, 1].view(num_blocks, hkv, d, 16)[pg, :, :, (pos % 16).to(DEV)] = v
        ctx = pk.pack([StepItem("a", [1] * new, old, [table])])
        out = torch.empty(new, hq * d, dtype=act, device=DEV)
        ops.paged_attention(qkv, out, kv, ctx, 0, hq, hkv, d, 50.0, window)
        for h in range(hkv):
            got = out[qi].view(hq, d)[h * group]
            if seen:
                assert rel(got, v[far, h]) < 2e-2, f"query {q_pos}, planted key {far}, kv head {h}: not found"
            else:
                lo = q_pos - window + 1
                s = (qkv[qi, h * group * d: h * group * d + d].double() @ kk[lo:q_pos + 1, h].double().T) * 50.0
                want = torch.softmax(s, -1) @ v[lo:q_pos + 1, h].double()
                assert rel(got, want) < 2e-2, f"query {q_pos}, planted key {far} outside the window was seen"
                assert rel(got, v[far, h]) > 0.5


# --------------------------------------------------------------------- sampling

@pytest.mark.parametrize("vocab", [1237, 50257, 3])
def test_sampling_kernel(ops, vocab):
    """One run of the vocabulary, many runs of a length that is no multiple of 4 (so rows and
    runs start at odd alignments), and a vocabulary smaller than anything the kernel tiles by."""
    from plain.llama_plain import sample_plain

    rows = 6
    logits = rnd(rows, vocab, seed=4, scale=3.0)
    if vocab == 3:
        logits[0, 1] = logits[0, 2] = 50.0
        logits_tie = 1
    else:
        logits[0, 77] = logits[0, 900] = 50.0                       # a tie: the lowest index wins
        logits_tie = 77
    temps = torch.tensor([0.0, 0.0, 0.8, 0.8, 1.5, 0.3], device=DEV)
    us = torch.tensor([0.0, 0.5, 0.1234, 0.9999, 0.5, 0.0], device=DEV)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops.sample(logits, temps, us, out)
    got = out.tolist()
    assert got[0] == logits_tie and got[1] == int(torch.argmax(logits[1]))
    lg = logits.cpu().numpy()
    for r in range(2, rows):
        want = sample_plain(lg[r], float(temps[r]), float(us[r]))
        if got[r] != want:                                          # only a rounding of the CDF edge may differ
            z = lg[r].astype(np.float64) / float(temps[r])
            c = np.cumsum(np.exp(z - z.max()))
            target = float(us[r]) * c[-1]
            lo, hi = min(got[r], want), max(got[r], want)
            assert hi - lo == 1 and abs(c[lo] - target) < 1e-5 * c[-1]
    out2 = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops.argmax(logits, out2)
    assert out2.tolist() == [logits_tie] + torch.argmax(logits[1:], -1).tolist()


@pytest.mark.parametrize("vocab", [5, 5000, 40001])
def test_sampling_of_rows_without_a_maximum_stays_in_the_vocabulary(ops, vocab):
    """Rows of NaN or of -inf have no largest entry. The token is fed to the next step's
    embedding on the device, so whatever is returned must be an index of the row."""
    logits = rnd(6, vocab, seed=9)
    logits[0] = float("nan")
    logits[1] = float("-inf")
    logits[2] = float("nan")
    logits[3] = float("-inf")
    logits[4, : vocab // 2] = float("nan")                          # NaNs beside numbers: a number wins
    temps = torch.tensor([0.0, 0.0, 0.9, 0.9, 0.0, 0.0], device=DEV)
    us = torch.tensor([0.0, 0.0, 0.7, 0.7, 0.0, 0.0], device=DEV)
    out = torch.full((6,), -7, dtype=torch.int32, device=DEV)
    ops.sample(logits, temps, us, out)
    got = out.tolist()
    assert all(0 <= t < vocab for t in got), got
    assert got[0] == 0 and got[1] == 0
    assert got[4] == vocab // 2 + int(torch.argmax(logits[4, vocab // 2:]))
    assert got[5] == int(torch.argmax(logits[5]))


def test_embed_reads_the_nearest_row_for_an_id_outside_the_table(ops):
    table = rnd(7, 24).to(torch.bfloat16)
    ids = torch.tensor([3, -5, 0x7FFFFFFF, 6, 7], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 24, device=DEV)
    ops.embed(ids, table, out)
    assert torch.equal(out, table[[3, 0, 6, 6, 6]].float())


def test_sampling_frequencies(ops):
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]], device=DEV).repeat(4000, 1).contiguous()
    g = torch.Generator().manual_seed(0)
    us = torch.rand(4000, generator=g).to(DEV)
    temps = torch.full((4000,), 0.7, device=DEV)
    out = torch.empty(4000, dtype=torch.int32, device=DEV)
    ops.sample(logits, temps, us, out)
    freq = torch.bincount(out.long().cpu(), minlength=5).double() / 4000
    want = torch.softmax(logits[0].double().cpu() / 0.7, 0)
    assert float((freq - want).abs().max()) < 0.03


def test_kernels_refuse_what_they_do_not_take(ops):
    from prefixserve_amd.kernels.ops import KernelError

    with pytest.raises(KernelError):
        ops.linear(rnd(2, 8), rnd(4, 9), torch.empty(2, 4, device=DEV))
    with pytest.raises(KernelError):
        ops.embed(torch.zeros(2, dtype=torch.int64, device=DEV), rnd(4, 8), torch.empty(2, 8, device=DEV))
    with pytest.raises(KernelError):
        ops.add_rmsnorm(rnd(2, 8).to(torch.bfloat16), None, rnd(8), 1e-5, torch.empty(2, 8, device=DEV))
    x = rnd(2, 8).to(torch.float16)
    with pytest.raises(KernelError):
        ops.swiglu(x, torch.empty(2, 4, dtype=torch.float16, device=DEV))
