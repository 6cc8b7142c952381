"""Each HIP kernel alone against a plain float64 reference of the same operation, at sizes other
than the tiny models' (widths that are no power of two, odd row counts, several head sizes)."""
import math
import numpy as np

import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from inferflux_amd.kernels import ops

DEV = "cuda"
F32, BF16 = torch.float32, torch.bfloat16


def tol(dtype):
    # float32: rounding of a few dozen operations; bfloat16: one rounding of the result (2^-9 relative)
    return dict(rtol=2e-5, atol=2e-6) if dtype == F32 else dict(rtol=8e-3, atol=1e-3)


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_embedding(dtype):
    g = gen(1)
    table = torch.randn(77, 100, generator=g).to(dtype)
    ids = torch.tensor([0, 76, 5, 5, 33], dtype=torch.int32)
    out = ops.embedding(ids.to(DEV), table.to(DEV))
    assert out.dtype == F32 and torch.equal(out.cpu(), table.float()[ids.long()])
    wide = torch.randn(6, 9001, generator=g).to(dtype)              # rows of more than one run of 4,096 columns
    pick = torch.tensor([5, 0, 3], dtype=torch.int32)
    assert torch.equal(ops.embedding(pick.to(DEV), wide.to(DEV)).cpu(), wide.float()[pick.long()])


@pytest.mark.parametrize("T,H", [(1, 104), (5, 896), (16, 3584), (9, 9008)])
def test_embedding_that_prepares_the_first_norm(T, H):
    """The stream as ``embedding`` gives it, the rows times the norm's weight, and sums of squares by runs of 4,096
    columns that add up to each row's (zeros for the rows a step of fewer than 16 tokens does not have); what a product
    makes of such rows is the norm's output times the weight."""
    g = gen(3)
    eps = 1e-5
    table = torch.randn(50, H, generator=g).to(BF16)
    nw = (1 + 0.3 * torch.randn(H, generator=g)).to(BF16)
    ids = torch.randint(0, 50, (T,), generator=g).to(torch.int32)
    stream, scaled = ops.embedding_scaled(ids.to(DEV), table.to(DEV), nw.to(DEV), eps)
    x = table.float()[ids.long()]
    assert torch.equal(stream.cpu(), x)
    assert torch.equal(scaled.rows.cpu(), (x * nw.float()).to(BF16))
    pieces = scaled.pieces.cpu().double()
    assert pieces.shape == (-(-H // 4096), 16) and bool((pieces[:, T:] == 0).all())
    assert torch.allclose(pieces.sum(0)[:T], (x.double() ** 2).sum(-1), rtol=1e-5)
    assert scaled.width == H and scaled.eps == eps
    w = (torch.randn(64, H, generator=g) * 0.1).to(BF16)
    got = ops.linear(scaled, ops.prepare_linear(w.to(DEV)), F32).cpu().double()
    want = pm.rms_norm(x.double(), nw.double(), eps) @ w.double().t()
    assert float((got - want).abs().max()) <= 1e-2 * float(want.abs().max())
    with pytest.raises(ops.KernelError, match="at most 16"):
        ops.embedding_scaled(torch.zeros(17, dtype=torch.int32, device=DEV), table.to(DEV), nw.to(DEV), eps)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("H", [100, 3584])
@pytest.mark.parametrize("wdtype", [F32, BF16])
def test_add_rmsnorm(dtype, H, wdtype):
    g = gen(2)
    T, eps = 7, 1e-5
    res = torch.randn(T, H, generator=g)
    delta = torch.randn(T, H, generator=g).to(dtype)
    w = (1 + 0.3 * torch.randn(H, generator=g)).to(wdtype)
    want_res = res.double() + delta.double()
    want = pm.rms_norm(want_res, w.double(), eps)
    r = res.to(DEV)
    out = ops.add_rmsnorm(r, delta.to(DEV), w.to(DEV), eps, dtype)
    assert torch.allclose(r.cpu().double(), want_res, rtol=1e-6, atol=1e-6)        # the stream took the delta
    assert torch.allclose(out.cpu().double(), want, **tol(dtype))
    out2 = ops.add_rmsnorm(res.to(DEV), None, w.to(DEV), eps, dtype)                # no delta
    assert torch.allclose(out2.cpu().double(), pm.rms_norm(res.double(), w.double(), eps), **tol(dtype))
    rows = torch.tensor([6, 0, 3], dtype=torch.int32)
    r3 = res.to(DEV)
    out3 = ops.add_rmsnorm(r3, delta.to(DEV), w.to(DEV), eps, dtype, rows.to(DEV))  # gathered rows: stream untouched
    assert torch.equal(r3.cpu(), res)
    assert torch.allclose(out3.cpu().double(), want[rows.long()], **tol(dtype))


@pytest.mark.parametrize("seed", range(30))
def test_add_rmsnorm_random_shapes(seed):
    """Residual add and norm at widths of 1-9,000 (the vector form takes multiples of 8, the plain form the others),
    1-300 rows, a delta that is bf16, float, partial sums of 2-9 slices, or absent, and a gathered subset of rows;
    against float64."""
    import random
    rng = random.Random(1100 + seed)
    T = rng.choice([1, rng.randint(2, 20), rng.randint(21, 300)])
    H = rng.choice([rng.randint(1, 64), 8 * rng.randint(8, 600), rng.randint(65, 9000), 8 * rng.randint(601, 1100)])
    out_dtype, wdtype = rng.choice([F32, BF16]), rng.choice([F32, BF16])
    kind = rng.choice(["bf16", "f32", "slices", "slices", "none"])
    eps = rng.choice([1e-6, 1e-5, 1e-2])
    g = gen(1200 + seed)
    res = torch.randn(T, H, generator=g) * 3
    w = (1 + 0.3 * torch.randn(H, generator=g)).to(wdtype)
    delta, want_res = None, res.double()
    if kind == "slices":
        parts = torch.randn(rng.randint(2, 9), T, H, generator=g)
        delta = ops.SliceSums(parts.to(DEV), out_dtype)
        want_res = res.double() + parts.double().sum(0)
    elif kind != "none":
        d = torch.randn(T, H, generator=g).to(BF16 if kind == "bf16" else F32)
        delta, want_res = d.to(DEV), res.double() + d.double()
    want = pm.rms_norm(want_res, w.double(), eps)
    r = res.to(DEV)
    out = ops.add_rmsnorm(r, delta, w.to(DEV), eps, out_dtype)
    case = (T, H, kind, out_dtype, wdtype)
    assert torch.allclose(r.cpu().double(), want_res, rtol=1e-6, atol=1e-5), case          # the stream took the delta
    assert torch.allclose(out.cpu().double(), want, **tol(out_dtype)), case
    rows = torch.tensor([rng.randrange(T) for _ in range(rng.randint(1, 5))], dtype=torch.int32)
    r2 = res.to(DEV)
    out2 = ops.add_rmsnorm(r2, delta, w.to(DEV), eps, out_dtype, rows.to(DEV))             # gathered rows: stream untouched
    assert torch.equal(r2.cpu(), res), case
    assert torch.allclose(out2.cpu().double(), want[rows.long()], **tol(out_dtype)), case


def test_rmsnorm_eps_is_inside_the_root():
    x = torch.full((1, 64), 1e-4)
    w = torch.ones(64)
    a = ops.add_rmsnorm(x.to(DEV), None, w.to(DEV), 1e-6, F32).cpu()
    assert torch.allclose(a, x / math.sqrt(1e-8 + 1e-6), rtol=1e-5)


def cache_rows(k_cache, v_cache, slots, page_size):
    """Read back [T, nKV, d] keys and values from the two page layouts."""
    pages, offs = slots // page_size, slots % page_size
    k = k_cache[pages.long(), :, offs.long(), :]
    v = v_cache[pages.long(), :, :, offs.long()]
    return k, v


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("style,rot", [("split_half", None), ("consecutive", None), ("split_half", 8), ("none", None)])
@pytest.mark.parametrize("bias", [True, False])
def test_rope_append(dtype, style, rot, bias):
    g = gen(3)
    T, nH, nKV, d, P, pages, theta = 9, 5, 1, 24, 16, 6, 1e6
    width = (nH + 2 * nKV) * d
    qkv = torch.randn(T, width, generator=g).to(dtype)
    b = (0.5 * torch.randn(width, generator=g)).to(dtype) if bias else None
    positions = torch.tensor([0, 1, 2, 40, 41, 300, 7, 8, 1000], dtype=torch.int32)
    slots = torch.tensor([5, 17, 95, 0, 31, 32, 64, 80, 47], dtype=torch.int32)
    kc = torch.zeros(pages, nKV, P, d, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, nKV, d, P, dtype=dtype, device=DEV)
    rd = rot or d
    inv_freq = (1.0 / torch.pow(torch.tensor(theta, dtype=torch.float64), 2.0 * torch.arange(rd // 2, dtype=torch.float64) / rd)).float()
    code = {"split_half": ops.ROPE_SPLIT_HALF, "consecutive": ops.ROPE_CONSECUTIVE, "none": ops.ROPE_NONE}[style]
    cs, sn = ops.rope_table(positions.to(DEV), inv_freq.to(DEV)) if style != "none" else (None, None)
    q = ops.rope_append(qkv.to(DEV), b.to(DEV) if bias else None, slots.to(DEV), cs, sn, code, rd, nH, nKV, d, kc, vc, P)
    x = qkv.double() + (b.double() if bias else 0)
    xq, xk, xv = x[:, : nH * d].view(T, nH, d), x[:, nH * d: (nH + nKV) * d].view(T, nKV, d), x[:, (nH + nKV) * d:].view(T, nKV, d)

    def rope(t):
        if style == "none":
            return t
        fn = pm.rope_split_half if style == "split_half" else pm.rope_consecutive
        return torch.cat([fn(t[..., :rd], positions.tolist(), theta), t[..., rd:]], dim=-1)

    # angles are formed in float (position * rounded frequency): allow that on top of the result's rounding
    t = dict(rtol=tol(dtype)["rtol"], atol=tol(dtype)["atol"] + 2e-4)
    assert torch.allclose(q.cpu().double(), rope(xq), **t)
    k_got, v_got = cache_rows(kc.cpu(), vc.cpu(), slots, P)
    assert torch.allclose(k_got.double(), rope(xk), **t)
    assert torch.allclose(v_got.double(), xv, **tol(dtype))
    written = torch.zeros(pages * P, dtype=torch.bool); written[slots.long()] = True
    assert torch.all(kc.cpu().permute(0, 2, 1, 3).reshape(pages * P, -1)[~written] == 0)   # nothing else touched
    assert torch.all(vc.cpu().permute(0, 3, 1, 2).reshape(pages * P, -1)[~written] == 0)


@pytest.mark.parametrize("d,nH,nKV", [(16, 3, 1), (32, 4, 2), (128, 7, 1)])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("P", [16, 32, 128])
def test_rope_append_in_pieces(d, nH, nKV, bias, P):
    """bfloat16, split-half over the whole head, head size a multiple of 16: the kernel's 16-byte path.  Slots:
    an aligned run of 16 (written as pieces of the transposed page), a run that starts at an odd offset, scattered
    ones, one token without a slot."""
    g = gen(31)
    T, pages, theta = 133, 256 // P, 1e4
    width = (nH + 2 * nKV) * d
    qkv = torch.randn(T, width, generator=g).to(BF16)
    b = (0.5 * torch.randn(width, generator=g)).to(BF16) if bias else None
    positions = torch.cat([torch.arange(100, 116), torch.arange(3, 11), torch.randint(0, 2000, (109,), generator=g)]).to(torch.int32)
    scattered = (48 + torch.randperm(pages * P - 48, generator=g)[:109]).tolist()
    slots = torch.tensor(list(range(32, 48)) + list(range(3, 11)) + scattered, dtype=torch.int32)
    slots[30] = -1
    kc = torch.zeros(pages, nKV, P, d, dtype=BF16, device=DEV)
    vc = torch.zeros(pages, nKV, d, P, dtype=BF16, device=DEV)
    inv_freq = (1.0 / torch.pow(torch.tensor(theta, dtype=torch.float64), 2.0 * torch.arange(d // 2, dtype=torch.float64) / d)).float()
    cs, sn = ops.rope_table(positions.to(DEV), inv_freq.to(DEV))
    q = ops.rope_append(qkv.to(DEV), b.to(DEV) if bias else None, slots.to(DEV), cs, sn, ops.ROPE_SPLIT_HALF, d, nH, nKV, d, kc, vc, P)
    x = qkv.double() + (b.double() if bias else 0)
    xq, xk, xv = x[:, : nH * d].view(T, nH, d), x[:, nH * d: (nH + nKV) * d].view(T, nKV, d), x[:, (nH + nKV) * d:].view(T, nKV, d)
    t = dict(rtol=tol(BF16)["rtol"], atol=tol(BF16)["atol"] + 2e-4)
    assert torch.allclose(q.cpu().double(), pm.rope_split_half(xq, positions.tolist(), theta), **t)
    live = slots >= 0
    k_got, v_got = cache_rows(kc.cpu(), vc.cpu(), slots[live], P)
    assert torch.allclose(k_got.double(), pm.rope_split_half(xk, positions.tolist(), theta)[live], **t)
    assert torch.allclose(v_got.double(), xv[live], **tol(BF16))
    written = torch.zeros(pages * P, dtype=torch.bool); written[slots[live].long()] = True
    assert torch.all(kc.cpu().permute(0, 2, 1, 3).reshape(pages * P, -1)[~written] == 0)   # nothing else touched
    assert torch.all(vc.cpu().permute(0, 3, 1, 2).reshape(pages * P, -1)[~written] == 0)


@pytest.mark.parametrize("seed", range(30))
def test_rope_append_random_shapes(seed):
    """Bias, rotation and cache write at shapes drawn at random: head sizes of 2-256 (the 16-byte path takes bfloat16
    heads of a multiple of 16 rotated whole; the plain path the rest), 1-40 query heads on 1-8 kv heads, either rotation
    style over the whole head or a part of it, pages of 16-128, q/k/v given whole or as partial sums, slots scattered
    with some rows unwritten; against float64."""
    import random
    rng = random.Random(1500 + seed)
    dtype = rng.choice([F32, BF16, BF16])
    d = rng.choice([16 * rng.randint(1, 16), 16 * rng.randint(1, 8), 2 * rng.randint(1, 40)])
    nKV = rng.choice([1, 2, 3, 4, 8])
    nH = nKV * rng.choice([1, 2, 5, 7])
    style = rng.choice(["split_half", "split_half", "consecutive"])
    rd = rng.choice([d, d, 2 * rng.randint(1, d // 2)])
    bias = rng.random() < 0.6
    P = rng.choice([16, 32, 64, 128])
    T = rng.choice([1, rng.randint(2, 16), rng.randint(17, 150)])
    pages, theta = -(-(T + 40) // P) + 1, rng.choice([1e4, 1e6])
    g = gen(1600 + seed)
    width = (nH + 2 * nKV) * d
    qkv = torch.randn(T, width, generator=g).to(dtype)
    b = (0.5 * torch.randn(width, generator=g)).to(dtype) if bias else None
    positions = torch.randint(0, 40000, (T,), generator=g).to(torch.int32)
    slots = torch.randperm(pages * P, generator=g)[:T].to(torch.int32)
    if T > 3:
        slots[rng.randrange(T)] = -1
    run = min(T, 16)
    if rng.random() < 0.5 and pages * P >= 32:                 # an aligned run of 16 slots: written as pieces of the page
        slots[:run] = torch.arange(16, 16 + run, dtype=torch.int32)
        taken = set(slots[:run].tolist())
        rest = [x for x in torch.randperm(pages * P, generator=g).tolist() if x not in taken][: T - run]
        slots[run:] = torch.tensor(rest, dtype=torch.int32)
    kc = torch.zeros(pages, nKV, P, d, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, nKV, d, P, dtype=dtype, device=DEV)
    inv_freq = (1.0 / torch.pow(torch.tensor(theta, dtype=torch.float64), 2.0 * torch.arange(rd // 2, dtype=torch.float64) / rd)).float()
    code = {"split_half": ops.ROPE_SPLIT_HALF, "consecutive": ops.ROPE_CONSECUTIVE}[style]
    cs, sn = ops.rope_table(positions.to(DEV), inv_freq.to(DEV))
    given = qkv.to(DEV)
    want_in = qkv.double()
    if rng.random() < 0.4:                                     # partial sums of a product cut along K
        parts = torch.randn(rng.randint(2, 8), T, width, generator=g)
        given, want_in = ops.SliceSums(parts.to(DEV), dtype), parts.double().sum(0)
    q = ops.rope_append(given, b.to(DEV) if bias else None, slots.to(DEV), cs, sn, code, rd, nH, nKV, d, kc, vc, P)
    x = want_in + (b.double() if bias else 0)
    xq, xk, xv = x[:, : nH * d].view(T, nH, d), x[:, nH * d: (nH + nKV) * d].view(T, nKV, d), x[:, (nH + nKV) * d:].view(T, nKV, d)

    def rope(t):
        fn = pm.rope_split_half if style == "split_half" else pm.rope_consecutive
        return torch.cat([fn(t[..., :rd], positions.tolist(), theta), t[..., rd:]], dim=-1)

    case = (seed, dtype, d, nH, nKV, style, rd, bias, P, T, isinstance(given, ops.SliceSums))
    # angles are formed in float (position * rounded frequency, positions up to 40,000): allow that on top of the rounding
    t = dict(rtol=tol(dtype)["rtol"], atol=tol(dtype)["atol"] + 2e-2)
    assert torch.allclose(q.cpu().double(), rope(xq), **t), case
    live = slots >= 0
    k_got, v_got = cache_rows(kc.cpu(), vc.cpu(), slots[live], P)
    assert torch.allclose(k_got.double(), rope(xk)[live], **t), case
    assert torch.allclose(v_got.double(), xv[live], **tol(dtype)), case
    written = torch.zeros(pages * P, dtype=torch.bool); written[slots[live].long()] = True
    assert torch.all(kc.cpu().permute(0, 2, 1, 3).reshape(pages * P, -1)[~written] == 0), case   # nothing else touched
    assert torch.all(vc.cpu().permute(0, 3, 1, 2).reshape(pages * P, -1)[~written] == 0), case


def test_rope_queries_only():
    g = gen(4)
    T, nH, d = 4, 3, 16
    qo = torch.randn(T, nH * d, generator=g)
    pos = torch.tensor([3, 4, 5, 6], dtype=torch.int32)
    inv = (1.0 / torch.pow(torch.tensor(1e4, dtype=torch.float64), 2.0 * torch.arange(d // 2, dtype=torch.float64) / d)).float()
    cs, sn = ops.rope_table(pos.to(DEV), inv.to(DEV))
    q = ops.rope_append(qo.to(DEV), None, None, cs, sn, ops.ROPE_SPLIT_HALF, d, nH, 0, d, None, None, 16)
    assert torch.allclose(q.cpu().double(), pm.rope_split_half(qo.double().view(T, nH, d), pos.tolist(), 1e4), atol=1e-5)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_swiglu(dtype):
    g = gen(5)
    gu = (3 * torch.randn(5, 2 * 37, generator=g)).to(dtype)
    out = ops.swiglu(gu.to(DEV)).cpu().double()
    gate, up = gu.double()[:, :37], gu.double()[:, 37:]
    assert torch.allclose(out, gate / (1 + torch.exp(-gate)) * up, **tol(dtype))
    out = ops.swiglu(gu.to(DEV), interleaved=True).cpu().double()
    gate, up = gu.double()[:, 0::2], gu.double()[:, 1::2]
    assert torch.allclose(out, gate / (1 + torch.exp(-gate)) * up, **tol(dtype))


@pytest.mark.parametrize("M,N,K", [(1, 50, 33), (7, 64, 16), (65, 130, 257), (130, 3, 1000)])
@pytest.mark.parametrize("adtype", [F32, BF16])
def test_gemm_f32(M, N, K, adtype):
    g = gen(6)
    x = torch.randn(M, K, generator=g).to(adtype)
    w = torch.randn(N, K, generator=g)
    b = torch.randn(N, generator=g)
    out = ops.gemm_f32(x.to(DEV), w.to(DEV), b.to(DEV), F32).cpu().double()
    want = x.double() @ w.double().t() + b.double()
    assert torch.allclose(out, want, rtol=1e-5, atol=1e-5 * math.sqrt(K))
    # a row's result does not depend on how many rows are in the product
    one = ops.gemm_f32(x[:1].contiguous().to(DEV), w.to(DEV), b.to(DEV), F32).cpu().double()
    assert torch.equal(one[0], out[0])


def test_gemm_f32_is_true_32_bit():
    """Products whose exact value needs more than 10 or 8 mantissa bits survive: no reduced-precision matrix mode."""
    K = 64
    x = torch.full((1, K), 1.0 + 2.0 ** -12)
    w = torch.full((3, K), 1.0 + 2.0 ** -11)
    out = ops.gemm_f32(x.to(DEV), w.to(DEV), None, F32).cpu().double()
    want = (x.double() @ w.double().t())
    assert torch.allclose(out, want, rtol=3e-7, atol=0)
    assert not torch.allclose(out, torch.full_like(out, float(K)), rtol=1e-4, atol=0)


# ---- attention ------------------------------------------------------------------------------
def paged_case(seed, lens_q, lens_past, nH, nKV, d, P, dtype, window=None, n_pages=None, sharp=None, garbage=False):
    """Random q/k/v for several requests, keys and values scattered into shuffled pages.
    Returns device operands and the plain float64 result for this step's rows.
    ``garbage``: everything of the cache that no request holds (pages no table names, the slots of a last page past
    its request's length) is filled with what a kernel must never let through: NaN keys and values of +-1e30."""
    g = gen(seed)
    R = len(lens_q)
    kv_lens = [a + b for a, b in zip(lens_q, lens_past)]
    blocks = [-(-n // P) for n in kv_lens]
    n_pages = n_pages or sum(blocks) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    kc = torch.zeros(n_pages, nKV, P, d, dtype=dtype)
    vc = torch.zeros(n_pages, nKV, d, P, dtype=dtype)
    if garbage:
        kc.fill_(float("nan"))
        vc.copy_(torch.where(torch.rand(vc.shape, generator=g) < 0.5, 1e30, -1e30))
    width = max(blocks)
    table = torch.full((R, width), -1, dtype=torch.int32)
    qs, outs, row_req, positions = [], [], [], []
    for r in range(R):
        n, nq = kv_lens[r], lens_q[r]
        k = torch.randn(n, nKV, d, generator=g).to(dtype)
        v = torch.randn(n, nKV, d, generator=g).to(dtype)
        q = torch.randn(nq, nH, d, generator=g).to(dtype)
        if sharp is not None:
            # plant one far key that every query of head 0 must find: a wrong page, mask or offset changes the result
            j = sharp if sharp >= 0 else n + sharp
            if 0 <= j < n:
                k[j, 0] = (4.0 * q[-1, 0] / q[-1, 0].float().norm() * math.sqrt(d)).to(dtype)
        pages = [perm.pop() for _ in range(blocks[r])]
        table[r, : blocks[r]] = torch.tensor(pages, dtype=torch.int32)
        for j in range(n):
            kc[pages[j // P], :, j % P, :] = k[j]
            vc[pages[j // P], :, :, j % P] = v[j]
        qpos = list(range(n - nq, n))
        outs.append(pm.attention(q.double(), k.double(), v.double(), window=window, q_positions=qpos, k_positions=list(range(n))))
        qs.append(q); row_req += [r] * nq; positions += qpos
    q_all = torch.cat(qs)
    want = torch.cat(outs).reshape(q_all.shape[0], nH * d)
    dev = lambda t: t.to(DEV)
    return (dev(q_all), dev(kc), dev(vc), dev(torch.tensor(row_req, dtype=torch.int32)),
            dev(torch.tensor(positions, dtype=torch.int32)), dev(table)), want, dict(q_lens=lens_q, kv_lens=kv_lens)


def close_rows(out, want):
    """Row attention against float64: element by element, and the largest error against the largest value (a bound
    that follows the data: outputs here are 0.1-1 in size)."""
    return torch.allclose(out, want, rtol=1e-2, atol=1e-2) and float((out - want).abs().max()) <= 1e-2 * float(want.abs().max())


ATTN_CASES = [
    # lens_q, lens_past, nH, nKV, d, P, window, sharp
    ([1], [0], 4, 2, 16, 16, None, None),                       # a single key: the output is its value
    ([5, 1, 2], [0, 63, 17], 4, 2, 16, 16, None, None),
    ([33, 1], [40, 200], 7, 1, 40, 16, None, 3),                # MQA 7:1, head size 40, far planted key
    ([64, 2, 1, 16], [0, 62, 129, 48], 6, 3, 32, 16, None, None),
    ([20, 1, 3], [30, 100, 45], 6, 3, 32, 16, 24, None),        # window's edge inside and across pages
    ([1, 1], [70, 23], 2, 2, 64, 32, 5, -5),                    # planted key at the window's last visible place
    ([1, 1], [70, 23], 2, 2, 64, 32, 5, -6),                    # ... and just outside it
    ([7], [250], 28, 4, 128, 16, None, 0),                      # the 7B head layout, planted key at position 0
]


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("case", ATTN_CASES)
def test_attention_plain(dtype, case):
    lens_q, lens_past, nH, nKV, d, P, window, sharp = case
    (q, kc, vc, row_req, positions, table), want, _ = paged_case(7, lens_q, lens_past, nH, nKV, d, P, dtype, window, sharp=sharp)
    out = ops.attention_plain(q, kc, vc, row_req, positions, table, window, 1.0 / math.sqrt(d)).cpu().double()
    t = dict(rtol=1e-4, atol=1e-5) if dtype == F32 else dict(rtol=1e-2, atol=1e-2)
    assert torch.isfinite(out).all()
    assert torch.allclose(out, want, **t), float((out - want).abs().max())


@pytest.mark.parametrize("seed", range(24))
def test_attention_plain_random_cases(seed):
    """The plain attention kernel (the 32-bit path's, and the reference beside the matrix-core ones) at shapes drawn at
    random: head sizes of 1-256, pages of any size from 1 (no power of two), 1-3 requests of 1-60 rows behind pasts of
    0-400 keys, with and without a window and a planted far key; float32 and bfloat16, against float64."""
    import random
    rng = random.Random(1700 + seed)
    dtype = rng.choice([F32, F32, BF16])
    d = rng.choice([rng.randint(1, 24), 8 * rng.randint(1, 32), rng.randint(25, 256)])
    P = rng.choice([1, 3, 16, 24, 50, 64])
    nKV = rng.choice([1, 2, 3])
    nH = nKV * rng.choice([1, 2, 4, 7])
    n_req = rng.randint(1, 3)
    lens_q = [rng.randint(1, rng.choice([2, 20, 60])) for _ in range(n_req)]
    lens_past = [rng.choice([0, rng.randint(1, 60), rng.randint(61, 400)]) for _ in range(n_req)]
    window = rng.choice([None, None, rng.randint(1, 200)])
    sharp = rng.choice([None, 0, 2, -3])
    (q, kc, vc, row_req, positions, table), want, _ = paged_case(1800 + seed, lens_q, lens_past, nH, nKV, d, P, dtype, window, sharp=sharp)
    out = ops.attention_plain(q, kc, vc, row_req, positions, table, window, 1.0 / math.sqrt(d))
    t = dict(rtol=1e-4, atol=1e-5) if dtype == F32 else dict(rtol=1e-2, atol=1e-2)
    assert torch.allclose(out.cpu().double(), want, **t), (seed, dtype, d, P, nH, nKV, lens_q, lens_past, window, sharp,
                                                            float((out.cpu().double() - want).abs().max()))


@pytest.mark.parametrize("seed", range(16))
def test_gemm_f32_random_shapes(seed):
    """The 32-bit product at shapes drawn at random (1-300 rows, 1-3,000 weight rows, any K up to 5,000), float32 or
    bfloat16 activations, with and without a bias; against float64, and the same row gives the same bits whatever else
    is in the batch."""
    import random
    rng = random.Random(1900 + seed)
    M = rng.choice([1, rng.randint(2, 20), rng.randint(21, 300)])
    N = rng.choice([rng.randint(1, 40), rng.randint(41, 3000)])
    K = rng.choice([rng.randint(1, 70), rng.randint(71, 5000)])
    adtype = rng.choice([F32, BF16])
    g = gen(2000 + seed)
    x = torch.randn(M, K, generator=g).to(adtype)
    w = torch.randn(N, K, generator=g) * 0.2
    b = torch.randn(N, generator=g) if rng.random() < 0.5 else None
    want = x.double() @ w.double().t() + (b.double() if b is not None else 0)
    got = ops.gemm_f32(x.to(DEV), w.to(DEV), b.to(DEV) if b is not None else None)
    assert got.dtype == adtype or got.dtype == F32
    t = dict(rtol=1e-4, atol=2e-5 * max(1.0, K ** 0.5)) if got.dtype == F32 else dict(rtol=1e-2, atol=0.05 * max(1.0, (K / 500) ** 0.5))
    assert torch.allclose(got.cpu().double(), want, **t), (M, N, K, adtype, float((got.cpu().double() - want).abs().max()))
    r = rng.randrange(M)
    alone = ops.gemm_f32(x[r:r + 1].to(DEV), w.to(DEV), b.to(DEV) if b is not None else None)
    assert torch.equal(alone[0], got[r]), (M, N, K, r)


# ---- sampling -------------------------------------------------------------------------------
def test_argmax_lowest_index_wins_ties():
    l = torch.zeros(3, 1500)
    l[0, [700, 20, 1400]] = 5.0
    l[1, 1499] = 1.0
    l[2] = -float("inf")
    assert ops.argmax(l.to(DEV)).cpu().tolist() == [20, 1499, 0]
    g = gen(8)
    r = torch.randn(6, 152064, generator=g)
    assert ops.argmax(r.to(DEV)).cpu().tolist() == r.argmax(-1).tolist()


def test_penalties_and_logit_bias():
    l = torch.tensor([[2.0, -2.0, 1.0, 0.5], [1.0, 1.0, 1.0, 1.0]])
    d = l.to(DEV)
    i32 = lambda *v: torch.tensor(v, dtype=torch.int32, device=DEV)
    f32 = lambda *v: torch.tensor(v, dtype=torch.float32, device=DEV)
    ops.apply_penalties(d, i32(0, 0, 1), i32(0, 1, 3), i32(1, 2, 4), f32(2.0, 1.0), f32(0.25, 0.5), f32(0.5, 0.0))
    want0 = pm.apply_penalties(l[0], [0, 1, 1], 2.0, 0.25, 0.5)
    want1 = pm.apply_penalties(l[1], [3, 3, 3, 3], 1.0, 0.5, 0.0)
    assert torch.allclose(d.cpu(), torch.stack([want0, want1]))
    ops.add_logit_bias(d, i32(1), i32(2), f32(-100.0))
    assert float(d[1, 2]) == pytest.approx(1.0 - 100.0)


@pytest.mark.parametrize("V", [1000, 152064])
def test_sample_matches_the_plain_rule(V):
    g = gen(9)
    R = 12
    logits = 3.0 * torch.randn(R, V, generator=g)
    temps = torch.tensor([0.0, 1.0, 0.7, 1.3, 1.0, 1.0, 0.8, 1.0, 1.0, 0.5, 1.0, 2.0])
    top_k = torch.tensor([0, 0, 0, 40, 0, 5, 50, 0, 1, 0, 0, 0], dtype=torch.int32)
    top_p = torch.tensor([1.0, 1.0, 0.9, 1.0, 0.3, 0.95, 0.8, 1.0, 1.0, 1.0, 0.999, 1.0])
    min_p = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.02, 0.1, 0.0, 0.0, 0.0, 0.0])
    u = torch.rand(R, generator=g)
    got = ops.sample(logits.to(DEV), temps.to(DEV), top_k.to(DEV), top_p.to(DEV), min_p.to(DEV), u.to(DEV)).cpu().tolist()
    assert got[0] == int(logits[0].argmax())
    assert got[8] == int(logits[8].argmax())            # top_k = 1
    for r in range(1, R):
        w = pm.filtered_probs(logits[r], float(temps[r]), int(top_k[r]), float(top_p[r]), float(min_p[r]))
        assert w[got[r]] > 0, (r, "a filtered-out token was drawn")
        cum = torch.cumsum(w, 0) / w.sum()
        lo = float(cum[got[r] - 1]) if got[r] > 0 else 0.0
        hi = float(cum[got[r]])
        assert lo - 1e-4 <= float(u[r]) <= hi + 1e-4, (r, got[r], lo, float(u[r]), hi)


@pytest.mark.parametrize("seed", range(20))
def test_sample_random_vocabularies_and_filters(seed):
    """The draw against the plain rule at vocabularies of 2-200,000 (no multiple of anything), 1-40 rows, and
    temperatures, top-k, top-p and min-p drawn at random, several filters at once; the greedy rows beside them."""
    import random
    rng = random.Random(1300 + seed)
    V = rng.choice([rng.randint(2, 70), rng.randint(71, 5000), rng.randint(5001, 200000)])
    R = rng.randint(1, 40)
    g = gen(1400 + seed)
    logits = rng.choice([1.0, 3.0, 8.0]) * torch.randn(R, V, generator=g)
    temps = torch.tensor([rng.choice([0.0, 0.3, 0.7, 1.0, 1.5, 2.5]) for _ in range(R)])
    top_k = torch.tensor([rng.choice([0, 0, 1, 2, 5, 40, 1000]) for _ in range(R)], dtype=torch.int32)
    top_p = torch.tensor([rng.choice([1.0, 1.0, 0.999, 0.9, 0.5, 0.1]) for _ in range(R)])
    min_p = torch.tensor([rng.choice([0.0, 0.0, 0.01, 0.1, 0.5]) for _ in range(R)])
    u = torch.rand(R, generator=g)
    got = ops.sample(logits.to(DEV), temps.to(DEV), top_k.to(DEV), top_p.to(DEV), min_p.to(DEV), u.to(DEV)).cpu().tolist()
    assert ops.argmax(logits.to(DEV)).cpu().tolist() == logits.argmax(-1).tolist()
    for r in range(R):
        case = (seed, V, r, float(temps[r]), int(top_k[r]), float(top_p[r]), float(min_p[r]))
        assert 0 <= got[r] < V, case
        if float(temps[r]) == 0.0 or int(top_k[r]) == 1:
            assert got[r] == int(logits[r].argmax()), case
            continue
        w = pm.filtered_probs(logits[r], float(temps[r]), int(top_k[r]), float(top_p[r]), float(min_p[r]))
        assert w[got[r]] > 0, (case, "a filtered-out token was drawn")
        cum = torch.cumsum(w, 0) / w.sum()
        lo = float(cum[got[r] - 1]) if got[r] > 0 else 0.0
        assert lo - 1e-4 <= float(u[r]) <= float(cum[got[r]]) + 1e-4, (case, got[r], lo, float(u[r]), float(cum[got[r]]))


SAMPLE_SHAPES = [
    # (name, V, logits builder, temperature, top_k, top_p, min_p)
    ("flat under top-p", 40001, lambda g, V: 0.01 * torch.randn(V, generator=g), 1.0, 0, 0.9, 0.0),
    ("flat under a wide top-k", 40001, lambda g, V: 0.01 * torch.randn(V, generator=g), 0.7, 20000, 1.0, 0.0),
    ("flat under both", 30003, lambda g, V: 0.02 * torch.randn(V, generator=g), 1.0, 12000, 0.95, 0.0),
    ("one token far above", 152064, lambda g, V: torch.randn(V, generator=g).index_fill_(0, torch.tensor([77777]), 40.0), 1.0, 50, 0.9, 0.0),
    ("mostly masked", 9999, lambda g, V: torch.where(torch.rand(V, generator=g) < 0.9, torch.tensor(-float("inf")), 2.0 * torch.randn(V, generator=g)), 0.8, 40, 0.9, 0.0),
    ("top-p alone, peaked", 152064, lambda g, V: 6.0 * torch.randn(V, generator=g), 0.6, 0, 0.95, 0.0),
    ("top-p alone, wide", 152064, lambda g, V: 1.5 * torch.randn(V, generator=g), 1.0, 0, 0.9, 0.0),
    # a nearly flat row is all candidates: as many as fit, and one more (which takes the passes over the whole row)
    ("as many tokens as candidates fit", 3072, lambda g, V: 0.05 * torch.randn(V, generator=g), 1.0, 3000, 0.999, 0.0),
    ("one token more than candidates fit", 3073, lambda g, V: 0.05 * torch.randn(V, generator=g), 1.0, 3000, 0.999, 0.0),
    ("wide nucleus inside a wide top-k", 100003, lambda g, V: 0.7 * torch.randn(V, generator=g), 1.3, 60000, 0.97, 0.0),
]


@pytest.mark.parametrize("case", range(len(SAMPLE_SHAPES)), ids=[c[0] for c in SAMPLE_SHAPES])
def test_sample_rows_of_every_shape(case):
    """Rows that the thresholds' two ways take differently: few candidates above the thresholds' bins (gathered and
    bisected by one wave) and more than fit (bisected over the whole row), equal weights (kept or dropped together), rows
    that are mostly masked, and a vocabulary that is no multiple of four (rows that start at any address)."""
    name, V, build, temp, k, p, mp = SAMPLE_SHAPES[case]
    g = gen(1500 + case)
    R = 5
    logits = torch.stack([build(g, V) for _ in range(R)])
    u = torch.tensor([0.0, 0.25, 0.5, 0.75, 0.999999])
    full = lambda v, dt: torch.full((R,), v, dtype=dt, device=DEV)
    args = (logits.to(DEV), full(temp, torch.float32), full(k, torch.int32), full(p, torch.float32), full(mp, torch.float32), u.to(DEV))
    got = ops.sample(*args).cpu().tolist()
    assert ops.sample(*args, any_greedy=False).cpu().tolist() == got        # (no row here has temperature 0)
    # the same rows among twenty: large vocabularies are then drawn by one workgroup a row instead of sixteen
    many = [torch.cat([t, t, t, t]) for t in args]
    among = ops.sample(*many).cpu().tolist()
    assert among[:R] == among[R:2 * R] == among[3 * R:]
    for r in range(R):
        w = pm.filtered_probs(logits[r], temp, k, p, mp)
        assert w[got[r]] > 0 and w[among[r]] > 0, (name, r, "a filtered-out token was drawn")
        if among[r] != got[r]:                   # only a draw on the edge between two kept tokens may differ between the forms
            cum = torch.cumsum(w.double(), 0) / w.double().sum()
            a, b = min(among[r], got[r]), max(among[r], got[r])
            assert abs(float(cum[a]) - float(u[r])) < 1e-4 and float(w[a + 1:b].sum()) == 0.0, (name, r, among[r], got[r])
        cum = torch.cumsum(w.double(), 0) / w.double().sum()
        lo = float(cum[got[r] - 1]) if got[r] > 0 else 0.0
        assert lo - 1e-4 <= float(u[r]) <= float(cum[got[r]]) + 1e-4, (name, r, got[r], lo, float(u[r]), float(cum[got[r]]))


@pytest.mark.parametrize("V,every,k,p", [(5000, 1, 10, 0.5), (20000, 7, 100, 0.8), (152064, 3, 0, 0.3)])
def test_sample_keeps_equal_weights_together(V, every, k, p):
    """Tokens of equal weight are kept or dropped together: with every ``every``-th token at one logit and the rest far
    below, top-k and top-p smaller than that group keep all of it, and the draw falls evenly over it.  (All threads
    of a wave then add to one bin of the histogram: the slowest row there is.)"""
    logits = torch.where(torch.arange(V) % every == 0, torch.tensor(3.0), torch.tensor(-9.0)).repeat(4, 1)
    u = torch.tensor([0.0, 0.3, 0.6, 0.95])
    full = lambda v, dt: torch.full((4,), v, dtype=dt, device=DEV)
    got = ops.sample(logits.to(DEV), full(1.0, torch.float32), full(k, torch.int32), full(p, torch.float32),
                     full(0.0, torch.float32), u.to(DEV)).cpu().tolist()
    n = (V + every - 1) // every
    for r in range(4):
        assert got[r] % every == 0, (r, got[r])
        assert abs(got[r] // every - float(u[r]) * n) <= 1 + 1e-4 * n, (r, got[r], float(u[r]) * n)


def test_sample_histogram_follows_the_probabilities():
    g = gen(10)
    V, N = 50, 4000
    logits = torch.randn(V, generator=g)
    rows = logits.repeat(N, 1)
    ones = torch.ones(N)
    u = torch.rand(N, generator=g)
    got = ops.sample(rows.to(DEV), ones.to(DEV), torch.zeros(N, dtype=torch.int32, device=DEV), ones.to(DEV),
                     torch.zeros(N, device=DEV), u.to(DEV)).cpu()
    freq = torch.bincount(got.long(), minlength=V).double() / N
    p = torch.softmax(logits.double(), -1)
    chi2 = float((N * (freq - p) ** 2 / p).sum())
    assert chi2 < 100.0, chi2                            # 49 degrees of freedom: 100 is far in the tail


# ---- matrix-core attention --------------------------------------------------------------------
MFMA_CASES = [c for c in ATTN_CASES if c[4] % 16 == 0 and c[4] <= 128] + [
    ([100, 64, 17], [0, 100, 300], 4, 2, 16, 16, None, None),      # tiles that end inside a page, head size 16
    ([130], [61], 8, 2, 48, 16, None, 5),                          # head size 48 (half-empty last step), planted key
    ([70, 1], [200, 1000], 28, 4, 128, 16, None, None),            # 7B head layout
    ([64, 64], [0, 192], 3, 3, 64, 32, 40, None),                  # window across tiles, pages of 32
    ([33], [90], 40, 2, 32, 16, None, 64),                         # 20 query heads per kv head: two passes of 16
    ([2, 70], [9000, 8200], 4, 2, 64, 16, None, 4500),             # long contexts: many splits, planted key mid-way
    ([1, 1], [5000, 300], 2, 1, 128, 64, 1000, None),              # a window inside a long context, pages of 64
    ([40, 3], [30, 170], 6, 3, 96, 16, None, 20),                  # head sizes between the prebuilt ones
    ([90], [75], 5, 1, 80, 32, 50, None),
    # head size 128, where tiles of 128 rows are the kernel that loads straight into LDS: requests that end inside a
    # tile, pages of 32, a window across tiles, a long past with a planted key, seven query heads to a kv head
    ([300, 130], [500, 0], 8, 2, 128, 32, None, 100),
    ([129], [260], 4, 4, 128, 16, 200, None),
    ([260, 17], [3000, 40], 14, 2, 128, 16, None, 1500),
    # pages larger than a tile of 64 keys: where a tile's keys start inside their page changes from tile to tile
    ([200, 40], [300, 1000], 4, 2, 128, 128, None, 50),
    ([150], [700], 6, 2, 128, 256, 500, None),
    # steps of single tokens (every request one row: the row kernel then looks its pages up before it knows the position)
    ([1] * 9, [0, 5, 130, 700, 64, 31, 2000, 15, 16], 28, 4, 128, 16, None, 3),
    ([1] * 5, [300, 1, 1030, 77, 512], 6, 3, 32, 64, None, None),
]


def run_rows(q, kc, vc, row_req, positions, table, window, scale, rows=None, chunk=128, waves=0, extra_splits=0):
    """``waves`` 0: one wave per split of ``chunk`` keys and the merge launch (``extra_splits``: the grid reaches that
    many splits past the longest row, as a captured step's does); 1-8: one workgroup of that many waves per (row, kv head).
    Where every request brings one row the kernel is told so, as the engine tells it."""
    T, nH, d = q.shape
    req_is_row = bool(torch.equal(row_req.cpu(), torch.arange(T, dtype=torch.int32)))
    out = torch.zeros(T, nH * d, dtype=q.dtype, device=DEV)
    n = T if rows is None else rows.shape[0]
    max_kv = int(positions.max()) + 1
    ops.attention_rows(q, kc, vc, out, rows, n, row_req, positions, table, window, scale, chunk,
                       -(-max_kv // chunk) + extra_splits, waves, req_is_row)
    return out


@pytest.mark.parametrize("chunk,waves", [(32, 0), (128, 0), (1024, 0), (128, 1), (128, 2), (128, 3), (128, 4), (128, 8)])
@pytest.mark.parametrize("case", MFMA_CASES)
def test_attention_rows(case, chunk, waves):
    """Every launch shape of the row kernel: one wave per split and the merge launch, and one workgroup of several
    waves per (row, kv head) whose waves share the row's keys and meet in LDS."""
    lens_q, lens_past, nH, nKV, d, P, window, sharp = case
    (q, kc, vc, row_req, positions, table), want, _ = paged_case(7, lens_q, lens_past, nH, nKV, d, P, BF16, window, sharp=sharp)
    waves = ops.row_waves_fit(nH, nKV, d, waves)
    out = run_rows(q, kc, vc, row_req, positions, table, window, 1.0 / math.sqrt(d), chunk=chunk, waves=waves)
    assert torch.isfinite(out).all()
    assert close_rows(out.cpu().double(), want), float((out.cpu().double() - want).abs().max())
    # the same launch again, with a grid that reaches past the longest row: the same bits
    again = run_rows(q, kc, vc, row_req, positions, table, window, 1.0 / math.sqrt(d), chunk=chunk, waves=waves, extra_splits=3)
    assert torch.equal(again, out)


@pytest.mark.parametrize("seed", range(30))
def test_attention_rows_random_cases(seed):
    """The row kernels at shapes drawn at random: one to five requests of 1-15 rows behind pasts of 0-2,500 keys, head
    sizes 16-128, pages of 16-256, with and without a window, 1-20 query heads to a kv head, splits of 32-1,024 keys
    with the merge launch or workgroups of 1-8 waves that take a row whole, all rows or a subset; against float64."""
    import random
    rng = random.Random(500 + seed)
    d = rng.choice([16, 32, 64, 128])
    P = rng.choice([16, 16, 32, 64, 128, 256])
    nKV = rng.choice([1, 2, 3])
    nH = nKV * rng.choice([1, 2, 5, 7, 8, 20])
    n_req = rng.randint(1, 5)
    lens_q = [rng.randint(1, 15) for _ in range(n_req)]
    lens_past = [rng.choice([0, rng.randint(1, 200), rng.randint(200, 2500)]) for _ in range(n_req)]
    window = rng.choice([None, None, rng.randint(5, 900)])
    chunk = rng.choice([32, 64, 128, 256, 1024])
    waves = ops.row_waves_fit(nH, nKV, d, rng.choice([1, 2, 4, 5, 8])) if seed % 2 else 0
    (q, kc, vc, row_req, positions, table), want, _ = paged_case(600 + seed, lens_q, lens_past, nH, nKV, d, P, BF16, window,
                                                                 sharp=rng.choice([None, 2, -50]))
    T = q.shape[0]
    rows = None
    if rng.random() < 0.4 and T > 1:
        rows = torch.tensor(sorted(rng.sample(range(T), rng.randint(1, T - 1))), dtype=torch.int32, device=DEV)
    out = run_rows(q, kc, vc, row_req, positions, table, window, 1.0 / math.sqrt(d), rows=rows, chunk=chunk, waves=waves,
                   extra_splits=seed % 3).cpu().double()
    sel = list(range(T)) if rows is None else rows.cpu().tolist()
    assert torch.isfinite(out).all()
    assert close_rows(out[sel], want[sel]), (seed, d, P, nH, nKV, lens_q, lens_past, window, chunk, waves,
                                             float((out[sel] - want[sel]).abs().max()))
    rest = [i for i in range(T) if i not in sel]
    assert torch.all(out[rest] == 0)


def test_attention_rows_subset_leaves_other_rows_alone():
    (q, kc, vc, row_req, positions, table), want, _ = paged_case(8, [5, 1, 3], [10, 99, 40], 6, 2, 32, 16, BF16)
    rows = torch.tensor([5, 0, 8], dtype=torch.int32, device=DEV)
    out = run_rows(q, kc, vc, row_req, positions, table, None, 1.0 / math.sqrt(32), rows=rows).cpu().double()
    assert close_rows(out[[5, 0, 8]], want[[5, 0, 8]])
    rest = [i for i in range(9) if i not in (5, 0, 8)]
    assert torch.all(out[rest] == 0)


@pytest.mark.parametrize("qt", [1, 2])
@pytest.mark.parametrize("split_chunk", [0, 64, 192])
@pytest.mark.parametrize("case", MFMA_CASES)
def test_attention_tiles(case, qt, split_chunk):
    """``split_chunk``: the keys cut into splits of that many, run as workgroups of their own and merged."""
    lens_q, lens_past, nH, nKV, d, P, window, sharp = case
    (q, kc, vc, row_req, positions, table), want, info = paged_case(7, lens_q, lens_past, nH, nKV, d, P, BF16, window, sharp=sharp)
    T = q.shape[0]
    out = torch.zeros(T, nH * d, dtype=BF16, device=DEV)
    q_len = torch.tensor(info["q_lens"], dtype=torch.int32)
    q_start = torch.cumsum(q_len, 0, dtype=torch.int32) - q_len
    tiles = [(r, q0) for r, n in enumerate(info["q_lens"]) for q0 in range(0, n, ops.attention_tile_rows(d, qt))]
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    splits = {}
    if split_chunk:
        splits = dict(chunk=split_chunk, max_splits=-(-max(info["kv_lens"]) // split_chunk),
                      rows=torch.arange(T, dtype=torch.int32, device=DEV), row_req=row_req, positions=positions)
    call = (q, kc, vc, out, dev([t[0] for t in tiles]), dev([t[1] for t in tiles]), q_start.to(DEV),
            q_len.to(DEV), dev(info["kv_lens"]), table, window, 1.0 / math.sqrt(d), qt)
    ops.attention_tiles(*call, **splits)
    plain_order = out.clone()
    out = out.cpu().double()
    assert torch.isfinite(out).all()
    assert close_rows(out, want), float((out - want).abs().max())
    # the same launch with its workgroups in the balanced order, and in a shuffled one with gaps: the same bits
    import numpy as np
    from inferflux_amd.kernels.attention import tile_order
    first = np.asarray([info["kv_lens"][r] - info["q_lens"][r] + q0 for r, q0 in tiles])
    last = np.asarray([min(f + ops.attention_tile_rows(d, qt), info["kv_lens"][r]) - 1 for f, (r, _) in zip(first, tiles)])
    n_splits = splits.get("max_splits", 1)
    balanced = tile_order(first, last, nH, window, n_splits, split_chunk, period=3)
    n_items = len(tiles) * nH * n_splits
    assert sorted(balanced[balanced >= 0].tolist()) == list(range(n_items))
    rng = np.random.default_rng(3)
    shuffled = np.full(8 * (n_items // 8 + 3), -1, np.int32)
    shuffled[rng.permutation(shuffled.shape[0])[:n_items]] = rng.permutation(n_items)
    for order in (balanced, shuffled):
        again = torch.zeros(T, nH * d, dtype=BF16, device=DEV)
        ops.attention_tiles(*call[:3], again, *call[4:], **splits, order=torch.from_numpy(order).to(DEV))
        assert torch.equal(again, plain_order)


@pytest.mark.parametrize("seed", range(40))
def test_attention_tiles_random_cases(seed):
    """The tile kernels at shapes drawn at random (the first 24: tiles of 128 rows at head size 128, the kernel that
    loads its tiles straight into LDS; the others: either tiling at head sizes 16-128): several requests of 16-400
    rows behind pasts of 0-1,500 keys, pages of 16-256, with and without a window, one to eight query heads to a kv
    head, whole and in key splits, in the engine's workgroup order; against float64."""
    import random
    import numpy as np
    from inferflux_amd.kernels.attention import tile_order
    rng = random.Random(100 + seed)
    d, P = 128, rng.choice([16, 16, 32, 64, 128, 256])
    qt = 2
    if seed >= 24:
        d, qt = rng.choice([16, 32, 64, 128]), rng.choice([1, 2])
    nKV = rng.choice([1, 2, 4])
    nH = nKV * rng.choice([1, 2, 5, 7, 8])
    n_req = rng.randint(1, 3)
    lens_q = [rng.randint(16, rng.choice([40, 150, 400])) for _ in range(n_req)]
    lens_past = [rng.choice([0, rng.randint(1, 300), rng.randint(300, 1500)]) for _ in range(n_req)]
    window = rng.choice([None, None, rng.randint(20, 700)])
    sharp = rng.choice([None, 3, -200])
    (q, kc, vc, row_req, positions, table), want, info = paged_case(300 + seed, lens_q, lens_past, nH, nKV, d, P, BF16, window, sharp=sharp)
    T = q.shape[0]
    q_len = torch.tensor(info["q_lens"], dtype=torch.int32)
    q_start = torch.cumsum(q_len, 0, dtype=torch.int32) - q_len
    rows = ops.attention_tile_rows(d, qt)
    tiles = [(r, q0) for r, n in enumerate(info["q_lens"]) for q0 in range(0, n, rows)]
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    first = np.asarray([info["kv_lens"][r] - info["q_lens"][r] + q0 for r, q0 in tiles])
    last = np.asarray([min(f + rows, info["kv_lens"][r]) - 1 for f, (r, _) in zip(first, tiles)])
    for chunk in (0, rng.choice([64, 128, 320, 512])):
        splits = {}
        n_splits = 1
        if chunk:
            n_splits = -(-max(info["kv_lens"]) // chunk)
            splits = dict(chunk=chunk, max_splits=n_splits, rows=torch.arange(T, dtype=torch.int32, device=DEV), row_req=row_req,
                          positions=positions)
        order = torch.from_numpy(tile_order(first, last, nH, window, n_splits, chunk)).to(DEV)
        out = torch.zeros(T, nH * d, dtype=BF16, device=DEV)
        ops.attention_tiles(q, kc, vc, out, dev([t[0] for t in tiles]), dev([t[1] for t in tiles]), q_start.to(DEV), q_len.to(DEV),
                            dev(info["kv_lens"]), table, window, 1.0 / math.sqrt(d), qt, order=order, **splits)
        out = out.cpu().double()
        assert torch.isfinite(out).all()
        assert close_rows(out, want), (seed, chunk, d, qt, lens_q, lens_past, nH, nKV, P, window, float((out - want).abs().max()))


GARBAGE_CASES = [
    # lens_q, lens_past, nH, nKV, d, P, window: requests that end inside a page, a window that starts inside one
    ([1, 1, 3], [70, 1000, 45], 6, 3, 32, 16, None),
    ([1, 1], [500, 23], 14, 2, 128, 64, 100),
    ([70, 20], [200, 1000], 28, 4, 128, 16, None),
    ([130, 33], [61, 900], 8, 2, 128, 32, 300),
    ([100, 17], [300, 41], 4, 2, 64, 128, 77),
]


@pytest.mark.parametrize("case", GARBAGE_CASES)
def test_attention_kernels_let_nothing_through_from_outside_tables_and_lengths(case):
    """The cache holds NaN keys and values of +-1e30 wherever no request's table and length reach (other pages, the
    rest of a last page), and inside the pages before a window.  Every matrix-core kernel (rows in splits and whole,
    tiles of both heights, whole and in key splits) and the plain one still give the float64 result: what lies outside
    is dropped by a select on the score, never multiplied in."""
    lens_q, lens_past, nH, nKV, d, P, window = case
    (q, kc, vc, row_req, positions, table), want, info = paged_case(21, lens_q, lens_past, nH, nKV, d, P, BF16, window, garbage=True)
    scale = 1.0 / math.sqrt(d)
    T = q.shape[0]
    if window:           # the pages wholly before every window of a request: as a windowed cache group hands them back
        first_needed = [(n - nq - window + 1) // P for n, nq in zip(info["kv_lens"], info["q_lens"])]
        for r, b in enumerate(first_needed):
            for blk in range(max(b, 0)):
                kc[int(table[r, blk])] = float("nan")
                vc[int(table[r, blk])] = 1e30
    out = ops.attention_plain(q, kc, vc, row_req, positions, table, window, scale).cpu().double()
    assert torch.isfinite(out).all() and close_rows(out, want), "plain"
    for chunk, waves in ((32, 0), (128, 0), (128, 2), (128, 8)):
        out = run_rows(q, kc, vc, row_req, positions, table, window, scale, chunk=chunk, waves=ops.row_waves_fit(nH, nKV, d, waves),
                       extra_splits=1).cpu().double()
        assert torch.isfinite(out).all() and close_rows(out, want), ("rows", chunk, waves, float((out - want).abs().max()))
    q_len = torch.tensor(info["q_lens"], dtype=torch.int32)
    q_start = torch.cumsum(q_len, 0, dtype=torch.int32) - q_len
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    for qt in (1, 2):
        tiles = [(r, q0) for r, n in enumerate(info["q_lens"]) for q0 in range(0, n, ops.attention_tile_rows(d, qt))]
        for split_chunk in (0, 128):
            splits = {}
            if split_chunk:
                splits = dict(chunk=split_chunk, max_splits=-(-max(info["kv_lens"]) // split_chunk) + 1,
                              rows=torch.arange(T, dtype=torch.int32, device=DEV), row_req=row_req, positions=positions)
            out = torch.zeros(T, nH * d, dtype=BF16, device=DEV)
            ops.attention_tiles(q, kc, vc, out, dev([t[0] for t in tiles]), dev([t[1] for t in tiles]), q_start.to(DEV), q_len.to(DEV),
                                dev(info["kv_lens"]), table, window, scale, qt, **splits)
            out = out.cpu().double()
            assert torch.isfinite(out).all() and close_rows(out, want), ("tiles", qt, split_chunk, float((out - want).abs().max()))


def test_attention_tiles_refuses_splits_it_cannot_merge():
    (q, kc, vc, row_req, positions, table), _, info = paged_case(7, [64], [100], 4, 2, 16, 16, BF16, None)
    dev = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    args = (q, kc, vc, torch.zeros(64, 64, dtype=BF16, device=DEV), dev([0]), dev([0]), dev([0]), dev([64]), dev([164]), table, None, 0.25, 1)
    with pytest.raises(ops.KernelError, match="multiple of 64"):
        ops.attention_tiles(*args, chunk=100, max_splits=2, rows=dev(list(range(64))), row_req=row_req, positions=positions)
    with pytest.raises(ops.KernelError, match="rows to merge"):
        ops.attention_tiles(*args, chunk=128, max_splits=2)
    with pytest.raises(ops.KernelError, match="cannot hold"):
        ops.attention_tiles(*args, order=torch.full((40,), -1, dtype=torch.int32, device=DEV))   # 5 places per XCD for 4 items
    with pytest.raises(ops.KernelError, match="each of 8"):
        ops.attention_tiles(*args, order=torch.full((12,), -1, dtype=torch.int32, device=DEV))


def test_mfma_attention_refuses_what_it_cannot_do():
    q = torch.zeros(1, 2, 24, dtype=BF16, device=DEV)
    kc = torch.zeros(2, 1, 16, 24, dtype=BF16, device=DEV)
    vc = torch.zeros(2, 1, 24, 16, dtype=BF16, device=DEV)
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(ops.KernelError, match="head_dim"):
        ops.attention_rows(q, kc, vc, torch.zeros(1, 48, dtype=BF16, device=DEV), None, 1, z, z, z.view(1, 1), None, 1.0, 128, 1)
    q = torch.zeros(1, 2, 32, dtype=BF16, device=DEV)
    kc, vc = torch.zeros(2, 1, 16, 32, dtype=BF16, device=DEV), torch.zeros(2, 1, 32, 16, dtype=BF16, device=DEV)
    with pytest.raises(ops.KernelError, match="waves per workgroup"):
        ops.attention_rows(q, kc, vc, torch.zeros(1, 64, dtype=BF16, device=DEV), None, 1, z, z, z.view(1, 1), None, 1.0, 128, 1, waves=9)
    q = torch.zeros(1, 32, 128, dtype=BF16, device=DEV)           # 16 heads of 128 per pass: eight waves' results exceed the LDS
    kc, vc = torch.zeros(2, 1, 16, 128, dtype=BF16, device=DEV), torch.zeros(2, 1, 128, 16, dtype=BF16, device=DEV)
    assert ops.row_waves_fit(32, 1, 128, 8) == 4
    with pytest.raises(ops.KernelError, match="waves per workgroup"):
        ops.attention_rows(q, kc, vc, torch.zeros(1, 4096, dtype=BF16, device=DEV), None, 1, z, z, z.view(1, 1), None, 1.0, 128, 1, waves=8)


# ---- weight-streaming matrix product ---------------------------------------------------------
@pytest.mark.parametrize("M", [1, 5, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(50, 64), (3, 8), (130, 200), (577, 1000), (4608, 3584)])
@pytest.mark.parametrize("out_dtype", [BF16, F32])
def test_skinny_gemm(M, N, K, out_dtype):
    g = gen(11)
    x = torch.randn(M, K, generator=g).to(BF16)
    w = torch.randn(N, K, generator=g).to(BF16)
    want = x.double() @ w.double().t()
    out = ops.skinny_gemm(x.to(DEV), w.to(DEV), out_dtype).cpu().double()
    t = dict(rtol=1e-2, atol=1e-2 * math.sqrt(K)) if out_dtype == BF16 else dict(rtol=1e-4, atol=1e-4 * math.sqrt(K))
    assert torch.allclose(out, want, **t), float((out - want).abs().max())


@pytest.mark.parametrize("nt,waves,unroll", [(1, 1, 4), (2, 4, 2), (1, 16, 2), (2, 8, 4), (1, 3, 4)])
def test_skinny_gemm_every_launch_shape_gives_the_same_product(nt, waves, unroll):
    g = gen(12)
    x = torch.randn(9, 1096, generator=g).to(BF16)
    w = torch.randn(333, 1096, generator=g).to(BF16)
    want = x.double() @ w.double().t()
    out = ops.skinny_gemm(x.to(DEV), w.to(DEV), F32, nt=nt, waves=waves, unroll=unroll).cpu().double()
    assert torch.allclose(out, want, rtol=1e-4, atol=3e-3)


def test_tile_weights_layout():
    """Piece (tile t, k-tile kt, 16 g + col) of the tiled copy is row 16 t + col at k = 32 kt + 8 g; padding is zero."""
    g = gen(15)
    N, K = 37, 72                                      # 3 row tiles (11 padded rows), 4 k-tiles (56 padded values)
    w = torch.randn(N, K, generator=g).to(BF16)
    t = ops.tile_weights(w.to(DEV)).cpu().float().view(3, 4, 4, 16, 8)      # [t, kt, g, col, 8]
    want = torch.zeros(48, 128)
    want[:N, :K] = w.float()
    want = want.view(3, 16, 4, 4, 8).permute(0, 2, 3, 1, 4)                 # [t, col, kt, g, 8] -> [t, kt, g, col, 8]
    assert torch.equal(t, want)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(50, 64), (3, 8), (130, 200), (577, 1000), (4608, 3584)])
@pytest.mark.parametrize("tile_rows", [16, 14, 8])
def test_skinny_gemm_from_the_tiled_copy_equals_from_rows(M, N, K, tile_rows):
    g = gen(16)
    x = torch.randn(M, K, generator=g).to(BF16).to(DEV)
    w = torch.randn(N, K, generator=g).to(BF16).to(DEV)
    tiled = ops.tile_weights(w, tile_rows=tile_rows)
    want = x.double().cpu() @ w.double().cpu().t()
    skinny = ops.skinny_gemm
    ops_skinny = lambda *a, **kw: skinny(*a, tile_rows=tile_rows, **kw)
    out = ops_skinny(x, w, F32, tiled=tiled).cpu().double()
    assert torch.allclose(out, want, rtol=1e-4, atol=1e-4 * math.sqrt(K)), float((out - want).abs().max())
    mt = (M + 15) // 16
    for nt, waves, unroll in [(1, 1, 4), (2, 4, 2), (1, 16, 2)]:
        if (mt >= 3 and unroll == 4) or (mt == 4 and nt == 2):     # shapes the kernel is not built for
            with pytest.raises(ops.KernelError, match="no kernel"):
                ops_skinny(x, w, F32, nt=nt, waves=waves, unroll=unroll, tiled=tiled)
            continue
        a = ops_skinny(x, w, F32, nt=nt, waves=waves, unroll=unroll, tiled=tiled).cpu().double()
        assert torch.allclose(a, want, rtol=1e-4, atol=1e-4 * math.sqrt(K))
    if N % 2 == 0 and M <= 16:                     # gate/up pairs from the same copy
        pairs = ops_skinny(x, w, F32, swiglu_pairs=True, tiled=tiled).cpu().double()
        assert torch.allclose(pairs, torch.nn.functional.silu(want[:, 0::2]) * want[:, 1::2], rtol=1e-4, atol=1e-3 * math.sqrt(K))


def test_tiled_copies_of_other_tile_heights():
    """A tile of p rows is stored as 4 runs of p 16-byte pieces per 32 k-values; p is chosen below 16 where 16-row
    tiles would leave compute units without a tile; what is not a height, or a height with an order, is refused."""
    g = gen(21)
    N, K = 30, 72                                      # K pads to 128: 4 k-tiles
    w = torch.randn(N, K, generator=g).to(BF16).to(DEV)
    for p in ops.TILE_ROWS:
        t = ops.tile_weights(w, tile_rows=p).cpu()
        n_tiles = -(-N // p)
        assert t.numel() == n_tiles * p * 128
        t = t.view(n_tiles, 4, 4, p, 8)                # [row tile][k-tile][group of 8 k][row][8 k-values]
        full = torch.zeros(n_tiles * p, 128, dtype=BF16)
        full[:N, :K] = w.cpu()
        assert torch.equal(t.permute(0, 3, 1, 2, 4).reshape(n_tiles * p, 128), full)
    assert [ops.choose_tile_rows(n) for n in (3584, 2048, 5120, 37888, 152064, 4096, 3000, 64)] == [14, 8, 16, 16, 16, 16, 12, 8]
    with pytest.raises(ops.KernelError, match="rows to a tile"):
        ops.tile_weights(w, tile_rows=7)
    with pytest.raises(ops.KernelError, match="rows to a tile"):
        ops.tile_weights(w, torch.arange(3, dtype=torch.int32, device=DEV), tile_rows=10)
    x = torch.randn(4, K, generator=g).to(BF16).to(DEV)
    with pytest.raises(ops.KernelError, match="tiled"):
        ops.skinny_gemm(x, w, F32, tiled=ops.tile_weights(w, tile_rows=10), tile_rows=12)    # not that copy's size
    lw = ops.prepare_linear(w)
    assert lw.tile_rows == 8 and ops.prepare_linear(w, tile_rows=12).tile_rows == 12
    assert ops.prepare_linear(w, torch.tensor([1, 0], dtype=torch.int32, device=DEV)).tile_rows == 16


def test_tiled_copy_in_another_row_tile_order():
    """A permuted copy gives the same product (the kernel writes tile t to the rows order[t] names) and lays
    its tiles out as the order says."""
    g = gen(20)
    N, K = 150, 136                                    # 10 row tiles, the last with 6 rows
    w = torch.randn(N, K, generator=g).to(BF16).to(DEV)
    order = torch.tensor([3, 9, 0, 7, 1, 8, 2, 6, 5, 4], dtype=torch.int32, device=DEV)
    tiled = ops.tile_weights(w, order)
    plain = ops.tile_weights(w).view(10, -1)
    assert torch.equal(tiled.view(10, -1), plain[order.long()])
    for M in (1, 9, 16, 40):
        x = torch.randn(M, K, generator=g).to(BF16).to(DEV)
        want = x.double().cpu() @ w.double().cpu().t()
        got = ops.skinny_gemm(x, w, F32, tiled=tiled, order=order).cpu().double()
        assert torch.allclose(got, want, rtol=1e-4, atol=2e-3)
        assert torch.allclose(ops.linear(x, ops.LinearWeight(w, tiled, order), out_dtype=F32).cpu().double(), want, rtol=1e-4, atol=2e-3)
    with pytest.raises(ops.KernelError, match="permutation"):
        ops.tile_weights(w, torch.zeros(10, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("d,nH,nKV,K", [(32, 3, 1, 72), (128, 7, 1, 264), (64, 4, 2, 128)])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("P_", [16, 64, 128])
def test_qkv_projection_with_rotation_and_cache_write_as_its_epilogue(M, d, nH, nKV, K, bias, P_):
    """The fused kernel against the product followed by the rotary + append kernel (itself checked against the
    plain formulas above): same q, same cache, nothing else touched; and queries only."""
    g = gen(21)
    pages, theta = 5, 1e4
    heads = nH + 2 * nKV
    w = (torch.randn(heads * d, K, generator=g) / math.sqrt(K)).to(BF16).to(DEV)
    b = (0.5 * torch.randn(heads * d, generator=g)).to(BF16).to(DEV) if bias else None
    x = torch.randn(M, K, generator=g).to(BF16).to(DEV)
    positions = torch.randint(0, 3000, (M,), generator=g).to(torch.int32).to(DEV)
    slots = torch.randperm(pages * P_, generator=g)[:M].to(torch.int32)
    if M > 2:
        slots[1] = -1
    slots = slots.to(DEV)
    inv_freq = (1.0 / torch.pow(torch.tensor(theta, dtype=torch.float64), 2.0 * torch.arange(d // 2, dtype=torch.float64) / d)).float()
    cs, sn = ops.rope_table(positions, inv_freq.to(DEV))
    lw = ops.prepare_linear(w, torch.tensor(ops.pair_tile_order(heads, d), dtype=torch.int32, device=DEV))

    def caches():
        return (torch.zeros(pages, nKV, P_, d, dtype=BF16, device=DEV), torch.zeros(pages, nKV, d, P_, dtype=BF16, device=DEV))
    kc, vc = caches()
    q = ops.qkv_rope_append(x, lw, b, slots, cs, sn, nH, nKV, d, kc, vc, P_)
    # the unfused path rounds the product to bf16 before the bias: compare with that path in float, at bf16's rounding
    qkv32 = ops.skinny_gemm(x, w, F32)
    kc2f, vc2f = (c.float() for c in caches())
    q2 = ops.rope_append(qkv32, b.float() if bias else None, slots, cs, sn, ops.ROPE_SPLIT_HALF, d, nH, nKV, d, kc2f, vc2f, P_)
    t = dict(rtol=1e-2, atol=1e-2)
    assert torch.allclose(q.float().view(M, -1), q2.view(M, -1), **t)
    assert torch.allclose(kc.float(), kc2f, **t) and torch.allclose(vc.float(), vc2f, **t)
    assert torch.equal(kc == 0, kc2f == 0) and torch.equal(vc == 0, vc2f == 0)      # the same elements written
    for waves, unroll in [(1, 2), (4, 4), (16, 2)]:
        ka, va = caches()
        qa = ops.qkv_rope_append(x, lw, b, slots, cs, sn, nH, nKV, d, ka, va, P_, waves=waves, unroll=unroll)
        assert torch.allclose(qa.float(), q.float(), rtol=1e-2, atol=1e-2) and torch.allclose(ka.float(), kc.float(), rtol=1e-2, atol=1e-2)
    # queries only: the first nH heads of the weight, no cache
    lq = ops.prepare_linear(w[: nH * d], torch.tensor(ops.pair_tile_order(nH, d), dtype=torch.int32, device=DEV))
    qq = ops.qkv_rope_append(x, lq, b[: nH * d] if bias else None, None, cs, sn, nH, 0, d, None, None, P_)
    assert torch.allclose(qq.float(), q.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("seed", range(24))
def test_fused_qkv_random_shapes(seed):
    """The q/k/v product with bias, rotation and cache write as its epilogue, at shapes drawn at random (1-16 rows,
    head sizes of 32-256 in steps of 32, 1-40 query heads, K a multiple of 8 up to 4,000, pages of 16-128); against
    the plain formulas in float64."""
    import random
    rng = random.Random(2100 + seed)
    M = rng.randint(1, 16)
    d = 32 * rng.choice([1, 2, 2, 3, 4, 4, 8])
    nKV = rng.choice([1, 2, 4, 8])
    nH = nKV * rng.choice([1, 2, 5, 7])
    K = 8 * rng.choice([rng.randint(1, 30), rng.randint(31, 500)])
    P_ = rng.choice([16, 32, 64, 128])
    bias = rng.random() < 0.6
    pages, theta = 3, rng.choice([1e4, 1e6])
    g = gen(2200 + seed)
    heads = nH + 2 * nKV
    w = (torch.randn(heads * d, K, generator=g) / math.sqrt(K)).to(BF16)
    b = (0.5 * torch.randn(heads * d, generator=g)).to(BF16) if bias else None
    x = torch.randn(M, K, generator=g).to(BF16)
    positions = torch.randint(0, 3000, (M,), generator=g).to(torch.int32)
    slots = torch.randperm(pages * P_, generator=g)[:M].to(torch.int32)
    if M > 2:
        slots[rng.randrange(M)] = -1
    inv_freq = (1.0 / torch.pow(torch.tensor(theta, dtype=torch.float64), 2.0 * torch.arange(d // 2, dtype=torch.float64) / d)).float()
    cs, sn = ops.rope_table(positions.to(DEV), inv_freq.to(DEV))
    lw = ops.prepare_linear(w.to(DEV), torch.tensor(ops.pair_tile_order(heads, d), dtype=torch.int32, device=DEV))
    kc, vc = torch.zeros(pages, nKV, P_, d, dtype=BF16, device=DEV), torch.zeros(pages, nKV, d, P_, dtype=BF16, device=DEV)
    q = ops.qkv_rope_append(x.to(DEV), lw, b.to(DEV) if bias else None, slots.to(DEV), cs, sn, nH, nKV, d, kc, vc, P_)
    qkv = x.double() @ w.double().t() + (b.double() if bias else 0)
    xq, xk, xv = qkv[:, : nH * d].view(M, nH, d), qkv[:, nH * d: (nH + nKV) * d].view(M, nKV, d), qkv[:, (nH + nKV) * d:].view(M, nKV, d)
    case = (seed, M, d, nH, nKV, K, P_, bias)
    t = dict(rtol=1e-2, atol=1e-2)
    assert torch.allclose(q.cpu().double(), pm.rope_split_half(xq, positions.tolist(), theta), **t), case
    live = slots >= 0
    k_got, v_got = cache_rows(kc.cpu(), vc.cpu(), slots[live], P_)
    assert torch.allclose(k_got.double(), pm.rope_split_half(xk, positions.tolist(), theta)[live], **t), case
    assert torch.allclose(v_got.double(), xv[live], **t), case
    written = torch.zeros(pages * P_, dtype=torch.bool); written[slots[live].long()] = True
    assert torch.all(kc.cpu().permute(0, 2, 1, 3).reshape(pages * P_, -1)[~written] == 0), case   # nothing else touched
    assert torch.all(vc.cpu().permute(0, 3, 1, 2).reshape(pages * P_, -1)[~written] == 0), case


@pytest.mark.parametrize("M", [9, 17, 32, 33, 50, 64, 65, 81, 100, 128])
@pytest.mark.parametrize("N,K", [(50, 64), (130, 200), (577, 1000), (4608, 3584), (200, 2104), (4100, 136),
                                 (9000, 264)])                     # tall enough for workgroups of fewer than 8 waves at 33-64 rows
@pytest.mark.parametrize("out_dtype", [BF16, F32])
@pytest.mark.parametrize("tile_rows", [16, 14, 10])
def test_wide_gemm(M, N, K, out_dtype, tile_rows):
    g = gen(40)
    x = torch.randn(M, K, generator=g).to(BF16)
    w = (torch.randn(N, K, generator=g) * 0.3).to(BF16)
    want = x.double() @ w.double().t()
    lw = ops.prepare_linear(w.to(DEV), tile_rows=tile_rows)
    assert lw.tile_rows == tile_rows
    t = dict(rtol=1e-4, atol=3e-3) if out_dtype == F32 else dict(rtol=1e-2, atol=0.1)
    got = ops.wide_gemm(x.to(DEV), lw, out_dtype).cpu().double()
    assert got.shape == (M, N) and torch.allclose(got, want, **t), float((got - want).abs().max())
    if M > 16:
        assert torch.equal(ops.linear(x.to(DEV), lw, out_dtype).cpu().double(), got)   # what linear picks at these rows


@pytest.mark.parametrize("waves,slices,M", [(8, 1, 41), (8, 3, 41), (11, 2, 41), (16, 1, 41), (16, 8, 41), (8, 1, 113), (8, 4, 113), (8, 9, 70),
                                            (4, 1, 41), (5, 2, 17), (6, 1, 64), (7, 3, 33), (4, 9, 50), (5, 1, 100)])
def test_wide_gemm_every_launch_shape_gives_the_same_product(waves, slices, M):
    g = gen(41)
    N, K = 333, 1096                           # 9 rounds of 128 k-values, the last one short; 21 row tiles, the last one short
    x = torch.randn(M, K, generator=g).to(BF16)
    w = torch.randn(N, K, generator=g).to(BF16)
    lw = ops.prepare_linear(w.to(DEV))
    got = ops.wide_gemm(x.to(DEV), lw, F32, waves=waves, slices=slices).cpu().double()
    assert torch.allclose(got, x.double() @ w.double().t(), rtol=1e-4, atol=3e-3)
    lw.rows = torch.zeros_like(lw.rows)                                               # it reads the copy, not the rows
    assert torch.equal(ops.wide_gemm(x.to(DEV), lw, F32, waves=waves, slices=slices).cpu().double(), got)


def test_wide_gemm_gate_up_pairs_and_tile_order():
    g = gen(42)
    M, I2, K = 37, 2 * 301, 264
    x = torch.randn(M, K, generator=g).to(BF16)
    w = (torch.randn(I2, K, generator=g) * 0.2).to(BF16)
    ref = x.double() @ w.double().t()
    gt, up = ref[:, 0::2], ref[:, 1::2]
    got = ops.linear_swiglu(x.to(DEV), ops.prepare_linear(w.to(DEV))).cpu().double()
    assert got.shape == (M, I2 // 2) and torch.allclose(got, gt / (1 + torch.exp(-gt)) * up, rtol=2e-2, atol=2e-2)
    heads, d = 5, 32                                                                   # 160 rows in pair order, as q/k/v has them
    wq = (torch.randn(heads * d, K, generator=g) * 0.2).to(BF16)
    order = torch.tensor(ops.pair_tile_order(heads, d), dtype=torch.int32, device=DEV)
    lq = ops.prepare_linear(wq.to(DEV), order)
    out = ops.linear(x.to(DEV), lq, F32).cpu().double()
    assert torch.allclose(out, x.double() @ wq.double().t(), rtol=1e-4, atol=3e-3)
    with pytest.raises(ops.KernelError, match="wide_gemm"):
        ops.wide_gemm(x.to(DEV), lq, BF16, swiglu_pairs=True)                          # pairs in a permuted copy
    with pytest.raises(ops.KernelError, match="wide_gemm"):
        ops.wide_gemm(torch.zeros(129, K, dtype=BF16, device=DEV), lq)
    x65 = torch.randn(65, K, generator=g).to(BF16).to(DEV)
    assert torch.equal(ops.wide_gemm(x65, lq, F32, waves=16), ops.wide_gemm(x65, lq, F32))   # beyond 64 rows: taken as 8 waves
    assert torch.equal(ops.wide_gemm(x.to(DEV), lq, F32, waves=3).cpu().double(), out)    # fewer than 4 waves: taken as 4


def test_partial_sums_of_a_product_are_added_by_the_kernel_that_reads_them():
    """A product cut into slices of K may leave its partial sums to the norm or the rotary kernel that follows."""
    g = gen(43)
    M, H, K, eps = 23, 200, 1096, 1e-5
    x = torch.randn(M, K, generator=g).to(BF16)
    w = (torch.randn(H, K, generator=g) * 0.1).to(BF16)
    lw = ops.prepare_linear(w.to(DEV))
    sums = ops.wide_gemm(x.to(DEV), lw, BF16, slices=4, keep_slices=True)
    assert isinstance(sums, ops.SliceSums) and sums.parts.shape == (3, M, H) and sums.shape == (M, H)   # 9 rounds: 3 slices of 3
    prod = x.double() @ w.double().t()
    assert torch.allclose(sums.sum(F32).cpu().double(), prod, rtol=1e-4, atol=3e-3)
    assert torch.equal(sums.sum(), ops.wide_gemm(x.to(DEV), lw, BF16, slices=4))
    one = ops.wide_gemm(x.to(DEV), lw, BF16, slices=1, keep_slices=True)
    assert torch.is_tensor(one)                                                       # a single slice is a plain result
    # as the delta of a norm
    res = torch.randn(M, H, generator=g)
    nw = (1 + 0.3 * torch.randn(H, generator=g)).to(BF16)
    r = res.to(DEV)
    out = ops.add_rmsnorm(r, sums, nw.to(DEV), eps, BF16)
    want_res = res.double() + prod
    assert torch.allclose(r.cpu().double(), want_res, rtol=1e-5, atol=2e-3)
    assert torch.allclose(out.cpu().double(), pm.rms_norm(want_res, nw.double(), eps), **tol(BF16))
    rows = torch.tensor([22, 0, 7], dtype=torch.int32)
    r2 = res.to(DEV)
    out2 = ops.add_rmsnorm(r2, sums, nw.to(DEV), eps, BF16, rows.to(DEV))               # gathered rows: stream untouched
    assert torch.equal(r2.cpu(), res)
    assert torch.allclose(out2.cpu().double(), pm.rms_norm(want_res, nw.double(), eps)[rows.long()], **tol(BF16))
    # as the q/k/v of the rotary kernel
    nH, nKV, d, P = 3, 1, 40, 16                                                      # 5 heads of 40 = 200 columns
    bias = torch.randn(H, generator=g).to(BF16)
    cos, sin = ops.rope_table(torch.arange(M, dtype=torch.int32, device=DEV) + 5, (1.0 / 10000 ** (torch.arange(d // 2) * 2.0 / d)).to(DEV))
    slots = torch.arange(M, dtype=torch.int32, device=DEV) + 3

    def run(qkv):
        kc, vc = torch.zeros(2, nKV, P, d, dtype=BF16, device=DEV), torch.zeros(2, nKV, d, P, dtype=BF16, device=DEV)
        q = ops.rope_append(qkv, bias.to(DEV), slots, cos, sin, ops.ROPE_SPLIT_HALF, d, nH, nKV, d, kc, vc, P)
        return q.float().cpu(), kc.float().cpu(), vc.float().cpu()

    got, ref = run(sums), run(sums.sum(F32).to(BF16))                                   # the second rounds the sums first
    for a, b in zip(got, ref):
        assert torch.allclose(a, b, rtol=2e-2, atol=3e-2)
    qkv = prod + bias.double()
    c, sn = cos.cpu().double(), sin.cpu().double()
    qq = qkv[:, : nH * d].reshape(M, nH, d)
    lo, hi = qq[..., : d // 2], qq[..., d // 2:]
    want_q = torch.cat([lo * c[:, None] - hi * sn[:, None], lo * sn[:, None] + hi * c[:, None]], -1)
    assert torch.allclose(got[0].double(), want_q, **tol(BF16))


def test_linear_weight_uses_the_copy_for_few_rows_and_the_rows_beyond():
    g = gen(17)
    w = torch.randn(200, 136, generator=g).to(BF16).to(DEV)
    lw = ops.prepare_linear(w)
    assert lw.tiled is not None and lw.rows is w
    lw.rows = torch.zeros_like(w)                      # few rows must not read this; many rows must
    x = torch.randn(5, 136, generator=g).to(BF16).to(DEV)
    want = x.double().cpu() @ w.double().cpu().t()
    assert torch.allclose(ops.linear(x, lw, out_dtype=F32).cpu().double(), want, rtol=1e-4, atol=2e-3)
    big = torch.randn(200, 136, generator=g).to(BF16).to(DEV)
    assert torch.all(ops.linear(big, lw) == 0)
    mid = torch.randn(100, 136, generator=g).to(BF16).to(DEV)          # 65-128 rows of a weight with few rows: the copy again
    assert torch.allclose(ops.linear(mid, lw, out_dtype=F32).cpu().double(), mid.double().cpu() @ w.double().cpu().t(), rtol=1e-4, atol=2e-3)
    pairs = ops.prepare_linear(w)
    got = ops.linear_swiglu(x, pairs).cpu().double()
    gt, up = want[:, 0::2], want[:, 1::2]
    assert torch.allclose(got, gt / (1 + torch.exp(-gt)) * up, rtol=2e-2, atol=2e-2)
    old = ops.decode_weight_copy
    try:
        ops.decode_weight_copy = False
        assert ops.prepare_linear(w).tiled is None
    finally:
        ops.decode_weight_copy = old
    assert ops.prepare_linear(w.float()).tiled is None  # a 32-bit weight has no copy


@pytest.mark.parametrize("M,N,K", [(130, 200, 4096), (512, 136, 16384), (300, 520, 8192 + 4096), (1000, 64, 4096)])
def test_linear_cuts_deep_narrow_products_of_many_rows_into_slices(M, N, K):
    """Many rows times a weight with few rows and a long K: the library runs it as a batch of K slices with float32
    partial sums, which the caller's norm kernel adds; the sum is the product, and without ``keep_slices`` nothing is cut."""
    g = gen(51)
    x = torch.randn(M, K, generator=g).to(BF16)
    w = (torch.randn(N, K, generator=g) * 0.05).to(BF16)
    want = x.double() @ w.double().t()
    S = ops.library_k_slices(M, N, K)
    assert S > 1
    got = ops.linear(x.to(DEV), w.to(DEV), keep_slices=True)
    assert isinstance(got, ops.SliceSums) and got.parts.shape == (S, M, N) and got.parts.dtype == F32
    assert torch.allclose(got.parts.cpu().double().sum(0), want, rtol=1e-4, atol=2e-3 * (K / 4096) ** 0.5)
    assert torch.allclose(got.sum().cpu().double(), want, rtol=1e-2, atol=0.1)
    plain = ops.linear(x.to(DEV), w.to(DEV))
    assert isinstance(plain, torch.Tensor) and torch.allclose(plain.cpu().double(), want, rtol=1e-2, atol=0.1)
    res = torch.randn(M, N, generator=g)
    nw = (1 + 0.3 * torch.randn(N, generator=g)).to(BF16)
    r = res.to(DEV)
    out = ops.add_rmsnorm(r, got, nw.to(DEV), 1e-5, BF16)                       # the consumer: adds the slices in order
    assert torch.allclose(r.cpu().double(), res.double() + want, rtol=1e-4, atol=2e-3 * (K / 4096) ** 0.5)
    assert torch.allclose(out.cpu().double(), pm.rms_norm(res.double() + want, nw.double(), 1e-5), **tol(BF16))


def test_linear_picks_by_weight_type_and_rows():
    g = gen(13)
    w = torch.randn(96, 72, generator=g)
    for M in (3, 64, 65, 200):
        x = torch.randn(M, 72, generator=g)
        want = x.bfloat16().double() @ w.bfloat16().double().t()
        got = ops.linear(x.bfloat16().to(DEV), w.bfloat16().to(DEV))
        assert got.dtype == BF16 and torch.allclose(got.cpu().double(), want, rtol=1e-2, atol=0.1)
        logits = ops.linear(x.bfloat16().to(DEV), w.bfloat16().to(DEV), out_dtype=F32)
        assert logits.dtype == F32 and torch.allclose(logits.cpu().double(), want, rtol=1e-4, atol=1e-3)   # no bf16 rounding
        mixed = ops.linear(x.bfloat16().to(DEV), w.to(DEV))                  # a float32 weight in bf16 mode
        assert mixed.dtype == BF16 and torch.allclose(mixed.cpu().double(), x.bfloat16().double() @ w.double().t(), rtol=1e-2, atol=0.1)


@pytest.mark.parametrize("seed", range(40))
def test_linear_random_shapes(seed):
    """``linear`` and ``linear_swiglu`` at shapes drawn at random: 1-150 rows (the streaming kernels up to 64 and, for
    the weight's copy, 128; the library beyond), 1-6,000 weight rows, K a multiple of 8 up to 4,800, with and without the streamed copy in whatever
    tile height ``prepare_linear`` picks for the weight, partial sums kept or added, bf16 or float out; against
    float64."""
    import random
    rng = random.Random(500 + seed)
    M = rng.choice([1, rng.randint(2, 16), rng.randint(17, 64), rng.randint(65, 128), rng.randint(129, 150)])
    N = rng.choice([rng.randint(1, 40), rng.randint(41, 700), rng.randint(701, 6000)])
    K = 8 * rng.choice([rng.randint(1, 16), rng.randint(17, 150), rng.randint(151, 600)])
    out_dtype = rng.choice([BF16, F32])
    g = gen(600 + seed)
    x = torch.randn(M, K, generator=g).to(BF16)
    w = (torch.randn(N, K, generator=g) * 0.3).to(BF16)
    want = x.double() @ w.double().t()
    t = dict(rtol=1e-4, atol=3e-3 * max(1.0, K / 1000)) if out_dtype == F32 else dict(rtol=1e-2, atol=0.1 * max(1.0, (K / 1000) ** 0.5))
    weight = ops.prepare_linear(w.to(DEV)) if rng.random() < 0.75 else w.to(DEV)
    got = ops.linear(x.to(DEV), weight, out_dtype, keep_slices=rng.random() < 0.5)
    if isinstance(got, ops.SliceSums):
        got = got.sum()
    got = got.cpu().double()
    assert got.shape == (M, N) and torch.allclose(got, want, **t), (M, N, K, out_dtype, float((got - want).abs().max()))
    if N % 2 == 0:
        act = ops.linear_swiglu(x.to(DEV), weight).cpu().double()
        gt, up = want[:, 0::2], want[:, 1::2]
        ref = gt / (1 + torch.exp(-gt)) * up
        assert act.shape == (M, N // 2) and torch.allclose(act, ref, rtol=2e-2, atol=2e-2 * max(1.0, float(ref.abs().max()) / 8)), \
            (M, N, K, float((act - ref).abs().max()))


@pytest.mark.parametrize("M", [1, 8, 16, 40, 100])
def test_linear_swiglu_pairs(M):
    g = gen(14)
    I, K = 1000 if M != 8 else 37, 144
    x = torch.randn(M, K, generator=g).to(BF16)
    wg, wu = torch.randn(I, K, generator=g).to(BF16) * 0.2, torch.randn(I, K, generator=g).to(BF16) * 0.2
    pairs = torch.stack([wg, wu], dim=1).reshape(2 * I, K).contiguous()
    got = ops.linear_swiglu(x.to(DEV), pairs.to(DEV)).cpu().double()
    gt, up = x.double() @ wg.double().t(), x.double() @ wu.double().t()
    assert got.shape == (M, I) and torch.allclose(got, gt / (1 + torch.exp(-gt)) * up, rtol=2e-2, atol=2e-2)
    got32 = ops.linear_swiglu(x.float().to(DEV), pairs.float().to(DEV)).cpu().double()     # the 32-bit path
    assert torch.allclose(got32, gt / (1 + torch.exp(-gt)) * up, rtol=1e-4, atol=1e-4)


def _stream_case(M, N, K, seed, copy):
    """``copy``: False (the weight's rows) or the rows to a tile of the streamed copy."""
    g = gen(seed)
    x = torch.randn(M, K, generator=g).to(BF16)
    w = (torch.randn(N, K, generator=g) * 0.1).to(BF16)
    stream = torch.randn(M, N, generator=g) * 2.0
    nw = (1 + 0.3 * torch.randn(N, generator=g)).to(BF16)
    p = 16 if copy in (False, True) else copy
    lw = ops.LinearWeight(w.to(DEV), ops.tile_weights(w.to(DEV), tile_rows=p) if copy else None, None, p)
    return x, w, stream, nw, lw


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("N,K", [(100, 72), (3584, 512), (36, 1000), (4100, 64)])
@pytest.mark.parametrize("copy", [False, True, 14, 8])
def test_product_added_to_the_stream_with_the_next_norm_prepared(M, N, K, copy):
    x, w, stream, nw, lw = _stream_case(M, N, K, 30, copy)
    p = lw.tile_rows
    s = stream.to(DEV)
    got = ops.linear_into_stream(x.to(DEV), lw, s, nw.to(DEV), 1e-5)
    want = stream.double() + x.double() @ w.double().t()
    assert torch.allclose(s.cpu().double(), want, rtol=1e-5, atol=1e-5)               # float sums, no rounding of the delta
    assert got.rows.dtype == BF16 and got.width == N
    assert torch.allclose(got.rows.cpu().double(), want * nw.double(), **tol(BF16))   # one rounding
    assert got.pieces.shape == (-(-N // p), 16)                                        # one piece per row tile of the weight
    sq = torch.nn.functional.pad(want ** 2, (0, -N % p)).reshape(M, -1, p).sum(-1)     # [M, pieces]
    assert torch.allclose(got.pieces.cpu().double()[:, :M], sq.t(), rtol=1e-5, atol=1e-7)
    assert float(got.pieces[:, M:].abs().max()) == 0.0 if M < 16 else True


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("copy", [False, True, 10])
def test_row_factors_are_applied_by_the_product_that_reads_the_rows(M, copy):
    """The norm's factor per row, applied to sums instead of to the input: the same as norm, then product."""
    H, I, eps = 200, 300, 1e-3
    x, w, stream, nw, lw = _stream_case(M, H, 136, 31, copy)
    s = stream.to(DEV)
    scaled = ops.linear_into_stream(x.to(DEV), lw, s, nw.to(DEV), eps)
    rows = scaled.rows.cpu().double()
    normed = pm.rms_norm(s.cpu().double(), nw.double(), eps)              # what the norm's own kernel would give
    factor = torch.rsqrt((s.cpu().double() ** 2).mean(-1, keepdim=True) + eps)
    assert torch.allclose(rows * factor, normed, **tol(BF16))
    g = gen(32)
    w2 = (torch.randn(I, H, generator=g) * 0.2).to(BF16)
    lw2 = ops.LinearWeight(w2.to(DEV), ops.tile_weights(w2.to(DEV), tile_rows=lw.tile_rows) if copy else None, None, lw.tile_rows)
    assert ops.takes_scaled_rows(M, lw2) and not ops.takes_scaled_rows(17, lw2)
    got = ops.linear(scaled, lw2).cpu().double()
    assert torch.allclose(got, (rows @ w2.double().t()) * factor, **tol(BF16))         # same rounded inputs: one rounding
    assert torch.allclose(got, normed @ w2.double().t(), rtol=2e-2, atol=2e-2)         # and the function it stands for
    got32 = ops.linear(scaled, lw2, torch.float32).cpu().double()
    assert torch.allclose(got32, (rows @ w2.double().t()) * factor, rtol=1e-4, atol=1e-4)
    gt, up = (rows @ w2[0::2].double().t()) * factor, (rows @ w2[1::2].double().t()) * factor
    act = ops.linear_swiglu(scaled, lw2).cpu().double()
    assert torch.allclose(act, gt / (1 + torch.exp(-gt)) * up, **tol(BF16))


@pytest.mark.parametrize("seed", range(25))
def test_stream_add_and_row_factors_random_shapes(seed):
    """A product added into the stream with the next norm prepared, then the products that take the rows with their
    factors, at widths, row counts and tile heights drawn at random; against float64."""
    import random
    rng = random.Random(700 + seed)
    M = rng.randint(1, 16)
    H = 8 * rng.choice([rng.randint(1, 12), rng.randint(13, 120), rng.randint(121, 450)])
    K = 8 * rng.choice([rng.randint(1, 20), rng.randint(21, 300)])
    I = 2 * rng.choice([rng.randint(1, 30), rng.randint(31, 1200)])
    copy = rng.choice([False, True, 14, 10, 8])
    eps = rng.choice([1e-6, 1e-3])
    x, w, stream, nw, lw = _stream_case(M, H, K, 800 + seed, copy)
    s = stream.to(DEV)
    scaled = ops.linear_into_stream(x.to(DEV), lw, s, nw.to(DEV), eps)
    want = stream.double() + x.double() @ w.double().t()
    assert torch.allclose(s.cpu().double(), want, rtol=1e-5, atol=1e-4 * max(1.0, K / 500)), (M, H, K, copy)
    rows = scaled.rows.cpu().double()
    factor = torch.rsqrt((s.cpu().double() ** 2).mean(-1, keepdim=True) + eps)
    assert torch.allclose(rows * factor, pm.rms_norm(s.cpu().double(), nw.double(), eps), **tol(BF16)), (M, H, K, copy)
    g = gen(900 + seed)
    w2 = (torch.randn(I, H, generator=g) * 0.2).to(BF16)
    lw2 = ops.LinearWeight(w2.to(DEV), ops.tile_weights(w2.to(DEV), tile_rows=lw.tile_rows) if copy else None, None, lw.tile_rows)
    ref = (rows @ w2.double().t()) * factor
    big = max(1.0, float(ref.abs().max()))
    got = ops.linear(scaled, lw2, torch.float32).cpu().double()
    assert torch.allclose(got, ref, rtol=1e-4, atol=1e-4 * big), (M, H, K, I, copy, float((got - ref).abs().max()))
    gt, up = ref[:, 0::2], ref[:, 1::2]
    act = ops.linear_swiglu(scaled, lw2).cpu().double()
    want_act = gt / (1 + torch.exp(-gt)) * up
    assert torch.allclose(act, want_act, rtol=8e-3, atol=1e-3 * max(1.0, float(want_act.abs().max()))), (M, H, K, I, copy)


@pytest.mark.parametrize("M", [1, 9, 16])
@pytest.mark.parametrize("copy", [True, 14, 8])
def test_row_factors_in_the_product_that_shares_x_through_lds(M, copy):
    """The product that large tall weights take from 9 rows on applies the norm's factor per row like the other one:
    every number of waves (the waves' shares of the sums of squares meet in LDS), both outputs, SwiGLU, a width whose
    pieces do not fill a wave's loads and one that needs several rounds of them."""
    for H, I, eps in ((200, 300, 1e-3), (4104, 72, 1e-6)):
        x, w, stream, nw, lw = _stream_case(M, H, 136, 35, copy)
        s = stream.to(DEV)
        scaled = ops.linear_into_stream(x.to(DEV), lw, s, nw.to(DEV), eps)
        rows = scaled.rows.cpu().double()
        factor = torch.rsqrt((s.cpu().double() ** 2).mean(-1, keepdim=True) + eps)
        g = gen(36)
        w2 = (torch.randn(I, H, generator=g) * 0.2).to(BF16)
        lw2 = ops.LinearWeight(w2.to(DEV), ops.tile_weights(w2.to(DEV), tile_rows=lw.tile_rows), None, lw.tile_rows)
        ref = (rows @ w2.double().t()) * factor
        big = max(1.0, float(ref.abs().max()))
        gt, up = ref[:, 0::2], ref[:, 1::2]
        want_act = gt / (1 + torch.exp(-gt)) * up
        for waves in (0, 4, 5, 8, 11, 16):
            got32 = ops.wide_gemm(scaled, lw2, torch.float32, waves=waves, slices=1 if waves else 0).cpu().double()
            assert torch.allclose(got32, ref, rtol=1e-4, atol=1e-4 * big), (H, waves, float((got32 - ref).abs().max()))
            got = ops.wide_gemm(scaled, lw2, BF16, waves=waves, slices=1 if waves else 0).cpu().double()
            assert torch.allclose(got, ref, rtol=8e-3, atol=8e-3 * big), (H, waves)
            act = ops.wide_gemm(scaled, lw2, BF16, waves=waves, slices=1 if waves else 0, swiglu_pairs=True).cpu().double()
            assert torch.allclose(act, want_act, rtol=8e-3, atol=1e-3 * max(1.0, float(want_act.abs().max()))), (H, waves)
        sliced = ops.wide_gemm(scaled, lw2, torch.float32, waves=8, slices=2).cpu().double()      # the factor on partial sums
        assert torch.allclose(sliced, ref, rtol=1e-4, atol=1e-4 * big)
        other = ops.skinny_gemm(scaled, lw2.rows, torch.float32, tiled=lw2.tiled, tile_rows=lw2.tile_rows).cpu().double()
        assert torch.allclose(other, got32, rtol=1e-4, atol=1e-4 * big)                              # the two kernels agree
    with pytest.raises(ops.KernelError, match="at most 16"):
        ops.wide_gemm(ops.ScaledRows(torch.zeros(17, H, dtype=BF16, device=DEV), scaled.pieces, H, 1e-3), lw2)


def test_few_rows_of_large_tall_weights_take_the_product_that_shares_x(monkeypatch):
    """The choice between the two products for up to 16 rows, and that ``linear`` / ``linear_swiglu`` follow it with
    scaled rows (forced here for a small weight by lowering the size from which it applies)."""
    assert ops._small_m_kernel(9, 37888, 3584, True) == "wide" and ops._small_m_kernel(8, 37888, 3584, True) == "skinny"
    assert ops._small_m_kernel(16, 37888, 3584, False) == "skinny"                     # no tiled copy
    assert ops._small_m_kernel(16, 22016, 2048, True) == "skinny"                      # a smaller weight
    assert ops._small_m_kernel(11, 152064, 3584, True) == "skinny" and ops._small_m_kernel(12, 152064, 3584, True) == "wide"
    assert ops._small_m_kernel(16, 3584, 18944, True) == "skinny"                      # few rows of W: K would need slices
    assert not ops._tile_pairs_fit(27648) and ops._tile_pairs_fit(37888)              # 1,728 tiles: 7 to a unit one by one, 8 in pairs
    assert ops._small_m_kernel(6, 27648, 5120, True) == "wide" and ops._small_m_kernel(5, 27648, 5120, True) == "skinny"
    # large weights of few rows whose 16-row tiles lie unevenly on the 256 units (5,120 rows: 320 tiles) are cut into slices of K
    assert ops._small_m_kernel(8, 5120, 27648, True) == "wide" and ops._small_m_kernel(7, 5120, 27648, True) == "skinny"
    assert ops._small_m_kernel(9, 5120, 13824, True) == "wide" and ops._small_m_kernel(8, 5120, 13824, True) == "skinny"
    assert ops._small_m_kernel(16, 5120, 5120, True) == "skinny" and ops._small_m_kernel(16, 8192, 29568, True) == "skinny"
    lw = ops.LinearWeight(torch.empty(5120, 27648, dtype=BF16, device="meta"), torch.empty(1, device="meta"), None, 16)
    nw = torch.empty(5120, dtype=BF16, device="meta")
    assert ops.adds_into_stream(7, lw, nw) and not ops.adds_into_stream(8, lw, nw)
    M, H, eps = 12, 136, 1e-5
    x, w, stream, nw, lw = _stream_case(M, H, 72, 37, True)
    s = stream.to(DEV)
    scaled = ops.linear_into_stream(x.to(DEV), lw, s, nw.to(DEV), eps)
    w2 = (torch.randn(16400, H, generator=gen(38)) * 0.2).to(BF16)
    lw2 = ops.prepare_linear(w2.to(DEV))
    before = ops.linear(scaled, lw2, torch.float32)
    calls = []
    real = ops.wide_gemm
    monkeypatch.setattr(ops, "wide_gemm", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    monkeypatch.setattr(ops, "WIDE_FEW_ROWS_MIN_WEIGHT", 1)
    assert ops.takes_scaled_rows(M, lw2)
    after = ops.linear(scaled, lw2, torch.float32)
    act = ops.linear_swiglu(scaled, lw2)
    assert len(calls) == 2
    big = float(before.abs().max())
    assert torch.allclose(after, before, rtol=1e-5, atol=1e-5 * big)
    gt, up = before.double()[:, 0::2], before.double()[:, 1::2]
    assert torch.allclose(act.double(), gt / (1 + torch.exp(-gt)) * up, rtol=8e-3, atol=1e-3 * big)


def test_row_factors_in_the_fused_qkv_product():
    M, d, nH, nKV, K, P, eps = 6, 32, 3, 1, 96, 16, 1e-6
    g = gen(33)
    x, w, stream, nw, lw = _stream_case(M, K, 40, 33, True)
    s = stream.to(DEV)
    scaled = ops.linear_into_stream(x.to(DEV), lw, s, nw.to(DEV), eps)
    heads = nH + 2 * nKV
    wq = (torch.randn(heads * d, K, generator=g) * 0.2).to(BF16)
    bias = torch.randn(heads * d, generator=g).to(BF16)
    order = torch.tensor(ops.pair_tile_order(heads, d), dtype=torch.int32, device=DEV)
    lq = ops.prepare_linear(wq.to(DEV), order)
    cos, sin = ops.rope_table(torch.arange(M, dtype=torch.int32, device=DEV) + 3, (1.0 / 10000 ** (torch.arange(d // 2) * 2.0 / d)).to(DEV))
    slots = torch.arange(M, dtype=torch.int32, device=DEV)

    def run(h):
        kc, vc = torch.zeros(1, nKV, P, d, dtype=BF16, device=DEV), torch.zeros(1, nKV, d, P, dtype=BF16, device=DEV)
        return ops.qkv_rope_append(h, lq, bias.to(DEV), slots, cos, sin, nH, nKV, d, kc, vc, P), kc, vc

    q1, k1, v1 = run(scaled)
    # the same with the factor applied to the rows beforehand, in float, by a weight that cannot round: compare with the
    # plain product on the normalised rows
    factor = torch.rsqrt((s.cpu().double() ** 2).mean(-1, keepdim=True) + eps)
    qkv = (scaled.rows.cpu().double() @ wq.double().t()) * factor + bias.double()
    want_v = qkv[:, (nH + nKV) * d:].reshape(M, nKV, d)
    assert torch.allclose(v1[0, :, :, :M].permute(2, 0, 1).cpu().double(), want_v, **tol(BF16))
    c, sn = cos.cpu().double(), sin.cpu().double()
    qq = qkv[:, : nH * d].reshape(M, nH, d)
    lo, hi = qq[..., : d // 2], qq[..., d // 2:]
    want_q = torch.cat([lo * c[:, None] - hi * sn[:, None], lo * sn[:, None] + hi * c[:, None]], -1)
    assert torch.allclose(q1.cpu().double(), want_q, **tol(BF16))


def test_scaled_rows_are_refused_where_no_kernel_applies_them():
    x, w, stream, nw, lw = _stream_case(4, 64, 32, 34, True)
    scaled = ops.linear_into_stream(x.to(DEV), lw, stream.to(DEV), nw.to(DEV), 1e-5)
    with pytest.raises(ops.KernelError, match="scaled rows"):
        ops.linear(scaled, torch.randn(8, 64, device=DEV))                          # a float32 weight
    with pytest.raises(ops.KernelError, match="scaled rows"):
        ops.linear(scaled, torch.randn(8, 64, device=DEV).bfloat16())               # a bare tensor
    with pytest.raises(ops.KernelError, match="linear_into_stream"):
        ops.linear_into_stream(torch.zeros(17, 32, dtype=BF16, device=DEV), lw, torch.zeros(17, 64, device=DEV), nw.to(DEV), 1e-5)
    with pytest.raises(ops.KernelError, match="linear_into_stream"):               # a float32 norm weight
        ops.linear_into_stream(x.to(DEV), lw, stream.to(DEV), nw.float().to(DEV), 1e-5)


@pytest.mark.parametrize("M", [1, 7, 16, 33, 64])
@pytest.mark.parametrize("N,K,slices", [(50, 64, 0), (3, 8, 0), (130, 200, 2), (577, 1000, 0), (4608, 3584, 0), (200, 2104, 5)])
@pytest.mark.parametrize("out_dtype", [BF16, F32])
def test_staged_gemm(M, N, K, slices, out_dtype):
    g = gen(15)
    x = torch.randn(M, K, generator=g).to(BF16)
    w = torch.randn(N, K, generator=g).to(BF16)
    want = x.double() @ w.double().t()
    out = ops.staged_gemm(x.to(DEV), w.to(DEV), out_dtype, slices=slices).cpu().double()
    t = dict(rtol=1e-2, atol=1e-2 * math.sqrt(K)) if out_dtype == BF16 else dict(rtol=1e-4, atol=1e-4 * math.sqrt(K))
    assert torch.allclose(out, want, **t), float((out - want).abs().max())


def test_staged_gemm_swiglu_pairs_and_unrolls():
    g = gen(16)
    I, K = 300, 520
    x = torch.randn(40, K, generator=g).to(BF16)
    wg, wu = torch.randn(I, K, generator=g).to(BF16) * 0.1, torch.randn(I, K, generator=g).to(BF16) * 0.1
    pairs = torch.stack([wg, wu], dim=1).reshape(2 * I, K).contiguous()
    gt, up = x.double() @ wg.double().t(), x.double() @ wu.double().t()
    want = gt / (1 + torch.exp(-gt)) * up
    for unroll in (2, 4, 6):
        got = ops.staged_gemm(x.to(DEV), pairs.to(DEV), BF16, unroll=unroll, swiglu_pairs=True).cpu().double()
        assert got.shape == (40, I) and torch.allclose(got, want, rtol=2e-2, atol=2e-2)


def test_logprobs_against_log_softmax_and_topk():
    g = gen(17)
    R, V = 5, 3000
    logits = 2.0 * torch.randn(R, V, generator=g)
    logits[1, 100] = logits[1, 7] = logits[1].max() + 1.0          # a tie at the top: index 7 first
    chosen = torch.tensor([0, 100, 5, 2999, 17], dtype=torch.int32)
    lp, ids, tlp = (t.cpu() for t in ops.logprobs(logits.to(DEV), chosen.to(DEV), 6))
    want = torch.log_softmax(logits.double(), -1)
    assert torch.allclose(lp.double(), want[torch.arange(R), chosen.long()], atol=1e-4)
    for r in range(R):
        order = sorted(range(V), key=lambda i: (-float(logits[r, i]), i))[:6]
        assert ids[r].tolist() == order
        assert torch.allclose(tlp[r].double(), want[r, order], atol=1e-4)
    assert ids[1, :2].tolist() == [7, 100]
    assert ops.logprobs(logits.to(DEV), chosen.to(DEV), 0)[1].shape == (R, 0)


LOGPROB_ROWS = [
    ("wide", 152064, lambda g, V: 3.0 * torch.randn(V, generator=g)),
    ("one token far above", 152063, lambda g, V: torch.randn(V, generator=g).index_fill_(0, torch.tensor([40000]), 60.0)),
    ("flat: more near-equal logits than candidates fit", 30001, lambda g, V: 1e-3 * torch.randn(V, generator=g)),
    ("all equal", 9000, lambda g, V: torch.zeros(V)),
    ("fewer finite logits than ranks", 5000, lambda g, V: torch.full((V,), -float("inf")).index_put_((torch.tensor([3, 4000, 77]),), torch.tensor([1.0, 2.0, 1.0]))),
    ("fewer tokens than ranks", 5, lambda g, V: torch.randn(V, generator=g)),
    ("the ranks far apart", 70000, lambda g, V: (-200.0 + torch.randn(V, generator=g)).index_put_((torch.arange(8) * 9000,), 100.0 - 35.0 * torch.arange(8.0))),
]


@pytest.mark.parametrize("case", range(len(LOGPROB_ROWS)), ids=[c[0] for c in LOGPROB_ROWS])
def test_logprobs_rows_of_every_shape(case):
    """The most probable tokens where they are picked from few candidates and where the whole row is searched per rank:
    order by value, then index; ranks beyond the vocabulary come back as -1 and -inf."""
    name, V, build = LOGPROB_ROWS[case]
    g = gen(1600 + case)
    R, N = 3, 8
    logits = torch.stack([build(g, V) for _ in range(R)])
    chosen = torch.tensor([int(logits[r].argmax()) for r in range(R)], dtype=torch.int32)
    lp, ids, tlp = (t.cpu() for t in ops.logprobs(logits.to(DEV), chosen.to(DEV), N))
    want = torch.log_softmax(logits.double(), -1)
    assert torch.allclose(lp.double(), want[torch.arange(R), chosen.long()], atol=1e-4), name
    for r in range(R):
        order = sorted(range(V), key=lambda i: (-float(logits[r, i]), i))[:N]
        assert ids[r, :len(order)].tolist() == order, (name, r)              # (masked tokens rank last, by index)
        assert torch.allclose(tlp[r, :len(order)].double(), want[r, order], atol=1e-4, rtol=1e-5), (name, r)
        assert ids[r, len(order):].tolist() == [-1] * (N - len(order)) and bool((tlp[r, len(order):] == -float("inf")).all())


def test_sample_draws_its_own_numbers_as_the_host_does():
    """Given seeds and counters instead of numbers in [0, 1), the kernel makes the number params.philox_uniform makes:
    the same tokens either way, with seeds and counters beyond 32 bits among them."""
    from inferflux_amd.sampling.params import philox_uniform
    R, V = 64, 5000
    g = gen(31)
    logits = 0.5 * torch.randn(R, V, generator=g)
    seeds = np.array([0, 1, 2**32 - 1, 2**32, 2**63 + 5, 2**64 - 1] + [int(x) for x in torch.randint(0, 2**62, (R - 6,), generator=g)], dtype=np.uint64)
    steps = np.array([0, 2**32, 7, 2**40 + 3, 1, 2**64 - 1] + list(range(R - 6)), dtype=np.uint64)
    draws = torch.from_numpy(np.stack([seeds, steps], 1).view(np.uint32).view(np.int32).reshape(R, 4)).to(DEV)
    u = torch.from_numpy(philox_uniform(seeds, steps)).to(DEV)
    full = lambda v, dt: torch.full((R,), v, dtype=dt, device=DEV)
    a = (logits.to(DEV), full(1.0, torch.float32), full(0, torch.int32), full(1.0, torch.float32), full(0.0, torch.float32))
    by_kernel = ops.sample(*a, draws=draws).cpu().tolist()
    assert by_kernel == ops.sample(*a, uniform=u).cpu().tolist()
    assert len(set(by_kernel)) > R // 2                                  # and they are not all one token
    with pytest.raises(ops.KernelError, match="either"):
        ops.sample(*a)
    with pytest.raises(ops.KernelError, match="either"):
        ops.sample(*a, uniform=u, draws=draws)


def test_measurement_kernels_copy_what_they_read():
    g = gen(23)
    src = torch.randn(5 * 2048 * 3, generator=g).to(DEV)           # 15 rounds of 8 KB: no multiple of the grid
    for streaming in (False, True):
        for waves in (1, 4, 64):
            dst = torch.zeros_like(src)
            ops.stream_copy(src, dst, waves, streaming)
            assert torch.equal(dst, src)
            ops.stream_read(src, waves, streaming)
    with pytest.raises(ops.KernelError, match="multiple of"):
        ops.stream_read(src[:1000], 4, False)
    with pytest.raises(ops.KernelError, match="overlap"):
        ops.stream_copy(src[:4096], src[2048:6144], 4, False)
