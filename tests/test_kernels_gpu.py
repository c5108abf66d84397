"""Each kernel alone against its plain reference, at other sizes than the engine's."""

import math

import numpy as np
import pytest
import torch

import plain_llama as P
from halite_amd.kernels import attention as attn_kernels
from halite_amd.kernels import ops

pytestmark = pytest.mark.gpu
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def close(got, want, tol, what=""):
    got, want = got.float().cpu(), want.float().cpu()
    err = float((got - want).abs().max()) / max(1.0, float(want.abs().max()))
    assert err == err and err <= tol, f"{what}: error {err:.3e} > {tol:.1e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("vocab,d", [(331, 120), (1000, 4096), (17, 8)])
def test_embedding(gpu, dtype, vocab, d):
    table = rnd(vocab, d, seed=1).to(DT[dtype])
    ids = torch.randint(0, vocab, (37,), generator=torch.Generator().manual_seed(2), dtype=torch.int32)
    out = ops.embedding(ids.to(gpu), table.to(gpu))
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), P.embed(ids.long(), table.float()))
    bad = ops.embedding(torch.tensor([vocab], dtype=torch.int32, device=gpu), table.to(gpu))
    assert torch.isnan(bad).all()  # an id outside the table shows, it does not fault


def test_take_tokens(gpu):
    src = torch.randint(0, 50000, (300,), generator=torch.Generator().manual_seed(3), dtype=torch.int32)
    rows = torch.randperm(300, generator=torch.Generator().manual_seed(4))[:270].to(torch.int32)
    tokens = rows.to(gpu)
    ops.take_tokens(src.to(gpu), tokens)
    assert torch.equal(tokens.cpu(), src[rows.long()])
    outside = torch.tensor([300, -1, 5], dtype=torch.int32, device=gpu)
    ops.take_tokens(src.to(gpu), outside)
    assert outside.tolist() == [0, 0, int(src[5])]  # a row outside the source reads nothing


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [120, 1000, 4096])
def test_rmsnorm(gpu, dtype, d):
    dt = DT[dtype]
    h = rnd(9, d, seed=3, scale=2.0)
    delta = rnd(9, d, seed=4).to(dt)
    w = (1 + 0.2 * rnd(d, seed=5)).to(dt)
    eps = 3e-6
    tol = 1e-6 if dtype == "float32" else 1e-2
    # plain: statistics in float32, rounded to the activation type, then the weight
    x = h + delta.float()
    want = P.rms_norm(x.to(dt), w, eps) if dtype == "float32" else (w.float() * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)).to(dt).float())
    hg = h.to(gpu).clone()
    out = ops.rmsnorm(hg, w.to(gpu), eps, dt, delta=delta.to(gpu))
    close(out, want, tol, "norm with add")
    close(hg, x, 1e-7, "stream after add")
    # no delta: the stream stays
    hg = h.to(gpu).clone()
    out = ops.rmsnorm(hg, w.to(gpu), eps, dt)
    close(out, P.rms_norm(h, w.float(), eps), tol, "norm")
    assert torch.equal(hg.cpu(), h)
    # gathered rows: only those, and the stream stays
    rows = torch.tensor([7, 0, 7, 3], dtype=torch.int32)
    hg = h.to(gpu).clone()
    out = ops.rmsnorm(hg, w.to(gpu), eps, dt, delta=delta.to(gpu), rows=rows.to(gpu))
    close(out, want[rows.long()], tol, "gathered norm")
    assert torch.equal(hg.cpu(), h)
    # a 32-bit weight with bfloat16 activations
    if dtype == "bfloat16":
        out = ops.rmsnorm(h.to(gpu).clone(), w.float().to(gpu), eps, dt)
        close(out, P.rms_norm(h, w.float(), eps), tol, "norm, 32-bit weight")
    # many rows (a prompt): smaller blocks, several vectors per thread
    many, dm = rnd(300, d, seed=6, scale=2.0), rnd(300, d, seed=7).to(dt)
    xm = many + dm.float()
    want = P.rms_norm(xm.to(dt), w, eps) if dtype == "float32" else (w.float() * (xm * torch.rsqrt(xm.pow(2).mean(-1, keepdim=True) + eps)).to(dt).float())
    hg = many.to(gpu).clone()
    close(ops.rmsnorm(hg, w.to(gpu), eps, dt, delta=dm.to(gpu)), want, tol, "norm of many rows")
    close(hg, xm, 1e-7, "stream of many rows after add")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_silu_mul_and_residual_add(gpu, dtype):
    dt = DT[dtype]
    gu = rnd(11, 2 * 352, seed=6, scale=3.0).to(dt)
    g, u = gu[:, :352].float(), gu[:, 352:].float()
    close(ops.silu_mul(gu.to(gpu)), u * g * torch.sigmoid(g), 1e-6 if dtype == "float32" else 5e-3)
    odd = rnd(7, 2 * 353, seed=16, scale=3.0).to(dt)  # a width that is no multiple of 4
    g, u = odd[:, :353].float(), odd[:, 353:].float()
    close(ops.silu_mul(odd.to(gpu)), u * g * torch.sigmoid(g), 1e-6 if dtype == "float32" else 5e-3)
    for rows, F in ((7, 348), (301, 1000), (2048, 1432)):  # multiples of 4 only and of 8; many rows
        big = rnd(rows, 2 * F, seed=17, scale=3.0).to(dt)
        g, u = big[:, :F].float(), big[:, F:].float()
        close(ops.silu_mul(big.to(gpu)), u * g * torch.sigmoid(g), 1e-6 if dtype == "float32" else 5e-3)
    h, d = rnd(5, 77, seed=7), rnd(5, 77, seed=8).to(dt)
    close(ops.residual_add(h.to(gpu).clone(), d.to(gpu)), h + d.float(), 1e-7)


def paged_cache(k, v, page_size, seed, n_extra=3, dtype=torch.float32, poison=True):
    """Scatters dense keys/values [n, K, D] of ONE request over randomly chosen pages.
    Returns (k_pages, v_pages, table row) with NaN in every slot that holds nothing."""
    n, K, D = k.shape
    n_logical = -(-n // page_size)
    n_pages = n_logical + n_extra + 1
    perm = torch.randperm(n_pages - 1, generator=torch.Generator().manual_seed(seed))[:n_logical] + 1
    fill = float("nan") if poison else 0.0
    kp = torch.full((n_pages, K, page_size, D), fill)
    vp = torch.full((n_pages, K, D, page_size), fill)
    for j in range(n):
        p, o = int(perm[j // page_size]), j % page_size
        kp[p, :, o, :] = k[j]
        vp[p, :, :, o] = v[j]
    return kp.to(dtype), vp.to(dtype), perm.to(torch.int32)


def tiled_maps(page, D):
    """Where element (slot, d) of one kv head's part of a page lies in the tiled page
    layout: per block of 32 slots, keys as [16-key tile][32-dim step][dim quad][key][8 dims]
    with slot r = key (r/8)*4 + r%4 of tile (r%8)/4, values as [16-dim tile][8-key group]
    [dim][8 keys].  Both maps are permutations of the page's elements."""
    slot, d = torch.arange(page).view(-1, 1), torch.arange(D).view(1, -1)
    r = slot % 32
    tile, key = (r % 8) // 4, (r // 8) * 4 + r % 4
    kmap = (slot // 32) * 32 * D + ((tile * (D // 32) + d // 32) * 64 + ((d % 32) // 8) * 16 + key) * 8 + d % 8
    vmap = (slot // 32) * 32 * D + ((d // 16) * 64 + (r // 8) * 16 + d % 16) * 8 + r % 8
    for m in (kmap, vmap):
        assert sorted(m.flatten().tolist()) == list(range(page * D))
    return kmap.flatten(), vmap.flatten()


def to_tiled(kp, vp):
    """Plain pages (keys [P, K, page, D], values [P, K, D, page]) in the tiled layout
    (same shapes, other order of the elements of a (page, kv head))."""
    P_, K, page, D = kp.shape
    kmap, vmap = tiled_maps(page, D)
    kt, vt = torch.empty(P_, K, page * D, dtype=kp.dtype), torch.empty(P_, K, page * D, dtype=vp.dtype)
    kt[:, :, kmap] = kp.reshape(P_, K, page * D)
    vt[:, :, vmap] = vp.transpose(2, 3).reshape(P_, K, page * D)
    return kt.view(P_, K, page, D), vt.view(P_, K, D, page)


def from_tiled(kt, vt):
    P_, K, page, D = kt.shape
    kmap, vmap = tiled_maps(page, D)
    kp = kt.reshape(P_, K, page * D)[:, :, kmap].view(P_, K, page, D)
    vp = vt.reshape(P_, K, page * D)[:, :, vmap].view(P_, K, page, D).transpose(2, 3)
    return kp, vp


def rope_case(gpu, dtype, interleaved, H, K, D, rot, page, tiled, lens, starts):
    dt = DT[dtype]
    n_seg = len(lens)
    reach = max(s + n for s, n in zip(starts, lens))  # positions in use
    table_w = -(-reach // page)
    T = sum(lens)
    qkv = rnd(T, (H + 2 * K) * D, seed=9).to(dt)
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)]).to(torch.int32)
    token_seg = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)]).to(torch.int32)
    n_pages = n_seg * table_w + 8
    bt = torch.randperm(n_pages - 1, generator=torch.Generator().manual_seed(1))[: n_seg * table_w].view(n_seg, table_w) + 1
    inv = P.inverse_frequencies(rot, 10000.0)
    cos, sin = P.rotation_table(torch.arange(reach), inv)
    kp = torch.zeros(n_pages, K, page, D, dtype=dt, device=gpu)
    vp = torch.zeros(n_pages, K, D, page, dtype=dt, device=gpu)
    got = qkv.to(gpu).clone()
    ops.rope_append(got, positions.to(gpu), cos.to(gpu), sin.to(gpu), H, K, D, rot, interleaved,
                    token_seg=token_seg.to(gpu), block_table=bt.to(torch.int32).to(gpu),
                    k_pages=kp, v_pages=vp, page_size=page, tiled=tiled)
    q = qkv[:, : H * D].float().view(T, H, D)
    k = qkv[:, H * D : (H + K) * D].float().view(T, K, D)
    v = qkv[:, (H + K) * D :].float().view(T, K, D)
    rotate = P.rotate_interleaved if interleaved else P.rotate_half_split
    c, s = cos[positions.long()], sin[positions.long()]
    rq = torch.cat((rotate(q[..., :rot], c, s), q[..., rot:]), -1)
    rk = torch.cat((rotate(k[..., :rot], c, s), k[..., rot:]), -1)
    tol = 1e-6 if dtype == "float32" else 8e-3
    close(got[:, : H * D].view(T, H, D), rq, tol, "rotated q")
    close(got[:, H * D : (H + K) * D].view(T, K, D), rk, tol, "rotated k")
    assert torch.equal(got[:, (H + K) * D :].cpu(), qkv[:, (H + K) * D :])  # v untouched
    kpc, vpc = kp.float().cpu(), vp.float().cpu()
    if tiled:
        kpc, vpc = from_tiled(kpc, vpc)
    pg = bt[token_seg.long(), positions.long() // page]
    off = positions.long() % page
    close(kpc[pg, :, off, :], rk, tol, "k pages")
    assert torch.equal(vpc[pg, :, :, off], v.to(dt).float())
    written = torch.zeros(n_pages, page, dtype=torch.bool)
    written[pg, off] = True
    assert float(kpc.abs().sum(dim=(1, 3))[~written].sum()) == 0  # nothing else was written
    assert float(vpc.abs().sum(dim=(1, 2))[~written].sum()) == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("H,K,D,rot,page,tiled", [
    (4, 2, 16, 16, 4, False), (6, 2, 48, 48, 16, False), (3, 1, 32, 16, 8, False), (8, 8, 128, 128, 64, False),
    (8, 8, 128, 128, 64, True), (3, 1, 32, 16, 32, True), (4, 2, 64, 64, 32, True), (2, 1, 96, 40, 64, True)])
def test_rope_append(gpu, dtype, interleaved, H, K, D, rot, page, tiled):
    # runs of eight aligned positions and ragged ends
    rope_case(gpu, dtype, interleaved, H, K, D, rot, page, tiled, [5, 1, 9, 20], [3, 40, 0, 6])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("H,K,D,rot,page,tiled", [
    (6, 2, 48, 48, 16, False), (8, 8, 128, 128, 64, True), (4, 2, 64, 64, 32, True), (2, 1, 96, 40, 64, True),
    (3, 1, 32, 16, 8, False)])
def test_rope_append_of_many_tokens(gpu, dtype, interleaved, H, K, D, rot, page, tiled):
    """Steps of many tokens take a kernel of their own (eight tokens to a workgroup): runs of
    eight positions that start inside one workgroup's tokens and end in the next one's,
    segments that end in the middle of a workgroup's tokens, a last workgroup with fewer."""
    rope_case(gpu, dtype, interleaved, H, K, D, rot, page, tiled, [705, 1, 303, 611, 5], [3, 40, 0, 26, 8])
    rope_case(gpu, dtype, interleaved, H, K, D, rot, page, tiled, [2048], [512])


@pytest.mark.parametrize("M", [1, 5, 16, 17, 32])
@pytest.mark.parametrize("H,K,D,width,page,tiled", [
    (4, 2, 16, 64, 8, False), (6, 3, 48, 120, 16, False), (5, 1, 80, 200, 4, False),
    (8, 2, 64, 352, 32, True), (32, 8, 128, 4096, 64, True), (2, 2, 160, 96, 64, True),
])
def test_qkv_rope_append_in_one_kernel(gpu, M, H, K, D, width, page, tiled):
    """Projection, rotation and append in one kernel against the three steps one by one
    (the same kernels' unfused forms) and against the plain rotation."""
    dt = torch.bfloat16
    n_seg, table_w = 3, -(-64 // page)
    # tokens of three requests: a run of neighbouring positions, and single ones
    lens = [M - 2, 1, 1] if M > 2 else [M]
    starts = [11, 40, 0][: len(lens)]
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)]).to(torch.int32)
    token_seg = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)]).to(torch.int32)
    n_pages = n_seg * table_w + 5
    bt = (torch.randperm(n_pages - 1, generator=torch.Generator().manual_seed(2))[: n_seg * table_w]
          .view(n_seg, table_w) + 1).to(torch.int32)
    w = (rnd((H + 2 * K) * D, width, seed=3) * 0.2).to(dt).to(gpu)
    x = rnd(M, width, seed=4).to(dt).to(gpu)
    cos, sin = P.rotation_table(torch.arange(64), P.inverse_frequencies(D, 10000.0))
    cos, sin = cos.contiguous().to(gpu), sin.contiguous().to(gpu)
    pages = lambda: (torch.zeros(n_pages, K, page, D, dtype=dt, device=gpu), torch.zeros(n_pages, K, D, page, dtype=dt, device=gpu))

    paired = ops.tile_weight(ops.pair_rows_for_rotation(w, D))
    kp, vp = pages()
    q = ops.qkv_rope_append(x, paired, positions.to(gpu), cos, sin, H, K, D, token_seg.to(gpu), bt.to(gpu),
                            kp, vp, page, tiled)

    qkv = ops.gemm_bf16_skinny(x, ops.tile_weight(w), tiled_shape=tuple(w.shape))
    plain_qkv = qkv.float().cpu()
    kp2, vp2 = pages()
    ops.rope_append(qkv, positions.to(gpu), cos, sin, H, K, D, D, False, token_seg=token_seg.to(gpu),
                    block_table=bt.to(gpu), k_pages=kp2, v_pages=vp2, page_size=page, tiled=tiled)
    # the same sums in the same order, rounded at the same places
    close(q, qkv[:, : H * D], 4e-3, "rotated q, fused against unfused")
    close(kp, kp2, 4e-3, "key pages")
    if M <= 16:  # the same sums in the same order; beyond, the unfused product splits K otherwise
        assert torch.equal(vp, vp2)
    close(vp, vp2, 4e-3, "value pages")
    # and the rotation itself against the plain one, from the unrotated product
    c, s_ = cos.cpu()[positions.long()], sin.cpu()[positions.long()]
    want_q = P.rotate_half_split(plain_qkv[:, : H * D].view(M, H, D), c, s_)
    close(q.view(M, H, D), want_q, 8e-3, "rotated q against the plain rotation")
    assert float(kp.float().abs().sum()) > 0


@pytest.mark.parametrize("M", [1, 7, 16, 19, 32])
@pytest.mark.parametrize("d,F,wdt", [(64, 96, "float32"), (120, 352, "bfloat16"), (4096, 1024, "bfloat16"), (1000, 200, "bfloat16"),
                                     (8192, 512, "bfloat16")])  # the last: more partial sums than a thread asks for ahead
def test_norm_folded_into_the_products_around_it(gpu, M, d, F, wdt):
    """product -> add into the stream -> RMSNorm -> product (plain and gated), with the norm
    done by the two products, against the same chain with the norm's own kernel and
    against plain arithmetic."""
    dt = torch.bfloat16
    eps = 1e-5
    a = rnd(M, F, seed=1).to(dt).to(gpu)                      # what the first product reads
    w1 = (rnd(d, F, seed=2) * 0.3).to(dt).to(gpu)             # into the stream
    w2 = (rnd(F, d, seed=3) * 0.3).to(dt).to(gpu)             # out of the norm (gate)
    w3 = (rnd(F, d, seed=4) * 0.3).to(dt).to(gpu)             # out of the norm (up)
    nw = (1.0 + 0.5 * rnd(d, seed=5)).to(DT[wdt]).to(gpu)
    h0 = (rnd(M, d, seed=6) * 3.0).to(gpu)
    h0[0, 3] = 40.0  # one large element: a row's scale must come from the whole row
    t1, t2, t3 = ops.tile_weight(w1), ops.tile_weight(w2), ops.tile_weight(w3)

    # the norm's own kernel between the products
    h_ref = h0.clone()
    delta = ops.gemm_bf16_skinny(a, t1, tiled_shape=(d, F))
    y = ops.rmsnorm(h_ref, nw, eps, dt, delta=delta)
    plain_out = ops.gemm_bf16_skinny(y, t2, tiled_shape=(F, d))
    gated_out = ops.gemm_bf16_skinny(y, t2, w_up=t3, tiled_shape=(F, d))

    # folded
    h = h0.clone()
    rows = ops.gemm_bf16_skinny_norm(a, t1, (d, F), next_norm=ops.NextNorm(h, nw, eps))
    assert isinstance(rows, ops.NormedRows) and rows.ss_parts.shape == (-(-d // 16), 16 * -(-M // 16))
    if M <= 16:  # the same sums, rounded at the same place, added to the same stream
        assert torch.equal(h, h_ref)
    close(h, h_ref, 1e-3, "the stream")  # beyond 16 rows the unfused product splits K otherwise
    close(rows.ss_parts.sum(0)[:M], (h_ref.double() ** 2).sum(1), 1e-5, "sums of squares")
    assert float(rows.ss_parts[:, M:].abs().sum()) == 0
    close(rows.materialize(), y, 1.2e-2, "rows made whole")
    scaled = rows.x.float() * torch.rsqrt(rows.ss_parts.double().sum(0)[:M] / d + eps).float()[:, None]
    off = (rows.materialize().float() - scaled.to(dt).float()).abs() / scaled.abs().clamp_min(1e-6)
    assert float(off.max()) <= 2 ** -7, "rows made whole: more than one bf16 step from x * rstd"
    got_plain = ops.gemm_bf16_skinny_norm(rows, t2, (F, d))
    got_gated = ops.gemm_bf16_skinny_norm(rows, t2, (F, d), w_up_tiled=t3)
    close(got_plain, plain_out, 1.5e-2, "plain product after the folded norm")
    close(got_gated, gated_out, 2e-2, "gated product after the folded norm")

    # plain arithmetic in float64 from the same stream
    hd = h_ref.double().cpu()
    n64 = hd * torch.rsqrt((hd ** 2).mean(1, keepdim=True) + eps) * nw.double().cpu()
    close(got_plain, n64 @ w2.double().cpu().T, 1.5e-2, "against float64")
    g, u = n64 @ w2.double().cpu().T, n64 @ w3.double().cpu().T
    close(got_gated, u * g * torch.sigmoid(g), 2e-2, "gated against float64")
    # through linear(): the same two calls, and a reader without a tiled copy gets whole rows
    h = h0.clone()
    rows2 = ops.linear(a, w1, tiled=t1, next_norm=ops.NextNorm(h, nw, eps))
    if ops.norm_folds(M, d, F, t1):
        assert torch.equal(rows2.x, rows.x) and float((h - h_ref).abs().max()) <= 1e-3 * float(h_ref.abs().max())
    else:  # beyond 16 rows linear() folds only where that is the faster way; the result is then as ever
        assert isinstance(rows2, torch.Tensor) and torch.equal(h, h0)
        close(rows2, delta, 4e-3, "the product alone")
    if ops.norm_folds(M, F, d, t2):
        assert torch.equal(ops.linear(rows, w2, tiled=t2), got_plain)
    close(ops.linear(rows, w2), plain_out, 1.5e-2, "materialised rows")
    assert isinstance(ops.linear(a, w1, next_norm=ops.NextNorm(h0.clone(), nw, eps)), torch.Tensor)


def attention_case(gpu, dtype, H, K, D, page, segs, window, seed, use, tiled=False):
    """``segs``: list of (cached before, new tokens).  Builds one dense sequence per
    segment, pages it, and compares the rows of the new tokens with plain attention
    over the whole sequence."""
    dt = DT[dtype]
    scale = D**-0.5
    qs, tables, kps, vps, want, pos, seg_of = [], [], [], [], [], [], []
    page_base = 0
    all_k, all_v = [], []
    for i, (before, new) in enumerate(segs):
        n = before + new
        q = rnd(n, H, D, seed=seed + 3 * i).to(dt).float()
        k = rnd(n, K, D, seed=seed + 3 * i + 1).to(dt).float()
        v = rnd(n, K, D, seed=seed + 3 * i + 2).to(dt).float()
        if n > 40:  # one far key stands out: a kernel that drops or misplaces it shows
            far = 3
            k[far] = 0
            k[far, :, 0] = 6.0
            q[-1, :, :] = 0
            q[-1, :, 0] = 6.0 * math.sqrt(D) / 6.0 * 2.0
            v[far] = 5.0
        ref = P.causal_attention(q, k, v, window=window or None)
        want.append(ref[before:].reshape(new, H * D))
        qs.append(q[before:].reshape(new, H * D))
        kp, vp, row = paged_cache(k, v, page, seed + i, dtype=dt)
        tables.append(row + page_base)
        page_base += kp.shape[0]
        kps.append(kp), vps.append(vp)
        pos.append(torch.arange(before, n))
        seg_of.append(torch.full((new,), i))
    width = max(len(t) for t in tables)
    bt = torch.full((len(segs), width), -1, dtype=torch.int32)
    for i, t in enumerate(tables):
        bt[i, : len(t)] = t
    k_pages, v_pages = torch.cat(kps), torch.cat(vps)
    if window:
        # pages that the window of a segment's first new token has passed are given back in
        # the engine; here their entries name a page of NaN, so that a kernel that uses one shows
        k_pages = torch.cat((k_pages, torch.full_like(k_pages[:1], float("nan"))))
        v_pages = torch.cat((v_pages, torch.full_like(v_pages[:1], float("nan"))))
        for i, (before, new) in enumerate(segs):
            bt[i, : max(0, before - window + 1) // page] = k_pages.shape[0] - 1
    if tiled:
        k_pages, v_pages = to_tiled(k_pages, v_pages)
    k_pages, v_pages, is_tiled = k_pages.to(gpu), v_pages.to(gpu), tiled
    q = torch.cat(qs).to(dt).to(gpu)
    positions = torch.cat(pos).to(torch.int32).to(gpu)
    token_seg = torch.cat(seg_of).to(torch.int32).to(gpu)
    if use in ("simple", "rows"):
        # as the engine calls it: the fewest tokens of a request decide between the kernel of
        # the vector units and, for steps of prompts alone, the one of the matrix cores;
        # "rows" claims many tokens whatever the step holds, which is wrong and must cost time only
        fewest = 10**6 if use == "rows" else min(new for _, new in segs)
        out = ops.attention_simple(q, H * D, positions, token_seg, bt.to(gpu), k_pages, v_pages, H, scale, window,
                                   max_kv_len=max(b + n for b, n in segs), min_q_len=fewest)
    else:
        q_len = np.array([n for _, n in segs], dtype=np.int32)
        kv_len = np.array([b + n for b, n in segs], dtype=np.int32)
        plan = attn_kernels.plan_items(q_len, kv_len, H // K, K, window, attn_kernels.rows_per_big_item(D))
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)

        class Ctx:
            n_tokens = int(q_len.sum())
            seg_q_start = dev(np.concatenate(([0], np.cumsum(q_len)[:-1])).astype(np.int32))
            seg_q_len = dev(q_len)
            seg_kv_len = dev(kv_len)

        class Group:
            block_table = bt.to(gpu)

        class KV:
            k, v, tiled = k_pages, v_pages, is_tiled

        out = attn_kernels.attention_mfma(q, H * D, attn_kernels.upload_plan(plan, gpu), Ctx, Group, KV, H, scale, window)
    close(out, torch.cat(want), 5e-6 if dtype == "float32" else 1.2e-2, f"attention {use}")


SHAPES = [(4, 2, 16), (6, 2, 48), (4, 1, 32), (8, 8, 64), (32, 8, 128), (5, 5, 80), (20, 1, 16), (4, 2, 256), (6, 3, 112), (2, 1, 160)]
SEGS = [[(0, 1)], [(0, 70)], [(63, 1), (0, 33), (64, 64), (129, 2), (200, 1)], [(700, 1), (5, 300)]]
PROMPTS = [[(0, 200)], [(37, 130), (0, 64), (500, 90)], [(0, 9), (100, 8), (31, 33)], [(1000, 129)]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("segs", SEGS + PROMPTS[:2])
@pytest.mark.parametrize("H,K,D", SHAPES[:5])
def test_attention_simple(gpu, dtype, H, K, D, segs):
    for page, window in ((1, 0), (4, 0), (16, 0), (64, 0), (16, 37), (4, 1)):
        attention_case(gpu, dtype, H, K, D, page, segs, window, seed=20, use="simple")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("segs", [[(2000, 1), (900, 1), (40, 1), (1199, 2), (383, 1)], [(1300, 1)], [(255, 1), (256, 1), (127, 2)]])
@pytest.mark.parametrize("H,K,D", SHAPES[:5] + [(20, 1, 16), (4, 2, 256), (2, 1, 320)])
def test_attention_simple_pieces_of_decode_tokens(gpu, dtype, H, K, D, segs):
    """Steps of few tokens: every piece of a row's keys is a workgroup of its own and a second
    kernel joins them; the fewer the rows, the smaller the pieces (512, 256 or 128 keys).  With
    windows that begin inside a piece, and pages smaller and larger than a block."""
    for page, window in ((1, 0), (16, 0), (64, 0), (16, 300), (4, 37), (64, 130)):
        attention_case(gpu, dtype, H, K, D, page, segs, window, seed=27, use="simple")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("segs", SEGS + PROMPTS)
@pytest.mark.parametrize("H,K,D", SHAPES[:7] + [(7, 1, 24), (3, 3, 128), (256, 1, 8)])
def test_attention_of_many_rows_a_request(gpu, dtype, H, K, D, segs):
    """The 32-bit kernel on the matrix cores, which steps of prompts alone take: every head
    size it serves (multiples of 8 up to 128), groups that fill a wave's 32 rows unevenly or
    are more than a workgroup's 128, and steps that it would not be given (single tokens)."""
    for page, window in ((1, 0), (4, 0), (16, 0), (64, 0), (16, 37), (4, 1), (8, 70)):
        attention_case(gpu, dtype, H, K, D, page, segs, window, seed=25, use="rows")


@pytest.mark.parametrize("segs", SEGS)
@pytest.mark.parametrize("H,K,D", SHAPES)
def test_attention_mfma(gpu, H, K, D, segs):
    for page, window in ((8, 0), (16, 0), (64, 0), (24, 0), (16, 37), (8, 1), (64, 300)):
        attention_case(gpu, "bfloat16", H, K, D, page, segs, window, seed=30, use="mfma")
    if D % 32 == 0:  # the pages in the kernel's own order
        for page, window in ((32, 0), (64, 0), (128, 0), (64, 300), (32, 37)):
            attention_case(gpu, "bfloat16", H, K, D, page, segs, window, seed=31, use="mfma", tiled=True)


@pytest.mark.parametrize("H,K,D", SHAPES)
def test_attention_mfma_pieces_of_decode_tokens(gpu, H, K, D):
    """Decode tokens against key ranges of one piece (joined in the workgroup, some of its four
    quarters empty) and of several (joined there into partial results, which the workgroup that
    comes last merges), at every
    head size, with windows that start a range in the middle of a block."""
    segs = [(2000, 1), (900, 1), (40, 1), (1199, 2), (383, 1)]
    if 2 * (H // K) <= 16:  # every segment is one tile: three of the ranges are cut
        q_len, kv_len = np.array([n for _, n in segs]), np.array([b + n for b, n in segs])
        plan = attn_kernels.plan_items(q_len, kv_len, H // K, K, 0, attn_kernels.rows_per_big_item(D))
        assert plan.n_big == 0 and plan.n_items == 4 * 12
        if K * 5 * 8 >= 256:  # few enough pieces a tile that the attention kernel merges them itself
            assert sorted(set(plan.items[:, 9].tolist())) == [0, 2, 3, 5] and plan.n_merges == 0
        else:
            assert sorted(plan.merges[:, 3].tolist()) == [2, 3, 5] and not plan.merged_in_kernel
    for page, window, tiled in ((16, 0, False), (64, 0, D % 32 == 0), (8, 37, False), (64, 1000, D % 32 == 0), (24, 601, False)):
        attention_case(gpu, "bfloat16", H, K, D, page, segs, window, seed=33, use="mfma", tiled=tiled)


def test_attention_mfma_merges_in_the_kernel_the_same_every_time(gpu):
    """Eight decode tokens against a few thousand keys each: every tile's key range has four
    pieces, and the workgroup that finishes a tile last merges them.  Which one that is
    varies from launch to launch; the result must not."""
    H, K, D, page = 32, 8, 128, 64
    lens = [3000, 4100, 2047, 3500, 1600, 4096, 2500, 3999]
    rng = torch.Generator().manual_seed(70)
    n_pages = sum(-(-n // page) for n in lens)
    k_pages = (torch.randn((n_pages, K, page, D), generator=rng) * 0.5).to(torch.bfloat16).to(gpu)
    v_pages = torch.randn((n_pages, K, D, page), generator=rng).to(torch.bfloat16).to(gpu)  # (values are kept transposed)
    order = torch.randperm(n_pages, generator=rng).to(torch.int32)
    width = max(-(-n // page) for n in lens)
    bt = torch.full((len(lens), width), -1, dtype=torch.int32)
    at = 0
    for i, n in enumerate(lens):
        bt[i, : -(-n // page)] = order[at : at + -(-n // page)]
        at += -(-n // page)
    q = torch.randn((len(lens), H * D), generator=rng).to(torch.bfloat16)
    # one key in the third of the first request's four pieces gets most of the weight: a piece
    # that is dropped, or merged with a wrong maximum, shows
    far = 1700
    far_page, far_off = int(bt[0, far // page]), far % page
    k_pages[far_page, :, far_off, :] = 0
    k_pages[far_page, :, far_off, 1] = 8.0
    v_pages[far_page, :, :, far_off] = 3.0
    q[0].view(H, D)[:, 1] = 12.0
    q = q.to(gpu)
    q_len, kv_len = np.ones(len(lens), dtype=np.int32), np.array(lens, dtype=np.int32)
    plan = attn_kernels.plan_items(q_len, kv_len, H // K, K, 0, attn_kernels.rows_per_big_item(D))
    assert plan.merged_in_kernel and plan.n_merges == 0 and (plan.items[:, 9] == 4).all()
    holds_far = plan.items[(plan.items[:, 0] == 0) & (plan.items[:, 2] <= far) & (far < plan.items[:, 3])]
    assert len(holds_far) == 1 and holds_far[0, 4] - holds_far[0, 8] == 2  # the third piece's slot
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)

    class Ctx:
        n_tokens = len(lens)
        seg_q_start = dev(np.arange(len(lens), dtype=np.int32))
        seg_q_len = dev(q_len)
        seg_kv_len = dev(kv_len)

    class Group:
        block_table = bt.to(gpu)

    class KV:
        k, v, tiled = k_pages, v_pages, False

    plan_dev = attn_kernels.upload_plan(plan, gpu)
    first = attn_kernels.attention_mfma(q, H * D, plan_dev, Ctx, Group, KV, H, D**-0.5, 0)
    # against plain attention over the gathered keys
    for i, n in enumerate(lens):
        pages = bt[i, : -(-n // page)].long()
        k = k_pages[pages].permute(0, 2, 1, 3).reshape(-1, K, D)[:n].float().cpu()
        v = v_pages[pages].permute(0, 3, 1, 2).reshape(-1, K, D)[:n].float().cpu()
        qi = q[i].float().cpu().view(H, D)
        want = torch.stack([torch.softmax(k[:, h // (H // K)] @ qi[h] * D**-0.5, 0) @ v[:, h // (H // K)] for h in range(H)])
        close(first[i].view(H, D), want, 1.2e-2, f"request {i}")
        if i == 0:
            assert float(want.abs().min()) > 0.5  # the far key decides
    for _ in range(300):
        again = attn_kernels.attention_mfma(q, H * D, plan_dev, Ctx, Group, KV, H, D**-0.5, 0)
        assert torch.equal(again, first)
    assert int(attn_kernels._counters(gpu).abs().sum()) == 0  # every count was set back


def test_attention_mfma_split_keys(gpu):
    # few rows and many keys: the key range is cut and merged (so few tiles that a tile may have
    # more pieces than the attention kernel merges itself: the merge kernel's work)
    segs = [(3000, 1), (1500, 2), (4000, 1)]
    plan = attn_kernels.plan_items(np.array([1, 2, 1]), np.array([3001, 1502, 4001]), 4, 2, 0)
    assert plan.n_merges == 3 and plan.n_big == 0 and not plan.merged_in_kernel
    attention_case(gpu, "bfloat16", 8, 2, 128, 64, segs, 0, seed=40, use="mfma")
    attention_case(gpu, "bfloat16", 8, 2, 128, 16, segs, 1000, seed=41, use="mfma")
    # a short portion against a long context: tiles of 64 rows, cut and merged
    attention_case(gpu, "bfloat16", 8, 2, 128, 64, [(5000, 40), (2500, 100)], 0, seed=42, use="mfma")
    attention_case(gpu, "bfloat16", 6, 2, 48, 16, [(3000, 50)], 700, seed=43, use="mfma")
    attention_case(gpu, "bfloat16", 8, 2, 128, 64, segs, 0, seed=44, use="mfma", tiled=True)
    attention_case(gpu, "bfloat16", 8, 2, 128, 64, [(5000, 40), (2500, 100)], 0, seed=45, use="mfma", tiled=True)
    attention_case(gpu, "bfloat16", 4, 1, 64, 32, [(3000, 50), (0, 600)], 700, seed=46, use="mfma", tiled=True)
    # few partial results per row: the merge kernel of one wave per row
    for segs, heads in (([(512, 256)], (8, 2)), ([(300, 200), (0, 64)], (4, 1))):
        q_len, kv_len = np.array([n for _, n in segs]), np.array([b + n for b, n in segs])
        plan = attn_kernels.plan_items(q_len, kv_len, heads[0] // heads[1], heads[1], 0, attn_kernels.rows_per_big_item(128))
        assert 1 < plan.max_parts <= 8 and plan.n_merges > 0
        attention_case(gpu, "bfloat16", heads[0], heads[1], 128, 64, segs, 0, seed=47, use="mfma")
        attention_case(gpu, "bfloat16", heads[0], heads[1], 128, 64, segs, 0, seed=48, use="mfma", tiled=True)


@pytest.mark.parametrize("tiled", [False, True])
def test_attention_mfma_hundred_thousand_keys(gpu, tiled):
    """One decoded token against 100,003 cached keys: the key range is cut into far more
    pieces than a wave of the merge kernel joins at once.  The key that decides the
    result lies in the middle of a piece far from both ends."""
    H, K, D, page, n = 8, 2, 128, 64, 100_003
    dt = torch.bfloat16
    k = rnd(n, K, D, seed=60).to(dt).float()
    v = rnd(n, K, D, seed=61).to(dt).float()
    q = rnd(1, H, D, seed=62).to(dt).float()
    far = 61_007
    k[far] = 0
    k[far, :, 1] = 10.0
    q[0, :, 1] = 16.0  # the far key gets about as much weight as all the others together
    v[far] = 3.0
    scale = D**-0.5
    want = torch.empty(H, D, dtype=torch.float64)
    for h in range(H):
        g = h // (H // K)
        p = torch.softmax((k[:, g].double() @ q[0, h].double()) * scale, dim=0)
        want[h] = p @ v[:, g].double()
    assert float(want.abs().max()) > 1.0  # the far key carries weight
    n_logical = -(-n // page)
    perm = torch.randperm(n_logical + 3, generator=torch.Generator().manual_seed(63))[:n_logical] + 1
    pad = n_logical * page - n
    kl = torch.cat((k, torch.full((pad, K, D), float("nan")))).view(n_logical, page, K, D)
    vl = torch.cat((v, torch.full((pad, K, D), float("nan")))).view(n_logical, page, K, D)
    kp = torch.full((n_logical + 4, K, page, D), float("nan"))
    vp = torch.full((n_logical + 4, K, D, page), float("nan"))
    kp[perm] = kl.permute(0, 2, 1, 3)
    vp[perm] = vl.permute(0, 2, 3, 1)
    kp, vp = kp.to(dt), vp.to(dt)
    if tiled:
        kp, vp = to_tiled(kp, vp)
    q_len, kv_len = np.array([1], dtype=np.int32), np.array([n], dtype=np.int32)
    plan = attn_kernels.plan_items(q_len, kv_len, H // K, K, 0, attn_kernels.rows_per_big_item(D))
    assert plan.n_merges == 1 and plan.n_items > 64  # more than 64 partial results per row
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(gpu)

    class Ctx:
        n_tokens = 1
        seg_q_start = dev(np.array([0], dtype=np.int32))
        seg_q_len = dev(q_len)
        seg_kv_len = dev(kv_len)

    class Group:
        block_table = perm.to(torch.int32).view(1, -1).to(gpu)

    class KV:
        pass

    KV.k, KV.v, KV.tiled = kp.to(gpu), vp.to(gpu), tiled
    out = attn_kernels.attention_mfma(q.view(1, H * D).to(dt).to(gpu), H * D, attn_kernels.upload_plan(plan, gpu),
                                      Ctx, Group, KV, H, scale, 0)
    close(out, want.float().view(1, H * D), 1.2e-2, "attention over 100,003 keys")


@pytest.mark.parametrize("M,N,K", [(1, 256, 64), (5, 331, 120), (8, 257, 1000), (9, 130, 36), (16, 1000, 352), (17, 96, 64),
                                   (64, 200, 352), (130, 96, 1000), (3, 4096, 4096), (2, 50, 30),
                                   # columns enough for two waves, and for one, on a set of columns
                                   (7, 8200, 2308), (13, 9001, 260), (4, 16400, 1028), (16, 17003, 520),
                                   # many rows: tiles of the matrix cores, whole and in part; a k that is no multiple of 4
                                   (65, 128, 32), (300, 517, 2052), (1024, 260, 1028), (129, 129, 36), (200, 96, 1001)])
def test_gemm_f32(gpu, M, N, K):
    a, w = rnd(M, K, seed=50), rnd(N, K, seed=51)
    want = (a.double() @ w.double().T).float()
    close(ops.gemm_f32(a.to(gpu), w.to(gpu)), want, 3e-6, "gemm_f32")
    # a row's result does not depend on the other rows of the batch, bit for bit: with
    # other rows beside it (the same kernel, at most 16 rows or more) ...
    whole = ops.gemm_f32(a.to(gpu), w.to(gpu))
    others = a.clone()
    others[1:] = rnd(M, K, seed=52)[1:] * 3.0
    assert torch.equal(whole[:1].cpu(), ops.gemm_f32(others.to(gpu), w.to(gpu))[:1].cpu())
    # ... and alone, where both take the kernel for few rows (the two kernels add in
    # different orders: the last bits may differ between them)
    alone = ops.gemm_f32(a[:1].to(gpu).contiguous(), w.to(gpu))
    if M <= 16:
        assert torch.equal(alone.cpu(), whole[:1].cpu())
    close(alone, whole[:1], 2e-6, "a row alone and in a larger batch")


@pytest.mark.parametrize("M,N,K", [(8, 512, 4096), (16, 512, 14336), (48, 512, 4096), (2048, 384, 4096), (1500, 256, 14336),
                                   (17, 9000, 4096), (100, 300, 14336), (128, 96, 4100), (33, 40, 36)])
def test_gemm_f32_with_rows_as_long_as_the_models(gpu, M, N, K):
    """Every kernel of the 32-bit product against the product in 64-bit, at the row lengths
    of the 8B shape.  One row of W is made of ones and A's entries are positive there, so
    that a kernel which dropped or doubled a stretch of k would show in a sum without
    cancellation."""
    a, w = rnd(M, K, seed=53), rnd(N, K, seed=54)
    w[5] = 1.0
    a[3] = a[3].abs()
    want = (a.double() @ w.double().T).float()
    got = ops.gemm_f32(a.to(gpu), w.to(gpu)).cpu()
    close(got, want, 3e-6, "gemm_f32")
    exact = float(a[3].double().sum())
    assert abs(float(got[3, 5]) - exact) <= 2e-6 * exact


@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(256, 64), (331, 120), (1000, 352), (4096, 4096), (200, 14336)])
def test_gemm_bf16_skinny(gpu, M, N, K):
    x = rnd(M, K, seed=60).to(torch.bfloat16)
    w = rnd(N, K, seed=61, scale=0.05).to(torch.bfloat16)
    w2 = rnd(N, K, seed=62, scale=0.05).to(torch.bfloat16)
    want = x.float() @ w.float().T
    xg, wg, w2g = x.to(gpu), w.to(gpu), w2.to(gpu)
    close(ops.gemm_bf16_skinny(xg, wg, out_dtype=torch.float32), want, 2e-5, "skinny f32")
    close(ops.gemm_bf16_skinny(xg, wg), want, 5e-3, "skinny bf16")
    base = rnd(M, N, seed=63)
    acc = base.to(gpu).clone()
    ops.gemm_bf16_skinny(xg, wg, add_to=acc)
    close(acc, base + want, 2e-5, "skinny add")
    up = x.float() @ w2.float().T
    close(ops.gemm_bf16_skinny(xg, wg, w_up=w2g, out_dtype=torch.float32), up * want * torch.sigmoid(want), 3e-5, "skinny gated")
    with pytest.raises(ops.KernelError):
        ops.gemm_bf16_skinny(rnd(65, K).to(torch.bfloat16).to(gpu), wg)
    # the tiled copy of the weights gives the same sums in the same order
    tw, tw2 = ops.tile_weight(wg), ops.tile_weight(w2g)
    assert tw.numel() == (-(-N // 16) * 16) * (-(-K // 32) * 32)
    a = ops.gemm_bf16_skinny(xg, wg, out_dtype=torch.float32)
    b = ops.gemm_bf16_skinny(xg, tw, out_dtype=torch.float32, tiled_shape=(N, K))
    assert torch.equal(a, b)
    a = ops.gemm_bf16_skinny(xg, wg, w_up=w2g)
    b = ops.gemm_bf16_skinny(xg, tw, w_up=tw2, tiled_shape=(N, K))
    assert torch.equal(a, b)


def test_linear_dispatch(gpu):
    x = rnd(100, 352, seed=70).to(torch.bfloat16).to(gpu)
    w = rnd(331, 352, seed=71, scale=0.05)
    want = x.float().cpu() @ w.to(torch.bfloat16).float().T
    close(ops.linear(x, w.to(torch.bfloat16).to(gpu)), want, 8e-3, "library product")
    close(ops.linear(x, w.to(torch.bfloat16).to(gpu), out_dtype=torch.float32), want, 3e-5, "float32 output in passes")
    # a 32-bit weight under bfloat16 activations runs the 32-bit kernel
    close(ops.linear(x, w.to(gpu), out_dtype=torch.float32), x.float().cpu() @ w.T, 3e-6, "32-bit weight")
    assert ops.linear(x, w.to(gpu)).dtype == torch.bfloat16


def _sample(gpu, logits, spread=False, **kw):
    n = logits.shape[0]
    f = lambda v, dt: torch.full((n,), v, dtype=dt, device=gpu) if not torch.is_tensor(v) else v.to(gpu)
    return ops.sample(
        logits.to(gpu), f(kw.get("temperature", 1.0), torch.float32), f(kw.get("top_k", -1), torch.int32),
        f(kw.get("top_p", 1.0), torch.float32), f(kw.get("min_p", 0.0), torch.float32),
        f(kw.get("seed", 7), torch.int64), kw.get("draw", torch.arange(n, dtype=torch.int32)).to(gpu),
        spread=spread,
    )


@pytest.mark.parametrize("vocab", [331, 1000, 128256])
def test_sample_greedy(gpu, vocab):
    logits = rnd(6, vocab, seed=80, scale=2.0)
    logits[1, 5] = logits[1, 300] = 50.0  # a tie: the first index wins, as torch.argmax
    logits[2, 17] = float("nan")
    tok, lp = _sample(gpu, logits, temperature=0.0)
    clean = torch.where(torch.isnan(logits), torch.full_like(logits, -1e5), logits)
    assert tok.cpu().tolist() == torch.argmax(clean, -1).tolist() and tok[1] == 5
    want = torch.log_softmax(clean.double(), -1).gather(1, tok.cpu().long()[:, None])[:, 0]
    close(lp, want.float(), 1e-5, "greedy logprob")
    tok2, _ = _sample(gpu, logits, temperature=0.9, top_k=1)
    assert torch.equal(tok, tok2)
    # the rows spread over many blocks (what the engine uses when no row samples)
    n = logits.shape[0]
    f = lambda v, dt: torch.full((n,), v, dtype=dt, device=gpu)
    tok3, lp3 = ops.sample(logits.to(gpu), f(0.0, torch.float32), f(-1, torch.int32), f(1.0, torch.float32),
                           f(0.0, torch.float32), f(7, torch.int64), f(0, torch.int32), all_greedy=True)
    assert torch.equal(tok, tok3)
    close(lp3, want.float(), 1e-5, "greedy logprob, many blocks")


@pytest.mark.parametrize("kw", [{}, {"top_k": 5}, {"top_p": 0.7}, {"top_k": 40, "top_p": 0.9}, {"min_p": 0.1},
                                {"top_k": 9, "top_p": 0.8, "min_p": 0.05}, {"temperature": 0.6, "top_p": 0.5}])
def test_sample_matches_the_plain_sampler(gpu, kw):
    vocab, n = 1000, 400
    base = rnd(1, vocab, seed=81, scale=2.5)[0]
    logits = base[None].repeat(n, 1)
    # one block per row, and the rows spread over many blocks
    both_ways = [_sample(gpu, logits, seed=11, **kw), _sample(gpu, logits, seed=11, spread=True, **kw)]
    for tok, lp in both_ways:
        _compare_with_plain(base, kw, tok, lp, n)


def _compare_with_plain(base, kw, tok, lp, n):
    params = {"temperature": 1.0, "seed": 11, **kw}
    probs = P.filtered_probabilities(base, params["temperature"], params.get("top_k", -1), params.get("top_p", 1.0), params.get("min_p", 0.0))
    agree = 0
    for i in range(n):
        t, logprob, margin = P.sample_token(base, params, i)
        assert probs[int(tok[i])] > 0, "a filtered token was sampled"
        if margin > 2e-5:
            assert int(tok[i]) == t, f"draw {i}: kernel {int(tok[i])}, plain {t}"
            assert abs(float(lp[i]) - logprob) < 1e-4
            agree += 1
    assert agree > 0.85 * n


@pytest.mark.parametrize("vocab", [50257, 128256])
def test_sample_large_vocabulary(gpu, vocab):
    """Many tokens per thread: the filters' thresholds and the drawn tokens against the
    plain sampler, with and without the room for keys between the passes."""
    base = rnd(1, vocab, seed=83, scale=3.0)[0]
    base[vocab // 3] = float("nan")
    n = 24
    logits = base[None].repeat(n, 1)
    for kw in ({"top_p": 0.9, "temperature": 0.8}, {"top_k": 50}, {"top_k": 200, "top_p": 0.6, "min_p": 0.02}, {}):
        params = {"temperature": 1.0, "seed": 5, **kw}
        clean = torch.where(torch.isnan(base), torch.full_like(base, -1e5), base)
        probs = P.filtered_probabilities(clean, params["temperature"], params.get("top_k", -1), params.get("top_p", 1.0), params.get("min_p", 0.0))
        tok, lp = _sample(gpu, logits, seed=5, **kw)
        f = lambda v, dt: torch.full((n,), v, dtype=dt, device=gpu)
        tok_again, _ = ops.sample(
            logits.to(gpu), f(params["temperature"], torch.float32), f(kw.get("top_k", -1), torch.int32),
            f(kw.get("top_p", 1.0), torch.float32), f(kw.get("min_p", 0.0), torch.float32), f(5, torch.int64),
            torch.arange(n, dtype=torch.int32, device=gpu), key_scratch=False,  # the keys are derived again in every pass
        )
        assert torch.equal(tok, tok_again)
        ways = [(tok, lp), _sample(gpu, logits, seed=5, spread=True, **kw)]  # and spread over many blocks
        for tok, lp in ways:
            agree = 0
            for i in range(n):
                t, logprob, margin = P.sample_token(clean, params, i)
                assert probs[int(tok[i])] > 0, f"{kw}: a filtered token was sampled"
                if margin > 2e-5:
                    assert int(tok[i]) == t, f"{kw} draw {i}: kernel {int(tok[i])}, plain {t}"
                    assert abs(float(lp[i]) - logprob) < 2e-4
                    agree += 1
            assert agree > 0.8 * n


@pytest.mark.parametrize("vocab", [331, 1000, 50257, 128256])
def test_sample_unfiltered_rows_over_many_blocks(gpu, vocab):
    """Rows without filters (greedy ones among them) spread over many blocks: the tokens and
    log-probabilities of the plain sampler, and of the one-block kernel wherever the draw is
    not within rounding of a token's edge."""
    n = 48
    base = rnd(1, vocab, seed=85, scale=3.0)[0]
    base[vocab // 5] = float("nan")
    clean = torch.where(torch.isnan(base), torch.full_like(base, -1e5), base)
    logits = base[None].repeat(n, 1)
    temps = torch.tensor([0.0 if i % 6 == 5 else (0.7 if i % 2 else 1.3) for i in range(n)])
    top_k = torch.tensor([1 if i % 12 == 0 else (-1 if i % 3 else vocab) for i in range(n)], dtype=torch.int32)
    f = lambda v, dt: torch.full((n,), v, dtype=dt, device=gpu)
    args = (logits.to(gpu), temps.to(gpu), top_k.to(gpu), f(1.0, torch.float32), f(0.0, torch.float32),
            f(9, torch.int64), torch.arange(n, dtype=torch.int32, device=gpu))
    tok, lp = ops.sample(*args, unfiltered=True)
    tok1, lp1 = ops.sample(*args)
    agree = 0
    for i in range(n):
        greedy = float(temps[i]) == 0.0 or int(top_k[i]) == 1
        params = {"temperature": 0.0 if greedy else float(temps[i]), "seed": 9}
        t, logprob, margin = P.sample_token(clean, params, i)
        if greedy or margin > 2e-5:
            assert int(tok[i]) == t == int(tok1[i]), f"row {i}: many blocks {int(tok[i])}, one block {int(tok1[i])}, plain {t}"
            assert abs(float(lp[i]) - logprob) < 2e-4 and abs(float(lp[i]) - float(lp1[i])) < 2e-4
            agree += 1
    assert agree > 0.6 * n  # with 128 k tokens many a draw lies within rounding of an edge


def test_sample_rows_that_hold_nothing(gpu):
    """A row of nothing but -inf (no distribution at all) and a row of nothing but NaN
    (uniform, by the NaN rule): every way of sampling still returns a token of the vocabulary."""
    vocab = 1000
    logits = torch.full((4, vocab), float("-inf"))
    logits[1] = float("nan")
    logits[2] = rnd(1, vocab, seed=3)[0]
    logits[3, 1:] = float("-inf")
    logits[3, 0] = 0.5
    for kw in ({"temperature": 0.0}, {}, {"top_k": 5}, {"top_p": 0.5}, {"min_p": 0.2}):
        for spread in (False, True):
            tok, _ = _sample(gpu, logits, spread=spread, **kw)
            assert all(0 <= int(t) < vocab for t in tok), (kw, spread, tok.tolist())
            assert int(tok[3]) == 0
        n = logits.shape[0]
        f = lambda v, dt: torch.full((n,), v, dtype=dt, device=gpu)
        tok, _ = ops.sample(logits.to(gpu), f(kw.get("temperature", 1.0), torch.float32), f(-1, torch.int32),
                            f(1.0, torch.float32), f(0.0, torch.float32), f(7, torch.int64), f(0, torch.int32),
                            unfiltered=True, all_greedy=kw.get("temperature") == 0.0)
        assert all(0 <= int(t) < vocab for t in tok) and int(tok[3]) == 0


def test_sample_logprob_of_a_row_that_starts_with_minus_infinity(gpu):
    """-inf logits seen before any finite one (a thread's first logit is -inf, a later one
    of the same thread is finite): the sum of the exponentials stays finite and the
    log-probability is the plain softmax's, in the one-block kernel and in the spread ones."""
    vocab = 6000
    logits = torch.full((3, vocab), float("-inf"))
    logits[0, 4096] = 1.0  # thread 0 sees index 0 (-inf) first, then this one
    logits[0, 5000] = 2.0
    logits[1, :7] = float("-inf")
    logits[1, 7:] = rnd(1, vocab - 7, seed=9)[0]
    logits[2] = rnd(1, vocab, seed=10)[0]
    logits[2, ::2] = float("-inf")
    ref = torch.log_softmax(logits.double(), dim=-1)
    for kw in ({"temperature": 0.0}, {}, {"top_k": 50}):
        for spread in (False, True):
            tok, lp = (t.cpu() for t in _sample(gpu, logits, spread=spread, **kw))
            assert torch.isfinite(lp).all(), (kw, spread, lp.tolist())
            if kw.get("temperature") == 0.0:
                assert tok.tolist() == ref.argmax(-1).tolist()
            if "top_k" not in kw:
                want = ref.gather(1, tok.long()[:, None])[:, 0]
                assert torch.allclose(lp.double(), want, atol=1e-4), (kw, spread)


def test_sample_rows_are_independent(gpu):
    logits = rnd(8, 331, seed=82, scale=2.0)
    temp = torch.tensor([0.0, 1.0, 0.5, 2.0, 1.0, 0.0, 1.0, 0.7])
    topk = torch.tensor([-1, -1, 10, -1, 1, -1, 50, -1], dtype=torch.int32)
    seeds = torch.arange(8, dtype=torch.int64) * 1000 + 3
    draw = torch.tensor([0, 5, 2, 9, 1, 0, 7, 3], dtype=torch.int32)
    tok, lp = _sample(gpu, logits, temperature=temp, top_k=topk, seed=seeds, draw=draw)
    for r in range(8):  # the same row alone gives the same token
        t1, l1 = _sample(gpu, logits[r : r + 1], temperature=temp[r : r + 1], top_k=topk[r : r + 1],
                         seed=seeds[r : r + 1], draw=draw[r : r + 1])
        assert int(t1[0]) == int(tok[r]) and abs(float(l1[0]) - float(lp[r])) < 1e-6
