"""Each HIP kernel alone against a plain float64 torch reference of the same operation, at
sizes other than the engine tests use (widths and vocabularies that are no power of two,
head sizes 32..256, group sizes 1..8, page sizes 8..64, shuffled page order)."""
import random

import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"


def ops():
    from dinfer_amd.kernels import ops as o
    return o


def tol(dtype):
    # bf16: one rounding of the result (2^-8 relative) plus input rounding noise
    return dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=1e-5, atol=1e-5)


DTYPES = [torch.float32, torch.bfloat16]


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(dtype):
    V, W = 1000, 200  # rows of 400 / 800 bytes: vector path for both dtypes; plus an odd width below
    for width in (W, 201):
        table = torch.randn(V, width, device=DEV).to(dtype)
        ids = torch.randint(0, V, (17,), device=DEV, dtype=torch.int32)
        out = torch.empty(17, width, device=DEV, dtype=dtype)
        ops().embedding(ids, table, out)
        assert torch.equal(out, table[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [1536, 100, 4096, 5120, 20000])
def test_rmsnorm(dtype, width):
    T, eps = 13, 1e-5
    x = (torch.randn(T, width, device=DEV) * 2).to(dtype)
    res = torch.randn(T, width, device=DEV).to(dtype)
    w = (torch.rand(width, device=DEV) + 0.5).to(dtype)
    out = torch.empty(T, width, device=DEV, dtype=dtype)
    ops().rmsnorm(x, w, out, eps, T)
    want = plain.rms_norm(x.double(), w.double(), eps)
    torch.testing.assert_close(out.double(), want, **tol(dtype))
    # fused add: the residual is rounded first, and the rounded sum is normed
    res2 = res.clone()
    ops().rmsnorm(x, w, out, eps, T, residual=res2)
    summed = (x.float() + res.float()).to(dtype)
    assert torch.equal(res2, summed)
    torch.testing.assert_close(out.double(), plain.rms_norm(summed.double(), w.double(), eps), **tol(dtype))
    # gather, with a gain stored in 32-bit and an offset of 1
    rows = torch.tensor([12, 0, 5], device=DEV, dtype=torch.int32)
    out3 = torch.empty(3, width, device=DEV, dtype=dtype)
    ops().rmsnorm(x, w.float(), out3, eps, 3, rows=rows, weight_offset=1.0)
    torch.testing.assert_close(out3.double(), plain.rms_norm(x[rows.long()].double(), w.double() + 1.0, eps), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_act(dtype):
    for T, I in ((11, 2048), (3, 136), (5, 12288)):
        x = torch.randn(T, 2 * I, device=DEV).to(dtype)
        out = torch.empty(T, I, device=DEV, dtype=dtype)
        ops().gated_act(x, out, T)
        want = plain.silu(x[:, :I].double()) * x[:, I:].double()
        torch.testing.assert_close(out.double(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_ref(dtype):
    for M, N, K in ((33, 96, 512), (1, 331, 80), (70, 100, 37)):
        a = torch.randn(M, K, device=DEV).to(dtype)
        w = (torch.randn(N, K, device=DEV) * 0.05).to(dtype)
        out = torch.empty(M, N, device=DEV, dtype=dtype)
        ops().gemm_ref(a, w, out, M)
        want = a.double() @ w.double().T
        torch.testing.assert_close(out.double(), want, **tol(dtype))
        out32 = torch.empty(M, N, device=DEV, dtype=torch.float32)
        ops().gemm_ref(a, w, out32, M)
        torch.testing.assert_close(out32.double(), want, rtol=1e-5, atol=1e-5)


# ---- qkv_post: per-head norm, rotation, cache write -----------------------------------------------
def rope_table(max_pos, rd, theta):
    ang = plain.rope_angles(list(range(max_pos)), rd, theta)
    return torch.cat([ang.cos(), ang.sin()], dim=1).float()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,D,page", [(16, 8, 128, 16), (6, 2, 48, 4), (5, 5, 80, 8), (4, 1, 256, 32), (7, 1, 64, 8),
                                         (3, 3, 320, 8)])
def test_qkv_post(dtype, H, Hkv, D, page):
    T, theta, eps, nblocks = 6, 1e6, 1e-6, 4
    width = (H + 2 * Hkv) * D
    qkv_in = torch.randn(T, width, device=DEV).to(dtype)
    wq = (torch.rand(D, device=DEV) + 0.5).to(dtype)
    wk = (torch.rand(D, device=DEV) + 0.5).to(dtype)
    pos = torch.tensor([0, 3, 7, 15, 31, 100], device=DEV, dtype=torch.int32)
    slots = torch.tensor([0, 1, 2, page + 1, page + 2, -1], device=DEV, dtype=torch.int64)  # the last token is not cached
    table = rope_table(128, D, theta).to(DEV)
    kc = torch.zeros(ops().k_cache_shape(nblocks, Hkv, page, D), device=DEV, dtype=dtype)
    vc = torch.zeros(nblocks, Hkv, D, page, device=DEV, dtype=dtype)
    qkv = qkv_in.clone()
    ops().qkv_post(qkv, T, heads=H, kv_heads=Hkv, head_dim=D, q_off=0, k_off=H * D, v_off=(H + Hkv) * D, q_gain=wq,
                   k_gain=wk, eps=eps, gain_offset=0.0, positions=pos, cos_sin=table, rotary_dim=D, rope_style=0,
                   k_cache=kc, v_cache=vc, slot_mapping=slots, page_size=page)
    x = qkv_in.double().cpu()
    ang = plain.rope_angles(pos.tolist(), D, theta)
    q = plain.rope_neox(plain.rms_norm(x[:, :H * D].view(T, H, D), wq.double().cpu(), eps), ang)
    k = plain.rope_neox(plain.rms_norm(x[:, H * D:(H + Hkv) * D].view(T, Hkv, D), wk.double().cpu(), eps), ang)
    v = x[:, (H + Hkv) * D:].view(T, Hkv, D)
    torch.testing.assert_close(qkv[:, :H * D].double().cpu().view(T, H, D), q, **tol(dtype))
    want_k = torch.zeros(nblocks, Hkv, page, D, dtype=torch.float64)
    want_v = torch.zeros(nblocks, Hkv, D, page, dtype=torch.float64)
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            want_k[s // page, :, s % page, :] = k[t]
            want_v[s // page, :, :, s % page] = v[t]
    torch.testing.assert_close(ops().k_cache_rows(kc).double().cpu(), want_k, **tol(dtype))
    assert torch.equal(vc.double().cpu(), want_v)  # v is copied, not computed


def test_qkv_post_partial_and_interleaved_rotation():
    """rotary_dim smaller than the head, interleaved pairs, no norm: parameters, not constants."""
    T, H, Hkv, D, RD, theta = 4, 2, 1, 64, 32, 1e4
    qkv_in = torch.randn(T, (H + 2 * Hkv) * D, device=DEV)
    pos = torch.tensor([5, 0, 9, 77], device=DEV, dtype=torch.int32)
    table = rope_table(128, RD, theta).to(DEV)
    for style in (0, 1):
        qkv = qkv_in.clone()
        ops().qkv_post(qkv, T, heads=H, kv_heads=Hkv, head_dim=D, q_off=0, k_off=H * D, v_off=(H + Hkv) * D,
                       q_gain=None, k_gain=None, eps=0.0, gain_offset=0.0, positions=pos, cos_sin=table, rotary_dim=RD,
                       rope_style=style, k_cache=None, v_cache=None, slot_mapping=None, page_size=8)
        x = qkv_in[:, :H * D].double().cpu().view(T, H, D)
        ang = plain.rope_angles(pos.tolist(), RD, theta)
        want = x.clone()
        if style == 0:
            want[..., :RD] = plain.rope_neox(x[..., :RD], ang)
        else:
            a, b = x[..., 0:RD:2], x[..., 1:RD:2]
            c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
            want[..., 0:RD:2], want[..., 1:RD:2] = a * c - b * s, b * c + a * s
        torch.testing.assert_close(qkv[:, :H * D].double().cpu().view(T, H, D), want, rtol=1e-5, atol=1e-5)


# ---- attention ------------------------------------------------------------------------------------
def paged_case(dtype, H, Hkv, D, page, hist, new, seed=0, spike=None, sharp=1.0):
    """Requests with `hist` cached tokens and `new` rows each; pages in shuffled order.
    Returns q [T, H*D], caches, metadata tensors and the expected output [T, H, D] in float64.
    sharp: the queries are that much larger, so that among thousands of keys a few, anywhere, carry a row's softmax
    (the mean of thousands of random values is as small as the tolerance, whatever keys went into it)."""
    g = torch.Generator().manual_seed(seed)
    B = len(hist)
    total = [h + n for h, n in zip(hist, new)]
    max_blocks = max(-(-t // page) for t in total) + 1
    nblocks = sum(-(-t // page) for t in total) + 3
    order = list(range(nblocks))
    random.Random(seed).shuffle(order)
    kc = torch.randn(nblocks, Hkv, page, D, generator=g).to(dtype)  # stale content everywhere
    vc = torch.randn(nblocks, Hkv, D, page, generator=g).to(dtype)
    bt = torch.full((B, max_blocks), -1, dtype=torch.int32)
    qs, outs = [], []
    for b in range(B):
        k = torch.randn(total[b], Hkv, D, generator=g).to(dtype)
        v = torch.randn(total[b], Hkv, D, generator=g).to(dtype)
        q = (torch.randn(new[b], H, D, generator=g) * sharp).to(dtype)
        sp = spike.get(b) if isinstance(spike, dict) else spike   # one for all requests, or {request: (key, amp)}
        if sp is not None and total[b] > sp[0] and new[b] > 0:
            # one far key that must win: scale a query and that key so that one score stands out
            key, amp = sp
            k[key] = k[key] * 0 + q[-1, ::H // Hkv][:, :].float().to(dtype) * amp
        for i in range(-(-total[b] // page)):
            blk = order.pop()
            bt[b, i] = blk
            n = min(page, total[b] - i * page)
            kc[blk, :, :n] = k[i * page:i * page + n].transpose(0, 1)
            vc[blk, :, :, :n] = v[i * page:i * page + n].permute(1, 2, 0)
        qs.append(q)
        outs.append((q.double(), k.double(), v.double()))
    cu = torch.tensor([0] + list(torch.tensor(new).cumsum(0)), dtype=torch.int32)
    meta = dict(bt=bt.to(DEV), cu=cu.to(DEV), sl=torch.tensor(total, dtype=torch.int32, device=DEV))
    q_all = torch.cat(qs).reshape(sum(new), H * D).to(DEV)
    return q_all, ops().k_cache_pack(kc).to(DEV), vc.to(DEV), meta, outs


def expected_attention(outs, hist, scale, window, device="cpu"):
    """float64 softmax attention of every request, rows [sum of new, H, D] on the CPU (device: where it is computed;
    thousands of rows against thousands of keys take the CPU minutes)."""
    res = []
    for (q, k, v), h in zip(outs, hist):
        q, k, v = q.to(device), k.to(device), v.to(device)
        Tq, H, D = q.shape
        G = H // k.shape[1]
        o = torch.zeros_like(q)
        pos = h + torch.arange(Tq, device=device)[:, None]
        j = torch.arange(k.shape[0], device=device)[None, :]
        hidden = j > pos
        if window:
            hidden = hidden | (j <= pos - window)
        for hh in range(H):
            s = (q[:, hh] @ k[:, hh // G].T) * scale
            s = s.masked_fill(hidden, float("-inf"))
            o[:, hh] = torch.softmax(s, -1) @ v[:, hh // G]
        res.append(o.cpu())
    return torch.cat(res)


GEOS = [(4, 2, 32, 8), (16, 8, 128, 16), (6, 2, 48, 8), (5, 1, 64, 64), (8, 8, 96, 24), (16, 2, 256, 16)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [0, 40])
def test_attention_plain_kernel(dtype, window):
    H, Hkv, D, page = 6, 2, 40, 4  # a head size the MFMA kernels do not take
    hist, new = [11, 0, 70, 6], [3, 17, 1, 1]
    q, kc, vc, m, outs = paged_case(dtype, H, Hkv, D, page, hist, new)
    out = torch.empty(sum(new), H * D, device=DEV, dtype=dtype)
    ops().attn_paged_ref(q, out, kc, vc, m["bt"], m["cu"], m["sl"], len(hist), sum(new), scale=D ** -0.5,
                         window=window, heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    want = expected_attention(outs, hist, D ** -0.5, window)
    torch.testing.assert_close(out.double().cpu().view(-1, H, D), want, **tol(dtype))


@pytest.mark.parametrize("window", [0, 50])
@pytest.mark.parametrize("H,Hkv,D,page", GEOS)
def test_attention_flash(H, Hkv, D, page, window):
    # prompts without history (70 / 33 / 5: several tiles, ragged tail, idle waves), portions with
    # history that ends inside a page, single rows, and a long run that needs the two-tile kernel
    hist, new = [0, 0, 0, 40, 70, 300, 129, 7], [70, 33, 5, 5, 1, 1, 150, 64]
    q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, new, seed=3)
    out = torch.zeros(sum(new), H * D, device=DEV, dtype=torch.bfloat16)
    ops().attn_flash(q, out, kc, vc, m["bt"], m["cu"], m["sl"], len(hist), sum(new), max(new), scale=D ** -0.5,
                     window=window, heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    want = expected_attention(outs, hist, D ** -0.5, window)
    torch.testing.assert_close(out.double().cpu().view(-1, H, D), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("window", [0, 100])
@pytest.mark.parametrize("H,Hkv,D,page", GEOS)
def test_attention_decode_split_k(H, Hkv, D, page, window):
    # 300 / 70 / 1: several splits, a short one, a single key; then 1..64 at batch 32
    for hist, splits in (([299, 69, 0, 1000], 7), ([random.Random(7).randrange(64) for _ in range(32)], 2),
                         ([5000, 31, 32], 64), ([100, 200], 1),
                         # up to four parts meet inside the workgroup (no merge kernel): with empty parts, a single key
                         ([0, 45, 1000, 130], 4), ([70, 2, 500, 33, 64], 3)):
        new = [1] * len(hist)
        q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, new, seed=5)
        out = torch.zeros(len(hist), H * D, device=DEV, dtype=torch.bfloat16)
        part = torch.full((len(hist) * H * splits * (D + 4),), float("nan"), device=DEV)  # empty parts stay NaN
        ops().attn_decode(q, out, part, kc, vc, m["bt"], None, m["sl"], len(hist), splits, scale=D ** -0.5,
                          window=window, heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
        want = expected_attention(outs, hist, D ** -0.5, window)
        torch.testing.assert_close(out.double().cpu().view(-1, H, D), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("gains", ["bf16", "none"])
@pytest.mark.parametrize("window", [0, 100])
@pytest.mark.parametrize("H,Hkv,D,page", [(16, 8, 128, 16), (5, 1, 64, 64), (16, 2, 256, 16), (8, 8, 64, 24)])
def test_attention_decode_takes_norm_rotation_and_cache_write_along(H, Hkv, D, page, window, gains):
    """A step of single rows straight from the q|k|v product: one kernel norms and rotates q and the new key, writes
    key and value into their pages and attends. Against the plain functions, and against the two kernels it stands for
    (whose page contents it must reproduce bit for bit). The slot of the new key holds stale content beforehand; one
    request writes nothing (slot -1: its pages hold the key already)."""
    # parts of several blocks, a part of one block (the store is waited for at once), a single key, many short ones
    rng = random.Random(3)
    for hist, splits in (([299, 69, 0, 1000], 7), ([rng.randrange(64) for _ in range(32)], 2),
                         ([0, 45, 1000, 130], 4), ([100, 31, 32, 33], 1),
                         # 32 requests and more (the new key is dealt with inside the walk) with parts that a merge
                         # kernel combines: parts of one and two blocks, then of three to five
                         ([rng.randrange(200) for _ in range(33)], 6), ([300 + rng.randrange(400) for _ in range(34)], 5)):
        decode_post_case(H, Hkv, D, page, window, gains, hist, splits)


def decode_post_case(H, Hkv, D, page, window, gains, hist, splits, device="cpu", spike=None, sharp=1.0):
    """One launch of the decode kernel that norms, rotates and writes the cache, against the plain functions and, bit
    for bit, against the two kernels it stands for. Request 1 writes nothing (slot -1)."""
    theta, eps, scale = 1e4, 1e-5, D ** -0.5
    B = len(hist)
    _, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, [1] * B, seed=11)
    g = torch.Generator().manual_seed(B)
    raw = torch.randn(B, (H + 2 * Hkv) * D, generator=g).to(torch.bfloat16)
    wq = wk = None
    if gains != "none":
        wq = ((torch.rand(D, generator=g) + 0.5) * sharp).to(torch.bfloat16)   # (a norm undoes any scale of q itself)
        wk = (torch.rand(D, generator=g) + 0.5).to(torch.bfloat16)
    else:
        raw[:, :H * D] = (raw[:, :H * D].float() * sharp).to(torch.bfloat16)
    pos = [h for h in hist]
    table = rope_table(max(hist) + 25, D, theta).to(DEV)
    slots = []
    for b in range(B):
        blk = int(m["bt"][b, hist[b] // page])
        slots.append(blk * page + hist[b] % page)
    slots[1] = -1
    # what the plain functions make of the rows
    x = raw.double()
    ang = plain.rope_angles(pos, D, theta)
    norm = (lambda t, w: plain.rms_norm(t, w.double(), eps)) if wq is not None else (lambda t, w: t)
    q = plain.rope_neox(norm(x[:, :H * D].view(B, H, D), wq), ang).to(torch.bfloat16).double()
    k = plain.rope_neox(norm(x[:, H * D:(H + Hkv) * D].view(B, Hkv, D), wk), ang).to(torch.bfloat16).double()
    v = x[:, (H + Hkv) * D:].view(B, Hkv, D)
    want_outs = []
    for b, (_, kk, vv) in enumerate(outs):
        kk, vv = kk.clone(), vv.clone()
        if slots[b] >= 0:
            kk[-1], vv[-1] = k[b], v[b]
        sp = spike.get(b) if isinstance(spike, dict) else spike
        if sp is not None:   # a cached key along the row's first query head of each group, as it is after norm and rotation
            key, amp = sp
            kk[key] = (q[b, ::H // Hkv] * amp).to(torch.bfloat16).double()
            blk, off = int(m["bt"][b, key // page]), key % page
            kc[blk, :, :, off, :] = kk[key].to(torch.bfloat16).view(Hkv, D // 8, 8).to(DEV)
        want_outs.append((q[b:b + 1], kk, vv))
    want = expected_attention(want_outs, hist, scale, window, device)
    dev = lambda t: None if t is None else t.to(DEV)
    args = dict(heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    post = dict(q_off=0, k_off=H * D, v_off=(H + Hkv) * D, q_gain=dev(wq), k_gain=dev(wk), eps=eps, gain_offset=0.0,
                positions=torch.tensor(pos, dtype=torch.int32, device=DEV))
    slot_t = torch.tensor(slots, dtype=torch.int64, device=DEV)
    part = torch.full((B * H * splits * (D + 4),), float("nan"), device=DEV)
    # the two kernels
    kc2, vc2, qkv2 = kc.clone(), vc.clone(), raw.to(DEV)
    out2 = torch.zeros(B, H * D, device=DEV, dtype=torch.bfloat16)
    ops().qkv_post(qkv2, B, **args, **post, cos_sin=table, rotary_dim=D, rope_style=0, k_cache=kc2, v_cache=vc2,
                   slot_mapping=slot_t, token_runs=False)
    ops().attn_decode(qkv2, out2, part, kc2, vc2, m["bt"], None, m["sl"], B, splits, scale=scale, window=window,
                      **args)
    # the one
    kc1, vc1, qkv1 = kc.clone(), vc.clone(), raw.to(DEV)
    out1 = torch.zeros(B, H * D, device=DEV, dtype=torch.bfloat16)
    part.fill_(float("nan"))
    ops().attn_decode_post(qkv1, out1, part, kc1, vc1, m["bt"], m["sl"], B, splits, scale=scale, window=window,
                           **args, **post, cos_sin=table, slot_mapping=slot_t)
    assert torch.equal(qkv1.cpu(), raw), "the product's rows are left as they were"
    assert torch.equal(vc1, vc2) and torch.equal(kc1, kc2), "the pages hold the same bits as after the two kernels"
    torch.testing.assert_close(out1.double().cpu().view(-1, H, D), want, rtol=2e-2, atol=2e-2)
    assert torch.equal(out1, out2), f"differs from the two kernels by {float((out1.float() - out2.float()).abs().max())}"


@pytest.mark.parametrize("window", [0, 200])
@pytest.mark.parametrize("H,Hkv,D,page", [(8, 2, 128, 16), (5, 5, 64, 8), (6, 1, 128, 24), (4, 2, 256, 16)])
def test_attention_flash_long_portions(H, Hkv, D, page, window):
    """Long portions: a whole prompt of 700, a portion of 300 on top of a history of 333, short requests in
    the same launch (idle waves), and a single row behind 1000 keys."""
    hist, new = [0, 333, 0, 77, 1000], [700, 300, 5, 130, 1]
    q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, new, seed=13)
    out = torch.zeros(sum(new), H * D, device=DEV, dtype=torch.bfloat16)
    ops().attn_flash(q, out, kc, vc, m["bt"], m["cu"], m["sl"], len(hist), sum(new), max(new), scale=D ** -0.5,
                     window=window, heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    want = expected_attention(outs, hist, D ** -0.5, window)
    torch.testing.assert_close(out.double().cpu().view(-1, H, D), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("page", [16, 24])
@pytest.mark.parametrize("window", [0, 300])
def test_attention_flash_three_row_tiles_a_workgroup(window, page):
    """Head size 128 with enough rows for several rounds of workgroups: 48 rows a workgroup (three row tiles share every
    key and value fragment). Rows with and without history, a request that ends inside a tile, one shorter than a tile;
    pages of a power of two and not."""
    H, Hkv, D = 16, 4, 128
    hist, new = [0, 100, 555, 31, 7, 0], [1000, 700, 300, 49, 120, 33]     # ceil(1000 / 48) x 16 heads x 6 requests = 2,016 workgroups
    q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, new, seed=9)
    out = torch.zeros(sum(new), H * D, device=DEV, dtype=torch.bfloat16)
    ops().attn_flash(q, out, kc, vc, m["bt"], m["cu"], m["sl"], len(hist), sum(new), max(new), scale=D ** -0.5,
                     window=window, heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    want = expected_attention(outs, hist, D ** -0.5, window)
    torch.testing.assert_close(out.double().cpu().view(-1, H, D), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("splits", [5, 3])   # parts merged by a kernel of their own, and inside the workgroup
def test_attention_mixed_routes_single_rows_to_split_k(splits):
    H, Hkv, D, page = 16, 4, 128, 16
    hist, new = [500, 0, 64, 900, 33, 10], [1, 40, 1, 1, 20, 1]
    q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, new, seed=9)
    out = torch.zeros(sum(new), H * D, device=DEV, dtype=torch.bfloat16)
    part = torch.zeros(len(hist) * H * splits * (D + 4), device=DEV)
    geo = dict(scale=D ** -0.5, window=0, heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    ops().attn_decode(q, out, part, kc, vc, m["bt"], m["cu"], m["sl"], len(hist), splits, **geo)
    ops().attn_flash(q, out, kc, vc, m["bt"], m["cu"], m["sl"], len(hist), sum(new), max(new), skip_single=True, **geo)
    want = expected_attention(outs, hist, D ** -0.5, 0)
    torch.testing.assert_close(out.double().cpu().view(-1, H, D), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("kernel", ["plain", "flash", "decode"])
def test_attention_finds_one_far_key(kernel):
    """Random scores hide a key that is skipped or read from the wrong slot. Here key 5 of 700 is
    made to dominate the last row's softmax, so the output must be (nearly) that key's value."""
    H, Hkv, D, page = 8, 2, 64, 16
    hist, new = [699], [1]
    q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, new, seed=11, spike=(5, 3.0))
    out = torch.zeros(1, H * D, device=DEV, dtype=torch.bfloat16)
    geo = dict(scale=D ** -0.5, window=0, heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    if kernel == "plain":
        ops().attn_paged_ref(q, out, kc, vc, m["bt"], m["cu"], m["sl"], 1, 1, **geo)
    elif kernel == "flash":
        ops().attn_flash(q, out, kc, vc, m["bt"], m["cu"], m["sl"], 1, 1, 1, **geo)
    else:
        part = torch.zeros(H * 11 * (D + 4), device=DEV)
        ops().attn_decode(q, out, part, kc, vc, m["bt"], None, m["sl"], 1, 11, **geo)
    want = expected_attention(outs, hist, D ** -0.5, 0)
    torch.testing.assert_close(out.double().cpu().view(-1, H, D), want, rtol=2e-2, atol=2e-2)
    # the spiked heads (one per kv head) really are dominated by key 5
    (qq, kk, vv) = outs[0]
    got = out.double().cpu().view(H, D)
    for hk in range(Hkv):
        assert (got[hk * (H // Hkv)] - vv[5, hk]).abs().max() < 0.1


@pytest.mark.parametrize("kernel", ["plain", "flash", "decode"])
@pytest.mark.parametrize("inside", [True, False], ids=["first_key_inside", "last_key_outside"])
def test_attention_window_edge(kernel, inside):
    """A window of W keys ends exactly W - 1 keys before the row: the key at that place is made to dominate the last
    row's softmax and must decide the output; the key one place earlier, made to dominate instead, must not count
    at all (with random scores one key more or less among 150 changes the output by less than the tolerance).
    The edge lies in the middle of a 32-key block and of a page, and the window starts in another split."""
    H, Hkv, D, page, W = 8, 2, 64, 16, 150
    total = 700
    pos = total - 1                                   # the last row's position
    key = pos - W + 1 if inside else pos - W          # first key inside the window / last key outside it
    hist, new = ([total - 1], [1]) if kernel != "flash" else ([total - 40], [40])
    q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, new, seed=21, spike=(key, 3.0))
    out = torch.zeros(new[0], H * D, device=DEV, dtype=torch.bfloat16)
    geo = dict(scale=D ** -0.5, window=W, heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    if kernel == "plain":
        ops().attn_paged_ref(q, out, kc, vc, m["bt"], m["cu"], m["sl"], 1, new[0], **geo)
    elif kernel == "flash":
        ops().attn_flash(q, out, kc, vc, m["bt"], m["cu"], m["sl"], 1, new[0], new[0], **geo)
    else:
        part = torch.zeros(H * 7 * (D + 4), device=DEV)
        ops().attn_decode(q, out, part, kc, vc, m["bt"], None, m["sl"], 1, 7, **geo)
    want = expected_attention(outs, hist, D ** -0.5, W)
    torch.testing.assert_close(out.double().cpu().view(-1, H, D), want, rtol=2e-2, atol=2e-2)
    (qq, kk, vv) = outs[0]
    got = out.double().cpu().view(-1, H, D)[-1]
    for hk in range(Hkv):
        near = (got[hk * (H // Hkv)] - vv[key, hk]).abs().max()
        assert (near < 0.1) == inside, f"kv head {hk}: the spiked key {'does not decide' if inside else 'decides'} the output"


# ---- sampling -------------------------------------------------------------------------------------
def table_refetches(k_lo, k_hi, page):
    """Where a wave that walks the keys [k_lo, k_hi) in blocks of 32 with the block-table entries of 64 pages on board
    takes the next 64: the first key of each block that no longer fits (csrc/attention.hip, Pages::ensure). Used to put
    a spiked key on each side of such a line; if the rule here were wrong the spikes would only sit somewhere else."""
    lines, base = [], (k_lo & ~31) // page
    for kb in range(k_lo & ~31, k_hi, 32):
        if (kb + 31) // page - base >= 64:
            base = kb // page
            lines.append(kb)
    return lines


def decode_parts(seq, window, splits):
    """The parts [lo, hi) a request's visible keys are cut into (csrc/attention.hip, split_range)."""
    first = max(seq - window, 0) if window else 0
    base = first & ~31
    per = (-(-(seq - base) // splits) + 31) & ~31
    parts = [(max(base + s * per, first), min(base + (s + 1) * per, seq)) for s in range(splits)]
    return [(lo, hi) for lo, hi in parts if lo < hi]


LONG_DECODE = [
    # 64 requests of 2,064 keys in two parts each: the parts meet inside a workgroup and the keys are read past the caches
    ([2063] * 64, 2),
    # one part walks the whole request; three parts of 1,376 keys
    ([4095, 2063, 70], 1), ([4095, 2063, 70], 3),
]


@pytest.mark.parametrize("entry", ["plain", "post"])
@pytest.mark.parametrize("side", [0, 1], ids=["spike_before_the_line", "spike_behind_the_line"])
@pytest.mark.parametrize("window", [0, 3000])
@pytest.mark.parametrize("page", [16, 8])
def test_attention_decode_parts_longer_than_64_pages(page, window, side, entry):
    """Contexts of 2,064 and 4,096 keys with so few parts that one wave walks more than 64 pages and takes the next
    block-table entries on the way. Sharp scores: each row's softmax rests on a few keys anywhere in its context; and
    in every request the key just before (or just behind) the first such line of one of its parts decides the row."""
    H, Hkv, D = 8, 2, 128
    for hist, splits in LONG_DECODE:
        B, spikes, with_line = len(hist), {}, 0
        for b, h in enumerate(hist):
            lines = [l for lo, hi in decode_parts(h + 1, window, splits) for l in table_refetches(lo, hi, page)]
            with_line += bool(lines)
            spikes[b] = ((lines[b % len(lines)] if lines else h // 2) - 1 + side, 3.0)
        assert with_line >= 1 or splits == 3, "the case must make waves walk more than 64 pages"
        if entry == "post":
            decode_post_case(H, Hkv, D, page, window, "bf16", hist, splits, device=DEV, spike=spikes, sharp=3.0)
            continue
        q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, [1] * B, seed=17, spike=spikes, sharp=3.0)
        out = torch.zeros(B, H * D, device=DEV, dtype=torch.bfloat16)
        part = torch.full((B * H * splits * (D + 4),), float("nan"), device=DEV)
        ops().attn_decode(q, out, part, kc, vc, m["bt"], None, m["sl"], B, splits, scale=D ** -0.5, window=window,
                          heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
        want = expected_attention(outs, hist, D ** -0.5, window, DEV)
        got = out.double().cpu().view(B, H, D)
        torch.testing.assert_close(got, want, rtol=2e-2, atol=2e-2)
        for b, (_, _, vv) in enumerate(outs):
            for hk in range(Hkv):
                assert (got[b, hk * (H // Hkv)] - vv[spikes[b][0], hk]).abs().max() < 0.1, f"request {b}: the spiked key"


@pytest.mark.parametrize("entry", ["plain", "post"])
@pytest.mark.parametrize("window", [0, 3230])
def test_attention_decode_reads_past_the_caches_from_100_mb_a_step(window, entry):
    """Where a request's visible keys times the number of requests come to 100 MB of keys and values (8 requests of
    3,200 keys of 8 kv heads of 128: 105 MB) a wave of the decode kernel reads them with non-temporal loads; the short
    requests of the same launch take the other walk. Sharp scores, and in every request one key anywhere decides the
    row."""
    H, Hkv, D, page, splits = 16, 8, 128, 16, 16
    hist = [3300, 500, 3210, 64, 3500, 0, 3250, 1000]
    B = len(hist)
    first = lambda h: max(h + 1 - window, 0) if window else 0      # the row stands at position h
    spikes = {b: (first(h) + (h - first(h)) * (b + 1) // (B + 1), 3.0) for b, h in enumerate(hist) if h > 0}
    if entry == "post":
        decode_post_case(H, Hkv, D, page, window, "bf16", hist, splits, device=DEV, spike=spikes, sharp=3.0)
        return
    q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, [1] * B, seed=29, spike=spikes, sharp=3.0)
    out = torch.zeros(B, H * D, device=DEV, dtype=torch.bfloat16)
    part = torch.full((B * H * splits * (D + 4),), float("nan"), device=DEV)
    ops().attn_decode(q, out, part, kc, vc, m["bt"], None, m["sl"], B, splits, scale=D ** -0.5, window=window,
                      heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    want = expected_attention(outs, hist, D ** -0.5, window, DEV)
    got = out.double().cpu().view(B, H, D)
    torch.testing.assert_close(got, want, rtol=2e-2, atol=2e-2)
    for b, (key, _) in spikes.items():
        for hk in range(Hkv):
            assert (got[b, hk * (H // Hkv)] - outs[b][2][key, hk]).abs().max() < 0.1, f"request {b}: the spiked key"


def flash_wave_runs(hist, q_len, window, rows):
    """The runs of keys the four waves of the last workgroup of a request walk (csrc/attention.hip, attn_flash_kernel)."""
    q0 = (q_len - 1) // rows * rows
    lo = max(hist + q0 - window + 1, 0) if window else 0
    hi = hist + q_len
    b0, b1 = lo >> 5, (hi + 31) >> 5
    per = (b1 - b0 + 3) >> 2
    runs = [(max((b0 + w * per) * 32, lo), min((b0 + (w + 1) * per) * 32, hi)) for w in range(4)]
    return [(a, b) for a, b in runs if a < b]


@pytest.mark.parametrize("side", [0, 1], ids=["spike_before_the_line", "spike_behind_the_line"])
@pytest.mark.parametrize("windowed", [False, True])
@pytest.mark.parametrize("page,rows", [(16, 4500), (8, 4500), (24, 6400)])
def test_attention_flash_a_prompt_of_thousands_of_rows(page, rows, windowed, side):
    """One prompt of 4,500 (6,400) rows of 24 heads of 128: 48 rows a workgroup, and the waves of the late row tiles
    walk more than 64 pages each. Sharp scores; the last row's softmax rests on the key beside a wave's refetch line."""
    H, Hkv, D = 24, 4, 128
    window = rows - 300 if windowed else 0
    lines = [l for lo, hi in flash_wave_runs(0, rows, window, 48) for l in table_refetches(lo, hi, page)]
    assert lines, "the case must make a wave walk more than 64 pages"
    key = lines[len(lines) // 2] - 1 + side
    q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, [0], [rows], seed=23, spike=(key, 3.0), sharp=3.0)
    out = torch.zeros(rows, H * D, device=DEV, dtype=torch.bfloat16)
    ops().attn_flash(q, out, kc, vc, m["bt"], m["cu"], m["sl"], 1, rows, rows, scale=D ** -0.5, window=window, heads=H,
                     kv_heads=Hkv, head_dim=D, page_size=page)
    want = expected_attention(outs, [0], D ** -0.5, window, DEV)
    got = out.double().cpu().view(rows, H, D)
    torch.testing.assert_close(got, want, rtol=2e-2, atol=2e-2)
    for hk in range(Hkv):
        assert (got[-1, hk * (H // Hkv)] - outs[0][2][key, hk]).abs().max() < 0.1


@pytest.mark.parametrize("side", [0, 1], ids=["spike_before_the_line", "spike_behind_the_line"])
@pytest.mark.parametrize("window", [0, 4200])
@pytest.mark.parametrize("page", [16, 8])
def test_attention_flash_a_portion_behind_thousands_of_keys(page, window, side):
    """600 rows behind 4,000 keys (32 rows a workgroup: every wave walks 1,150 keys), beside a short request."""
    H, Hkv, D = 8, 2, 128
    hist, new = [4000, 20], [600, 40]
    lines = [l for lo, hi in flash_wave_runs(hist[0], new[0], window, 32) for l in table_refetches(lo, hi, page)]
    assert lines
    key = lines[len(lines) // 2] - 1 + side
    q, kc, vc, m, outs = paged_case(torch.bfloat16, H, Hkv, D, page, hist, new, seed=29, spike={0: (key, 3.0)}, sharp=3.0)
    out = torch.zeros(sum(new), H * D, device=DEV, dtype=torch.bfloat16)
    ops().attn_flash(q, out, kc, vc, m["bt"], m["cu"], m["sl"], 2, sum(new), max(new), scale=D ** -0.5, window=window,
                     heads=H, kv_heads=Hkv, head_dim=D, page_size=page)
    want = expected_attention(outs, hist, D ** -0.5, window, DEV)
    got = out.double().cpu().view(sum(new), H, D)
    torch.testing.assert_close(got, want, rtol=2e-2, atol=2e-2)
    for hk in range(Hkv):
        assert (got[new[0] - 1, hk * (H // Hkv)] - outs[0][2][key, hk]).abs().max() < 0.1


@pytest.mark.parametrize("V", [163841, 16385, 4096 * 4, 1000])
@pytest.mark.parametrize("spread", [False, True])
def test_argmax_ties_to_lowest_index(V, spread):
    """One workgroup a row, and a row spread over many workgroups in two launches (long rows, with scratch): equal
    entries go to the lowest index, also across the pieces; a row of -inf gives 0; rows that start at any alignment."""
    logits = torch.randn(7, V, device=DEV) * 3
    logits[2, 100] = logits[2, V - 7] = 50.0
    logits[3, :] = 1.0
    logits[4, :] = float("-inf")
    logits[5, V - 1] = 60.0                     # in the last, short piece
    logits[6, 4095:4097] = 70.0 if V > 4097 else logits[6, 4095:4097]     # across a piece's edge
    out = torch.full((7,), -1, device=DEV, dtype=torch.int32)
    scratch = ops().argmax_scratch(7, V, DEV) if spread else None
    ops().argmax(logits, out, 7, scratch)
    want = logits.argmax(-1).tolist()
    want[2], want[3], want[4], want[5] = 100, 0, 0, V - 1
    if V > 4097:
        want[6] = 4095
    assert out.tolist() == want
    if spread:      # fewer rows than the scratch was made for, and a view with a row stride of its own
        wide = torch.randn(3, V + 13, device=DEV)
        view = wide[:, 5:5 + V]
        ops().argmax(view, out, 3, scratch)
        assert out[:3].tolist() == view.argmax(-1).tolist()


PATHS = ["one_workgroup", "spread", "spread_forced_generic"]


def draw(logits, temperature, seeds, offsets, path="spread", **kw):
    """path: the kernel with one workgroup a row; the launches that spread a row over many workgroups (what the
    sampler uses); the latter with every row sent down its built-in one-workgroup branch."""
    import numpy as np
    R, V = logits.shape
    out = torch.empty(R, device=DEV, dtype=torch.int32)
    work = torch.empty(R, V, device=DEV)
    f = lambda xs, dt: torch.tensor(xs, device=DEV, dtype=dt)
    if path == "one_workgroup":
        ops().sample(logits, work, out, R, temperature=f(temperature, torch.float32), seeds=f(seeds, torch.int64),
                     offsets=f(offsets, torch.int64),
                     **{k: f(v, torch.int32 if k == "top_k" else torch.float32) for k, v in kw.items()})
        return out.tolist()
    rec = np.zeros(R, dtype=ops().SAMPLE_ROW)
    rec["temperature"], rec["seed"], rec["offset"] = temperature, [x & (2**64 - 1) for x in seeds], offsets
    rec["top_k"], rec["top_p"], rec["min_p"] = kw.get("top_k", -1), kw.get("top_p", 1.0), kw.get("min_p", 0.0)
    packed = torch.from_numpy(rec.view(np.uint8)).to(DEV)
    scratch = torch.empty(ops().sample_scratch_bytes(R, V), dtype=torch.uint8, device=DEV)
    ops().sample_rows(logits, work, scratch, packed, out, R, force_generic=path == "spread_forced_generic")
    return out.tolist()


@pytest.mark.parametrize("path", PATHS)
def test_sample_follows_the_inverse_cdf_rule(path):
    """Each draw must be the token whose interval of the running sum holds u * total, with u from the
    plain Philox. Draws whose target lies within rounding of an interval's edge are not judged."""
    V = 331
    logits = torch.randn(64, V, device=DEV) * 2
    temps = [0.7] * 64
    seeds = [12345 + i for i in range(64)]
    offsets = [i * 3 for i in range(64)]
    got = draw(logits, temps, seeds, offsets, path)
    judged = 0
    for r in range(64):
        tok, slack = plain.sample_row(logits[r].cpu(), temps[r], seeds[r], offsets[r])
        if slack > 1e-5:
            judged += 1
            assert got[r] == tok, f"row {r}: kernel chose {got[r]}, the rule says {tok}"
    assert judged > 55


@pytest.mark.parametrize("path", PATHS)
def test_sample_does_not_depend_on_batch_position(path):
    V = 1000
    row = torch.randn(1, V, device=DEV)
    other = torch.randn(5, V, device=DEV)
    alone = draw(row, [0.9], [777], [4], path)[0]
    batch = torch.cat([other[:3], row, other[3:]])
    mixed = draw(batch, [1.0, 0.0, 0.5, 0.9, 1.3, 0.0], [1, 2, 3, 777, 5, 6], [0, 0, 0, 4, 0, 0], path)
    assert mixed[3] == alone
    assert mixed[1] == int(batch[1].argmax()) and mixed[5] == int(batch[5].argmax())  # greedy rows untouched


@pytest.mark.parametrize("path", PATHS[:2])
def test_sample_frequencies_match_softmax(path):
    """100k draws of one 64-token row at temperature 0.8: L1 distance to softmax below 0.03
    (the reference's statistical test, crates/kernels/tests/ref_tests.rs:225-252)."""
    V, N = 64, 100_000
    row = torch.randn(V, device=DEV) * 2
    counts = torch.zeros(V)
    for chunk in range(N // 1000):
        toks = draw(row.expand(1000, V).contiguous(), [0.8] * 1000, [42] * 1000, list(range(chunk * 1000, chunk * 1000 + 1000)), path)
        counts += torch.bincount(torch.tensor(toks), minlength=V).float()
    want = torch.softmax(row.cpu() / 0.8, -1)
    assert (counts / N - want).abs().sum() < 0.03


@pytest.mark.parametrize("path", PATHS)
def test_sample_candidate_sets(path):
    """min_p, top-k and top-p: every draw falls in the set the plain rule keeps."""
    V = 512
    logits = torch.randn(6, V, device=DEV) * 3
    cases = [dict(top_k=1, top_p=1.0, min_p=0.0), dict(top_k=50, top_p=1.0, min_p=0.0),
             dict(top_k=-1, top_p=0.9, min_p=0.0), dict(top_k=5, top_p=0.5, min_p=0.0),
             dict(top_k=-1, top_p=1.0, min_p=0.2), dict(top_k=40, top_p=0.8, min_p=0.05)]
    for r, c in enumerate(cases):
        keep = plain.candidate_mask(logits[r].cpu().double() / 0.9, **c)
        seen = set()
        for off in range(0, 200, 50):
            toks = draw(logits[r].expand(50, V).contiguous(), [0.9] * 50, [9] * 50, list(range(off, off + 50)), path,
                        top_k=[c["top_k"]] * 50, top_p=[c["top_p"]] * 50, min_p=[c["min_p"]] * 50)
            seen |= set(toks)
        outside = [t for t in seen if not keep[t]]
        # a token on the very edge of top-p may fall either way in 32-bit; allow the reference's margin
        assert len(outside) <= max(2, int(0.001 * keep.sum())), f"case {c}: drew {outside} outside the kept set"
        if c["top_k"] == 1:
            assert seen == {int(logits[r].argmax())}


def test_sample_spread_over_workgroups_at_a_large_vocabulary():
    """At a vocabulary of many segments (and no multiple of one): peaked rows, whose top-k / top-p sets are short
    lists, and a flat row whose nucleus is too wide for a list and takes the built-in one-workgroup branch.
    Every option alone and together; each judged draw is the plain rule's token."""
    V = 151936 + 3
    g = torch.Generator().manual_seed(5)
    base = torch.randn(V, generator=g) * 2.0
    peaked = base.clone()
    peaked[torch.randperm(V, generator=g)[:40]] += torch.rand(40, generator=g) * 6 + 6     # a few dozen likely tokens
    flat = base * 0.2
    cases = [dict(), dict(min_p=0.02), dict(top_k=1), dict(top_k=20), dict(top_k=3000), dict(top_p=0.9), dict(top_p=0.3),
             dict(top_k=50, top_p=0.95), dict(top_k=50, top_p=0.9, min_p=0.01), dict(top_k=V - 1), dict(top_p=0.999)]
    rows, opts = [], []
    for i, c in enumerate(cases):
        for src in (peaked, flat):
            rows.append(src)
            opts.append({**dict(top_k=-1, top_p=1.0, min_p=0.0), **c})
    logits = torch.stack(rows).to(DEV)
    R = len(rows)
    seeds, offsets, temps = [100 + i for i in range(R)], [i % 7 for i in range(R)], [0.8] * R
    kw = {k: [o[k] for o in opts] for k in ("top_k", "top_p", "min_p")}
    got = draw(logits, temps, seeds, offsets, "spread", **kw)
    slow = draw(logits, temps, seeds, offsets, "one_workgroup", **kw)
    judged = 0
    for r in range(R):
        tok, slack = plain.sample_row(logits[r].cpu(), temps[r], seeds[r], offsets[r], **opts[r])
        keep = plain.candidate_mask(logits[r].cpu().double() / temps[r], **opts[r])
        assert keep[got[r]], f"row {r} {opts[r]}: drew {got[r]} outside the kept set"
        if slack > 1e-5:
            judged += 1
            assert got[r] == tok, f"row {r} {opts[r]}: drew {got[r]}, the rule says {tok} (one workgroup: {slow[r]})"
        else:
            # an interval narrower than 32-bit sums resolve (a flat row: 1 / V each): the target must lie
            # within rounding of the drawn token's interval
            z = logits[r].cpu().double() / temps[r]
            pr = torch.where(keep, torch.exp(z - z[keep].max()), torch.zeros_like(z))
            cum = pr.cumsum(-1)
            target = plain.uniform(seeds[r], offsets[r]) * float(cum[-1])
            lo, hi = float(cum[got[r]] - pr[got[r]]), float(cum[got[r]])
            assert max(lo - target, target - hi, 0.0) < 2e-5 * float(cum[-1]), f"row {r} {opts[r]}: drew {got[r]}, rule {tok}"
    assert judged >= R // 2


def test_sample_paths_agree_on_random_options():
    """The spread launches against the one-workgroup kernel over random rows and options: the same token, but for
    the few draws whose target lies within rounding of an interval's edge (the sums are taken in another order)."""
    V, R = 40000 + 17, 96
    rng = random.Random(8)
    logits = (torch.randn(R, V) * torch.tensor([rng.choice([0.3, 1.0, 3.0, 6.0]) for _ in range(R)])[:, None]).to(DEV)
    logits[5, 100:200] = float("-inf")
    logits[6, :] = 1.5                                                     # all equal: every filter keeps all ties
    temps = [rng.choice([0.0, 0.3, 0.8, 1.0, 1.7]) for _ in range(R)]
    kw = dict(top_k=[rng.choice([-1, -1, 1, 7, 64, 1000, 30000]) for _ in range(R)],
              top_p=[rng.choice([1.0, 1.0, 0.95, 0.7, 0.1]) for _ in range(R)],
              min_p=[rng.choice([0.0, 0.0, 0.05, 0.3]) for _ in range(R)])
    seeds, offsets = [rng.getrandbits(64) - (1 << 63) for _ in range(R)], [rng.randrange(500) for _ in range(R)]
    a = draw(logits, temps, seeds, offsets, "one_workgroup", **kw)
    b = draw(logits, temps, seeds, offsets, "spread", **kw)
    c = draw(logits, temps, seeds, offsets, "spread_forced_generic", **kw)
    assert a == c
    differ = [r for r in range(R) if a[r] != b[r]]
    assert len(differ) <= 2, [(r, a[r], b[r], temps[r], {k: v[r] for k, v in kw.items()}) for r in differ]


def test_sample_paths_agree_at_the_edges_of_the_options():
    """Very cold and very hot rows, a nucleus of almost nothing, min_p of 1, top-k of 1 on a tie, rows of equal
    logits and rows that are -inf but for one entry: the spread launches give the one-workgroup kernel's token."""
    V = 20011
    g = torch.Generator().manual_seed(21)
    base = torch.randn(V, generator=g) * 4
    tie = base.clone()
    tie[[17, 4000, 19999]] = base.max() + 1.0                  # three equal maxima
    lonely = torch.full((V,), float("-inf"))
    lonely[12345] = 0.3
    flat = torch.zeros(V)
    cases = [(base, 1e-4, {}), (base, 50.0, {}), (base, 1.0, dict(top_p=1e-6)), (base, 1.0, dict(min_p=1.0)),
             (tie, 1.0, dict(top_k=1)), (tie, 0.7, dict(top_p=1e-6)), (tie, 0.7, dict(min_p=1.0)), (flat, 1.0, dict(top_k=5)),
             (flat, 1.0, dict(top_p=0.5)), (lonely, 1.0, {}), (lonely, 0.5, dict(top_k=3, top_p=0.9, min_p=0.1)),
             (base, 1e-4, dict(top_k=40, top_p=0.9)), (base, 50.0, dict(top_k=V - 1, top_p=0.99999))]
    logits = torch.stack([c[0] for c in cases]).to(DEV)
    temps = [c[1] for c in cases]
    kw = {k: [c[2].get(k, d) for c in cases] for k, d in (("top_k", -1), ("top_p", 1.0), ("min_p", 0.0))}
    for seed in (1, 2, 3):
        seeds, offsets = [seed * 100 + i for i in range(len(cases))], [seed] * len(cases)
        a = draw(logits, temps, seeds, offsets, "one_workgroup", **kw)
        b = draw(logits, temps, seeds, offsets, "spread", **kw)
        differ = [(i, a[i], b[i]) for i in range(len(cases)) if a[i] != b[i]]
        # the hot rows and the flat ones have intervals of 1 / V: a target within rounding of an edge may fall either way
        assert all(i in (1, 7, 8, 12) for i, _, _ in differ) and len(differ) <= 2, differ
        assert b[4] in (17, 4000, 19999) and b[5] in (17, 4000, 19999) and b[6] in (17, 4000, 19999)
        assert b[9] == 12345 and b[10] == 12345 and b[0] == int(base.argmax()) and b[3] == int(base.argmax())


def test_penalties_match_plain_rule():
    import numpy as np
    V = 512
    logits = torch.randn(5, V, device=DEV) * 3
    hist = [([1, 5, 9, 5], [9, 9, 20]), ([3], []), ([7, 7, 7], [7, 100]), ([], [2, 4, 6, 4]), ([8], [8])]
    rep, freq, pres = [1.5, 1.0, 1.2, 1.0, 2.0], [0.0, 0.0, 0.3, 0.5, 1.0], [0.0, 0.0, 0.2, 0.1, 0.5]
    slots = [2, 0, 3, 1, -1]                                # the last row takes no penalties at all
    history = torch.zeros(4, V, dtype=torch.int32, device=DEV)
    entries = [(s, t, 0) for s, (p, _) in zip(slots, hist) if s >= 0 for t in set(p)]
    entries += [(s, t, 1) for s, (_, o) in zip(slots, hist) if s >= 0 for t in o]
    ops().history_add(history, torch.tensor(entries, dtype=torch.int32, device=DEV))
    pen = np.array(list(zip(slots, rep, freq, pres)), dtype=ops().PENALTY_ROW)
    got = logits.clone()
    ops().penalties_dense(got, 5, history, torch.from_numpy(pen.view(np.uint8)).to(DEV))
    for r, (p, o) in enumerate(hist):
        want = logits[r].cpu().double() if slots[r] < 0 else plain.apply_penalties(logits[r].cpu().double(), p, o, rep[r], freq[r], pres[r])
        torch.testing.assert_close(got[r].cpu().double(), want, rtol=1e-6, atol=1e-6)


def test_penalties_from_a_history_on_the_device():
    """The sampler keeps what each request has seen on the device and sends only what is new: requests come, take
    steps in changing company, end, and their slots are used again; every step's penalised logits are the plain
    rule's over the request's whole prompt and outputs."""
    from dinfer_amd.sampling.params import SamplingParams
    from dinfer_amd.sampling.sampler import Sampler
    V = 331
    rng = random.Random(2)
    s = Sampler(DEV, 3, V)
    sp = {"a": SamplingParams(temperature=0.0, repetition_penalty=1.4),
          "b": SamplingParams(temperature=0.0, frequency_penalty=0.6, presence_penalty=0.3),
          "c": SamplingParams(temperature=0.0),                                    # no penalties: no slot
          "d": SamplingParams(temperature=0.0, repetition_penalty=0.8, frequency_penalty=0.2, presence_penalty=1.0),
          "e": SamplingParams(temperature=0.0, presence_penalty=2.0)}
    prompts = {k: [rng.randrange(V) for _ in range(rng.randint(1, 60))] for k in sp}
    outputs = {k: [] for k in sp}
    plan = [["a"], ["a", "b"], ["b", "c", "a"], ["d", "a", "b"], ["d"], ["e", "d", "c"], ["e", "d", "b"]]
    ends = {3: ["a"], 4: ["b"], 6: ["e"]}      # after step 3 a is over (then d and e need its slot) ...
    for step, live in enumerate(plan):
        if step == 6:                         # ... and b comes back under its old name as a new request
            prompts["b"], outputs["b"] = [rng.randrange(V) for _ in range(9)], []
        logits = torch.randn(len(live), V, device=DEV) * 3
        want = []
        for i, k in enumerate(live):
            p = sp[k]
            z = plain.apply_penalties(logits[i].cpu().double(), prompts[k], outputs[k], p.repetition_penalty,
                                      p.frequency_penalty, p.presence_penalty)
            want.append(int(z.argmax()))
        toks = s.sample(logits, [(sp[k], len(outputs[k]), prompts[k], outputs[k], 0, k) for k in live])
        assert toks == want, (step, live, toks, want)
        for k, t in zip(live, toks):
            outputs[k].append(t)
            outputs[k].append(prompts[k][0])   # and one the sampler did not choose (a forced token): counted all the same
        for k in ends.get(step, []):
            s.forget(k)
    assert len(s._slots) == 2 and len(s._free) == 1
    # rows without a name send their whole history and keep no slot
    logits = torch.randn(2, V, device=DEV) * 3
    rows = [(sp["d"], 3, [5, 6, 7], [7, 7, 8], 0), (sp["e"], 0, [1], [], 0)]
    want = [int(plain.apply_penalties(logits[i].cpu().double(), r[2], r[3], r[0].repetition_penalty, r[0].frequency_penalty,
                                      r[0].presence_penalty).argmax()) for i, r in enumerate(rows)]
    with pytest.raises(RuntimeError, match="live requests with penalties"):
        s.sample(logits, rows)               # one slot is free, two are needed
    s.forget("d")
    assert s.sample(logits, rows) == want and len(s._free) == 2


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 64])
def test_gemm_small_m(M, out_dtype):
    """Weight-streaming MFMA product against float64, at sizes that are no multiples of its tiles."""
    for N, K in ((96, 512), (331, 80), (4096, 4096), (1000, 1096), (50, 8), (6144, 64), (5000, 128), (10240, 64), (9001, 72)):
        a = torch.randn(M, K, device=DEV).to(torch.bfloat16)
        w = (torch.randn(N, K, device=DEV) * 0.05).to(torch.bfloat16)
        want = a.double() @ w.double().T
        for rt, waves in ((0, 0), (1, 1), (2, 4), (1, 16), (4, 2) if M <= 32 else (2, 8)):
            out = torch.full((M, N), float("nan"), device=DEV, dtype=out_dtype)
            ops().gemm_small_m(a, w, out, M, row_tiles=rt, waves=waves)
            t = dict(rtol=2e-2, atol=2e-2) if out_dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
            torch.testing.assert_close(out.double(), want, **t, msg=lambda m_: f"M={M} N={N} K={K} rt={rt} waves={waves}: {m_}")


def test_library_gemm_with_measured_algorithm(tmp_path):
    """Products of many rows: the vendor library called directly. Inside `measuring()` (the engine's warm-up) the
    candidates of a shape are timed once and the choice goes to the plan file; outside it nothing is timed: a shape
    runs what it was given, or the library's first suggestion. Rows may be rounded up to a bucket inside scratch
    buffers: the rows asked for are right, rows past the bucket untouched."""
    import json
    from dinfer_amd.kernels import blaslt, gemm
    blaslt.configure(tuning="measured", plan_file=str(tmp_path / "plans.json"))
    blaslt._plans.clear()                                                    # what earlier tests of this process met
    assert blaslt.available()
    a = torch.randn(200, 1096, device=DEV).to(torch.bfloat16)
    w = (torch.randn(1000, 1096, device=DEV) * 0.05).to(torch.bfloat16)
    out = torch.empty(200, 1000, device=DEV, dtype=torch.bfloat16)
    gemm.matmul_nt(a, w, out, 200)                                           # outside: no measurement
    assert not any(p and p.tuned for p in blaslt._plans.values())
    with blaslt.measuring():
        _library_gemm_cases(gemm)
    stored = json.loads((tmp_path / "plans.json").read_text())
    assert any(k.startswith("520,1000,1096,") for k in stored) and all(0 <= v["index"] < 32 for v in stored.values())
    # a process that starts with the file takes its choices without measuring: forget the plans, keep the file
    measured = {k: p.index for k, p in blaslt._plans.items() if p and p.tuned}
    blaslt._plans.clear()
    _library_gemm_cases(gemm)
    again = {k: p.index for k, p in blaslt._plans.items() if p and p.tuned}
    assert again == measured and all(p.times is None for p in blaslt._plans.values() if p)
    blaslt.configure(plan_file=None)


def _library_gemm_cases(gemm):
    from dinfer_amd.kernels import blaslt
    for M, N, K in ((130, 200, 264), (520, 1000, 1096), (33, 96, 512), (257, 4096, 512), (70, 50, 100), (40, 33, 6), (35, 7, 1)):
        a = torch.randn(M + 70, K, device=DEV).to(torch.bfloat16)
        w = (torch.randn(N, K, device=DEV) * 0.05).to(torch.bfloat16)
        want = a[:M].double() @ w.double().T
        for pad in (False, True):
            out = torch.full((M + 70, N), 7.0, device=DEV, dtype=torch.bfloat16)
            for _ in range(2):                                   # the second call replays the choice of the first
                gemm.matmul_nt(a, w, out, M, may_pad=pad)
            torch.testing.assert_close(out[:M].double(), want, rtol=2e-2, atol=2e-2, msg=lambda m_: f"{M}x{N}x{K} pad={pad}: {m_}")
            last = gemm.row_bucket(M) if pad else M
            assert bool((out[last:] == 7.0).all()), f"{M}x{N}x{K} pad={pad}: rows past {last} were written"
    assert any(p and p.tuned for p in blaslt._plans.values())        # the larger shapes above were measured
    assert any(p and not p.tuned for p in blaslt._plans.values())    # the tiny ones took the library's first suggestion
    # float32 out (logits at many positions): not rounded to bfloat16 on the way
    a = torch.randn(100, 264, device=DEV).to(torch.bfloat16)
    w = (torch.randn(1000, 264, device=DEV) * 0.05).to(torch.bfloat16)
    out = torch.empty(100, 1000, device=DEV)
    gemm.matmul_nt(a, w, out, 100)
    torch.testing.assert_close(out.double(), a.double() @ w.double().T, rtol=1e-4, atol=1e-4)


def test_library_gemm_adds_into_its_output(tmp_path):
    """stream += a . w^T through the library: a shape that is measured times the candidates on a copy (the stream
    itself gets the product once), later calls add once each; rows past the bucket are untouched; the few-row and
    tall shapes are refused (other kernels serve them)."""
    from dinfer_amd.kernels import blaslt, gemm
    blaslt.configure(tuning="measured", plan_file=str(tmp_path / "plans.json"))
    blaslt._plans.clear()
    assert blaslt.available()
    with blaslt.measuring():
        _library_add_cases(gemm)
    assert any(p and p.tuned for key, p in blaslt._plans.items() if key[-1])   # an adding product was measured too
    blaslt.configure(plan_file=None)
    a = torch.randn(32, 64, device=DEV).to(torch.bfloat16)
    assert not gemm.add_nt(a, torch.zeros(48, 64, device=DEV, dtype=torch.bfloat16), torch.zeros(32, 48, device=DEV, dtype=torch.bfloat16), 32)
    assert not gemm.add_nt(a.float(), torch.zeros(48, 64, device=DEV), torch.zeros(32, 48, device=DEV), 32)


def _library_add_cases(gemm):
    for M, N, K in ((520, 1000, 1096), (130, 200, 264), (40, 33, 8), (257, 4096, 512)):
        a = torch.randn(M + 70, K, device=DEV).to(torch.bfloat16)
        w = (torch.randn(N, K, device=DEV) * 0.05).to(torch.bfloat16)
        start = torch.randn(M + 70, N, device=DEV).to(torch.bfloat16)
        prod = a[:M].double() @ w.double().T
        stream = start.clone()
        last = gemm.row_bucket(M)
        for call in (1, 2):
            before = stream[:M].double()
            assert gemm.add_nt(a, w, stream, M)
            want = before + prod
            # one rounding of (float sum of products + stream) per call
            err = (stream[:M].double() - want).abs()
            assert bool((err <= 2.0 ** -8 * want.abs() + 1e-3 * prod.abs().mean()).all()), f"{M}x{N}x{K} call {call}: {err.max()}"
            assert torch.equal(stream[last:], start[last:]), f"{M}x{N}x{K}: rows past {last} were written"


@pytest.mark.parametrize("M", [1, 8, 16, 17, 32])
def test_gemm_small_m_gated(M):
    """Both projections of a gated feed-forward and silu(gate) * up in one kernel, against float64."""
    for N, K in ((136, 4096), (1000, 1096), (12288, 512), (20, 8)):
        a = torch.randn(M, K, device=DEV).to(torch.bfloat16)
        w = (torch.randn(2 * N, K, device=DEV) * 0.05).to(torch.bfloat16)
        z = a.double() @ w.double().T
        want = plain.silu(z[:, :N]) * z[:, N:]
        for waves in (0, 1, 8):
            out = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
            ops().gemm_small_m_gated(a, w, out, M, waves=waves)
            # one rounding of the result; the operands are exact here, so the sums are exact to float
            err = (out.double() - want).abs()
            assert bool((err <= 1e-2 * want.abs() + 1e-3 * want.std()).all()), f"M={M} N={N} K={K}: {float(err.max())}"


@pytest.mark.parametrize("M", [1, 8, 16, 17, 32])
def test_gemm_small_m_carries_the_norm(M):
    """A product that adds into the residual stream and leaves what the next RMSNorm needs (the stream times the gain,
    sums of squares per 16 or 8 columns), and the product that takes those: together they equal add, norm and product, to
    rounding, at widths that are no multiples of the tiles, with the gain in either dtype and an offset. (Consumers of
    4,097 to 6,144 outputs take 24 weight rows a workgroup at up to 16 tokens: 6,144, 5,000 and 4,120 end their last
    workgroup at 24, 8 and 16 rows; so do producers of that width: 5,120 and 4,108, whose last workgroup has 4 rows.
    A producer of 9,000 columns in two tiles a workgroup ends with a tile that has no column: it leaves no sum. A
    consumer of 8,193 to 10,240 outputs takes 40 rows a workgroup: 10,240 and 9,000. Up to 2,048 rows a workgroup
    takes 8, producer or consumer.)"""
    eps = 1e-5
    for N, K, N2 in ((96, 512, 136), (328, 80, 1000), (4096, 4096, 6144), (1000, 1096, 50), (200, 64, 5000), (72, 128, 4120),
                     (5120, 256, 64), (4108, 64, 32), (64, 72, 10240), (9000, 64, 9000)):
        for gain_dtype, offset in ((torch.float32, 0.0), (torch.bfloat16, 1.0)):
            a = torch.randn(M, K, device=DEV).to(torch.bfloat16)
            w = (torch.randn(N, K, device=DEV) * 0.05).to(torch.bfloat16)
            h0 = torch.randn(M + 1, N, device=DEV).to(torch.bfloat16)
            gain = (torch.randn(N, device=DEV) * 0.1 + (1.0 - offset)).to(gain_dtype)
            h = h0.clone()
            xg = torch.full((M + 1, N), 7.0, device=DEV, dtype=torch.bfloat16)
            stats = torch.full((M + 1, -(-N // 8) + 3), 7.0, device=DEV)
            cols = ops().gemm_small_m_sink(a, w, h, xg, gain, stats, M, gain_offset=offset)
            per = 8 if cols == -(-N // 8) else 16         # the 24-row form counts per 8 columns
            assert cols == -(-N // per) and (per == 8) == (M <= 16 and (N <= 2048 or 4096 < N <= 6144))
            want_h = (h0[:M].double() + a.double() @ w.double().T)
            err = (h[:M].double() - want_h).abs()
            # one rounding of a float sum of K products
            assert bool((err <= 2 ** -8 * want_h.abs() + 1e-5 * want_h.abs().mean()).all()), f"stream M={M} N={N} K={K}: {float(err.max())}"
            assert torch.equal(h[M:], h0[M:]) and bool((xg[M:] == 7.0).all()) and bool((stats[M:] == 7.0).all())
            assert bool((stats[:M, cols:] == 7.0).all())
            hs = h[:M].double()                                       # from here on the stream as it was stored
            pad = torch.zeros(M, cols * per - N, device=DEV, dtype=torch.float64)
            want_stats = torch.cat([hs, pad], dim=1).reshape(M, cols, per).pow(2).sum(-1)
            torch.testing.assert_close(stats[:M, :cols].double(), want_stats, rtol=1e-5, atol=1e-6)
            want_xg = hs * (gain.double() + offset)
            assert bool(((xg[:M].double() - want_xg).abs() <= 2 ** -8 * want_xg.abs() + 1e-6).all())
            if N % 8:
                continue                                              # the consumer reads 16 bytes at a time
            normed = hs / (hs.pow(2).mean(-1, keepdim=True) + eps).sqrt() * (gain.double() + offset)
            rstd = (stats[:M, :cols].double().sum(-1, keepdim=True) / N + eps).rsqrt()
            for gated in (False, True):
                w2 = (torch.randn((2 if gated else 1) * N2, N, device=DEV) * 0.05).to(torch.bfloat16)
                out = torch.full((M + 1, N2), 7.0, device=DEV, dtype=torch.bfloat16)
                ops().gemm_small_m_scaled(xg, w2, out, M, stats, cols, eps, N, gated=gated)
                assert bool((out[M:] == 7.0).all())
                # the kernel itself, on the operands as they are stored: only the result is rounded
                z = (xg[:M].double() @ w2.double().T) * rstd
                want = plain.silu(z[:, :N2]) * z[:, N2:] if gated else z
                err = (out[:M].double() - want).abs()
                assert bool((err <= 1e-2 * want.abs() + 1e-3 * want.std()).all()), f"M={M} N={N} N2={N2} gated={gated}: {float(err.max())}"
                if not gated:
                    # and the pair against norm, then product: the operand is rounded once more, as a norm's output is
                    want = normed @ w2.double().T
                    err = (out[:M].double() - want).abs()
                    assert bool((err <= 2e-2 * want.abs() + 2e-2 * want.abs().mean()).all()), f"M={M} N={N} N2={N2}: {float(err.max())}"


@pytest.mark.parametrize("M", [1, 17, 32, 33, 48, 64])
def test_gemm_mid_m(M):
    """The product that keeps a slice of the activations in LDS, plain and gated, against float64: sizes that are no
    multiples of its tiles, slices that end inside a 64-wide step, one slice and many, every form it has."""
    from dinfer_amd.kernels.lib import KernelError
    ran = 0
    for N, K in ((96, 512), (332, 80), (4096, 4096), (1000, 1096), (52, 8), (260, 2600)):
        a = torch.randn(M, K, device=DEV).to(torch.bfloat16)
        w = (torch.randn(2 * N, K, device=DEV) * 0.05).to(torch.bfloat16)
        z = a.double() @ w.double().T
        for gated in (False, True):
            want = plain.silu(z[:, :N]) * z[:, N:] if gated else z[:, :N]
            for ks, rt in ((0, 0), (1024, 1), (1024, 2), (64, 4), (2048, 1), (1536, 2), (256, 1)):
                try:
                    need = ops().gemm_mid_m_workspace(M, N, K, gated=gated, ks=ks, rt=rt)
                except KernelError:
                    assert M > 32 and ks > 1024          # only a slice that LDS does not hold is refused
                    continue
                ws = torch.full((need // 4 + 8,), float("nan"), device=DEV)
                for out_dtype in (torch.bfloat16,) if gated else (torch.bfloat16, torch.float32):
                    out = torch.full((M + 2, N), 7.0, device=DEV, dtype=out_dtype)
                    ops().gemm_mid_m(a, w if gated else w[:N], out, M, ws, gated=gated, ks=ks, rt=rt)
                    err = (out[:M].double() - want).abs()
                    tol = 1e-2 * want.abs() + 1e-3 * want.std() if out_dtype == torch.bfloat16 else 1e-4 * want.abs() + 1e-4
                    assert bool((err <= tol).all()), f"M={M} N={N} K={K} gated={gated} ks={ks} rt={rt}: {float(err.max())}"
                    assert bool((out[M:] == 7.0).all())
                    ran += 1
                with pytest.raises(KernelError):             # a workspace that is too small is refused, not overrun
                    ops().gemm_mid_m(a, w if gated else w[:N], out, M, ws[:max(need // 4 - 16, 0)], gated=gated, ks=ks, rt=rt)
    assert ran >= 60


@pytest.mark.parametrize("gain_dtype,offset", [(torch.bfloat16, 0.0), (torch.float32, 1.0)])
@pytest.mark.parametrize("M", [1, 17, 33, 50, 64])
def test_gemm_mid_m_adds_into_the_stream_and_norms_it(M, gain_dtype, offset):
    """The LDS-resident product whose pass over the partial sums is also the add into the residual stream and the
    RMSNorm that reads the stream next: the stream against float64 (one rounding), the norm's output against the plain
    norm of the stream the kernel left, rows beyond m and columns beyond N untouched; rows of very different sizes."""
    g = torch.Generator().manual_seed(M)
    for N, K, ks, rt in ((96, 512, 0, 0), (332, 1096, 256, 1), (4096, 12288, 1024, 2), (4096, 12288, 1536, 1),
                         (1000, 2600, 1024, 1), (5120, 1024, 0, 0), (8192, 512, 0, 0)):
        if ks > 1024 and M > 32:
            continue
        a = torch.randn(M + 1, K, generator=g).to(torch.bfloat16).to(DEV)
        w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
        rows = torch.exp(torch.randn(M + 2, 1, generator=g) * 2)
        whole = (torch.randn(M + 2, N + 8, generator=g) * rows).to(torch.bfloat16).to(DEV)
        before = whole.clone()
        stream = whole[:, :N]
        gain = (torch.rand(N, generator=g) + 0.5 - offset).to(gain_dtype).to(DEV)
        out_whole = torch.full((M + 2, N + 4), 7.0, dtype=torch.bfloat16, device=DEV)
        out = out_whole[:, :N]
        need = ops().gemm_mid_m_workspace(M, N, K, ks=ks, rt=rt)
        ws = torch.full((need // 4 + 8,), float("nan"), device=DEV)
        ops().gemm_mid_m_sink(a, w, stream, out, gain, offset, 1e-5, M, ws, ks=ks, rt=rt)
        want = before[:M, :N].double() + a[:M].double() @ w.double().T
        err = (stream[:M].double() - want).abs()
        assert bool((err <= 1e-2 * want.abs() + 1e-3 * want.std()).all()), f"stream, N={N} K={K}: {float(err.max())}"
        assert torch.equal(whole[M:], before[M:]) and torch.equal(whole[:, N:], before[:, N:]), "wrote beside the stream"
        normed = plain.rms_norm(stream[:M].double(), gain.double() + offset, 1e-5)
        err = (out[:M].double() - normed).abs()
        assert bool((err <= 1e-2 * normed.abs() + 1e-3).all()), f"norm, N={N} K={K}: {float(err.max())}"
        assert bool((out_whole[M:] == 7.0).all()) and bool((out_whole[:, N:] == 7.0).all()), "wrote beside the norm's output"
    from dinfer_amd.kernels.lib import KernelError
    with pytest.raises(KernelError):      # more columns than a workgroup of the second kernel holds
        N, K = 8192 + 64, 512
        ops().gemm_mid_m_sink(torch.zeros(M, K, dtype=torch.bfloat16, device=DEV), torch.zeros(N, K, dtype=torch.bfloat16, device=DEV),
                              torch.zeros(M, N, dtype=torch.bfloat16, device=DEV), torch.zeros(M, N, dtype=torch.bfloat16, device=DEV),
                              torch.ones(N, dtype=gain_dtype, device=DEV), 0.0, 1e-5, M, torch.zeros(1 << 22, device=DEV))


@pytest.mark.parametrize("M", [1, 17, 33, 48, 49, 64])
def test_gemm_wide(M):
    """The product for up to 64 rows whose waves stage their own activations in LDS: plain with bf16 and float output,
    gated, and as the consumer of a carried norm; a weight whose last workgroup has tiles to spare (N / 16 no multiple
    of six or three), K of one, two and three steps a wave."""
    g = torch.Generator().manual_seed(M)
    for N, K in ((16 * 13, 512), (16 * 31, 1024), (16 * 97, 1536)):
        a = (torch.randn(M + 3, K, generator=g) * 0.5).to(torch.bfloat16).to(DEV)
        w = (torch.randn(2 * N, K, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
        assert ops().gemm_wide_supports(M, N, K) and not ops().gemm_wide_supports(M, N + 8, K)
        assert not ops().gemm_wide_supports(M, N, K + 64) and not ops().gemm_wide_supports(65, N, K)
        ad, wd = a[:M].double().cpu(), w.double().cpu()
        for dtype in (torch.bfloat16, torch.float32):
            out = torch.full((M + 3, 2 * N), 7.0, dtype=dtype, device=DEV)
            ops().gemm_wide(a, w, out, M)
            torch.testing.assert_close(out[:M].double().cpu(), ad @ wd.T, rtol=2e-2, atol=2e-2)
            assert bool((out[M:] == 7.0).all()), "rows beyond m are left alone"
        gate, up = ad @ wd[:N].T, ad @ wd[N:].T
        out = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
        ops().gemm_wide(a, w, out, M, gated=True)
        torch.testing.assert_close(out.double().cpu(), plain.silu(gate) * up, rtol=2e-2, atol=2e-2)
        # the consumer of a carried norm: rows scaled by rsqrt(sum of the partial sums / width + eps)
        stats = torch.rand(M, 11, generator=g).to(DEV) * 40
        scale = torch.rsqrt(stats[:, :9].double().cpu().sum(-1, keepdim=True) / 300 + 1e-5)
        ops().gemm_wide(a, w, out, M, gated=True, stats=stats, cols=9, eps=1e-5, width=300)
        torch.testing.assert_close(out.double().cpu(), plain.silu(gate * scale) * (up * scale), rtol=2e-2, atol=2e-2)
        plainout = torch.zeros(M, 2 * N, dtype=torch.bfloat16, device=DEV)
        ops().gemm_wide(a, w, plainout, M, stats=stats, cols=9, eps=1e-5, width=300)
        torch.testing.assert_close(plainout.double().cpu(), (ad @ wd.T) * scale, rtol=2e-2, atol=2e-2)


def test_gemm_wide_at_the_size_it_runs_at():
    """The gate and up projections of the 8B sizes (256 workgroups, eight steps of k a wave, every wave's fragments of the
    activations landing in LDS one step ahead of their use) at the row counts the rule sends there, on four weights in
    turn so that the memory system is busy: a fragment read before it has landed would be the fragment of the step
    before, an error as large as the result."""
    N, K = 12288, 4096
    g = torch.Generator().manual_seed(5)
    ws = [(torch.randn(2 * N, K, generator=g) * 0.03).to(torch.bfloat16).to(DEV) for _ in range(4)]
    for M in (33, 48, 64):
        a = torch.randn(64, K, generator=g).to(torch.bfloat16).to(DEV)
        outs = [torch.zeros(64, N, dtype=torch.bfloat16, device=DEV) for _ in ws]
        for _ in range(3):
            for w, out in zip(ws, outs):
                ops().gemm_wide(a, w, out, M, gated=True)
        for w, out in zip(ws, outs):
            z = a[:M].double() @ w.double().T
            want = plain.silu(z[:, :N]) * z[:, N:]
            err = (out[:M].double() - want).abs()
            assert bool((err <= 2e-2 * want.abs() + 2e-3 * want.std()).all()), f"{M} rows: {float(err.max())}"


def test_gemm_wide_random_sizes_and_pitches():
    """Sixty products of random sizes (1 to 64 rows, N a multiple of 16 up to 6,400, K of 1 to 12 steps), operands and
    result with row pitches beyond their widths, plain, gated and as the consumer of a carried norm, bfloat16 and float
    out: the result against float64, and nothing written beside it."""
    import random
    rng = random.Random(11)
    for it in range(60):
        M, N, K = rng.randint(1, 64), 16 * rng.randint(1, 400), 512 * rng.randint(1, 12)
        pad_a, pad_w, pad_c = rng.choice([0, 8, 64]), rng.choice([0, 8, 128]), rng.choice([0, 4, 32])
        gated, scaled = rng.random() < 0.5, rng.random() < 0.4
        f32 = not gated and rng.random() < 0.3
        g = torch.Generator().manual_seed(it)
        a = (torch.randn(M + 2, K + pad_a, generator=g) * 0.5).to(torch.bfloat16).to(DEV)[:, :K]
        w = (torch.randn(2 * N if gated else N, K + pad_w, generator=g) * 0.1).to(torch.bfloat16).to(DEV)[:, :K]
        whole = torch.full((M + 2, N + pad_c), 7.0, dtype=torch.float32 if f32 else torch.bfloat16, device=DEV)
        out, kw = whole[:, :N], {}
        scale = torch.ones(M, 1, dtype=torch.float64, device=DEV)
        if scaled:
            cols, width = rng.randint(1, 40), rng.randint(100, 5000)
            stats = (torch.rand(M, cols + 3, generator=g) * 50).to(DEV)
            kw = dict(stats=stats, cols=cols, eps=1e-5, width=width)
            scale = torch.rsqrt(stats[:, :cols].double().sum(-1, keepdim=True) / width + 1e-5)
        ops().gemm_wide(a, w, out, M, gated=gated, **kw)
        z = (a[:M].double() @ w.double().T) * scale
        want = plain.silu(z[:, :N]) * z[:, N:] if gated else z
        err = (out[:M].double() - want).abs()
        tol = 1e-4 * want.abs() + 1e-3 * want.std() if f32 else 2e-2 * want.abs() + 2e-3 * want.std() + 1e-6
        assert bool((err <= tol).all()), f"case {it}: {M}x{N}x{K} gated {gated} scaled {scaled}: {float(err.max())}"
        assert bool((whole[M:] == 7.0).all()) and bool((whole[:, N:] == 7.0).all()), f"case {it}: wrote beside the result"


def test_products_of_17_to_64_rows_by_the_rule_of_sizes():
    """Between the few-row kernel and the library, a weight far wider than high goes to the LDS-resident kernel;
    whichever runs, the product is right, plain and gated, bfloat16 and float32 out, rows past the bucket untouched."""
    from dinfer_amd.kernels import gemm
    seen, wide = set(), set()
    for M in (17, 32, 33, 50, 64):
        # (the last: 10,000 gated columns are 209 workgroups of the kernel for wide weights, a round three quarters full)
        for N, K in ((96, 512), (1000, 1096), (333, 264), (2048, 8192), (1024, 16384), (10000, 512)):
            seen.add(gemm._tall(M, 2 * N, K))
            wide.add(gemm._wide(M, N, K))
            a = torch.randn(M + 70, K, device=DEV).to(torch.bfloat16)
            w = (torch.randn(2 * N, K, device=DEV) * 0.05).to(torch.bfloat16)
            z = a[:M].double() @ w.double().T
            for out_dtype in (torch.bfloat16, torch.float32):
                out = torch.full((M + 70, 2 * N), 7.0, device=DEV, dtype=out_dtype)
                gemm.matmul_nt(a, w, out, M, may_pad=True)
                t = dict(rtol=2e-2, atol=2e-2) if out_dtype == torch.bfloat16 else dict(rtol=1e-4, atol=2e-4)
                torch.testing.assert_close(out[:M].double(), z, **t, msg=lambda m_: f"{M}x{2 * N}x{K}: {m_}")
                assert bool((out[96:] == 7.0).all())
            want = plain.silu(z[:, :N]) * z[:, N:]
            act = torch.full((M + 70, N), 7.0, device=DEV, dtype=torch.bfloat16)
            scratch = torch.empty(M + 70, 2 * N, device=DEV, dtype=torch.bfloat16)
            gemm.gated_nt(a, w, act, scratch, M, "silu")
            err = (act[:M].double() - want).abs()
            assert bool((err <= 2e-2 * want.abs() + 2e-3 * want.std()).all()), f"gated {M}x{N}x{K}: {float(err.max())}"
            assert bool((act[M:] == 7.0).all())
    assert seen == {True, False} and wide == {True, False}          # both sides of each rule were met
    assert gemm._wide(64, 12288, 4096) and not gemm._wide(64, 17408, 5120)
    assert gemm._wide(17, 12288, 4096) and not gemm._wide(16, 12288, 4096)


def test_a_graph_keeps_its_partial_sums_when_the_buffer_grows():
    """A decode graph captured while the buffer for partial sums was small must still be right after a larger
    product has made the buffer grow: the old buffer stays where it is and belongs to nobody else."""
    from dinfer_amd.kernels import gemm
    M, N, K = 20, 2048, 8192
    assert gemm._tall(M, N, K)
    a = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) * 0.05).to(torch.bfloat16)
    out = torch.zeros(M, N, device=DEV, dtype=torch.bfloat16)
    gemm._workspace.pop(a.device, None)                  # as in a new process: the first product sizes the buffer
    gemm.matmul_nt(a, w, out, M)
    want = out.clone()
    small = gemm._workspace[a.device]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        gemm.matmul_nt(a, w, out, M)
    a2 = torch.randn(64, 4 * K, device=DEV).to(torch.bfloat16)
    w2 = (torch.randn(N, 4 * K, device=DEV) * 0.05).to(torch.bfloat16)
    gemm.matmul_nt(a2, w2, torch.empty(64, N, device=DEV, dtype=torch.bfloat16), 64)   # needs more: the buffer grows
    assert gemm._workspace[a.device] is not small and gemm._workspace[a.device].numel() > small.numel()
    del small
    others = [torch.full((1 << 20,), 3.0, device=DEV) for _ in range(16)]                # would land in freed memory
    for _ in range(2):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
    assert all(bool((t == 3.0).all()) for t in others)


@pytest.mark.parametrize("start", [0, 8, 3])
def test_qkv_post_many_tokens_writes_v_transposed(start):
    """From 64 tokens on, V is written by the gathering kernel: slots that start on a multiple of 8
    (16-byte rows of V^T), slots that do not (element stores), pages in shuffled order, a ragged tail
    and a token without a slot."""
    H, Hkv, D, page, T = 8, 2, 128, 16, 77
    qkv_in = torch.randn(T, (H + 2 * Hkv) * D, device=DEV).to(torch.bfloat16)
    pos = torch.arange(start, start + T, device=DEV, dtype=torch.int32)
    nblocks = 8
    order = [5, 2, 7, 0, 3, 6, 1, 4]
    slots = [order[p // page] * page + p % page for p in range(start, start + T)]
    slots[40] = -1
    slots_t = torch.tensor(slots, device=DEV, dtype=torch.int64)
    table = rope_table(128, D, 1e6).to(DEV)
    kc = torch.zeros(ops().k_cache_shape(nblocks, Hkv, page, D), device=DEV, dtype=torch.bfloat16)
    vc = torch.zeros(nblocks, Hkv, D, page, device=DEV, dtype=torch.bfloat16)
    qkv = qkv_in.clone()
    ops().qkv_post(qkv, T, heads=H, kv_heads=Hkv, head_dim=D, q_off=0, k_off=H * D, v_off=(H + Hkv) * D, q_gain=None,
                   k_gain=None, eps=0.0, gain_offset=0.0, positions=pos, cos_sin=table, rotary_dim=D, rope_style=0,
                   k_cache=kc, v_cache=vc, slot_mapping=slots_t, page_size=page)
    v = qkv_in[:, (H + Hkv) * D:].view(T, Hkv, D)
    want_v = torch.zeros_like(vc)
    for t, s in enumerate(slots):
        if s >= 0:
            want_v[s // page, :, :, s % page] = v[t]
    assert torch.equal(vc, want_v)
    k = plain.rope_neox(qkv_in[:, H * D:(H + Hkv) * D].double().cpu().view(T, Hkv, D), plain.rope_angles(pos.tolist(), D, 1e6))
    for t, s in enumerate(slots):
        if s >= 0:
            torch.testing.assert_close(ops().k_cache_rows(kc)[s // page, :, s % page, :].double().cpu(), k[t], rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_widen_fill(dtype):
    a = torch.randn(5, 331, device=DEV).to(dtype)
    b = torch.randn(5, 331, device=DEV).to(dtype)
    want = (a.float() + b.float()).to(dtype)            # summed in float, one rounding
    ops().add_inplace(a, b)
    assert torch.equal(a, want)
    wide = torch.empty(5, 331, device=DEV)
    ops().widen(b, wide)
    assert torch.equal(wide, b.float())
    ops().fill_zero(wide)
    assert not wide.any()


@pytest.mark.parametrize("dtype", DTYPES)
def test_scale_and_soft_cap(dtype):
    x = (torch.randn(5, 333, device=DEV) * 20).to(dtype)
    for scale, cap in ((0.5, None), (1.0, 30.0), (3.0, 7.5)):
        got = x.clone()
        ops().scale_softcap(got, 4, scale, cap)
        want = x[:4].double() * scale
        if cap:
            want = cap * torch.tanh(want / cap)
        torch.testing.assert_close(got[:4].double(), want, **tol(dtype))
        assert torch.equal(got[4], x[4]), "rows beyond the count are left alone"
        assert cap is None or float(got[:4].float().abs().max()) <= cap


def test_measured_ceilings_are_plausible():
    """The two kernels that measure what the chip gives a kernel that only reads and one that only multiplies:
    between a fifth of the vendor's figures and the figures themselves."""
    hbm = ops().measured_hbm_read(DEV, nbytes=1 << 30)
    assert 1.6e12 < hbm < 8.0e12, hbm
    mfma = ops().measured_mfma_bf16(DEV)
    assert 0.5e15 < mfma < 2.5e15, mfma


@pytest.mark.parametrize("V", [331, 4097, 151936])
def test_logprobs_of_chosen_and_most_probable_tokens(V):
    """Log-softmax of the row as given: the chosen token's value and rank, the k most probable in falling order.
    Equal logits (planted at the top and around the chosen token) go by index; a row that asks nothing is left
    alone; k = 0 gives the chosen token only."""
    g = torch.Generator().manual_seed(V)
    logits = torch.randn(6, V, generator=g) * 4
    ks = [-1, 0, 3, 20, 7, 32]
    chosen = [5, V - 1, 17, 0, 200, 9]
    logits[2, [40, 3, 300]] = logits[2].max() + 1.0            # three equal best: 3, 40, 300 in that order
    logits[4, [100, 200, 250]] = float(logits[4].topk(5).values[-1])   # the chosen one has twins of equal value
    logits[5, 1:] = logits[5, 0]                                # a flat row: every rank is 0, the top is 0, 1, 2, ...
    stride = 33
    ids = torch.full((6, stride), -7, dtype=torch.int32, device=DEV)
    lps = torch.full((6, stride), 7.0, dtype=torch.float32, device=DEV)
    rank = torch.full((6,), -7, dtype=torch.int32, device=DEV)
    i32 = lambda xs: torch.tensor(xs, device=DEV, dtype=torch.int32)
    ops().logprobs(logits.to(DEV), i32(chosen), i32(ks), ids, lps, rank, 6)
    ids, lps, rank = ids.cpu(), lps.cpu(), rank.cpu()
    assert (ids[0] == -7).all() and (lps[0] == 7.0).all() and rank[0] == -7
    for r in range(1, 6):
        lp, rk, top = plain.token_logprobs(logits[r], chosen[r], ks[r])
        assert ids[r, 0] == chosen[r] and rank[r] == rk, (r, int(rank[r]), rk)
        assert abs(float(lps[r, 0]) - lp) < 2e-5
        assert ids[r, 1:ks[r] + 1].tolist() == [t for t, _ in top], r
        torch.testing.assert_close(lps[r, 1:ks[r] + 1].double(), torch.tensor([v for _, v in top], dtype=torch.float64),
                                   rtol=0, atol=2e-5)
        assert (ids[r, ks[r] + 1:] == -7).all()
    assert ids[2, 1:4].tolist() == [3, 40, 300] and rank[5] == 0 and ids[5, 1:5].tolist() == [0, 1, 2, 3]


def test_logprobs_of_a_vocabulary_smaller_than_k():
    logits = torch.tensor([[0.0, 1.0, -1.0]])
    ids = torch.zeros((1, 6), dtype=torch.int32, device=DEV)
    lps = torch.zeros((1, 6), dtype=torch.float32, device=DEV)
    rank = torch.zeros(1, dtype=torch.int32, device=DEV)
    i32 = lambda xs: torch.tensor(xs, device=DEV, dtype=torch.int32)
    ops().logprobs(logits.to(DEV), i32([2]), i32([5]), ids, lps, rank, 1)
    assert ids.cpu()[0].tolist() == [2, 1, 0, 2, -1, -1] and rank.item() == 2
    assert lps.cpu()[0, 4:].tolist() == [float("-inf")] * 2


def test_logit_bias_adds_to_the_named_logits_only():
    V = 1000
    logits = torch.randn(3, V)
    entries = [(0, 5, 2.5), (2, 999, -100.0), (2, 0, 100.0), (1, 17, 0.25), (3, 4, 9.0), (1, 1000, 9.0), (-1, 3, 9.0)]
    got = logits.to(DEV)
    ops().logit_bias(got, 3, torch.tensor([(r, t) for r, t, _ in entries], dtype=torch.int32, device=DEV),
                     torch.tensor([b for *_, b in entries], dtype=torch.float32, device=DEV))
    want = logits.clone()
    for r, bias in ((0, {5: 2.5}), (1, {17: 0.25}), (2, {999: -100.0, 0: 100.0})):      # the rest names no cell
        want[r] = plain.apply_logit_bias(logits[r], bias)
    torch.testing.assert_close(got.cpu(), want, rtol=0, atol=0)


def test_sampler_with_bias_penalties_and_logprobs_in_one_batch():
    """Rows of every kind side by side: the token comes from the logits after bias and penalties, the
    log-probabilities from the logits as they were given."""
    from dinfer_amd.sampling.params import SamplingParams
    from dinfer_amd.sampling.sampler import Sampler
    V = 777
    s = Sampler(DEV, 6, V)
    g = torch.Generator().manual_seed(9)
    for turn in range(3):                       # (the pinned buffers alternate: both are used, and one again)
        logits = torch.randn(5, V, generator=g) * 3
        best = logits.argmax(-1).tolist()
        sps = [SamplingParams(temperature=0.0, logprobs=2),
               SamplingParams(temperature=0.0, logit_bias={best[1]: -100.0}, logprobs=0),
               SamplingParams(temperature=0.0, logit_bias={3: 100.0}),
               SamplingParams(temperature=0.0, repetition_penalty=2.0, presence_penalty=2.0, logprobs=20),
               SamplingParams(temperature=0.9, seed=5, logit_bias=[(7, 1.5), (8, -1.5)], logprobs=1)]
        prompt, output = [best[3], 4], [best[3], 9]
        rows = [(p, turn, prompt, output, p.seed or 0) for p in sps]
        launched = s.launch(logits.to(DEV), rows)
        toks, about = launched.tokens(), launched.logprobs()
        z1 = plain.apply_logit_bias(logits[1].double(), sps[1].logit_bias)
        z3 = plain.apply_penalties(logits[3].double(), prompt, output, 2.0, 0.0, 2.0)
        z4 = plain.apply_logit_bias(logits[4].double(), sps[4].logit_bias)
        want4, slack = plain.sample_row(z4, 0.9, 5, turn)
        assert toks[0] == best[0] and toks[1] == int(z1.argmax()) != best[1] and toks[2] == 3
        assert toks[3] == int(z3.argmax()) != best[3]
        assert toks[4] == want4 or slack < 1e-5
        assert about[2] is None
        for r in (0, 1, 3, 4):
            lp, rk, top = plain.token_logprobs(logits[r], toks[r], sps[r].logprobs)
            a = about[r]
            assert a.token_id == toks[r] and a.rank == rk and abs(a.logprob - lp) < 2e-5
            assert [t for t, _ in a.top] == [t for t, _ in top]
        assert about[0].rank == 0 and about[1].rank == 1 and about[3].rank >= 1
