"""Each HIP kernel alone against a plain float reference of the same op, at sizes other than the
engine's (odd widths, head sizes in steps of 16, vocabularies that are no power of two)."""
import math

import numpy as np

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from llm_infrence_engine_amd.kernels import ops

    return ops


def tol(dtype):
    # float: sums of a few hundred products; bfloat16: one rounding of the result (2^-8 relative) on top
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=1.6e-2)


DTYPES = [torch.float32, torch.bfloat16]


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(ops, dtype):
    g = torch.Generator().manual_seed(0)
    table = torch.randn(331, 72, generator=g).to(dtype).to(DEV)
    ids = torch.randint(0, 331, (13,), generator=g).to(torch.int32).to(DEV)
    out = torch.empty(13, 72, dtype=torch.float32, device=DEV)
    ops.embed(ids, table, out)
    assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [72, 896, 1500, 16384, 20000])
def test_rms_norm(ops, dtype, H):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(9, H, generator=g) * 3).to(DEV)
    w = (1 + 0.1 * torch.randn(H, generator=g)).to(DEV)
    out = torch.empty(9, H, dtype=dtype, device=DEV)
    ops.rms_norm(x, w, 1e-5, out)
    want = w.double() * (x.double() * torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5))
    torch.testing.assert_close(out.double(), want, **tol(dtype))
    # with the residual sum fused, and rows gathered
    delta = torch.randn(9, H, generator=g).to(dtype).to(DEV)
    x2 = x.clone()
    ops.rms_norm(x2, w, 1e-5, out, delta=delta)
    s = x.double() + delta.double()
    torch.testing.assert_close(x2.double(), s, atol=1e-6, rtol=1e-6)
    want = w.double() * (s * torch.rsqrt((s ** 2).mean(-1, keepdim=True) + 1e-5))
    torch.testing.assert_close(out.double(), want, **tol(dtype))
    rows = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
    out3 = torch.empty(3, H, dtype=dtype, device=DEV)
    ops.rms_norm(x2, w, 1e-5, out3, rows=rows)
    torch.testing.assert_close(out3.double(), want[rows.long()], **tol(dtype))
    # the sum formed but not kept, from two partial sums
    x3 = x.clone()
    halves = torch.stack((delta.float() * 0.25, delta.float() * 0.75)).to(dtype)
    ops.rms_norm(x3, w, 1e-5, out, delta=halves, write_back=False)
    assert torch.equal(x3, x)
    s = x.double() + halves[0].double() + halves[1].double()
    want = w.double() * (s * torch.rsqrt((s ** 2).mean(-1, keepdim=True) + 1e-5))
    torch.testing.assert_close(out.double(), want, **tol(dtype))


def test_rms_norm_eps_inside_root(ops):
    x = torch.full((1, 16), 1e-6, device=DEV)
    out = torch.empty(1, 16, device=DEV)
    ops.rms_norm(x, torch.ones(16, device=DEV), 1e-2, out)
    torch.testing.assert_close(out, x / math.sqrt(1e-12 + 1e-2), rtol=1e-6, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(ops, dtype):
    g = torch.Generator().manual_seed(2)
    gu = (torch.randn(7, 2 * 200, generator=g) * 2).to(dtype).to(DEV)
    out = torch.empty(7, 200, dtype=dtype, device=DEV)
    ops.silu_mul(gu, out)
    a = gu.double()
    want = torch.nn.functional.silu(a[:, 0::2]) * a[:, 1::2]
    torch.testing.assert_close(out.double(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,N,K", [(1, 331, 72), (5, 64, 120), (70, 200, 896), (130, 151, 50), (3, 1000, 4864)])
def test_gemm_generic(ops, dtype, M, N, K):
    g = torch.Generator().manual_seed(3)
    a = torch.randn(M, K, generator=g).to(dtype).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    want = a.double() @ w.double().T
    out = torch.empty(M, N, dtype=dtype, device=DEV)
    ops.gemm_generic(a, w, out)
    torch.testing.assert_close(out.double(), want, **tol(dtype))
    ops.gemm_generic(a, w, out, bias=bias)
    torch.testing.assert_close(out.double(), want + bias.double(), **tol(dtype))
    acc = torch.randn(M, N, generator=g).to(DEV)
    acc0 = acc.clone()
    ops.gemm_generic(a, w, acc, accumulate=True)  # float result whatever the inputs are
    torch.testing.assert_close(acc.double(), acc0.double() + want, atol=2e-5, rtol=2e-5)


def test_gemm_row_does_not_depend_on_the_batch(ops):
    g = torch.Generator().manual_seed(4)
    a = torch.randn(77, 192, generator=g).to(DEV)
    w = torch.randn(331, 192, generator=g).to(DEV)
    full = torch.empty(77, 331, device=DEV)
    one = torch.empty(1, 331, device=DEV)
    ops.gemm_generic(a, w, full)
    ops.gemm_generic(a[40:41], w, one)
    assert torch.equal(full[40:41], one)


def rope_reference(x, pos, rot, inv):
    ang = pos.double()[:, None] * inv[None]
    cos, sin = torch.cat((ang, ang), -1).cos()[:, None], torch.cat((ang, ang), -1).sin()[:, None]
    xr = x[..., :rot]
    half = rot // 2
    rotated = xr * cos + torch.cat((-xr[..., half:], xr[..., :half]), -1) * sin
    return torch.cat((rotated, x[..., rot:]), -1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("vt", [False, True])
@pytest.mark.parametrize("nh,nkv,d,rot", [(4, 2, 16, 16), (5, 1, 48, 48), (6, 3, 80, 32), (3, 1, 20, 20), (2, 2, 24, 12),
                                          (14, 2, 64, 64), (2, 1, 256, 256)])
def test_rope_store(ops, dtype, nh, nkv, d, rot, vt):
    """Sizes that the 16-byte kernel takes and sizes that fall to the element-wise one; values pages plain and
    transposed; with and without a late bias; one token that is not stored."""
    g = torch.Generator().manual_seed(5)
    N, page_size, pages = 11, 4, 9
    qkv = torch.randn(N, (nh + 2 * nkv) * d, generator=g).to(dtype)
    pos = torch.tensor([0, 1, 2, 3, 8191, 5, 100, 7, 4000, 9, 10], dtype=torch.int32)
    slots = torch.randperm(pages * page_size, generator=g)[:N].to(torch.int32)
    slots[3] = -1
    theta = 1e6
    inv_freq = (1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot))).float()
    kp = torch.zeros(pages, nkv, page_size, d, dtype=dtype, device=DEV)
    vp = torch.zeros(pages, nkv, d, page_size, dtype=dtype, device=DEV) if vt else torch.zeros_like(kp)
    dev = qkv.to(DEV)
    bias = torch.randn((nh + 2 * nkv) * d, generator=g) if rot != 16 else None   # with and without a late bias
    ops.rope_store(dev, nh, nkv, d, rot, pos.to(DEV), inv_freq.to(DEV), slots.to(DEV), kp, vp, v_transposed=vt,
                   bias=None if bias is None else bias.to(DEV))
    x = qkv.double().view(N, nh + 2 * nkv, d)
    if bias is not None:
        x = x + bias.double().view(1, nh + 2 * nkv, d)
    want_q = rope_reference(x[:, :nh], pos, rot, inv_freq.double())
    want_k = rope_reference(x[:, nh:nh + nkv], pos, rot, inv_freq.double())
    got = dev.double().cpu().view(N, nh + 2 * nkv, d)
    # the angle is a float product of position and frequency: at position 8191 its rounding is ~2.4e-4 rad
    t = dict(atol=2e-3, rtol=0) if dtype == torch.float32 else dict(atol=3e-2, rtol=1.6e-2)
    torch.testing.assert_close(got[:, :nh], want_q, **t)
    torch.testing.assert_close(got[:, nh:nh + nkv], want_k, **t)
    small = pos < 200  # there the float angle is exact to ~1e-5
    torch.testing.assert_close(got[small][:, :nh], want_q[small], **tol(dtype))
    torch.testing.assert_close(got[:, nh + nkv:], x[:, nh + nkv:], **(tol(dtype) if bias is not None else dict(atol=0, rtol=0)))
    for n in range(N):
        s = int(slots[n])
        if s < 0:
            continue
        p, o = divmod(s, page_size)
        assert torch.equal(kp[p, :, o].cpu().double(), got[n, nh:nh + nkv])
        assert torch.equal((vp[p, :, :, o] if vt else vp[p, :, o]).cpu().double(), got[n, nh + nkv:])
    used = torch.zeros(pages * page_size, dtype=torch.bool)
    used[slots[slots >= 0].long()] = True
    assert (kp.cpu().permute(0, 2, 1, 3).reshape(pages * page_size, -1)[~used] == 0).all()


def attention_reference(q, k, v, scale, window=None):
    """q [nh, T, d], k/v [nkv, S, d] with the T queries at the last T of S positions."""
    nh, T, d = q.shape
    S = k.shape[1]
    rep = nh // k.shape[0]
    k, v = k.repeat_interleave(rep, 0), v.repeat_interleave(rep, 0)
    s = torch.einsum("htd,hsd->hts", q, k) * scale
    i = torch.arange(S - T, S)[:, None]
    j = torch.arange(S)[None]
    vis = j <= i
    if window:
        vis = vis & (j > i - window)
    s = s.masked_fill(~vis[None], float("-inf"))
    return torch.einsum("hts,hsd->htd", s.softmax(-1), v)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page_size,window", [(4, 2, 16, 4, None), (6, 2, 32, 8, None), (5, 1, 48, 16, None),
                                                        (3, 3, 80, 4, 7), (8, 2, 128, 16, 40)])
def test_paged_attention_generic(ops, dtype, nh, nkv, d, page_size, window):
    """Three requests in one batch: a whole prompt, a portion after a cached prefix, one decoded token;
    pages handed out in shuffled order and the pool pre-filled with large values that must never be read."""
    g = torch.Generator().manual_seed(6)
    ctx = [70, 133, 201]       # keys each request holds after this step
    qlen = [70, 9, 1]          # its new tokens
    pages_per = [-(-c // page_size) for c in ctx]
    P = sum(pages_per) + 5
    order = torch.randperm(P - 1, generator=g) + 1
    kp = torch.full((P, nkv, page_size, d), 1e4, dtype=dtype)
    vp = torch.full((P, nkv, page_size, d), -1e4, dtype=dtype)
    table = torch.zeros(3, max(pages_per), dtype=torch.int32)
    scale = 1.0 / math.sqrt(d)
    q_all, req_all, pos_all, want = [], [], [], []
    used = 0
    for r in range(3):
        k = torch.randn(nkv, ctx[r], d, generator=g).to(dtype)
        v = torch.randn(nkv, ctx[r], d, generator=g).to(dtype)
        q = (torch.randn(nh, qlen[r], d, generator=g) * 2).to(dtype)
        # one far key stands out for the last query of each request
        far = 3
        k[:, far] = (q[::nh // nkv, -1].float() * 1.5).to(dtype)
        pages = order[used:used + pages_per[r]]
        used += pages_per[r]
        table[r, :pages_per[r]] = pages.to(torch.int32)
        for j in range(ctx[r]):
            kp[pages[j // page_size], :, j % page_size] = k[:, j]
            vp[pages[j // page_size], :, j % page_size] = v[:, j]
        q_all.append(q.transpose(0, 1).reshape(qlen[r], nh * d))
        req_all += [r] * qlen[r]
        pos_all += list(range(ctx[r] - qlen[r], ctx[r]))
        want.append(attention_reference(q.double(), k.double(), v.double(), scale, window).transpose(0, 1).reshape(qlen[r], nh * d))
    q = torch.cat(q_all).to(DEV)
    N = q.shape[0]
    # q as a row slice of a wider matrix, as in the fused projection
    wide = torch.zeros(N, nh * d + 24, dtype=dtype, device=DEV)
    wide[:, :nh * d] = q
    out = torch.empty(N, nh * d, dtype=dtype, device=DEV)
    ops.paged_attention_generic(wide, kp.to(DEV), vp.to(DEV), table.to(DEV),
                                torch.tensor(req_all, dtype=torch.int32, device=DEV),
                                torch.tensor(pos_all, dtype=torch.int32, device=DEV), out, nh, scale, window)
    torch.testing.assert_close(out.double().cpu(), torch.cat(want), **tol(dtype))


def test_sample_greedy_and_vectors(ops):
    lg = torch.tensor([[0.1, 2.0, 0.5], [3.0, 0.0, 0.0], [1.0, 1.0, 1.0]], device=DEV)
    out = torch.empty(3, dtype=torch.int32, device=DEV)
    ops.sample(lg, out)
    assert out.tolist() == [1, 0, 0]  # first maximum on ties
    g = torch.Generator().manual_seed(7)
    big = torch.randn(5, 151936, generator=g).to(DEV)
    out = torch.empty(5, dtype=torch.int32, device=DEV)
    ops.sample(big, out)
    assert out.tolist() == big.argmax(-1).tolist()


def _draws_of_row(ops, row, n, temperature, top_k, top_p, seed=5, first_draw=0):
    """``n`` draws from one row of logits: the row repeated, each copy with a draw index of its own."""
    V = row.numel()
    lg = row.to(DEV).float().expand(n, V).contiguous()
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ops.sample(lg, out, torch.full((n,), temperature, device=DEV), torch.full((n,), top_k, dtype=torch.int32, device=DEV),
               torch.full((n,), top_p, device=DEV), torch.full((n,), seed, dtype=torch.int64, device=DEV),
               torch.arange(first_draw, first_draw + n, dtype=torch.int32, device=DEV))
    return out.cpu().long()


@pytest.mark.parametrize("V", [50, 1000, 151936])
@pytest.mark.parametrize("temperature,top_k,top_p", [(0.8, 50, 0.9), (1.3, 0, 0.7), (1.0, 5, 1.0), (1.0, 0, 1.0), (0.5, 7, 0.3)])
def test_sampler_draws_from_the_plain_distribution(ops, V, temperature, top_k, top_p):
    """Draws land only on tokens the plain rule keeps (temperature, top-k, top-p in the reference's order,
    src/miniserve/sampler.py:23-41) and as often as its probabilities say."""
    from tests.plain import qwen2_plain as P

    g = torch.Generator().manual_seed(V + top_k)
    row = torch.randn(V, generator=g) * 2.5
    want = P.logits_to_probs(row[None], temperature, top_k, top_p)[0]
    n = 8192
    got = _draws_of_row(ops, row, n, temperature, top_k, top_p)
    kept = (want > 0).nonzero().flatten()
    assert set(got.tolist()) <= set(kept.tolist()), "a token was drawn that the plain rule drops"
    freq = torch.bincount(got, minlength=V).double() / n
    # the tokens that carry the mass: each within five standard deviations of its probability
    for tok in want.topk(min(20, kept.numel())).indices.tolist():
        pr = float(want[tok])
        assert abs(float(freq[tok]) - pr) < 5 * math.sqrt(pr * (1 - pr) / n) + 2e-4, (tok, pr, float(freq[tok]))
    if kept.numel() <= 64:                                  # few enough that every kept token should appear
        assert (freq[kept] > 0).all() or float(want[kept].min()) * n < 8


def test_sampler_ties_thresholds_and_mixed_rows(ops):
    """Ties at the k-th value are all kept; the token at which the running mass reaches top_p is kept with all its
    equals; top_k = 1 and a tiny top_p are the greedy choice; rows without temperature take the first maximum
    beside rows that draw; and a draw does not depend on the rows beside it (nor on how many blocks a row is
    spread over)."""
    row = torch.tensor([1.0, 3.0, 2.0, 2.0, 0.5, 2.0, -1.0, 3.0])
    got = _draws_of_row(ops, row, 2048, 1.0, 3, 1.0)               # the third largest is 2.0, three times: five tokens stay
    assert set(got.tolist()) == {1, 2, 3, 5, 7}
    got = _draws_of_row(ops, row, 2048, 1.0, 0, 0.59)              # the two 3.0s hold 0.599 of the mass: they stay, nothing else
    assert set(got.tolist()) == {1, 7}
    got = _draws_of_row(ops, row, 2048, 1.0, 0, 0.61)              # a little more: the three 2.0s come in together
    assert set(got.tolist()) == {1, 2, 3, 5, 7}
    assert set(_draws_of_row(ops, row, 256, 2.0, 1, 1.0).tolist()) == {1, 7}      # both maxima tie at k = 1
    g = torch.Generator().manual_seed(3)
    big = torch.randn(151936, generator=g) * 3
    assert set(_draws_of_row(ops, big, 64, 1.5, 1, 1.0).tolist()) == {int(big.argmax())}
    assert set(_draws_of_row(ops, big, 64, 1.0, 0, 1e-6).tolist()) == {int(big.argmax())}
    # mixed rows, and the same draws alone and in company
    rows = torch.stack([big, big.flip(0), big * 0.5, big])
    lg = rows.to(DEV)
    temp = torch.tensor([0.9, 0.0, 1.2, -1.0], device=DEV)
    k = torch.tensor([40, 40, 0, 3], dtype=torch.int32, device=DEV)
    pp = torch.tensor([0.95, 0.5, 0.8, 0.9], device=DEV)
    seeds = torch.tensor([11, 12, 13, 14], dtype=torch.int64, device=DEV)
    draw = torch.tensor([3, 3, 9, 0], dtype=torch.int32, device=DEV)
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    ops.sample(lg, out, temp, k, pp, seeds, draw)
    together = out.tolist()
    assert together[1] == int(rows[1].argmax()) and together[3] == int(rows[3].argmax())
    for r in (0, 2):
        alone = torch.empty(1, dtype=torch.int32, device=DEV)
        ops.sample(lg[r:r + 1].contiguous(), alone, temp[r:r + 1], k[r:r + 1], pp[r:r + 1], seeds[r:r + 1], draw[r:r + 1])
        assert alone.item() == together[r]
        many = torch.empty(200, dtype=torch.int32, device=DEV)          # 200 rows: fewer blocks to a row
        ops.sample(lg[r:r + 1].expand(200, -1).contiguous(), many, temp[r:r + 1].expand(200).contiguous(),
                   k[r:r + 1].expand(200).contiguous(), pp[r:r + 1].expand(200).contiguous(),
                   seeds[r:r + 1].expand(200).contiguous(), draw[r:r + 1].expand(200).contiguous())
        assert set(many.tolist()) == {together[r]}
    # a row that holds nothing to draw from falls back to index 0, like the greedy choice
    nothing = torch.full((1, 5000), float("-inf"), device=DEV)
    ops.sample(nothing, alone, temp[:1], k[:1], pp[:1], seeds[:1], draw[:1])
    assert alone.item() == 0


def test_argmax_in_two_stages(ops):
    """Ties across and inside the slices of the first stage go to the smallest index; a row of -inf or NaN gives
    index 0; vocabularies that are no multiple of the slice count."""
    for V in (1000, 4097, 151936, 200003):
        lg = torch.zeros(6, V, device=DEV)
        lg[0, V - 1] = 1.0
        lg[1, [V // 3, V // 3 + 1, V - 2]] = 2.0            # the first of three equal maxima
        lg[2, :] = -5.0                                      # all equal: index 0
        lg[3, :] = float("-inf")
        lg[4, :] = float("nan")
        lg[5, [7, V // 2]] = torch.tensor([3.0, 3.0], device=DEV)
        out = torch.full((6,), -1, dtype=torch.int32, device=DEV)
        ops.sample(lg, out)
        assert out.tolist() == [V - 1, V // 3, 0, 0, 0, 7], V


@pytest.mark.parametrize("dtype", DTYPES)
def test_bias_add_and_residual_add(ops, dtype):
    g = torch.Generator().manual_seed(12)
    x = torch.randn(7, 331, generator=g).to(dtype).to(DEV)
    b = torch.randn(331, generator=g).to(DEV)
    want = (x.double() + b.double())
    ops.bias_add(x, b)
    torch.testing.assert_close(x.double(), want, **tol(dtype))
    stream = torch.randn(7, 331, generator=g).to(DEV)
    delta = torch.randn(7, 331, generator=g).to(dtype).to(DEV)
    want = stream.double() + delta.double()
    ops.residual_add(stream, delta)
    torch.testing.assert_close(stream.double(), want, atol=1e-6, rtol=1e-6)   # the sum itself is float


@pytest.mark.parametrize("page_size", [4, 16, 48])
@pytest.mark.parametrize("through_rows", [False, True])
def test_decode_advance(ops, page_size, through_rows):
    """Between two decode steps of one launch: live rows move on by one position, take the token just chosen and
    get their slot from their block table (also across a page's edge, in every cache group; the table's row is
    the batch's row or the one ``table_rows`` names); other rows stay."""
    g = torch.Generator().manual_seed(page_size)
    R, width, live = 9, 6, 6
    pos = torch.tensor([0, page_size - 2, page_size - 1, 2 * page_size - 1, 3 * page_size + 1, 5, 7, 8, 9], dtype=torch.int32)
    rows = torch.randperm(R + 4, generator=g)[:R].to(torch.int32) if through_rows else torch.arange(R, dtype=torch.int32)
    tables = [torch.randint(1, 500, (R + 4 if through_rows else R, width), generator=g, dtype=torch.int32) for _ in range(2)]
    prev = torch.randint(0, 1000, (R,), generator=g, dtype=torch.int32)
    toks = torch.randint(0, 1000, (R,), generator=g, dtype=torch.int32)
    ctx = pos + 1
    slots = [torch.full((R,), -7, dtype=torch.int32) for _ in range(2)]
    dev = lambda t: t.clone().to(DEV)
    d_tok, d_pos, d_ctx, d_slots = dev(toks), dev(pos), dev(ctx), [dev(s_) for s_ in slots]
    draws = torch.arange(10, 10 + R, dtype=torch.int32, device=DEV)
    ops.decode_advance(dev(prev), d_tok, d_pos, d_ctx, torch.tensor([live], dtype=torch.int32, device=DEV),
                       dev(rows) if through_rows else None, [dev(t) for t in tables], d_slots, page_size,
                       draws if through_rows else None)
    assert draws.tolist() == [10 + r + (1 if r < live and through_rows else 0) for r in range(R)]
    for r in range(R):
        if r < live:
            p = int(pos[r]) + 1
            assert (int(d_pos[r]), int(d_ctx[r]), int(d_tok[r])) == (p, p + 1, int(prev[r]))
            for t, sl in zip(tables, d_slots):
                assert int(sl[r]) == int(t[int(rows[r]), p // page_size]) * page_size + p % page_size
        else:
            assert (int(d_pos[r]), int(d_ctx[r]), int(d_tok[r])) == (int(pos[r]), int(ctx[r]), int(toks[r]))
            assert all(int(sl[r]) == -7 for sl in d_slots)


def test_table_update_and_zero_rows(ops):
    """The device's block tables take the entries that changed (counts on the device; an index past the table or
    negative is left alone), and state slots are zeroed by row (as many as a device count says)."""
    g = torch.Generator().manual_seed(4)
    tables = [torch.randint(1, 99, (7, 11), generator=g, dtype=torch.int32) for _ in range(3)]
    want = [t.clone() for t in tables]
    U = 300
    index, value, counts = [], [], []
    for gi, t in enumerate(want):
        n = (0, 40, 77)[gi]
        ix = torch.randperm(77, generator=g)[:n].to(torch.int32)
        v = torch.randint(100, 999, (n,), generator=g, dtype=torch.int32)
        t.view(-1)[ix.long()] = v
        pad_i = torch.full((U - n,), -1, dtype=torch.int32)
        pad_i[:3] = torch.tensor([77, 5000, -9])             # would be out of the table: never written
        index.append(torch.cat([ix, pad_i])); value.append(torch.cat([v, torch.full((U - n,), 12345, dtype=torch.int32)]))
        counts.append(n + (3 if gi == 1 else 0))              # group 1 also counts its three bad indices
    dev_tables = [t.to(DEV) for t in tables]
    ops.table_update(dev_tables, [i.to(DEV) for i in index], [v.to(DEV) for v in value],
                     torch.tensor(counts, dtype=torch.int32, device=DEV), U)
    for got, w in zip(dev_tables, want):
        assert torch.equal(got.cpu(), w)
    for dtype, shape in ((torch.float32, (9, 5, 3)), (torch.bfloat16, (9, 6)), (torch.int32, (9,))):
        t = torch.ones(shape, dtype=dtype, device=DEV)
        rows = torch.tensor([7, 2, 4, 0], dtype=torch.int32, device=DEV)
        ops.zero_rows(t, rows, torch.tensor([3], dtype=torch.int32, device=DEV))
        live = t.reshape(9, -1).float().abs().sum(1).cpu() > 0
        assert live.tolist() == [True, True, False, True, False, True, True, False, True]
        ops.zero_rows(t, rows)
        assert float(t.reshape(9, -1)[0].float().abs().sum()) == 0


def _draws(ops, logits, n, temperature=1.0, top_k=0, top_p=1.0, seed=0):
    M = n
    lg = logits.to(DEV).expand(M, -1).contiguous()
    out = torch.empty(M, dtype=torch.int32, device=DEV)
    ops.sample(lg, out, torch.full((M,), temperature, device=DEV), torch.full((M,), top_k, dtype=torch.int32, device=DEV),
               torch.full((M,), top_p, device=DEV), torch.full((M,), seed, dtype=torch.int64, device=DEV),
               torch.arange(M, dtype=torch.int32, device=DEV))
    return out.cpu()


def test_sample_distribution_and_filters(ops):
    # vectors of the reference's tests/test_sampler.py
    assert set(_draws(ops, torch.tensor([[0.1, 2.0, 0.5]]), 20, top_k=1).tolist()) == {1}
    assert set(_draws(ops, torch.tensor([[2.0, 1.0, 0.0, -1.0]]), 300, top_p=0.7).tolist()) == {0, 1}
    assert set(_draws(ops, torch.tensor([[10.0, 0.0, 0.0]]), 50, top_p=1e-4).tolist()) == {0}
    d = _draws(ops, torch.log(torch.tensor([[0.7, 0.2, 0.1]])), 4000, seed=123)
    freq = torch.bincount(d, minlength=3).float() / 4000
    assert torch.allclose(freq, torch.tensor([0.7, 0.2, 0.1]), atol=0.03)
    # temperature sharpens: T = 0.5 squares the odds
    d = _draws(ops, torch.log(torch.tensor([[0.5, 0.5 / 3]])), 4000, temperature=0.5, seed=5)
    assert abs((d == 0).float().mean().item() - 0.9) < 0.03
    # same seed and draw index, same token; top-k = 2 on a wide row leaves two tokens
    row = torch.randn(1, 5000, generator=torch.Generator().manual_seed(8))
    a, b = _draws(ops, row, 64, seed=9), _draws(ops, row, 64, seed=9)
    assert torch.equal(a, b) and len(set(a.tolist())) > 10
    top2 = set(row[0].topk(2).indices.tolist())
    assert set(_draws(ops, row, 200, top_k=2, seed=1).tolist()) == top2


def test_ops_refuse_cpu_tensors_and_wrong_shapes(ops):
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.silu_mul(torch.zeros(2, 4), torch.zeros(2, 2))
    with pytest.raises(ValueError):
        ops.silu_mul(torch.zeros(2, 4, device=DEV), torch.zeros(2, 3, device=DEV))
    with pytest.raises(RuntimeError, match="unsupported"):
        kp = torch.zeros(2, 1, 4, 6, device=DEV)  # head size 6 is no multiple of 4
        ops.paged_attention_generic(torch.zeros(1, 6, device=DEV), kp, kp, torch.zeros(1, 1, dtype=torch.int32, device=DEV),
                                    torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV),
                                    torch.zeros(1, 6, device=DEV), 1, 1.0)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(1152, 896), (331, 72), (896, 4864), (50, 200), (9728, 104), (17000, 64)])
def test_gemm_skinny(ops, M, N, K):
    g = torch.Generator().manual_seed(M * 1000 + N)
    a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    want = a.double() @ w.double().T
    out = ops.gemm_skinny(a, w, bias)
    torch.testing.assert_close(out.double(), want + bias.double(), **tol(torch.bfloat16))
    f = ops.gemm_skinny(a, w, None, out_dtype=torch.float32)
    assert f.dtype == torch.float32
    torch.testing.assert_close(f.double(), want, atol=2e-5, rtol=2e-5)
    x = torch.randn(M, N, generator=g).to(DEV)
    x0 = x.clone()
    ops.gemm_skinny(a, w, bias, ops.EPI_RESIDUAL, residual=x)
    torch.testing.assert_close(x.double(), x0.double() + want + bias.double(), atol=2e-5, rtol=2e-5)
    if N % 2 == 0:
        act = ops.gemm_skinny(a, w, None, ops.EPI_SWIGLU)
        wantact = torch.nn.functional.silu(want[:, 0::2]) * want[:, 1::2]
        torch.testing.assert_close(act.double(), wantact, **tol(torch.bfloat16))
    # a row slice of a wider matrix, and the same row alone: the same bits whatever else is in the batch
    wide = torch.zeros(M, K + 8, dtype=torch.bfloat16, device=DEV)
    wide[:, :K] = a
    assert torch.equal(ops.gemm_skinny(wide[:, :K], w, bias), out)
    assert torch.equal(ops.gemm_skinny(a[M - 1:], w, bias), out[M - 1:])


@pytest.mark.parametrize("M", [3, 40])
@pytest.mark.parametrize("shape", [(4, 4, 0), (4, 8, 0), (3, 4, 0), (3, 8, 0), (2, 8, 0), (2, 16, 0), (1, 8, 0), (1, 16, 0),
                                   (4, 8, 1), (3, 8, 1), (2, 8, 2)])
def test_gemm_skinny_block_shapes(ops, M, shape):
    """Every block shape on offer (tiles per block, waves, token groups per block) gives the same numbers (to
    float rounding of another summation order), also with the gated epilogue and the folded norm.  A forced
    shape also keeps few rows in this kernel; unforced they go to the streaming kernel, which must agree."""
    from llm_infrence_engine_amd.kernels import build

    lib = build.load()
    g = torch.Generator().manual_seed(sum(shape) + M)
    N, K = 1000, 1544
    a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    want = a.double() @ w.double().T + bias.double()
    x0 = torch.randn(M, N, generator=g).to(DEV)
    try:
        lib.ms_gemm_skinny_force(*shape)
        x = x0.clone()
        try:
            ops.gemm_skinny(a, w, bias, ops.EPI_RESIDUAL, residual=x)
        except RuntimeError as e:      # a shape that does not fit LDS with this many token groups is refused
            assert "unsupported" in str(e) and (shape[1] - 1) * shape[0] * (shape[2] or (1 if M <= 16 else 4)) > 60
            return
        torch.testing.assert_close(x.double(), x0.double() + want, atol=3e-5, rtol=3e-5)
        f = ops.gemm_skinny(a, w, bias, out_dtype=torch.float32)
        torch.testing.assert_close(f.double(), want, atol=3e-5, rtol=3e-5)
        # gated epilogue over interleaved rows, norm folded in: against the default shape
        x32 = torch.randn(M, K, generator=g).to(DEV)
        nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
        got = ops.gemm_skinny_norm(x32, nw, 1e-6, w, None, ops.EPI_SWIGLU)
        lib.ms_gemm_skinny_force(0, 0, 0)
        ref = ops.gemm_skinny_norm(x32, nw, 1e-6, w, None, ops.EPI_SWIGLU)
        torch.testing.assert_close(got.double(), ref.double(), atol=1e-2, rtol=1e-2)
    finally:
        lib.ms_gemm_skinny_force(0, 0, 0)


@pytest.mark.parametrize("M", [1, 5, 8, 16])
@pytest.mark.parametrize("N,K", [(896, 4864), (1152, 896), (330, 72), (52, 200), (9728, 904), (1000, 9000), (4000, 2056),
                                 (16384, 64)])
def test_gemm_stream(ops, M, N, K):
    """The streaming kernel at every shape it can compute: one or several stages, a last k-step that K fills in
    part, one to four tiles of rows to a block, rows that run out in the last block; every epilogue, the folded
    norm with gathered rows; a row's numbers do not depend on the rest of the batch."""
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    want = a.double() @ w.double().T
    out = ops.gemm_stream(a, w, bias)
    torch.testing.assert_close(out.double(), want + bias.double(), **tol(torch.bfloat16))
    f = ops.gemm_stream(a, w, None, out_dtype=torch.float32)
    torch.testing.assert_close(f.double(), want, atol=3e-5, rtol=3e-5)
    x = torch.randn(M, N, generator=g).to(DEV)
    x0 = x.clone()
    ops.gemm_stream(a, w, bias, ops.EPI_RESIDUAL, residual=x)
    torch.testing.assert_close(x.double(), x0.double() + want + bias.double(), atol=3e-5, rtol=3e-5)
    act = ops.gemm_stream(a, w, None, ops.EPI_SWIGLU)
    torch.testing.assert_close(act.double(), torch.nn.functional.silu(want[:, 0::2]) * want[:, 1::2], **tol(torch.bfloat16))
    assert torch.equal(ops.gemm_stream(a[M - 1:], w, bias), out[M - 1:])
    # the folded norm over gathered rows of a taller residual stream
    xs = torch.randn(M + 3, K, generator=g).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
    rows = torch.randperm(M + 3, generator=g)[:M].to(torch.int32).to(DEV)
    xr = xs[rows.long()].double()
    h = (xr * nw.double()).float().bfloat16().double() * torch.rsqrt((xr * xr).mean(-1, keepdim=True) + 1e-5)
    got = ops.gemm_stream(xs, w, bias, out_dtype=torch.float32, norm_weight=nw, eps=1e-5, rows=rows)
    torch.testing.assert_close(got.double(), h @ w.double().T + bias.double(), atol=2e-4, rtol=2e-4)
    gated = ops.gemm_stream(xs, w, None, ops.EPI_SWIGLU, norm_weight=nw, eps=1e-5, rows=rows)
    hw = h @ w.double().T
    torch.testing.assert_close(gated.double(), torch.nn.functional.silu(hw[:, 0::2]) * hw[:, 1::2], **tol(torch.bfloat16))


def test_gemm_stream_refuses_what_it_cannot_take(ops):
    w = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="unsupported"):
        ops.gemm_stream(torch.zeros(17, 64, dtype=torch.bfloat16, device=DEV), w)            # more than 16 rows
    with pytest.raises(RuntimeError, match="unsupported"):
        ops.gemm_stream(torch.zeros(2, 36, dtype=torch.bfloat16, device=DEV),
                        torch.zeros(8, 36, dtype=torch.bfloat16, device=DEV))                 # K no multiple of 8
    with pytest.raises(RuntimeError, match="unsupported"):                                   # not the shape it is for
        ops.gemm_stream(torch.zeros(2, 64, dtype=torch.bfloat16, device=DEV), w, any_shape=False)


@pytest.mark.parametrize("M", [17, 32, 41, 64])
@pytest.mark.parametrize("N,K", [(7000, 96), (4100, 200), (330, 256), (48, 896), (16 * 256 * 17 + 6, 64), (1000, 1000)])
def test_gemm_panel(ops, M, N, K):
    """The kernel that holds the activations in LDS, at every shape it can compute: blocks of one tile, of a few
    tiles whose k-steps several waves share, and of more tiles than waves; a last k-step that K fills in part;
    rows of W that run out inside the last tile; every epilogue, the folded norm with gathered rows; a row's
    numbers do not depend on the rest of the batch."""
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    want = a.double() @ w.double().T
    out = ops.gemm_panel(a, w, bias)
    torch.testing.assert_close(out.double(), want + bias.double(), **tol(torch.bfloat16))
    f = ops.gemm_panel(a, w, None, out_dtype=torch.float32)
    torch.testing.assert_close(f.double(), want, atol=3e-5, rtol=3e-5)
    x = torch.randn(M, N, generator=g).to(DEV)
    x0 = x.clone()
    ops.gemm_panel(a, w, bias, ops.EPI_RESIDUAL, residual=x)
    torch.testing.assert_close(x.double(), x0.double() + want + bias.double(), atol=3e-5, rtol=3e-5)
    act = ops.gemm_panel(a, w, None, ops.EPI_SWIGLU)
    torch.testing.assert_close(act.double(), torch.nn.functional.silu(want[:, 0::2]) * want[:, 1::2], **tol(torch.bfloat16))
    assert torch.equal(ops.gemm_panel(a[M - 3:], w, bias), out[M - 3:])
    # the folded norm over gathered rows of a taller residual stream
    xs = torch.randn(M + 3, K, generator=g).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
    rows = torch.randperm(M + 3, generator=g)[:M].to(torch.int32).to(DEV)
    xr = xs[rows.long()].double()
    h = (xr * nw.double()).float().bfloat16().double() * torch.rsqrt((xr * xr).mean(-1, keepdim=True) + 1e-5)
    got = ops.gemm_panel(xs, w, bias, out_dtype=torch.float32, norm_weight=nw, eps=1e-5, rows=rows)
    torch.testing.assert_close(got.double(), h @ w.double().T + bias.double(), atol=2e-4, rtol=2e-4)
    gated = ops.gemm_panel(xs, w, None, ops.EPI_SWIGLU, norm_weight=nw, eps=1e-5, rows=rows)
    hw = h @ w.double().T
    torch.testing.assert_close(gated.double(), torch.nn.functional.silu(hw[:, 0::2]) * hw[:, 1::2], **tol(torch.bfloat16))


@pytest.mark.parametrize("M,N,K", [(20, 300, 1200), (33, 4100, 1528), (18, 500, 2040),
                                   (64, 4300, 3584), (40, 700, 5120), (64, 4096 + 16 * 256 * 2, 2600), (17, 90, 4872),
                                   (50, 16 * 256 * 33 + 40, 2400), (40, 16 * 256 * 50, 1840)])
def test_gemm_panel_long_rows(ops, M, N, K):
    """Rows of three and four 512-column parts (with three a quarter of the waves sit the loading out), and rows
    that do not fit LDS whole and go through it in chunks: a last chunk that is shorter, blocks with whole and
    shared tiles, two and three whole tiles to a wave."""
    g = torch.Generator().manual_seed(K)
    xs = torch.randn(M, K, generator=g).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
    h = (xs.double() * nw.double()).float().bfloat16().double() * torch.rsqrt((xs.double() ** 2).mean(-1, keepdim=True) + 1e-6)
    got = ops.gemm_panel(xs, w, None, out_dtype=torch.float32, norm_weight=nw, eps=1e-6)
    torch.testing.assert_close(got.double(), h @ w.double().T, atol=2e-4, rtol=2e-4)
    a = xs.bfloat16()
    plain = ops.gemm_panel(a, w, None, out_dtype=torch.float32)
    torch.testing.assert_close(plain.double(), a.double() @ w.double().T, atol=3e-5, rtol=3e-5)


@pytest.mark.parametrize("M,N,K", [(8, 5120, 13824), (64, 3584, 18944), (33, 5120, 27648), (17, 900, 8200), (64, 16, 9000),
                                   (5, 8192, 16384), (64, 3584, 3584), (40, 4608, 3584), (64, 7168, 5120), (33, 3100, 3080)])
def test_gemm_with_the_columns_split_over_blocks(ops, M, N, K):
    """Long rows against few of them: blocks take parts of the columns, a second kernel adds the partial sums in
    order.  Every epilogue that has no gate; a row's numbers do not depend on the rest of the batch; parts of
    uneven length, a vocabulary-free odd N, one tile only."""
    from llm_infrence_engine_amd.kernels import build
    assert build.load().ms_gemm_panel_splitk_parts(M, N, K) > 1
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    want = a.double() @ w.double().T
    out = ops.gemm_skinny(a, w, bias)
    torch.testing.assert_close(out.double(), want + bias.double(), **tol(torch.bfloat16))
    f = ops.gemm_skinny(a, w, None, out_dtype=torch.float32)
    torch.testing.assert_close(f.double(), want, atol=5e-5, rtol=5e-5)
    x = torch.randn(M, N, generator=g).to(DEV)
    x0 = x.clone()
    ops.gemm_skinny(a, w, bias, ops.EPI_RESIDUAL, residual=x)
    torch.testing.assert_close(x.double(), x0.double() + want + bias.double(), atol=5e-5, rtol=5e-5)
    assert torch.equal(ops.gemm_skinny(a[M - 1:], w, bias), out[M - 1:]) or M > 16   # the same kernel for one row
    unsplit = ops.gemm_skinny(a, w, None, out_dtype=torch.float32, split_columns=False)
    torch.testing.assert_close(unsplit.double(), want, atol=5e-5, rtol=5e-5)


def test_columns_are_split_only_where_it_pays(ops):
    from llm_infrence_engine_amd.kernels import build
    parts = build.load().ms_gemm_panel_splitk_parts
    assert parts(8, 896, 4864) == 0          # rows too short
    assert parts(8, 3584, 18944) == 0        # few tokens and a tile for nearly every CU: as well unsplit
    assert parts(8, 37888, 3584) == 0        # and here, with tiles enough for every CU besides
    assert parts(65, 3584, 18944) == 0       # too many tokens
    assert parts(8, 16384, 18944) == 0       # more than two tiles per CU
    assert parts(64, 3584, 3584) == 4 and parts(64, 5120, 5120) == 4   # shorter rows: only with more than 32 tokens ...
    assert parts(32, 3584, 3584) == 0 and parts(64, 2048, 2048) == 0 and parts(64, 896, 4864) == 0   # ... long enough, and a tile to most CUs


def test_gemm_panel_refuses_what_it_cannot_take(ops):
    w = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="unsupported"):
        ops.gemm_panel(torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV), w)             # more than 64 rows
    with pytest.raises(RuntimeError, match="unsupported"):           # in chunks, and too many tiles to a block
        ops.gemm_panel(torch.zeros(64, 2400, dtype=torch.bfloat16, device=DEV),
                       torch.zeros(16 * 256 * 48, 2400, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(RuntimeError, match="unsupported"):                                   # not the shape it is for
        ops.gemm_panel(torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV), w, any_shape=False)


def test_gemm_skinny_refuses_what_it_cannot_take(ops):
    a = torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError, match="at most 64 rows"):
        ops.gemm_skinny(a, w)
    with pytest.raises(ValueError, match="multiple of 8"):
        ops.gemm_skinny(a[:4, :60], w[:, :60].contiguous())


@pytest.mark.parametrize("tile", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("M,N,K", [(65, 662, 64), (300, 2 * 331, 192), (257, 130, 896), (1000, 2 * 4864, 896), (2051, 1026, 128),
                                   (130, 16, 64), (513, 4100, 1536), (4100, 2 * 331, 64), (6200, 1300, 128)])
def test_gemm_tiled(ops, M, N, K, tile):
    """The many-rows product and its gated epilogue with every tile shape (256, 128, 64, 192 and 160 features wide:
    the last two store a lane's results in pieces of 8 and 4 bytes): rows and features that fill no whole tile, rows
    of the result that start at odd addresses, one step of 64 columns and many, and so many tokens that the tiles are
    laid over the XCDs in two and in four rows."""
    force = ops._get("ms_gemm_tiled_force")
    force.restype = None
    g = torch.Generator().manual_seed(M + N)
    a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    a[M - 1] *= 3.0                                        # the last row is told apart from a repeated one before it
    want = a.double() @ w.double().T
    force(tile)
    try:
        out = ops.gemm_tiled(a, w)
        act = ops.gemm_tiled(a, w, ops.EPI_SWIGLU)
    finally:
        force(0)
    assert out.shape == (M, N) and act.shape == (M, N // 2) and out.dtype == act.dtype == torch.bfloat16
    torch.testing.assert_close(out.double(), want, **tol(torch.bfloat16))
    torch.testing.assert_close(act.double(), torch.nn.functional.silu(want[:, 0::2]) * want[:, 1::2], **tol(torch.bfloat16))
    # a row's result does not depend on what else is in the batch
    assert torch.equal(ops.gemm_tiled(a[M - 70:], w), out[M - 70:])


def test_gemm_tiled_refuses_what_it_cannot_take_and_linear_goes_on(ops):
    from llm_infrence_engine_amd.kernels import linear

    g = torch.Generator().manual_seed(5)
    a = torch.randn(100, 72, generator=g).bfloat16().to(DEV)
    w = (torch.randn(60, 72, generator=g) / 8).bfloat16().to(DEV)
    with pytest.raises(ops.UnsupportedShape):
        ops.gemm_tiled(a, w)                               # 72 columns: no multiple of 64
    assert not ops.gemm_tiled_pays(a, w)
    with pytest.raises(TypeError):
        ops.gemm_tiled(a.float(), w)
    # the dispatcher: wide enough rows of a narrow model go to the tiled kernel, others to the library
    a2 = torch.randn(200, 128, generator=g).bfloat16().to(DEV)
    w2 = (torch.randn(96, 128, generator=g) / 11).bfloat16().to(DEV)
    assert ops.gemm_tiled_pays(a2, w2)
    got = linear.linear_swiglu(a2, w2)
    ref = a2.double() @ w2.double().T
    torch.testing.assert_close(got.double(), torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2], **tol(torch.bfloat16))
    assert torch.equal(got, ops.gemm_tiled(a2, w2, ops.EPI_SWIGLU))
    assert linear.fallback_count() == 0 or all(k[3] != "tiled gated product" for k in linear.fallbacks)


def test_linear_picks_a_kernel_for_every_shape(ops):
    from llm_infrence_engine_amd.kernels import linear

    g = torch.Generator().manual_seed(11)
    for dtype in DTYPES:
        for M, N, K in [(3, 40, 72), (100, 40, 72), (200, 331, 120), (5, 33, 60), (70, 33, 60)]:
            a = torch.randn(M, K, generator=g).to(dtype).to(DEV)
            w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype).to(DEV)
            b = torch.randn(N, generator=g).to(DEV)
            want = a.double() @ w.double().T + b.double()
            torch.testing.assert_close(linear.linear(a, w, b).double(), want, **tol(dtype))
            lg = linear.linear(a, w, b, out_dtype=torch.float32)
            assert lg.dtype == torch.float32
            torch.testing.assert_close(lg.double(), want, **(tol(torch.float32) if dtype == torch.float32 or M <= 64 else tol(dtype)))
            x = torch.randn(M, N, generator=g).to(DEV)
            x0 = x.clone()
            r = linear.linear_residual(a, w, b, x)
            got = x.double() - x0.double() if r is None else r.double()
            assert (r is None) == (dtype == torch.bfloat16 and M <= 64 and K % 8 == 0)
            torch.testing.assert_close(got, want, **tol(dtype))
        for M in (4, 90):
            a = torch.randn(M, 72, generator=g).to(dtype).to(DEV)
            gate = (torch.randn(50, 72, generator=g) / 8).to(dtype).to(DEV)
            up = (torch.randn(50, 72, generator=g) / 8).to(dtype).to(DEV)
            got = linear.linear_swiglu(a, linear.interleave_rows(gate, up))
            want = torch.nn.functional.silu(a.double() @ gate.double().T) * (a.double() @ up.double().T)
            torch.testing.assert_close(got.double(), want, **tol(dtype))


def _paged_case(g, dtype, nh, nkv, d, page_size, ctx, qlen, fill):
    """Random requests laid out in shuffled pages (values transposed); returns what the kernels take and
    the plain answer.  Unused slots, the tails of last pages and the null page hold ``fill``."""
    R = len(ctx)
    pages_per = [-(-c // page_size) for c in ctx]
    P = sum(pages_per) + 4
    order = torch.randperm(P - 1, generator=g) + 1
    kp = torch.full((P, nkv, page_size, d), fill, dtype=dtype)
    vt = torch.full((P, nkv, d, page_size), fill, dtype=dtype)
    table = torch.zeros(R, max(pages_per), dtype=torch.int32)
    qs, ks, vs, q_rows, req, pos = [], [], [], [], [], []
    used = 0
    for r in range(R):
        k = torch.randn(nkv, ctx[r], d, generator=g).to(dtype)
        v = torch.randn(nkv, ctx[r], d, generator=g).to(dtype)
        q = (torch.randn(nh, qlen[r], d, generator=g) * 2).to(dtype)
        k[:, min(3, ctx[r] - 1)] = (q[::nh // nkv, -1].float() * 1.5).to(dtype)   # one far key stands out
        pages = order[used:used + pages_per[r]]
        used += pages_per[r]
        table[r, :pages_per[r]] = pages.to(torch.int32)
        for j in range(ctx[r]):
            kp[pages[j // page_size], :, j % page_size] = k[:, j]
            vt[pages[j // page_size], :, :, j % page_size] = v[:, j]
        qs.append(q); ks.append(k); vs.append(v)
        q_rows.append(q.transpose(0, 1).reshape(qlen[r], nh * d))
        req += [r] * qlen[r]
        pos += list(range(ctx[r] - qlen[r], ctx[r]))
    return dict(kp=kp, vt=vt, table=table, q=torch.cat(q_rows), req=req, pos=pos, qs=qs, ks=ks, vs=vs)


@pytest.mark.parametrize("nh,nkv,d,page_size,window", [(14, 2, 64, 16, None), (6, 2, 32, 16, None), (8, 8, 128, 32, None),
                                                        (4, 1, 64, 16, 40), (28, 4, 128, 16, None), (5, 5, 32, 64, 100),
                                                        (6, 2, 64, 48, None)])
@pytest.mark.parametrize("shape", ["mixed", "decode", "long"])
def test_paged_attention_mfma(ops, nh, nkv, d, page_size, window, shape):
    g = torch.Generator().manual_seed(nh * 100 + d)
    if shape == "mixed":
        ctx, qlen = [70, 133, 201, 300], [70, 9, 1, 150]
    elif shape == "decode":
        ctx, qlen = [1, 31, 32, 33, 600, 1000, 64, 17], [1] * 8
    else:   # few requests with long contexts: keys split over blocks and combined
        ctx, qlen = [2500, 1, 300], [1] * 3
    c = _paged_case(g, torch.bfloat16, nh, nkv, d, page_size, ctx, qlen, float("nan"))
    scale = 1.0 / math.sqrt(d)
    assert ops.attention_splits_keys(len(ctx), nkv, nh // nkv, max(qlen), max(ctx)) == (shape == "long")
    want = torch.cat([attention_reference(q.double(), k.double(), v.double(), scale, window).transpose(0, 1).reshape(-1, nh * d)
                      for q, k, v in zip(c["qs"], c["ks"], c["vs"])])
    N = c["q"].shape[0]
    wide = torch.zeros(N, (nh + 2 * nkv) * d, dtype=torch.bfloat16, device=DEV)
    wide[:, :nh * d] = c["q"].to(DEV)
    out = torch.full((N, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    q_start = torch.tensor([0] + list(np.cumsum(qlen)), dtype=torch.int32, device=DEV)
    ops.paged_attention_mfma(wide, c["kp"].to(DEV), c["vt"].to(DEV), c["table"].to(DEV), q_start,
                             torch.tensor(ctx, dtype=torch.int32, device=DEV), out, nh, scale, max(qlen), max(ctx), window)
    torch.testing.assert_close(out.double().cpu(), want, **tol(torch.bfloat16))
    # the generic kernel reads the same transposed pages
    out2 = torch.empty_like(out)
    ops.paged_attention_generic(wide, c["kp"].to(DEV), c["vt"].to(DEV), c["table"].to(DEV),
                                torch.tensor(c["req"], dtype=torch.int32, device=DEV),
                                torch.tensor(c["pos"], dtype=torch.int32, device=DEV), out2, nh, scale, window, v_transposed=True)
    torch.testing.assert_close(out2.double().cpu(), want, **tol(torch.bfloat16))


@pytest.mark.parametrize("nh,nkv,d,page_size,window", [(14, 2, 64, 16, None), (6, 2, 32, 16, 50), (8, 2, 128, 32, None)])
@pytest.mark.parametrize("shape", ["mixed", "decode", "long", "many"])
def test_attention_of_a_padded_batch_through_table_rows(ops, nh, nkv, d, page_size, window, shape):
    """A batch as a captured graph sees it: the block table has a row per request the engine can hold and the
    step's requests name theirs; requests without tokens or keys pad the batch, tokens past the last request's
    belong to nobody and their output rows are left alone; the launch is sized for more and longer portions
    than there are.  Matrix-core and generic kernels alike."""
    g = torch.Generator().manual_seed(nh + d)
    if shape == "mixed":
        ctx, qlen = [70, 133, 201, 300], [70, 9, 1, 150]
    elif shape == "decode":
        ctx, qlen = [1, 31, 600, 1000, 64], [1] * 5
    elif shape == "long":
        ctx, qlen = [2500, 1, 300], [1] * 3
    else:   # more requests than a wave has lanes, most of them short portions: the tile search goes round twice
        ctx = [int(v) for v in torch.randint(5, 90, (70,), generator=g)]
        qlen = [min(c, int(v)) for c, v in zip(ctx, torch.randint(1, 6, (70,), generator=g))]
        qlen[40] = ctx[40] = 77
    c = _paged_case(g, torch.bfloat16, nh, nkv, d, page_size, ctx, qlen, float("nan"))
    scale = 1.0 / math.sqrt(d)
    want = torch.cat([attention_reference(q.double(), k.double(), v.double(), scale, window).transpose(0, 1).reshape(-1, nh * d)
                      for q, k, v in zip(c["qs"], c["ks"], c["vs"])])
    R, N = len(ctx), c["q"].shape[0]
    pad_r, pad_n = 3, (0 if shape in ("decode", "long") else 45)       # a decode graph pads requests, not tokens
    if shape in ("decode", "long"):
        pad_n = pad_r                                                    # ... each padding request's row is a padding token
    rows_total = R + pad_r + 2
    perm = torch.randperm(rows_total - 1, generator=g)[:R]              # the last row stays all null pages
    table = torch.zeros(rows_total, c["table"].shape[1] + 3, dtype=torch.int32)
    table[perm, :c["table"].shape[1]] = c["table"]
    table_rows = torch.cat([perm.to(torch.int32), torch.full((pad_r,), rows_total - 1, dtype=torch.int32)]).to(DEV)
    q = torch.full((N + pad_n, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    q[:N] = c["q"].to(DEV)
    q_start = torch.tensor([0] + list(np.cumsum(qlen)) + [N] * pad_r, dtype=torch.int32, device=DEV)
    ctx_all = torch.tensor(ctx + [0] * pad_r, dtype=torch.int32, device=DEV)
    room = table.shape[1] * page_size                                   # what a request's table row can hold
    cap_q = max(qlen) if shape in ("decode", "long") else min(N + pad_n, room)
    cap_ctx = room
    out = torch.full((N + pad_n, nh * d), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.paged_attention_mfma(q, c["kp"].to(DEV), c["vt"].to(DEV), table.to(DEV), q_start, ctx_all, out, nh, scale,
                             cap_q, cap_ctx, window, table_rows)
    torch.testing.assert_close(out[:N].double().cpu(), want, **tol(torch.bfloat16))
    assert (out[N:] == 7.0).all()
    out2 = torch.full_like(out, 7.0)
    req = torch.tensor(c["req"] + [R + pad_r - 1] * pad_n, dtype=torch.int32, device=DEV)
    pos = torch.tensor(c["pos"] + [0] * pad_n, dtype=torch.int32, device=DEV)
    ops.paged_attention_generic(q, c["kp"].to(DEV), c["vt"].to(DEV), table.to(DEV), req, pos, out2, nh, scale, window,
                                v_transposed=True, table_rows=table_rows, n_live_tokens=q_start[R + pad_r:R + pad_r + 1])
    torch.testing.assert_close(out2[:N].double().cpu(), want, **tol(torch.bfloat16))
    assert (out2[N:] == 7.0).all()


@pytest.mark.parametrize("R,nh,nkv,d,window", [(40, 6, 2, 64, None), (64, 4, 2, 32, None), (21, 8, 4, 128, 700)])
def test_split_decode_attention_of_a_large_uneven_batch(ops, R, nh, nkv, d, window):
    """Many requests whose contexts differ widely, some far beyond the length from which keys are split over
    blocks: few splits per request (a number that is no power of two), short requests that use one of them."""
    g = torch.Generator().manual_seed(R)
    ctx = [int(v) for v in torch.randint(1, 1500, (R,), generator=g)]
    ctx[3], ctx[R - 1] = 2300, 1
    qlen = [1] * R
    assert ops.attention_splits_keys(R, nkv, nh // nkv, 1, max(ctx))
    c = _paged_case(g, torch.bfloat16, nh, nkv, d, 16, ctx, qlen, float("nan"))
    want = torch.cat([attention_reference(q.double(), k.double(), v.double(), 1.0 / math.sqrt(d), window).transpose(0, 1).reshape(-1, nh * d)
                      for q, k, v in zip(c["qs"], c["ks"], c["vs"])])
    torch.testing.assert_close(_run_mfma(ops, c, nh, d, ctx, qlen, window), want, **tol(torch.bfloat16))


@pytest.mark.parametrize("longest,splits_window", [(17000, None), (70000, None), (70000, 30000)])
def test_split_decode_attention_of_very_long_contexts(ops, longest, splits_window):
    """Tens of thousands of keys: more splits than at a few thousand (32 and 128), beside a short request that
    uses one of them."""
    nh, nkv, d = 4, 2, 64
    g = torch.Generator().manual_seed(longest)
    ctx, qlen = [longest, 40], [1, 1]
    c = _paged_case(g, torch.bfloat16, nh, nkv, d, 16, ctx, qlen, float("nan"))
    want = torch.cat([attention_reference(q.double(), k.double(), v.double(), 1.0 / math.sqrt(d), splits_window).transpose(0, 1).reshape(-1, nh * d)
                      for q, k, v in zip(c["qs"], c["ks"], c["vs"])])
    torch.testing.assert_close(_run_mfma(ops, c, nh, d, ctx, qlen, splits_window), want, **tol(torch.bfloat16))


@pytest.mark.parametrize("nh,nkv,d,window", [(4, 2, 64, None), (2, 1, 128, None), (4, 4, 32, None), (4, 2, 64, 700)])
def test_prompt_attention_of_thousands_of_tokens(ops, nh, nkv, d, window):
    """A whole prompt of 3,300 tokens in one step (more column tiles than CUs, late tiles first, every wave of a
    block many key blocks deep) beside a portion of 1,500 tokens behind a prefix of 1,100, with a far key that
    stands out for the last query of each."""
    g = torch.Generator().manual_seed(d + nh)
    ctx, qlen = [3300, 2600], [3300, 1500]
    c = _paged_case(g, torch.bfloat16, nh, nkv, d, 16, ctx, qlen, float("nan"))
    scale = 1.0 / math.sqrt(d)
    want = torch.cat([attention_reference(q.double(), k.double(), v.double(), scale, window).transpose(0, 1).reshape(-1, nh * d)
                      for q, k, v in zip(c["qs"], c["ks"], c["vs"])])
    torch.testing.assert_close(_run_mfma(ops, c, nh, d, ctx, qlen, window), want, **tol(torch.bfloat16))


def _run_mfma(ops, c, nh, d, ctx, qlen, window=None):
    N = c["q"].shape[0]
    out = torch.full((N, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    q_start = torch.tensor([0] + list(np.cumsum(qlen)), dtype=torch.int32, device=DEV)
    ops.paged_attention_mfma(c["q"].to(DEV), c["kp"].to(DEV), c["vt"].to(DEV), c["table"].to(DEV), q_start,
                             torch.tensor(ctx, dtype=torch.int32, device=DEV), out, nh, 1.0 / math.sqrt(d), max(qlen),
                             max(ctx), window)
    return out.double().cpu()


@pytest.mark.parametrize("d,shape", [(32, (4, 4, 1)), (32, (2, 4, 1)), (32, (2, 8, 1)), (32, (1, 8, 1)), (32, (1, 16, 1)),
                                     (64, (4, 4, 1)), (64, (2, 4, 1)), (64, (2, 8, 1)), (64, (1, 4, 1)), (64, (1, 8, 1)),
                                     (64, (1, 16, 1)), (128, (2, 4, 1)), (128, (1, 4, 1)), (128, (1, 8, 1)),
                                     (32, (1, 16, 2)), (64, (1, 16, 2)), (64, (1, 16, 4)), (64, (1, 8, 2)), (64, (1, 8, 4)),
                                     (128, (1, 8, 2)), (128, (1, 8, 4))])
def test_attention_mfma_tile_shapes(ops, d, shape):
    """Every tile width, wave count and number of blocks to a narrow tile on the menu gives the same answer (the
    choice by size picks among them)."""
    from llm_infrence_engine_amd.kernels import build
    nh, nkv = 6, 2
    g = torch.Generator().manual_seed(d + shape[0] * 7 + shape[1] + shape[2] * 1000)
    ctx, qlen = [300, 97, 520], [130, 1, 45]
    c = _paged_case(g, torch.bfloat16, nh, nkv, d, 16, ctx, qlen, float("nan"))
    want = torch.cat([attention_reference(q.double(), k.double(), v.double(), 1.0 / math.sqrt(d), None).transpose(0, 1).reshape(-1, nh * d)
                      for q, k, v in zip(c["qs"], c["ks"], c["vs"])])
    lib = build.load()
    lib.ms_attention_mfma_force(*shape)
    try:
        got = _run_mfma(ops, c, nh, d, ctx, qlen)
    finally:
        lib.ms_attention_mfma_force(0, 0, 0)
    torch.testing.assert_close(got, want, **tol(torch.bfloat16))


@pytest.mark.parametrize("ramp", [0.5, 6.0, 60.0])
def test_attention_mfma_when_the_maximum_keeps_rising(ops, ramp):
    """Scores that grow along the context by ``ramp`` log2 units in all: the running reference of the softmax
    stays (small ramp), moves once or moves at almost every block, and late keys dwarf the early ones."""
    nh, nkv, d = 4, 2, 64
    g = torch.Generator().manual_seed(int(ramp * 10))
    ctx, qlen = [640, 333], [200, 1]
    c = _paged_case(g, torch.bfloat16, nh, nkv, d, 16, ctx, qlen, float("nan"))
    scale = 1.0 / math.sqrt(d)
    # all queries share a direction u; key j carries (j / ctx) * ramp * ln2 / scale along it
    u = torch.zeros(d); u[5] = 1.0
    for r in range(len(ctx)):
        c["qs"][r] = (c["qs"][r].float() * 0.05 + u).to(torch.bfloat16)
        steps = torch.arange(ctx[r]).float() / ctx[r] * ramp * math.log(2.0) / scale
        c["ks"][r] = (c["ks"][r].float() * 0.05 + steps[None, :, None] * u).to(torch.bfloat16)
    # lay the changed keys and queries out again
    rows, p = [], 0
    for r in range(len(ctx)):
        for j in range(ctx[r]):
            c["kp"][c["table"][r, j // 16].item(), :, j % 16] = c["ks"][r][:, j]
        rows.append(c["qs"][r].transpose(0, 1).reshape(qlen[r], nh * d))
    c["q"] = torch.cat(rows)
    want = torch.cat([attention_reference(q.double(), k.double(), v.double(), scale, None).transpose(0, 1).reshape(-1, nh * d)
                      for q, k, v in zip(c["qs"], c["ks"], c["vs"])])
    got = _run_mfma(ops, c, nh, d, ctx, qlen)
    torch.testing.assert_close(got, want, **tol(torch.bfloat16))


def test_attention_mfma_support_matrix(ops):
    assert ops.attention_mfma_supported(64, 16) and ops.attention_mfma_supported(128, 32)
    assert not ops.attention_mfma_supported(48, 16) and not ops.attention_mfma_supported(64, 8)


@pytest.mark.parametrize("M", [1, 8, 33, 64])
@pytest.mark.parametrize("N,K", [(1152, 896), (330, 72), (50, 200)])
def test_gemm_skinny_with_the_norm_folded_in(ops, M, N, K):
    g = torch.Generator().manual_seed(M + N)
    x = (torch.randn(M + 5, K, generator=g) * 3).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    rows = torch.randperm(M + 5, generator=g)[:M].to(torch.int32).to(DEV)
    xd = x.double()
    h = nw.double() * (xd * torch.rsqrt((xd ** 2).mean(-1, keepdim=True) + 1e-5))
    want = h @ w.double().T + bias.double()
    t = dict(atol=3e-2, rtol=2e-2)   # the operand x * weight is rounded to bfloat16 before the product
    got = ops.gemm_skinny_norm(x[:M].contiguous(), nw, 1e-5, w, bias)
    torch.testing.assert_close(got.double(), want[:M], **t)
    got = ops.gemm_skinny_norm(x, nw, 1e-5, w, bias, out_dtype=torch.float32, rows=rows)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.double(), want[rows.long()], **t)
    if N % 2 == 0:
        act = ops.gemm_skinny_norm(x, nw, 1e-5, w, None, ops.EPI_SWIGLU, rows=rows)
        p = (h @ w.double().T)[rows.long()]
        torch.testing.assert_close(act.double(), torch.nn.functional.silu(p[:, 0::2]) * p[:, 1::2], **t)
    # against the unfused pair of kernels: the same up to the rounding of the operand
    hb = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
    ops.rms_norm(x, nw, 1e-5, hb, rows=rows)
    unfused = ops.gemm_skinny(hb, w, bias, out_dtype=torch.float32)
    torch.testing.assert_close(got, unfused, atol=3e-2, rtol=2e-2)


@pytest.mark.parametrize("M", [1, 8, 40])
@pytest.mark.parametrize("nh,nkv,d,K,v_transposed", [(14, 2, 64, 896, True), (6, 3, 32, 72, False), (4, 1, 128, 200, True)])
@pytest.mark.parametrize("tiles", ["whole", "8+8"])
def test_qkv_rope_store_fused_equals_the_separate_kernels(ops, M, nh, nkv, d, K, v_transposed, tiles):
    """Both shapes of block: two whole tiles half a head apart, and one tile of 8 + 8 rows whose rotary pairs lie in
    two lanes (the choice between them goes by the number of blocks; here each is forced in turn)."""
    from llm_infrence_engine_amd.kernels import build

    lib = build.load()
    lib.ms_qkv_rope_store_force(0 if tiles == "whole" else 1)
    try:
        _qkv_fused_case(ops, M, nh, nkv, d, K, v_transposed)
    finally:
        lib.ms_qkv_rope_store_force(-1)


def _qkv_fused_case(ops, M, nh, nkv, d, K, v_transposed):
    g = torch.Generator().manual_seed(M + d)
    page_size, pages = 16, 12
    x = (torch.randn(M, K, generator=g) * 2).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
    w = (torch.randn((nh + 2 * nkv) * d, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    bias = torch.randn((nh + 2 * nkv) * d, generator=g).to(DEV)
    pos = torch.randint(0, 3000, (M,), generator=g).to(torch.int32).to(DEV)
    slots = torch.randperm(pages * page_size, generator=g)[:M].to(torch.int32)
    if M > 2:
        slots[2] = -1
    slots = slots.to(DEV)
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float64) / d))).float().to(DEV)
    vshape = (pages, nkv, d, page_size) if v_transposed else (pages, nkv, page_size, d)
    kp1, vp1 = torch.zeros(pages, nkv, page_size, d, dtype=torch.bfloat16, device=DEV), torch.zeros(vshape, dtype=torch.bfloat16, device=DEV)
    kp2, vp2 = torch.zeros_like(kp1), torch.zeros_like(vp1)
    q = ops.qkv_rope_store(x, nw, 1e-6, w, bias, nh, nkv, d, pos, inv_freq, slots, kp1, vp1, v_transposed)
    # the separate kernels, in float between them so that only the final rounding differs
    qkv = ops.gemm_skinny_norm(x, nw, 1e-6, w, bias, out_dtype=torch.float32)
    exact = qkv.double().view(M, nh + 2 * nkv, d).cpu()
    rot = rope_reference(exact[:, :nh + nkv], pos.cpu(), d, inv_freq.double().cpu())
    torch.testing.assert_close(q.double().cpu().view(M, nh, d), rot[:, :nh], atol=3e-2, rtol=1.6e-2)
    for n in range(M):
        s = int(slots[n])
        if s < 0:
            continue
        p, o = divmod(s, page_size)
        torch.testing.assert_close(kp1[p, :, o].double().cpu(), rot[n, nh:], atol=3e-2, rtol=1.6e-2)
        v = vp1[p, :, :, o] if v_transposed else vp1[p, :, o]
        torch.testing.assert_close(v.double().cpu(), exact[n, nh + nkv:], atol=3e-2, rtol=1.6e-2)
    untouched = torch.ones(pages * page_size, dtype=torch.bool)
    untouched[slots[slots >= 0].long().cpu()] = False
    assert (kp1.permute(0, 2, 1, 3).reshape(pages * page_size, -1)[untouched.to(DEV)] == 0).all()


@pytest.mark.parametrize("M", [65, 130, 700])
@pytest.mark.parametrize("nh,nkv,d,K,v_transposed,tile", [(14, 2, 64, 896, True, 0), (3, 1, 64, 128, False, 2),
                                                            (5, 5, 64, 192, True, 3), (3, 1, 128, 256, True, 0),
                                                            (2, 2, 128, 64, False, 0)])
def test_gemm_tiled_qkv_equals_product_rotation_and_store(ops, M, nh, nkv, d, K, v_transposed, tile):
    """The many-rows q/k/v product with bias, rotation and cache store as its epilogue, against a double product
    and the plain rotation: every tile shape, tokens and heads that fill no whole tile, one token not stored, pages
    plain and transposed, positions up to thousands."""
    g = torch.Generator().manual_seed(M + d + K)
    page_size = 16
    pages = (M + page_size - 1) // page_size + 3
    a = torch.randn(M, K, generator=g).bfloat16().to(DEV)
    w = (torch.randn((nh + 2 * nkv) * d, K, generator=g) / math.sqrt(K)).bfloat16().to(DEV)
    bias = torch.randn((nh + 2 * nkv) * d, generator=g).to(DEV) if K != 128 else None
    pos = torch.randint(0, 3000, (M,), generator=g).to(torch.int32).to(DEV)
    slots = torch.randperm(pages * page_size, generator=g)[:M].to(torch.int32)
    slots[2] = -1
    slots = slots.to(DEV)
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float64) / d))).float().to(DEV)
    vshape = (pages, nkv, d, page_size) if v_transposed else (pages, nkv, page_size, d)
    kp = torch.zeros(pages, nkv, page_size, d, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros(vshape, dtype=torch.bfloat16, device=DEV)
    assert ops.gemm_tiled_qkv_pays(a, w, d, d, kp)
    assert not ops.gemm_tiled_qkv_pays(a, w, d, d // 2, kp)       # a rotation over part of the head is not taken
    force = ops._get("ms_gemm_tiled_force")
    force(tile)
    try:
        table = ops.rope_table(pos, inv_freq)
        q = ops.gemm_tiled_qkv(a, w, bias, nh, nkv, d, table, slots, kp, vp, v_transposed)
    finally:
        force(0)
    ang = pos.cpu().float()[:, None] * inv_freq.cpu()[None]      # the float product, as the kernel forms it
    torch.testing.assert_close(table.cpu().double(), torch.stack((ang.double().cos(), ang.double().sin()), -1),
                               atol=1e-6, rtol=0)
    exact = a.double().cpu() @ w.double().cpu().T
    if bias is not None:
        exact = exact + bias.double().cpu()
    exact = exact.view(M, nh + 2 * nkv, d)
    rot = rope_reference(exact[:, :nh + nkv], pos.cpu(), d, inv_freq.double().cpu())
    t = dict(atol=3e-2, rtol=1.6e-2)
    torch.testing.assert_close(q.double().cpu().view(M, nh, d), rot[:, :nh], **t)
    sl = slots.cpu()
    stored = sl >= 0
    pg, off = (sl[stored] // page_size).long(), (sl[stored] % page_size).long()
    torch.testing.assert_close(kp.cpu()[pg, :, off].double(), rot[stored][:, nh:], **t)
    v = vp.cpu().permute(0, 1, 3, 2) if v_transposed else vp.cpu()
    torch.testing.assert_close(v[pg, :, off].double(), exact[stored][:, nh + nkv:], **t)
    untouched = torch.ones(pages * page_size, dtype=torch.bool)
    untouched[sl[stored].long()] = False
    assert (kp.cpu().permute(0, 2, 1, 3).reshape(pages * page_size, -1)[untouched] == 0).all()
    assert (v.permute(0, 2, 1, 3).reshape(pages * page_size, -1)[untouched] == 0).all()


# the products of a decode step at the shapes of the published checkpoints: (rows of W, columns) of the packed
# q/k/v, o, interleaved gate/up, down and head matrices
MODEL_PRODUCTS = {
    "0.5b": [(1152, 896), (896, 896), (9728, 896), (896, 4864), (151936, 896)],
    "7b": [(4608, 3584), (3584, 3584), (37888, 3584), (3584, 18944), (152064, 3584)],
    "32b": [(7168, 5120), (5120, 5120), (55296, 5120), (5120, 27648), (152064, 5120)],
}


@pytest.mark.parametrize("shape", sorted(MODEL_PRODUCTS))
def test_every_row_count_of_the_model_products_has_a_kernel(ops, shape):
    """1 to 64 rows against every product of the three model shapes, through ``kernels.linear`` as the parts call it:
    right against a double-precision product, and never by falling back to the vector-ALU kernel."""
    from llm_infrence_engine_amd.kernels import linear

    g = torch.Generator(device=DEV).manual_seed(len(shape))
    before = linear.fallback_count()
    for N, K in MODEL_PRODUCTS[shape]:
        w = (torch.randn(N, K, generator=g, device=DEV) / math.sqrt(K)).bfloat16()
        a = torch.randn(64, K, generator=g, device=DEV).bfloat16()
        want = a.double() @ w.double().T                                    # rows are independent: one reference for all M
        x = torch.randn(64, N, generator=g, device=DEV) if N < 100000 else None
        rows = (range(1, 65) if N < 100000 else (1, 2, 7, 8, 9, 16, 17, 31, 32, 33, 48, 63, 64))
        for M in rows:
            got = linear.linear(a[:M], w, out_dtype=torch.float32)
            err = (got.double() - want[:M]).abs().max().item()
            assert err < 5e-5 * max(1.0, want[:M].abs().max().item()) + 2e-5, (shape, "store", M, N, K, err)
            if x is not None:
                r = x[:M].clone()
                assert linear.linear_residual(a[:M], w, None, r) is None
                err = (r.double() - x[:M].double() - want[:M]).abs().max().item()
                assert err < 1e-4, (shape, "residual", M, N, K, err)
            if N % 2 == 0 and N > K and x is not None:                      # the gated product of gate/up
                act = linear.linear_swiglu(a[:M], w)
                ref = torch.nn.functional.silu(want[:M, 0::2]) * want[:M, 1::2]
                assert (act.double() - ref).abs().max().item() < 0.02 * max(1.0, ref.abs().max().item()), (shape, "gated", M, N, K)
        del w, a, want
    assert linear.fallback_count() == before, linear.fallbacks


def test_random_product_shapes_are_right_whatever_kernel_takes_them(ops):
    """A few hundred random shapes of up to 64 rows: ``kernels.linear`` finds a kernel for each (falling back to the
    vector-ALU kernel where the few-rows kernels have no variant, which is counted, not an error)."""
    from llm_infrence_engine_amd.kernels import linear

    rng = np.random.default_rng(17)
    g = torch.Generator(device=DEV).manual_seed(17)
    for case in range(300):
        M = int(rng.integers(1, 65))
        N = int(rng.choice([rng.integers(1, 64), rng.integers(64, 5000), rng.integers(5000, 40000)]))
        K = int(rng.choice([rng.integers(1, 40), rng.integers(40, 2000), rng.integers(2000, 12000)]))
        if rng.random() < 0.7:
            K = max(8, K // 8 * 8)
        a = torch.randn(M, K, generator=g, device=DEV).bfloat16()
        w = (torch.randn(N, K, generator=g, device=DEV) / math.sqrt(K)).bfloat16()
        b = torch.randn(N, generator=g, device=DEV) if rng.random() < 0.5 else None
        want = a.double() @ w.double().T + (b.double() if b is not None else 0.0)
        got = linear.linear(a, w, b, out_dtype=torch.float32)
        err = (got.double() - want).abs().max().item()
        assert err < 5e-5 * max(1.0, want.abs().max().item()) + 2e-5, (case, M, N, K, err)
        x = torch.randn(M, N, generator=g, device=DEV)
        r = x.clone()
        d = linear.linear_residual(a, w, b, r)
        total = r.double() if d is None else x.double() + d.double()
        assert (total - x.double() - want).abs().max().item() < (1e-4 if d is None else 0.05), (case, M, N, K)


def test_random_gated_products_of_many_rows(ops):
    """Random shapes of more than 64 rows through ``linear_swiglu``: the tiled kernel where it takes the sizes
    (columns in steps of 64) and pays, the library's product and the activation kernel otherwise."""
    from llm_infrence_engine_amd.kernels import linear

    rng = np.random.default_rng(23)
    g = torch.Generator(device=DEV).manual_seed(23)
    tiled = 0
    for case in range(60):
        M = int(rng.choice([rng.integers(65, 300), rng.integers(300, 3000)]))
        inter = int(rng.choice([rng.integers(1, 200), rng.integers(200, 6000)]))
        K = int(rng.choice([64 * rng.integers(1, 40), 8 * rng.integers(1, 300)]))
        a = torch.randn(M, K, generator=g, device=DEV).bfloat16()
        gate = (torch.randn(inter, K, generator=g, device=DEV) / math.sqrt(K)).bfloat16()
        up = (torch.randn(inter, K, generator=g, device=DEV) / math.sqrt(K)).bfloat16()
        w = linear.interleave_rows(gate, up)
        tiled += ops.gemm_tiled_pays(a, w)
        got = linear.linear_swiglu(a, w)
        want = torch.nn.functional.silu(a.double() @ gate.double().T) * (a.double() @ up.double().T)
        assert got.shape == (M, inter)
        err = (got.double() - want).abs().max().item()
        # the result is rounded to bfloat16 once; where the library writes the product first, that is rounded too
        assert err < 2.5e-2 * max(1.0, want.abs().max().item()), (case, M, inter, K, err)
    assert 15 < tiled < 60


def test_read_probe_reads_everything_once(ops):
    t = torch.randint(-2 ** 31, 2 ** 31 - 1, (1 << 20,), dtype=torch.int32, device=DEV)
    for n in (1 << 20, 4 * 1000, 4):
        got = np.bitwise_xor.reduce(ops.read_probe(t[:n]).cpu().numpy().view(np.uint32))
        assert got == np.bitwise_xor.reduce(t[:n].cpu().numpy().view(np.uint32))
    with pytest.raises(ValueError, match="16 bytes"):
        ops.read_probe(t[:3])
