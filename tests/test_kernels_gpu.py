"""Each HIP kernel alone against a plain torch reference of the same operation, at sizes
other than the engine's test models (widths and vocabularies that are no power of two,
head sizes in steps of 16, odd head counts)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def K():
    from jax_vllm_amd.ops import kernels

    return kernels


def tol(dtype, f32=1e-5, bf16=2e-2):
    return dict(rtol=f32, atol=f32) if dtype == torch.float32 else dict(rtol=bf16, atol=bf16)


def randn(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,vocab", [(72, 333), (4096, 1000), (70, 50), (12, 19)])
def test_embedding(dtype, hidden, vocab):
    table = randn(vocab, hidden, dtype=dtype)
    ids = torch.tensor([0, vocab - 1, 5, 5, 17], dtype=torch.int32).cuda()
    h = torch.empty(5, hidden, dtype=torch.float32).cuda()
    K().embedding(h, table, ids)
    torch.testing.assert_close(h, table[ids.long()].float(), rtol=0, atol=0)
    # an id that no row has (the sampling kernel's answer for a row of logits without a maximum is the
    # vocabulary size) reads nothing: its row is NaN, the other rows are untouched by it
    bad = torch.tensor([3, vocab, -1, 2 ** 31 - 1, 1], dtype=torch.int32).cuda()
    K().embedding(h, table, bad)
    assert torch.isnan(h[1:4]).all()
    torch.testing.assert_close(h[[0, 4]], table[[3, 1]].float(), rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [80, 1000, 4096])
def test_add_rmsnorm(dtype, hidden):
    n, eps = 7, 1e-5
    h = randn(n, hidden, seed=1)
    delta = randn(n, hidden, dtype=dtype, seed=2)
    w = 1 + 0.1 * randn(hidden, seed=3)
    h0 = h.clone()
    out = torch.empty(n, hidden, dtype=dtype).cuda()
    K().add_rmsnorm(h, delta, w, out, eps)
    x = h0 + delta.float()
    ref = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w
    torch.testing.assert_close(h, x, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(out.float(), ref, **tol(dtype))
    # first layer: no delta, h untouched
    h1 = h0.clone()
    K().add_rmsnorm(h1, None, w, out, eps)
    torch.testing.assert_close(h1, h0, rtol=0, atol=0)
    ref1 = h0 * torch.rsqrt((h0 * h0).mean(-1, keepdim=True) + eps) * w
    torch.testing.assert_close(out.float(), ref1, **tol(dtype))
    # selected rows: h untouched, sum redone on the fly
    rows = torch.tensor([6, 0, 3], dtype=torch.int32).cuda()
    h2 = h0.clone()
    out2 = torch.empty(3, hidden, dtype=dtype).cuda()
    K().add_rmsnorm(h2, delta, w, out2, eps, rows)
    torch.testing.assert_close(h2, h0, rtol=0, atol=0)
    torch.testing.assert_close(out2.float(), ref[rows.long()], **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_last_axis(dtype):
    x = randn(5, 3, 48, dtype=dtype, seed=4)
    w = 1 + 0.2 * randn(48, seed=5)
    out = K().rmsnorm(x, w, 1e-6)
    xf = x.float()
    ref = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + 1e-6) * w
    torch.testing.assert_close(out.float(), ref, **tol(dtype))


def gate_activation(name, g):
    """The library routine a gate activation of the kernels reduces to."""
    return torch.nn.functional.silu(g) if name == "silu" else torch.nn.functional.gelu(g, approximate="tanh")


ACTIVATIONS = ["silu", "gelu_tanh"]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [176, 12288, 77])
@pytest.mark.parametrize("act", ACTIVATIONS)
def test_gated_mul(dtype, inter, act):
    gu = randn(9, 2 * inter, dtype=dtype, seed=6, scale=3.0)
    out = K().gated_mul(gu, activation=act)
    g, u = gu.float()[:, :inter], gu.float()[:, inter:]
    torch.testing.assert_close(out.float(), gate_activation(act, g) * u, **tol(dtype))
    # gate and up alternating along the row
    out2 = K().gated_mul(gu, interleaved=True, activation=act)
    g2, u2 = gu.float()[:, 0::2], gu.float()[:, 1::2]
    torch.testing.assert_close(out2.float(), gate_activation(act, g2) * u2, **tol(dtype))
    with pytest.raises(ValueError):
        K().gated_mul(gu, activation="relu")


@pytest.mark.parametrize("m,n,k", [(1, 50, 70), (5, 333, 80), (70, 130, 257), (130, 64, 16)])
def test_gemm_f32_is_true_32bit(m, n, k):
    a, w = randn(m, k, seed=7), randn(n, k, seed=8)
    out = K().gemm_f32(a, w)
    ref = (a.double() @ w.double().T)
    # float accumulation over k terms: error far below any 16- or 19-bit matrix mode (~1e-3)
    torch.testing.assert_close(out.double(), ref, rtol=1e-5, atol=1e-5 * math.sqrt(k))
    # a row's result does not depend on the other rows of the batch
    if m > 1:
        single = K().gemm_f32(a[:1].contiguous(), w)
        torch.testing.assert_close(single, out[:1], rtol=0, atol=0)


@pytest.mark.parametrize("m,n,k", [(1, 96, 64), (8, 224, 96), (33, 512, 96)])
def test_linear_bf16(m, n, k):
    a, w = randn(m, k, dtype=torch.bfloat16, seed=9), randn(n, k, dtype=torch.bfloat16, seed=10)
    out = K().linear(a, w)
    ref = a.float() @ w.float().T
    torch.testing.assert_close(out.float(), ref, rtol=2e-2, atol=2e-2 * math.sqrt(k) / 8)


# ------------------------------------------------------------------ q/k norm + rotation + page write
def rope_reference(x, pos, inv_freq, rotary_dim, interleaved):
    """x [T, heads, D] float; rotation of the first rotary_dim elements of each head."""
    ang = pos.float()[:, None] * inv_freq[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    half = rotary_dim // 2
    if interleaved:
        a, b = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
        out[..., 0:rotary_dim:2] = a * cos - b * sin
        out[..., 1:rotary_dim:2] = b * cos + a * sin
    else:
        a, b = x[..., :half], x[..., half:rotary_dim]
        out[..., :half] = a * cos - b * sin
        out[..., half:rotary_dim] = b * cos + a * sin
    return out


ROPE_CASES = [(4, 2, 16, 16, False, True, 11), (5, 5, 48, 48, False, True, 11), (6, 2, 128, 128, False, True, 11),
              (3, 1, 80, 32, False, False, 11), (4, 4, 32, 32, True, True, 11), (8, 2, 256, 64, True, False, 11),
              (8, 2, 256, 256, False, True, 11), (4, 4, 256, 128, False, True, 11), (32, 8, 128, 128, False, True, 300),
              (5, 1, 128, 128, False, False, 260), (2, 2, 64, 64, False, True, 270)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,rotary_dim,interleaved,with_norm,t", ROPE_CASES)
def test_qk_norm_rope_write(dtype, nq, nkv, d, rotary_dim, interleaved, with_norm, t):
    page_size, eps = 4, 1e-5
    pages = t + 2
    qkv = randn(t, (nq + 2 * nkv) * d, dtype=dtype, seed=11)
    g = torch.Generator().manual_seed(t)
    pos_list = ([0, 1, 2, 3, 100, 101, 4095, 7, 8, 9, 31999] + torch.randint(0, 200, (max(0, t - 11),), generator=g).tolist())[:t]
    slot_list = (torch.randperm((pages - 1) * page_size, generator=g)[:t] + page_size).tolist()   # distinct, none in page 0
    slot_list[7] = -1
    pos = torch.tensor(pos_list, dtype=torch.int32).cuda()
    slots = torch.tensor(slot_list, dtype=torch.int32).cuda()
    qw = (1 + 0.1 * randn(d, seed=12)) if with_norm else None
    kw = (1 + 0.1 * randn(d, seed=13)) if with_norm else None
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))).cuda()
    k_pages = torch.zeros(pages, nkv, page_size, d, dtype=dtype).cuda()
    v_pages = torch.zeros(pages, nkv, d, page_size, dtype=dtype).cuda()
    x = qkv.float().view(t, nq + 2 * nkv, d).clone()
    table = K().rope_table(pos, inv_freq)
    ang = pos.float()[:, None] * inv_freq[None, :]
    torch.testing.assert_close(table, torch.cat([torch.cos(ang), torch.sin(ang)], dim=1), rtol=1e-5, atol=2e-6)
    K().qk_norm_rope_write(qkv, slots, qw, kw, eps, table, rotary_dim, interleaved, k_pages, v_pages,
                           page_size, nq, nkv, d)
    q, k, v = x[:, :nq], x[:, nq:nq + nkv], x[:, nq + nkv:]
    if with_norm:
        q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * qw
        k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * kw
    q = rope_reference(q, pos, inv_freq, rotary_dim, interleaved)
    k = rope_reference(k, pos, inv_freq, rotary_dim, interleaved)
    got_q = qkv.float().view(t, nq + 2 * nkv, d)[:, :nq]
    # large positions: the angle itself carries float rounding (pos * inv_freq ~ 3e4 * 1 has ulp 2e-3)
    big = dict(rtol=1e-2, atol=1e-2) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    small = tol(dtype, f32=2e-5, bf16=2e-2)
    near = (pos.cpu() < 200).cuda()
    torch.testing.assert_close(got_q[near], q[near], **small)
    torch.testing.assert_close(got_q, q, **big)
    exp_k = torch.zeros(pages, nkv, page_size, d).cuda()
    exp_v = torch.zeros(pages, nkv, d, page_size).cuda()     # values are stored transposed
    for i, s_ in enumerate(slot_list):
        if s_ >= 0:
            exp_k[s_ // page_size, :, s_ % page_size] = k[i]
            exp_v[s_ // page_size, :, :, s_ % page_size] = v[i]
    torch.testing.assert_close(k_pages.float(), exp_k, **big)
    torch.testing.assert_close(v_pages.float(), exp_v, rtol=0, atol=0)  # values are copied untouched
    # without pages nothing is stored and q is still prepared (a run that reads another's cache)
    qkv2 = x.reshape(t, -1).to(dtype).contiguous()
    K().qk_norm_rope_write(qkv2, None, qw, kw, eps, table, rotary_dim, interleaved, None, None, page_size, nq, nkv, d)
    torch.testing.assert_close(qkv2.float().view(t, nq + 2 * nkv, d)[:, :nq], got_q, rtol=0, atol=0)


def _slot_pattern(kind: str, t: int, page_size: int):
    base = 2 * page_size
    if kind == "prompt":            # one prompt from the start of a page: every 8 tokens are one aligned run
        return [base + i for i in range(t)]
    if kind == "offset":            # a portion that starts in the middle of a page: no aligned run at all
        return [base + 3 + i for i in range(t)]
    if kind == "two_requests":      # a boundary between requests inside a group of 8, the second one unaligned
        first = 130
        second_base = base + 40 * page_size + 5
        return [base + i for i in range(first)] + [second_base + i for i in range(t - first)]
    g = torch.Generator().manual_seed(t + page_size)
    slots = (torch.randperm(t + 64, generator=g)[:t] + base).tolist()
    for i in (7, 8, 100, t - 1):
        slots[i] = -1
    return slots


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [8, 16, 64])
@pytest.mark.parametrize("kind", ["prompt", "offset", "two_requests", "scattered"])
@pytest.mark.parametrize("nq,nkv,d,t", [(4, 2, 128, 300), (2, 3, 80, 259), (5, 3, 64, 270), (3, 1, 256, 257)])
def test_values_of_many_tokens_reach_their_pages(dtype, page_size, kind, nq, nkv, d, t):
    """From 256 tokens on the v heads go to their transposed pages 8 tokens at a time where 8
    consecutive tokens have 8 consecutive, aligned slots, and one by one elsewhere, and q and k of
    fully rotated heads of 64, 128 or 256 are prepared 16 bytes a lane: all must give what the
    token-by-token path gives (the same call on portions below 256 tokens), v as an untouched copy."""
    eps = 1e-6
    slot_list = _slot_pattern(kind, t, page_size)
    pages = max(slot_list) // page_size + 2
    qkv = randn(t, (nq + 2 * nkv) * d, dtype=dtype, seed=31)
    slots = torch.tensor(slot_list, dtype=torch.int32).cuda()
    pos = torch.arange(t, dtype=torch.int32).cuda()
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).cuda()
    table = K().rope_table(pos, inv_freq)
    qw, kw = 1 + 0.1 * randn(d, seed=32), 1 + 0.1 * randn(d, seed=33)

    def run(portions):
        x = qkv.clone()
        kp = torch.zeros(pages, nkv, page_size, d, dtype=dtype).cuda()
        vp = torch.zeros(pages, nkv, d, page_size, dtype=dtype).cuda()
        for a, b in portions:
            part = x[a:b].contiguous()
            K().qk_norm_rope_write(part, slots[a:b].contiguous(), qw, kw, eps, table[a:b].contiguous(), d, False,
                                   kp, vp, page_size, nq, nkv, d)
            x[a:b] = part
        return x, kp, vp

    whole = run([(0, t)])
    pieces = run([(0, 101), (101, 250), (250, t)])
    # q and k: the two paths add the squares of a head in different orders
    torch.testing.assert_close(whole[0].float(), pieces[0].float(), **tol(dtype, f32=2e-5, bf16=2e-2))
    torch.testing.assert_close(whole[1].float(), pieces[1].float(), **tol(dtype, f32=2e-5, bf16=2e-2))
    torch.testing.assert_close(whole[2], pieces[2], rtol=0, atol=0)
    exp_v = torch.zeros(pages, nkv, d, page_size, dtype=dtype).cuda()
    v = qkv.view(t, nq + 2 * nkv, d)[:, nq + nkv:]
    for i, s_ in enumerate(slot_list):
        if s_ >= 0:
            exp_v[s_ // page_size, :, :, s_ % page_size] = v[i]
    torch.testing.assert_close(whole[2], exp_v, rtol=0, atol=0)


@pytest.mark.parametrize("nq,nkv,d,n_parts,t,with_norm", [(6, 2, 128, 2, 5, True), (4, 4, 256, 4, 16, True),
                                                         (32, 8, 128, 4, 8, True), (3, 1, 128, 3, 9, False)])
def test_qk_norm_rope_write_from_partial_products(nq, nkv, d, n_parts, t, with_norm):
    """The projection arrives as float partial products: their ordered sum must give what the
    whole bfloat16 projection gives, up to the rounding the whole one has and the parts do not."""
    bf = torch.bfloat16
    page_size, eps, width = 8, 1e-6, (nq + 2 * nkv) * d
    pages = t + 2
    parts = randn(n_parts, t, width, seed=40, scale=0.7)
    whole = (parts[0].cpu() + parts[1].cpu())
    for q in range(2, n_parts):
        whole = whole + parts[q].cpu()
    g = torch.Generator().manual_seed(t)
    pos = torch.randint(0, 3000, (t,), generator=g).to(torch.int32).cuda()
    slots = (torch.randperm((pages - 1) * page_size, generator=g)[:t] + page_size).to(torch.int32).cuda()
    qw = (1 + 0.1 * randn(d, seed=12)) if with_norm else None
    kw = (1 + 0.1 * randn(d, seed=13)) if with_norm else None
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))).cuda()
    table = K().rope_table(pos, inv_freq)
    outs = []
    for use_parts in (True, False):
        k_pages = torch.zeros(pages, nkv, page_size, d, dtype=bf).cuda()
        v_pages = torch.zeros(pages, nkv, d, page_size, dtype=bf).cuda()
        qkv = torch.zeros(t, width, dtype=bf).cuda() if use_parts else whole.to(bf).cuda()
        K().qk_norm_rope_write(qkv, slots, qw, kw, eps, table, d, False, k_pages, v_pages, page_size, nq, nkv, d,
                               parts=parts if use_parts else None)
        outs.append((qkv.float().view(t, nq + 2 * nkv, d)[:, :nq].cpu(), k_pages.float().cpu(), v_pages.float().cpu()))
    for a, b in zip(*outs):
        torch.testing.assert_close(a, b, rtol=3e-2, atol=3e-2)
    # and against the float formula directly
    x = whole.view(t, nq + 2 * nkv, d)
    qf = x[:, :nq]
    if with_norm:
        qf = qf * torch.rsqrt((qf * qf).mean(-1, keepdim=True) + eps) * qw.cpu()
    qf = rope_reference(qf.cuda(), pos, inv_freq, d, False).cpu()
    torch.testing.assert_close(outs[0][0], qf, rtol=1e-2, atol=1e-2)
    assert not K().rope_takes_parts(torch.bfloat16, 64, False, 64, True)
    assert not K().rope_takes_parts(torch.bfloat16, 128, True, 128, True)
    assert not K().rope_takes_parts(torch.float32, 128, False, 128, True)


# ------------------------------------------------------------------ paged attention
def build_paged(k, v, page_size, seed=0, extra_pages=3):
    """Scatter per-request [T, nkv, D] keys/values over shuffled pages; returns pages and tables."""
    g = torch.Generator().manual_seed(seed)
    need = [-(-kk.shape[0] // page_size) for kk in k]
    total = sum(need) + extra_pages + 1
    order = (torch.randperm(total - 1, generator=g) + 1).tolist()
    nkv, d = k[0].shape[1], k[0].shape[2]
    k_pages = torch.randn(total, nkv, page_size, d, generator=g) * 50  # garbage where no key lives
    v_pages = torch.randn(total, nkv, d, page_size, generator=g) * 50  # values are stored transposed
    tables = torch.zeros(len(k), max(need), dtype=torch.int32)
    for r, (kk, vv) in enumerate(zip(k, v)):
        for p in range(need[r]):
            page = order.pop()
            tables[r, p] = page
            chunk = slice(p * page_size, min((p + 1) * page_size, kk.shape[0]))
            n = chunk.stop - chunk.start
            k_pages[page, :, :n] = kk[chunk].transpose(0, 1)
            v_pages[page, :, :, :n] = vv[chunk].permute(1, 2, 0)
    return k_pages, v_pages, tables


def attention_reference(q, k, v, positions, scale, window=None):
    """q [Tq, nq, D] at absolute ``positions``; k, v [Tk, nkv, D]; float64."""
    nq, nkv = q.shape[1], k.shape[1]
    kk = torch.repeat_interleave(k.double(), nq // nkv, dim=1)
    vv = torch.repeat_interleave(v.double(), nq // nkv, dim=1)
    s = torch.einsum("qhd,khd->hqk", q.double(), kk) * scale
    j = torch.arange(k.shape[0])[None, :]
    p = positions[:, None]
    mask = j <= p
    if window:
        mask &= j > p - window
    s = s.masked_fill(~mask[None], float("-inf"))
    return torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), vv)


ATT_CASES = [
    # nq, nkv, d, page_size, [(context_len, q_len)], window
    (4, 2, 16, 8, [(0, 5), (0, 17), (0, 33)], None),
    (6, 2, 32, 16, [(0, 1), (9, 1), (40, 24), (0, 64), (100, 1)], None),
    (5, 5, 48, 32, [(37, 2), (0, 70)], None),
    (8, 2, 128, 16, [(300, 1), (0, 130), (255, 3)], None),
    (3, 1, 80, 4, [(20, 9), (3, 1)], None),
    (4, 2, 64, 16, [(50, 10), (0, 40), (200, 1)], 24),
    (16, 2, 256, 16, [(10, 3)], None),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", ATT_CASES, ids=[f"h{c[0]}g{c[1]}d{c[2]}p{c[3]}w{c[5]}" for c in ATT_CASES])
def test_paged_attention_generic(dtype, case):
    nq, nkv, d, page_size, reqs, window = case
    scale = 1.0 / math.sqrt(d)
    g = torch.Generator().manual_seed(5)
    ks = [torch.randn(c + q, nkv, d, generator=g).to(dtype).float() for c, q in reqs]
    vs = [torch.randn(c + q, nkv, d, generator=g).to(dtype).float() for c, q in reqs]
    qs = [torch.randn(q, nq, d, generator=g).to(dtype).float() for c, q in reqs]
    k_pages, v_pages, tables = build_paged(ks, vs, page_size)
    n = sum(q for _, q in reqs)
    # q rows live inside a fused qkv-like buffer: row stride larger than nq * d
    stride = (nq + 2 * nkv) * d
    qbuf = torch.zeros(n, stride)
    positions, token_req, refs, at = [], [], [], 0
    for r, (c, ql) in enumerate(reqs):
        qbuf[at:at + ql, :nq * d] = qs[r].reshape(ql, nq * d)
        pos = torch.arange(c, c + ql)
        positions += pos.tolist()
        token_req += [r] * ql
        refs.append(attention_reference(qs[r], ks[r], vs[r], pos, scale, window))
        at += ql
    ref = torch.cat(refs).reshape(n, nq * d)
    out = torch.empty(n, nq * d, dtype=dtype).cuda()
    K().paged_attention_generic(
        out, qbuf.to(dtype).cuda(), stride, k_pages.to(dtype).cuda(), v_pages.to(dtype).cuda(), tables.cuda(),
        torch.tensor(token_req, dtype=torch.int32).cuda(), torch.tensor(positions, dtype=torch.int32).cuda(),
        nq, nkv, d, scale, window or 0)
    torch.testing.assert_close(out.double().cpu(), ref, **tol(dtype, f32=2e-5, bf16=2e-2))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("far_key", [0, 15, 16, 17, 255, 256, 511, 640])
def test_attention_finds_one_far_key(dtype, far_key):
    """One key among hundreds is made to dominate: the output must be that key's value, wherever
    in its page (first slot, last slot) and however far back it lies."""
    nq, nkv, d, page_size, ctx = 4, 2, 64, 16, 641
    g = torch.Generator().manual_seed(far_key)
    k = torch.randn(ctx, nkv, d, generator=g) * 0.1
    v = torch.randn(ctx, nkv, d, generator=g)
    q = torch.randn(1, nq, d, generator=g) * 0.1
    q[0, :, 0] = 40.0
    k[far_key, :, 0] = 40.0          # score 1600/8 = 200 above the rest
    k_pages, v_pages, tables = build_paged([k], [v], page_size, seed=far_key)
    out = torch.empty(1, nq * d, dtype=dtype).cuda()
    K().paged_attention_generic(
        out, q.reshape(1, -1).to(dtype).cuda(), nq * d, k_pages.to(dtype).cuda(), v_pages.to(dtype).cuda(),
        tables.cuda(), torch.zeros(1, dtype=torch.int32).cuda(), torch.tensor([ctx - 1], dtype=torch.int32).cuda(),
        nq, nkv, d, 1.0 / math.sqrt(d))
    expect = torch.repeat_interleave(v[far_key].to(dtype).float(), nq // nkv, dim=0).reshape(1, -1)
    torch.testing.assert_close(out.float().cpu(), expect, rtol=1e-3, atol=1e-3)


# ------------------------------------------------------------------ sampling
def test_greedy_is_argmax_lowest_index_on_ties():
    logits = randn(6, 777, seed=20)
    logits[2, 100] = logits[2, 500] = 99.0
    logits[4, 776] = 50.0
    out = K().sample(logits)
    ref = torch.argmax(logits, dim=-1)
    assert out.tolist()[:2] == ref.tolist()[:2]
    assert out[2].item() == 100 and out[4].item() == 776


def test_a_row_without_a_maximum_is_an_error_not_a_token():
    """A row of NaN logits has no winner: the kernel answers with the vocabulary size and the
    sampler above it raises at once, instead of handing on a token that no table has."""
    from jax_vllm_amd.sampling.sampler import Sampler

    logits = randn(3, 300, seed=21)
    logits[1] = float("nan")
    assert K().sample(logits).tolist()[1] == 300
    with pytest.raises(FloatingPointError, match=r"row\(s\) \[1\] of 3"):
        Sampler(logits.device).sample(logits, [0.0, 0.0, 0.0], [1, 2, 3])
    logits[1] = 0.0
    logits[1, 7] = float("nan")                       # one NaN among numbers never wins
    assert Sampler(logits.device).sample(logits, [0.0, 0.0, 0.0], [1, 2, 3])[1] == 0


def test_temperature_sampling_matches_softmax():
    v, n, temp = 11, 20000, 0.8
    logits1 = randn(1, v, seed=21, scale=1.5)
    logits = logits1.expand(n, v).contiguous()
    keys = torch.arange(n, dtype=torch.int64).cuda() * 7919 + 3
    t = torch.full((n,), temp, dtype=torch.float32).cuda()
    out = K().sample(logits, t, keys)
    freq = torch.bincount(out.long().cpu(), minlength=v).double() / n
    p = torch.softmax(logits1[0].double().cpu() / temp, -1)
    # binomial standard deviation of a frequency is at most 0.5 / sqrt(n) = 0.0035
    assert (freq - p).abs().max().item() < 0.015
    # the draw depends on key and logits only: same keys in another order, another batch size
    perm = torch.randperm(n)[:100].cuda()
    out2 = K().sample(logits[perm].contiguous(), t[:100].contiguous(), keys[perm].contiguous())
    assert out2.tolist() == out[perm].tolist()
    # temperature 0 rows beside sampled rows are greedy
    t2 = t.clone()
    t2[::2] = 0.0
    out3 = K().sample(logits, t2, keys)
    assert (out3[::2] == torch.argmax(logits1[0])).all()
    assert out3[1::2].tolist() == out[1::2].tolist()


# ------------------------------------------------------------------ matrix-core attention (bfloat16)
def _mfma_inputs(nq, nkv, d, page_size, reqs, seed=5):
    g = torch.Generator().manual_seed(seed)
    bf = torch.bfloat16
    ks = [torch.randn(c + q, nkv, d, generator=g).to(bf).float() for c, q in reqs]
    vs = [torch.randn(c + q, nkv, d, generator=g).to(bf).float() for c, q in reqs]
    qs = [torch.randn(q, nq, d, generator=g).to(bf).float() for c, q in reqs]
    k_pages, v_pages, tables = build_paged(ks, vs, page_size, seed=seed)
    n = sum(q for _, q in reqs)
    stride = (nq + 2 * nkv) * d
    qbuf = torch.zeros(n, stride)
    cu, at = [0], 0
    for r, (c, ql) in enumerate(reqs):
        qbuf[at:at + ql, :nq * d] = qs[r].reshape(ql, nq * d)
        at += ql
        cu.append(at)
    dev = dict(
        q=qbuf.to(bf).cuda(), k_pages=k_pages.to(bf).cuda(), v_pages=v_pages.to(bf).cuda(), tables=tables.cuda(),
        cu=torch.tensor(cu, dtype=torch.int32).cuda(),
        ctx=torch.tensor([c for c, _ in reqs], dtype=torch.int32).cuda(), stride=stride, n=n,
    )
    return qs, ks, vs, dev


def _mfma_reference(qs, ks, vs, reqs, scale, window, nq, d):
    refs = []
    for r, (c, ql) in enumerate(reqs):
        refs.append(attention_reference(qs[r], ks[r], vs[r], torch.arange(c, c + ql), scale, window))
    return torch.cat(refs).reshape(-1, nq * d)


MFMA_PREFILL_CASES = [c for c in ATT_CASES if c[3] % 8 == 0] + [
    (32, 8, 128, 16, [(0, 200), (1000, 50)], None),
    (4, 4, 112, 24, [(30, 40), (0, 3)], None),
    (8, 1, 64, 8, [(5, 70)], 17),
    (40, 2, 32, 16, [(10, 9)], None),      # 20 heads per group: rows of one query span two 16-row tiles
    (8, 2, 128, 16, [(0, 700)], None),     # 44 groups: light ones paired with heavy ones
    (8, 2, 64, 16, [(100, 300)], 50),      # window: paired groups far apart leave a gap of key tiles between them
    (4, 1, 128, 32, [(64, 129), (0, 64)], 40),
    (2, 1, 16, 8, [(17000, 40)], None),    # more pages than the kernel keeps of the table at a time
    (2, 1, 16, 8, [(17000, 200)], 100),
    # head sizes of the kernel with 32-row tiles, in each of its ways of finding a key's page
    (6, 2, 96, 16, [(70, 90), (0, 5)], None),       # keys of 12 chunks: a load instruction spans pages
    (4, 2, 128, 24, [(100, 140)], None),            # a page size that is no power of two
    (4, 1, 64, 128, [(200, 100), (0, 129)], None),  # pages larger than a key tile
    (4, 2, 128, 8, [(3, 150)], 90),
    (6, 3, 32, 16, [(1, 260), (500, 33)], None),    # one load instruction a tile and wave
    (2, 1, 32, 8, [(9000, 70)], None),              # more pages than the general path keeps of the table at a time
    (10, 2, 64, 16, [(64, 64), (63, 65), (0, 2)], None),   # 5 heads a group: a query's rows cross the 32-row tiles
    (32, 8, 128, 16, [(1900, 300)], 1024),          # window wider than the portion: early tiles drop out one by one
]


def _prefill_work(reqs, g, d, window, plan):
    """Work items of the prefill kernel: by the engine's planner (in both its ways of pairing groups),
    one group per item, every group in the item's second place, or the first group with the last."""
    from jax_vllm_amd.parts.attention_backend import prefill_work_items

    group_rows, per_item = K().attn_prefill_geometry(d)
    singles = [(r, m0) for r, (c, ql) in enumerate(reqs) for m0 in range(0, ql * g, group_rows)]
    if plan in ("planner", "neighbours"):       # light groups paired with heavy ones, or neighbours paired
        items = prefill_work_items([ql for _, ql in reqs], [c for c, _ in reqs], g, window or 0, group_rows, per_item,
                                   balance=plan == "planner")
        items += [(r, 0, -1) for r, (c, ql) in enumerate(reqs) if ql == 1]      # the planner leaves these to decode
    elif plan == "second" and per_item > 1:
        items = [(r, -1, m0) for r, m0 in singles]
    elif plan == "far" and per_item > 1:         # first with last, window or not
        items = []
        for r in range(len(reqs)):
            mine = [m0 for rr, m0 in singles if rr == r]
            while len(mine) > 1:
                items.append((r, mine.pop(0), mine.pop(-1)))
            items += [(r, m0, -1) for m0 in mine]
    else:
        items = [(r, m0, -1) for r, m0 in singles]
    covered = sorted((r, m0) for r, a, b in items for m0 in (a, b) if m0 >= 0)
    assert covered == sorted(singles)
    return torch.tensor([x for it in items for x in it], dtype=torch.int32).cuda(), len(items)


@pytest.mark.parametrize("plan", ["planner", "neighbours", "single", "second", "far"])
@pytest.mark.parametrize("case", MFMA_PREFILL_CASES,
                         ids=[f"h{c[0]}g{c[1]}d{c[2]}p{c[3]}w{c[5]}n{len(c[4])}" for c in MFMA_PREFILL_CASES])
def test_mfma_prefill_attention(case, plan):
    nq, nkv, d, page_size, reqs, window = case
    scale = 1.0 / math.sqrt(d)
    qs, ks, vs, dev = _mfma_inputs(nq, nkv, d, page_size, reqs)
    work, n_work = _prefill_work(reqs, nq // nkv, d, window, plan)
    out = torch.full((dev["n"], nq * d), float("nan"), dtype=torch.bfloat16).cuda()
    K().attn_prefill_mfma(out, dev["q"], dev["stride"], dev["k_pages"], dev["v_pages"], dev["tables"], dev["cu"],
                          dev["ctx"], work, n_work, nq, nkv, d, scale, window or 0)
    ref = _mfma_reference(qs, ks, vs, reqs, scale, window, nq, d)
    torch.testing.assert_close(out.double().cpu(), ref, rtol=2e-2, atol=2e-2)


MFMA_DECODE_CASES = [
    # nq, nkv, d, page_size, contexts, window
    (4, 2, 16, 8, [0, 1, 7, 8, 33, 200], None),
    (6, 2, 32, 16, [9, 100, 31, 32, 1234], None),
    (5, 5, 48, 32, [37, 0, 500], None),
    (32, 8, 128, 16, [1023, 1024, 1500, 3], None),
    (16, 2, 256, 16, [130, 64], None),
    (40, 2, 64, 16, [77, 300], None),      # 20 heads per group: two row tiles per kv head
    (8, 2, 64, 16, [50, 200, 1000], 24),
    (4, 4, 80, 40, [99, 160], None),
]


@pytest.mark.parametrize("splits", [1, 3, 8])
@pytest.mark.parametrize("case", MFMA_DECODE_CASES,
                         ids=[f"h{c[0]}g{c[1]}d{c[2]}p{c[3]}w{c[5]}" for c in MFMA_DECODE_CASES])
def test_mfma_decode_attention(case, splits):
    nq, nkv, d, page_size, contexts, window = case
    reqs = [(c, 1) for c in contexts]
    scale = 1.0 / math.sqrt(d)
    qs, ks, vs, dev = _mfma_inputs(nq, nkv, d, page_size, reqs, seed=9)
    # the work list names the requests in another order than they lie in the batch
    order = list(reversed(range(len(reqs))))
    scratch = None
    if splits > 1:
        scratch = torch.full((K().attn_decode_scratch_floats(len(reqs), nq, splits, d),), float("nan")).cuda()
    out = torch.full((dev["n"], nq * d), float("nan"), dtype=torch.bfloat16).cuda()
    K().attn_decode_mfma(out, dev["q"], dev["stride"], dev["k_pages"], dev["v_pages"], dev["tables"], dev["cu"],
                         dev["ctx"], torch.tensor(order, dtype=torch.int32).cuda(), len(order), nq, nkv, d, scale,
                         window or 0, splits, scratch)
    ref = _mfma_reference(qs, ks, vs, reqs, scale, window, nq, d)
    torch.testing.assert_close(out.double().cpu(), ref, rtol=2e-2, atol=2e-2)
    # a step of decoded tokens only needs no work list: request r's token is row r
    again = torch.full((dev["n"], nq * d), float("nan"), dtype=torch.bfloat16).cuda()
    K().attn_decode_mfma(again, dev["q"], dev["stride"], dev["k_pages"], dev["v_pages"], dev["tables"], dev["cu"],
                         dev["ctx"], None, len(order), nq, nkv, d, scale, window or 0, splits, scratch)
    assert torch.equal(again, out)


def test_mfma_decode_attention_with_a_table_wider_than_a_block_keeps():
    """More than 4,096 pages: a block copies only the entries of its own split's keys, so few splits are
    refused and enough of them give the same result as everywhere else."""
    from jax_vllm_amd.ops.kernels import KernelArgumentError, attn_decode_min_splits

    nq, nkv, d, page_size = 2, 1, 16, 8
    reqs = [(40000, 1), (33, 1), (36111, 1)]
    scale = 1.0 / math.sqrt(d)
    qs, ks, vs, dev = _mfma_inputs(nq, nkv, d, page_size, reqs, seed=11)
    assert dev["tables"].shape[1] > 4096 and attn_decode_min_splits(dev["tables"].shape[1], page_size) == 2
    ref = _mfma_reference(qs, ks, vs, reqs, scale, None, nq, d)
    for splits in (2, 5, 16):
        scratch = torch.full((K().attn_decode_scratch_floats(len(reqs), nq, splits, d),), float("nan")).cuda()
        out = torch.full((dev["n"], nq * d), float("nan"), dtype=torch.bfloat16).cuda()
        K().attn_decode_mfma(out, dev["q"], dev["stride"], dev["k_pages"], dev["v_pages"], dev["tables"], dev["cu"],
                             dev["ctx"], None, len(reqs), nq, nkv, d, scale, 0, splits, scratch)
        torch.testing.assert_close(out.double().cpu(), ref, rtol=2e-2, atol=2e-2)
    with pytest.raises(KernelArgumentError, match="at least 2 splits"):
        K().attn_decode_mfma(out, dev["q"], dev["stride"], dev["k_pages"], dev["v_pages"], dev["tables"], dev["cu"],
                             dev["ctx"], None, len(reqs), nq, nkv, d, scale, 0, 1, None)


@pytest.mark.parametrize("far_key", [0, 15, 16, 31, 32, 63, 64, 255, 256, 511, 640])
@pytest.mark.parametrize("kernel", ["prefill", "decode1", "decode5"])
def test_mfma_attention_finds_one_far_key(kernel, far_key):
    nq, nkv, d, page_size, ctx = 4, 2, 64, 16, 641
    g = torch.Generator().manual_seed(far_key)
    k = (torch.randn(ctx, nkv, d, generator=g) * 0.1)
    v = torch.randn(ctx, nkv, d, generator=g)
    q = torch.randn(1, nq, d, generator=g) * 0.1
    q[0, :, 0] = 40.0
    k[far_key, :, 0] = 40.0
    bf = torch.bfloat16
    k_pages, v_pages, tables = build_paged([k.to(bf).float()], [v.to(bf).float()], page_size, seed=far_key)
    out = torch.empty(1, nq * d, dtype=bf).cuda()
    args = (out, q.reshape(1, -1).to(bf).cuda(), nq * d, k_pages.to(bf).cuda(), v_pages.to(bf).cuda(), tables.cuda(),
            torch.tensor([0, 1], dtype=torch.int32).cuda(), torch.tensor([ctx - 1], dtype=torch.int32).cuda())
    scale = 1.0 / math.sqrt(d)
    if kernel == "prefill":
        K().attn_prefill_mfma(*args, torch.tensor([0, 0, -1], dtype=torch.int32).cuda(), 1, nq, nkv, d, scale)
    else:
        splits = int(kernel[-1])
        scratch = torch.empty(max(1, K().attn_decode_scratch_floats(1, nq, splits, d))).cuda()
        K().attn_decode_mfma(*args, torch.tensor([0], dtype=torch.int32).cuda(), 1, nq, nkv, d, scale, 0, splits,
                             scratch)
    expect = torch.repeat_interleave(v[far_key].to(bf).float(), nq // nkv, dim=0).reshape(1, -1)
    torch.testing.assert_close(out.float().cpu(), expect, rtol=1e-2, atol=1e-2)


def _loud_key_case(nq, nkv, d, ctx, ql, qi, key, seed):
    """Random small q, k; query ``qi`` and key ``key`` get one large matching component, so that
    the key decides the query's output if (and only if) the query may see it."""
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(ctx + ql, nkv, d, generator=g) * 0.1
    v = torch.randn(ctx + ql, nkv, d, generator=g)
    q = torch.randn(ql, nq, d, generator=g) * 0.1
    q[qi, :, 0] = 40.0
    k[key, :, 0] = 40.0
    bf = torch.bfloat16
    return q.to(bf).float(), k.to(bf).float(), v.to(bf).float()


EDGES = ["self", "future", "window_first", "before_window"]


@pytest.mark.parametrize("kernel", ["generic", "prefill", "decode1", "decode3"])
@pytest.mark.parametrize("edge", EDGES)
def test_attention_edges_of_visibility(edge, kernel):
    """A loud key is put exactly on, and exactly one beyond, the causal limit and the window's
    first key of a query, for queries on both sides of the kernels' row and key tile borders.
    An edge that is off by one gives the wrong key's value, not a small error."""
    nq, nkv, d, page_size, window = 4, 2, 64, 16, 64
    scale = 1.0 / math.sqrt(d)
    bf = torch.bfloat16
    decode = kernel.startswith("decode")
    cases = [(c, 1, 0) for c in (70, 127, 128, 129, 200)] if decode else \
        [(70, 70, qi) for qi in (0, 7, 8, 31, 32, 33, 68)]
    for ctx, ql, qi in cases:
        pos = ctx + qi
        key = {"self": pos, "future": pos + 1, "window_first": pos - window + 1, "before_window": pos - window}[edge]
        if key >= ctx + ql:
            continue                                   # the last query has no future key in the cache
        q, k, v = _loud_key_case(nq, nkv, d, ctx, ql, qi, key, seed=pos)
        positions = torch.arange(ctx, ctx + ql)
        ref = attention_reference(q, k, v, positions, scale, window).reshape(ql, nq * d)
        visible = edge in ("self", "window_first")
        if visible:                                    # the oracle itself must show the effect
            torch.testing.assert_close(ref[qi].float().reshape(nq, d),
                                       torch.repeat_interleave(v[key], nq // nkv, dim=0), rtol=1e-3, atol=1e-3)
        k_pages, v_pages, tables = build_paged([k], [v], page_size, seed=pos)
        out = torch.full((ql, nq * d), float("nan"), dtype=bf).cuda()
        args = (out, q.reshape(ql, -1).to(bf).cuda(), nq * d, k_pages.to(bf).cuda(), v_pages.to(bf).cuda(),
                tables.cuda())
        cu = torch.tensor([0, ql], dtype=torch.int32).cuda()
        cl = torch.tensor([ctx], dtype=torch.int32).cuda()
        if kernel == "generic":
            K().paged_attention_generic(*args, torch.zeros(ql, dtype=torch.int32).cuda(),
                                        positions.to(torch.int32).cuda(), nq, nkv, d, scale, window)
        elif kernel == "prefill":
            work, n_work = _prefill_work([(ctx, ql)], nq // nkv, d, window, "single")
            K().attn_prefill_mfma(*args, cu, cl, work, n_work, nq, nkv, d, scale, window)
        else:
            splits = int(kernel[-1])
            scratch = torch.empty(max(1, K().attn_decode_scratch_floats(1, nq, splits, d))).cuda()
            K().attn_decode_mfma(*args, cu, cl, torch.tensor([0], dtype=torch.int32).cuda(), 1, nq, nkv, d, scale,
                                 window, splits, scratch)
        torch.testing.assert_close(out.double().cpu(), ref, rtol=2e-2, atol=2e-2,
                                   msg=lambda m: f"context {ctx}, query {qi}, key {key}: {m}")


@pytest.mark.parametrize("kernel", ["prefill", "decode1", "decode4", "decode16"])
@pytest.mark.parametrize("heads", [(8, 2), (16, 2)], ids=["4-a-group", "8-a-group"])
@pytest.mark.parametrize("ctx", [8191, 16400, 32767])
def test_mfma_attention_over_long_contexts_at_head_size_128(kernel, ctx, heads):
    """Heads of 128, 4 or 8 per kv head (the 8B/14B and the 32B geometry), pages of 16, behind 8 k to 32 k keys.  Among thousands of random
    keys a missing page would change nothing that a tolerance sees, so every checked query has TWO
    loud keys far apart (the first key, a page's last slot in the middle, a page's first slot, the
    newest key): its output is the mean of their two values, and a key that is lost, read from a
    wrong page or merged with a wrong weight shows as an error of half a value."""
    (nq, nkv), d, page_size = heads, 128, 16
    scale = 1.0 / math.sqrt(d)
    bf = torch.bfloat16
    decode = kernel.startswith("decode")
    ql = 1 if decode else 130
    mid = (ctx // 2) // page_size * page_size
    pairs = [(0, ctx + ql - 1), (mid - 1, mid), (15, ctx - 16), (mid + 16, ctx // 4 * 3 + 5)]
    g = torch.Generator().manual_seed(ctx)
    reqs, qs, ks, vs, checked = [], [], [], [], []
    for r, (a, b) in enumerate(pairs if decode else pairs[:2]):
        k = torch.randn(ctx + ql, nkv, d, generator=g) * 0.1
        v = torch.randn(ctx + ql, nkv, d, generator=g)
        q = torch.randn(ql, nq, d, generator=g) * 0.1
        for qi, comp in ((0, 0),) if decode else ((0, 0), (64, 1), (129, 2)):
            hi = min(b, ctx + qi)                      # a query cannot see beyond itself
            q[qi, :, comp] = 40.0
            k[a, :, comp] = 40.0
            k[hi, :, comp] = 40.0
            checked.append((r, qi))
        reqs.append((ctx, ql))
        qs.append(q.to(bf).float()), ks.append(k.to(bf).float()), vs.append(v.to(bf).float())
    k_pages, v_pages, tables = build_paged(ks, vs, page_size, seed=ctx)
    n = len(reqs) * ql
    out = torch.full((n, nq * d), float("nan"), dtype=bf).cuda()
    qbuf = torch.cat([q.reshape(ql, nq * d) for q in qs]).to(bf).cuda()
    cu = torch.tensor([i * ql for i in range(len(reqs) + 1)], dtype=torch.int32).cuda()
    cl = torch.tensor([ctx] * len(reqs), dtype=torch.int32).cuda()
    args = (out, qbuf, nq * d, k_pages.to(bf).cuda(), v_pages.to(bf).cuda(), tables.cuda(), cu, cl)
    if decode:
        splits = int(kernel[6:])
        scratch = torch.full((max(1, K().attn_decode_scratch_floats(len(reqs), nq, splits, d)),), float("nan")).cuda()
        K().attn_decode_mfma(*args, None, len(reqs), nq, nkv, d, scale, 0, splits, scratch)
    else:
        work, n_work = _prefill_work(reqs, nq // nkv, d, None, "planner")
        K().attn_prefill_mfma(*args, work, n_work, nq, nkv, d, scale, 0)
    got = out.double().cpu().reshape(len(reqs), ql, nq * d)
    for r, qi in checked:
        ref = attention_reference(qs[r][qi:qi + 1], ks[r], vs[r], torch.tensor([ctx + qi]), scale).reshape(nq * d)
        assert float(ref.abs().max()) > 0.5            # the oracle's answer is a mean of two values, not of thousands
        torch.testing.assert_close(got[r, qi], ref, rtol=2e-2, atol=2e-2, msg=lambda m: f"request {r}, query {qi}: {m}")


def test_mfma_attention_ignores_garbage_past_the_context():
    """Slots of the last page beyond the context hold NaN and infinity: they must not leak."""
    nq, nkv, d, page_size = 4, 2, 64, 16
    reqs = [(0, 21), (37, 1)]
    qs, ks, vs, dev = _mfma_inputs(nq, nkv, d, page_size, reqs, seed=3)
    for r, (c, ql) in enumerate(reqs):
        n = c + ql
        page = int(dev["tables"][r, n // page_size])
        dev["k_pages"][page, :, n % page_size:] = float("nan")
        dev["v_pages"][page, :, :, n % page_size:] = float("inf")
    scale = 1.0 / math.sqrt(d)
    ref = _mfma_reference(qs, ks, vs, reqs, scale, None, nq, d)
    out = torch.zeros(dev["n"], nq * d, dtype=torch.bfloat16).cuda()
    K().attn_prefill_mfma(out, dev["q"], dev["stride"], dev["k_pages"], dev["v_pages"], dev["tables"], dev["cu"],
                          dev["ctx"], torch.tensor([0, 0, -1], dtype=torch.int32).cuda(), 1, nq, nkv, d, scale)
    K().attn_decode_mfma(out, dev["q"], dev["stride"], dev["k_pages"], dev["v_pages"], dev["tables"], dev["cu"],
                         dev["ctx"], torch.tensor([1], dtype=torch.int32).cuda(), 1, nq, nkv, d, scale)
    torch.testing.assert_close(out.double().cpu(), ref, rtol=2e-2, atol=2e-2)


def test_mfma_attention_refuses_what_it_cannot_do():
    from jax_vllm_amd.ops.kernels import KernelArgumentError, mfma_attention_supported

    assert not mfma_attention_supported(torch.bfloat16, 80, 4)       # page size not a multiple of 8
    assert not mfma_attention_supported(torch.bfloat16, 72, 16)      # head size not a multiple of 16
    assert not mfma_attention_supported(torch.bfloat16, 272, 16)     # head size above 256
    assert not mfma_attention_supported(torch.float32, 64, 16)
    nq, nkv, d, page_size = 3, 1, 80, 4
    qs, ks, vs, dev = _mfma_inputs(nq, nkv, d, page_size, [(3, 2)])
    out = torch.zeros(dev["n"], nq * d, dtype=torch.bfloat16).cuda()
    with pytest.raises(KernelArgumentError, match="multiple of 8"):
        K().attn_prefill_mfma(out, dev["q"], dev["stride"], dev["k_pages"], dev["v_pages"], dev["tables"], dev["cu"],
                              dev["ctx"], torch.tensor([0, 0, -1], dtype=torch.int32).cuda(), 1, nq, nkv, d, 0.1)


# ------------------------------------------------------------------ weight-streaming matrix product
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("m,n,k,shape", [
    (1, 96, 64, (0, 0, 0)), (8, 224, 96, (0, 0, 0)), (33, 520, 136, (2, 3, 2)), (64, 100, 4096, (0, 0, 0)),
    (5, 777, 80, (1, 16, 2)), (17, 64, 12288, (1, 8, 4)), (3, 30, 264, (1, 1, 8)), (16, 48, 2056, (0, 0, 0)),
    (8, 24576, 512, (0, 0, 0)), (48, 6144, 1024, (4, 2, 2)), (1, 6144, 4096, (1, 8, 4)), (9, 160, 4096, (4, 4, 8)),
    (1, 8200, 4096, (0, 0, 0)), (2, 100, 4096, (-1, 8, 16)), (8, 333, 1000, (-1, 16, 4)), (16, 64, 12288, (-1, 4, 8)),
    (11, 50, 72, (-1, 3, 4)), (8, 24576, 512, (-2, 64, 4)), (16, 333, 4096, (-2, 7, 16)), (5, 777, 2000, (-2, 1000, 8)),
    (3, 100, 72, (-2, 3, 4)), (1, 8200, 4096, (-2, 256, 16)), (17, 333, 1000, (-2, 40, 4)), (32, 4096, 2048, (-2, 256, 8)),
    (25, 50, 1200, (-2, 9, 5)), (40, 333, 1000, (-2, 40, 4)), (64, 200, 1280, (-2, 30, 5)), (49, 77, 1016, (-2, 3, 4)), (8, 200, 4904, (-2, 16, 20)),
    # 17..32 rows with 12 or 16 pieces a wave: W goes through four slots
    (24, 777, 4096, (-2, 20, 16)), (32, 300, 4000, (-2, 5, 16)), (17, 200, 3072, (-2, 3, 12)), (30, 64, 2904, (-2, 100, 12))])
def test_gemm_skinny(m, n, k, shape, out_dtype):
    x = randn(m, k, dtype=torch.bfloat16, seed=30, scale=0.5)
    w = randn(n, k, dtype=torch.bfloat16, seed=31, scale=0.5)
    out = K().gemm_skinny(x, w, out_dtype, block_shape=shape)
    ref = x.double() @ w.double().T
    if out_dtype == torch.float32:
        # float accumulation of exact bf16 products
        torch.testing.assert_close(out.double(), ref, rtol=1e-4, atol=1e-4 * math.sqrt(k))
    else:
        torch.testing.assert_close(out.double(), ref, rtol=1e-2, atol=1e-2 * math.sqrt(k) / 4)
    # a row's result does not depend on the other rows of the batch: bit for bit with a fixed
    # block shape (fixed summation order), to rounding when the shape is chosen from M
    if m > 1:
        one = K().gemm_skinny(x[2:3].contiguous() if m > 2 else x[:1].contiguous(), w, out_dtype, block_shape=shape)
        exact = dict(rtol=0, atol=0) if shape != (0, 0, 0) else dict(rtol=1e-2, atol=1e-3)
        torch.testing.assert_close(one, out[2:3] if m > 2 else out[:1], **exact)


@pytest.mark.parametrize("m,n,k,shape,ksplit", [(8, 4096, 4096, (-1, 4, 4), 4), (1, 100, 12288, (-1, 4, 4), 4),
                                                (16, 333, 1000, (-1, 8, 2), 2), (5, 64, 2560, (-1, 4, 4), 3),
                                                (3, 48, 1000, (-1, 2, 2), 4), (8, 4096, 4096, (-2, 512, 4), 4),
                                                (16, 130, 3000, (-2, 10, 4), 3), (2, 64, 12288, (-2, 30, 16), 3),
                                                (32, 4096, 4096, (-2, 256, 4), 4), (20, 136, 5120, (-2, 33, 5), 4),
                                                (64, 520, 4096, (-2, 256, 4), 4), (41, 136, 4800, (-2, 7, 5), 4),
                                                (24, 136, 12288, (-2, 4, 16), 3), (32, 100, 9000, (-2, 3, 12), 3)])
def test_gemm_skinny_shares_out_the_inner_size(m, n, k, shape, ksplit):
    """Partial products [ksplit, M, N] in float: part s covers its own columns only, and the
    ordered sum is the product."""
    x = randn(m, k, dtype=torch.bfloat16, seed=34, scale=0.5)
    w = randn(n, k, dtype=torch.bfloat16, seed=35, scale=0.5)
    parts = K().gemm_skinny(x, w, torch.float32, block_shape=shape, ksplit=ksplit)
    assert parts.shape == (ksplit, m, n) and parts.dtype == torch.float32
    if shape[0] == -2:
        k_per = 256 * shape[2]                   # 8 waves x pieces x 32 columns per group
    else:
        kp = shape[1] * shape[2] * 32
        k_per = -(-(-(-k // kp)) // ksplit) * kp
    for s in range(ksplit):
        lo, hi = s * k_per, min(k, (s + 1) * k_per)
        ref = x[:, lo:hi].double() @ w[:, lo:hi].double().T
        torch.testing.assert_close(parts[s].double().cpu(), ref.cpu(), rtol=1e-4, atol=1e-3)
    again = K().gemm_skinny(x, w, torch.float32, block_shape=shape, ksplit=ksplit)
    assert torch.equal(parts, again)
    from jax_vllm_amd.ops.kernels import KernelArgumentError
    with pytest.raises((KernelArgumentError, RuntimeError)):
        K().gemm_skinny(x, w, torch.float32, block_shape=shape, ksplit=1000)   # more parts than phases


TILE64_CASES = [(17, 64, 256, 1), (64, 128, 2048, 4), (33, 200, 1000, 2), (48, 72, 3080, 3), (64, 64, 264, 2),
                (20, 4096, 12288, 4), (1, 130, 520, 1), (64, 5120, 17408, 3)]


@pytest.mark.parametrize("m,n,k,ksplit", TILE64_CASES)
def test_gemm_tile64(m, n, k, ksplit):
    """Blocks of 64 rows of w against up to 64 rows of x: whole products and partial products of a
    shared-out inner size, at sizes that end inside a tile of w, inside a row tile of x, inside a
    chunk of 256 columns and inside a 32-column step; rows of x and w beyond the sizes and columns
    beyond a block's share must contribute nothing."""
    x = randn(m, k, dtype=torch.bfloat16, seed=51, scale=0.5)
    w = randn(n, k, dtype=torch.bfloat16, seed=52, scale=0.1)
    ref = x.double() @ w.double().T
    out_dtype = torch.float32 if ksplit > 1 else torch.bfloat16
    y = K().gemm_tile64(x, w, out_dtype, ksplit=ksplit)
    if ksplit > 1:
        assert y.shape == (ksplit, m, n) and y.dtype == torch.float32
        torch.testing.assert_close(y.sum(0).double(), ref, rtol=1e-3, atol=2e-3 * math.sqrt(k) / 8)
        # every group holds its own columns only: group 0 equals the product over its share
        share = -(-(-(-k // 256)) // ksplit) * 256
        torch.testing.assert_close(y[0].double(), x[:, :share].double() @ w[:, :share].double().T,
                                   rtol=1e-3, atol=2e-3 * math.sqrt(k) / 8)
    else:
        assert y.shape == (m, n) and y.dtype == torch.bfloat16
        torch.testing.assert_close(y.double(), ref, rtol=2e-2, atol=2e-2 * math.sqrt(k) / 8)
        yf = K().gemm_tile64(x, w, torch.float32)
        torch.testing.assert_close(yf.double(), ref, rtol=1e-3, atol=2e-3 * math.sqrt(k) / 8)
    # the same call again gives the same bits (fixed order of every sum)
    torch.testing.assert_close(K().gemm_tile64(x, w, out_dtype, ksplit=ksplit), y, rtol=0, atol=0)


@pytest.mark.parametrize("act", ACTIVATIONS)
def test_gemm_tile64_activation_epilogue_and_refusals(act):
    x = randn(40, 1024, dtype=torch.bfloat16, seed=53, scale=0.5)
    w = randn(300, 1024, dtype=torch.bfloat16, seed=54, scale=0.1)
    g, u = w[0::2].double(), w[1::2].double()
    want = gate_activation(act, x.double() @ g.T) * (x.double() @ u.T)
    got = K().gemm_tile64(x, w, gate_pairs=act)
    assert got.shape == (40, 150)
    torch.testing.assert_close(got.double(), want, rtol=2e-2, atol=2e-2)
    with pytest.raises(ValueError):
        K().gemm_tile64(x, w, gate_pairs="relu")                                    # no such kernel
    with pytest.raises(ValueError):
        K().gemm_tile64(randn(65, 1024, dtype=torch.bfloat16), w)                    # more than 64 rows
    with pytest.raises(ValueError):
        K().gemm_tile64(x, w, torch.float32, ksplit=5)                              # 4 chunks of 256 for 5 groups
    with pytest.raises(ValueError):
        K().gemm_tile64(x, w, torch.bfloat16, ksplit=2)                             # partial products are float32
    with pytest.raises(ValueError):
        K().gemm_tile64(x, w, gate_pairs=act, ksplit=2, out_dtype=torch.float32)   # no activation of a partial sum


@pytest.mark.parametrize("m,hidden,n_parts", [(8, 4096, 4), (1, 512, 2), (16, 5120, 3), (5, 8192, 1)])
def test_residual_step_that_leaves_the_scale_to_the_product(m, hidden, n_parts):
    """``add_parts_unscaled`` adds the partial products to the residual stream and hands on h * weight
    with the shares of each row's sum of squares; a product by the blocks that stay multiplies its
    output rows by the norm's scale.  Together they equal norm-then-product."""
    kern = K()
    h = randn(m, hidden, seed=70, scale=2.0)
    parts = randn(n_parts, m, hidden, seed=71)
    weight = 1 + 0.1 * randn(hidden, seed=72)
    eps = 1e-5
    total = parts[0]
    for q in range(1, n_parts):
        total = total + parts[q]
    want_h = h + total
    h2 = h.clone()
    rows = kern.add_parts_unscaled(h2, parts, weight, eps)
    torch.testing.assert_close(h2, want_h, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(rows.x.float(), (want_h * weight).to(torch.bfloat16).float(), rtol=0, atol=0)
    assert rows.ssq.shape == (m, 16) and rows.shares == hidden // 512
    torch.testing.assert_close(rows.ssq[:, :rows.shares].sum(-1), (want_h * want_h).sum(-1), rtol=1e-5, atol=1e-5)
    # the product: qkv-like (partial products) and gate/up-like (activation as epilogue)
    inv = torch.rsqrt((want_h.double() ** 2).mean(-1, keepdim=True) + eps)
    xn = rows.x.double() * inv                      # what the reader multiplies, to the rounding of x
    n = 1024
    w = randn(n, hidden, dtype=torch.bfloat16, seed=73, scale=0.05)
    assert kern.linear_takes_unscaled_rows(m, w, partial_ok=True) == (hidden != 512)     # no piece count covers 512 columns
    if kern.linear_takes_unscaled_rows(m, w, partial_ok=True):
        y = kern.linear(rows, w, partial_ok=True)
        y = y.sum(0) if y.dim() == 3 else y.float()
        torch.testing.assert_close(y.double(), xn @ w.double().T, rtol=2e-2, atol=2e-2)
    wide = randn(2 * 16 * 4 * 256, hidden, dtype=torch.bfloat16, seed=74, scale=0.05)     # 1,024 row tiles: the wide plan
    if kern.linear_takes_unscaled_rows(m, wide, gate_pairs=True):
        z = kern.linear(rows, wide, gate_pairs="silu")
        full = xn @ wide.double().T
        gate, up = full[:, 0::2], full[:, 1::2]
        torch.testing.assert_close(z.double(), gate / (1 + torch.exp(-gate)) * up, rtol=3e-2, atol=3e-2)
    # rows that were not made for this x are refused, and so is a plan that cannot scale
    other = kern.UnscaledRows(rows.x.clone(), rows.ssq, hidden, eps)
    with pytest.raises(kern.KernelArgumentError, match="does not belong"):
        kern.gemm_skinny(rows.x, w, torch.float32, block_shape=(-2, 64, 4), ksplit=max(1, -(-hidden // 1024)), row_scale=other)


def test_linear_takes_blocks_of_64_rows_for_a_long_inner_size():
    """17..64 rows against a narrow matrix with a long inner size (the feed-forward's second product):
    ``linear`` hands out partial products from ``gemm_tile64`` that ``add_rmsnorm`` adds; the same
    product without a reader for partial sums is the library's."""
    kern = K()
    m, n, k = 40, 1024, 12288
    x = randn(m, k, dtype=torch.bfloat16, seed=55, scale=0.5)
    w = randn(n, k, dtype=torch.bfloat16, seed=56, scale=0.05)
    plan = kern.streaming_plan(m, n, k, partial_ok=True, device=x.device)
    assert plan == (kern.TILE64, 4)
    assert kern.streaming_plan(m, n, k, partial_ok=False, device=x.device) is None
    assert kern.streaming_plan(m, n, 4096, partial_ok=True, device=x.device) == ((-2, 256, 4), 4)   # too few columns a block of 64 rows: staying blocks
    assert kern.streaming_plan(m, n, 8192, partial_ok=True, device=x.device) is None      # ... unless x would not fit their registers
    few = kern.streaming_plan(12, 5120, 17408, partial_ok=True, device=x.device)     # not the library's either
    assert few is not None and few[1] == 4 and few[0][0] in (-1, -2)
    parts = kern.linear(x, w, partial_ok=True)
    assert parts.shape == (4, m, n) and parts.dtype == torch.float32
    ref = x.double() @ w.double().T
    torch.testing.assert_close(parts.sum(0).double(), ref, rtol=1e-3, atol=2e-2)
    torch.testing.assert_close(kern.linear(x, w).double(), ref, rtol=2e-2, atol=2e-1)
    # the reader: residual + ordered sum of the parts, then the norm
    h = randn(m, n, seed=57)
    weight = 1 + 0.1 * randn(n, seed=58)
    h2 = h.clone()
    out = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    kern.add_rmsnorm(h2, parts, weight, out, 1e-6)
    want_h = h + ((parts[0] + parts[1]) + parts[2]) + parts[3]
    torch.testing.assert_close(h2, want_h, rtol=1e-6, atol=1e-6)
    want = want_h * torch.rsqrt((want_h * want_h).mean(-1, keepdim=True) + 1e-6) * weight
    torch.testing.assert_close(out.float(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("k", [512, 1000, 1024, 2560, 3072, 5120, 6152, 12288])
def test_linear_at_every_size_runs_a_plan_the_library_accepts(k):
    """Whatever ``streaming_plan`` picks for a size must be a plan the kernels accept and must give
    the product: rows 1..64, widths and inner sizes that are no powers of two, inner sizes that do
    not share out evenly (3,072 = 6 phases for 4 groups), with and without a reader of partial
    products, with and without the silu epilogue."""
    kern = K()
    for n in (64, 1000, 1024, 4104):
        w = randn(n, k, dtype=torch.bfloat16, seed=n + k, scale=0.05)
        for m in (1, 5, 8, 12, 16, 17, 40, 64):
            x = randn(m, k, dtype=torch.bfloat16, seed=m, scale=0.5)
            ref = x.double() @ w.double().T
            tol_ = dict(rtol=2e-2, atol=2e-2 * math.sqrt(k) / 8)
            y = kern.linear(x, w, partial_ok=True)
            y = y.sum(0) if y.dim() == 3 else y
            torch.testing.assert_close(y.double(), ref, **tol_)
            torch.testing.assert_close(kern.linear(x, w).double(), ref, **tol_)
            act = kern.linear(x, w, gate_pairs="silu")
            want = torch.nn.functional.silu(ref[:, 0::2]) * ref[:, 1::2]
            torch.testing.assert_close(act.double(), want, rtol=3e-2, atol=3e-2 * math.sqrt(k) / 8)


def test_linear_follows_its_plan_and_all_roads_agree():
    """``linear`` at few rows: the staying blocks, the shared-out inner size, the staged chunks and
    the library must give the same numbers up to rounding, with and without the silu epilogue."""
    kern = K()
    x = randn(8, 4096, dtype=torch.bfloat16, seed=36, scale=0.5)
    wide = randn(16640, 4096, dtype=torch.bfloat16, seed=37, scale=0.1)      # 1,040 row tiles: blocks that stay
    narrow = randn(512, 4096, dtype=torch.bfloat16, seed=38, scale=0.1)      # 32 row tiles: inner size shared out
    assert kern.streaming_plan(8, 16640, 4096, gate_pairs=True, device=x.device)[0][0] == -2
    plan = kern.streaming_plan(8, 512, 4096, partial_ok=True, device=x.device)
    assert plan[1] == 4 and kern.streaming_plan(8, 512, 4096, partial_ok=False, device=x.device) == ((0, 0, 0), 1)
    assert kern.streaming_plan(17, 512, 4096, device=x.device) is None       # the library's
    ref = x.double() @ narrow.double().T
    parts = kern.linear(x, narrow, partial_ok=True)
    assert plan[0][0] == -2 and parts.shape == (4, 8, 512) and parts.dtype == torch.float32
    torch.testing.assert_close(parts.sum(0).double(), ref, rtol=1e-3, atol=1e-2)
    torch.testing.assert_close(kern.linear(x, narrow).double(), ref, rtol=2e-2, atol=5e-2)
    g, u = wide[0::2].double(), wide[1::2].double()
    ref_act = torch.nn.functional.silu(x.double() @ g.T) * (x.double() @ u.T)
    assert kern.streaming_plan(24, 16640, 4096, gate_pairs=True, device=x.device)[0] == (-2, kern.compute_units(x.device), 16)
    assert kern.streaming_plan(40, 16640, 4096, gate_pairs=True, device=x.device) is None
    for rows in (8, 24, 40):                    # staying blocks; the same with two row tiles of x; library + activation kernel
        xi = x if rows == 8 else randn(rows, 4096, dtype=torch.bfloat16, seed=39, scale=0.5)
        want = ref_act if rows == 8 else torch.nn.functional.silu(xi.double() @ g.T) * (xi.double() @ u.T)
        got = kern.linear(xi, wide, gate_pairs="silu")
        assert got.shape == (rows, 8320) and got.dtype == torch.bfloat16
        torch.testing.assert_close(got.double(), want, rtol=2e-2, atol=5e-2)


@pytest.mark.parametrize("m,inter,k,shape", [(1, 176, 80, (0, 0, 0)), (8, 12288, 96, (0, 0, 0)), (40, 224, 104, (0, 0, 0)),
                                             (16, 1000, 4096, (0, 0, 0)), (8, 1000, 4096, (-2, 256, 16)),
                                             (3, 177, 1000, (-2, 5, 4)), (24, 1000, 4096, (-2, 256, 16)),
                                             (32, 177, 3000, (-2, 5, 12))])
@pytest.mark.parametrize("act", ACTIVATIONS)
def test_gemm_skinny_activation_epilogue(m, inter, k, shape, act):
    """Rows of w alternate gate and up rows; the product comes out as act(gate) * up."""
    x = randn(m, k, dtype=torch.bfloat16, seed=32, scale=0.7)
    wg = randn(inter, k, dtype=torch.bfloat16, seed=33, scale=0.3)
    wu = randn(inter, k, dtype=torch.bfloat16, seed=34, scale=0.3)
    w = torch.stack([wg, wu], dim=1).reshape(2 * inter, k).contiguous()
    out = K().gemm_skinny(x, w, torch.bfloat16, gate_pairs=act, block_shape=shape)
    assert out.shape == (m, inter)
    ref = gate_activation(act, x.double() @ wg.double().T) * (x.double() @ wu.double().T)
    torch.testing.assert_close(out.double(), ref, rtol=2e-2, atol=2e-2 * math.sqrt(k) / 4)
