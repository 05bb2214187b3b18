"""Each kernel alone against a plain float32 torch formula, at sizes other than the engine's."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_llama as P  # noqa: E402

PAGE = 64


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from fms_amd.kernels import load, ops as _ops

    load()
    return _ops


def dev(t):
    return t.to("cuda")


def tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


# --------------------------------------------------------------------------
def test_embed(ops):
    torch.manual_seed(0)
    for dtype in (torch.float32, torch.bfloat16):
        table = torch.randn(37, 24).to(dtype)
        ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32)
        out = ops.embed(dev(ids), dev(table)).cpu()
        assert out.dtype == torch.float32
        assert torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("width", [24, 100, 4096, 9000, 20000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_norm(ops, width, dtype):
    torch.manual_seed(1)
    T = 5
    resid = torch.randn(T, width) * 2
    branch = torch.randn(T, width).to(dtype)
    weight = (1 + 0.3 * torch.randn(width)).to(dtype)
    eps = 1e-3
    want_resid = resid + branch.float()
    want = P.rms_norm(want_resid, weight.float(), eps)
    r = dev(resid.clone())
    out = ops.add_norm(r, dev(branch), dev(weight), None, eps, dtype)
    torch.testing.assert_close(r.cpu(), want_resid)
    torch.testing.assert_close(out.cpu().float(), want, **tol(dtype))
    # no branch; selected rows only; the stream is left alone
    r2 = dev(resid.clone())
    rows = torch.tensor([3, 0], dtype=torch.int32)
    out2 = ops.add_norm(r2, dev(branch), dev(weight), None, eps, dtype, rows=dev(rows))
    torch.testing.assert_close(out2.cpu().float(), want[rows.long()], **tol(dtype))
    assert torch.equal(r2.cpu(), resid)
    out3 = ops.add_norm(dev(resid.clone()), None, dev(weight), None, eps, dtype)
    torch.testing.assert_close(out3.cpu().float(), P.rms_norm(resid, weight.float(), eps), **tol(dtype))


def test_add_norm_with_mean_and_shift(ops):
    torch.manual_seed(2)
    x = torch.randn(3, 48) + 1.5
    w, b = torch.randn(48), torch.randn(48)
    out = ops.add_norm(dev(x.clone()), None, dev(w), dev(b), 1e-5, torch.float32, use_mean=True)
    torch.testing.assert_close(out.cpu(), torch.nn.functional.layer_norm(x, (48,), w, b, 1e-5), atol=1e-5, rtol=1e-5)
    # a float32 weight with bfloat16 activations (a tensor the checkpoint keeps in 32-bit)
    out = ops.add_norm(dev(x.clone()), None, dev(w), None, 1e-5, torch.bfloat16)
    torch.testing.assert_close(out.cpu().float(), P.rms_norm(x, w, 1e-5), atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_act(ops, dtype):
    torch.manual_seed(3)
    gu = torch.randn(7, 2 * 44).to(dtype)
    bias = torch.randn(2 * 44).to(dtype)
    out = ops.gated_act(dev(gu), dev(bias), "swish").cpu().float()
    g = gu.float() + bias.float()
    torch.testing.assert_close(out, P.silu(g[:, :44]) * g[:, 44:], **tol(dtype))
    out = ops.gated_act(dev(gu), None, "silu").cpu().float()
    torch.testing.assert_close(out, P.silu(gu.float()[:, :44]) * gu.float()[:, 44:], **tol(dtype))


def test_cast_and_bias(ops):
    x = torch.randn(1000)
    assert torch.equal(ops.cast(dev(x), torch.bfloat16).cpu(), x.to(torch.bfloat16))
    assert torch.equal(ops.cast(dev(x.to(torch.bfloat16)), torch.float32).cpu(), x.to(torch.bfloat16).float())
    m = torch.randn(4, 10)
    b = torch.randn(10)
    torch.testing.assert_close(ops.bias_add_(dev(m.clone()), dev(b)).cpu(), m + b)


def test_rope_table(ops):
    freqs = P.rope_frequencies(24, 500000.0)
    cos, sin = ops.rope_table(dev(freqs), 300)
    angles = torch.outer(torch.arange(300).float(), freqs)
    torch.testing.assert_close(cos.cpu(), torch.cos(angles), atol=2e-6, rtol=0)
    torch.testing.assert_close(sin.cpu(), torch.sin(angles), atol=2e-6, rtol=0)
    # large angles keep their accuracy (positions in the thousands times frequency one)
    cos, sin = ops.rope_table(dev(torch.tensor([1.0, 0.37])), 9000)
    a = torch.outer(torch.arange(9000).float(), torch.tensor([1.0, 0.37]))
    torch.testing.assert_close(cos.cpu(), torch.cos(a.double()).float(), atol=5e-7, rtol=0)


# --------------------------------------------------------------------------
# paged cache helpers
# --------------------------------------------------------------------------
def make_pages(lengths, K, D, dtype, seed=0, extra_pages=3):
    """Random page assignment: returns (block_table [B, P] int32, n_pages)."""
    g = torch.Generator().manual_seed(seed)
    per_seq = [-(-n // PAGE) for n in lengths]
    total = sum(per_seq) + extra_pages
    perm = torch.randperm(total, generator=g).tolist()
    width = max(per_seq)
    table = torch.full((len(lengths), width), -1, dtype=torch.int32)
    it = iter(perm)
    for b, n in enumerate(per_seq):
        for i in range(n):
            table[b, i] = next(it)
    return table, total


def fill_cache(table, ks, vs, n_pages, dtype):
    """ks[b]: [len, K, D] -> caches in the kernels' layout."""
    K, D = ks[0].shape[1:]
    kc = torch.zeros(n_pages, K, PAGE, D, dtype=dtype)
    vc = torch.zeros(n_pages, K, D, PAGE, dtype=dtype)
    for b, (k, v) in enumerate(zip(ks, vs)):
        for pos in range(k.shape[0]):
            page = int(table[b, pos // PAGE])
            kc[page, :, pos % PAGE, :] = k[pos].to(dtype)
            vc[page, :, :, pos % PAGE] = v[pos].to(dtype)
    return kc, vc


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,K,D,rot", [(4, 2, 16, 16), (3, 1, 24, 24), (2, 2, 32, 16), (2, 1, 6, 6), (8, 2, 128, 128), (3, 3, 256, 64)])
@pytest.mark.parametrize("starts,lens", [([0, 70, 5], [9, 3, 130]), ([0, 64, 8, 3], [200, 72, 56, 13])])
def test_rope_kv_write(ops, dtype, H, K, D, rot, starts, lens):
    """The second layout has runs of tokens that start at multiples of 8 places of their pages and cross page
    borders (whole 16-byte pieces of the transposed value pages), the first has none to speak of."""
    torch.manual_seed(4)
    total = [s + n for s, n in zip(starts, lens)]
    table, n_pages = make_pages(total, K, D, dtype, seed=1)
    T = sum(lens)
    qkv = torch.randn(T, (H + 2 * K) * D).to(dtype)
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)]).int()
    seq = torch.cat([torch.full((n,), b) for b, n in enumerate(lens)]).int()
    freqs = P.rope_frequencies(rot, 10000.0)
    cos, sin = ops.rope_table(dev(freqs), 256)
    kc = torch.zeros(n_pages, K, PAGE, D, dtype=dtype, device="cuda")
    vc = torch.zeros(n_pages, K, D, PAGE, dtype=dtype, device="cuda")
    q_dev = dev(qkv.clone())
    ops.rope_kv_write(q_dev, dev(positions), dev(seq), dev(table), cos, sin, rot, kc, vc, H, K, D)
    out = q_dev.cpu().float()
    x = qkv.float()
    q = x[:, : H * D].reshape(T, H, D)
    k = x[:, H * D : (H + K) * D].reshape(T, K, D)
    v = x[:, (H + K) * D :].reshape(T, K, D)

    def rotate(t):
        r = P.rope_rotate(t[..., :rot], positions, freqs)
        return torch.cat([r, t[..., rot:]], dim=-1)

    torch.testing.assert_close(out[:, : H * D].reshape(T, H, D), rotate(q), **tol(dtype))
    # v columns of qkv untouched
    assert torch.equal(out[:, (H + K) * D :], x[:, (H + K) * D :])
    kc, vc = kc.cpu().float(), vc.cpu().float()
    rk = rotate(k)
    for t in range(T):
        page = int(table[int(seq[t]), int(positions[t]) // PAGE])
        off = int(positions[t]) % PAGE
        torch.testing.assert_close(kc[page, :, off, :], rk[t], **tol(dtype))
        torch.testing.assert_close(vc[page, :, :, off], v[t].to(dtype).float(), **tol(dtype))
    # pages of no sequence stay zero: nothing was written elsewhere
    used = set(int(p) for p in table.flatten() if p >= 0)
    for p in range(n_pages):
        if p not in used:
            assert float(kc[p].abs().sum()) == 0 and float(vc[p].abs().sum()) == 0


@pytest.mark.parametrize("M", [1, 8, 20, 32, 40, 64, 81, 128, 129, 150, 161, 192])
@pytest.mark.parametrize("H,K,D,rot,E", [(4, 2, 16, 16, 64), (3, 1, 48, 48, 40), (8, 8, 32, 16, 256), (40, 4, 128, 128, 32), (30, 2, 136, 136, 32)])
def test_qkv_rope_write_equals_the_separate_kernels(ops, M, H, K, D, rot, E):
    """The decode-time fusion (projection + rotation + cache write) against linear followed by rope_kv_write."""
    torch.manual_seed(11)
    dtype = torch.bfloat16
    N = (H + 2 * K) * D
    x = torch.randn(M, E).to(dtype)
    w = (torch.randn(N, E) * 0.2).to(dtype)
    bias = torch.randn(N).to(dtype)
    positions = torch.randint(0, 200, (M,)).int()
    seq = torch.arange(M).int()
    if M > 2:
        seq[1] = -1  # a padding row: nothing of it may reach the cache
        seq[2:] -= 1
    n_seqs = int(seq.max()) + 1
    table, n_pages = make_pages([256] * n_seqs, K, D, dtype, seed=3)
    freqs = P.rope_frequencies(rot, 10000.0)
    cos, sin = ops.rope_table(dev(freqs), 256)
    for b in (None, bias):
        caches = []
        outs = []
        for fused in (False, True):
            kc = torch.zeros(n_pages, K, PAGE, D, dtype=dtype, device="cuda")
            vc = torch.zeros(n_pages, K, D, PAGE, dtype=dtype, device="cuda")
            args = (dev(positions), dev(seq), dev(table), cos, sin, rot, kc, vc, H, K, D)
            if fused:
                qkv = ops.qkv_rope_write(dev(x), dev(w), None if b is None else dev(b), *args)
            else:
                qkv = ops.linear(dev(x), dev(w), None if b is None else dev(b))
                ops.rope_kv_write(qkv, *args)
            outs.append(qkv[:, : H * D].cpu().float()[seq >= 0])  # a padding row's queries are never read
            caches.append((kc.cpu().float(), vc.cpu().float()))
        # The separate kernels round the projection to bfloat16 before they rotate it, the fused kernel rotates the
        # float32 sums: an element that the rotation makes small out of two large ones differs by up to the rounding
        # of those two, half a bfloat16 step (2^-9 of the largest value) each.
        step = 2.0 ** -8 * max(float(outs[0].abs().max()), float(caches[0][0].abs().max()))
        torch.testing.assert_close(outs[1], outs[0], atol=step, rtol=2e-2)
        torch.testing.assert_close(caches[1][0], caches[0][0], atol=step, rtol=2e-2)
        torch.testing.assert_close(caches[1][1], caches[0][1], atol=2e-2, rtol=2e-2)
        assert float(caches[0][0].abs().sum()) > 0


# --------------------------------------------------------------------------
def reference_attention(qs, ks, vs, starts, H, K, scale=None, window=0):
    """qs[b]: [n_b, H, D] queries at positions starts[b]..; ks/vs[b]: [len_b, K, D] all keys."""
    outs = []
    for q, k, v, s in zip(qs, ks, vs, starts):
        n = q.shape[0]
        full_q = torch.zeros(k.shape[0], H, q.shape[2])
        full_q[s : s + n] = q
        o = P.causal_attention(full_q, k.float(), v.float(), scale=scale, window=window)
        outs.append(o[s : s + n])
    return torch.cat(outs).reshape(sum(q.shape[0] for q in qs), -1)


def reference_attention_rows(qs, ks, vs, starts, H, K, scale=None, window=0):
    """The same attention for the query rows only (fms/modules/attention.py:215-294: head h reads kv head
    h // (H / K), key j is visible to the query at position p if j <= p, and p - j < window if there is one):
    for contexts so long that the whole square of scores of causal_attention would not fit."""
    outs = []
    for q, k, v, s in zip(qs, ks, vs, starts):
        n, _, D = q.shape
        sc = scale if scale is not None else 1 / math.sqrt(D)
        pos = torch.arange(s, s + n)[:, None]
        key = torch.arange(k.shape[0])[None, :]
        visible = key <= pos
        if window:
            visible &= pos - key < window
        o = torch.zeros(n, H, D)
        for h in range(H):
            kh = h // (H // K)
            scores = (q[:, h].double() @ k[:, kh].double().t()) * sc
            probs = torch.softmax(scores.masked_fill(~visible, float("-inf")), dim=-1)
            o[:, h] = (probs @ v[:, kh].double()).float()
        outs.append(o)
    return torch.cat(outs).reshape(sum(q.shape[0] for q in qs), -1)


def test_the_two_attention_references_agree():
    torch.manual_seed(3)
    ks, vs = [torch.randn(90, 2, 16)], [torch.randn(90, 2, 16)]
    qs = [torch.randn(7, 4, 16)]
    for window in (0, 20):
        torch.testing.assert_close(reference_attention_rows(qs, ks, vs, [83], 4, 2, window=window),
                                   reference_attention(qs, ks, vs, [83], 4, 2, window=window), atol=1e-5, rtol=1e-5)


def attention_case(ops, dtype, H, K, D, starts, lens, window=0, decode=False, scale=None, spike=False, **kw):
    torch.manual_seed(5)
    totals = [s + n for s, n in zip(starts, lens)]
    table, n_pages = make_pages(totals, K, D, dtype, seed=2)
    ks = [torch.randn(n, K, D).to(dtype).float() for n in totals]
    vs = [torch.randn(n, K, D).to(dtype).float() for n in totals]
    qs = [torch.randn(n, H, D).to(dtype).float() for n in lens]
    if spike:
        # one far key decides the result: a kernel that loses it (a split, a page, a mask edge) fails visibly
        for b in range(len(lens)):
            far = totals[b] // 3
            qs[b][-1, :, :] = 0
            qs[b][-1, :, 0] = 8.0
            ks[b][:, :, 0] = -1.0
            ks[b][far, :, 0] = 8.0
    kc, vc = fill_cache(table, ks, vs, n_pages, dtype)
    T = sum(lens)
    q_flat = torch.cat([q.reshape(q.shape[0], H * D) for q in qs]).to(dtype)
    # queries sit inside wider rows, as in the fused qkv buffer
    wide = torch.zeros(T, (H + 2 * K) * D, dtype=dtype)
    wide[:, : H * D] = q_flat
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)]).int()
    seq = torch.cat([torch.full((n,), b) for b, n in enumerate(lens)]).int()
    qblock = kw.pop("qblock", None) or ops.prefill_qblock(H, K, D, T)
    qb_start, qb_len, base = [], [], 0
    for n in lens:
        for off in range(0, n, qblock):
            qb_start.append(base + off)
            qb_len.append(min(qblock, n - off))
        base += n
    sc = scale if scale is not None else 1 / math.sqrt(D)
    out = ops.attention(
        dev(wide), dev(positions), dev(seq), dev(table), dev(kc), dev(vc), H, K, D, sc, window,
        decode=decode, max_context=max(totals),
        qblock_start=dev(torch.tensor(qb_start, dtype=torch.int32)), qblock_len=dev(torch.tensor(qb_len, dtype=torch.int32)), qblock_tokens=qblock, **kw,
    )
    rows_only = max(totals) > 3000  # the whole square of scores of a long context is too much for the plain function
    want = (reference_attention_rows if rows_only else reference_attention)(qs, ks, vs, starts, H, K, scale=sc, window=window)
    torch.testing.assert_close(out.cpu().float(), want, **(dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)))


@pytest.mark.parametrize("H,K,D", [(4, 2, 16), (4, 1, 24), (3, 3, 40), (2, 1, 8)])
def test_attention_generic_f32(ops, H, K, D):
    attention_case(ops, torch.float32, H, K, D, starts=[0, 0, 60], lens=[70, 1, 9])
    attention_case(ops, torch.float32, H, K, D, starts=[299, 64], lens=[1, 1], decode=True)


@pytest.mark.parametrize("H,K,D", [(4, 2, 16), (4, 1, 48), (6, 3, 128), (2, 2, 64), (32, 1, 32), (2, 1, 256), (5, 5, 80), (8, 2, 128), (12, 2, 64),
                                   (16, 2, 128), (4, 4, 128), (24, 1, 128)])
def test_attention_prefill_bf16(ops, H, K, D):
    attention_case(ops, torch.bfloat16, H, K, D, starts=[0, 0, 0], lens=[200, 1, 33])
    # a chunk that continues a cached prefix
    attention_case(ops, torch.bfloat16, H, K, D, starts=[100, 64, 0], lens=[70, 5, 129])
    attention_case(ops, torch.bfloat16, H, K, D, starts=[0, 30], lens=[300, 100])


@pytest.mark.parametrize("H,K,D", [(4, 2, 16), (4, 1, 48), (8, 2, 128), (2, 2, 64), (40, 2, 32), (2, 1, 256), (5, 5, 80),
                                   (16, 2, 128), (4, 4, 128), (24, 1, 128)])
def test_attention_decode_bf16(ops, H, K, D):
    attention_case(ops, torch.bfloat16, H, K, D, starts=[0, 63, 64, 700], lens=[1, 1, 1, 1], decode=True)
    attention_case(ops, torch.bfloat16, H, K, D, starts=[1500, 2], lens=[1, 1], decode=True, pages_per_block=2, waves=1)
    attention_case(ops, torch.bfloat16, H, K, D, starts=[1500, 2], lens=[1, 1], decode=True, pages_per_block=5, waves=3)
    attention_case(ops, torch.bfloat16, H, K, D, starts=[1500, 2], lens=[1, 1], decode=True, pages_per_block=24, waves=8)
    attention_case(ops, torch.bfloat16, H, K, D, starts=[1500, 2, 600], lens=[1, 1, 1], decode=True, pages_per_block=16, waves=4)
    # the order in which the blocks take the rows changes nothing; several pages a wave run as a pipeline
    attention_case(ops, torch.bfloat16, H, K, D, starts=[40, 1500, 2, 600], lens=[1, 1, 1, 1], decode=True, pages_per_block=24, waves=2,
                   row_order=dev(torch.tensor([1, 3, 0, 2], dtype=torch.int32)))
    if D == 128:
        # pages by way of LDS: blocks of up to 4 and of up to 8 waves, whole and partly filled pages, splits
        for pages, waves in ((64, 8), (64, 3), (5, 2), (2, 1), (16, 4)):
            attention_case(ops, torch.bfloat16, H, K, D, starts=[1500, 2, 600, 63, 64, 190], lens=[1, 1, 1, 1, 1, 1], decode=True,
                           pages_per_block=pages, waves=waves, staged=True)


@pytest.mark.parametrize("dtype,decode", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
def test_attention_far_key_and_window(ops, dtype, decode):
    lens = [1, 1] if decode else [40, 3]
    if decode:
        attention_case(ops, dtype, 8, 2, 128, starts=[900, 130], lens=lens, decode=True, spike=True, staged=True)
        attention_case(ops, dtype, 8, 2, 128, starts=[900, 130], lens=lens, decode=True, window=70, staged=True)
    attention_case(ops, dtype, 4, 2, 32, starts=[900, 130], lens=lens, decode=decode, spike=True)
    attention_case(ops, dtype, 4, 2, 32, starts=[900, 130], lens=lens, decode=decode, window=100)
    attention_case(ops, dtype, 4, 2, 32, starts=[900, 130], lens=lens, decode=decode, window=64, scale=0.3)
    attention_case(ops, dtype, 4, 2, 32, starts=[900, 130], lens=lens, decode=decode, window=1)


def test_attention_over_long_contexts(ops):
    """Contexts of 8200, 12000 and 20000 tokens beside short ones: the decode kernel with the split that the wrapper
    picks for such a bound and with others, pages through LDS and not, a far key that decides the result, a window
    whose edge lies thousands of tokens back; the prefill kernel for a chunk behind a cached prefix of 8000 tokens and for a prompt of 3200 tokens;
    the float32 kernel."""
    bf, f32 = torch.bfloat16, torch.float32
    attention_case(ops, bf, 8, 2, 128, starts=[8199, 19999, 2], lens=[1, 1, 1], decode=True, spike=True)
    attention_case(ops, bf, 8, 2, 128, starts=[8199, 19999, 2, 700], lens=[1, 1, 1, 1], decode=True, staged=True)
    attention_case(ops, bf, 8, 2, 128, starts=[8199, 19999, 2], lens=[1, 1, 1], decode=True, staged=True, window=5000)
    attention_case(ops, bf, 8, 2, 128, starts=[19999, 64], lens=[1, 1], decode=True, staged=True, pages_per_block=40, waves=8, spike=True)
    attention_case(ops, bf, 4, 1, 64, starts=[11999, 0], lens=[1, 1], decode=True, spike=True)
    attention_case(ops, bf, 6, 2, 80, starts=[9000], lens=[1], decode=True, window=4097)
    attention_case(ops, bf, 8, 2, 128, starts=[8000, 0], lens=[200, 70], spike=True)
    attention_case(ops, bf, 8, 2, 128, starts=[0, 0], lens=[3200, 33], spike=True)  # a long prompt whole: a hundred query blocks
    attention_case(ops, bf, 4, 4, 32, starts=[5000], lens=[100], window=3000)
    attention_case(ops, f32, 4, 2, 16, starts=[9000, 5], lens=[3, 2], spike=True)
    attention_case(ops, f32, 4, 2, 16, starts=[9000], lens=[1], decode=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_score_terms(ops, dtype):
    """Further terms of the scores (fms/modules/positions.py:9-36, the reference's adjusted_mask; :78-105: a bias of
    -|key position - query position| * scale[head]): a slope per head times the distance, and a soft cap.  Against
    softmax(cap * tanh(q.k * scale / cap) - slope * distance) written out; the special cases: slope 0 and a cap far
    above the scores is plain attention, a steep slope leaves every query its own value."""
    torch.manual_seed(9)
    H, K, D = 6, 2, 16
    starts, lens = [0, 130, 5], [70, 2, 1]
    totals = [s + n for s, n in zip(starts, lens)]
    table, n_pages = make_pages(totals, K, D, dtype, seed=4)
    ks = [torch.randn(n, K, D).to(dtype).float() for n in totals]
    vs = [torch.randn(n, K, D).to(dtype).float() for n in totals]
    qs = [2 * torch.randn(n, H, D).to(dtype).float() for n in lens]
    kc, vc = fill_cache(table, ks, vs, n_pages, dtype)
    q_flat = torch.cat([q.reshape(q.shape[0], H * D) for q in qs]).to(dtype)
    positions = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)]).int()
    seq = torch.cat([torch.full((n,), b) for b, n in enumerate(lens)]).int()
    sc = 1 / math.sqrt(D)

    def run(slopes, cap):
        sl = dev(torch.tensor(slopes, dtype=torch.float32)) if slopes is not None else None
        return ops.attention(dev(q_flat), dev(positions), dev(seq), dev(table), dev(kc), dev(vc), H, K, D, sc, 0,
                             score_slopes=sl, soft_cap=cap, force_generic=True).cpu().float()

    def want(slopes, cap):
        outs = []
        for q, k, v, s in zip(qs, ks, vs, starts):
            n = q.shape[0]
            pos = torch.arange(s, s + n)[:, None]
            key = torch.arange(k.shape[0])[None, :]
            o = torch.zeros(n, H, D)
            for h in range(H):
                kh = h // (H // K)
                scores = (q[:, h].double() @ k[:, kh].double().t()) * sc
                if cap:
                    scores = cap * torch.tanh(scores / cap)
                if slopes is not None:
                    scores = scores - slopes[h] * (pos - key).abs()
                probs = torch.softmax(scores.masked_fill(key > pos, float("-inf")), dim=-1)
                o[:, h] = (probs @ v[:, kh].double()).float()
            outs.append(o.reshape(n, H * D))
        return torch.cat(outs)

    tolerance = dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    slopes = [2.0 ** -(i + 1) for i in range(H)]
    plain = run(None, 0.0)
    torch.testing.assert_close(plain, want(None, 0.0), **tolerance)
    for sl, cap in ((slopes, 0.0), (None, 1.5), (slopes, 1.5)):
        got = run(sl, cap)
        torch.testing.assert_close(got, want(sl, cap), **tolerance)
        assert float((got - plain).abs().max()) > 0.05  # the term did something
    torch.testing.assert_close(run([0.0] * H, 1e4), plain, **tolerance)
    own = torch.cat([v[s : s + n].repeat_interleave(H // K, dim=1).reshape(n, H * D) for v, s, n in zip(vs, starts, lens)])
    torch.testing.assert_close(run([200.0] * H, 0.0), own, **tolerance)
    with pytest.raises(ValueError):
        run(slopes[:-1], 0.0)


def test_attention_generic_bf16_agrees(ops):
    attention_case(ops, torch.bfloat16, 4, 2, 16, starts=[0, 10], lens=[70, 3], force_generic=True)


# --------------------------------------------------------------------------
@pytest.mark.parametrize("M,N,K", [(1, 40, 24), (5, 100, 176), (64, 64, 64), (130, 257, 96), (70, 4096, 40)])
def test_gemm_f32(ops, M, N, K):
    torch.manual_seed(6)
    x, w, b = torch.randn(M, K), torch.randn(N, K), torch.randn(N)
    out = ops.linear(dev(x), dev(w), dev(b)).cpu()
    torch.testing.assert_close(out, (x.double() @ w.double().t() + b.double()).float(), atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("M", [1, 3, 16, 17, 33, 48, 64, 65, 96, 100, 128, 129, 144, 160, 170, 192, 193, 300])
@pytest.mark.parametrize("N,K", [(40, 24), (100, 176), (257, 96), (384, 96), (4096 + 16, 512), (20000, 64)])
def test_gemm_bf16(ops, M, N, K):
    torch.manual_seed(7)
    x = torch.randn(M, K).to(torch.bfloat16)
    w = (torch.randn(N, K) * 0.1).to(torch.bfloat16)
    b = torch.randn(N).to(torch.bfloat16)
    want = x.double() @ w.double().t()
    for out_dtype in (torch.bfloat16, torch.float32):
        for allow_library in (True, False):
            out = ops.linear(dev(x), dev(w), None, out_dtype=out_dtype, allow_library=allow_library).cpu()
            assert out.dtype == out_dtype
            torch.testing.assert_close(out.double(), want, atol=3e-2 if out_dtype == torch.bfloat16 else 2e-3, rtol=1e-2)
    out = ops.linear(dev(x), dev(w), dev(b), out_dtype=torch.float32, allow_library=False).cpu()
    torch.testing.assert_close(out.double(), want + b.double(), atol=2e-3, rtol=1e-2)
    # a float32 bias with bfloat16 weights, and a float32 weight with bfloat16 activations
    out = ops.linear(dev(x), dev(w), dev(b.float()), out_dtype=torch.float32).cpu()
    torch.testing.assert_close(out.double(), want + b.double(), atol=2e-3, rtol=1e-2)
    out = ops.linear(dev(x), dev(w.float()), None).cpu()
    assert out.dtype == torch.bfloat16
    torch.testing.assert_close(out.double(), want, atol=3e-2, rtol=1e-2)


@pytest.mark.parametrize("M", [1, 5, 17, 64, 70, 200])
@pytest.mark.parametrize("N,K", [(37, 12), (100, 44), (60, 50), (301, 1000 + 4)])
def test_gemm_bf16_of_widths_that_are_no_multiple_of_8(ops, M, N, K):
    """Rows of such widths are not 16-byte aligned, which the MFMA kernels need: an element-wise kernel takes
    them, so that no width a configuration allows is refused.  Also a view whose row stride is odd."""
    torch.manual_seed(17)
    x = torch.randn(M, K).to(torch.bfloat16)
    w = (torch.randn(N, K) * 0.1).to(torch.bfloat16)
    b = torch.randn(N).to(torch.bfloat16)
    want = x.double() @ w.double().t()
    for out_dtype in (torch.bfloat16, torch.float32):
        out = ops.linear(dev(x), dev(w), None, out_dtype=out_dtype).cpu()
        assert out.dtype == out_dtype
        torch.testing.assert_close(out.double(), want, atol=3e-2 if out_dtype == torch.bfloat16 else 2e-3, rtol=1e-2)
    for bias in (b, b.float()):
        out = ops.linear(dev(x), dev(w), dev(bias), out_dtype=torch.float32).cpu()
        torch.testing.assert_close(out.double(), want + b.double(), atol=2e-3, rtol=1e-2)
    wide = dev(torch.randn(M, K + 3).to(torch.bfloat16))
    out = ops.linear(wide[:, :K], dev(w), None, out_dtype=torch.float32).cpu()
    torch.testing.assert_close(out.double(), wide[:, :K].cpu().double() @ w.double().t(), atol=2e-3, rtol=1e-2)
    if N % 2 == 0:
        out = ops.gated_linear(dev(x), dev(w), dev(b), "swish").cpu().float()
        gu = x.float() @ w.float().t() + b.float()
        want = P.silu(gu[:, : N // 2]) * gu[:, N // 2 :]
        torch.testing.assert_close(out, want, atol=4e-2, rtol=2e-2)


@pytest.mark.parametrize("M", [1, 8, 20, 40, 64, 100, 128, 130, 150, 177, 192, 200])
@pytest.mark.parametrize("hidden,K", [(44, 24), (77, 40), (176, 64), (1000, 96)])
def test_gated_linear(ops, M, hidden, K):
    torch.manual_seed(8)
    for dtype in (torch.bfloat16, torch.float32):
        x = torch.randn(M, K).to(dtype)
        w = (torch.randn(2 * hidden, K) * 0.2).to(dtype)
        b = torch.randn(2 * hidden).to(dtype)
        for bias in (None, b):
            out = ops.gated_linear(dev(x), dev(w), None if bias is None else dev(bias), "swish").cpu().float()
            gu = x.float() @ w.float().t() + (0 if bias is None else bias.float())
            want = P.silu(gu[:, :hidden]) * gu[:, hidden:]
            torch.testing.assert_close(out, want, **(dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=4e-2, rtol=2e-2)))


@pytest.mark.parametrize("M", [1, 7, 16, 17, 32, 33, 64, 90, 128, 140, 165, 192])
@pytest.mark.parametrize("N,K,eps", [(48, 24, 1e-5), (96, 176, 1e-6), (4096 + 40, 64, 1e-5), (100, 96, 1e-3), (6144, 32, 1e-5)])
def test_linear_into_stream_and_deferred_row_norm(ops, M, N, K, eps):
    """The last product of a branch adds to the float32 stream and leaves the next norm's input; the
    products that read it (plain, gated, qkv with rotation) finish the norm.  Against the plain formulas:
    stream' = stream + x W^T + b;  y = rms_norm(stream') V^T."""
    torch.manual_seed(12)
    x = torch.randn(M, K).to(torch.bfloat16)
    w = (torch.randn(N, K) * 0.2).to(torch.bfloat16)
    b = torch.randn(N).to(torch.bfloat16)
    resid = torch.randn(M, N) * 3
    resid[0] *= 40  # rows of very different size: a row scale applied to the wrong row shows
    for norm_w in (torch.randn(N).abs().to(torch.bfloat16), torch.randn(N).abs(), None):
        for bias in (None, b):
            stream = dev(resid.clone())
            scaled, row_norm = ops.linear_into_stream(dev(x), dev(w), None if bias is None else dev(bias), stream,
                                                      None if norm_w is None else dev(norm_w), eps)
            want_stream = resid.double() + x.double() @ w.double().t() + (0 if bias is None else bias.double())
            torch.testing.assert_close(stream.cpu().double(), want_stream, atol=2e-3, rtol=1e-4)
            got = stream.cpu()
            torch.testing.assert_close(row_norm.partials.cpu().sum(-1), got.pow(2).sum(-1), rtol=1e-5, atol=1e-5)
            nw = torch.ones(N) if norm_w is None else norm_w.float()
            torch.testing.assert_close(scaled.cpu().float(), (got * nw).to(torch.bfloat16).float(), atol=0, rtol=1e-2)
            if N % 8:
                continue
            # consumers: what they make of (scaled, row_norm) against the product of the normed stream
            normed = P.rms_norm(got, nw, eps)
            N2 = 80
            v = (torch.randn(N2, N) * 0.2).to(torch.bfloat16)
            vb = torch.randn(N2).to(torch.bfloat16)
            bound = dict(atol=0.02 * float((normed @ v.float().t()).abs().max()) + 1e-3, rtol=2e-2)
            out = ops.linear(scaled, dev(v), dev(vb), row_norm=row_norm).cpu().float()
            torch.testing.assert_close(out, normed @ v.float().t() + vb.float(), **bound)
            out = ops.linear(scaled, dev(v), None, out_dtype=torch.float32, row_norm=row_norm).cpu()
            torch.testing.assert_close(out, normed @ v.float().t(), **bound)
            out = ops.gated_linear(scaled, dev(v), dev(vb), "swish", row_norm=row_norm).cpu().float()
            gu = normed @ v.float().t() + vb.float()
            want = P.silu(gu[:, :N2 // 2]) * gu[:, N2 // 2:]  # a product of two rounded values: its own scale
            torch.testing.assert_close(out, want, atol=0.02 * float(want.abs().max()) + 1e-3, rtol=2e-2)
            # the chain: a second product into the stream that reads the first one's rows
            stream2 = dev(resid.clone())
            w2 = (torch.randn(N, N) * 0.1).to(torch.bfloat16)
            ops.linear_into_stream(scaled, dev(w2), None, stream2, None, eps, row_norm=row_norm)
            torch.testing.assert_close(stream2.cpu(), resid + normed @ w2.float().t(), **bound)


@pytest.mark.parametrize("E,F,H,K", [(5120, 13824, 40, 40), (8192, 28672, 64, 8), (2560, 10240, 32, 32)])
def test_decode_products_at_the_layer_sizes_of_other_variants(ops, E, F, H, K):
    """The four products of a layer as a decode step runs them, at the sizes of the 13B, 70B and granite 3B variants
    (the 8B and 7B sizes run through whole models in test_model_shapes_gpu.py): output projection into the stream,
    gate/up with the activation and the deferred norm, down projection into the stream, qkv with rotation and cache
    write and the deferred norm.  Row counts of the kernels for up to 16 rows, for 17 to 32, for 33 to 128 and for 129 to 192.
    References are float32 products of the same operands, on the GPU."""
    torch.manual_seed(31)
    D = E // H
    eps = 1e-5
    wo = (torch.randn(E, E, device="cuda") * 0.02).bfloat16()
    wgu = (torch.randn(2 * F, E, device="cuda") * 0.02).bfloat16()
    wd = (torch.randn(E, F, device="cuda") * 0.02).bfloat16()
    wqkv = (torch.randn((H + 2 * K) * D, E, device="cuda") * 0.02).bfloat16()
    nw = (1 + 0.1 * torch.randn(E, device="cuda")).bfloat16()
    cos, sin = ops.rope_table(dev(P.rope_frequencies(D, 10000.0)), 512)
    for M in (8, 24, 80, 150):
        attn = torch.randn(M, E, device="cuda").bfloat16()
        resid = torch.randn(M, E, device="cuda") * 2
        resid[0] *= 20
        stream = resid.clone()
        # output projection: stream += attn Wo^T, scaled = stream * norm weight, partial sums of squares
        scaled, row_norm = ops.linear_into_stream(attn, wo, None, stream, nw, eps)
        want_stream = resid + attn.float() @ wo.float().t()
        torch.testing.assert_close(stream, want_stream, atol=2e-3, rtol=1e-4)
        normed = want_stream * torch.rsqrt(want_stream.pow(2).mean(-1, keepdim=True) + eps) * nw.float()
        # gate/up with the deferred norm
        hidden = ops.gated_linear(scaled, wgu, None, "swish", row_norm=row_norm)
        gu = normed @ wgu.float().t()
        want_hidden = P.silu(gu[:, :F]) * gu[:, F:]
        torch.testing.assert_close(hidden.float(), want_hidden, atol=0.02 * float(want_hidden.abs().max()) + 1e-3, rtol=2e-2)
        # down projection into the stream
        stream2 = want_stream.clone()
        ops.linear_into_stream(hidden, wd, None, stream2, nw, eps)
        torch.testing.assert_close(stream2, want_stream + hidden.float() @ wd.float().t(), atol=3e-3, rtol=1e-4)
        # qkv with rotation and cache write, against the product followed by the separate rotation kernel
        positions = torch.randint(0, 300, (M,)).int()
        seq = torch.arange(M).int()
        table, n_pages = make_pages([320] * M, K, D, torch.bfloat16, seed=4)
        res = []
        for fused in (True, False):
            kc = torch.zeros(n_pages, K, PAGE, D, dtype=torch.bfloat16, device="cuda")
            vc = torch.zeros(n_pages, K, D, PAGE, dtype=torch.bfloat16, device="cuda")
            args = (dev(positions), dev(seq), dev(table), cos, sin, D, kc, vc, H, K, D)
            if fused:
                qkv = ops.qkv_rope_write(scaled, wqkv, None, *args, row_norm=row_norm)
            else:
                qkv = (normed @ wqkv.float().t()).bfloat16()
                ops.rope_kv_write(qkv, *args)
            res.append((qkv[:, : H * D].float(), kc.float(), vc.float()))
        step = 2.0 ** -7 * max(float(res[1][0].abs().max()), float(res[1][1].abs().max()))  # see test_qkv_rope_write
        for a, b in zip(res[0], res[1]):
            assert float(b.abs().max()) > 0
            torch.testing.assert_close(a, b, atol=step, rtol=2e-2)


def test_qkv_rope_write_takes_a_deferred_row_norm(ops):
    torch.manual_seed(13)
    M, H, K, D, E, eps = 5, 4, 2, 32, 96, 1e-5
    N = (H + 2 * K) * D
    resid = torch.randn(M, E) * 2
    resid[3] *= 30
    nw = torch.randn(E).abs().to(torch.bfloat16)
    x0 = torch.zeros(M, 8).to(torch.bfloat16)
    stream = dev(resid.clone())
    scaled, row_norm = ops.linear_into_stream(dev(x0), dev(torch.zeros(E, 8).to(torch.bfloat16)), None, stream, dev(nw), eps)
    normed = ops.add_norm(dev(resid.clone()), None, dev(nw), None, eps, torch.bfloat16)
    w = (torch.randn(N, E) * 0.2).to(torch.bfloat16)
    positions = torch.randint(0, 200, (M,)).int()
    seq = torch.arange(M).int()
    table, n_pages = make_pages([256] * M, K, D, torch.bfloat16, seed=3)
    cos, sin = ops.rope_table(dev(P.rope_frequencies(D, 10000.0)), 256)
    res = []
    for x, rn in ((normed, None), (scaled, row_norm)):
        kc = torch.zeros(n_pages, K, PAGE, D, dtype=torch.bfloat16, device="cuda")
        vc = torch.zeros(n_pages, K, D, PAGE, dtype=torch.bfloat16, device="cuda")
        qkv = ops.qkv_rope_write(x, dev(w), None, dev(positions), dev(seq), dev(table), cos, sin, D, kc, vc, H, K, D, row_norm=rn)
        res.append((qkv[:, : H * D].cpu().float(), kc.cpu().float(), vc.cpu().float()))
    for a, b in zip(*res):
        assert a.abs().max() > 0
        torch.testing.assert_close(a, b, atol=0.02 * float(a.abs().max()), rtol=2e-2)


@pytest.mark.parametrize("vocab,width", [(128256, 4096), (32000, 4096), (49152, 2560)])
def test_output_head_at_served_vocabularies(ops, vocab, width):
    """The last product of a step at the vocabularies and widths of the registered variants: float32 logits from
    bfloat16 rows, for the row counts of decode batches (the weight-streaming kernels, 1 to 192 rows, in blocks of
    thousands) and above (this package's MFMA kernel), against the float32 product of the same operands; and the
    token choice on those logits."""
    torch.manual_seed(21)
    w = (torch.randn(vocab, width, device="cuda") * 0.02).bfloat16()
    wf = w.float()
    for M in (1, 8, 17, 33, 64, 128, 130, 192, 200):
        x = torch.randn(M, width, device="cuda").bfloat16()
        got = ops.linear(x, w, None, out_dtype=torch.float32)
        want = x.float() @ wf.t()
        assert got.dtype == torch.float32 and tuple(got.shape) == (M, vocab)
        torch.testing.assert_close(got, want, atol=2e-3, rtol=2e-3)
        assert ops.sample(got, False).tolist() == got.argmax(-1).tolist()
    del wf


# --------------------------------------------------------------------------
def test_argmax(ops):
    torch.manual_seed(9)
    logits = torch.randn(6, 1000)
    logits[2, 17] = logits[2, 900] = 50.0  # equal maxima: the lowest index wins
    out = ops.sample(dev(logits), False).cpu()
    want = logits.argmax(-1)
    want[2] = 17
    assert out.tolist() == want.tolist()
    big = torch.randn(2, 128256)
    assert ops.sample(dev(big), False).cpu().tolist() == big.argmax(-1).tolist()


@pytest.mark.parametrize("vocab,top_k,temperature", [(50, 0, 1.0), (384, 10, 0.8), (5000, 3, 2.0), (128256, 50, 0.7), (300, 1000, 1.0),
                                                     (128256, 0, 0.8), (128256, 10, 1.0), (32000, 256, 1.3), (5000, 300, 1.0), (128256, 512, 1.0), (49152, 700, 0.9),
                                                     (1031, 1030, 0.9), (64, 5, 1.0), (65, 64, 1.0)])
def test_sampling(ops, vocab, top_k, temperature):
    torch.manual_seed(10)
    rows = 64
    logits = torch.randn(rows, vocab) * 3
    seeds = [1234 + 7 * r for r in range(rows)]
    counters = [r % 5 for r in range(rows)]
    rng = torch.tensor([[s, c] for s, c in zip(seeds, counters)], dtype=torch.int64)
    rng_dev = dev(rng)
    out = ops.sample(dev(logits), True, temperature, top_k, rng_dev).cpu().tolist()
    assert rng_dev.cpu()[:, 1].tolist() == [c + 1 for c in counters]
    for r in range(rows):
        p = P.sampling_distribution(logits[r], temperature, top_k).double()
        cdf = torch.cumsum(p, 0)
        u = P.draw_uniform(seeds[r], counters[r])  # the plain implementation's own statement of the generator
        tok = out[r]
        assert p[tok] > 0, "a token outside the kept set was drawn"
        lo = float(cdf[tok] - p[tok])
        hi = float(cdf[tok])
        assert lo - 1e-5 <= u <= hi + 1e-5, (r, tok, u, lo, hi)
    if top_k == 3:
        kept = [set(torch.topk(logits[r], 3).indices.tolist()) for r in range(rows)]
        assert all(out[r] in kept[r] for r in range(rows))


def test_sampling_ties_at_threshold_survive(ops):
    logits = torch.full((1, 100), -5.0)
    logits[0, [3, 50, 77]] = 2.0  # top_k=2 but three equal maxima: all three stay
    seen = set()
    for c in range(200):
        rng = dev(torch.tensor([[99, c]], dtype=torch.int64))
        seen.add(int(ops.sample(dev(logits), True, 1.0, 2, rng).cpu()[0]))
    assert seen == {3, 50, 77}


@pytest.mark.parametrize("vocab", [900, 6000])
def test_sampling_with_many_equal_values(ops, vocab):
    """top_k far below the number of equal maxima: every one of them stays, so the draw is uniform over them, in
    index order.  600 of them fit the kernel's short list of candidates (which it has to put in index order);
    4000 do not, and the threshold is found over the whole row."""
    logits = torch.full((1, vocab), 1.5)
    logits[0, ::3] = -4.0  # a third are low values, the others equal maxima
    kept = [i for i in range(vocab) if i % 3]
    for c in range(40):
        rng = dev(torch.tensor([[5, c]], dtype=torch.int64))
        tok = int(ops.sample(dev(logits), True, 0.5, 7, rng).cpu()[0])
        u = P.draw_uniform(5, c)
        assert tok % 3, "a low value was drawn"
        assert abs(kept.index(tok) - u * len(kept)) <= 1.5, (c, tok, u)


def test_sampling_finds_a_far_value(ops):
    """One value stands out at each of many places of a large row, the row's ends and the borders of the stretches
    that the kernel cuts it into among them: with top_k=1 it is drawn whatever the uniform number is."""
    vocab = 128256
    places = [0, 1, 63, 64, 8063, 8064, 8065, 16127, 64512, 120959, 120960, 128191, 128192, vocab - 2, vocab - 1]
    torch.manual_seed(12)
    logits = torch.randn(len(places), vocab)
    for r, at in enumerate(places):
        logits[r, at] = 9.0
    rng = dev(torch.tensor([[77, r] for r in range(len(places))], dtype=torch.int64))
    assert ops.sample(dev(logits), True, 0.9, 1, rng).cpu().tolist() == places
    # and without top_k, at a temperature that leaves the others no mass to speak of
    rng = dev(torch.tensor([[78, r] for r in range(len(places))], dtype=torch.int64))
    assert ops.sample(dev(logits * 20), True, 0.05, 0, rng).cpu().tolist() == places


def test_kernels_refuse_what_they_cannot_do(ops):
    from fms_amd.kernels import KernelError

    with pytest.raises((KernelError, ValueError)):  # a deferred row norm needs rows the MFMA kernels can load
        ops.linear(dev(torch.zeros(2, 12, dtype=torch.bfloat16)), dev(torch.zeros(8, 12, dtype=torch.bfloat16)),
                   row_norm=ops.RowNorm(dev(torch.zeros(2, 1)), 1e-5))
    with pytest.raises(RuntimeError):
        ops.embed(torch.zeros(2, dtype=torch.int32), torch.zeros(4, 4))  # CPU tensors: no CPU path
    with pytest.raises((KernelError, ValueError)):
        ops.sample(dev(torch.zeros(1, 8)), True, 0.0, 0, dev(torch.zeros(1, 2, dtype=torch.int64)))


def test_the_probes_measure_this_gpu(ops):
    """What the benchmark divides by: a kernel that only reads and one that only issues matrix instructions.  On an
    MI355X the first lies between a quarter of and the whole published 8 TB/s, the second between a fifth of and the
    whole published 2.5 PFLOP/s; a probe whose loop the compiler removed, or that counts its work wrongly, falls outside."""
    read, mfma = ops.measured_peaks(read_mib=256, repeats=3)
    assert 2.0e12 < read < 8.0e12, f"a pure read measured at {read / 1e12:.2f} TB/s"
    assert 0.5e15 < mfma < 2.5e15, f"matrix instructions measured at {mfma / 1e15:.2f} PFLOP/s"

