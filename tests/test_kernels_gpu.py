"""Each HIP kernel alone against a plain float reference, at sizes other than the tiny models'."""

import math

import numpy as np
import pytest
import torch

from tests.plain import llama_plain as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 1e-5, torch.bfloat16: 1.6e-2}


def ops():
    from paged_llm_amd.csrc import ops as _ops
    return _ops


def rel_err(got, want):
    got, want = got.float().cpu(), want.float().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def rnd(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


# ----------------------------------------------------------------------------------- rows
@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_gather(dtype):
    table = rnd(301, 72, dtype=dtype).cuda()
    ids = torch.tensor([0, 300, 7, 7, 150], dtype=torch.int32).cuda()
    out = ops().embed_gather(ids, table)
    assert torch.equal(out.cpu(), table.cpu()[ids.cpu().long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [48, 200, 2048, 5000, 8200, 16384, 20001])
def test_rmsnorm(dtype, hidden):
    x = rnd(9, hidden, seed=1, dtype=dtype, scale=3.0)
    w = 1 + 0.3 * rnd(hidden, seed=2)
    eps = 1e-3
    out = ops().rmsnorm(x.cuda(), w.cuda(), eps)
    want = plain.rms_norm(x.float(), w, eps)
    assert rel_err(out, want) <= TOL[dtype]
    # the library routine the formula reduces to
    lib = torch.nn.functional.rms_norm(x.float(), (hidden,), w, eps)
    assert rel_err(want, lib) <= 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_with_residual_sum_and_row_choice(dtype):
    hidden = 136
    x = rnd(12, hidden, seed=3, dtype=dtype)
    d = rnd(12, hidden, seed=4, dtype=dtype)
    w = 1 + 0.3 * rnd(hidden, seed=5)
    xg = x.cuda().clone()
    out = ops().rmsnorm(xg, w.cuda(), 1e-5, delta=d.cuda())
    summed = (x.float() + d.float()).to(dtype)                 # the residual is rounded once
    assert torch.equal(xg.cpu(), summed)
    assert rel_err(out, plain.rms_norm(summed.float(), w, 1e-5)) <= TOL[dtype]
    # chosen rows, residual left alone
    idx = torch.tensor([11, 0, 5], dtype=torch.int32)
    xg = x.cuda().clone()
    out = ops().rmsnorm(xg, w.cuda(), 1e-5, delta=d.cuda(), row_index=idx.cuda(), write_residual=False)
    assert torch.equal(xg.cpu(), x)
    assert rel_err(out, plain.rms_norm(summed.float()[idx.long()], w, 1e-5)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [136, 2048, 8200, 99])
def test_rmsnorm_adds_partial_sums_in_order(dtype, hidden):
    """The residual's addend as float partial sums [ranges, rows, hidden] of a product cut along its inner dimension:
    added in order in float, then with x, rounded once (every kernel form: rows in registers, a row per workgroup, and
    widths that are no multiple of a 16-byte piece)."""
    x = rnd(21, hidden, seed=7, dtype=dtype)
    parts = rnd(3 * 21, hidden, seed=8).view(3, 21, hidden).contiguous()
    w = 1 + 0.3 * rnd(hidden, seed=9)
    summed = (x.float() + ((parts[0] + parts[1]) + parts[2])).to(dtype)
    xg = x.cuda().clone()
    out = ops().rmsnorm(xg, w.cuda(), 1e-5, delta=parts.cuda())
    assert torch.equal(xg.cpu(), summed)
    assert rel_err(out, plain.rms_norm(summed.float(), w, 1e-5)) <= TOL[dtype]
    idx = torch.tensor([20, 0, 5, 5], dtype=torch.int32)
    xg = x.cuda().clone()
    out = ops().rmsnorm(xg, w.cuda(), 1e-5, delta=parts.cuda(), row_index=idx.cuda(), write_residual=False)
    assert torch.equal(xg.cpu(), x)
    assert rel_err(out, plain.rms_norm(summed.float()[idx.long()], w, 1e-5)) <= TOL[dtype]
    with pytest.raises(ops().KernelError):
        ops().rmsnorm(xg, w.cuda(), 1e-5, delta=parts[:, :20].contiguous().cuda())


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    inter = 150
    gu = rnd(7, 2 * inter, seed=6, dtype=dtype, scale=2.0)
    out = ops().silu_mul(gu.cuda())
    want = torch.nn.functional.silu(gu.float()[:, :inter]) * gu.float()[:, inter:]
    assert rel_err(out, want) <= TOL[dtype]
    out = ops().gate_mul(gu.cuda(), "gelu_tanh")
    want = torch.nn.functional.gelu(gu.float()[:, :inter], approximate="tanh") * gu.float()[:, inter:]
    assert rel_err(out, want) <= TOL[dtype]
    with pytest.raises(ops().KernelError):
        ops().gate_mul(gu.cuda(), "gelu")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("slots", ["shuffled", "runs"])
@pytest.mark.parametrize("heads,kv_heads,d,bs", [(4, 2, 16, 16), (3, 1, 48, 8), (8, 8, 128, 32)])
def test_rope_and_cache_write(dtype, heads, kv_heads, d, bs, slots):
    """``runs``: the slots of prompt portions (consecutive positions): a portion from a page's start, one that
    starts 3 slots into a page, and between them a token that writes nothing.  Enough tokens for the form that
    writes the values of 16 tokens at a time: whole rows where their slots follow each other inside a page, single
    elements where they do not (shuffled slots, a portion that starts inside a page, the token without a slot)."""
    from paged_llm_amd.parts.registry import BuildEnv
    from paged_llm_amd.parts.rope import RotaryEncoding
    n1, n2 = 272, 270                                            # (the 16-at-a-time form is taken from 512 tokens on)
    second = (n1 + bs - 1) // bs                                 # the second portion's first page
    T, pages = (531, (531 + bs - 1) // bs + 2) if slots == "shuffled" else (n1 + 1 + n2, second + (3 + n2 + bs - 1) // bs + 1)
    rope = RotaryEncoding({"head_dim": d, "theta": 10000.0, "scaling": None}, BuildEnv(64, dtype, torch.device("cuda"), 512, {}))
    rope.prepare(512)
    width = (heads + 2 * kv_heads) * d
    qkv = rnd(T, width, seed=7, dtype=dtype)
    positions = torch.tensor([(5 * t + 3) % 500 for t in range(T)], dtype=torch.int32)
    perm = torch.randperm(pages * bs, generator=torch.Generator().manual_seed(8))[:T].to(torch.int32)
    if slots == "runs":
        order = torch.randperm(pages, generator=torch.Generator().manual_seed(8)).tolist()
        def portion(first_page, start, n):                       # n consecutive positions from `start` of a request
            table = order[first_page:]
            return [table[(start + i) // bs] * bs + (start + i) % bs for i in range(n)]
        perm = torch.tensor(portion(0, 0, n1) + [-1] + portion(second, 3, n2), dtype=torch.int32)
        assert perm.numel() == T
    k_pages = torch.zeros(pages, kv_heads, bs, d, dtype=dtype).cuda()
    v_pages = torch.zeros(pages, kv_heads, d, bs, dtype=dtype).cuda()
    g = qkv.cuda().clone()
    ops().rope_scatter(g, positions.cuda(), rope.cos, rope.sin, heads, kv_heads, d, perm.cuda(), k_pages, v_pages, bs)

    inv = plain.inverse_frequencies(d, 10000.0, None)
    ang = plain.rotary_angles(positions, inv)
    q = plain.apply_rotary(qkv.float()[:, :heads * d].view(T, heads, d), ang)
    k = plain.apply_rotary(qkv.float()[:, heads * d:(heads + kv_heads) * d].view(T, kv_heads, d), ang)
    v = qkv.float()[:, (heads + kv_heads) * d:].view(T, kv_heads, d)
    assert rel_err(g[:, :heads * d].view(T, heads, d), q) <= TOL[dtype]
    kp, vp = k_pages.float().cpu(), v_pages.float().cpu()
    for t in range(T):
        if int(perm[t]) < 0:
            continue
        page, off = int(perm[t]) // bs, int(perm[t]) % bs
        assert rel_err(kp[page, :, off, :], k[t]) <= TOL[dtype]
        assert torch.equal(vp[page, :, :, off], v[t].to(dtype).float()), f"token {t}"
    # untouched slots stay zero
    written = torch.zeros(pages * bs, dtype=torch.bool)
    written[perm[perm >= 0].long()] = True
    assert kp.permute(0, 2, 1, 3).reshape(pages * bs, -1)[~written].abs().max() == 0
    assert vp.permute(0, 3, 1, 2).reshape(pages * bs, -1)[~written].abs().max() == 0


def test_copy_pages():
    pages = rnd(6, 2, 8, 16, seed=9).cuda()
    before = pages.cpu().clone()
    ops().copy_pages(pages, torch.tensor([0, 3], dtype=torch.int32).cuda(), torch.tensor([5, 1], dtype=torch.int32).cuda())
    after = pages.cpu()
    assert torch.equal(after[5], before[0]) and torch.equal(after[1], before[3])
    assert torch.equal(after[[0, 2, 3, 4]], before[[0, 2, 3, 4]])


# ----------------------------------------------------------------------------------- products
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 7, 5), (3, 130, 64), (65, 64, 33), (200, 96, 176), (17, 517, 96)])
def test_gemm_generic(dtype, m, n, k):
    a, w = rnd(m, k, seed=10, dtype=dtype), rnd(n, k, seed=11, dtype=dtype)
    want = a.double() @ w.double().T
    out = ops().gemm_generic(a.cuda(), w.cuda())
    assert rel_err(out, want) <= TOL[dtype]
    out32 = ops().gemm_generic(a.cuda(), w.cuda(), out_dtype=torch.float32)
    assert out32.dtype == torch.float32 and rel_err(out32, want) <= 1e-5


def test_gemm_generic_rows_do_not_depend_on_the_batch():
    a, w = rnd(70, 200, seed=12), rnd(90, 200, seed=13)
    whole = ops().gemm_generic(a.cuda(), w.cuda()).cpu()
    for lo, hi in [(0, 1), (5, 7), (63, 70)]:
        part = ops().gemm_generic(a[lo:hi].cuda(), w.cuda()).cpu()
        assert torch.equal(part, whole[lo:hi])


# ----------------------------------------------------------------------------------- attention
def paged_case(seq_lens_k, num_q, heads, kv_heads, d, bs, dtype, seed=0, spare=3):
    """Keys and values in shuffled pages (test vectors of the reference's
    tests/test_attention_reference.py:10-28, in this engine's page layout)."""
    g = torch.Generator().manual_seed(seed)
    nblocks = [(L + bs - 1) // bs for L in seq_lens_k]
    total = sum(nblocks) + spare
    perm = torch.randperm(total, generator=g)
    tables = torch.zeros(len(seq_lens_k), max(nblocks), dtype=torch.int32)
    p = 0
    for s, nb in enumerate(nblocks):
        tables[s, :nb] = perm[p:p + nb]
        p += nb
    k_pages = torch.randn(total, kv_heads, bs, d, generator=g).to(dtype)
    v_pages = torch.randn(total, kv_heads, d, bs, generator=g).to(dtype)
    q = torch.randn(sum(num_q), heads * d, generator=g).to(dtype)
    cu = torch.tensor([0] + list(np.cumsum(num_q)), dtype=torch.int32)
    return q, k_pages, v_pages, tables, cu, torch.tensor(seq_lens_k, dtype=torch.int32)


def dense_attention(q, k_pages, v_pages, tables, cu, lens, heads, kv_heads, d, scale, window=None, **score_terms):
    bs = k_pages.shape[2]
    out = torch.empty(q.shape[0], heads * d)
    for s in range(len(lens)):
        L, lo, hi = int(lens[s]), int(cu[s]), int(cu[s + 1])
        idx = torch.arange(L)
        page, off = tables[s][idx // bs].long(), idx % bs
        k = k_pages.float()[page, :, off, :]                       # [L, kv, d]
        v = v_pages.float()[page, :, :, off]                       # [L, kv, d]
        q_full = torch.zeros(L, heads, d)
        q_full[L - (hi - lo):] = q[lo:hi].float().view(-1, heads, d)
        if score_terms:
            from tests.toy_plain import attention_with_score_terms
            o = attention_with_score_terms(q_full, k, v, scale, window, **score_terms)
        else:
            o = plain.causal_attention(q_full, k, v, scale, window)
        out[lo:hi] = o[L - (hi - lo):].reshape(hi - lo, heads * d)
    return out


CASES = [([5], [5]), ([33, 8, 17], [33, 8, 17]), ([40, 9, 64], [1, 1, 1]), ([40, 9, 64], [8, 1, 3]),
         ([7], [7]), ([129, 300, 17], [129, 300, 17]), ([1000, 33, 2048, 5], [1, 1, 1, 1]), ([500, 64, 77], [37, 1, 12]),
         ([1], [1])]
SHAPES = [(4, 2, 32, 8), (8, 8, 64, 16), (32, 4, 64, 16), (3, 1, 48, 32), (5, 5, 16, 4), (6, 2, 128, 16), (2, 1, 256, 16)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,d,bs", SHAPES)
@pytest.mark.parametrize("lens,num_q", CASES)
def test_paged_attention_generic(dtype, heads, kv_heads, d, bs, lens, num_q):
    if sum(lens) * heads * d > 3_000_000 and (heads, d) not in ((32, 64),):
        pytest.skip("long case kept for one shape")
    q, kp, vp, tables, cu, sl = paged_case(lens, num_q, heads, kv_heads, d, bs, dtype, seed=1)
    scale = 1 / math.sqrt(d)
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, scale)
    got = ops().paged_attention_generic(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads,
                                        d, scale)
    assert rel_err(got, want) <= (2e-5 if dtype == torch.float32 else 1.6e-2)


@pytest.mark.parametrize("window", [1, 5, 64, 100])
def test_paged_attention_generic_window(window):
    heads, kv_heads, d, bs = 4, 2, 32, 16
    q, kp, vp, tables, cu, sl = paged_case([150, 70, 9], [30, 1, 9], heads, kv_heads, d, bs, torch.float32, seed=2)
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, 0.2, window)
    got = ops().paged_attention_generic(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads,
                                        d, 0.2, window)
    assert rel_err(got, want) <= 2e-5


def test_attention_ignores_table_padding_and_stale_slots():
    """Garbage in table entries past the context and in slots past it must not change anything
    (tests/test_triton_kernel.py:37-44 of the reference)."""
    heads, kv_heads, d, bs = 4, 2, 32, 16
    q, kp, vp, tables, cu, sl = paged_case([20, 5], [1, 1], heads, kv_heads, d, bs, torch.float32, seed=3)
    args = (heads, kv_heads, d, 0.3)
    a = ops().paged_attention_generic(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), *args)
    t2 = tables.clone()
    t2[1, 1:] = 999_999
    kp2, vp2 = kp.clone(), vp.clone()
    kp2[tables[1, 0], :, 5:, :] = float("nan")            # slots behind the 5 tokens of request 1
    vp2[tables[1, 0], :, :, 5:] = float("nan")
    b = ops().paged_attention_generic(q.cuda(), kp2.cuda(), vp2.cuda(), t2.cuda(), cu.cuda(), sl.cuda(), *args)
    assert torch.equal(a.cpu(), b.cpu())


def test_attention_one_far_key_stands_out():
    """One key among 700 is made to dominate: the output must be that key's value row."""
    heads, kv_heads, d, bs = 2, 1, 32, 16
    q, kp, vp, tables, cu, sl = paged_case([700], [1], heads, kv_heads, d, bs, torch.float32, seed=4)
    far = 3
    page, off = int(tables[0, far // bs]), far % bs
    kp[page, 0, off, :] = q[0, :d] * 50
    got = ops().paged_attention_generic(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads,
                                        d, 1.0).cpu()
    assert torch.allclose(got[0, :d], vp[page, 0, :, off], atol=1e-5)


def score_terms_case(which, heads, seed=0):
    """(keyword arguments of the plain attention, the kernels' ScoreTerms) for one of "cap", "slopes", "sinks", "all"."""
    g = torch.Generator().manual_seed(seed)
    cap = 0.8 if which in ("cap", "all") else 0.0
    slopes = (0.002 * 4.0 ** torch.linspace(0, 2, heads)) if which in ("slopes", "all") else None      # 0.002 .. 0.032 a position
    # (sinks as heavy as a few hundred keys together: leaving one out shows at long contexts too)
    sinks = 7.0 + 1.5 * torch.randn(heads, generator=g) if which in ("sinks", "all") else None
    on_gpu = lambda t: None if t is None else t.float().cuda().contiguous()
    return dict(cap=cap, slopes=slopes, sinks=sinks), ops().ScoreTerms(cap, on_gpu(slopes), on_gpu(sinks))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["cap", "slopes", "sinks", "all"])
@pytest.mark.parametrize("window", [0, 40])
def test_paged_attention_generic_with_score_terms(dtype, which, window):
    """Further terms of the scores (a cap, a slope times the distance, a sink per head), each alone and together, with
    and without a window, against the plain attention with the same terms; each term must matter."""
    heads, kv_heads, d, bs = 6, 2, 24, 8
    lens, num_q = [150, 70, 9, 33], [30, 1, 9, 33]
    q, kp, vp, tables, cu, sl = paged_case(lens, num_q, heads, kv_heads, d, bs, dtype, seed=21)
    q = q * 2                                                   # scores of a few units: the cap has something to hold
    scale = 1 / math.sqrt(d)
    plain_terms, terms = score_terms_case(which, heads, seed=22)
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, scale, window or None, **plain_terms)
    without = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, scale, window or None)
    tol = 2e-5 if dtype == torch.float32 else 1.6e-2
    assert rel_err(without, want) > 5 * tol
    got = ops().paged_attention_generic(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, scale,
                                        window, terms=terms)
    assert rel_err(got, want) <= tol


def test_score_terms_are_checked():
    heads, kv_heads, d, bs = 4, 2, 32, 16
    q, kp, vp, tables, cu, sl = paged_case([20], [1], heads, kv_heads, d, bs, torch.bfloat16, seed=23)
    args = (q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, 1.0, 0)
    o = ops()
    for bad in (o.ScoreTerms(-1.0), o.ScoreTerms(float("nan")), o.ScoreTerms(0.0, torch.zeros(heads + 1, device="cuda")),
                o.ScoreTerms(0.0, None, torch.zeros(heads, device="cuda", dtype=torch.bfloat16)),
                o.ScoreTerms(0.0, torch.zeros(heads))):
        with pytest.raises(o.KernelError):
            o.paged_attention_generic(*args, terms=bad)
        with pytest.raises(o.KernelError):
            o.paged_attention_mfma(*args, 1, terms=bad)
    assert not o.ScoreTerms().any() and o.ScoreTerms(0.5).any()


# ----------------------------------------------------------------------------------- sampling
@pytest.mark.parametrize("vocab", [1000, 1001, 32000, 128256, 5003])
def test_argmax_takes_the_first_maximum(vocab):
    z = rnd(5, vocab, seed=14)
    z[1, 17] = z[1, 900] = 50.0
    z[2, :] = 0.0
    z[3, vocab - 1] = 60.0                                             # the last element of a row
    z[4, vocab - 2] = z[4, vocab - 1] = 70.0
    got = ops().argmax(z.cuda()).cpu()
    assert got.tolist() == [int(z[0].argmax()), 17, 0, vocab - 1, vocab - 2]
    # rows of a larger matrix: a row stride that leaves rows unaligned when the vocabulary is odd
    wide = torch.zeros(5, vocab + 3)
    wide[:, 1:vocab + 1] = z
    assert ops().argmax(wide.cuda()[:, 1:vocab + 1].contiguous()).cpu().tolist() == got.tolist()


def sample_rows(z, temperature, top_k, top_p, draws, seed=0):
    n = z.shape[0]
    out = []
    zg = z.cuda()
    t = torch.full((n,), temperature, dtype=torch.float32).cuda()
    k = torch.full((n,), top_k, dtype=torch.int32).cuda()
    p = torch.full((n,), top_p, dtype=torch.float32).cuda()
    keys = torch.arange(n, dtype=torch.int64).cuda()
    for step in range(draws):
        s = torch.full((n,), step, dtype=torch.int32).cuda()
        out.append(ops().sample(zg, t, k, p, keys, s, seed).cpu())
    return torch.stack(out)            # [draws, n]


def test_sampling_reduces_to_argmax():
    z = rnd(4, 333, seed=15)
    assert sample_rows(z, 0.0, -1, 1.0, 1)[0].tolist() == z.argmax(-1).tolist()
    assert sample_rows(z, 1.0, 1, 1.0, 3).tolist() == [z.argmax(-1).tolist()] * 3
    assert sample_rows(z, 1.0, -1, 1e-6, 3).tolist() == [z.argmax(-1).tolist()] * 3


def test_sampling_same_seed_same_tokens_other_seed_other_tokens():
    z = rnd(6, 97, seed=16)
    a, b, c = sample_rows(z, 1.0, -1, 1.0, 20, seed=1), sample_rows(z, 1.0, -1, 1.0, 20, seed=1), sample_rows(z, 1.0, -1, 1.0, 20, seed=2)
    assert torch.equal(a, b) and not torch.equal(a, c)


@pytest.mark.parametrize("vocab", [24, 40000, 33001])
@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, -1, 1.0), (0.7, -1, 1.0), (1.3, 5, 1.0), (1.0, -1, 0.6), (0.9, 8, 0.8)])
def test_sampling_frequencies_follow_the_filtered_distribution(temperature, top_k, top_p, vocab):
    """24 tokens that matter.  In the long rows (which the kernel reads again in every pass instead of holding them in
    registers: one a multiple of four, read in pieces of 16 bytes, one not) they are spread over the row among tokens
    whose logits lie 40 to 50 below and share a few values, so that the search for the threshold starts far away."""
    draws = 4000
    few = rnd(1, 24, seed=17, scale=1.5)
    if vocab == 24:
        z = few
    else:
        z = -45.0 + 5.0 * torch.round(rnd(1, vocab, seed=18) * 2).clamp(-2, 2) / 2
        z[0, (torch.arange(24) * 1663 + 11) % vocab] = few[0]
    probs = plain.filtered_probabilities(z[0], temperature, top_k, top_p).numpy()
    got = sample_rows(z, temperature, top_k, top_p, draws)[:, 0].numpy()
    counts = np.bincount(got, minlength=vocab)
    assert counts[probs == 0].sum() == 0, "a filtered token was drawn"
    keep = probs > 0
    chi2 = float(((counts[keep] - draws * probs[keep]) ** 2 / (draws * probs[keep])).sum())
    dof = int(keep.sum()) - 1
    assert chi2 < dof + 5 * math.sqrt(2 * max(dof, 1)) + 5, f"chi-square {chi2:.1f} for {dof} degrees of freedom"


@pytest.mark.parametrize("vocab", [1000, 32000, 50001, 128256])
@pytest.mark.parametrize("top_k,top_p", [(50, 1.0), (-1, 0.9), (40, 0.95), (-1, 0.999), (3, 0.2)])
def test_sampling_draws_only_and_all_of_the_kept_tokens(vocab, top_k, top_p):
    """Rows of real sizes: every drawn token belongs to the kept set of the plain implementation, and where that set is
    small all of it is drawn in the end."""
    z = rnd(3, vocab, seed=19, scale=3.0)
    z[1] = z[1] * 0.05                                                  # a flat row: the kept set of top-p is most of it
    z[2, ::7] = float("-inf")                                           # tokens that are ruled out beforehand
    draws = 300
    got = sample_rows(z, 0.8, top_k, top_p, draws)
    for row in range(3):
        probs = plain.filtered_probabilities(z[row], 0.8, top_k, top_p)
        assert bool((probs[got[:, row].long()] > 0).all()), f"row {row}: a filtered token was drawn"
        kept = int((probs > 0).sum())
        if kept <= 6:
            assert set(got[:, row].tolist()) == set(torch.nonzero(probs > 0).flatten().tolist()), f"row {row}"


@pytest.mark.parametrize("vocab", [97, 40000])
def test_sampling_keeps_or_drops_equal_logits_together(vocab):
    """A token stays if fewer than top_k tokens have a larger logit: with the second and third largest equal and
    top_k = 2 both stay (one token is larger than each), and the fourth goes."""
    z = torch.full((1, vocab), -20.0)
    z[0, 5], z[0, vocab // 2], z[0, vocab - 3], z[0, 70] = 3.0, 2.5, 2.5, 2.0
    draws = 4000
    got = sample_rows(z, 1.0, 2, 1.0, draws)[:, 0]
    assert set(got.tolist()) == {5, vocab // 2, vocab - 3}
    # ... and the draw is renormalised over that larger set (the reference cuts by sorted rank, pagedllm/sampler.py:25-31,
    # keeps exactly top_k tokens and so one of the two equal ones, whichever its sort puts first)
    want = torch.softmax(torch.tensor([3.0, 2.5, 2.5]), 0).numpy() * draws
    counts = np.array([(got == i).sum().item() for i in (5, vocab // 2, vocab - 3)])
    assert float(((counts - want) ** 2 / want).sum()) < 2 + 5 * math.sqrt(4) + 5
    # the same for the mass filter: the two equal tokens pass or fail the cumulative mass together
    mass = torch.softmax(z[0].double(), 0)
    p_between = float(mass[5] + 0.5 * mass[vocab // 2])            # reached inside the tie group
    assert set(sample_rows(z, 1.0, -1, p_between, 300)[:, 0].tolist()) == {5, vocab // 2, vocab - 3}


def kept_by_the_stated_rule(z_row, temperature, top_k, top_p):
    """Probabilities under the rule the kernel states for itself: a token stays if fewer than top_k tokens have a larger
    logit and the tokens with a larger logit weigh at most top_p; equal logits stay or go together (where no tie lies at
    the cut this is the reference's distribution, pagedllm/sampler.py:21-35)."""
    zz = z_row.double() / max(temperature, 1e-5)
    n = zz.numel()
    sz, idx = zz.sort(descending=True)
    probs = torch.softmax(sz, 0)
    exclusive = probs.cumsum(0) - probs
    starts = torch.ones(n, dtype=torch.bool)
    starts[1:] = sz[1:] != sz[:-1]
    first = torch.cummax(torch.where(starts, torch.arange(n), torch.zeros(n, dtype=torch.long)), 0).values      # where each run of equal logits begins
    keep = (first < (top_k if top_k > 0 else n)) & (exclusive[first] <= top_p)
    out = torch.zeros(n, dtype=torch.double)
    out[idx[keep]] = torch.softmax(sz[keep], 0)
    return out


@pytest.mark.parametrize("vocab", [32000, 50001, 128256, 262144])
@pytest.mark.parametrize("top_k,top_p", [(50, 0.9), (64, 1.0), (1, 1.0), (20, 0.3)])
def test_sampling_by_candidates_keeps_what_the_whole_row_keeps(vocab, top_k, top_p):
    """Rows of a long vocabulary with a small top_k are cut into chunks that hand on their largest logits, and the search
    and the draw run over those.  Three kinds of row: noise, a row in which few tokens carry the mass, and a row with
    a group of equal logits across the cut at top_k (all of them stay).  Every drawn token belongs to the kept set, a
    small kept set is drawn in full with frequencies that follow its probabilities, and the rows did go by their
    candidates; a row of equal logits, whose chunks have too many candidates, goes the long way."""
    z = rnd(4, vocab, seed=41, scale=1.0)
    z[1] = z[1] * 0.1
    z[1, (torch.arange(12) * 2503 + 7) % vocab] += torch.linspace(9.0, 6.0, 12)
    tie = torch.topk(z[2], top_k + 3).indices[max(top_k - 2, 0):]        # ranks top_k - 1 .. top_k + 3 share one logit
    z[2, tie] = z[2, tie].max()
    z[3] = 1.5
    draws = 400
    got = sample_rows(z, 0.8, top_k, top_p, draws)
    by_candidates = ops().rows_sampled_by_candidates(4, vocab, "cuda:0")
    assert by_candidates == [True, True, True, False], by_candidates
    for row in range(4):
        probs = kept_by_the_stated_rule(z[row], 0.8, top_k, top_p)
        if row < 2:                                                   # (no equal logits at the cut: the reference's own support)
            assert torch.equal(probs > 0, plain.filtered_probabilities(z[row], 0.8, top_k, top_p) > 0)
        drawn = got[:, row].long()
        assert bool((probs[drawn] > 0).all()), f"row {row}: a filtered token was drawn"
        kept = torch.nonzero(probs > 0).flatten()
        if 0 < len(kept) <= 12:
            assert set(drawn.tolist()) == set(kept.tolist()), f"row {row}"
            counts = np.array([(drawn == i).sum().item() for i in kept])
            want = probs[kept].numpy() * draws
            chi2, dof = float(((counts - want) ** 2 / want).sum()), len(kept) - 1
            assert chi2 < dof + 5 * math.sqrt(2 * max(dof, 1)) + 5, f"row {row}: chi-square {chi2:.1f} for {dof} degrees of freedom"
    # the same rows walked whole: other draws (the tokens stand in another order), the same kept sets
    zg = z.cuda()
    t, k, p = torch.full((4,), 0.8).cuda(), torch.full((4,), top_k, dtype=torch.int32).cuda(), torch.full((4,), top_p).cuda()
    keys = torch.arange(4, dtype=torch.int64).cuda()
    kept_sets = [kept_by_the_stated_rule(z[row], 0.8, top_k, top_p) > 0 for row in range(4)]
    for step in range(40):
        whole = ops().sample(zg, t, k, p, keys, torch.full((4,), step, dtype=torch.int32).cuda(), 0, candidates=False).cpu()
        for row in range(4):
            assert bool(kept_sets[row][int(whole[row])]), (step, row)


@pytest.mark.parametrize("vocab", [70000, 128256])
@pytest.mark.parametrize("top_k,top_p", [(-1, 0.9), (200, 0.8), (-1, 0.999)])
def test_long_rows_cut_by_their_mass_try_the_candidates(vocab, top_k, top_p):
    """A long row under top_p alone (or with a top_k beyond the candidates' reach) goes by the candidates of its 64 largest
    logits when fewer than 64 tokens stay, and is walked whole when not; either way what is drawn is what the plain
    implementation keeps.  Rows: a dozen tokens carry the mass; noise (thousands stay); a row where exactly the 64
    largest carry it, equal among themselves (the candidates do not settle that one)."""
    z = rnd(3, vocab, seed=43, scale=1.0)
    z[0] = z[0] * 0.2
    z[0, (torch.arange(12) * 3001 + 5) % vocab] += torch.linspace(14.0, 9.0, 12)
    z[2] = z[2] * 0.01
    z[2, (torch.arange(64) * 997 + 3) % vocab] = 20.0
    draws = 300
    got = sample_rows(z, 0.8, top_k, top_p, draws)
    for row in range(3):
        probs = kept_by_the_stated_rule(z[row], 0.8, top_k, top_p)
        if row < 2:
            assert torch.equal(probs > 0, plain.filtered_probabilities(z[row], 0.8, top_k, top_p) > 0)
        drawn = got[:, row].long()
        assert bool((probs[drawn] > 0).all()), f"row {row}: a filtered token was drawn"
        kept = torch.nonzero(probs > 0).flatten()
        if row == 2:
            assert len(kept) == 64
        if 0 < len(kept) <= 12:
            counts = np.array([(drawn == i).sum().item() for i in kept])
            want = probs[kept].numpy() * draws
            likely = want >= 5                                      # (tokens that 300 draws can be expected to show)
            assert bool((counts[likely] > 0).all()), f"row {row}: a token that stays was never drawn"
            chi2, dof = float(((counts[likely] - want[likely]) ** 2 / want[likely]).sum()), int(likely.sum())
            assert chi2 < dof + 5 * math.sqrt(2 * max(dof, 1)) + 5, f"row {row}: chi-square {chi2:.1f} for {dof} degrees of freedom"
    assert len(set(got[:, 1].tolist())) > 100 and len(set(got[:, 2].tolist())) > 40      # (many of the tokens that stay were drawn)


def test_sampling_rows_do_not_depend_on_their_neighbours():
    z = rnd(5, 50001, seed=23, scale=2.0)
    alone = torch.stack([sample_rows(z[r:r + 1], 0.9, 30, 0.9, 4)[:, 0] for r in range(5)], dim=1)
    keys = torch.arange(5, dtype=torch.int64)
    # the same rows in one launch, in another order, with the same request keys
    order = [3, 0, 4, 1, 2]
    zg = z[order].cuda()
    t, k, pp = torch.full((5,), 0.9).cuda(), torch.full((5,), 30, dtype=torch.int32).cuda(), torch.full((5,), 0.9).cuda()
    for step in range(4):
        s_ = torch.full((5,), step, dtype=torch.int32).cuda()
        got = ops().sample(zg, t, k, pp, keys[order].cuda(), s_, 0).cpu()
        for j, r in enumerate(order):
            # alone, row r was drawn with request key 0: draw it again in the batch with key r and alone with key r
            one = ops().sample(z[r:r + 1].cuda(), t[:1], k[:1], pp[:1], keys[r:r + 1].cuda(), s_[:1], 0).cpu()
            assert int(got[j]) == int(one[0]), (step, r)
    assert alone.shape == (4, 5)


# ----------------------------------------------------------------------------------- bfloat16 products for many rows
@pytest.mark.parametrize("m", [17, 64, 200])
@pytest.mark.parametrize("n,k", [(100, 96), (517, 176), (2048, 5632), (96, 1000), (33, 37)])
def test_library_product_float_and_bfloat16_out(m, n, k):
    a, w = rnd(m, k, seed=20, dtype=torch.bfloat16), rnd(n, k, seed=21, dtype=torch.bfloat16)
    want = a.double() @ w.double().T
    assert rel_err(ops().gemm_bf16(a.cuda(), w.cuda(), torch.float32), want) <= 2e-5
    out16 = ops().gemm_bf16(a.cuda(), w.cuda())
    assert out16.dtype == torch.bfloat16 and rel_err(out16, want) <= 1e-2


def test_library_product_strided_rows():
    big = rnd(40, 300, seed=24, dtype=torch.bfloat16).cuda()
    a, w = big[:, 41:41 + 176], rnd(64, 176, seed=25, dtype=torch.bfloat16).cuda()          # row stride and offset of no special form
    assert rel_err(ops().gemm_bf16(a, w, torch.float32), a.double().cpu() @ w.double().cpu().T) <= 2e-5


def test_large_bf16_product_and_float_rows():
    a, w = rnd(200, 256, seed=28, dtype=torch.bfloat16), rnd(130, 256, seed=29, dtype=torch.bfloat16)
    want = a.double() @ w.double().T
    assert rel_err(ops().gemm_bf16(a.cuda(), w.cuda()), want) <= 1e-2
    out = ops().gemm_bf16(a.cuda(), w.cuda(), torch.float32)
    assert out.dtype == torch.float32 and rel_err(out, want) <= 2e-5


# ----------------------------------------------------------------------------------- attention on the matrix cores
MFMA_SHAPES = [(4, 2, 32, 16), (8, 8, 64, 16), (32, 4, 64, 16), (3, 1, 48, 32), (5, 5, 16, 16), (6, 2, 128, 64), (2, 1, 256, 16),
               (16, 1, 80, 16), (40, 1, 64, 16), (1, 1, 112, 16), (6, 2, 112, 16), (3, 3, 96, 16)]


@pytest.mark.parametrize("heads,kv_heads,d,bs", MFMA_SHAPES)
@pytest.mark.parametrize("lens,num_q", CASES)
def test_paged_attention_mfma(heads, kv_heads, d, bs, lens, num_q):
    if sum(lens) * heads * d > 3_000_000 and (heads, d) not in ((32, 64),):
        pytest.skip("long case kept for one shape")
    q, kp, vp, tables, cu, sl = paged_case(lens, num_q, heads, kv_heads, d, bs, torch.bfloat16, seed=1)
    scale = 1 / math.sqrt(d)
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, scale)
    args = (q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, scale, 0, max(num_q))
    assert rel_err(ops().paged_attention_mfma(*args), want) <= 1.6e-2
    for size in (64, 256):
        parts = (max(lens) + size - 1) // size
        assert rel_err(ops().paged_attention_mfma(*args, size, parts), want) <= 1.6e-2, f"partition {size}"
    if max(num_q) * (heads // kv_heads) <= 64:
        cols = max(num_q) * (heads // kv_heads)
        ncb = 1 if cols <= 16 else (2 if cols <= 32 else 4)
        for waves in (4, 8):
            if ops()._merge_lds_bytes(ncb, waves, d) <= 160 * 1024:
                assert rel_err(ops().paged_attention_mfma(*args, 0, 1, waves), want) <= 1.6e-2, f"{waves} wavefronts"
                parts = (max(lens) + 255) // 256
                assert rel_err(ops().paged_attention_mfma(*args, 256, parts, waves), want) <= 1.6e-2, f"{waves} wavefronts, partitions"


@pytest.mark.parametrize("window", [1, 5, 64, 100])
def test_paged_attention_mfma_window(window):
    heads, kv_heads, d, bs = 4, 2, 32, 16
    q, kp, vp, tables, cu, sl = paged_case([150, 70, 9, 300], [30, 1, 9, 1], heads, kv_heads, d, bs, torch.bfloat16, seed=2)
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, 0.2, window)
    args = (q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, 0.2, window, 30)
    assert rel_err(ops().paged_attention_mfma(*args), want) <= 1.6e-2
    assert rel_err(ops().paged_attention_mfma(*args, 64, 5), want) <= 1.6e-2
    args = args[:-1] + (2,)
    q2 = torch.cat([q[28:30], q[30:31], q[38:40], q[40:41]])          # at most two queries per sequence: 16 columns
    cu2 = torch.tensor([0, 2, 3, 5, 6], dtype=torch.int32)
    want2 = torch.cat([want[28:30], want[30:31], want[38:40], want[40:41]])
    got = ops().paged_attention_mfma(q2.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu2.cuda(), sl.cuda(), heads, kv_heads, d, 0.2,
                                     window, 2, 0, 1, 8)
    assert rel_err(got, want2) <= 1.6e-2


def test_mfma_attention_ignores_table_padding_and_stale_slots():
    heads, kv_heads, d, bs = 4, 2, 32, 16
    q, kp, vp, tables, cu, sl = paged_case([20, 5, 70], [1, 1, 3], heads, kv_heads, d, bs, torch.bfloat16, seed=3)
    def run(kp, vp, tables, *split):
        return ops().paged_attention_mfma(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads,
                                          d, 0.3, 0, 3, *split).cpu()
    t2 = tables.clone()
    t2[0, 2:] = 999_999
    t2[1, 1:] = 999_999
    kp2, vp2 = kp.clone(), vp.clone()
    kp2[tables[1, 0], :, 5:, :] = float("nan")
    vp2[tables[1, 0], :, :, 5:] = float("nan")
    kp2[tables[0, 1], :, 4:, :] = float("inf")
    vp2[tables[0, 1], :, :, 4:] = float("nan")
    for split in ((), (64, 2), (0, 1, 4), (64, 2, 4)):
        assert torch.equal(run(kp, vp, tables, *split), run(kp2, vp2, t2, *split))


@pytest.mark.parametrize("far", [3, 64, 200, 699])
def test_mfma_attention_one_far_key_stands_out(far):
    heads, kv_heads, d, bs = 8, 1, 64, 16
    q, kp, vp, tables, cu, sl = paged_case([700], [1], heads, kv_heads, d, bs, torch.bfloat16, seed=4)
    page, off = int(tables[0, far // bs]), far % bs
    kp[page, 0, off, :] = (q[0, 5 * d:6 * d].float() * 40).to(torch.bfloat16)       # head 5 looks at that key only
    for split in ((), (128, 6), (0, 1, 8), (256, 3, 4)):
        got = ops().paged_attention_mfma(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads,
                                         d, 1.0, 0, 1, *split).cpu().float()
        assert torch.allclose(got[0, 5 * d:6 * d], vp[page, 0, :, off].float(), atol=2e-2)


@pytest.mark.parametrize("heads,kv_heads,d", [(8, 2, 64), (6, 2, 128), (4, 4, 32)])
@pytest.mark.parametrize("which", ["cap", "slopes", "sinks", "all"])
@pytest.mark.parametrize("window", [0, 200])
def test_paged_attention_mfma_with_score_terms(heads, kv_heads, d, which, window):
    """The matrix-core kernels with further score terms (compiled into a library of their own), in every form a step
    may take: decoded tokens in one piece, in partitions (the sink then belongs to the partition that holds a query's
    first visible key: with a window not the first one), with several wavefronts; prompt portions as workgroups that
    share their keys, whole and in partitions."""
    bs = 16
    group = heads // kv_heads
    plain_terms, terms = score_terms_case(which, heads, seed=24)
    scale = 1 / math.sqrt(d)
    # decoding and small portions
    lens, num_q = [700, 33, 1030, 5, 64], [1, 1, 2, 1, 2]
    q, kp, vp, tables, cu, sl = paged_case(lens, num_q, heads, kv_heads, d, bs, torch.bfloat16, seed=25)
    q = q * 2
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, scale, window or None, **plain_terms)
    assert rel_err(dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, scale, window or None), want) > 8e-2
    args = (q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, scale, window, max(num_q))
    cols = max(num_q) * group
    ncb = 1 if cols <= 16 else (2 if cols <= 32 else 4)
    for split in ((), (64, 17), (256, 5), (0, 1, 4), (0, 1, 8), (256, 5, 4), (128, 9, 8)):
        if len(split) == 3 and ops()._merge_lds_bytes(ncb, split[2], d) > 160 * 1024:
            continue
        assert rel_err(ops().paged_attention_mfma(*args, *split, terms=terms), want) <= 1.6e-2, f"decode {split}"
    # prompt portions: whole prompts and portions behind a context
    lens, num_q = [300, 1100, 130], [300, 200, 64 // group + 3]
    q, kp, vp, tables, cu, sl = paged_case(lens, num_q, heads, kv_heads, d, bs, torch.bfloat16, seed=26)
    q = q * 2
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, scale, window or None, **plain_terms)
    args = (q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, scale, window, max(num_q))
    for split in ((0, 1, 1, 2), (128, 9, 1, 2), (512, 3, 1, 2), (0, 1, 1, 4)):
        assert rel_err(ops().paged_attention_mfma(*args, *split, terms=terms), want) <= 1.6e-2, f"prompt {split}"


def test_score_terms_through_the_planned_launch():
    """Decoded tokens at long contexts beside prompt portions, launched as the engine launches a step (two launches,
    partitions as planned), with all score terms at once."""
    import types
    heads, kv_heads, d, bs = 8, 2, 64, 16
    plain_terms, terms = score_terms_case("all", heads, seed=27)
    q_lens, k_lens = [1, 1, 2, 100, 300], [3000, 17, 4100, 2000, 300]
    q, kp, vp, tables, cu, sl = paged_case(k_lens, q_lens, heads, kv_heads, d, bs, torch.bfloat16, seed=28)
    q = q * 2
    ctx = types.SimpleNamespace(num_seqs=len(q_lens), max_q_len=max(q_lens), max_k_len=max(k_lens), q_lens=q_lens, k_lens=k_lens,
                                capturing=False, device=torch.device("cuda"))
    got = ops().paged_attention(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, 0.125, 0, ctx,
                                terms=terms)
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, 0.125, None, **plain_terms)
    assert rel_err(got, want) <= 1.6e-2


@pytest.mark.parametrize("heads,kv_heads,d", [(32, 4, 64), (8, 2, 128), (6, 1, 96)])
@pytest.mark.parametrize("batch", [1, 9])
def test_long_contexts_through_the_planned_launch(heads, kv_heads, d, batch):
    """Decoding at contexts of thousands of keys, launched as the engine launches it (partitions, wavefronts
    and merge as planned for the batch).  In every sequence one head looks at one key only, somewhere among
    the thousands (the first, both sides of a block and of a partition edge, the last): its output must be
    that key's value.  All heads of the first and the last sequence are compared with dense attention."""
    import types
    bs = 16
    lens = [6000 + 517 * i for i in range(batch)]
    q, kp, vp, tables, cu, sl = paged_case(lens, [1] * batch, heads, kv_heads, d, bs, torch.bfloat16, seed=9)
    far = [0, 63, 64, 255, 256, 4095, 4096, 5999, 2048][:batch]
    for s, n in enumerate(far):
        page, off = int(tables[s, n // bs]), n % bs
        head = s % heads
        kp[page, head // (heads // kv_heads), off, :] = (q[s, head * d:(head + 1) * d].float() * 40).to(torch.bfloat16)
    ctx = types.SimpleNamespace(num_seqs=batch, max_q_len=1, max_k_len=max(lens), q_lens=[1] * batch, k_lens=lens, capturing=False, device=torch.device("cuda"))
    got = ops().paged_attention(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d,
                                1.0, 0, ctx).cpu().float()
    for s, n in enumerate(far):
        page, off = int(tables[s, n // bs]), n % bs
        head = s % heads
        assert torch.allclose(got[s, head * d:(head + 1) * d], vp[page, head // (heads // kv_heads), :, off].float(), atol=2e-2), \
            f"sequence {s}: key {n} of {lens[s]}"
    pick = sorted({0, batch - 1})                              # dense attention of the first and the last sequence
    want = dense_attention(q[pick], kp, vp, tables[pick], torch.arange(len(pick) + 1, dtype=torch.int32), sl[pick], heads,
                           kv_heads, d, 1.0)
    assert rel_err(got[pick], want) <= 1.6e-2


def test_an_outgrown_partition_buffer_stays_allocated():
    """The buffer of the partitions' partial results grows with the batch; a captured graph still holds the
    address of the one it was captured with, so an outgrown buffer must not go back to the allocator."""
    o = ops()
    heads, kv_heads, d, bs = 4, 1, 16, 16
    def run(batch, parts):
        lens = [parts * 64] * batch
        q, kp, vp, tables, cu, sl = paged_case(lens, [1] * batch, heads, kv_heads, d, bs, torch.bfloat16, seed=3)
        got = o.paged_attention_mfma(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, 1.0, 0, 1,
                                     64, parts).cpu().float()
        pick = sorted({0, batch - 1})
        want = dense_attention(q[pick], kp, vp, tables[pick], torch.arange(len(pick) + 1, dtype=torch.int32), sl[pick], heads,
                               kv_heads, d, 1.0)
        assert rel_err(got[pick], want) <= 1.6e-2
    run(2, 2)
    first = o._attn_scratch["cuda:0"]
    need = first.numel() // (heads * (d + 2)) + 64            # rows x partitions that no longer fit
    run(need // 16 + 1, 16)
    assert o._attn_scratch["cuda:0"].numel() > first.numel()
    assert any(t is first for t in o._attn_scratch_retired)


@pytest.mark.parametrize("heads,kv_heads,d", [(32, 4, 64), (8, 2, 128), (6, 1, 96), (4, 4, 32)])
def test_decoded_tokens_beside_prompt_portions(heads, kv_heads, d):
    """A step with decoded tokens (long contexts, cut into partitions) and small portions beside prompt portions:
    launched in two parts, sequences with few queries first.  One decoded token looks at a single far key."""
    import types
    bs = 16
    group = heads // kv_heads
    few_q = [1, 1, 2, 1, 64 // group]                          # the last one fills the decode kernel's tile exactly
    few_k = [3000, 17, 700, 4096, 900]
    many_q = [64 // group + 1, 100, 300]
    many_k = [2000, 100, 1300]
    q_lens, k_lens = few_q + many_q, few_k + many_k
    q, kp, vp, tables, cu, sl = paged_case(k_lens, q_lens, heads, kv_heads, d, bs, torch.bfloat16, seed=12)
    n = 1234                                                   # sequence 0, head 1 sees key 1234 only
    page, off = int(tables[0, n // bs]), n % bs
    kp[page, 1 // group, off, :] = (q[0, d:2 * d].float() * 40).to(torch.bfloat16)
    ctx = types.SimpleNamespace(num_seqs=len(q_lens), max_q_len=max(q_lens), max_k_len=max(k_lens), q_lens=q_lens, k_lens=k_lens,
                                capturing=False, device=torch.device("cuda"))
    got = ops().paged_attention(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d,
                                1.0, 0, ctx).cpu().float()
    assert torch.allclose(got[0, d:2 * d], vp[page, 1 // group, :, off].float(), atol=2e-2)
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, 1.0)
    assert rel_err(got, want) <= 1.6e-2
    # the same batch in one launch (sequences not in that order): the same numbers up to rounding
    order = [5, 0, 6, 1, 2, 7, 3, 4]
    rows = [list(range(int(cu[s]), int(cu[s + 1]))) for s in order]
    q2 = q[[r for rs in rows for r in rs]]
    cu2 = torch.tensor([0] + list(np.cumsum([len(rs) for rs in rows])), dtype=torch.int32)
    ctx2 = types.SimpleNamespace(num_seqs=len(order), max_q_len=max(q_lens), max_k_len=max(k_lens), q_lens=[q_lens[s] for s in order],
                                 k_lens=[k_lens[s] for s in order], capturing=False, device=torch.device("cuda"))
    got2 = ops().paged_attention(q2.cuda(), kp.cuda(), vp.cuda(), tables[order].contiguous().cuda(), cu2.cuda(), sl[order].cuda(), heads,
                                 kv_heads, d, 1.0, 0, ctx2).cpu().float()
    back = torch.empty_like(got2)
    back[[r for rs in rows for r in rs]] = got2
    assert rel_err(back, want) <= 1.6e-2


@pytest.mark.parametrize("heads,kv_heads,d", [(32, 4, 64), (8, 2, 128), (6, 1, 96), (4, 4, 32)])
@pytest.mark.parametrize("window", [0, 700])
def test_prompt_portions_with_key_partitions(heads, kv_heads, d, window):
    """Prompt portions behind long contexts with their keys cut into partitions that the merge kernel joins: partitions
    that end inside, at and beyond a sequence's context, a sequence that starts at position 0, a window, one query
    that looks at a single far key, and stale slots full of NaN behind a context's end."""
    bs = 16
    group = heads // kv_heads
    q_lens, k_lens = [200, 64 // group + 3, 130], [2300, 1024, 130]
    q, kp, vp, tables, cu, sl = paged_case(k_lens, q_lens, heads, kv_heads, d, bs, torch.bfloat16, seed=13)
    n, row, head = 777 if window == 0 else 2100, 150, 1 % heads           # row 150 of sequence 0 (position 2250) sees key n only
    page, off = int(tables[0, n // bs]), n % bs
    kp[page, head // group, off, :] = (q[row, head * d:(head + 1) * d].float() * 40).to(torch.bfloat16)
    stale = int(tables[2, 130 // bs])                                   # the slots behind sequence 2's 130 keys
    kp[stale, :, 130 % bs:, :], vp[stale, :, :, 130 % bs:] = float("nan"), float("nan")
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, 1.0, window or None)
    for size in (128, 512, 640, 4096):
        parts = (max(k_lens) + size - 1) // size
        got = ops().paged_attention_mfma(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, 1.0,
                                         window, max(q_lens), size, parts, 1, 2).cpu().float()
        assert torch.allclose(got[row, head * d:(head + 1) * d], vp[page, head // group, :, off].float(), atol=2e-2), f"partition {size}"
        assert rel_err(got, want) <= 1.6e-2, f"partition {size}"


def test_prompt_portion_with_more_partitions_than_a_wavefront_has_lanes():
    """A portion behind 9,000 cached positions in 71 partitions of 128 keys: the merge walks them 64 at a time."""
    heads, kv_heads, d, bs = 4, 1, 32, 16
    q, kp, vp, tables, cu, sl = paged_case([9000], [80], heads, kv_heads, d, bs, torch.bfloat16, seed=14)
    n, row, head = 8321, 40, 2                                         # one query looks at a key in the 66th partition only
    page, off = int(tables[0, n // bs]), n % bs
    kp[page, 0, off, :] = (q[row, head * d:(head + 1) * d].float() * 40).to(torch.bfloat16)
    want = dense_attention(q, kp, vp, tables, cu, sl, heads, kv_heads, d, 1.0)
    got = ops().paged_attention_mfma(q.cuda(), kp.cuda(), vp.cuda(), tables.cuda(), cu.cuda(), sl.cuda(), heads, kv_heads, d, 1.0,
                                     0, 80, 128, 71, 1, 2).cpu().float()
    assert torch.allclose(got[row, head * d:(head + 1) * d], vp[page, 0, :, off].float(), atol=2e-2)
    assert rel_err(got, want) <= 1.6e-2


def test_prompt_partitions_are_chosen_to_fill_the_gpu():
    pp = ops().prompt_partitions
    assert pp(512, 4, 2048, 256) == (0, 1)                              # a whole prompt: tiles enough
    assert pp(16, 4, 2048, 256) == (512, 4)                             # 256 tokens behind 2048: 64 workgroups -> 256
    assert pp(16, 4, 600, 256) == (0, 1)                                # too short to cut
    size, parts = pp(2, 8, 100_000, 256)
    assert size % 128 == 0 and size >= 512 and (parts - 1) * size < 100_000 <= parts * size and parts <= 16


def test_decode_attention_kernel_leaves_room_for_two_workgroups():
    """At head size 64 the decode kernel keeps two blocks of keys and values in registers; two of its workgroups of
    four wavefronts share a compute unit only while it takes at most 256 registers per lane, vector and accumulation
    registers together (the plan for large batches counts on that: a version that took a few more was measured half
    as fast in the same launch)."""
    assert 0 < ops().attention_decode_registers(64, 4) <= 256


@pytest.mark.parametrize("head_dim", [64, 128])
def test_decode_attention_kernel_spills_no_registers(head_dim):
    """The forms that decoding uses (16 columns, four or eight wavefronts) must fit their registers: at head size 128
    the eight-wavefront form takes all 256, and a change that made it spill four of them cost 12 % of its speed
    at 64 sequences."""
    for waves in (4, 8):
        assert ops().attention_decode_spill_bytes(head_dim, waves) == 0, (head_dim, waves)


def test_attention_plan():
    plan = ops().attention_plan
    lds = 160 * 1024
    assert plan(8, 4, 1, 2048, 8, 64, lds) == (4, 256, 8)       # decoding: partitions for workgroups, blocks for wavefronts
    assert plan(64, 4, 1, 2048, 8, 64, lds) == (8, 0, 1)         # enough sequences: wavefronts only
    assert plan(64, 8, 1, 2048, 4, 64, lds) == (4, 0, 1)         # two work items per compute unit: smaller workgroups
    assert plan(64, 8, 1, 2048, 4, 128, lds) == (8, 0, 1)        # large heads keep eight (one block under way per wavefront)
    assert plan(1, 4, 1, 2048, 8, 64, lds) == (4, 256, 8)
    assert plan(8, 4, 1, 200, 8, 64, lds) == (4, 0, 1)
    assert plan(1, 4, 2048, 2048, 8, 64, lds) == (1, 0, 1)      # a long prompt portion: one wavefront per query tile
    assert plan(2, 4, 1, 50, 8, 64, lds) == (1, 0, 1)
    assert plan(8, 8, 1, 2048, 4, 128, lds) == (8, 512, 4)
    assert plan(1, 8, 1, 100000, 4, 128, lds) == (8, 4096, 25)
    assert plan(24, 4, 1, 2048, 8, 64, lds) == (8, 1024, 2)      # work items x partitions fill the compute units once, not twice
    assert plan(48, 4, 1, 2048, 8, 64, lds) == (8, 0, 1)
    assert plan(96, 4, 1, 2048, 8, 64, lds) == (4, 0, 1)         # more work items than compute units: two small workgroups each
    assert plan(40, 8, 1, 2048, 4, 128, lds) == (8, 0, 1)
    assert plan(48, 4, 1, 2048, 8, 64, lds, 304) == (8, 0, 1) and plan(24, 4, 1, 2048, 8, 64, lds, 64) == (4, 0, 1)


# ----------------------------------------------------------------------------------- fused decode products
@pytest.mark.parametrize("m", [1, 3, 8, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("n,k", [(16, 64), (100, 96), (517, 176), (2560, 2048), (2048, 5632), (96, 1000)])
def test_decode_linear_plain(m, n, k):
    o = ops()
    x, w = rnd(m, k, seed=30, dtype=torch.bfloat16), rnd(n, k, seed=31, dtype=torch.bfloat16)
    assert o.decode_linear_takes(m, k, x.cuda(), w.cuda(), staged=False)
    want = x.double() @ w.double().T
    assert rel_err(o.decode_linear(x.cuda(), w.cuda(), o.EPI_F32), want) <= 2e-5
    assert rel_err(o.decode_linear(x.cuda(), w.cuda(), o.EPI_BF16), want) <= 1e-2


@pytest.mark.parametrize("m", [1, 8, 13])
@pytest.mark.parametrize("k", [96, 2048])
def test_decode_linear_with_residual_sum_norm_and_row_choice(m, k):
    o = ops()
    x, d = rnd(m, k, seed=32, dtype=torch.bfloat16), rnd(m, k, seed=33, dtype=torch.bfloat16)
    nw, w = 1 + 0.3 * rnd(k, seed=34), rnd(130, k, seed=35, dtype=torch.bfloat16, scale=k ** -0.5)
    summed = (x.float() + d.float()).to(torch.bfloat16)
    h = plain.rms_norm(summed.float(), nw, 1e-4).to(torch.bfloat16)
    want = h.double() @ w.double().T
    x_out = torch.zeros(m, k, dtype=torch.bfloat16).cuda()
    got = o.decode_linear(x.cuda(), w.cuda(), o.EPI_F32, delta=d.cuda(), norm_weight=nw.cuda(), eps=1e-4, x_out=x_out)
    assert torch.equal(x_out.cpu(), summed)
    assert rel_err(got, want) <= 1e-2                      # h differs from the plain one by its bfloat16 rounding at most
    # no delta, chosen rows
    idx = torch.tensor(list(range(m - 1, -1, -2)), dtype=torch.int32)
    h2 = plain.rms_norm(x.float()[idx.long()], nw, 1e-4).to(torch.bfloat16)
    got = o.decode_linear(x.cuda(), w.cuda(), o.EPI_F32, norm_weight=nw.cuda(), eps=1e-4, row_index=idx.cuda())
    assert rel_err(got, h2.double() @ w.double().T) <= 1e-2
    # the fused norm against the norm kernel followed by the plain product: the same numbers up to where
    # the rounding to bfloat16 happens (the norm kernel rounds x * w / rms, the fused kernel rounds x * w and
    # scales the finished sums by 1 / rms), so each is held to the exact result
    sep = o.decode_linear(o.rmsnorm(x.cuda(), nw.cuda(), 1e-4), w.cuda(), o.EPI_F32)
    fused = o.decode_linear(x.cuda(), w.cuda(), o.EPI_F32, norm_weight=nw.cuda(), eps=1e-4)
    exact = plain.rms_norm(x.double(), nw.double(), 1e-4) @ w.double().T
    assert rel_err(fused, exact) <= 4e-3 and rel_err(sep, exact) <= 4e-3


@pytest.mark.parametrize("m", [1, 8, 16, 24, 41, 64])
@pytest.mark.parametrize("inter,k", [(176, 64), (250, 96), (5632, 2048)])
def test_decode_linear_gated(m, inter, k):
    o = ops()
    x = rnd(m, k, seed=36, dtype=torch.bfloat16)
    w = rnd(2 * inter, k, seed=37, dtype=torch.bfloat16, scale=k ** -0.5)
    want = torch.nn.functional.silu(x.double() @ w[:inter].double().T) * (x.double() @ w[inter:].double().T)
    assert rel_err(o.decode_linear(x.cuda(), w.cuda(), o.EPI_GATED), want) <= 1e-2


@pytest.mark.parametrize("heads,kv_heads,d,bs", [(4, 2, 32, 16), (32, 4, 64, 16), (3, 1, 96, 32), (8, 8, 128, 16), (5, 1, 48, 16), (2, 2, 16, 8)])
@pytest.mark.parametrize("m", [1, 7, 16, 20, 47, 64])
def test_decode_linear_rotary_and_cache_write(heads, kv_heads, d, bs, m):
    from paged_llm_amd.parts.registry import BuildEnv
    from paged_llm_amd.parts.rope import RotaryEncoding
    o = ops()
    k_in, pages = 256, 12
    rope = RotaryEncoding({"head_dim": d, "theta": 10000.0, "scaling": None}, BuildEnv(64, torch.bfloat16, torch.device("cuda"), 512, {}))
    rope.prepare(512)
    width = (heads + 2 * kv_heads) * d
    x = rnd(m, k_in, seed=38, dtype=torch.bfloat16)
    w = rnd(width, k_in, seed=39, dtype=torch.bfloat16, scale=k_in ** -0.5)
    positions = torch.tensor([(37 * t + 11) % 500 for t in range(m)], dtype=torch.int32)
    slots = torch.randperm(pages * bs, generator=torch.Generator().manual_seed(40))[:m].to(torch.int32)
    def run_fused():
        kp = torch.zeros(pages, kv_heads, bs, d, dtype=torch.bfloat16).cuda()
        vp = torch.zeros(pages, kv_heads, d, bs, dtype=torch.bfloat16).cuda()
        q = o.decode_linear(x.cuda(), w.cuda(), o.EPI_ROPE_KV, rope=dict(
            positions=positions.cuda(), cos=rope.cos, sin=rope.sin, slots=slots.cuda(), k_pages=kp, v_pages=vp, num_heads=heads,
            num_kv_heads=kv_heads, head_dim=d, block_size=bs))
        return q, kp, vp
    def run_apart():
        kp = torch.zeros(pages, kv_heads, bs, d, dtype=torch.bfloat16).cuda()
        vp = torch.zeros(pages, kv_heads, d, bs, dtype=torch.bfloat16).cuda()
        qkv = o.decode_linear(x.cuda(), w.cuda(), o.EPI_BF16)
        o.rope_scatter(qkv, positions.cuda(), rope.cos, rope.sin, heads, kv_heads, d, slots.cuda(), kp, vp, bs)
        return qkv[:, :heads * d], kp, vp
    for a, b in zip(run_fused(), run_apart()):
        assert torch.equal(a.cpu(), b.cpu())


# ----------------------------------------------------------------------------------- streaming products (17 rows and more)
STREAM_SHAPES = [(48, 64), (100, 96), (517, 160), (2560, 2048), (2048, 5632), (96, 992), (33, 32)]


@pytest.mark.parametrize("m", [1, 17, 33, 64, 100, 128, 200, 264])
@pytest.mark.parametrize("n,k", STREAM_SHAPES)
def test_stream_linear_plain_float_and_partial(m, n, k):
    """Tiled weights, every number of rows (tiles of 32 rows, blocks of up to 128 along y), every blocking of the weight
    rows that the rows' number allows, widths that are no multiple of the stage of 256 columns, and K cut into ranges."""
    o = ops()
    x, w = rnd(m, k, seed=50, dtype=torch.bfloat16), rnd(n, k, seed=51, dtype=torch.bfloat16)
    tiled = o.tile_weight(w.cuda())
    assert tiled.blocks % 24 == 0 and tiled.out_features == n
    want = x.double() @ w.double().T
    rows_per_block = -(-m // -(-m // 128))
    for nt in (1, 2, 3, 4):
        if nt >= 3 and rows_per_block > 64:
            with pytest.raises(o.KernelError):
                o.stream_linear(x.cuda(), tiled, o.SL_F32, nt=nt)
            continue
        assert rel_err(o.stream_linear(x.cuda(), tiled, o.SL_F32, nt=nt), want) <= 2e-5, nt
    assert rel_err(o.stream_linear(x.cuda(), tiled, o.SL_BF16), want) <= 1e-2
    stages = -(-k // 256)
    for splits in {1, 2, stages} - {0}:
        if splits > stages or -(-stages // splits) * (splits - 1) >= stages:
            continue
        parts = o.stream_linear(x.cuda(), tiled, o.SL_PARTIAL, splits=splits)
        assert parts.shape == (splits, m, n) and parts.dtype == torch.float32
        assert rel_err(parts.double().sum(0), want) <= 2e-5, splits


def test_stream_linear_does_not_depend_on_the_other_rows():
    """A row's sums are taken in an order that depends on its place in the matrix only: alone, among 40 or among 200 rows,
    first or last, the same bits."""
    o = ops()
    x, w = rnd(200, 2048, seed=52, dtype=torch.bfloat16), rnd(300, 2048, seed=53, dtype=torch.bfloat16)
    tiled = o.tile_weight(w.cuda())
    whole = o.stream_linear(x.cuda(), tiled, o.SL_F32).cpu()
    for lo, hi in ((0, 40), (150, 200), (77, 78), (0, 17)):
        assert torch.equal(o.stream_linear(x[lo:hi].contiguous().cuda(), tiled, o.SL_F32).cpu(), whole[lo:hi]), (lo, hi)


@pytest.mark.parametrize("m", [17, 41, 64, 128])
@pytest.mark.parametrize("inter,k", [(176, 64), (250, 96), (5632, 2048)])
def test_stream_linear_gated(m, inter, k):
    o = ops()
    x = rnd(m, k, seed=54, dtype=torch.bfloat16)
    w = rnd(2 * inter, k, seed=55, dtype=torch.bfloat16, scale=k ** -0.5)
    want = torch.nn.functional.silu(x.double() @ w[:inter].double().T) * (x.double() @ w[inter:].double().T)
    tiled = o.tile_weight(w.cuda(), "gated")
    for nt in (2, 3):
        if nt == 3 and m > 64:
            continue
        assert rel_err(o.stream_linear(x.cuda(), tiled, o.SL_GATED, nt=nt), want) <= 1e-2
    with pytest.raises(o.KernelError):
        o.stream_linear(x.cuda(), tiled, o.SL_BF16)              # the rows are not in the plain order


@pytest.mark.parametrize("heads,kv_heads,d,bs", [(4, 2, 32, 16), (32, 4, 64, 16), (3, 1, 96, 32), (8, 8, 128, 16), (5, 1, 48, 16), (2, 2, 16, 8)])
@pytest.mark.parametrize("m", [17, 47, 64, 130])
def test_stream_linear_rotary_and_cache_write(heads, kv_heads, d, bs, m):
    """Against the product, then the rotary kernel: the same bits in q and in the pages (both round the projection to
    bfloat16 before the rotation)."""
    from paged_llm_amd.parts.registry import BuildEnv
    from paged_llm_amd.parts.rope import RotaryEncoding
    o = ops()
    k_in, pages = 256, 24
    rope = RotaryEncoding({"head_dim": d, "theta": 10000.0, "scaling": None}, BuildEnv(64, torch.bfloat16, torch.device("cuda"), 512, {}))
    rope.prepare(512)
    width = (heads + 2 * kv_heads) * d
    x = rnd(m, k_in, seed=56, dtype=torch.bfloat16)
    w = rnd(width, k_in, seed=57, dtype=torch.bfloat16, scale=k_in ** -0.5)
    positions = torch.tensor([(37 * t + 11) % 500 for t in range(m)], dtype=torch.int32)
    slots = torch.randperm(pages * bs, generator=torch.Generator().manual_seed(58))[:m].to(torch.int32)
    slots[3] = -1                                                   # a row that writes nothing (padding of a replayed step)
    tiled = o.tile_weight(w.cuda(), "rotary", head_dim=d)
    kp = torch.zeros(pages, kv_heads, bs, d, dtype=torch.bfloat16).cuda()
    vp = torch.zeros(pages, kv_heads, d, bs, dtype=torch.bfloat16).cuda()
    q = o.stream_linear(x.cuda(), tiled, o.SL_ROPE_KV, rope=dict(
        positions=positions.cuda(), cos=rope.cos, sin=rope.sin, slots=slots.cuda(), k_pages=kp, v_pages=vp, num_heads=heads,
        num_kv_heads=kv_heads, head_dim=d, block_size=bs))
    kp2, vp2 = torch.zeros_like(kp), torch.zeros_like(vp)
    qkv = o.stream_linear(x.cuda(), o.tile_weight(w.cuda()), o.SL_BF16)
    assert rel_err(qkv, x.double() @ w.double().T) <= 1e-2
    o.rope_scatter(qkv, positions.cuda(), rope.cos, rope.sin, heads, kv_heads, d, slots.cuda(), kp2, vp2, bs)
    assert torch.equal(q.cpu(), qkv[:, :heads * d].cpu()) and torch.equal(kp.cpu(), kp2.cpu()) and torch.equal(vp.cpu(), vp2.cpu())
    assert kp.float().abs().sum() > 0 and vp.float().abs().sum() > 0


@pytest.mark.parametrize("m", [1, 5, 8, 13, 16])
@pytest.mark.parametrize("n,k", [(48, 64), (517, 160), (2560, 2048), (2048, 5632), (96, 992)])
def test_decode_linear_streams_the_tiled_copy(m, n, k):
    """At most 16 rows with the weights from their tiled copy: plain and float out, with the sum and norm in front, and
    gated; the same sums in the same order as from the row-major matrix wherever that one is read in units of 16 rows too."""
    o = ops()
    x, w = rnd(m, k, seed=60, dtype=torch.bfloat16), rnd(n, k, seed=61, dtype=torch.bfloat16, scale=k ** -0.5)
    tiled = o.tile_weight(w.cuda())
    want = x.double() @ w.double().T
    got = o.decode_linear(x.cuda(), w.cuda(), o.EPI_F32, tiled=tiled)
    assert rel_err(got, want) <= 2e-5
    if m > 8:
        assert torch.equal(got.cpu(), o.decode_linear(x.cuda(), w.cuda(), o.EPI_F32).cpu())
    d, nw = rnd(m, k, seed=62, dtype=torch.bfloat16), 1 + 0.3 * rnd(k, seed=63)
    h = plain.rms_norm((x.float() + d.float()).to(torch.bfloat16).float(), nw, 1e-4).to(torch.bfloat16)
    if o.decode_linear_takes(m, k, x.cuda(), w.cuda()):                  # (the rows fit LDS)
        x_out = torch.zeros(m, k, dtype=torch.bfloat16).cuda()
        got = o.decode_linear(x.cuda(), w.cuda(), o.EPI_BF16, delta=d.cuda(), norm_weight=nw.cuda(), eps=1e-4, x_out=x_out, tiled=tiled)
        assert rel_err(got, h.double() @ w.double().T) <= 1.5e-2
    if n % 2 == 0:
        half = n // 2
        want = torch.nn.functional.silu(x.double() @ w[:half].double().T) * (x.double() @ w[half:].double().T)
        assert rel_err(o.decode_linear(x.cuda(), w.cuda(), o.EPI_GATED, tiled=o.tile_weight(w.cuda(), "gated")), want) <= 1e-2
        with pytest.raises(o.KernelError):
            o.decode_linear(x.cuda(), w.cuda(), o.EPI_GATED, tiled=tiled)      # the plain pairing does not go with the gated epilogue


@pytest.mark.parametrize("heads,kv_heads,d,bs", [(4, 2, 32, 16), (32, 4, 64, 16), (5, 1, 48, 16), (2, 2, 16, 8)])
@pytest.mark.parametrize("m", [1, 8, 16])
def test_decode_linear_rotary_from_the_tiled_copy(heads, kv_heads, d, bs, m):
    from paged_llm_amd.parts.registry import BuildEnv
    from paged_llm_amd.parts.rope import RotaryEncoding
    o = ops()
    k_in, pages = 256, 12
    rope = RotaryEncoding({"head_dim": d, "theta": 10000.0, "scaling": None}, BuildEnv(64, torch.bfloat16, torch.device("cuda"), 512, {}))
    rope.prepare(512)
    width = (heads + 2 * kv_heads) * d
    x = rnd(m, k_in, seed=64, dtype=torch.bfloat16)
    w = rnd(width, k_in, seed=65, dtype=torch.bfloat16, scale=k_in ** -0.5)
    positions = torch.tensor([(37 * t + 11) % 500 for t in range(m)], dtype=torch.int32)
    slots = torch.randperm(pages * bs, generator=torch.Generator().manual_seed(66))[:m].to(torch.int32)
    def run(tiled):
        kp = torch.zeros(pages, kv_heads, bs, d, dtype=torch.bfloat16).cuda()
        vp = torch.zeros(pages, kv_heads, d, bs, dtype=torch.bfloat16).cuda()
        q = o.decode_linear(x.cuda(), w.cuda(), o.EPI_ROPE_KV, tiled=tiled, rope=dict(
            positions=positions.cuda(), cos=rope.cos, sin=rope.sin, slots=slots.cuda(), k_pages=kp, v_pages=vp, num_heads=heads,
            num_kv_heads=kv_heads, head_dim=d, block_size=bs))
        return q.cpu().float(), kp.cpu().float(), vp.cpu().float()
    for a, b in zip(run(o.tile_weight(w.cuda(), "rotary", head_dim=d)), run(None)):
        assert (a - b).abs().max().item() <= 2e-2 * max(1.0, b.abs().max().item()) and b.abs().sum() > 0


@pytest.mark.parametrize("m", [17, 100, 129, 264, 300, 512, 640])
@pytest.mark.parametrize("n,k", STREAM_SHAPES)
def test_tile_linear_plain_float_and_partial(m, n, k):
    """Tiles of up to 128 rows x 128 weight rows with both operands through LDS: every number of rows, widths that are no
    multiple of a stage of 64 columns, fewer weight rows than a tile, and K cut into ranges."""
    o = ops()
    x, w = rnd(m, k, seed=70, dtype=torch.bfloat16), rnd(n, k, seed=71, dtype=torch.bfloat16)
    tiled = o.tile_weight(w.cuda())
    want = x.double() @ w.double().T
    assert rel_err(o.tile_linear(x.cuda(), tiled, o.SL_F32), want) <= 2e-5
    assert rel_err(o.tile_linear(x.cuda(), tiled, o.SL_BF16), want) <= 1e-2
    stages = -(-k // 64)
    for splits in {2, 3, stages}:
        if splits > stages or -(-stages // splits) * (splits - 1) >= stages:
            continue
        parts = o.tile_linear(x.cuda(), tiled, o.SL_PARTIAL, splits=splits)
        assert parts.shape == (splits, m, n) and rel_err(parts.double().sum(0), want) <= 2e-5, splits
    alone = o.tile_linear(x[m // 2:m // 2 + 5].contiguous().cuda(), tiled, o.SL_F32)
    assert torch.equal(alone.cpu(), o.tile_linear(x.cuda(), tiled, o.SL_F32)[m // 2:m // 2 + 5].cpu())     # a row's sums do not depend on the others


def test_tile_shapes_of_the_tiled_kernel():
    """A product in one range of K takes the tile shape with the most workgroups in one round of the compute units; the
    largest tiles when none fits; blocks of rows always cover the rows."""
    shape = ops().tile_linear_shape
    assert shape(264, 2560, 256) == (64, 64, 200)          # q/k/v of a 2048-wide model: 5 blocks of rows x 40 tiles
    assert shape(264, 11264, 256) == (144, 128, 176)       # its gate/up product: two blocks x 88 tiles of 128
    assert shape(128, 11264, 256) == (128, 64, 176)        # one block of rows: tiles of 64 weight rows
    assert shape(64, 28672, 256) == (64, 128, 224)         # a large matrix fills the GPU with tiles of 128
    assert shape(264, 28672, 256) == (144, 128, 448)       # nothing fits one round: the largest tiles
    rng = np.random.default_rng(3)
    for _ in range(500):
        m, n, cus = int(rng.integers(1, 700)), int(rng.integers(1, 40000)), int(rng.choice([64, 104, 256, 304]))
        rows, tile, wgs = shape(m, n, cus)
        assert rows % 16 == 0 and 32 <= rows <= 160 and tile in (64, 128)
        blocks, tiles = -(-m // rows), -(-n // tile)
        assert wgs == blocks * tiles and (blocks - 1) * rows < m <= blocks * rows
        if wgs > cus:                                      # then even the largest tiles do not fit one round
            assert -(-m // 160) * -(-n // 128) > cus and tile == 128


@pytest.mark.parametrize("m", [17, 24, 49, 64, 100, 130, 150, 264])
@pytest.mark.parametrize("size", ["small", "middle", "large"])
def test_tile_linear_gated_and_rotary(m, size):
    """The kernel takes the tile shape that gives the most workgroups in one round: small matrices end up with blocks of 32
    rows x tiles of 64 weight rows at every row count, matrices of a few thousand rows with tiles of 64 weight rows and
    blocks that grow with the rows, and matrices whose tiles of 128 need more than one round keep the largest tiles."""
    from paged_llm_amd.parts.registry import BuildEnv
    from paged_llm_amd.parts.rope import RotaryEncoding
    o = ops()
    wide = size == "large"
    inter, k = {"small": (250, 96), "middle": (5630, 64), "large": (16650, 64)}[size]
    if size == "middle":
        assert o.tile_linear_shape(m, 2 * inter, 256)[:2] == {17: (32, 64), 24: (32, 64), 49: (64, 64), 64: (64, 64), 100: (128, 64), 130: (96, 128),
                                                               150: (96, 128), 264: (144, 128)}[m]
    x = rnd(m, k, seed=72, dtype=torch.bfloat16)
    w = rnd(2 * inter, k, seed=73, dtype=torch.bfloat16, scale=k ** -0.5)
    want = torch.nn.functional.silu(x.double() @ w[:inter].double().T) * (x.double() @ w[inter:].double().T)
    assert rel_err(o.tile_linear(x.cuda(), o.tile_weight(w.cuda(), "gated"), o.SL_GATED), want) <= 1e-2
    heads, kv_heads, d, bs, pages, k_in = {"small": (5, 1, 48, 16, 24, 256), "middle": (100, 2, 48, 16, 24, 64), "large": (340, 3, 48, 16, 24, 64)}[size]
    rope = RotaryEncoding({"head_dim": d, "theta": 10000.0, "scaling": None}, BuildEnv(64, torch.bfloat16, torch.device("cuda"), 512, {}))
    rope.prepare(512)
    x = rnd(m, k_in, seed=74, dtype=torch.bfloat16)
    w = rnd((heads + 2 * kv_heads) * d, k_in, seed=75, dtype=torch.bfloat16, scale=k_in ** -0.5)
    positions = torch.tensor([(37 * t + 11) % 500 for t in range(m)], dtype=torch.int32)
    slots = torch.randperm(pages * bs, generator=torch.Generator().manual_seed(76))[:m].to(torch.int32)
    kp = torch.zeros(pages, kv_heads, bs, d, dtype=torch.bfloat16).cuda()
    vp = torch.zeros(pages, kv_heads, d, bs, dtype=torch.bfloat16).cuda()
    q = o.tile_linear(x.cuda(), o.tile_weight(w.cuda(), "rotary", head_dim=d), o.SL_ROPE_KV, rope=dict(
        positions=positions.cuda(), cos=rope.cos, sin=rope.sin, slots=slots.cuda(), k_pages=kp, v_pages=vp, num_heads=heads,
        num_kv_heads=kv_heads, head_dim=d, block_size=bs))
    kp2, vp2 = torch.zeros_like(kp), torch.zeros_like(vp)
    qkv = o.tile_linear(x.cuda(), o.tile_weight(w.cuda()), o.SL_BF16)
    o.rope_scatter(qkv, positions.cuda(), rope.cos, rope.sin, heads, kv_heads, d, slots.cuda(), kp2, vp2, bs)
    assert torch.equal(q.cpu(), qkv[:, :heads * d].cpu()) and torch.equal(kp.cpu(), kp2.cpu()) and torch.equal(vp.cpu(), vp2.cpu())
    assert kp.float().abs().sum() > 0
