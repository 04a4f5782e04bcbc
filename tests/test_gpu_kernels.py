"""Each HIP kernel alone against its plain float64 formula, at sizes other than the tiny models':
widths and vocabularies that are no power of two, head sizes in steps of 16, odd head groupings,
several page sizes, both storage types."""
import math

import pytest
import torch

from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float32) * scale


def tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def as_stored(x, dtype):
    """Round to the storage type and give both the device tensor and its exact float64 value."""
    dev = x.to(dtype).to(DEV)
    return dev, dev.cpu().to(F64)


@pytest.fixture(scope="module")
def k():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from pulse_infer_amd.ops import kernels, library
    library.load()
    return kernels


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_gather(k, dtype):
    table, ref = as_stored(rnd(37, 70), dtype)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32, device=DEV)
    out = torch.full((5, 70), 7.0, device=DEV)
    bad = torch.zeros(1, dtype=torch.int32, device=DEV)
    k.embed_gather(ids, table, out, bad)
    assert torch.equal(out.cpu().to(F64), ref[ids.cpu().long()]) and bad.item() == 0
    k.embed_gather(torch.tensor([3, 37, -1], dtype=torch.int32, device=DEV), table, out[:3], bad)
    # refused loudly, nothing read out of range: the flag, and rows that poison whatever is computed from them
    assert bad.item() == 1 and bool(out[1:3].isnan().all()) and torch.equal(out[0].cpu().to(F64), ref[3])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [48, 1000, 4100])
def test_add_rmsnorm(k, dtype, hidden):
    rows, eps = 9, 3e-5
    h = rnd(rows, hidden, seed=1).to(DEV)
    delta, dref = as_stored(rnd(rows, hidden, seed=2), dtype)
    w, wref = as_stored(1 + 0.1 * rnd(hidden, seed=3), dtype)
    want_sum = h.cpu().to(F64) + dref
    out = torch.empty(rows, hidden, dtype=dtype, device=DEV)
    hh = h.clone()
    k.add_rmsnorm(hh, delta, w, eps, out)
    assert torch.allclose(out.cpu().to(F64), P.rms_norm(want_sum, wref, eps), **tol(dtype))
    assert torch.allclose(hh.cpu().to(F64), want_sum, atol=1e-6)            # the residual keeps the sum, in float32
    # without delta nothing is written back; gathered rows leave h alone
    hh = h.clone()
    k.add_rmsnorm(hh, None, w, eps, out)
    assert torch.equal(hh, h)
    assert torch.allclose(out.cpu().to(F64), P.rms_norm(h.cpu().to(F64), wref, eps), **tol(dtype))
    pick = torch.tensor([8, 0, 3], dtype=torch.int32, device=DEV)
    out3 = torch.empty(3, hidden, dtype=dtype, device=DEV)
    k.add_rmsnorm(hh, delta, w, eps, out3, rows=pick)
    assert torch.equal(hh, h)
    assert torch.allclose(out3.cpu().to(F64), P.rms_norm(want_sum[[8, 0, 3]], wref, eps), **tol(dtype))


def test_residual_add_and_gather_rows(k):
    h = rnd(5, 33).to(DEV)
    d, dref = as_stored(rnd(5, 33, seed=1), torch.bfloat16)
    want = h.cpu().to(F64) + dref
    k.residual_add(h, d)
    assert torch.allclose(h.cpu().to(F64), want, atol=1e-6)
    out = torch.empty(2, 33, device=DEV)
    k.gather_rows(h, torch.tensor([4, 1], dtype=torch.int32, device=DEV), out)
    assert torch.equal(out, h[[4, 1]])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu(k, dtype):
    gu, ref = as_stored(rnd(7, 2 * 77, seed=4, scale=3.0), dtype)
    out = torch.empty(7, 77, dtype=dtype, device=DEV)
    k.swiglu(gu, out)
    assert torch.allclose(out.cpu().to(F64), P.silu(ref[:, :77]) * ref[:, 77:], **tol(dtype))


@pytest.mark.parametrize("shape", [(1, 7, 5), (3, 70, 33), (65, 129, 100), (130, 64, 257)])
@pytest.mark.parametrize("types", [(torch.float32, torch.float32, torch.float32),
                                   (torch.bfloat16, torch.bfloat16, torch.float32),
                                   (torch.float32, torch.bfloat16, torch.bfloat16)])
def test_gemm_f32(k, shape, types):
    m, n, kk = shape
    a, aref = as_stored(rnd(m, kk, seed=5), types[0])
    w, wref = as_stored(rnd(n, kk, seed=6), types[1])
    out = torch.empty(m, n, dtype=types[2], device=DEV)
    k.gemm_f32(a, w, out)
    assert torch.allclose(out.cpu().to(F64), aref @ wref.T, **(tol(types[2]) if types[2] == torch.bfloat16
                                                               else dict(atol=1e-4, rtol=1e-5)))


def test_gemm_f32_rows_do_not_depend_on_the_batch(k):
    a = rnd(40, 300, seed=7).to(DEV)
    w = rnd(90, 300, seed=8).to(DEV)
    full = torch.empty(40, 90, device=DEV)
    k.gemm_f32(a, w, full)
    one = torch.empty(1, 90, device=DEV)
    k.gemm_f32(a[17:18], w, one)
    assert torch.equal(one[0], full[17])                                   # same sums in the same order


def test_rope_table(k):
    theta, rot = 1e6, 48
    pos = torch.tensor([0, 1, 2, 1000, 40959], dtype=torch.int32, device=DEV)
    inv = torch.pow(torch.tensor(theta, dtype=F64), -torch.arange(rot // 2, dtype=F64) * 2 / rot).to(DEV)
    cos = torch.empty(5, rot // 2, device=DEV)
    sin = torch.empty_like(cos)
    k.rope_table(pos, inv, cos, sin)
    angle = pos.cpu().to(F64)[:, None] / theta ** (torch.arange(0, rot, 2, dtype=F64) / rot)
    assert torch.allclose(cos.cpu().to(F64), torch.cos(angle), atol=1e-7)
    assert torch.allclose(sin.cpu().to(F64), torch.sin(angle), atol=1e-7)


def _cache(pages, nkv, bs, d, dtype):
    return (torch.zeros(pages, nkv, bs, d, dtype=dtype, device=DEV),
            torch.zeros(pages, nkv, d, bs, dtype=dtype, device=DEV))


def _stale(kc, vc, seed=0):
    """What pages hold that have been used before, and worse: every page, its slots beyond a request's context
    included, is filled with ordinary values, with NaN, with +Inf or with -Inf before the requests' keys and values
    go in (a request that was fed an id outside the table leaves NaN behind).  Nothing of it may reach an output: a
    stale value times a weight of zero is not zero."""
    kinds = torch.randint(0, 4, (kc.shape[0],), generator=torch.Generator().manual_seed(1000 + seed)).tolist()
    kc.normal_()
    vc.normal_()
    for page, kind in enumerate(kinds):
        if kind:
            value = (float("nan"), float("inf"), float("-inf"))[kind - 1]
            kc[page].fill_(value)
            vc[page].fill_(value)


def _bits(t):
    """The tensor's bit patterns, so that NaN compares equal to itself."""
    return t.cpu().contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


def _tables(k, positions, theta, rot):
    inv = torch.pow(torch.tensor(theta, dtype=F64), -torch.arange(rot // 2, dtype=F64) * 2 / rot).to(DEV)
    cos = torch.empty(len(positions), rot // 2, device=DEV)
    sin = torch.empty_like(cos)
    k.rope_table(torch.tensor(positions, dtype=torch.int32, device=DEV), inv, cos, sin)
    return cos, sin


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [
    dict(nq=5, nkv=5, d=16, rot=16, pairing="interleaved", norm=True, bs=4),
    dict(nq=6, nkv=2, d=48, rot=48, pairing="interleaved", norm=True, bs=16),
    dict(nq=4, nkv=1, d=80, rot=32, pairing="interleaved", norm=True, bs=8),    # partial rotation, tail untouched
    dict(nq=3, nkv=3, d=160, rot=160, pairing="half", norm=False, bs=16),       # other pairing, no norm, > 128 channels
    dict(nq=2, nkv=1, d=32, rot=0, pairing="interleaved", norm=True, bs=2),     # no position encoding at all
    dict(nq=7, nkv=7, d=64, rot=32, pairing="half", norm=True, bs=16),          # other pairing, partial rotation
    dict(nq=5, nkv=1, d=128, rot=128, pairing="interleaved", norm=True, bs=16), # heads no multiple of a wavefront's share
    dict(nq=2, nkv=2, d=20, rot=12, pairing="half", norm=True, bs=4),           # sizes only the element-wise kernel takes
])
def test_qk_rope_kv(k, dtype, case):
    nq, nkv, d, rot, bs = case["nq"], case["nkv"], case["d"], case["rot"], case["bs"]
    eps, theta = 2e-5, 7e4
    # two requests in one step: 5 tokens from position 6 (crossing a page edge for small pages) and 1 token at 0
    positions = [6, 7, 8, 9, 10, 0]
    entry = [0, 0, 0, 0, 0, 1]
    width = 10 // bs + 1
    pages_a = list(range(3, 3 + width))
    table = torch.full((2, width), -1, dtype=torch.int32)
    table[0] = torch.tensor(pages_a, dtype=torch.int32)
    table[1, 0] = 1
    kc, vc = _cache(3 + width + 1, nkv, bs, d, dtype)
    qkv, ref = as_stored(rnd(6, (nq + 2 * nkv) * d + 8, seed=9), dtype)      # 8 spare columns: rows are strided
    qw, qwref = as_stored(1 + 0.1 * rnd(d, seed=10), dtype)
    kw, kwref = as_stored(1 + 0.1 * rnd(d, seed=11), dtype)
    cos, sin = _tables(k, positions, theta, rot) if rot else (None, None)
    k.qk_rope_kv(qkv, nq, nkv, d, qw if case["norm"] else None, kw if case["norm"] else None, eps, cos, sin, rot,
                 0 if case["pairing"] == "interleaved" else 1, kc, vc,
                 torch.tensor(positions, dtype=torch.int32, device=DEV), torch.tensor(entry, dtype=torch.int32, device=DEV),
                 table.to(DEV))
    q = ref[:, :nq * d].reshape(6, nq, d)
    kk = ref[:, nq * d:(nq + nkv) * d].reshape(6, nkv, d)
    vv = ref[:, (nq + nkv) * d:(nq + 2 * nkv) * d].reshape(6, nkv, d)
    if case["norm"]:
        q, kk = P.rms_norm(q, qwref, eps), P.rms_norm(kk, kwref, eps)
    if rot:
        q = P.rope(q, positions, theta, rot, case["pairing"])
        kk = P.rope(kk, positions, theta, rot, case["pairing"])
    got = qkv.cpu().to(F64)
    assert torch.allclose(got[:, :nq * d].reshape(6, nq, d), q, **tol(dtype))
    assert torch.equal(got[:, nq * d:], ref[:, nq * d:])                    # k, v and the spare columns stay as they were
    kcpu, vcpu = kc.cpu().to(F64), vc.cpu().to(F64)
    touched = torch.zeros(kc.shape[0], bs, dtype=torch.bool)
    for t, (p, e) in enumerate(zip(positions, entry)):
        page, slot = int(table[e, p // bs]), p % bs
        touched[page, slot] = True
        assert torch.allclose(kcpu[page, :, slot, :], kk[t], **tol(dtype))
        assert torch.equal(vcpu[page, :, :, slot], vv[t])                   # values are copied as they are
    assert torch.all(kcpu[~touched.unsqueeze(1).expand(-1, nkv, -1)] == 0)  # nothing else was written


def _fill_cache(kc, vc, keys, vals, table_row, bs):
    """Put keys/vals [S, nkv, d] of one request into its pages."""
    for j in range(keys.shape[0]):
        page, slot = table_row[j // bs], j % bs
        kc[page, :, slot, :] = keys[j]
        vc[page, :, :, slot] = vals[j]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [
    dict(nq=4, nkv=2, d=16, bs=4, window=0),
    dict(nq=6, nkv=1, d=32, bs=16, window=0),
    dict(nq=3, nkv=3, d=48, bs=8, window=7),
    dict(nq=8, nkv=2, d=128, bs=16, window=0),
    dict(nq=2, nkv=1, d=208, bs=32, window=40),
])
def test_attn_generic(k, dtype, case):
    nq, nkv, d, bs, window = case["nq"], case["nkv"], case["d"], case["bs"], case["window"]
    lens = [70, 131]                        # contexts of two requests; crossing the 64-key tile and page edges
    pages = [[126 - 2 * i for i in range((lens[0] + bs - 1) // bs)],       # descending even pages
             [2 * i + 1 for i in range((lens[1] + bs - 1) // bs)]]         # ascending odd pages
    width = max(len(p) for p in pages)
    kc, vc = _cache(128, nkv, bs, d, dtype)
    _stale(kc, vc)
    refs = []
    for r, n in enumerate(lens):
        ks, kref = as_stored(rnd(n, nkv, d, seed=20 + r), dtype)
        vs, vref = as_stored(rnd(n, nkv, d, seed=30 + r), dtype)
        _fill_cache(kc, vc, ks, vs, pages[r], bs)
        refs.append((kref, vref))
    table = torch.full((2, width), -1, dtype=torch.int32)
    for r, p in enumerate(pages):
        table[r, :len(p)] = torch.tensor(p, dtype=torch.int32)
    # request 0: its last 9 tokens as a portion; request 1: a single decoded token; and an early token of request 1
    positions = list(range(lens[0] - 9, lens[0])) + [lens[1] - 1]
    entry = [0] * 9 + [1]
    q, qref = as_stored(rnd(len(positions), nq * d + 16, seed=40), dtype)
    out = torch.zeros(len(positions), nq * d, dtype=dtype, device=DEV)
    scale = 0.37
    k.attn_generic(q, out, nq, nkv, d, kc, vc, torch.tensor(positions, dtype=torch.int32, device=DEV),
                   torch.tensor(entry, dtype=torch.int32, device=DEV), table.to(DEV), scale, window)
    got = out.cpu().to(F64).reshape(-1, nq, d)
    for t, (p, e) in enumerate(zip(positions, entry)):
        kref, vref = refs[e]
        want = P.causal_attention(qref[t:t + 1, :nq * d].reshape(1, nq, d), kref[:p + 1], vref[:p + 1], scale,
                                  window or None, [p])
        assert torch.allclose(got[t], want[0], **tol(dtype)), (t, p, e)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attn_generic_one_far_key_and_the_window_edge(k, dtype):
    """Random keys would hide a key that is skipped or read from the wrong page: make one score stand out."""
    nq, nkv, d, bs, n = 2, 1, 32, 16, 600
    pages = list(range(n // bs + 1))
    table = torch.tensor([pages], dtype=torch.int32, device=DEV)
    for target, window, seen in ((3, 0, True), (n - 100, 100, True), (n - 101, 100, False), (bs * 7, 0, True),
                                 (bs * 7 - 1, 0, True), (n - 1, 1, True)):
        kc, vc = _cache(len(pages), nkv, bs, d, dtype)
        keys = rnd(n, nkv, d, seed=50, scale=0.1)
        vals = rnd(n, nkv, d, seed=51)
        keys[target] = 0
        keys[target, 0, 0] = 30.0
        ks, kref = as_stored(keys, dtype)
        vs, vref = as_stored(vals, dtype)
        _fill_cache(kc, vc, ks, vs, pages, bs)
        qv = rnd(1, nq * d, seed=52, scale=0.1)
        qv[0, 0] = 30.0
        qv[0, d] = 30.0
        q, qref = as_stored(qv, dtype)
        out = torch.zeros(1, nq * d, dtype=dtype, device=DEV)
        k.attn_generic(q, out, nq, nkv, d, kc, vc, torch.tensor([n - 1], dtype=torch.int32, device=DEV),
                       torch.tensor([0], dtype=torch.int32, device=DEV), table, 1.0, window)
        got = out.cpu().to(F64).reshape(nq, d)
        close = torch.allclose(got, vref[target].expand(nq, d), atol=1e-2)
        assert close == seen, (target, window)
        want = P.causal_attention(qref.reshape(1, nq, d), kref, vref, 1.0, window or None, [n - 1])
        assert torch.allclose(got, want[0], **tol(dtype)), (target, window)


def test_argmax_takes_the_lowest_index_among_equals(k):
    logits = rnd(5, 1009, seed=60).to(DEV)
    logits[0, 17] = logits[0, 800] = 50.0
    logits[1, 1008] = 60.0
    logits[2, 0] = 60.0
    logits[3] = 1.25
    logits[4, 5] = float("nan")
    out = torch.empty(5, dtype=torch.int32, device=DEV)
    k.sample(logits, out)
    want = [17, 1008, 0, 0, int(torch.argmax(torch.nan_to_num(logits[4].cpu(), nan=-1e30)))]
    assert out.tolist() == want


def test_temperature_sampling_follows_the_softmax(k):
    vocab, rows = 700, 4000
    base = torch.full((vocab,), -30.0)
    base[[5, 123, 400, 699]] = torch.tensor([1.0, 2.0, 0.5, 1.5])
    logits = base.repeat(rows, 1).to(DEV)
    temperature = torch.full((rows,), 0.8, device=DEV)
    uniform = torch.rand(rows, generator=torch.Generator().manual_seed(1)).to(DEV)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    k.sample(logits, out, temperature=temperature, uniform=uniform)
    counts = torch.bincount(out.cpu().long(), minlength=vocab).double() / rows
    want = torch.softmax(base.double() / 0.8, dim=0)
    assert torch.allclose(counts, want, atol=0.03)
    # the same uniform number gives the same token, whatever else is in the batch
    again = torch.empty(1, dtype=torch.int32, device=DEV)
    k.sample(logits[7:8], again, temperature=temperature[7:8], uniform=uniform[7:8])
    assert again.item() == out[7].item()


def test_top_k_top_p_penalty_and_banned(k):
    vocab, rows = 333, 3000
    base = torch.linspace(-3, 3, vocab)[torch.randperm(vocab, generator=torch.Generator().manual_seed(2))]
    logits = base.repeat(rows, 1).to(DEV)
    uniform = torch.rand(rows, generator=torch.Generator().manual_seed(3)).to(DEV)
    temperature = torch.ones(rows, device=DEV)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    # top-k: only the k largest ever appear, with renormalised softmax frequencies
    k.sample(logits, out, temperature=temperature, uniform=uniform,
             top_k=torch.full((rows,), 5, dtype=torch.int32, device=DEV))
    top5 = torch.topk(base, 5).indices
    assert set(out.tolist()) <= set(top5.tolist())
    freq = torch.bincount(out.cpu().long(), minlength=vocab).double()[top5] / rows
    assert torch.allclose(freq, torch.softmax(base[top5].double(), 0), atol=0.03)
    # top-p: the shortest prefix of the sorted distribution whose mass reaches p
    probs = torch.softmax(base.double(), 0)
    order = torch.argsort(probs, descending=True)
    keep = order[: int((torch.cumsum(probs[order], 0) < 0.3).sum()) + 1]
    k.sample(logits, out, temperature=temperature, uniform=uniform, top_p=torch.full((rows,), 0.3, device=DEV))
    assert set(out.tolist()) == set(keep.tolist())
    # presence penalty: a seen token loses `penalty` before the choice; banned ids never appear
    words = (vocab + 31) // 32
    seen = torch.zeros(2, words, dtype=torch.int32, device=DEV)
    best = int(torch.argmax(base))
    second = int(torch.topk(base, 2).indices[1])
    k.mark_seen(seen, torch.tensor([1, 1], dtype=torch.int32, device=DEV),
                torch.tensor([best, 7], dtype=torch.int32, device=DEV), vocab)
    greedy = torch.empty(2, dtype=torch.int32, device=DEV)
    k.sample(logits[:2], greedy, penalty=torch.tensor([1.5, 1.5], device=DEV),
             seen_row=torch.tensor([0, 1], dtype=torch.int32, device=DEV), seen_masks=seen)
    assert greedy.tolist() == [best, second]
    banned = torch.zeros(words, dtype=torch.int32)
    banned[best >> 5] = 1 << (best & 31) if (best & 31) < 31 else -(1 << 31)
    k.sample(logits[:1], greedy[:1], banned=banned.to(DEV))
    assert greedy[0].item() == second


@pytest.mark.parametrize("mode,vocab,chunked", [
    ("temperature", 151936, False), ("top_k", 151936, False), ("top_k_top_p", 151936, False), ("top_p", 151936, False),
    ("top_p_peaked", 151936, False), ("ties", 151936, False), ("many_ties", 151936, False), ("penalty", 151936, False),
    # candidates found in chunks of the vocabulary: rows that fit, rows with too many equal values (left to the kernel
    # with a workgroup a row), a vocabulary of fewer chunks than k (the same), one of barely more; top-p alone on
    # peaked rows (the short list holds its share) and on flat ones (it does not)
    ("top_k", 151936, True), ("top_k_top_p", 151936, True), ("ties", 151936, True), ("many_ties", 151936, True),
    ("penalty", 151936, True), ("temperature", 151936, True), ("top_p", 151936, True), ("top_p_peaked", 151936, True),
    ("top_p_flat", 151936, True), ("top_p_peaked", 43000, True),
    ("top_k", 5000, True), ("top_k_top_p", 43000, True), ("top_k", 2048 * 20, True)])
def test_sampling_at_a_real_vocabulary(k, mode, vocab, chunked):
    """The draw of every row against the same steps in float64: kept set by thresholds (top-k, then top-p on what
    top-k kept), cumulative walk in vocabulary order.  The chosen token must be kept and the draw must fall into its
    interval of the cumulative sum (up to float32 rounding of the sums)."""
    rows = 48
    gen = torch.Generator().manual_seed(11)
    # flat enough that top-p alone needs thousands of tokens (the passes over the whole vocabulary), or peaked so that
    # a thousand hold its mass (the short list)
    logits = torch.randn(rows, vocab, generator=gen) * {"top_p_peaked": 8.0, "top_p_flat": 0.5}.get(mode, 2.5)
    if mode in ("ties", "many_ties"):        # the k-th largest value many times: all of its copies are kept
        logits[:, ::(97 if mode == "ties" else 40)] = 20.0
    temp = 0.7
    top_k = {"top_k": 20, "top_k_top_p": 50, "ties": 40, "many_ties": 40, "penalty": 20}.get(mode, 0)
    top_p = {"top_k_top_p": 0.9, "top_p": 0.8, "top_p_peaked": 0.9, "top_p_flat": 0.9, "penalty": 0.95}.get(mode, 0.0)
    uniform = torch.rand(rows, generator=gen)
    dev = lambda t: t.to(DEV)
    kw = dict(temperature=dev(torch.full((rows,), temp)), uniform=dev(uniform))
    if top_k:
        kw["top_k"] = dev(torch.full((rows,), top_k, dtype=torch.int32))
    if top_p:
        kw["top_p"] = dev(torch.full((rows,), top_p))
    ref = logits.to(F64).clone()
    if mode == "penalty":
        words = (vocab + 31) // 32
        seen = torch.zeros(rows, words, dtype=torch.int32, device=DEV)
        best = torch.argmax(logits, dim=1).to(torch.int32)
        k.mark_seen(seen, torch.arange(rows, dtype=torch.int32, device=DEV), dev(best), vocab)
        kw.update(penalty=dev(torch.full((rows,), 1.5)), seen_row=torch.arange(rows, dtype=torch.int32, device=DEV),
                  seen_masks=seen)
        ref[torch.arange(rows), best.long()] -= 1.5
    out = torch.full((rows,), -9, dtype=torch.int32, device=DEV)

    def draw(logits_dev, out_dev, **args):
        if not chunked:
            return k.sample(logits_dev, out_dev, **args)
        scratch = _chunked_scratch(k, out_dev.numel(), vocab)
        k.sample_chunked(logits_dev, out_dev, scratch, **args)
        if mode in ("top_k", "top_k_top_p", "penalty", "ties", "temperature", "top_p_peaked") and vocab >= 2048 * 50:
            assert bool((scratch["done"][: out_dev.numel()] == 1).all())     # these rows fit: no row was left over
        if mode in ("many_ties", "top_p_flat") or vocab == 5000:
            assert bool((scratch["done"][: out_dev.numel()] == 0).all())     # and these did not (top-p alone on a flat
                                                                             # row: thousands of tokens hold its share)

    draw(dev(logits), out, **kw)
    got = out.cpu().tolist()
    for r in range(rows):
        x = ref[r]
        kept = torch.ones(vocab, dtype=torch.bool)
        if top_k:
            kept &= x >= torch.topk(x, top_k).values[-1]
        w = torch.where(kept, torch.exp((x - x.max()) / temp), torch.zeros_like(x))
        if top_p:
            order = torch.argsort(w, descending=True)
            csum = torch.cumsum(w[order], 0)
            cut = int((csum < top_p * w.sum()).sum())                # the first place where the mass reaches p
            kept &= x >= x[order[cut]]
            w = torch.where(kept, w, torch.zeros_like(w))
        cum = torch.cumsum(w, 0)
        target = float(uniform[r]) * float(cum[-1])
        t = got[r]
        slack = 2e-5 * float(cum[-1])
        assert kept[t], (mode, r, t)
        assert float(cum[t]) - float(w[t]) - slack <= target <= float(cum[t]) + slack, (mode, r, t)
    again = torch.empty(1, dtype=torch.int32, device=DEV)            # a row's draw does not depend on the other rows
    one = {n: v[5:6] for n, v in kw.items() if n not in ("seen_masks",)}
    if "seen_masks" in kw:
        one["seen_masks"] = kw["seen_masks"]
    draw(dev(logits[5:6]), again, **one)
    assert again.item() == got[5]


def _chunked_scratch(k, rows, vocab):
    scratch = k.sample_chunked_scratch(rows, vocab, DEV)
    for t in scratch.values():                             # nothing that was not written is used
        t.fill_(float("nan") if t.dtype == torch.float32 else -3)
    return scratch


@pytest.mark.parametrize("vocab", [151936, 2048, 2049, 700])
def test_sampling_in_chunks(k, vocab):
    """Rows without top-k and top-p through the kernels that cut a row into chunks (a workgroup a chunk): greedy rows
    (ties, NaN, all banned) beside rows at a temperature, a presence penalty and banned ids; every draw against the
    same steps in float64, as for the kernel that takes a workgroup a row, and the same draw whatever else is batched."""
    rows = 40
    gen = torch.Generator().manual_seed(21)
    logits = torch.randn(rows, vocab, generator=gen) * 2.5
    logits[0, 17] = logits[0, vocab - 3] = 50.0            # greedy: the lowest index among equals
    logits[1, vocab - 1] = 60.0
    logits[2, 5] = float("nan")
    temp = torch.full((rows,), 0.7)
    temp[:4] = 0.0                                          # rows 0 to 3 are greedy
    temp[4] = 5.0                                           # a flat row
    uniform = torch.rand(rows, generator=gen)
    uniform[5] = 0.0
    uniform[6] = 0.99999994                                 # the last kept token, not beyond it
    words = (vocab + 31) // 32
    banned = torch.zeros(words, dtype=torch.int64)
    for tok in (3, 40, vocab - 1):
        banned[tok >> 5] |= 1 << (tok & 31)
    banned = torch.where(banned >= 2 ** 31, banned - 2 ** 32, banned).to(torch.int32)
    seen = torch.zeros(rows, words, dtype=torch.int32, device=DEV)
    best = torch.argmax(torch.nan_to_num(logits, nan=-1e30), dim=1).to(torch.int32)
    k.mark_seen(seen, torch.arange(rows, dtype=torch.int32, device=DEV), best.to(DEV), vocab)
    penalty = torch.zeros(rows)
    penalty[10:20] = 1.5
    ref = torch.nan_to_num(logits.to(F64), nan=float("-inf")).clone()
    ref[torch.arange(10, 20), best[10:20].long()] -= 1.5
    ref[:, [3, 40, vocab - 1]] = float("-inf")
    dev = lambda t: t.to(DEV)
    kw = dict(temperature=dev(temp), uniform=dev(uniform), penalty=dev(penalty),
              seen_row=torch.arange(rows, dtype=torch.int32, device=DEV), seen_masks=seen, banned=dev(banned))
    out = torch.full((rows,), -5, dtype=torch.int32, device=DEV)
    k.sample_chunked(dev(logits), out, _chunked_scratch(k, rows, vocab), **kw)
    got = out.cpu().tolist()
    for r in range(rows):
        x = ref[r]
        if float(temp[r]) <= 0:
            assert got[r] == int(torch.argmax(x)), r       # torch.argmax: the first of equals
            continue
        w = torch.exp((x - x.max()) / float(temp[r]))
        cum = torch.cumsum(w, 0)
        target = float(uniform[r]) * float(cum[-1])
        t = got[r]
        slack = 2e-5 * float(cum[-1])
        assert float(w[t]) > 0 and t not in (3, 40, vocab - 1), (r, t)
        assert float(cum[t]) - float(w[t]) - slack <= target <= float(cum[t]) + slack, (r, t)
    # the kernel with a workgroup a row agrees (its sums run in another order: draws at an interval's edge may differ)
    other = torch.empty(rows, dtype=torch.int32, device=DEV)
    k.sample(dev(logits), other, **kw)
    assert sum(a != b for a, b in zip(got, other.cpu().tolist())) <= 1
    # a row's draw does not depend on the other rows
    again = torch.empty(1, dtype=torch.int32, device=DEV)
    one = {n: v[12:13] for n, v in kw.items() if n not in ("seen_masks", "banned")}
    one["seen_row"] = torch.tensor([12], dtype=torch.int32, device=DEV)
    k.sample_chunked(dev(logits[12:13]), again, _chunked_scratch(k, 1, vocab), seen_masks=seen, banned=dev(banned), **one)
    assert again.item() == got[12]
    # nothing left of a row: -1
    everything = torch.full((words,), -1, dtype=torch.int32, device=DEV)
    k.sample_chunked(dev(logits[:2]), out[:2], _chunked_scratch(k, 2, vocab), temperature=dev(temp[4:6]),
                     uniform=dev(uniform[:2]), banned=everything)
    assert out[:2].tolist() == [-1, -1]


@pytest.mark.parametrize("vocab", [151936, 43000])
def test_rows_of_every_kind_in_one_step_draw_what_they_draw_alone(k, vocab):
    """Greedy rows, rows at a temperature, with top-k, with top-k and top-p, with top-p alone and rows whose
    candidates do not fit, in one call: every row draws the token that it draws in a call of its own, with and
    without the options that it does not use (a seeded request does not depend on what it is batched with)."""
    rows = 24
    gen = torch.Generator().manual_seed(5)
    logits = torch.randn(rows, vocab, generator=gen) * 2.5
    logits[20:, ::40] = 20.0                                # rows 20 to 23: too many equal values for a segment
    temp = torch.full((rows,), 0.8)
    temp[0:4] = 0.0
    top_k = torch.zeros(rows, dtype=torch.int32)
    top_k[8:16] = 20
    top_k[20:] = 40
    top_p = torch.zeros(rows)
    top_p[12:20] = 0.9
    uniform = torch.rand(rows, generator=gen)
    dev = lambda t: t.to(DEV)
    out = torch.full((rows,), -5, dtype=torch.int32, device=DEV)
    scratch = _chunked_scratch(k, rows, vocab)
    k.sample_chunked(dev(logits), out, scratch, temperature=dev(temp), top_k=dev(top_k), top_p=dev(top_p),
                     uniform=dev(uniform))
    got = out.cpu().tolist()
    done = scratch["done"].cpu().tolist()
    assert done[:16] == [1] * 16 and done[20:] == [0] * 4       # (top-p alone, rows 16 to 19: as the row's shape has it)
    for r in range(rows):
        alone = torch.empty(1, dtype=torch.int32, device=DEV)
        kw = dict(temperature=dev(temp[r:r + 1]), uniform=dev(uniform[r:r + 1]))
        if int(top_k[r]):
            kw["top_k"] = dev(top_k[r:r + 1])
        if float(top_p[r]):
            kw["top_p"] = dev(top_p[r:r + 1])
        k.sample_chunked(dev(logits[r:r + 1]), alone, _chunked_scratch(k, 1, vocab), **kw)
        assert alone.item() == got[r], r
        if float(temp[r]) <= 0:
            assert got[r] == int(torch.argmax(logits[r]))


def test_temperature_sampling_in_chunks_follows_the_softmax(k):
    vocab, rows = 5000, 4000
    base = torch.full((vocab,), -30.0)
    base[[5, 2047, 2048, 4999]] = torch.tensor([1.0, 2.0, 0.5, 1.5])     # on both sides of a chunk's edge
    logits = base.repeat(rows, 1).to(DEV)
    temperature = torch.full((rows,), 0.8, device=DEV)
    uniform = torch.rand(rows, generator=torch.Generator().manual_seed(1)).to(DEV)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    k.sample_chunked(logits, out, _chunked_scratch(k, rows, vocab), temperature=temperature, uniform=uniform)
    counts = torch.bincount(out.cpu().long(), minlength=vocab).double() / rows
    want = torch.softmax(base.double() / 0.8, dim=0)
    assert torch.allclose(counts, want, atol=0.03)


def test_kernels_refuse_what_they_cannot_do(k):
    from pulse_infer_amd.ops import KernelError
    with pytest.raises(KernelError, match="GPU"):
        k.swiglu(torch.zeros(2, 4), torch.zeros(2, 2))
    with pytest.raises(KernelError, match="storage type"):
        k.swiglu(torch.zeros(2, 4, dtype=torch.float16, device=DEV), torch.zeros(2, 2, dtype=torch.float16, device=DEV))
    with pytest.raises(KernelError, match="inner sizes"):
        k.gemm_f32(torch.zeros(2, 4, device=DEV), torch.zeros(3, 5, device=DEV), torch.zeros(2, 3, device=DEV))
    kc, vc = _cache(2, 1, 4, 1024, torch.float32)
    with pytest.raises(KernelError, match="head_dim"):
        k.attn_generic(torch.zeros(1, 1024, device=DEV), torch.zeros(1, 1024, device=DEV), 1, 1, 1024, kc, vc,
                       torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV),
                       torch.zeros(1, 1, dtype=torch.int32, device=DEV), 1.0)


# ------------------------------------------------------- matrix-core attention
def _mfma_case(k, nq, nkv, d, bs, window, lens, portion, split, seed=0, portion_split=0, made_for=None, planned=None):
    """Requests with contexts `lens`; request 0 brings its last `portion` tokens, the others one token each.
    ``portion_split``: request 0's portion goes through the prompt-portion kernel with its keys in splits of that size.
    ``made_for = (context, splits)``: the launch is made for contexts up to that (as a recorded step's is for its
    bucket) and is told the longest context there is through ``live_context``.  ``planned = (slots, first_wave,
    min_keys)``: such a launch with a plan made on the device instead."""
    from pulse_infer_amd.ops import attention_mfma as M
    dtype = torch.bfloat16
    pages_per = [(n + bs - 1) // bs for n in lens]
    total = sum(pages_per) + 3
    perm = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
    kc, vc = _cache(total, nkv, bs, d, dtype)
    _stale(kc, vc, seed)              # stale data everywhere, as in pages that are used again
    width = max(pages_per)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    refs, start = [], 0
    for r, n in enumerate(lens):
        pages = perm[start:start + pages_per[r]]
        start += pages_per[r]
        table[r, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
        ks, kref = as_stored(rnd(n, nkv, d, seed=100 + 7 * r + seed), dtype)
        vs, vref = as_stored(rnd(n, nkv, d, seed=200 + 7 * r + seed), dtype)
        _fill_cache(kc, vc, ks, vs, pages, bs)
        refs.append((kref, vref))
    positions = list(range(lens[0] - portion, lens[0])) + [n - 1 for n in lens[1:]]
    entry = [0] * portion + list(range(1, len(lens)))

    class E:  # what build_items needs of an entry
        def __init__(self, first_row, count):
            self.first_row, self.count = first_row, count
    entries = [E(0, portion)] + [E(portion + i, 1) for i in range(len(lens) - 1)]
    group = nq // nkv
    numbered = list(enumerate(entries))                 # (row of the block table, entry)
    items = torch.tensor(M.build_items(numbered, M.tokens_per_item(group)), dtype=torch.int32, device=DEV)
    q, qref = as_stored(rnd(len(positions), (nq + 2 * nkv) * d, seed=300 + seed), dtype)
    out = torch.zeros(len(positions), nq * d, dtype=dtype, device=DEV)
    max_ctx = max(lens)
    live = None
    if made_for is not None:
        max_ctx, n = made_for
        split = ((max_ctx + n - 1) // n + 31) // 32 * 32
        live = torch.tensor([max(lens)], dtype=torch.int32, device=DEV) if planned is None else None
    if split is None or split == "portion" or portion_split:
        split_size, n_splits = M.choose_splits(items.numel() // M.ITEM_INTS, nkv, group, max_ctx)
    else:
        split_size, n_splits = split, (max_ctx + split - 1) // split
    rows = len(positions) * nq * n_splits
    part_o = torch.full((rows, d), float("nan"), device=DEV)
    part_ml = torch.full((rows, 2), float("nan"), device=DEV)
    scale = d ** -0.5
    pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)
    if split == "portion" or portion_split:
        # request 0's portion through the kernel that shares keys through LDS, the single tokens through the other
        big = torch.tensor(M.build_items(numbered[:1], M.portion_tokens(group, d)), dtype=torch.int32, device=DEV)
        if portion_split:
            n_big = (lens[0] + portion_split - 1) // portion_split
            big_o = torch.full((len(positions) * nq * n_big, d), float("nan"), device=DEV)
            big_ml = torch.full((len(positions) * nq * n_big, 2), float("nan"), device=DEV)
            M.attn_prefill(q, out, nq, nkv, d, kc, vc, pos_t, table.to(DEV), big, scale, window, portion_split, n_big,
                           big_o, big_ml)
        else:
            M.attn_prefill(q, out, nq, nkv, d, kc, vc, pos_t, table.to(DEV), big, scale, window)
        if len(entries) > 1:
            small = torch.tensor(M.build_items(numbered[1:], M.tokens_per_item(group)), dtype=torch.int32, device=DEV)
            M.attn_mfma(q, out, nq, nkv, d, kc, vc, pos_t, table.to(DEV), small, scale, window, split_size,
                        n_splits, max_ctx, part_o, part_ml)
    else:
        plan = None
        if planned is not None:
            n_items = items.numel() // M.ITEM_INTS
            plan = torch.full((M.plan_ints(n_items, n_splits),), -77, dtype=torch.int32, device=DEV)
            M.attn_plan(items, pos_t, n_splits, planned[0], planned[1], plan, d, min_keys=planned[2])
        M.attn_mfma(q, out, nq, nkv, d, kc, vc, pos_t, table.to(DEV), items, scale, window, split_size,
                    n_splits, max_ctx, part_o, part_ml, live_context=live, plan=plan)
    got = out.cpu().to(F64).reshape(-1, nq, d)
    for t, (p, e) in enumerate(zip(positions, entry)):
        kref, vref = refs[e]
        want = P.causal_attention(qref[t:t + 1, :nq * d].reshape(1, nq, d), kref[:p + 1], vref[:p + 1], scale,
                                  window or None, [p])
        assert torch.allclose(got[t], want[0], atol=2e-2, rtol=2e-2), (t, p, e, float((got[t] - want[0]).abs().max()))


@pytest.mark.parametrize("case", [
    dict(nq=4, nkv=2, d=16, bs=16, window=0, lens=[70, 131, 33], portion=9),
    dict(nq=6, nkv=1, d=32, bs=16, window=0, lens=[150, 1, 64, 65], portion=70),      # 6 heads: 8 columns a token
    dict(nq=6, nkv=3, d=48, bs=32, window=24, lens=[170, 90, 24, 25], portion=40),     # window, head size 48
    dict(nq=32, nkv=8, d=128, bs=16, window=0, lens=[300, 513, 512, 31], portion=37),
    dict(nq=8, nkv=2, d=64, bs=32, window=40, lens=[333, 64], portion=150),              # wide portions: window, 32-key pages
    dict(nq=2, nkv=2, d=32, bs=16, window=0, lens=[190, 17], portion=129),               # one head a kv head: 16 tokens a tile
    dict(nq=16, nkv=2, d=128, bs=64, window=0, lens=[257, 100], portion=257),            # a whole prompt from position 0
    dict(nq=3, nkv=3, d=80, bs=16, window=0, lens=[97, 40], portion=1),                # no grouping: 16 tokens an item
    dict(nq=40, nkv=2, d=64, bs=64, window=0, lens=[200, 77], portion=5),              # 20 heads a kv head: two chunks
    dict(nq=16, nkv=1, d=224, bs=16, window=100, lens=[260, 130], portion=18),
])
@pytest.mark.parametrize("split", [None, 32, 128, "portion"])
def test_attn_mfma(k, case, split):
    _mfma_case(k, split=split, **case)


@pytest.mark.parametrize("case", [
    dict(nq=32, nkv=8, d=128, bs=16, window=0, lens=[300, 513, 512, 31], portion=3),
    dict(nq=6, nkv=3, d=48, bs=32, window=24, lens=[170, 90, 24, 25], portion=1),
    dict(nq=8, nkv=2, d=64, bs=16, window=0, lens=[5, 1, 2], portion=1),                 # far fewer keys than splits of a block
])
@pytest.mark.parametrize("made_for", [(1024, 4), (4096, 7), (520, 2), (2048, 64)])
def test_attn_mfma_made_for_longer_contexts_than_the_step_has(k, case, made_for):
    """A launch shaped for a context bucket (its number of splits, its scratch) that is told the longest context of the
    step: the kernel and the merge cut the keys that are there into even splits, and both must agree on where."""
    _mfma_case(k, split=None, made_for=made_for, **case)


@pytest.mark.parametrize("case", [
    dict(nq=32, nkv=8, d=128, bs=16, window=0, lens=[300, 513, 512, 31], portion=3),
    dict(nq=6, nkv=3, d=48, bs=32, window=24, lens=[170, 90, 24, 25], portion=1),     # splits that lie below the window
    dict(nq=8, nkv=2, d=64, bs=16, window=0, lens=[5, 1, 2], portion=1),
    dict(nq=4, nkv=2, d=32, bs=16, window=0, lens=[1500, 40, 33, 900, 64, 65, 7], portion=1),
])
@pytest.mark.parametrize("planned", [(4, 2, 32), (9, 3, 64), (64, 32, 256), (1000, 1, 32)])
def test_attn_mfma_with_a_plan_of_the_step(k, case, planned):
    """The kernel for decoded tokens and short portions with a plan made on the device from the step's positions:
    every item cut into as many splits as its length asks for, the (item, split) pairs in the plan's order; items of
    one split are finished by their workgroup, the others by the merge (the scratch starts as NaN)."""
    _mfma_case(k, split=None, made_for=(2048, 6), planned=planned, **case)


def test_attn_plan_cuts_and_orders(k):
    """The plan itself against the rule it follows: the smallest split length T (whole blocks of 32, at least
    min_keys) with at most `slots` pairs in all, items cut evenly into min(n_splits, ceil(context / T)) splits, pairs
    by length, longest first (ties: the earlier pair), the second `first_wave` turned round."""
    from pulse_infer_amd.ops import attention_mfma as M
    gen = torch.Generator().manual_seed(3)
    for n_items, n_splits, slots, first, min_keys, hi in ((32, 8, 64, 32, 256, 2304), (5, 4, 7, 2, 32, 700), (48, 8, 64, 32, 256, 4096),
                                                         (128, 8, 64, 32, 256, 3000), (3, 6, 64, 32, 256, 90), (20, 8, 64, 32, 256, 8000),
                                                         (64, 16, 100, 8, 128, 50000)):
        ctx = torch.randint(1, hi + 1, (n_items,), generator=gen).tolist()
        rows = torch.randperm(n_items, generator=gen).tolist()            # items in another order than their rows
        positions = torch.zeros(n_items, dtype=torch.int32)
        items = []
        for i, r in enumerate(rows):
            positions[r] = ctx[i] - 1
            items.extend((r, 1, i, 0))
        items = torch.tensor(items, dtype=torch.int32, device=DEV)
        plan = torch.full((M.plan_ints(n_items, n_splits),), -77, dtype=torch.int32, device=DEV)
        M.attn_plan(items, positions.to(DEV), n_splits, slots, first, plan, 128, min_keys=min_keys)
        got = plan.cpu().tolist()
        count = lambda t: sum(min(n_splits, -(-c // t)) for c in ctx)
        top = (max(ctx) + 31) // 32 * 32
        T = next(t for t in range(min((min_keys + 31) // 32 * 32, top), top + 1, 32) if count(t) <= slots or t == top)
        sizes, pairs = [], []
        for i, c in enumerate(ctx):
            n = min(n_splits, -(-c // T))
            size = (-(-c // n) + 31) // 32 * 32
            sizes.append(size)
            pairs.extend((min(size, c - z * size), i * n_splits + z) for z in range(-(-c // size)))
        order = sorted(range(len(pairs)), key=lambda j: (-pairs[j][0], j))
        end = min(2 * first, len(order))
        order = order[:first] + order[first:end][::-1] + order[end:]
        assert got[0] == len(pairs)
        assert got[1:1 + len(pairs)] == [pairs[j][1] for j in order]
        assert got[1 + n_items * n_splits:] == sizes


@pytest.mark.parametrize("case", [
    dict(nq=32, nkv=8, d=128, bs=16, window=0, lens=[300, 513, 512, 31], portion=37),
    dict(nq=32, nkv=8, d=128, bs=16, window=0, lens=[700, 20], portion=700),             # a whole prompt: early items finish in split 0
    dict(nq=8, nkv=2, d=64, bs=32, window=40, lens=[333, 64], portion=150),              # splits that lie below the window
    dict(nq=2, nkv=2, d=32, bs=16, window=0, lens=[390, 17], portion=129),
    dict(nq=16, nkv=2, d=128, bs=64, window=0, lens=[257, 100], portion=257),
    dict(nq=12, nkv=2, d=64, bs=16, window=100, lens=[450], portion=260),                # 6 heads a kv head, a window over several splits
])
@pytest.mark.parametrize("size", [64, 128, 192, 1024])
def test_attn_prefill_with_its_keys_in_splits(k, case, size):
    """The prompt-portion kernel with the keys cut into splits (a workgroup a split, a second kernel merges): splits of
    one block, of several, and one that holds everything; the scratch starts as NaN, so nothing unwritten is read."""
    _mfma_case(k, split=None, portion_split=size, **case)


@pytest.mark.parametrize("n", [2048, 8192])
def test_attn_prefill_at_the_benchmark_shape(k, n):
    """A whole prompt of 2,048 (and 8,192) tokens at 32 query heads over 8 kv heads of 128 (every workgroup of the chip busy, items
    of every length, one diagonal block each): rows at the edges of items, of key blocks and of pages against the
    plain formula.  (The profile of this kernel is taken from this test.)"""
    from pulse_infer_amd.ops import attention_mfma as M
    nq, nkv, d, bs = 32, 8, 128, 16
    dtype = torch.bfloat16
    pages = n // bs
    perm = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(9)).tolist()[:pages]
    kc, vc = _cache(pages + 3, nkv, bs, d, dtype)
    _stale(kc, vc)
    ks, kref = as_stored(rnd(n, nkv, d, seed=501), dtype)
    vs, vref = as_stored(rnd(n, nkv, d, seed=502), dtype)
    _fill_cache(kc, vc, ks, vs, perm, bs)
    q, qref = as_stored(rnd(n, nq * d, seed=503), dtype)
    out = torch.zeros(n, nq * d, dtype=dtype, device=DEV)
    table = torch.tensor([perm], dtype=torch.int32, device=DEV)

    class E:
        def __init__(self, first_row, count):
            self.first_row, self.count, self.start = first_row, count, 0
    entries = [(0, E(0, n))]
    portion = M.portion_tokens(nq // nkv, d)
    items = torch.tensor(M.build_items(entries, portion), dtype=torch.int32, device=DEV)
    # a full chip is not cut, but for the last quarter of the walks of a long prompt, which get a second split
    split_size, n_splits = M.choose_prefill_splits(entries, portion, nkv, nq // nkv, d, 0)
    assert (split_size, n_splits) == ((0, 1) if n < 4096 else (3 * n // 4, 2))
    part_o = torch.full((n * nq * n_splits, d), float("nan"), device=DEV) if n_splits > 1 else None
    part_ml = torch.full((n * nq * n_splits, 2), float("nan"), device=DEV) if n_splits > 1 else None
    pos = torch.arange(n, dtype=torch.int32, device=DEV)
    for _ in range(3):
        M.attn_prefill(q, out, nq, nkv, d, kc, vc, pos, table, items, d ** -0.5, 0, split_size, n_splits, part_o, part_ml)
    got = out.cpu().to(F64).reshape(n, nq, d)
    for t in (0, 1, 15, 16, 31, 32, 33, 63, 64, 65, 127, 128, 1000, 1023, 1024, 1055, 1056, 2015, 2016, 2046, 2047,
              3 * n // 4 - 33, 3 * n // 4 - 1, 3 * n // 4, 3 * n // 4 + 1, 3 * n // 4 + 63, 3 * n // 4 + 64, n - 33, n - 32, n - 1):
        want = P.causal_attention(qref[t:t + 1].reshape(1, nq, d), kref[:t + 1], vref[:t + 1], d ** -0.5, None, [t])
        assert torch.allclose(got[t], want[0], atol=2e-2, rtol=2e-2), (t, float((got[t] - want[0]).abs().max()))


@pytest.mark.parametrize("path", ["decode", "decode_raw", "portion", "portion_splits"])
def test_attn_mfma_one_far_key_in_a_long_context(k, path):
    """A context of 20,000 keys (scattered pages, many splits) in which one key's score stands out: the output is that
    key's value wherever it lies (the first block, a page's edge, a split's edge, the far end), and not when a window
    excludes it.  Through the kernel for decoded tokens, the same from the raw projection output, and the kernel for
    prompt portions (its last 40 tokens)."""
    from pulse_infer_amd.ops import attention_mfma as M
    nq, nkv, d, bs, n = 8, 2, 128, 16, 20000
    dtype = torch.bfloat16
    pages = torch.randperm(n // bs + 1, generator=torch.Generator().manual_seed(8)).tolist()
    table = torch.tensor([pages], dtype=torch.int32, device=DEV)
    group = nq // nkv
    rows = 1 if not path.startswith("portion") else 40
    positions = list(range(n - rows, n))
    pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)

    class E:
        def __init__(self, first_row, count):
            self.first_row, self.count = first_row, count
    per = M.tokens_per_item(group) if not path.startswith("portion") else M.portion_tokens(group, d)
    items = torch.tensor(M.build_items([(0, E(0, rows))], per), dtype=torch.int32, device=DEV)
    split_size, n_splits = M.choose_splits(1, nkv, group, n)
    assert n_splits > 8
    part_o = torch.empty(rows * nq * n_splits, d, device=DEV)
    part_ml = torch.empty(rows * nq * n_splits, 2, device=DEV)
    kc, vc = _cache(len(pages), nkv, bs, d, dtype)
    ks, _ = as_stored(rnd(n, nkv, d, seed=50, scale=0.05), dtype)
    vs, vref = as_stored(rnd(n, nkv, d, seed=51), dtype)
    order = torch.tensor(pages, device=DEV)[torch.arange(n, device=DEV) // bs]          # page of every key
    slots = torch.arange(n, device=DEV) % bs
    kc[order, :, slots, :] = ks
    vc[order, :, :, slots] = vs
    spike = torch.zeros(nkv, d, dtype=dtype, device=DEV)
    spike[:, 0] = 40.0
    for target, window, seen in ((0, 0, True), (31, 0, True), (32, 0, True), (split_size - 1, 0, True),
                                 (split_size, 0, True), (bs * 700 - 1, 0, True), (n - 3000, 3000 + rows, True),
                                 (n - 3001 - rows, 3000, False), (n - rows - 1, 0, True)):
        page, slot = pages[target // bs], target % bs
        kept = kc[page, :, slot, :].clone()
        kc[page, :, slot, :] = spike
        qv = rnd(rows, (nq + 2 * nkv) * d, seed=52, scale=0.05)
        qv[:, 0:nq * d:d] = 40.0                                   # channel 0 of every query head
        qv[:, nq * d:] = 0                                          # (raw path) the tokens' own keys and values: nothing
        q, qref = as_stored(qv, dtype)
        out = torch.zeros(rows, nq * d, dtype=dtype, device=DEV)
        if path == "portion":
            M.attn_prefill(q, out, nq, nkv, d, kc, vc, pos_t, table, items, 1.0, window)
        elif path == "portion_splits":
            assert split_size % 64 == 0
            M.attn_prefill(q, out, nq, nkv, d, kc, vc, pos_t, table, items, 1.0, window, split_size, n_splits,
                           part_o, part_ml)
        elif path == "decode":
            M.attn_mfma(q, out, nq, nkv, d, kc, vc, pos_t, table, items, 1.0, window, split_size, n_splits, n,
                        part_o, part_ml)
        else:
            M.attn_decode(q, out, nq, nkv, d, kc, vc, pos_t, table, items, 1.0, window, split_size, n_splits, n,
                          part_o, part_ml, None, None, 0.0, None, None, 0, 0, False)
        got = out.cpu().to(F64).reshape(rows, nq, d)
        heads = torch.arange(nq) // group
        close = torch.allclose(got[-1], vref[target][heads], atol=2e-2)
        assert close == seen, (path, target, window)
        kc[page, :, slot, :] = kept


def test_attn_mfma_refuses_other_sizes(k):
    from pulse_infer_amd.ops import KernelError
    from pulse_infer_amd.ops import attention_mfma as M
    assert not M.supported(40, 16, torch.bfloat16, torch.bfloat16)       # head size no multiple of 16
    assert not M.supported(64, 8, torch.bfloat16, torch.bfloat16)        # pages shorter than a key tile
    assert not M.supported(64, 16, torch.float32, torch.float32)         # the 32-bit path has its own kernel
    assert not M.supported(256, 16, torch.bfloat16, torch.bfloat16)
    kc, vc = _cache(2, 1, 8, 64, torch.bfloat16)
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(KernelError, match="not supported"):
        M.attn_mfma(torch.zeros(1, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(1, 64, dtype=torch.bfloat16, device=DEV),
                    1, 1, 64, kc, vc, z, torch.zeros(1, 1, dtype=torch.int32, device=DEV),
                    torch.tensor([0, 1, 0, 0], dtype=torch.int32, device=DEV), 1.0, 0, 32, 1, 1, None, None)


@pytest.mark.parametrize("case", [
    dict(nq=32, nkv=8, d=128, rot=128, pairing="interleaved", norm=True, bs=16, window=0, lens=[300, 1, 513, 512, 33]),
    dict(nq=8, nkv=2, d=64, rot=64, pairing="half", norm=True, bs=32, window=40, lens=[333, 64, 40, 41]),
    dict(nq=6, nkv=3, d=48, rot=16, pairing="interleaved", norm=True, bs=16, window=0, lens=[170, 17, 16]),
    dict(nq=6, nkv=1, d=32, rot=0, pairing="interleaved", norm=False, bs=16, window=0, lens=[150, 2]),
    dict(nq=4, nkv=4, d=128, rot=64, pairing="half", norm=False, bs=64, window=0, lens=[97, 200]),
    dict(nq=16, nkv=1, d=224, rot=224, pairing="interleaved", norm=True, bs=16, window=100, lens=[260, 130]),
    dict(nq=40, nkv=2, d=64, rot=32, pairing="interleaved", norm=True, bs=64, window=0, lens=[200, 77, 64]),  # 20 heads a kv head: two chunks
])
@pytest.mark.parametrize("split", [None, 32, 128, "bucket", "planned", "planned_short"])
@pytest.mark.parametrize("new_key", [True, False])
@pytest.mark.parametrize("listed", [True, False])
def test_attn_decode_from_raw(k, case, split, new_key, listed):
    """Decoded tokens straight from the raw projection output: per-head norm, rotation, the token's own key and
    value (used from registers, written to the page) inside the attention kernel, against the plain formulas and
    against what the separate preparation kernel writes.  With new_key False the pages already hold the token.
    "bucket": the launch is made for contexts of up to 2,048 in five splits, as a recorded step's is, and told the
    longest context there is: the split that holds a token's position, whose workgroup writes its key, moves with it.
    "planned": the same launch with a plan made on the device from the positions (every item its own split size, the
    workgroups in the plan's order, items of one split finished without the merge); "planned_short": splits down to a
    block of keys, so that every item is cut as far as the launch allows.  ``listed`` False: no list of items is given,
    item i is token i with row i of the block table."""
    from pulse_infer_amd.ops import attention_mfma as M
    nq, nkv, d, rot, bs, window, lens = (case[x] for x in ("nq", "nkv", "d", "rot", "bs", "window", "lens"))
    pairing = 0 if case["pairing"] == "interleaved" else 1
    dtype, eps, theta, scale = torch.bfloat16, 3e-5, 9e3, d ** -0.5
    assert M.decode_takes(d, rot, pairing)
    n = len(lens)
    pages_per = [(c + bs - 1) // bs for c in lens]
    total = sum(pages_per) + 2
    perm = torch.randperm(total, generator=torch.Generator().manual_seed(5)).tolist()
    kc, vc = _cache(total, nkv, bs, d, dtype)
    _stale(kc, vc)                                 # stale data, also in the slot the new key goes to
    table = torch.full((n, max(pages_per)), -1, dtype=torch.int32)
    positions = [c - 1 for c in lens]
    qkv, ref = as_stored(rnd(n, (nq + 2 * nkv) * d + 8, seed=41), dtype)
    qw, qwref = as_stored(1 + 0.1 * rnd(d, seed=42), dtype)
    kw, kwref = as_stored(1 + 0.1 * rnd(d, seed=43), dtype)
    if not case["norm"]:
        qw = kw = None
    cos, sin = _tables(k, positions, theta, rot) if rot else (None, None)
    q = ref[:, :nq * d].reshape(n, nq, d)
    knew = ref[:, nq * d:(nq + nkv) * d].reshape(n, nkv, d)
    vnew = ref[:, (nq + nkv) * d:(nq + 2 * nkv) * d].reshape(n, nkv, d)
    if case["norm"]:
        q, knew = P.rms_norm(q, qwref, eps), P.rms_norm(knew, kwref, eps)
    if rot:
        q = P.rope(q, positions, theta, rot, case["pairing"])
        knew = P.rope(knew, positions, theta, rot, case["pairing"])
    knew = knew.to(dtype).to(F64)                  # keys are stored rounded
    refs, start = [], 0
    for r, c in enumerate(lens):
        pages = perm[start:start + pages_per[r]]
        start += pages_per[r]
        table[r, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
        ks, kref = as_stored(rnd(c, nkv, d, seed=100 + 7 * r), dtype)
        vs, vref = as_stored(rnd(c, nkv, d, seed=200 + 7 * r), dtype)
        kref[c - 1], vref[c - 1] = knew[r], vnew[r]
        if not new_key:                            # the pages already hold the token
            ks[c - 1], vs[c - 1] = knew[r].to(dtype), vnew[r].to(dtype)
        _fill_cache(kc, vc, ks[:c if not new_key else c - 1], vs[:c if not new_key else c - 1], pages, bs)
        refs.append((kref, vref))
    before_k, before_v = kc.clone(), vc.clone()

    class E:
        def __init__(self, first_row, count):
            self.first_row, self.count = first_row, count
    group = nq // nkv
    items = torch.tensor(M.build_items(list(enumerate(E(i, 1) for i in range(n))), M.tokens_per_item(group)),
                         dtype=torch.int32, device=DEV)
    max_ctx = max(lens)
    live = None
    if split is None:
        split_size, n_splits = M.choose_splits(n, nkv, group, max_ctx)
    elif split == "bucket":
        live = torch.tensor([max_ctx], dtype=torch.int32, device=DEV)
        max_ctx, n_splits = 2048, 5
        split_size = 416
    elif split in ("planned", "planned_short"):
        max_ctx, n_splits = 2048, 5
        split_size = 416
    else:
        split_size, n_splits = split, (max_ctx + split - 1) // split
    part_o = torch.full((n * nq * n_splits, d), float("nan"), device=DEV)
    part_ml = torch.full((n * nq * n_splits, 2), float("nan"), device=DEV)
    out = torch.zeros(n, nq * d, dtype=dtype, device=DEV)
    pos_t = torch.tensor(positions, dtype=torch.int32, device=DEV)
    plan = None
    if split in ("planned", "planned_short"):
        plan = torch.full((M.plan_ints(n, n_splits),), -77, dtype=torch.int32, device=DEV)
        slots = 2 * n if split == "planned" else 1000
        M.attn_plan(items if listed else None, pos_t, n_splits, slots, 2, plan, d, min_keys=64 if split == "planned" else 32)
        sizes = plan[1 + n * n_splits:].tolist()
        assert all(sz % 32 == 0 and sz * n_splits >= c for sz, c in zip(sizes, lens))
        if split == "planned_short":
            assert sizes == [max(32, ((c + n_splits - 1) // n_splits + 31) // 32 * 32) for c in lens]
    raw = qkv.clone()
    M.attn_decode(qkv, out, nq, nkv, d, kc, vc, pos_t, table.to(DEV), items if listed else None, scale, window,
                  split_size, n_splits, max_ctx, part_o, part_ml, qw, kw, eps, cos, sin, rot, pairing, new_key,
                  live_context=live, plan=plan)
    assert torch.equal(qkv, raw)                   # the projection output stays raw
    got = out.cpu().to(F64).reshape(n, nq, d)
    for t, p in enumerate(positions):
        kref, vref = refs[t]
        want = P.causal_attention(q[t:t + 1], kref[:p + 1], vref[:p + 1], scale, window or None, [p])
        assert torch.allclose(got[t], want[0], atol=2e-2, rtol=2e-2), (t, p, float((got[t] - want[0]).abs().max()))
    # the pages: the token's slot holds its key and value, nothing else has changed
    touched = torch.zeros(kc.shape[0], bs, dtype=torch.bool)
    kcpu, vcpu = kc.cpu().to(F64), vc.cpu().to(F64)
    for t, p in enumerate(positions):
        page, slot = int(table[t, p // bs]), p % bs
        touched[page, slot] = new_key
        assert torch.allclose(kcpu[page, :, slot, :], knew[t], atol=2e-2, rtol=2e-2)
        assert torch.equal(vcpu[page, :, :, slot], vnew[t])
    same = ~touched.unsqueeze(1).expand(-1, nkv, -1)
    assert torch.equal(_bits(kc)[same], _bits(before_k)[same])
    assert torch.equal(_bits(vc).transpose(2, 3)[same], _bits(before_v).transpose(2, 3)[same])
    if new_key:
        # the separate preparation kernel writes the same pages (up to the last bit of a sum in another order)
        k.qk_rope_kv(raw, nq, nkv, d, qw, kw, eps, cos, sin, rot, pairing, before_k, before_v, pos_t,
                     torch.arange(n, dtype=torch.int32, device=DEV), table.to(DEV))
        assert torch.allclose(kc.float(), before_k.float(), atol=0, rtol=2 ** -7, equal_nan=True)
        assert torch.equal(_bits(vc), _bits(before_v))


def test_attn_decode_refuses_rotations_it_cannot_prepare(k):
    from pulse_infer_amd.ops import attention_mfma as M
    assert M.decode_takes(128, 128, 0) and M.decode_takes(128, 64, 1) and M.decode_takes(64, 0, 0)
    assert not M.decode_takes(128, 12, 0)          # slices of 8 channels are rotated whole
    assert not M.decode_takes(128, 32, 1)          # the partner of a channel must lie in the same lane
    assert not M.decode_takes(64, 128, 0)


# ------------------------------------------------------------ few-rows product
@pytest.mark.parametrize("m", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("n,kk", [(48, 64), (509, 96), (4096 + 16, 200), (96, 4096)])
def test_gemm_skinny(k, m, n, kk):
    a, aref = as_stored(rnd(m, kk, seed=70), torch.bfloat16)
    w, wref = as_stored(rnd(n, kk, seed=71), torch.bfloat16)
    want = aref @ wref.T
    out32 = torch.empty(m, n, device=DEV)
    k.gemm_skinny(a, w, out32)
    assert torch.allclose(out32.cpu().to(F64), want, atol=2e-3 * math.sqrt(kk), rtol=1e-5)   # float32 sums of exact products
    out16 = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    k.gemm_skinny(a, w, out16)
    assert torch.equal(out16, out32.to(torch.bfloat16))                # the same sums, rounded once
    base = rnd(m, n, seed=72).to(DEV)
    acc = base.clone()
    k.gemm_skinny(a, w, acc, add=True)
    assert torch.allclose(acc, base + out32, atol=1e-6, rtol=1e-6)
    again = torch.empty(m, n, device=DEV)
    k.gemm_skinny(a, w, again)
    assert torch.equal(again, out32)                                   # the same from run to run
    if m > 1:                                                          # strided rows (a view into a wider buffer)
        wide = torch.zeros(m, kk + 24, dtype=torch.bfloat16, device=DEV)
        wide[:, :kk] = a
        k.gemm_skinny(wide[:, :kk], w, again)
        assert torch.equal(again, out32)


@pytest.mark.parametrize("m", [1, 2, 3, 4, 7, 8, 11, 16])
@pytest.mark.parametrize("n,kk", [(40, 2048), (509, 1024), (96, 3072), (33, 4096)])
def test_gemm_skinny_streaming_variants(k, m, n, kk):
    """Every variant of the streaming kernel (slabs, wavefronts, k-steps a load of X) against the general kernel
    and float64: a lane that fetched the wrong row or k-step would change the sums."""
    a, aref = as_stored(rnd(m, kk, seed=76), torch.bfloat16)
    w, wref = as_stored(rnd(n, kk, seed=77), torch.bfloat16)
    want = aref @ wref.T
    general = torch.empty(m, n, device=DEV)
    k.gemm_skinny(a, w, general, tune=9)
    assert torch.allclose(general.cpu().to(F64), want, atol=2e-3 * math.sqrt(kk), rtol=1e-5)
    ran = 0
    for slabs in (1, 2):
        for kw in (4, 8):
            if kk % (256 * kw):
                continue
            for p in (1, 2, 3, 4):
                if m > 16 >> (p - 1):
                    continue
                out = torch.full((m, n), float("nan"), device=DEV)
                k.gemm_skinny(a, w, out, tune=slabs * 100 + kw * 10 + p)
                if kw == 4:      # the same split of K as the general kernel: the same sums in the same order
                    assert torch.equal(out, general), (slabs, kw, p)
                else:
                    assert torch.allclose(out.cpu().to(F64), want, atol=2e-3 * math.sqrt(kk), rtol=1e-5), (slabs, kw, p)
                ran += 1
    assert ran >= 2
    auto = torch.empty(m, n, device=DEV)
    k.gemm_skinny(a, w, auto)
    assert torch.allclose(auto.cpu().to(F64), want, atol=2e-3 * math.sqrt(kk), rtol=1e-5)
    with pytest.raises(Exception, match="does not fit|unknown tuning"):
        k.gemm_skinny(a, w, auto, tune=184 if m > 2 else 777)


@pytest.mark.parametrize("m", [1, 3, 8, 13, 16])
@pytest.mark.parametrize("n,kk,swiglu", [(48, 1024, False), (4096 + 32, 2048, False), (96, 3072, True)])
def test_gemm_skinny_rounded_copy_and_rows_scaled_behind_the_product(k, m, n, kk, swiglu):
    """The norm moved behind the product: the product that adds into the residual leaves the new rows once more in
    bfloat16 with their sums of squares, and the next product, given those, multiplies row m of its result by
    1 / sqrt(mean(x_m^2) + eps) before it stores it or applies SwiGLU.  Against the formula in float64."""
    eps = 3e-6
    h = (rnd(m, kk, seed=90) * 3).to(DEV)
    a, _ = as_stored(rnd(m, 2048, seed=91), torch.bfloat16)
    wo, _ = as_stored(rnd(kk, 2048, seed=92, scale=2048 ** -0.5), torch.bfloat16)
    w, wref = as_stored(rnd(n, kk, seed=93, scale=kk ** -0.5), torch.bfloat16)
    sums = torch.full((m, kk // 16), float("nan"), device=DEV)
    rounded = torch.full((m + 1, kk), float("nan"), dtype=torch.bfloat16, device=DEV)
    plain = h.clone()
    k.gemm_skinny(a, wo, plain, add=True)
    k.gemm_skinny(a, wo, h, add=True, sumsq_out=sums, copy_out=rounded[:m])
    assert torch.equal(h, plain)
    assert torch.equal(rounded[:m], h.to(torch.bfloat16))
    assert bool(torch.isnan(rounded[m]).all())        # nothing beyond the rows
    # with column factors (the weight of the norm that reads h next): multiplied in before the one rounding
    cs, _ = as_stored(1 + 0.5 * rnd(kk, seed=94), torch.bfloat16)
    again, weighted = h.clone(), torch.empty(m, kk, dtype=torch.bfloat16, device=DEV)
    k.gemm_skinny(a, wo, again, add=True, copy_out=weighted, copy_scale=cs)
    assert torch.equal(weighted, (again * cs.float()).to(torch.bfloat16))
    again = None
    want_sums = (h.cpu().to(F64) ** 2).view(m, kk // 16, 16).sum(-1)
    assert torch.allclose(sums.cpu().to(F64), want_sums, rtol=1e-5, atol=1e-6)      # 16 columns a part
    # the mean comes from the float32 rows, the product from their rounded copy
    inv = 1.0 / torch.sqrt((h.cpu().to(F64) ** 2).mean(-1, keepdim=True) + eps)
    y = (rounded[:m].cpu().to(F64) @ wref.to(F64).t()) * inv
    if swiglu:
        g = y.view(m, -1, 2, 16)[:, :, 0].reshape(m, -1)
        u = y.view(m, -1, 2, 16)[:, :, 1].reshape(m, -1)
        want = g / (1 + torch.exp(-g)) * u
        got = torch.full((m, n // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
        k.gemm_skinny(rounded[:m], w, got, swiglu=True, row_scale=(sums, eps))
        err = (got.cpu().to(F64) - want).abs()
        assert bool((err <= 2.0 ** -8 * want.abs() + 1e-5 * math.sqrt(kk)).all())   # one rounding to bfloat16
    else:
        got = torch.full((m, n), float("nan"), device=DEV)
        k.gemm_skinny(rounded[:m], w, got, row_scale=(sums, eps))
        assert torch.allclose(got.cpu().to(F64), y, atol=1e-5 * math.sqrt(kk), rtol=1e-5)
        # no scale: the plain product, which the factor 1 / rms tells apart
        bare = torch.empty_like(got)
        k.gemm_skinny(rounded[:m], w, bare)
        assert torch.allclose(bare.cpu().to(F64), y / inv, atol=1e-5 * math.sqrt(kk), rtol=1e-5)
    from pulse_infer_amd.ops import KernelError
    with pytest.raises(KernelError, match="fused"):
        k.gemm_skinny(rounded[:m, :512].contiguous(), w[:, :512].contiguous(), got, swiglu=swiglu, row_scale=(sums, eps))
    # sums of squares in another split of the row (parts that are no multiple of four) give the same
    odd = torch.zeros(m, 7, device=DEV)
    odd[:, 2] = sums.sum(-1)
    again = torch.full_like(got, float("nan"))
    k.gemm_skinny(rounded[:m], w, again, swiglu=swiglu, row_scale=(odd, eps))
    assert float((again.float() - got.float()).abs().max()) <= 2.0 ** -7 * float(got.float().abs().max())


@pytest.mark.parametrize("m", [1, 8, 20, 32])
@pytest.mark.parametrize("inter,kk", [(32, 64), (224, 96), (176, 80), (12288 // 8, 256), (48, 2048), (176, 1024)])
def test_gemm_skinny_swiglu(k, m, inter, kk):
    a, aref = as_stored(rnd(m, kk, seed=73), torch.bfloat16)
    gate, gref = as_stored(rnd(inter, kk, seed=74, scale=kk ** -0.5), torch.bfloat16)
    up, uref = as_stored(rnd(inter, kk, seed=75, scale=kk ** -0.5), torch.bfloat16)
    mixed = torch.stack([gate.view(-1, 16, kk), up.view(-1, 16, kk)], dim=1).reshape(2 * inter, kk).contiguous()
    out = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    k.gemm_skinny(a, mixed, out, swiglu=True)
    want = P.silu(aref @ gref.T) * (aref @ uref.T)
    assert torch.allclose(out.cpu().to(F64), want, atol=1e-2, rtol=1e-2)
    # the unfused way over the same interleaved layout gives the same, up to the rounding of gate and up
    gu = torch.empty(m, 2 * inter, dtype=torch.bfloat16, device=DEV)
    k.gemm_skinny(a, mixed, gu)
    z = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    k.swiglu(gu, z, slab=16)
    assert torch.allclose(z.cpu().to(F64), want, atol=2e-2, rtol=2e-2)


def test_gemm_skinny_refuses(k):
    from pulse_infer_amd.ops import KernelError
    a = torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV)
    assert not k.gemm_skinny_ok(a, w) and k.gemm_skinny_ok(a[:64], w)
    assert not k.gemm_skinny_ok(a[:4, :60], w[:, :60])                 # K no multiple of 8
    assert not k.gemm_skinny_ok(a[:4].float(), w)
    with pytest.raises(KernelError, match="at most 64 rows"):
        k.gemm_skinny(a, w, torch.zeros(65, 32, device=DEV))
    with pytest.raises(KernelError, match="float32 target"):
        k.gemm_skinny(a[:4], w, torch.zeros(4, 32, dtype=torch.bfloat16, device=DEV), add=True)


@pytest.mark.parametrize("m", [1, 16, 17, 33, 48, 64, 65, 100, 128, 150, 192])
@pytest.mark.parametrize("n,kk", [(200, 128), (4096 + 16, 384), (96, 4096), (64, 1536)])
def test_gemm_mid(k, m, n, kk):
    """The product for 17 to 64 rows (X shared through LDS) at every workgroup shape, whole and in shares of the
    inner dimension, against float64: a wavefront that took another's weight rows, a piece of X staged to the wrong
    place or a chunk used before it had landed would change the sums."""
    a, aref = as_stored(rnd(m, kk, seed=90), torch.bfloat16)
    w, wref = as_stored(rnd(n, kk, seed=91), torch.bfloat16)
    want = aref @ wref.T
    first = None
    for waves in ((0, 2, 3, 4, 6) if m <= 64 else (0, 4, 6)):  # more than 64 rows: four or six wavefronts, chunks of 64
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
        k.gemm_mid(a, w, out, waves=waves)
        assert torch.allclose(out.cpu().to(F64), want, atol=3e-2 * math.sqrt(kk / 128), rtol=1e-2), waves
        first = out if first is None else first
        assert torch.equal(out, first)                      # the sums do not depend on the workgroup's shape
    for splits in (1, 2, 3, 4, 12):
        if not k.gemm_mid_takes(m, n, kk, splits):
            continue
        parts = torch.full((splits, m, n), float("nan"), device=DEV)
        k.gemm_mid(a, w, parts, splits=splits)
        share = kk // splits
        for s_ in range(splits):                            # every share is the product over its part of K
            part = aref[:, s_ * share:(s_ + 1) * share] @ wref[:, s_ * share:(s_ + 1) * share].T
            assert torch.allclose(parts[s_].cpu().to(F64), part, atol=2e-3 * math.sqrt(share), rtol=1e-5), (splits, s_)
        again = torch.empty_like(parts)
        k.gemm_mid(a, w, again, splits=splits, waves=2 if m <= 64 else 6)
        assert torch.equal(again, parts)
    if m > 1:                                                # strided rows (a view into a wider buffer)
        wide = torch.zeros(m, kk + 24, dtype=torch.bfloat16, device=DEV)
        wide[:, :kk] = a
        out = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
        k.gemm_mid(wide[:, :kk], w, out)
        assert torch.equal(out, first)


@pytest.mark.parametrize("m", [3, 17, 40, 64, 90, 192])
@pytest.mark.parametrize("inter,kk", [(48, 128), (1008, 256), (96, 2048)])
def test_gemm_mid_swiglu(k, m, inter, kk):
    a, aref = as_stored(rnd(m, kk, seed=93), torch.bfloat16)
    gate, gref = as_stored(rnd(inter, kk, seed=94, scale=kk ** -0.5), torch.bfloat16)
    up, uref = as_stored(rnd(inter, kk, seed=95, scale=kk ** -0.5), torch.bfloat16)
    mixed = torch.stack([gate.view(-1, 16, kk), up.view(-1, 16, kk)], dim=1).reshape(2 * inter, kk).contiguous()
    want = P.silu(aref @ gref.T) * (aref @ uref.T)
    for waves in ((0, 2, 4, 6) if m <= 64 else (0, 4, 6)):
        out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
        k.gemm_mid(a, mixed, out, swiglu=True, waves=waves)
        assert torch.allclose(out.cpu().to(F64), want, atol=1e-2, rtol=1e-2), waves


@pytest.mark.parametrize("m", [1, 17, 33, 48, 64])
@pytest.mark.parametrize("n,kk", [(16, 256), (80, 512), (528, 2304), (6144, 4096)])
def test_gemm_rows(k, m, n, kk):
    """The product for 17 to 64 rows of a weight with few rows (a workgroup owns whole slabs and all of K, its
    wavefronts share K out and meet in LDS), at every number of slabs a workgroup, against float64: stored as
    bfloat16; added into float32 with the new rows' sums of squares (16 columns a part) and the rounded, scaled copy;
    and with its rows scaled by 1 / sqrt(mean + eps) from the parts of their sums of squares.  A wavefront that took
    another's share of K, a chunk of X staged to the wrong place or partial sums met in another order would show."""
    a, aref = as_stored(rnd(m, kk, seed=190), torch.bfloat16)
    w, wref = as_stored(rnd(n, kk, seed=191, scale=kk ** -0.5), torch.bfloat16)
    want = aref @ wref.T
    first = None
    for slabs in (0, 1, 2, 4):
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
        k.gemm_rows(a, w, out, slabs=slabs)
        assert torch.allclose(out.cpu().to(F64), want, atol=2e-2, rtol=1e-2), slabs
        first = out if first is None else first
        assert torch.equal(out, first)                      # the sums do not depend on the workgroup's shape
    # rows scaled behind the product: the parts of the rows' sums of squares in, 1 / sqrt(mean + eps) times the row out
    eps = 1e-5
    for parts in (1, 6, 64):
        sumsq = (torch.rand(m + 2, parts, generator=torch.Generator().manual_seed(parts)) * kk / parts).to(DEV)
        rstd = 1.0 / torch.sqrt(sumsq.cpu().to(F64)[:m].sum(dim=1) / kk + eps)
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
        k.gemm_rows(a, w, out, row_scale=(sumsq, eps))
        assert torch.allclose(out.cpu().to(F64), want * rstd[:, None], atol=2e-2, rtol=1e-2), parts
    # added into float32, with what the next product needs to do without a norm kernel
    base = rnd(m, n, seed=192).to(DEV)
    scale, sref = as_stored(1 + 0.1 * rnd(n, seed=193), torch.bfloat16)
    for slabs in (1, 2, 4):
        res = base.clone()
        sums = torch.full((m + 1, n // 16), float("nan"), device=DEV)
        copy = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
        k.gemm_rows(a, w, res, add=True, sumsq_out=sums, copy_out=copy, copy_scale=scale, slabs=slabs)
        new = base.cpu().to(F64) + want
        got = res.cpu().to(F64)
        assert torch.allclose(got, new, atol=1e-3, rtol=1e-5)
        assert torch.allclose(sums[:m].cpu().to(F64), (got ** 2).view(m, n // 16, 16).sum(dim=2), rtol=1e-5, atol=1e-6)
        assert bool(torch.isnan(sums[m]).all())                                     # nothing beyond the rows
        assert torch.equal(copy.cpu(), (res.cpu() * scale.cpu().float()).to(torch.bfloat16))   # one rounding of the float32 product
    plain = base.clone()
    k.gemm_rows(a, w, plain, add=True)
    assert torch.equal(plain, res)
    if m > 1:                                                # strided rows (views into wider buffers)
        wide = torch.zeros(m, kk + 24, dtype=torch.bfloat16, device=DEV)
        wide[:, :kk] = a
        out = torch.zeros(m, n + 8, dtype=torch.bfloat16, device=DEV)
        k.gemm_rows(wide[:, :kk], w, out[:, :n])
        assert torch.equal(out[:, :n], first) and bool((out[:, n:] == 0).all())


def test_gemm_rows_refuses(k):
    from pulse_infer_amd.ops import KernelError
    a = torch.zeros(65, 256, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 256, dtype=torch.bfloat16, device=DEV)
    assert k.gemm_rows_takes(64, 64, 256) and not k.gemm_rows_takes(65, 64, 256)
    assert not k.gemm_rows_takes(8, 72, 256) and not k.gemm_rows_takes(8, 64, 384)
    with pytest.raises(KernelError, match="not a shape"):
        k.gemm_rows(a, w, torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError, match="float32 target"):
        k.gemm_rows(a[:8], w, torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV), add=True)
    with pytest.raises(KernelError, match="come with add"):
        k.gemm_rows(a[:8], w, torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV), sumsq_out=torch.zeros(8, 4, device=DEV))
    with pytest.raises(KernelError, match="slabs"):
        k.gemm_rows(a[:8], w, torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV), slabs=3)


@pytest.mark.parametrize("m,n,kk", [(1, 32, 64), (256, 256, 64), (300, 520, 192), (257, 1056, 4160), (2048, 2304, 512),
                                    (2500, 264, 128)])
def test_gemm_tile(k, m, n, kk):
    """The product for many rows (output tiles of 256 x 256, four wavefronts, K in steps of 64 through two LDS stages
    filled straight from memory) against float64: bfloat16 results, float32 results of 1, 2 and 4 shares of K, rows
    that are views into wider buffers; tiles that hang over both edges, a single step of K and one more than the
    stages, panels of eight and of fewer tiles.  A piece of a row copied to another place than the operand reads look
    for it in, a quarter of the tile or a k group swapped, a stage read before its copies had landed or overwritten
    before its last read: all of them change results by their own size."""
    a, aref = as_stored(rnd(m, kk, seed=201), torch.bfloat16)
    w, wref = as_stored(rnd(n, kk, seed=202, scale=kk ** -0.5), torch.bfloat16)
    want = aref @ wref.T
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    k.gemm_tile(a, w, out)
    assert torch.allclose(out.cpu().to(F64), want, atol=2e-2, rtol=1e-2)
    again = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    k.gemm_tile(a, w, again)
    assert torch.equal(out, again)
    for splits in (1, 2, 4):
        if kk % (64 * splits):
            continue
        parts = torch.full((splits, m + 1, n), float("nan"), device=DEV)[:, :m]
        k.gemm_tile(a, w, parts)
        total = parts.cpu().to(F64).sum(dim=0)
        assert torch.allclose(total, want, atol=1e-4, rtol=1e-5), splits
        if splits == 1:
            assert torch.equal(parts[0].to(torch.bfloat16), out)      # the same sums, rounded once
            flat = torch.full((m, n), float("nan"), device=DEV)
            k.gemm_tile(a, w, flat)
            assert torch.equal(flat, parts[0])
    wide = torch.zeros(m, kk + 24, dtype=torch.bfloat16, device=DEV)
    wide[:, :kk] = a
    padded = torch.zeros(m, n + 8, dtype=torch.bfloat16, device=DEV)
    k.gemm_tile(wide[:, :kk], w, padded[:, :n])
    assert torch.equal(padded[:, :n], out) and bool((padded[:, n:] == 0).all())


@pytest.mark.parametrize("m,inter,kk", [(256, 128, 64), (700, 1008, 256), (1030, 2064, 1088)])
def test_gemm_tile_swiglu(k, m, inter, kk):
    """SwiGLU on the way out of the many-rows product, gate and up rows in alternating slabs of 16 (a tile's last
    pair of slabs included), against float64 and against the product followed by the SwiGLU kernel."""
    a, aref = as_stored(rnd(m, kk, seed=203), torch.bfloat16)
    gate, gref = as_stored(rnd(inter, kk, seed=204, scale=kk ** -0.5), torch.bfloat16)
    up, uref = as_stored(rnd(inter, kk, seed=205, scale=kk ** -0.5), torch.bfloat16)
    mixed = torch.stack([gate.view(-1, 16, kk), up.view(-1, 16, kk)], dim=1).reshape(2 * inter, kk).contiguous()
    want = P.silu(aref @ gref.T) * (aref @ uref.T)
    out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    k.gemm_tile(a, mixed, out, swiglu=True)
    assert torch.allclose(out.cpu().to(F64), want, atol=1e-2, rtol=1e-2)
    gu = torch.empty(m, 2 * inter, dtype=torch.bfloat16, device=DEV)
    k.gemm_tile(a, mixed, gu)
    z = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    k.swiglu(gu, z, slab=16)                                  # (this one rounds gate and up before it multiplies)
    assert torch.allclose(out.float(), z.float(), atol=1e-2, rtol=2e-2)


def test_gemm_tile_at_the_benchmark_shape(k):
    """gate and up of the benchmark's layer for a prompt of 2,048 tokens (768 tiles, three for every compute unit,
    64 steps of K each): SwiGLU inside against the float32 product of the same rounded operands followed by the
    formula, the bfloat16 product against the library's, and o's shape in two shares of K."""
    m, inter, kk = 2048, 12288, 4096
    a = rnd(m, kk, seed=206).to(torch.bfloat16).to(DEV)
    mixed = rnd(2 * inter, kk, seed=207, scale=kk ** -0.5).to(torch.bfloat16).to(DEV)
    ref = a.float() @ mixed.float().T                          # float32 on the device (no reduced-precision mode)
    slabs = ref.view(m, inter // 16, 2, 16)
    want = (torch.nn.functional.silu(slabs[:, :, 0]) * slabs[:, :, 1]).reshape(m, inter)
    out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    k.gemm_tile(a, mixed, out, swiglu=True)
    assert torch.allclose(out.float(), want, atol=1e-2, rtol=1e-2)
    plain = torch.full((m, 2 * inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    k.gemm_tile(a, mixed, plain)
    assert torch.allclose(plain.float(), ref, atol=2e-2, rtol=1e-2)
    library = torch.matmul(a, mixed.t())
    assert torch.allclose(plain.float(), library.float(), atol=2e-2, rtol=2e-2)
    del ref, slabs, want, out, plain, library
    w_o = mixed[:4096]
    parts = torch.full((2, m, 4096), float("nan"), device=DEV)
    k.gemm_tile(a, w_o, parts)
    assert torch.allclose(parts.sum(dim=0), a.float() @ w_o.float().T, atol=1e-3, rtol=1e-4)
    half = kk // 2
    assert torch.allclose(parts[1], a[:, half:].float() @ w_o[:, half:].float().T, atol=1e-3, rtol=1e-4)


def test_gemm_tile_refuses(k):
    from pulse_infer_amd.ops import KernelError
    a = torch.zeros(300, 192, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 192, dtype=torch.bfloat16, device=DEV)
    assert k.gemm_tile_takes(300, 64, 192) and not k.gemm_tile_takes(300, 64, 96) and not k.gemm_tile_takes(300, 60, 192)
    assert k.gemm_tile_takes(300, 64, 192, swiglu=True) and not k.gemm_tile_takes(300, 48, 192, swiglu=True)
    assert k.gemm_tile_takes(300, 60, 192, splits=3, float32=True) and not k.gemm_tile_takes(300, 64, 192, splits=2, float32=True)
    assert not k.gemm_tile_takes(300, 64, 192, splits=3)
    with pytest.raises(KernelError, match="not a shape"):
        k.gemm_tile(a[:, :96].contiguous(), w[:, :96].contiguous(), torch.zeros(300, 64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError, match="not a shape"):
        k.gemm_tile(a, w, torch.zeros(2, 300, 64, device=DEV))
    with pytest.raises(KernelError, match=r"out must be bfloat16 \[300, 32\]"):
        k.gemm_tile(a, w, torch.zeros(300, 64, dtype=torch.bfloat16, device=DEV), swiglu=True)
    with pytest.raises(KernelError, match="inner sizes"):
        k.gemm_tile(a, w[:, :128].contiguous(), torch.zeros(300, 64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError, match="float32 results go to"):
        k.gemm_tile(a, w, torch.zeros(3, 300, 32, device=DEV))


def test_gemm_mid_refuses(k):
    from pulse_infer_amd.ops import KernelError
    a = torch.zeros(193, 256, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 256, dtype=torch.bfloat16, device=DEV)
    assert k.gemm_mid_takes(192, 64, 256) and not k.gemm_mid_takes(193, 64, 256)
    assert not k.gemm_mid_takes(8, 64, 192) and not k.gemm_mid_takes(8, 64, 256, 3) and k.gemm_mid_takes(8, 64, 256, 2)
    with pytest.raises(KernelError, match="not a shape"):
        k.gemm_mid(a, w, torch.zeros(193, 64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError, match="4 or 6 wavefronts"):
        k.gemm_mid(a[:100], w, torch.zeros(100, 64, dtype=torch.bfloat16, device=DEV), waves=2)
    with pytest.raises(KernelError, match="partial sums"):
        k.gemm_mid(a[:8], w, torch.zeros(8, 64, device=DEV), splits=2)
    with pytest.raises(KernelError, match="bfloat16"):
        k.gemm_mid(a[:8], w, torch.zeros(8, 64, dtype=torch.bfloat16, device=DEV), splits=2)
    with pytest.raises(KernelError, match="wavefronts"):
        k.gemm_mid(a[:8], w, torch.zeros(8, 32, dtype=torch.bfloat16, device=DEV), swiglu=True, waves=3)


@pytest.mark.parametrize("hidden", [48, 4096])
def test_an_update_in_parts_is_added_in_order(k, hidden):
    """h + the parts of an update (the shares of a product whose inner dimension was split), in the norm's kernel
    and in the plain addition, with and without gathered rows."""
    rows, parts, eps = 20, 5, 1e-5
    h0 = rnd(rows, hidden, seed=96).to(DEV)
    delta = rnd(parts, rows, hidden, seed=97).to(DEV)
    w, wref = as_stored(1 + 0.1 * rnd(hidden, seed=98), torch.bfloat16)
    total = h0.clone()
    for p_ in range(parts):
        total += delta[p_]                                  # float32, in order: the kernel's own sums
    h = h0.clone()
    out = torch.empty(rows, hidden, dtype=torch.bfloat16, device=DEV)
    k.add_rmsnorm(h, delta, w, eps, out)
    assert torch.equal(h, total)
    assert torch.allclose(out.cpu().to(F64), P.rms_norm(total.cpu().to(F64), wref, eps), **tol(torch.bfloat16))
    pick = torch.tensor([19, 0, 7], dtype=torch.int32, device=DEV)
    h = h0.clone()
    some = torch.empty(3, hidden, dtype=torch.bfloat16, device=DEV)
    k.add_rmsnorm(h, delta, w, eps, some, rows=pick)
    assert torch.equal(h, h0) and torch.equal(some, out[pick.long()])
    h = h0.clone()
    k.residual_add(h, delta)
    assert torch.equal(h, total)


def test_two_stage_argmax(k):
    for rows, vocab in ((1, 5), (3, 2048), (8, 151936), (5, 4097)):
        logits = rnd(rows, vocab, seed=80 + rows).to(DEV)
        logits[0, vocab - 1] = logits[0, 0] = 99.0                       # equal maxima far apart: the lowest index wins
        if rows > 1:
            logits[1, vocab // 2] = float("nan")
        chunks = k.argmax_chunks(vocab)
        out = torch.empty(rows, dtype=torch.int32, device=DEV)
        k.argmax(logits, out, torch.empty(rows * chunks, device=DEV), torch.empty(rows * chunks, dtype=torch.int32, device=DEV))
        want = torch.argmax(torch.nan_to_num(logits.cpu(), nan=-1e30), dim=1).tolist()
        want[0] = 0
        assert out.tolist() == want
        single = torch.empty(rows, dtype=torch.int32, device=DEV)
        k.sample(logits, single)
        assert single.tolist() == want
