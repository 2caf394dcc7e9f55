"""GPU checks at the largest element counts the C ABI accepts: 2^32 - 1 for the dense
operators, 2^31 - 1 (int32 indices on the wire) for the sparse ones.  The CPU oracle would
take minutes and tens of GiB at these sizes, so the results are checked on the GPU with
plain torch arithmetic against what the operators' definitions fix element by element:
codes, residuals, decoded values, the sampled threshold, the selected set.  What these sizes
add to the other tests is index arithmetic beyond 2^31 and launches of a million tiles."""
import pytest
import torch

pytestmark = pytest.mark.gpu

CHUNK = 1 << 28


@pytest.fixture(scope="module")
def hp():
    import hipress_amd

    assert torch.cuda.is_available()
    hipress_amd._lib.lib()
    return hipress_amd


def _need(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * (1 << 30):
        pytest.skip(f"needs {gib} GiB of free device memory")


def _normal(n, std, seed):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    t = torch.empty(n, dtype=torch.float32, device="cuda")
    for lo in range(0, n, CHUNK):
        t[lo:lo + CHUNK].normal_(0.0, std, generator=gen)
    return t


def _chunks(n):
    for lo in range(0, n, CHUNK):
        yield lo, min(n, lo + CHUNK)


def _codes2(words, lo, hi):
    """2-bit codes of elements [lo, hi) from the packed words (code i in bits 2*(i%16) of word i/16);
    lo is a multiple of 16."""
    w = words[lo // 16:(hi + 15) // 16].to(torch.int64) & 0xFFFFFFFF
    sh = torch.arange(16, device=w.device, dtype=torch.int64) * 2
    return ((w[:, None] >> sh[None, :]) & 3).reshape(-1)[:hi - lo]


def _check_selection(v, acc, comp, n, ratio, cap):
    """comp holds what sampled-threshold selection at `ratio` sends of v (n elements), acc what it leaves
    behind; returns the indices sent."""
    head = comp[:16].view(torch.int32)
    nnz = head[0].item()
    assert head[1].item() == n and head[2].item() == cap and 0 < nnz <= cap
    # the threshold is the ks-th largest magnitude among the samples at 100 q + 50
    ns = n // 100
    ks = -(-ns // round(1 / ratio))  # ceil(ratio * ns)
    kth = torch.kthvalue(v[50::100][:ns].abs(), ns - ks + 1).values
    thr = comp[12:16].view(torch.float32)[0]
    assert thr.item() == kth.item()
    # everything at or above it (and nonzero) is sent, in index order, and leaves the accumulator
    idx = comp[16:16 + 4 * nnz].view(torch.int32)
    val = comp[16 + 4 * cap:16 + 4 * cap + 4 * nnz].view(torch.float32)
    sent = []
    for lo, hi in _chunks(n):
        x = v[lo:hi]
        sel = (x.abs() >= thr) & (x != 0)
        sent.append(torch.nonzero(sel).view(-1) + lo)
        assert torch.equal(acc[lo:hi], torch.where(sel, torch.zeros_like(x), x)), f"accumulator differs in [{lo}, {hi})"
    sent = torch.cat(sent)
    assert sent.numel() == nnz
    assert torch.equal(idx.to(torch.int64), sent)
    assert torch.equal(val, v[sent])
    return sent


def test_tbq_at_the_largest_element_count(hp):
    n = (1 << 32) - 1
    _need(80)
    tau = 0.05
    g = _normal(n, 0.05, 1)
    r = _normal(n, 0.01, 2)
    v = torch.empty_like(g)
    for lo, hi in _chunks(n):
        torch.add(r[lo:hi], g[lo:hi], out=v[lo:hi])
    comp = torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")
    hp.tbq_encode(g, r, comp, tau)
    out = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
    hp.tbq_decode(comp, out)
    torch.cuda.synchronize()
    head = comp[:16].view(torch.int32)
    assert head[0].item() == torch.tensor(tau, dtype=torch.float32).view(torch.int32).item()
    assert head[1].item() & 0xFFFFFFFF == n
    words = comp[16:].view(torch.int32)
    assert words.numel() == (n + 15) // 16
    t = torch.tensor(tau, dtype=torch.float32, device="cuda")
    for lo, hi in _chunks(n):
        x = v[lo:hi]
        pos, neg = x >= t, x <= -t
        code = pos.to(torch.int64) + 2 * neg.to(torch.int64)
        assert torch.equal(_codes2(words, lo, hi), code), f"codes differ in [{lo}, {hi})"
        keep = torch.where(pos, x - t, torch.where(neg, x + t, x))
        assert torch.equal(r[lo:hi].view(torch.int32), keep.view(torch.int32)), f"residual differs in [{lo}, {hi})"
        dec = torch.where(pos, t, torch.where(neg, -t, torch.zeros_like(x)))
        assert torch.equal(out[lo:hi], dec), f"decoded values differ in [{lo}, {hi})"
    # n mod 16 = 15: the last word's top code is padding
    assert (words[-1].item() >> 30) & 3 == 0


def test_onebit_at_the_largest_element_count(hp):
    n = (1 << 32) - 1
    _need(80)
    g = _normal(n, 0.02, 3)
    r = _normal(n, 0.005, 4)
    v = torch.empty_like(g)
    total = 0.0
    for lo, hi in _chunks(n):
        torch.add(r[lo:hi], g[lo:hi], out=v[lo:hi])
        total += v[lo:hi].abs().sum(dtype=torch.float64).item()
    comp = torch.zeros(hp.onebit_payload_bytes(n), dtype=torch.uint8, device="cuda")
    hp.onebit_encode(g, r, comp)
    out = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
    hp.onebit_decode(comp, out)
    torch.cuda.synchronize()
    head = comp[:16].view(torch.int32)
    s = comp[:4].view(torch.float32)[0]
    assert abs(s.item() - total / n) <= 1e-6 * (total / n)
    assert head[1].item() & 0xFFFFFFFF == n
    words = comp[16:].view(torch.int32)
    assert words.numel() == (n + 31) // 32
    sh = torch.arange(32, device="cuda", dtype=torch.int64)
    for lo, hi in _chunks(n):
        x = v[lo:hi]
        pos = x >= 0
        w = words[lo // 32:(hi + 31) // 32].to(torch.int64) & 0xFFFFFFFF
        bits = ((w[:, None] >> sh[None, :]) & 1).reshape(-1)[:hi - lo]
        assert torch.equal(bits, pos.to(torch.int64)), f"sign bits differ in [{lo}, {hi})"
        d = torch.where(pos, s, -s)
        assert torch.equal(r[lo:hi].view(torch.int32), (x - d).view(torch.int32)), f"residual differs in [{lo}, {hi})"
        assert torch.equal(out[lo:hi], d), f"decoded values differ in [{lo}, {hi})"
    assert (words[-1].item() >> 31) & 1 == 0  # n mod 32 = 31: one bit of padding


def test_graddrop_at_the_largest_element_count(hp):
    n = (1 << 31) - 1
    _need(60)
    ratio = 0.001
    g = _normal(n, 1e-3, 5)
    acc = _normal(n, 2e-4, 6)
    v = torch.empty_like(g)
    for lo, hi in _chunks(n):
        torch.add(acc[lo:hi], g[lo:hi], out=v[lo:hi])
    comp = torch.zeros(hp.sparse_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")
    hp.graddrop_encode(g, acc, comp, ratio)
    out = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
    hp.graddrop_decode(comp, out)
    torch.cuda.synchronize()
    sent = _check_selection(v, acc, comp, n, ratio, hp.sparse_capacity(n, ratio))
    for lo, hi in _chunks(n):
        x = v[lo:hi]
        mask = torch.zeros(hi - lo, dtype=torch.bool, device="cuda")
        mask[sent[(sent >= lo) & (sent < hi)] - lo] = True
        assert torch.equal(out[lo:hi], torch.where(mask, x, torch.zeros_like(x))), f"decoded values differ in [{lo}, {hi})"
    assert sent[-1].item() > (1 << 31) - 1 - 10_000_000  # the top of the index range is in use


def test_terngrad_at_the_largest_element_count(hp):
    n = (1 << 32) - 1
    _need(80)
    bucket = 512
    g = _normal(n, 1e-3, 7)
    u = torch.empty(n, dtype=torch.float32, device="cuda")
    gen = torch.Generator(device="cuda")
    gen.manual_seed(8)
    for lo, hi in _chunks(n):
        # 24 random bits / 2^24: strictly below one
        u[lo:hi] = torch.randint(0, 1 << 24, (hi - lo,), device="cuda", generator=gen, dtype=torch.int32).to(torch.float32) / 16777216.0
    comp = torch.zeros(hp.terngrad_payload_bytes(n, bucket), dtype=torch.uint8, device="cuda")
    hp.terngrad_encode(g, u, comp, bucket)
    out = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
    hp.terngrad_decode(comp, out)
    torch.cuda.synchronize()
    head = comp[:16].view(torch.int32)
    assert head[0].item() & 0xFFFFFFFF == n and head[1].item() == bucket
    nb = (n + bucket - 1) // bucket
    sbytes = (4 * nb + 15) // 16 * 16
    scale = comp[16:16 + 4 * nb].view(torch.float32)
    words = comp[16 + sbytes:].view(torch.int32)
    assert words.numel() == (n + 15) // 16
    for lo, hi in _chunks(n):  # CHUNK is a multiple of the bucket
        x, uu = g[lo:hi], u[lo:hi]
        a = x.abs()
        full = (hi - lo) // bucket * bucket
        s = a[:full].view(-1, bucket).amax(dim=1)
        if full < hi - lo:
            s = torch.cat([s, a[full:].amax().view(1)])
        assert torch.equal(scale[lo // bucket:lo // bucket + s.numel()], s), f"bucket scales differ in [{lo}, {hi})"
        se = s.repeat_interleave(bucket)[:hi - lo]
        keep = uu * se < a
        code = torch.where(keep, torch.where(x < 0, 2, 1), 0).to(torch.int64)
        assert torch.equal(_codes2(words, lo, hi), code), f"codes differ in [{lo}, {hi})"
        dec = torch.where(keep, torch.where(x < 0, -se, se), torch.zeros_like(x))
        assert torch.equal(out[lo:hi], dec), f"decoded values differ in [{lo}, {hi})"
    assert (words[-1].item() >> 30) & 3 == 0


def test_dgc_at_the_largest_element_count(hp):
    n = (1 << 31) - 1
    _need(80)
    ratio, mf = 0.001, 0.9
    g = _normal(n, 1e-3, 9)
    mom = _normal(n, 5e-4, 10)
    acc = _normal(n, 2e-4, 11)
    mm = torch.empty_like(g)  # fl(fl(mf * m) + g)
    v = torch.empty_like(g)   # acc + mm
    f = torch.tensor(mf, dtype=torch.float32, device="cuda")
    for lo, hi in _chunks(n):
        torch.mul(mom[lo:hi], f, out=mm[lo:hi])
        mm[lo:hi] += g[lo:hi]
        torch.add(acc[lo:hi], mm[lo:hi], out=v[lo:hi])
    comp = torch.zeros(hp.sparse_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")
    hp.dgc_encode(g, mom, acc, comp, mf, ratio)
    torch.cuda.synchronize()
    sent = _check_selection(v, acc, comp, n, ratio, hp.sparse_capacity(n, ratio))
    for lo, hi in _chunks(n):
        mask = torch.zeros(hi - lo, dtype=torch.bool, device="cuda")
        mask[sent[(sent >= lo) & (sent < hi)] - lo] = True
        assert torch.equal(mom[lo:hi], torch.where(mask, torch.zeros_like(mm[lo:hi]), mm[lo:hi])), f"momentum differs in [{lo}, {hi})"


def test_minmax_quantiser_at_the_largest_element_count(hp):
    n = (1 << 32) - 1
    _need(80)
    b = 2
    g = _normal(n, 1e-3, 12)
    u = torch.empty(n, dtype=torch.float32, device="cuda")
    gen = torch.Generator(device="cuda")
    gen.manual_seed(13)
    for lo, hi in _chunks(n):
        u[lo:hi] = torch.randint(0, 1 << 24, (hi - lo,), device="cuda", generator=gen, dtype=torch.int32).to(torch.float32) / 16777216.0
    comp = torch.zeros(hp.compll_payload_bytes(n, b), dtype=torch.uint8, device="cuda")
    hp.compll_terngrad_encode(g, u, comp, b)
    out = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
    hp.compll_terngrad_decode(comp, out)
    torch.cuda.synchronize()
    assert comp[0].item() == b and comp[1].item() == n % 4
    mn = comp[2:6].clone().view(torch.float32)[0]
    mx = comp[6:10].clone().view(torch.float32)[0]
    lo_ref = min(g[lo:hi].min().item() for lo, hi in _chunks(n))
    hi_ref = max(g[lo:hi].max().item() for lo, hi in _chunks(n))
    assert mn.item() == lo_ref and mx.item() == hi_ref
    gap = (mx - mn) / 3.0
    count = hp.compll_decoded_count(n, b)
    assert count == n - 2
    codes = comp[10:]
    assert codes.numel() == (n * b + 7) // 8
    sh = torch.arange(4, device="cuda", dtype=torch.int64) * 2
    for lo, hi in _chunks(n):  # CHUNK is a multiple of 4
        x = g[lo:hi]
        c = torch.floor((x - mn) / gap + u[lo:hi]).clamp_(0.0, 3.0).to(torch.int64)
        pad = (-(hi - lo)) % 4
        if pad:
            c = torch.cat([c, torch.zeros(pad, dtype=torch.int64, device="cuda")])
        byte = (c.view(-1, 4) << sh[None, :]).sum(dim=1).to(torch.uint8)
        assert torch.equal(codes[lo // 4:lo // 4 + byte.numel()], byte), f"code bytes differ in [{lo}, {hi})"
        top = min(hi, count)
        dec = c[:top - lo].to(torch.float32) * gap + mn
        assert torch.equal(out[lo:top], dec), f"decoded values differ in [{lo}, {top})"
    assert torch.all(out[count:] == 7.0)  # the reference's count stops two short of n here


def test_tbq_decode_merge_at_the_largest_element_count(hp):
    n = (1 << 32) - 1
    _need(90)
    taus = [0.05, 0.04, 0.06]
    g = torch.empty(n, dtype=torch.float32, device="cuda")
    r = torch.empty(n, dtype=torch.float32, device="cuda")
    comps = []
    gen = torch.Generator(device="cuda")
    for p, tau in enumerate(taus):
        gen.manual_seed(20 + p)
        for lo, hi in _chunks(n):
            g[lo:hi].normal_(0.0, 0.05, generator=gen)
        r.zero_()
        c = torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")
        hp.tbq_encode(g, r, c, tau)
        comps.append(c)
    agg = g.fill_(7.0)           # the merge overwrites it
    res = r                      # the aggregator's residual
    gen.manual_seed(30)
    for lo, hi in _chunks(n):
        res[lo:hi].normal_(0.0, 0.02, generator=gen)
    before = res.clone()
    tau_out = 0.05
    outc = torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")
    hp.tbq_decode_merge(comps, agg, res, outc, tau_out)
    torch.cuda.synchronize()
    words = [c[16:].view(torch.int32) for c in comps]
    out_words = outc[16:].view(torch.int32)
    t = torch.tensor(tau_out, dtype=torch.float32, device="cuda")
    for lo, hi in _chunks(n):
        e = torch.zeros(hi - lo, dtype=torch.float32, device="cuda")
        for w, tau in zip(words, taus):
            c = _codes2(w, lo, hi)
            tp = torch.tensor(tau, dtype=torch.float32, device="cuda")
            e = e + torch.where(c == 1, tp, torch.where(c == 2, -tp, torch.zeros_like(e)))
        assert torch.equal(agg[lo:hi], e), f"aggregate differs in [{lo}, {hi})"
        x = before[lo:hi] + e
        pos, neg = x >= t, x <= -t
        assert torch.equal(_codes2(out_words, lo, hi), pos.to(torch.int64) + 2 * neg.to(torch.int64)), f"codes differ in [{lo}, {hi})"
        keep = torch.where(pos, x - t, torch.where(neg, x + t, x))
        assert torch.equal(res[lo:hi].view(torch.int32), keep.view(torch.int32)), f"residual differs in [{lo}, {hi})"


def test_sparse_decode_merge_at_the_largest_element_count(hp):
    n = (1 << 31) - 1
    _need(60)
    ratio = 0.001
    g = torch.empty(n, dtype=torch.float32, device="cuda")
    a = torch.empty(n, dtype=torch.float32, device="cuda")
    comps = []
    gen = torch.Generator(device="cuda")
    for p in range(3):
        gen.manual_seed(40 + p)
        for lo, hi in _chunks(n):
            g[lo:hi].normal_(0.0, 1e-3, generator=gen)
        a.zero_()
        c = torch.zeros(hp.sparse_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")
        hp.graddrop_encode(g, a, c, ratio)
        comps.append(c)
    torch.cuda.synchronize()
    cap = hp.sparse_capacity(n, ratio)
    expect = torch.zeros(n, dtype=torch.float32, device="cuda")
    for c in comps:  # peer after peer; a peer's indices are distinct
        nnz = c[:4].view(torch.int32)[0].item()
        idx = c[16:16 + 4 * nnz].view(torch.int32).to(torch.int64)
        val = c[16 + 4 * cap:16 + 4 * cap + 4 * nnz].view(torch.float32)
        expect[idx] = expect[idx] + val
    agg = g.fill_(7.0)
    acc = a
    gen.manual_seed(50)
    for lo, hi in _chunks(n):
        acc[lo:hi].normal_(0.0, 2e-4, generator=gen)
    v = acc + expect
    outc = torch.zeros(hp.sparse_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")
    hp.graddrop_decode_merge(comps, agg, acc, outc, ratio)
    torch.cuda.synchronize()
    for lo, hi in _chunks(n):
        assert torch.equal(agg[lo:hi], expect[lo:hi]), f"aggregate differs in [{lo}, {hi})"
    _check_selection(v, acc, outc, n, ratio, cap)
