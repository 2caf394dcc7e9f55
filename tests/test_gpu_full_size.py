"""GPU parity at the sizes the benchmark configurations name: whole gradient sets
through the batched C ABI, compared with the CPU oracle where the oracle finishes
in seconds and through size-independent properties everywhere.  Also checks that
a captured HIP graph of encode+decode replays to the eager results."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

F = np.float32


@pytest.fixture(scope="module")
def hp():
    import hipress_amd

    assert torch.cuda.is_available()
    hipress_amd._lib.lib()
    return hipress_amd


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def test_onebit_vgg19_full_set_three_steps(hp):
    """configs[1]: onebit over the 38 VGG19 tensors, 143,667,240 elements, three steps with
    the residual carried, every tensor against the oracle."""
    from hipress_amd import workloads as W

    sizes = W.vgg19_sizes()
    dev = torch.device("cuda:0")
    ts = [{"gradient": torch.empty(n, device=dev), "residual": torch.zeros(n, device=dev), "out": torch.empty(n, device=dev),
           "compressed": torch.full((hp.onebit_payload_bytes(n),), 0xAB, dtype=torch.uint8, device="cuda")}
          for n in sizes]
    b = hp.Batch("onebit", ts)
    refs = [np.zeros(n, F) for n in sizes]
    for step in range(3):
        for t, g in zip(ts, W.normal_set(sizes, dev, step, log_sigma_range=(-4.0, -2.0))):
            t["gradient"].copy_(g)
        b.encode()
        b.decode()
        for i, (t, n) in enumerate(zip(ts, sizes)):
            g = host(t["gradient"])
            got = host(t["compressed"])
            s = got[:4].view(F)[0]
            s_ref = oracle.onebit_scale(g, refs[i])
            assert abs(float(s) - float(s_ref)) <= 1e-5 * float(s_ref), (step, n, s, s_ref)
            v = (refs[i] + g).astype(F)
            want, refs[i] = oracle.onebit_encode(g, refs[i], scale=s)
            np.testing.assert_array_equal(got, want, err_msg=f"payload, step {step} n={n}")
            res = host(t["residual"])
            np.testing.assert_array_equal(res, refs[i], err_msg=f"residual, step {step} n={n}")
            out = host(t["out"])
            # properties that hold at any size
            assert set(np.unique(out)).issubset({s, -s})
            np.testing.assert_array_equal(res, (v - out).astype(F))  # r' = v - d
    b.close()


def test_tbq_vgg19_full_set_three_steps(hp):
    """TBQ (threshold 0.05) over the 38 VGG19 tensors, three steps with the residual carried,
    every tensor against the oracle."""
    from hipress_amd import workloads as W

    sizes = W.vgg19_sizes()
    dev = torch.device("cuda:0")
    ts = [{"gradient": torch.empty(n, device=dev), "residual": torch.zeros(n, device=dev), "out": torch.empty(n, device=dev),
           "compressed": torch.full((hp.tbq_payload_bytes(n),), 0xAB, dtype=torch.uint8, device=dev)} for n in sizes]
    b = hp.Batch("tbq", ts, threshold=0.05)
    refs = [np.zeros(n, F) for n in sizes]
    for step in range(3):
        for t, g in zip(ts, W.normal_set(sizes, dev, 200 + step, sigma=0.02)):
            t["gradient"].copy_(g)
        b.encode()
        b.decode()
        for i, (t, n) in enumerate(zip(ts, sizes)):
            want, refs[i] = oracle.tbq_encode(host(t["gradient"]), refs[i], 0.05)
            np.testing.assert_array_equal(host(t["compressed"]), want, err_msg=f"payload, step {step} tensor {i}")
            np.testing.assert_array_equal(host(t["residual"]), refs[i], err_msg=f"residual, step {step} tensor {i}")
            np.testing.assert_array_equal(host(t["out"]), oracle.tbq_decode(want, n), err_msg=f"decode, step {step} tensor {i}")
    b.close()


def test_terngrad_resnet50_full_set(hp):
    """configs[2]: bucket 512, heavy-tailed gradients, explicit uniform tensor."""
    from hipress_amd import workloads as W

    sizes = W.resnet50_sizes()
    dev = torch.device("cuda:0")
    grads, unis = W.heavy_tailed_set(sizes, dev, 0), W.uniform_set(sizes, dev, 1000)
    ts = [{"gradient": g, "uniform": u, "out": torch.empty_like(g),
           "compressed": torch.full((hp.terngrad_payload_bytes(g.numel(), 512),), 0xAB, dtype=torch.uint8, device="cuda")}
          for g, u in zip(grads, unis)]
    b = hp.Batch("terngrad", ts, bucket=512)
    b.encode()
    b.decode()
    for t, n in zip(ts, sizes):
        g, u = host(t["gradient"]), host(t["uniform"])
        assert u.max() < 1.0
        want = oracle.terngrad_encode(g, u, 512)
        np.testing.assert_array_equal(host(t["compressed"]), want, err_msg=f"n={n}")
        out = host(t["out"])
        np.testing.assert_array_equal(out, oracle.terngrad_decode(want, n))
        # kept elements carry their bucket's scale with the gradient's sign
        nz = out != 0
        assert (np.sign(out[nz]) == np.sign(g[nz])).all()
    b.close()


def test_terngrad_vgg19_full_set(hp):
    """TernGrad (bucket 512) over the 38 VGG19 tensors, every tensor against the oracle."""
    from hipress_amd import workloads as W

    sizes = W.vgg19_sizes()
    dev = torch.device("cuda:0")
    grads, unis = W.normal_set(sizes, dev, 0, log_sigma_range=(-4.0, -2.0)), W.uniform_set(sizes, dev, 1000)
    ts = [{"gradient": g, "uniform": u, "out": torch.empty_like(g),
           "compressed": torch.full((hp.terngrad_payload_bytes(g.numel(), 512),), 0xAB, dtype=torch.uint8, device="cuda")}
          for g, u in zip(grads, unis)]
    b = hp.Batch("terngrad", ts, bucket=512)
    b.encode()
    b.decode()
    for t, n in zip(ts, sizes):
        want = oracle.terngrad_encode(host(t["gradient"]), host(t["uniform"]), 512)
        np.testing.assert_array_equal(host(t["compressed"]), want, err_msg=f"n={n}")
        np.testing.assert_array_equal(host(t["out"]), oracle.terngrad_decode(want, n), err_msg=f"decode n={n}")
    b.close()


def _sparse_full_set(hp, alg, sizes, grads_of_step, steps, ratio, m=0.9):
    """DGC or GradDrop over a whole gradient set for `steps` steps, EVERY tensor against the
    oracle: header, indices, values, state buffers and the decoded gradient."""
    dev = torch.device("cuda:0")
    ts = []
    for n in sizes:
        t = {"gradient": torch.empty(n, device=dev), "accumulator": torch.zeros(n, device=dev),
             "out": torch.empty(n, device=dev),
             "compressed": torch.zeros(hp.sparse_payload_bytes(n, ratio), dtype=torch.uint8, device=dev)}
        if alg == "dgc":
            t["momentum"] = torch.zeros(n, device=dev)
        ts.append(t)
    b = hp.Batch(alg, ts, momentum_factor=m, ratio=ratio)
    refs = [(np.zeros(n, F), np.zeros(n, F)) for n in sizes]
    for step in range(steps):
        for t, g in zip(ts, grads_of_step(step)):
            t["gradient"].copy_(g)
        b.encode()
        b.decode()
        total_nnz = 0
        for i, (t, n) in enumerate(zip(ts, sizes)):
            g = host(t["gradient"])
            where = f"{alg}, step {step} tensor {i} (n={n})"
            if alg == "dgc":
                want, mom, acc = oracle.dgc_encode(g, refs[i][0], refs[i][1], m, ratio)
                np.testing.assert_array_equal(host(t["momentum"]), mom, err_msg="momentum, " + where)
            else:
                want, acc = oracle.graddrop_encode(g, refs[i][1], ratio)
                mom = refs[i][0]
            refs[i] = (mom, acc)
            got_pay = host(t["compressed"])
            np.testing.assert_array_equal(got_pay[:16], want[:16], err_msg="header, " + where)
            got, w = oracle.sparse_unpack(got_pay), oracle.sparse_unpack(want)
            np.testing.assert_array_equal(got[4], w[4], err_msg="indices, " + where)
            np.testing.assert_array_equal(got[5], w[5], err_msg="values, " + where)
            np.testing.assert_array_equal(host(t["accumulator"]), acc, err_msg="accumulator, " + where)
            np.testing.assert_array_equal(host(t["out"]), oracle.sparse_decode(want, n), err_msg="decode, " + where)
            total_nnz += got[0]
        density = total_nnz / sum(sizes)
        assert 0.7 * ratio < density < 1.6 * ratio, density
    b.close()


def test_dgc_bert_large_full_set_two_steps(hp):
    """configs[3]: DGC 0.1 % with momentum 0.9 over the 391 BERT-large tensors (335,141,888
    elements), two steps, every tensor against the oracle."""
    from hipress_amd import workloads as W

    sizes = W.bert_large_sizes()
    _sparse_full_set(hp, "dgc", sizes, lambda step: W.normal_set(sizes, torch.device("cuda:0"), step, sigma=1e-3), 2, 0.001)


def test_graddrop_bert_large_full_set_two_steps(hp):
    """configs[3], second half: GradDrop with drop ratio 0.99 (1 % kept) on the same 391
    BERT-large tensors, two steps, every tensor against the oracle."""
    from hipress_amd import workloads as W

    sizes = W.bert_large_sizes()
    _sparse_full_set(hp, "graddrop", sizes, lambda step: W.normal_set(sizes, torch.device("cuda:0"), 50 + step, sigma=1e-3), 2, 0.01)


def test_dgc_vgg19_full_set_three_steps(hp):
    """DGC 0.1 % over the 38 VGG19 tensors (143,667,240 elements), three steps with momentum
    and accumulator carried, every tensor against the oracle."""
    from hipress_amd import workloads as W

    sizes = W.vgg19_sizes()
    _sparse_full_set(hp, "dgc", sizes,
                     lambda step: W.normal_set(sizes, torch.device("cuda:0"), 300 + step, log_sigma_range=(-4.0, -2.0)), 3, 0.001)


def test_graddrop_150m_elements_three_steps(hp):
    """One tensor of 150,000,000 elements (36,622 tiles, 367 workgroups in every threshold
    pass), three steps against the oracle: with this many workgroups a threshold pass that
    lets its last workgroup read the histogram before every other one's adds have landed
    picks a key a few ranks off."""
    n, ratio = 150_000_000, 0.01
    gen = torch.Generator(device="cuda").manual_seed(17)
    acc = torch.zeros(n, device="cuda")
    pay = torch.zeros(hp.graddrop_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")
    out = torch.empty(n, device="cuda")
    g = torch.empty(n, device="cuda")
    b = hp.Batch("graddrop", [{"gradient": g, "accumulator": acc, "compressed": pay, "out": out}], ratio=ratio)
    ref_acc = np.zeros(n, F)
    for step in range(3):
        g.normal_(0, 1e-3, generator=gen)
        b.encode()
        b.decode()
        want, ref_acc = oracle.graddrop_encode(host(g), ref_acc, ratio)
        got = host(pay)
        nnz, _, cap, thr, idx, val = oracle.sparse_unpack(got)
        w = oracle.sparse_unpack(want)
        assert (nnz, cap) == (w[0], w[2]) and thr.view(np.uint32) == w[3].view(np.uint32), f"step {step}"
        np.testing.assert_array_equal(idx, w[4])
        np.testing.assert_array_equal(val, w[5])
        np.testing.assert_array_equal(host(acc), ref_acc)
        o = host(out)
        assert np.count_nonzero(o) == nnz
        np.testing.assert_array_equal(o[idx], val)
    b.close()


def test_dgc_one_tensor_beyond_one_accumulate_launch(hp):
    """One tensor of 49,152 tiles + 12,345 elements through the per-tensor entry point: the
    accumulate pass is issued in two launches, the second starting in the middle of the
    tensor.  Two steps against the oracle."""
    n, ratio, m = 49152 * 4096 + 12345, 0.001, 0.9
    gen = torch.Generator(device="cuda").manual_seed(23)
    mom, acc = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    pay = torch.zeros(hp.dgc_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")
    g = torch.empty(n, device="cuda")
    ref_mom, ref_acc = np.zeros(n, F), np.zeros(n, F)
    for step in range(2):
        g.normal_(0, 1e-3, generator=gen)
        hp.dgc_encode(g, mom, acc, pay, m, ratio)
        want, ref_mom, ref_acc = oracle.dgc_encode(host(g), ref_mom, ref_acc, m, ratio)
        got, w = oracle.sparse_unpack(host(pay)), oracle.sparse_unpack(want)
        assert got[:3] == w[:3] and got[3].view(np.uint32) == w[3].view(np.uint32), f"step {step}"
        np.testing.assert_array_equal(got[4], w[4])
        np.testing.assert_array_equal(got[5], w[5])
        np.testing.assert_array_equal(host(acc), ref_acc)
        np.testing.assert_array_equal(host(mom), ref_mom)


def test_merge_vgg19_chunks_tbq(hp):
    """configs[4], TBQ half: 8 peers x 168 chunks of at most 4 MB, decode-and-merge with the
    fused re-encode; every chunk against the oracle, and the integer identity on all."""
    from hipress_amd import workloads as W

    sizes = W.chunk_sizes(W.vgg19_sizes())
    assert len(sizes) == 168
    dev = torch.device("cuda:0")
    tau, P = 0.05, 8
    chunks = [{"compressed": [torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device=dev) for _ in range(P)],
               "aggregate": torch.empty(n, device=dev), "state": torch.zeros(n, device=dev),
               "out_compressed": torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device=dev)} for n in sizes]
    for p in range(P):
        grads = W.normal_set(sizes, dev, p + 1, sigma=0.02)
        enc = hp.Batch("tbq", [{"gradient": g, "residual": torch.zeros_like(g), "compressed": c["compressed"][p]}
                               for g, c in zip(grads, chunks)], threshold=tau)
        enc.encode()
        torch.cuda.synchronize()
        enc.close()
    mb = hp.MergeBatch("tbq", chunks, threshold=tau)
    mb.run()
    for i, (c, n) in enumerate(zip(chunks, sizes)):
        agg = host(c["aggregate"])
        # every aggregate value is an integer multiple of tau between -8 tau and 8 tau
        k = np.rint(agg / F(tau))
        assert np.abs(k).max() <= P
        np.testing.assert_allclose(agg, k * np.float64(tau), rtol=1e-5, atol=0)
        pays = [host(p) for p in c["compressed"]]
        want_agg, want_out, want_r = oracle.tbq_decode_merge(pays, n, np.zeros(n, F), tau)
        np.testing.assert_array_equal(agg, want_agg, err_msg=f"aggregate, chunk {i}")
        np.testing.assert_array_equal(host(c["out_compressed"]), want_out, err_msg=f"payload, chunk {i}")
        np.testing.assert_array_equal(host(c["state"]), want_r, err_msg=f"residual, chunk {i}")
    mb.close()


def test_graddrop_vgg19_full_set_three_steps(hp):
    """GradDrop 1 % over the 38 VGG19 tensors (143,667,240 elements), three steps, every
    tensor against the oracle: payload, accumulator and decoded gradient."""
    from hipress_amd import workloads as W

    sizes = W.vgg19_sizes()
    dev = torch.device("cuda:0")
    ratio = 0.01
    ts = [{"gradient": torch.empty(n, device=dev), "accumulator": torch.zeros(n, device=dev),
           "out": torch.empty(n, device=dev),
           "compressed": torch.zeros(hp.graddrop_payload_bytes(n, ratio), dtype=torch.uint8, device=dev)} for n in sizes]
    b = hp.Batch("graddrop", ts, ratio=ratio)
    refs = [np.zeros(n, F) for n in sizes]
    for step in range(3):
        for t, g in zip(ts, W.normal_set(sizes, dev, 100 + step, log_sigma_range=(-4.0, -2.0))):
            t["gradient"].copy_(g)
        b.encode()
        b.decode()
        for i, (t, n) in enumerate(zip(ts, sizes)):
            want, refs[i] = oracle.graddrop_encode(host(t["gradient"]), refs[i], ratio)
            np.testing.assert_array_equal(host(t["compressed"])[:16], want[:16], err_msg=f"header, step {step} tensor {i}")
            got = oracle.sparse_unpack(host(t["compressed"]))
            w = oracle.sparse_unpack(want)
            np.testing.assert_array_equal(got[4], w[4], err_msg=f"indices, step {step} tensor {i}")
            np.testing.assert_array_equal(got[5], w[5], err_msg=f"values, step {step} tensor {i}")
            np.testing.assert_array_equal(host(t["accumulator"]), refs[i], err_msg=f"accumulator, step {step} tensor {i}")
            np.testing.assert_array_equal(host(t["out"]), oracle.sparse_decode(want, n), err_msg=f"decode, step {step} tensor {i}")
    b.close()


def test_merge_vgg19_chunks_dgc(hp):
    """configs[4], DGC half: 8 peers x 168 chunks, sparse decode-and-merge with the GradDrop-style
    re-encode of the aggregate; two rounds on the same batch object, every chunk against the oracle."""
    from hipress_amd import workloads as W

    sizes = W.chunk_sizes(W.vgg19_sizes())
    dev = torch.device("cuda:0")
    ratio, P = 0.001, 8
    chunks = [{"compressed": [torch.zeros(hp.dgc_payload_bytes(n, ratio), dtype=torch.uint8, device=dev) for _ in range(P)],
               "aggregate": torch.empty(n, device=dev), "state": torch.zeros(n, device=dev),
               "out_compressed": torch.zeros(hp.dgc_payload_bytes(n, ratio), dtype=torch.uint8, device=dev)} for n in sizes]
    mb = hp.MergeBatch("dgc", chunks, ratio=ratio)
    ref_acc = [np.zeros(n, F) for n in sizes]
    for rnd in range(2):
        for p in range(P):
            grads = W.normal_set(sizes, dev, 10 * rnd + p + 1, sigma=1e-3)
            enc = hp.Batch("dgc", [{"gradient": g, "momentum": torch.zeros_like(g), "accumulator": torch.zeros_like(g),
                                    "compressed": c["compressed"][p]} for g, c in zip(grads, chunks)],
                           momentum_factor=0.9, ratio=ratio)
            enc.encode()
            torch.cuda.synchronize()
            enc.close()
        mb.run()
        for i, (c, n) in enumerate(zip(chunks, sizes)):
            pays = [host(q) for q in c["compressed"]]
            agg, out, ref_acc[i] = oracle.sparse_decode_merge(pays, n, ref_acc[i], ratio)
            np.testing.assert_array_equal(host(c["aggregate"]), agg, err_msg=f"aggregate, round {rnd} chunk {i}")
            np.testing.assert_array_equal(host(c["out_compressed"])[:16], out[:16], err_msg=f"header, round {rnd} chunk {i}")
            got, w = oracle.sparse_unpack(host(c["out_compressed"])), oracle.sparse_unpack(out)
            np.testing.assert_array_equal(got[4], w[4], err_msg=f"indices, round {rnd} chunk {i}")
            np.testing.assert_array_equal(got[5], w[5], err_msg=f"values, round {rnd} chunk {i}")
            np.testing.assert_array_equal(host(c["state"]), ref_acc[i], err_msg=f"accumulator, round {rnd} chunk {i}")
    mb.close()


def test_hip_graph_replay_matches_eager(hp):
    """encode + decode enqueue only kernels (no allocation, no host synchronisation),
    so they can be captured in a HIP graph; every replay must equal the eager result."""
    n = 262144
    g = torch.randn(n, device="cuda", generator=torch.Generator(device="cuda").manual_seed(0)) * 0.02
    r = torch.zeros(n, device="cuda")
    pay = torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")
    out = torch.empty(n, device="cuda")
    # eager reference over three steps (the residual carries)
    eager = []
    for _ in range(3):
        hp.tbq_encode(g, r, pay, 0.05)
        hp.tbq_decode(pay, out)
        eager.append((host(pay).copy(), host(r).copy(), host(out).copy()))
    r.zero_()
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        hp.tbq_encode(g, r, pay, 0.05)  # warm-up on the capture stream
        hp.tbq_decode(pay, out)
        stream.synchronize()
        r.zero_()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            hp.tbq_encode(g, r, pay, 0.05)
            hp.tbq_decode(pay, out)
    for step in range(3):
        graph.replay()
        torch.cuda.synchronize()
        _ = (out * 2).sum().item()  # unrelated eager work between replays
        np.testing.assert_array_equal(host(pay), eager[step][0], err_msg=f"payload, replay {step}")
        np.testing.assert_array_equal(host(r), eager[step][1], err_msg=f"residual, replay {step}")
        np.testing.assert_array_equal(host(out), eager[step][2], err_msg=f"decode, replay {step}")


@pytest.mark.parametrize("bucket", [777, 100_000, 3_000_000])
def test_hip_graph_replay_of_terngrad_with_long_buckets(hp, bucket):
    """The encoders for bucket sizes that no wavefront covers (maxima gathered in LDS; beyond
    a tile, three launches that park per-tile maxima in the payload's word area) captured
    with the decode: each replay sees a new gradient in the same buffers and must give what
    the oracle gives for it, also where the scales shrink from one replay to the next."""
    n = 2_500_003
    rng = np.random.default_rng(bucket)
    g, u = torch.empty(n, device="cuda"), torch.empty(n, device="cuda")
    pay = torch.zeros(hp.terngrad_payload_bytes(n, bucket), dtype=torch.uint8, device="cuda")
    out = torch.empty(n, device="cuda")
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        g.zero_(); u.zero_()
        hp.terngrad_encode(g, u, pay, bucket)  # warm-up on the capture stream
        hp.terngrad_decode(pay, out)
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            hp.terngrad_encode(g, u, pay, bucket)
            hp.terngrad_decode(pay, out)
    for step, sigma in enumerate([1e-2, 1e-3, 1e-4]):
        gh, uh = rng.normal(0, sigma, n).astype(np.float32), rng.random(n, dtype=np.float32)
        g.copy_(torch.from_numpy(gh)); u.copy_(torch.from_numpy(uh))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _ = (out * 2).sum().item()  # unrelated eager work between replays
        want = oracle.terngrad_encode(gh, uh, bucket)
        np.testing.assert_array_equal(host(pay), want, err_msg=f"payload, replay {step}")
        np.testing.assert_array_equal(host(out), oracle.terngrad_decode(want, n), err_msg=f"decode, replay {step}")


def test_hip_graph_replay_of_a_sparse_batch(hp):
    """The batched DGC encode + decode (ten launches, idle dynamic LDS on some, a per-call
    counter in the decode) captured once and replayed: every replay equals the eager run
    that started from the same state."""
    sizes = [1000003, 262144, 4097]
    ratio, m = 0.001, 0.9
    gen = torch.Generator(device="cuda").manual_seed(3)
    grads = [torch.randn(n, device="cuda", generator=gen) * 1e-3 for n in sizes]

    def make():
        return [{"gradient": g, "momentum": torch.zeros_like(g), "accumulator": torch.zeros_like(g),
                 "out": torch.empty_like(g),
                 "compressed": torch.zeros(hp.dgc_payload_bytes(g.numel(), ratio), dtype=torch.uint8, device="cuda")}
                for g in grads]

    eager_ts = make()
    eb = hp.Batch("dgc", eager_ts, momentum_factor=m, ratio=ratio)
    eager = []
    for _ in range(3):
        eb.encode()
        eb.decode()
        eager.append([(host(t["compressed"]).copy(), host(t["accumulator"]).copy(), host(t["out"]).copy()) for t in eager_ts])
    eb.close()
    ts = make()
    b = hp.Batch("dgc", ts, momentum_factor=m, ratio=ratio)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        b.encode()  # warm-up on the capture stream, then back to the initial state
        b.decode()
        stream.synchronize()
        for t in ts:
            t["momentum"].zero_()
            t["accumulator"].zero_()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            b.encode()
            b.decode()
    for step in range(3):
        graph.replay()
        torch.cuda.synchronize()
        _ = (ts[0]["out"] * 2).sum().item()  # unrelated eager work between replays
        for t, (pay, acc, out) in zip(ts, eager[step]):
            np.testing.assert_array_equal(host(t["compressed"]), pay, err_msg=f"payload, replay {step}")
            np.testing.assert_array_equal(host(t["accumulator"]), acc, err_msg=f"accumulator, replay {step}")
            np.testing.assert_array_equal(host(t["out"]), out, err_msg=f"decode, replay {step}")
    b.close()


# ---------------------------------------------------------------- beyond the benchmark's sizes
# Above certain launch sizes the batched decoders are started with a different
# occupancy (the caps stop paying there).  The oracle would take minutes at these sizes:
# the batched decode is compared with the per-tensor entry point, which takes other
# launch paths (single-tensor kernels; zero fill + scatter for the sparse formats), and
# the encode with properties that hold at any size.

def _uniform_set(count, n, sigma, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    return [torch.randn(n, generator=gen, device="cuda") * sigma for _ in range(count)]


def test_graddrop_batch_decode_of_a_large_launch_matches_the_per_tensor_decode(hp):
    """~240 M elements at one per cent: more tiles than the sparse tile decode's cap covers."""
    sizes = [64 << 20, 64 << 20, 64 << 20, (48 << 20) + 1]
    ratio = 0.01
    ts = []
    for i, n in enumerate(sizes):
        g = _uniform_set(1, n, 1e-3, 40 + i)[0]
        ts.append({"gradient": g, "accumulator": torch.zeros_like(g), "out": torch.full_like(g, 7.0),
                   "compressed": torch.zeros(hp.graddrop_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")})
    b = hp.Batch("graddrop", ts, ratio=ratio)
    assert sum((n + 4095) // 4096 for n in sizes) > 57344
    b.encode()
    b.decode()
    for t in ts:
        n = t["gradient"].numel()
        single = torch.full_like(t["out"], -3.0)
        hp.graddrop_decode(t["compressed"], single)
        assert torch.equal(t["out"], single)
        nnz = int(t["compressed"][:4].view(torch.int32).item())
        assert 0.5 * ratio * n < nnz < 2.0 * ratio * n
        assert int((t["out"] != 0).sum().item()) == nnz
        # what was sent plus what stays is the gradient (first step: accumulator started at zero)
        assert torch.equal(t["out"] + t["accumulator"], t["gradient"])
    b.close()


def test_tbq_batch_decode_with_a_payload_beyond_the_cache_matches_the_per_tensor_decode(hp):
    """~870 M elements: 218 MB of packed words, more than the decoders' cap covers."""
    n, count, tau = 64 << 20, 13, 0.05
    ts = []
    for i in range(count):
        g = _uniform_set(1, n, 0.04, 60 + i)[0]
        ts.append({"gradient": g, "residual": torch.zeros_like(g), "out": torch.empty_like(g),
                   "compressed": torch.zeros(hp.tbq_payload_bytes(n), dtype=torch.uint8, device="cuda")})
    assert count * (n // 4) > (192 << 20)
    b = hp.Batch("tbq", ts, threshold=tau)
    b.encode()
    b.decode()
    single = torch.empty(n, device="cuda")
    for t in ts:
        hp.tbq_decode(t["compressed"], single)
        assert torch.equal(t["out"], single)
        g, out = t["gradient"], t["out"]
        want = torch.where(g >= tau, torch.full_like(g, tau), torch.where(g <= -tau, torch.full_like(g, -tau), torch.zeros_like(g)))
        assert torch.equal(out, want)
        assert torch.equal(t["residual"], g - out)
    b.close()


def test_dgc_batch_decode_of_a_very_large_launch_matches_the_per_tensor_decode(hp):
    """~1.14 G elements at 0.1 per cent: more tiles than the few-pairs cap covers."""
    n, count, ratio = 64 << 20, 17, 0.001
    ts = []
    for i in range(count):
        g = _uniform_set(1, n, 1e-3, 80 + i)[0]
        ts.append({"gradient": g, "momentum": torch.zeros_like(g), "accumulator": torch.zeros_like(g),
                   "out": torch.full_like(g, 7.0),
                   "compressed": torch.zeros(hp.dgc_payload_bytes(n, ratio), dtype=torch.uint8, device="cuda")})
    assert count * (n // 4096) > 262144
    b = hp.Batch("dgc", ts, momentum_factor=0.9, ratio=ratio)
    b.encode()
    b.decode()
    single = torch.empty(n, device="cuda")
    for t in ts:
        hp.dgc_decode(t["compressed"], single)
        assert torch.equal(t["out"], single)
        nnz = int(t["compressed"][:4].view(torch.int32).item())
        assert 0.5 * ratio * n < nnz < 2.0 * ratio * n
        assert int((t["out"] != 0).sum().item()) == nnz
        assert torch.equal(t["out"] + t["accumulator"], t["gradient"])
    b.close()
