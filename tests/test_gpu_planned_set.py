"""A gradient set under a SeCoPa plan on the GPU: every partition the plan cuts is
compressed on its own and equals the CPU oracle run on that slice; gradients the plan
leaves uncompressed are not touched."""
import numpy as np
import pytest
import torch

import oracle
from hipress_amd import planner

pytestmark = pytest.mark.gpu

F = np.float32

SIZES = [("conv_bias", 64), ("conv_weight", 36864), ("odd", 100003), ("dense_weight", 1200000), ("tiny_cut", 7)]
PLAN = ["conv_bias,64,n,4", "conv_weight,36864,y,1", "odd,100003,y,3", "dense_weight,1200000,y,4", "tiny_cut,7,y,16"]


@pytest.fixture(scope="module")
def hp():
    import hipress_amd

    assert torch.cuda.is_available()
    hipress_amd._lib.lib()
    return hipress_amd


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def gradients(seed, sigma=0.03):
    rng = np.random.default_rng(seed)
    return {name: (sigma * rng.standard_normal(n)).astype(F) for name, n in SIZES}


def test_partitions_follow_the_plan(hp):
    g = {k: torch.from_numpy(v).cuda() for k, v in gradients(0).items()}
    ps = hp.PlannedSet("tbq", PLAN, g, threshold=0.05)
    assert ps.uncompressed == ["conv_bias"]
    assert [p["length"] for p in ps.parts if p["name"] == "odd"] == [33336, 33336, 33331]
    assert [p["length"] for p in ps.parts if p["name"] == "tiny_cut"] == [4, 3]
    assert len(ps.compressed["dense_weight"]) == 4 and ps.elements == sum(n for _, n in SIZES) - 64
    assert "conv_bias" not in ps.compressed
    ps.close()


def test_tbq_plan_equals_the_oracle_per_partition_over_steps(hp):
    g = {k: torch.from_numpy(v).cuda() for k, v in gradients(0).items()}
    ps = hp.PlannedSet("tbq", PLAN, g, threshold=0.05)
    res = {name: np.zeros(n, F) for name, n in SIZES}
    for step in range(3):
        gs = gradients(step)
        for k, v in gs.items():
            g[k].copy_(torch.from_numpy(v))
        ps.encode()
        ps.decode()
        for p in ps.parts:
            name, i, off, ln = p["name"], p["index"], p["offset"], p["length"]
            want, r_new = oracle.tbq_encode(gs[name][off:off + ln], res[name][off:off + ln], 0.05)
            res[name][off:off + ln] = r_new
            np.testing.assert_array_equal(host(ps.compressed[name][i]), want, err_msg=f"{name}[{i}] step {step}")
            np.testing.assert_array_equal(host(ps.out[name])[off:off + ln], oracle.tbq_decode(want, ln))
        for name in ps.compressed:
            np.testing.assert_array_equal(host(ps.state[name]["residual"]), res[name])
        np.testing.assert_array_equal(host(g["conv_bias"]), gs["conv_bias"])
    ps.close()


def test_onebit_plan_has_one_scale_per_partition(hp):
    gs = gradients(5)
    g = {k: torch.from_numpy(v).cuda() for k, v in gs.items()}
    ps = hp.PlannedSet("onebit", PLAN, g)
    ps.encode()
    ps.decode()
    for p in ps.parts:
        name, i, off, ln = p["name"], p["index"], p["offset"], p["length"]
        got = host(ps.compressed[name][i])
        s = got[:4].view(F)[0]
        zero = np.zeros(ln, F)
        s_ref = oracle.onebit_scale(gs[name][off:off + ln], zero)
        assert abs(float(s) - float(s_ref)) <= 1e-5 * float(s_ref)
        want, r_new = oracle.onebit_encode(gs[name][off:off + ln], zero, scale=s)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(host(ps.state[name]["residual"])[off:off + ln], r_new)
    ps.close()


@pytest.mark.parametrize("alg", ["dgc", "graddrop"])
def test_sparse_plan_equals_the_oracle_per_partition(hp, alg):
    ratio = 0.01
    g = {k: torch.from_numpy(v).cuda() for k, v in gradients(0).items()}
    ps = hp.PlannedSet(alg, PLAN, g, ratio=ratio, momentum_factor=0.9)
    mom = {name: np.zeros(n, F) for name, n in SIZES}
    acc = {name: np.zeros(n, F) for name, n in SIZES}
    for step in range(2):
        gs = gradients(10 + step)
        for k, v in gs.items():
            g[k].copy_(torch.from_numpy(v))
        ps.encode()
        ps.decode()
        for p in ps.parts:
            name, i, off, ln = p["name"], p["index"], p["offset"], p["length"]
            sl = slice(off, off + ln)
            if alg == "dgc":
                want, m_new, a_new = oracle.dgc_encode(gs[name][sl], mom[name][sl], acc[name][sl], 0.9, ratio)
                mom[name][sl] = m_new
            else:
                want, a_new = oracle.graddrop_encode(gs[name][sl], acc[name][sl], ratio)
            acc[name][sl] = a_new
            got = host(ps.compressed[name][i])
            *hdr_g, idx_g, val_g = oracle.sparse_unpack(got)
            *hdr_w, idx_w, val_w = oracle.sparse_unpack(want)
            assert hdr_g == hdr_w, (name, i, step, hdr_g, hdr_w)
            np.testing.assert_array_equal(idx_g, idx_w)
            np.testing.assert_array_equal(val_g, val_w)
            np.testing.assert_array_equal(host(ps.out[name])[sl], oracle.sparse_decode(want, ln))
        for name in ps.compressed:
            np.testing.assert_array_equal(host(ps.state[name]["accumulator"]), acc[name])
            if alg == "dgc":
                np.testing.assert_array_equal(host(ps.state[name]["momentum"]), mom[name])
    ps.close()


def test_terngrad_plan_reads_the_noise_slice_of_each_partition(hp):
    gs = gradients(3)
    rng = np.random.default_rng(77)
    us = {name: rng.random(n, dtype=F) for name, n in SIZES}
    g = {k: torch.from_numpy(v).cuda() for k, v in gs.items()}
    u = {k: torch.from_numpy(v).cuda() for k, v in us.items()}
    ps = hp.PlannedSet("terngrad", PLAN, g, uniform=u, bucket=512)
    ps.encode()
    ps.decode()
    for p in ps.parts:
        name, i, off, ln = p["name"], p["index"], p["offset"], p["length"]
        want = oracle.terngrad_encode(gs[name][off:off + ln], us[name][off:off + ln], 512)
        np.testing.assert_array_equal(host(ps.compressed[name][i]), want)
        np.testing.assert_array_equal(host(ps.out[name])[off:off + ln], oracle.terngrad_decode(want, ln))
    ps.close()


def test_the_measured_vgg19_plan_runs_as_one_batch(hp):
    """The committed 4-node plan over the real VGG19 shapes: 18 weight tensors compressed in
    67 partitions, biases and the first convolution left alone; fc6's four partitions of
    25,690,112 elements against the oracle."""
    import os

    from hipress_amd import workloads as W

    plan = planner.read_plan(os.path.join(os.path.dirname(__file__), "golden", "plan_vgg19_tbq_ps4_mi355x.txt"))
    dev = torch.device("cuda:0")
    sizes = [size for _, size, _, _ in plan]
    assert sizes == W.vgg19_sizes()
    g = {name: t for (name, _, _, _), t in zip(plan, W.normal_set(sizes, dev, 0, log_sigma_range=(-4.0, -2.0)))}
    ps = hp.PlannedSet("tbq", plan, g, threshold=0.05)
    assert len(ps.uncompressed) == 20 and len(ps.compressed) == 18 and len(ps.parts) == 1 + 2 + 16 * 4
    ps.encode()
    ps.decode()
    name = "vgg0_dense0_weight"
    gh = host(g[name])
    for i, (off, ln) in enumerate(planner.partition_bounds(gh.size, 4)):
        want, r_new = oracle.tbq_encode(gh[off:off + ln], np.zeros(ln, F), 0.05)
        np.testing.assert_array_equal(host(ps.compressed[name][i]), want)
        np.testing.assert_array_equal(host(ps.state[name]["residual"][off:off + ln]), r_new)
    # every partition decodes to values of its own threshold grid and the residual identity holds
    for nm in ps.compressed:
        out, r = ps.out[nm], ps.state[nm]["residual"]
        assert bool(((out == 0) | (out.abs() == 0.05)).all())
        assert torch.equal(r, g[nm].view(-1) - out)
    ps.close()


@pytest.mark.parametrize("alg", ["tbq", "dgc"])
def test_planned_merge_sums_every_partition_in_peer_order_and_reencodes(hp, alg):
    """Three senders run the plan, the aggregator merges their partition payloads: every
    partition's sum, re-encoded payload and aggregator state equal the oracle's merge of the
    same payloads."""
    kw = {"threshold": 0.05} if alg == "tbq" else {"ratio": 0.01}
    senders, grads = [], []
    for p in range(3):
        g = {k: torch.from_numpy(v).cuda() for k, v in gradients(40 + p).items()}
        ps = hp.PlannedSet(alg, PLAN, g, **kw)
        ps.encode()
        senders.append(ps)
        grads.append(g)
    pm = hp.PlannedMerge(alg, PLAN, [s.compressed for s in senders], reencode=True, **kw)
    assert pm.uncompressed == ["conv_bias"] and len(pm.parts) == len(senders[0].parts)
    state = {name: np.zeros(n, F) for name, n in SIZES}
    for step in range(2):
        pm.run()
        for part in pm.parts:
            name, i, off, ln = part["name"], part["index"], part["offset"], part["length"]
            pays = [host(s.compressed[name][i]) for s in senders]
            if alg == "tbq":
                agg, out, r_new = oracle.tbq_decode_merge(pays, ln, state[name][off:off + ln], 0.05)
            else:
                agg, out, r_new = oracle.sparse_decode_merge(pays, ln, state[name][off:off + ln], 0.01)
            state[name][off:off + ln] = r_new
            np.testing.assert_array_equal(host(pm.aggregate[name])[off:off + ln], agg, err_msg=f"{name}[{i}] step {step}")
            got = host(pm.out_compressed[name][i])
            if alg == "tbq":
                np.testing.assert_array_equal(got, out)
            else:
                *hg, ig, vg = oracle.sparse_unpack(got)
                *hw, iw, vw = oracle.sparse_unpack(out)
                assert hg == hw
                np.testing.assert_array_equal(ig, iw)
                np.testing.assert_array_equal(vg, vw)
            np.testing.assert_array_equal(host(pm.state[name])[off:off + ln], r_new)
    pm.close()
    for s in senders:
        s.close()


def test_planned_merge_with_the_aggregators_own_gradient(hp):
    """A co-located server: two senders' payloads plus its own uncompressed gradients, partition by partition."""
    senders = []
    for p in range(2):
        ps = hp.PlannedSet("tbq", PLAN, {k: torch.from_numpy(v).cuda() for k, v in gradients(60 + p).items()}, threshold=0.05)
        ps.encode()
        senders.append(ps)
    mine = gradients(70)
    pm = hp.PlannedMerge("tbq", PLAN, [s.compressed for s in senders], reencode=True, threshold=0.05,
                         local={k: torch.from_numpy(v).cuda() for k, v in mine.items()})
    pm.run()
    for part in pm.parts:
        name, i, off, ln = part["name"], part["index"], part["offset"], part["length"]
        pays = [host(s.compressed[name][i]) for s in senders]
        agg, out, r_new = oracle.tbq_decode_merge(pays, ln, np.zeros(ln, F), 0.05, local=mine[name][off:off + ln])
        np.testing.assert_array_equal(host(pm.aggregate[name])[off:off + ln], agg)
        np.testing.assert_array_equal(host(pm.out_compressed[name][i]), out)
        np.testing.assert_array_equal(host(pm.state[name])[off:off + ln], r_new)
    pm.close()
    for s in senders:
        s.close()
