"""Writes tests/golden/operator_vectors.npz: inputs and the CPU oracle's outputs for every
operator on small fixed cases, so that a change to oracle and kernels in step (a bit order, a
header field, a tie rule) no longer passes unnoticed.

    python tests/golden/make_operator_vectors.py

Dense cases store inputs and outputs whole (n = 5003: a partial tile, a partial word, a
partial bucket).  The sampled-threshold path of the sparse compressors only starts at
262,144 elements, so those cases store the payload (a few KB) and SHA-256 digests of the
large arrays; their inputs come from the counter-based generator (hipress_amd.datagen) and
are digested too, so that a platform whose libm moves an input by one unit is told apart
from a wrong result.  Loaded with numpy.load(allow_pickle=False)."""
import hashlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402
from hipress_amd import datagen  # noqa: E402

F = np.float32
N_DENSE, N_SPARSE, PEERS = 5003, 300007, 3
CPU = torch.device("cpu")


def digest(a):
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest(), np.uint8).copy()


def normal(n, seed, tensor, sigma):
    return datagen.normal(n, CPU, seed, tensor, sigma).numpy().astype(F)


def uniform(n, seed, tensor):
    return datagen.uniform(n, CPU, seed, tensor).numpy().astype(F)


def main():
    out = {}
    n = N_DENSE
    g = [normal(n, 7, t, 0.03) for t in range(3)]
    # tbq: three steps with the residual carried, threshold 0.05
    r = np.zeros(n, F)
    for step in range(3):
        pay, r = oracle.tbq_encode(g[step], r, 0.05)
        out[f"tbq_gradient_{step}"], out[f"tbq_payload_{step}"] = g[step], pay
        out[f"tbq_residual_{step}"], out[f"tbq_decoded_{step}"] = r.copy(), oracle.tbq_decode(pay, n)
    # onebit: two steps; the scale is the oracle's own (a GPU result is compared within 1e-5, and
    # bit for bit after the oracle has been given the GPU's scale - see the test)
    r = normal(n, 7, 10, 1e-3)
    out["onebit_residual_in"] = r.copy()
    for step in range(2):
        gg = normal(n, 7, 11 + step, 1e-3)
        pay, r = oracle.onebit_encode(gg, r)
        out[f"onebit_gradient_{step}"], out[f"onebit_payload_{step}"] = gg, pay
        out[f"onebit_residual_{step}"], out[f"onebit_decoded_{step}"] = r.copy(), oracle.onebit_decode(pay, n)
    # terngrad: buckets of 512 and of 100 (the generic path), with heavy-tailed outliers
    gt = normal(n, 7, 20, 1e-3)
    pick = uniform(n, 7, 21) < 0.01
    gt[pick] = (normal(n, 7, 22, 1e-2))[pick]
    u = uniform(n, 7, 23)
    out["terngrad_gradient"], out["terngrad_uniform"] = gt, u
    for bucket in (512, 100):
        pay = oracle.terngrad_encode(gt, u, bucket)
        out[f"terngrad_payload_b{bucket}"], out[f"terngrad_decoded_b{bucket}"] = pay, oracle.terngrad_decode(pay, n)
    # the in-tree min/max quantiser, all four widths
    for b in (1, 2, 4, 8):
        pay = oracle.compll_encode(gt, u, b)
        out[f"compll_payload_b{b}"] = pay
        out[f"compll_decoded_b{b}"] = oracle.compll_decode(pay, n)
    # dense merges of three peers, TBQ with the re-encode
    peers = []
    for p in range(PEERS):
        pay, _ = oracle.tbq_encode(normal(n, 8, p, 0.04), np.zeros(n, F), 0.05)
        peers.append(pay)
        out[f"merge_tbq_peer_{p}"] = pay
    agg, outp, res = oracle.tbq_decode_merge(peers, n, np.zeros(n, F), 0.05)
    out["merge_tbq_aggregate"], out["merge_tbq_out_payload"], out["merge_tbq_residual"] = agg, outp, res
    # sparse: small (every element is a sample) and large (every 100th is), two steps each
    for tag, ns in (("small", N_DENSE), ("large", N_SPARSE)):
        mom, acc, acc_gd = np.zeros(ns, F), np.zeros(ns, F), np.zeros(ns, F)
        for step in range(2):
            gs = normal(ns, 9, step, 1e-3)
            out[f"sparse_{tag}_gradient_digest_{step}"] = digest(gs)
            if tag == "small":
                out[f"sparse_small_gradient_{step}"] = gs
            pay, mom, acc = oracle.dgc_encode(gs, mom, acc, 0.9, 0.001)
            out[f"dgc_{tag}_payload_{step}"] = pay
            out[f"dgc_{tag}_momentum_digest_{step}"], out[f"dgc_{tag}_accumulator_digest_{step}"] = digest(mom), digest(acc)
            out[f"dgc_{tag}_decoded_digest_{step}"] = digest(oracle.sparse_decode(pay, ns))
            pay, acc_gd = oracle.graddrop_encode(gs, acc_gd, 0.01)
            out[f"graddrop_{tag}_payload_{step}"] = pay
            out[f"graddrop_{tag}_accumulator_digest_{step}"] = digest(acc_gd)
    # sparse merge of three GradDrop payloads with the re-encode (large case)
    sp = [oracle.graddrop_encode(normal(N_SPARSE, 10, p, 1e-3), np.zeros(N_SPARSE, F), 0.01)[0] for p in range(PEERS)]
    for p in range(PEERS):
        out[f"merge_sparse_peer_{p}"] = sp[p]
    agg, outp, acc = oracle.sparse_decode_merge(sp, N_SPARSE, np.zeros(N_SPARSE, F), 0.01)
    out["merge_sparse_aggregate_digest"], out["merge_sparse_accumulator_digest"] = digest(agg), digest(acc)
    out["merge_sparse_out_payload"] = outp
    path = os.path.join(HERE, "operator_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
