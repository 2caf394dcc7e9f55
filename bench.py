#!/usr/bin/env python3
"""Throughput of the gradient-compression hot path on one MI355X.

A step is one pass of encode followed by decode over a whole synthetic gradient
set that is already resident in HBM.  The headline line is onebit over the
VGG19 gradient set; `--workload` selects another, and `others` in the JSON line
carries a shorter measurement of every other compressor / configuration.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-others] [--no-cpu]

Prints ONE JSON line.  value = 4 * elements * steps / elapsed, in GB/s of fp32
gradient through encode+decode.  `roofline` describes the dominant kernel:
algorithmic bytes per launch over its mean duration, measured with events on the
launch stream inside the timed steps, against the 8 TB/s HBM peak.
"""
import argparse
import ctypes
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs (summaries under profiles/), keyed by workload; absent = not
# measured.  (FETCH_SIZE KiB * 2.0 + WRITE_SIZE KiB * 1.0) * 1024, the factors
# being what the same counters read for a plain 1 GiB copy.
MEASURED_TRAFFIC = {
    "onebit_vgg19": 1747750092,           # onebit_quant_kernel
    "onebit_deferred_vgg19": 1748885811,  # onebit_deferred_kernel
    "tbq_vgg19": 1765707366,              # tbq_encode_kernel
    "terngrad_vgg19": 1193284403,         # terngrad_encode_kernel
    "dgc_vgg19": 2904932454,              # sparse_accum_kernel
    "graddrop_vgg19": 1755469209,         # sparse_accum_kernel
    "tbq_262144_x512": 1650560614,        # tbq_encode_kernel
    "terngrad_resnet50": 212500377,       # terngrad_encode_kernel
    "dgc_bert_large": 6782823833,         # sparse_accum_kernel
    "graddrop_bert_large": 4101445222,    # sparse_accum_kernel
    "merge_tbq_vgg19": 2090826240,        # dense_merge_kernel
    "merge_dgc_vgg19": 1780978995,        # sparse_merge_kernel
    "compll_b2_fc6": 848749465,           # compll_quant_kernel
    "compll_generated_b2_fc6": 848736665, # map_packed_kernel of the generated operator
    "merge_tbq_vgg19_payload_only": 1516136345,  # dense_merge_kernel
    "merge_dgc_vgg19_payload_only": 1206018662,  # sparse_merge_kernel
}


def _events(n):
    import torch

    return [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]


class SetWorkload:
    """encode+decode of one compressor over a list of tensor sizes through a Batch."""

    def __init__(self, name, alg, sizes, data, params, enc_bytes, dec_bytes, dominant_phase, dominant_kernel,
                 dominant_bytes, rotate=1, nphases=1, graph=False):
        self.graph = graph  # replay encode+decode from a captured HIP graph (one launch per step)
        self.name, self.alg, self.sizes, self.data, self.params = name, alg, sizes, data, params
        self.enc_bytes, self.dec_bytes = enc_bytes, dec_bytes  # algorithmic bytes per element
        self.dominant_phase, self.dominant_kernel, self.dominant_bytes = dominant_phase, dominant_kernel, dominant_bytes
        self.rotate, self.nphases = rotate, nphases
        self.elements = sum(sizes)

    def setup(self, dev):
        import torch

        import hipress_amd as hp
        from hipress_amd import workloads as W

        self.batches = []
        self.tensors = []
        for rot in range(self.rotate):
            seed = rot  # rotation 0 is the configuration's seed 0
            if self.data == "vgg":
                grads = W.normal_set(self.sizes, dev, seed, log_sigma_range=(-4.0, -2.0))
            elif self.data == "n0.02":
                grads = W.normal_set(self.sizes, dev, seed, sigma=0.02)
            elif self.data == "heavy":
                grads = W.heavy_tailed_set(self.sizes, dev, seed)
            else:
                grads = W.normal_set(self.sizes, dev, seed, sigma=1e-3)
            ts = []
            ratio = self.params.get("ratio", 0.001)
            for i, (n, g) in enumerate(zip(self.sizes, grads)):
                t = {"gradient": g, "out": torch.empty(n, device=dev)}
                if self.alg == "tbq":
                    t["residual"] = torch.zeros(n, device=dev)
                    nb = hp.tbq_payload_bytes(n)
                elif self.alg == "onebit":
                    t["residual"] = torch.zeros(n, device=dev)
                    nb = hp.onebit_payload_bytes(n)
                elif self.alg == "onebit_deferred":
                    t["state"] = torch.zeros(n, device=dev)
                    t["scale_state"] = torch.zeros(1, device=dev)
                    nb = hp.onebit_payload_bytes(n)
                elif self.alg == "terngrad":
                    nb = hp.terngrad_payload_bytes(n, self.params.get("bucket", 512))
                elif self.alg == "dgc":
                    t["momentum"] = torch.zeros(n, device=dev)
                    t["accumulator"] = torch.zeros(n, device=dev)
                    nb = hp.dgc_payload_bytes(n, ratio)
                else:
                    t["accumulator"] = torch.zeros(n, device=dev)
                    nb = hp.graddrop_payload_bytes(n, ratio)
                t["compressed"] = torch.zeros(nb, dtype=torch.uint8, device=dev)
                ts.append(t)
            if self.alg == "terngrad":
                for t, u in zip(ts, W.uniform_set(self.sizes, dev, 1000 + seed)):
                    t["uniform"] = u
            self.tensors.append(ts)
            self.batches.append(hp.Batch(self.alg, ts, **self.params))
        self.k = 0
        self.captured = None
        if self.graph:
            side = torch.cuda.Stream()
            b = self.batches[0]
            with torch.cuda.stream(side):
                b.encode()
                b.decode()
                side.synchronize()
                self.captured = torch.cuda.CUDAGraph()
                with torch.cuda.graph(self.captured, stream=side):
                    b.encode()
                    b.decode()
            torch.cuda.synchronize()

    def step(self, ev=None):
        if self.captured is not None:
            self.captured.replay()
            return
        b = self.batches[self.k % self.rotate]
        self.k += 1
        if ev is None:
            b.encode()
        else:
            for ph in range(self.nphases):
                if ph == self.dominant_phase:
                    ev[0].record()
                    b.encode_phase(ph)
                    ev[1].record()
                else:
                    b.encode_phase(ph)
        b.decode()

    def density(self):
        """Measured fraction of elements kept (sparse compressors)."""
        import torch

        nnz = 0
        for t in self.tensors[0]:
            nnz += int(t["compressed"][:4].view(torch.int32).item())
        return nnz / self.elements

    def close(self):
        self.captured = None
        for b in self.batches:
            b.close()
        self.batches, self.tensors = [], []


class MergeWorkload:
    """Decode-and-merge of 8 peer payloads per 4 MB chunk of the VGG19 set, with the
    fused re-encode for the next hop."""

    def __init__(self, name, alg, sizes, npeers=8, aggregate=True):
        self.name, self.alg, self.sizes, self.npeers = name, alg, sizes, npeers
        self.aggregate = aggregate  # False: only the re-encoded payload is produced (no fp32 sum written)
        self.elements = sum(sizes)
        self.dominant_phase = 0
        self.nphases = 1
        self.rotate = 1

    def setup(self, dev):
        import torch

        import hipress_amd as hp
        from hipress_amd import workloads as W

        tau, ratio = 0.05, 0.001
        self.ratio = ratio
        chunks = []
        for n in self.sizes:
            nb = hp.tbq_payload_bytes(n) if self.alg == "tbq" else hp.dgc_payload_bytes(n, ratio)
            chunks.append({"compressed": [torch.zeros(nb, dtype=torch.uint8, device=dev) for _ in range(self.npeers)],
                           "aggregate": torch.empty(n, device=dev) if self.aggregate else None,
                           "state": torch.zeros(n, device=dev),
                           "out_compressed": torch.zeros(nb, dtype=torch.uint8, device=dev)})
        # peer p's payloads come from that peer's own gradients (seed p) through the encoders
        for p in range(self.npeers):
            if self.alg == "tbq":
                grads = W.normal_set(self.sizes, dev, p + 1, sigma=0.02)
                ts = [{"gradient": g, "residual": torch.zeros_like(g), "compressed": c["compressed"][p]}
                      for g, c in zip(grads, chunks)]
                b = hp.Batch("tbq", ts, threshold=tau)
            else:
                grads = W.normal_set(self.sizes, dev, p + 1, sigma=1e-3)
                ts = [{"gradient": g, "momentum": torch.zeros_like(g), "accumulator": torch.zeros_like(g),
                       "compressed": c["compressed"][p]} for g, c in zip(grads, chunks)]
                b = hp.Batch("dgc", ts, momentum_factor=0.9, ratio=ratio)
            b.encode()
            torch.cuda.synchronize()
            b.close()
            del grads, ts
        self.chunks = chunks
        self.mb = hp.MergeBatch(self.alg, chunks, threshold=tau, ratio=ratio)
        agg_bytes = 4.0 if self.aggregate else 0.0
        if self.alg == "tbq":
            self.enc_bytes, self.dec_bytes = 0.25 * self.npeers + agg_bytes + 8.25, 0.0
            self.dominant_kernel, self.dominant_bytes = "dense_merge_kernel", self.enc_bytes
        else:
            self.enc_bytes, self.dec_bytes = 8.0 + agg_bytes, 0.0  # + 8*(P*rho + rho'), added after the run
            self.dominant_kernel, self.dominant_bytes = "sparse_merge_kernel", 8.0 + agg_bytes

    def step(self, ev=None):
        if ev is not None and self.alg == "tbq":
            ev[0].record()
            self.mb.run()
            ev[1].record()
        elif ev is not None:
            self.mb.run_phase(0)
            ev[0].record()
            self.mb.run_phase(1)
            ev[1].record()
            self.mb.run_phase(2)
        else:
            self.mb.run()

    def density(self):
        import torch

        nin = sum(int(p[:4].view(torch.int32).item()) for c in self.chunks for p in c["compressed"])
        nout = sum(int(c["out_compressed"][:4].view(torch.int32).item()) for c in self.chunks)
        return nin / self.elements, nout / self.elements

    def close(self):
        self.mb.close()
        self.chunks = []


class CompllWorkload:
    """The in-tree CompLL operator (bit width 2, 10-byte header) on the largest VGG19
    tensor through the per-tensor entry points."""

    def __init__(self, name, n, bitwidth=2, generated=False):
        self.name, self.sizes, self.elements, self.b, self.generated = name, [n], n, bitwidth, generated
        self.enc_bytes, self.dec_bytes = 8.0 + bitwidth / 8.0, 4.0 + bitwidth / 8.0
        self.dominant_kernel, self.dominant_bytes = "compll_quant_kernel", 8.0 + bitwidth / 8.0

    def setup(self, dev):
        import torch

        import hipress_amd as hp
        from hipress_amd import workloads as W

        self.hp = hp
        self.g = W.normal_set(self.sizes, dev, 0, sigma=1e-3)[0]
        self.u = W.uniform_set(self.sizes, dev, 1000)[0]
        self.pay = torch.zeros(hp.compll_payload_bytes(self.elements, self.b), dtype=torch.uint8, device=dev)
        self.out = torch.empty(self.elements, device=dev)
        if self.generated:
            from hipress_amd.compll import runtime

            self.gen = runtime.load()

    def step(self, ev=None):
        if self.generated:  # the same operator, generated from its program in the CompLL language
            self.gen.MinMaxQuantEncode(self.g, self.pay, self.b, uniform=self.u)
            self.gen.MinMaxQuantDecode(self.pay, self.out)
        else:
            self.hp.compll_terngrad_encode(self.g, self.u, self.pay, self.b)
            self.hp.compll_terngrad_decode(self.pay, self.out)

    def close(self):
        self.g = self.u = self.pay = self.out = None


class GeneratedTbqWorkload:
    """The error-feedback threshold quantiser generated from its CompLL program (one fused
    sweep for codes and residual) and its decoder, or the hand-written TBQ operator through
    the same per-tensor entry points, on the largest VGG19 tensor."""

    def __init__(self, name, n, generated):
        self.name, self.sizes, self.elements, self.generated = name, [n], n, generated
        self.enc_bytes, self.dec_bytes = 12.25, 4.25
        self.dominant_kernel, self.dominant_bytes = ("map_fused_kernel" if generated else "tbq_encode_kernel"), 12.25

    def setup(self, dev):
        import torch

        import hipress_amd as hp
        from hipress_amd import workloads as W
        from hipress_amd.compll import runtime

        self.hp, self.gen = hp, runtime.load()
        self.g = W.normal_set(self.sizes, dev, 0, sigma=0.02)[0]
        self.r = torch.zeros(self.elements, device=dev)
        nbytes = hp.tbq_payload_bytes(self.elements) if not self.generated else 4 + (2 * self.elements + 7) // 8
        self.pay = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        self.out = torch.empty(self.elements, device=dev)

    def step(self, ev=None):
        if self.generated:
            self.gen.ThresholdFeedbackEncode(self.g, self.r, self.pay, 0.05)
            self.gen.ThresholdTernaryDecode(self.pay, self.out)
        else:
            self.hp.tbq_encode(self.g, self.r, self.pay, 0.05)
            self.hp.tbq_decode(self.pay, self.out)

    def close(self):
        self.g = self.r = self.pay = self.out = None


def make_workload(name):
    from hipress_amd import workloads as W

    vgg, rn, bert = W.vgg19_sizes(), W.resnet50_sizes(), W.bert_large_sizes()
    if name == "onebit_vgg19":
        return SetWorkload(name, "onebit", vgg, "vgg", {}, 12.125, 4.125, 2, "onebit_quant_kernel", 12.125, nphases=3)
    if name == "onebit_deferred_vgg19":
        return SetWorkload(name, "onebit_deferred", vgg, "vgg", {}, 12.125, 4.125, 0, "onebit_deferred_kernel", 12.125, nphases=2)
    if name == "tbq_vgg19":
        return SetWorkload(name, "tbq", vgg, "vgg", {"threshold": 0.05}, 12.25, 4.25, 0, "tbq_encode_kernel", 12.25)
    if name == "terngrad_vgg19":
        return SetWorkload(name, "terngrad", vgg, "vgg", {"bucket": 512}, 8.2578, 4.2578, 0, "terngrad_encode_kernel", 8.2578)
    if name == "dgc_vgg19":
        return SetWorkload(name, "dgc", vgg, "vgg", {"momentum_factor": 0.9, "ratio": 0.001}, 20.0, 4.0, 0,
                           "sparse_accum_kernel", 20.0, nphases=7)
    if name == "graddrop_vgg19":
        return SetWorkload(name, "graddrop", vgg, "vgg", {"ratio": 0.01}, 12.0, 4.0, 0, "sparse_accum_kernel", 12.0, nphases=7)
    if name == "tbq_262144":
        return SetWorkload(name, "tbq", [262144], "n0.02", {"threshold": 0.05}, 12.25, 4.25, 0, "tbq_encode_kernel", 12.25)
    if name == "tbq_262144_graph":
        return SetWorkload(name, "tbq", [262144], "n0.02", {"threshold": 0.05}, 12.25, 4.25, 0, "tbq_encode_kernel", 12.25,
                           graph=True)
    if name == "tbq_262144_x512":
        return SetWorkload(name, "tbq", [262144] * 512, "n0.02", {"threshold": 0.05}, 12.25, 4.25, 0, "tbq_encode_kernel", 12.25)
    if name == "terngrad_resnet50":
        return SetWorkload(name, "terngrad", rn, "heavy", {"bucket": 512}, 8.2578, 4.2578, 0, "terngrad_encode_kernel",
                           8.2578, rotate=4)
    if name == "dgc_bert_large":
        return SetWorkload(name, "dgc", bert, "n1e-3", {"momentum_factor": 0.9, "ratio": 0.001}, 20.0, 4.0, 0,
                           "sparse_accum_kernel", 20.0, nphases=7)
    if name == "graddrop_bert_large":
        return SetWorkload(name, "graddrop", bert, "n1e-3", {"ratio": 0.01}, 12.0, 4.0, 0, "sparse_accum_kernel", 12.0, nphases=7)
    if name == "compll_b2_fc6":
        return CompllWorkload(name, max(vgg))
    if name == "compll_generated_b2_fc6":
        return CompllWorkload(name, max(vgg), generated=True)
    if name == "tbq_fc6":
        return GeneratedTbqWorkload(name, max(vgg), generated=False)
    if name == "tbq_generated_fc6":
        return GeneratedTbqWorkload(name, max(vgg), generated=True)
    if name == "merge_tbq_vgg19":
        return MergeWorkload(name, "tbq", W.chunk_sizes(vgg))
    if name == "merge_dgc_vgg19":
        return MergeWorkload(name, "dgc", W.chunk_sizes(vgg))
    if name == "merge_tbq_vgg19_payload_only":
        return MergeWorkload(name, "tbq", W.chunk_sizes(vgg), aggregate=False)
    if name == "merge_dgc_vgg19_payload_only":
        return MergeWorkload(name, "dgc", W.chunk_sizes(vgg), aggregate=False)
    raise SystemExit(f"unknown workload {name}")


ALL_WORKLOADS = [
    "onebit_vgg19", "onebit_deferred_vgg19", "tbq_vgg19", "terngrad_vgg19", "dgc_vgg19", "graddrop_vgg19", "tbq_262144", "tbq_262144_x512",
    "terngrad_resnet50", "dgc_bert_large", "graddrop_bert_large", "merge_tbq_vgg19", "merge_dgc_vgg19", "compll_b2_fc6",
    "compll_generated_b2_fc6", "tbq_fc6", "tbq_generated_fc6", "merge_tbq_vgg19_payload_only", "merge_dgc_vgg19_payload_only",
]


def measure(name, steps, warmup):
    import torch

    dev = torch.device("cuda:0")
    w = make_workload(name)
    w.setup(dev)
    for _ in range(warmup):
        w.step()
    evs = _events(steps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        w.step(evs[i])
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    enc_b, dec_b = w.enc_bytes, w.dec_bytes
    dom_b = w.dominant_bytes
    extra = {}
    if isinstance(w, SetWorkload) and w.alg in ("dgc", "graddrop"):
        rho = w.density()
        enc_b += 8 * rho
        dec_b += 8 * rho
        extra["density"] = rho
    if isinstance(w, MergeWorkload) and w.alg == "dgc":
        rin, rout = w.density()
        enc_b += 8 * (rin + rout)
        extra["density_in"], extra["density_out"] = rin, rout
    try:
        dom_ms = sum(a.elapsed_time(b) for a, b in evs) / steps
    except Exception:
        dom_ms = None  # the events were never recorded (no bracketed kernel for this workload)
    gbs = 4.0 * w.elements * steps / elapsed / 1e9
    alg_gbs = (enc_b + dec_b) * w.elements * steps / elapsed / 1e9
    res = {
        "workload": name,
        "value": gbs,
        "ms_per_step": elapsed / steps * 1e3,
        "elements": w.elements,
        "tensors": len(w.sizes),
        "algorithmic_bytes_per_element": enc_b + dec_b,
        "pct_of_hbm_roofline": 100.0 * alg_gbs / HBM_PEAK_GBS,
        **extra,
    }
    if dom_ms:
        ach = dom_b * w.elements / (dom_ms * 1e-3) / 1e9
        res["roofline"] = {"bound": "hbm", "kernel": w.dominant_kernel, "achieved": ach, "peak": HBM_PEAK_GBS,
                           "unit": "GB/s", "frac": ach / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC.get(name),
                           "kernel_ms": dom_ms, "algorithmic_bytes_per_launch": dom_b * w.elements}
    w.close()
    del w
    torch.cuda.empty_cache()
    return res


def cpu_baseline(budget_s=12.0):
    """The scalar CPU oracle (one thread, the execution model of the reference's
    registered CPU operator) on the headline workload: onebit encode+decode over the
    whole VGG19 set, same seeded values, repeated until the budget is used.  The same
    source built with OpenMP is timed beside it on all host cores (`all_cores`)."""
    import numpy as np
    import torch

    import oracle
    from hipress_amd import workloads as W

    sizes = W.vgg19_sizes()
    grads = W.normal_set(sizes, torch.device("cuda:0"), 0, log_sigma_range=(-4.0, -2.0))
    host = [g.cpu().numpy() for g in grads]
    del grads
    outs = [np.empty(n, np.float32) for n in sizes]
    pays = [np.zeros(oracle.onebit_payload_bytes(n), np.uint8) for n in sizes]
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)

    def run(L, budget, max_passes):
        res = [np.zeros(n, np.float32) for n in sizes]
        passes, t0 = 0, time.perf_counter()
        while True:
            for g, r, p, o in zip(host, res, pays, outs):
                L.hpo_onebit_encode(vp(g), vp(r), g.size, vp(p))
                L.hpo_onebit_decode(vp(p), vp(o), g.size)
            passes += 1
            el = time.perf_counter() - t0
            if el >= budget or passes >= max_passes:
                return passes, el

    passes, el = run(oracle.lib(), budget_s, 20)
    out = {"value": 4.0 * sum(sizes) * passes / el / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
           "sample": f"onebit encode+decode over the whole VGG19 set ({sum(sizes):,} elements), {passes} passes, "
                     f"{el:.1f} s, scalar C oracle built with gcc -O2"}
    try:
        Lo = oracle.omp_lib()
        threads = int(Lo.hpo_threads())
        run(Lo, 0.0, 1)  # first touch / thread start-up
        p2, e2 = run(Lo, budget_s / 3, 40)
        out["all_cores"] = {"value": 4.0 * sum(sizes) * p2 / e2 / 1e9, "unit": "GB/s", "cores": threads,
                            "sample": f"same workload, same source built with -fopenmp, {p2} passes, {e2:.1f} s"}
    except Exception as exc:  # the OpenMP build is optional
        out["all_cores"] = {"error": str(exc)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="onebit_vgg19", choices=ALL_WORKLOADS + ["tbq_262144_graph"])
    ap.add_argument("--no-others", action="store_true", help="measure only --workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--others-steps", type=int, default=10)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain 1 GiB device-to-device copy (a kernel of known traffic: 1 GiB read, "
                         "1 GiB written) so that rocprofv3 FETCH_SIZE / WRITE_SIZE can be scaled against it")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py: this build measures one GPU's share of the path; run with --gpus 1 "
                         "(collectives and sharding are not part of it)\n")
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py needs a GPU\n")
        sys.exit(2)
    import hipress_amd  # noqa: F401  (raises if libhipress_amd.so is missing)

    if args.calibrate_copy:
        src = torch.ones(1 << 28, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "torch copy_ of 2**28 fp32", "bytes_read": 4 << 28, "bytes_written": 4 << 28,
                          "launches": args.steps}))
        return

    main_res = measure(args.workload, args.steps, args.warmup)
    others = []
    if not args.no_others:
        for name in ALL_WORKLOADS:
            if name != args.workload:
                others.append(measure(name, args.others_steps, 3))
    line = {
        "metric": "fp32 grad GB/s through encode+decode",
        "value": main_res["value"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": args.workload, "elements": main_res["elements"], "tensors": main_res["tensors"],
                   "algorithmic_bytes_per_element": main_res["algorithmic_bytes_per_element"]},
        "pct_of_hbm_roofline": main_res["pct_of_hbm_roofline"],
        "roofline": {k: v for k, v in main_res.get("roofline", {}).items()},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline()
    if others:
        line["others"] = others
    print(json.dumps(line))


if __name__ == "__main__":
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    main()
