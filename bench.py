#!/usr/bin/env python3
"""Throughput of the gradient-compression hot path on one MI355X.

A step is one pass of encode followed by decode over a whole synthetic gradient
set that is already resident in HBM, through the calls a user of the library
makes (`Batch.encode()`, `Batch.decode()`, `MergeBatch.run()`).  The headline
line is TBQ over the VGG19 gradient set; `--workload` selects another, and
`others` in the JSON line carries a shorter measurement of every other
compressor / configuration (DGC over the same set first).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-others] [--no-cpu]

Prints ONE compact JSON line (under 4 KB) on stdout; the full per-workload records go to
a JSON file beside the other run outputs (its path is in the line as `detail`) and, one
JSON object per workload, to stderr.  value = 4 * elements * steps / elapsed over
exactly K steps bracketed by device synchronisation, in GB/s of fp32 gradient
through encode+decode; `median_ms_per_step` is the median of the same steps timed
one by one with events in a second run.  `roofline` describes the dominant kernel:
algorithmic bytes per launch over its mean duration against the 8 TB/s HBM peak.
Two durations are carried: `kernel_ms_events`, measured live with events on the
launch stream in a third run that issues the encode sequence launch by launch, and
`kernel_ms_profile`, the kernel's average in the committed rocprofv3 summary of the
same command (profiles/<workload>.md).  `frac` and `achieved` use the profile's
duration when the summary exists (anyone can re-derive them from the committed
table; `kernel_ms_source` names the file), the live one otherwise; `frac_events` is
always the live figure.  `traffic` is the HBM bytes per launch from the same
summary's counters and `traffic_ratio` its ratio to the algorithmic bytes.  Every
entry carries `cpu_baseline`: the scalar CPU oracle (one thread, the execution model
of the reference's registered CPU operator) on a bounded sample of the same
tensors, and the same source built with OpenMP on all host cores beside it.
"""
import argparse
import ctypes
import json
import os
import re
import statistics
import subprocess
import sys
import time

HBM_PEAK_GBS = 8000.0
ROOT = os.path.dirname(os.path.abspath(__file__))


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` as the rocprofv3 summary of this workload holds them
    (profiles/<workload>.md, table "HBM traffic per dispatch": (2.0 x FETCH_SIZE + 1.0 x
    WRITE_SIZE) x 1024, the factors being what the same counters read for a plain 1 GiB
    copy), or None when no summary with counters exists.  -> (bytes, source path)"""
    path = os.path.join(ROOT, "profiles", workload + ".md")
    try:
        text = open(path).read()
    except OSError:
        return None, None
    sect = text.split("HBM traffic per dispatch", 1)
    if len(sect) < 2:
        return None, None
    for line in sect[1].splitlines():
        cells = [c.strip() for c in line.split("|")]
        if len(cells) >= 6 and kernel in cells[1]:
            try:
                return int(cells[5].replace(",", "")), os.path.relpath(path, ROOT)
            except ValueError:
                return None, None
    return None, None


def profile_kernel_us(workload, kernel):
    """Average duration in microseconds of `kernel` in the "Kernel statistics" table of
    profiles/<workload>.md (rocprofv3 --kernel-trace --stats of `bench.py --workload
    <workload>`): the first row of that table whose name holds `kernel`, or None when there
    is no summary or no such row.  -> (microseconds, source path)"""
    path = os.path.join(ROOT, "profiles", workload + ".md")
    try:
        text = open(path).read()
    except OSError:
        return None, None
    sect = text.split("Kernel statistics", 1)
    if len(sect) < 2:
        return None, None
    for line in sect[1].split("HBM traffic per dispatch", 1)[0].splitlines():
        cells = [c.strip() for c in line.split("|")]
        if len(cells) >= 6 and kernel in cells[1]:
            try:
                return float(cells[3].replace(",", "")), os.path.relpath(path, ROOT)
            except ValueError:
                return None, None
    return None, None


def launches_per_step(w):
    """Launches of the dominant kernel in one step: the library issues a very long accumulate
    pass in equal parts of at most 49,152 tiles; everything else is one launch."""
    if w.dominant_kernel == "sparse_accum_kernel":
        return -(-sum(-(-n // 4096) for n in w.sizes) // 49152)
    return 1


def roofline_of(workload, kernel, bytes_per_launch, launches, events_ms):
    """The roofline record of one workload's dominant kernel.  bytes_per_launch: algorithmic
    bytes one launch moves; events_ms: its live mean duration per launch (None when the
    workload's calls do not expose the kernel on its own)."""
    prof_us, prof_src = profile_kernel_us(workload, kernel)
    traffic, traffic_src = measured_traffic(workload, kernel)
    ms = prof_us * 1e-3 if prof_us else events_ms
    if not ms:
        return None
    ach = bytes_per_launch / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "kernel": kernel, "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": ach / HBM_PEAK_GBS, "traffic": traffic,
            "traffic_ratio": traffic / bytes_per_launch if traffic else None, "traffic_source": traffic_src,
            "kernel_ms_source": prof_src if prof_us else "hipEvent",
            "kernel_ms_profile": prof_us * 1e-3 if prof_us else None, "kernel_ms_events": events_ms,
            "frac_events": bytes_per_launch / (events_ms * 1e-3) / 1e9 / HBM_PEAK_GBS if events_ms else None,
            "launches_per_step": launches, "algorithmic_bytes_per_launch": bytes_per_launch}


def _events(n):
    import torch

    return [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]


CPU_TENSOR_CAP = 4 << 20    # elements taken from the front of any one tensor for the CPU sample
CPU_SAMPLE_CAP = 24 << 20   # elements per CPU pass


def _vp(a):
    return a.ctypes.data_as(ctypes.c_void_p)


class CpuJob:
    """One pass of a workload's CPU restatement over a bounded sample; run(L) executes it
    with oracle build L (scalar or OpenMP) and carries state from pass to pass."""

    def __init__(self, elements, sample, run):
        self.elements, self.sample, self.run = elements, sample, run


def _sample_front(sizes):
    """The front of each tensor (at most CPU_TENSOR_CAP elements), tensors taken in order
    until CPU_SAMPLE_CAP elements are reached: [(tensor index, elements)]."""
    picks, total = [], 0
    for i, n in enumerate(sizes):
        if total >= CPU_SAMPLE_CAP:
            break
        k = min(n, CPU_TENSOR_CAP, CPU_SAMPLE_CAP - total)
        if k > 0:
            picks.append((i, k))
            total += k
    return picks, total


class SetWorkload:
    """encode+decode of one compressor over a list of tensor sizes through a Batch."""

    def __init__(self, name, alg, sizes, data, params, enc_bytes, dec_bytes, dominant_phase, dominant_kernel,
                 dominant_bytes, rotate=1, nphases=1, seeded=False):
        self.name, self.alg, self.sizes, self.data, self.params = name, alg, sizes, data, params
        self.seeded = seeded  # terngrad: no noise tensors, the kernels draw from a seed that changes every step
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
            if self.alg == "terngrad" and not self.seeded:
                for t, u in zip(ts, W.uniform_set(self.sizes, dev, 1000 + seed)):
                    t["uniform"] = u
            self.tensors.append(ts)
            self.batches.append(hp.Batch(self.alg, ts, **self.params))
        self.k = 0

    def step(self, ev=None):
        b = self.batches[self.k % self.rotate]
        self.k += 1
        if self.seeded:
            if ev is not None:
                ev[0].record()
            b.encode(seed=self.k)
            if ev is not None:
                ev[1].record()
        elif ev is None:
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

    def cpu_job(self):
        """The same compressor in the CPU oracle over the front of this set's tensors (the
        values the GPU run used, copied from the device)."""
        import numpy as np

        import oracle

        picks, total = _sample_front(self.sizes)
        ts = self.tensors[0]
        g = [ts[i]["gradient"][:k].cpu().numpy() for i, k in picks]
        u = None
        if self.alg == "terngrad":
            u = [np.empty(k, np.float32) if self.seeded else ts[i]["uniform"][:k].cpu().numpy() for i, k in picks]
        seeded = self.seeded
        zeros = lambda: [np.zeros(k, np.float32) for _, k in picks]
        s0, s1 = zeros(), zeros()
        out = [np.empty(k, np.float32) for _, k in picks]
        alg, pr = self.alg, self.params
        ratio = pr.get("ratio", 0.001)
        nbytes = {"tbq": oracle.tbq_payload_bytes, "onebit": oracle.onebit_payload_bytes,
                  "onebit_deferred": oracle.onebit_payload_bytes,
                  "terngrad": lambda n: oracle.terngrad_payload_bytes(n, pr.get("bucket", 512)),
                  "dgc": lambda n: oracle.sparse_payload_bytes(n, ratio),
                  "graddrop": lambda n: oracle.sparse_payload_bytes(n, ratio)}[alg]
        pay = [np.zeros(nbytes(k), np.uint8) for _, k in picks]

        def run(L):
            for j, (_, k) in enumerate(picks):
                if alg == "tbq":
                    L.hpo_tbq_encode(_vp(g[j]), _vp(s0[j]), k, _vp(pay[j]), pr["threshold"])
                    L.hpo_tbq_decode(_vp(pay[j]), _vp(out[j]), k)
                elif alg in ("onebit", "onebit_deferred"):
                    L.hpo_onebit_encode(_vp(g[j]), _vp(s0[j]), k, _vp(pay[j]))
                    L.hpo_onebit_decode(_vp(pay[j]), _vp(out[j]), k)
                elif alg == "terngrad":
                    if seeded:  # the draws are part of the operator
                        L.hpo_uniform_draws(1, j, _vp(u[j]), k)
                    L.hpo_terngrad_encode(_vp(g[j]), _vp(u[j]), k, _vp(pay[j]), pr.get("bucket", 512))
                    L.hpo_terngrad_decode(_vp(pay[j]), _vp(out[j]), k)
                elif alg == "dgc":
                    L.hpo_dgc_encode(_vp(g[j]), _vp(s0[j]), _vp(s1[j]), k, _vp(pay[j]), pr["momentum_factor"], ratio)
                    L.hpo_sparse_decode(_vp(pay[j]), _vp(out[j]), k)
                else:
                    L.hpo_graddrop_encode(_vp(g[j]), _vp(s1[j]), k, _vp(pay[j]), ratio)
                    L.hpo_sparse_decode(_vp(pay[j]), _vp(out[j]), k)

        what = (f"{alg} encode+decode over the first <= {CPU_TENSOR_CAP:,} elements of "
                f"{len(picks)} of the set's {len(self.sizes)} tensors ({total:,} elements per pass)")
        return CpuJob(total, what, run)

    def density(self):
        """Measured fraction of elements kept (sparse compressors)."""
        import torch

        nnz = 0
        for t in self.tensors[0]:
            nnz += int(t["compressed"][:4].view(torch.int32).item())
        return nnz / self.elements

    def close(self):
        for b in self.batches:
            b.close()
        self.batches, self.tensors = [], []


class PlannedWorkload(SetWorkload):
    """The VGG19 set as the planner cuts it for `nodes` nodes with the models measured on
    MI355X: gradients the plan marks `n` are left out, the others are compressed partition
    by partition (hipress_amd.PlannedSet), all partitions in one launch sequence."""

    def __init__(self, name, alg, params, enc_bytes, dec_bytes, dominant_kernel, nodes=4):
        from hipress_amd import planner
        from hipress_amd import workloads as W

        self.full_sizes = W.vgg19_sizes()
        names = [f"g{i}" for i in range(len(self.full_sizes))]
        self.plan = [planner.parse_plan_line(l) for l in
                     planner.Planner.from_measured(alg, nodes).plan(zip(names, self.full_sizes), "PS")]
        sizes = [ln for _, size, c, k in self.plan if c for _, ln in planner.partition_bounds(size, k)]
        super().__init__(name, alg, sizes, "vgg", params, enc_bytes, dec_bytes, 0, dominant_kernel, enc_bytes)

    def setup(self, dev):
        import hipress_amd as hp
        from hipress_amd import workloads as W

        grads = W.normal_set(self.full_sizes, dev, 0, log_sigma_range=(-4.0, -2.0))
        self.planned = hp.PlannedSet(self.alg, self.plan, {p[0]: g for p, g in zip(self.plan, grads)}, **self.params)
        self.batches = [self.planned._batch]
        self.tensors = [self.planned._batch._keep]
        self.k = 0

    def close(self):
        self.planned.close()
        self.batches, self.tensors = [], []


class MergeWorkload:
    """Decode-and-merge of 8 peer payloads per 4 MB chunk of the VGG19 set, with the
    fused re-encode for the next hop."""

    def __init__(self, name, alg, sizes, npeers=8, aggregate=True, local=False):
        self.name, self.alg, self.sizes, self.npeers = name, alg, sizes, npeers
        self.aggregate = aggregate  # False: only the re-encoded payload is produced (no fp32 sum written)
        self.local = local          # True: every sum starts from the aggregator's own fp32 gradient (a ring hop)
        self.elements = sum(sizes)
        self.dominant_phase = 0
        self.nphases = 1
        self.rotate = 1
        agg_bytes = (4.0 if aggregate else 0.0) + (4.0 if local else 0.0)
        if alg == "tbq":
            self.enc_bytes, self.dec_bytes = 0.25 * npeers + agg_bytes + 8.25, 0.0
            self.dominant_kernel, self.dominant_bytes = "dense_merge_kernel", self.enc_bytes
        elif alg == "terngrad":  # sum only: TernGrad keeps no state to re-encode against (buckets of 512)
            self.enc_bytes, self.dec_bytes = (0.25 + 4.0 / 512) * npeers + agg_bytes, 0.0
            self.dominant_kernel, self.dominant_bytes = "dense_merge_kernel", self.enc_bytes
        else:
            self.enc_bytes, self.dec_bytes = 8.0 + agg_bytes, 0.0  # + 8*(P*rho + rho'), added after the run
            self.dominant_kernel, self.dominant_bytes = "sparse_merge_kernel", 8.0 + agg_bytes

    def setup(self, dev):
        import torch

        import hipress_amd as hp
        from hipress_amd import workloads as W

        tau, ratio = 0.05, 0.001
        self.ratio = ratio
        chunks = []
        for n in self.sizes:
            nb = {"tbq": hp.tbq_payload_bytes(n), "terngrad": hp.terngrad_payload_bytes(n, 512)}.get(self.alg) or hp.dgc_payload_bytes(n, ratio)
            c = {"compressed": [torch.zeros(nb, dtype=torch.uint8, device=dev) for _ in range(self.npeers)],
                 "aggregate": torch.empty(n, device=dev) if self.aggregate else None}
            if self.alg != "terngrad":
                c["state"], c["out_compressed"] = torch.zeros(n, device=dev), torch.zeros(nb, dtype=torch.uint8, device=dev)
            chunks.append(c)
        if self.local:
            for c, g in zip(chunks, W.normal_set(self.sizes, dev, 0, sigma=0.02 if self.alg == "tbq" else 1e-3)):
                c["local"] = g
        # peer p's payloads come from that peer's own gradients (seed p) through the encoders
        for p in range(self.npeers):
            if self.alg == "tbq":
                grads = W.normal_set(self.sizes, dev, p + 1, sigma=0.02)
                ts = [{"gradient": g, "residual": torch.zeros_like(g), "compressed": c["compressed"][p]}
                      for g, c in zip(grads, chunks)]
                b = hp.Batch("tbq", ts, threshold=tau)
            elif self.alg == "terngrad":
                grads = W.normal_set(self.sizes, dev, p + 1, sigma=1e-3)
                ts = [{"gradient": g, "compressed": c["compressed"][p]} for g, c in zip(grads, chunks)]
                b = hp.Batch("terngrad", ts, bucket=512)  # no noise tensors: the peers draw from seed p
            else:
                grads = W.normal_set(self.sizes, dev, p + 1, sigma=1e-3)
                ts = [{"gradient": g, "momentum": torch.zeros_like(g), "accumulator": torch.zeros_like(g),
                       "compressed": c["compressed"][p]} for g, c in zip(grads, chunks)]
                b = hp.Batch("dgc", ts, momentum_factor=0.9, ratio=ratio)
            b.encode(seed=p) if self.alg == "terngrad" else b.encode()
            torch.cuda.synchronize()
            b.close()
            del grads, ts
        self.chunks = chunks
        self.mb = hp.MergeBatch(self.alg, chunks, threshold=tau, bucket=512, ratio=ratio)

    def step(self, ev=None):
        if ev is not None and self.alg in ("tbq", "terngrad"):
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

    def cpu_job(self):
        """decode-and-merge + re-encode of four full-sized chunks in the CPU oracle, on the very
        peer payloads the GPU run merges."""
        import numpy as np

        # four full-sized chunks: the set's first chunks are a few thousand elements each, which
        # times call overhead rather than the merge
        order = sorted(range(len(self.sizes)), key=lambda i: (-self.sizes[i], i))[:4]
        P, alg, ratio = self.npeers, self.alg, self.ratio
        jobs = []
        for i in sorted(order):
            n = self.sizes[i]
            pays = [p.cpu().numpy() for p in self.chunks[i]["compressed"]]
            arr = (ctypes.c_void_p * P)(*[p.ctypes.data for p in pays])
            loc = self.chunks[i]["local"].cpu().numpy() if self.local else None
            out_bytes = self.chunks[i]["out_compressed"].numel() if "out_compressed" in self.chunks[i] else 0
            jobs.append((n, pays, arr, np.empty(n, np.float32), np.zeros(n, np.float32), np.zeros(out_bytes, np.uint8), loc))
        total = sum(j[0] for j in jobs)

        def run(L):
            for n, _, arr, agg, state, outp, loc in jobs:
                lp = _vp(loc) if loc is not None else None
                if alg == "tbq":
                    L.hpo_tbq_decode_merge_local(arr, P, lp, _vp(agg), n, _vp(state), _vp(outp), 0.05)
                elif alg == "terngrad":
                    L.hpo_terngrad_decode_merge_local(arr, P, lp, _vp(agg), n)
                else:
                    L.hpo_sparse_decode_merge_local(arr, P, lp, _vp(agg), n, _vp(state), _vp(outp), ratio)

        what = (f"{alg} decode-and-merge of {P} peers{'' if alg == 'terngrad' else ' + re-encode'} over the {len(jobs)} largest of "
                f"{len(self.sizes)} chunks ({total:,} elements per pass)")
        return CpuJob(total, what, run)

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
        self.dominant_kernel = "map_packed_kernel" if generated else "compll_quant_kernel"
        self.dominant_bytes = 8.0 + bitwidth / 8.0

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

    def cpu_job(self):
        import numpy as np

        k = min(self.elements, 4 * CPU_TENSOR_CAP)
        g, u = self.g[:k].cpu().numpy(), self.u[:k].cpu().numpy()
        pay = np.zeros(10 + (k * self.b + 7) // 8, np.uint8)
        out = np.empty(k, np.float32)
        b = self.b

        def run(L):
            L.hpo_compll_encode(_vp(g), _vp(u), k, _vp(pay), b)
            L.hpo_compll_decode(_vp(pay), pay.size, _vp(out), k)

        return CpuJob(k, f"min/max {b}-bit quantiser encode+decode over the first {k:,} elements of the tensor", run)

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

    def cpu_job(self):
        import numpy as np

        import oracle

        k = min(self.elements, 4 * CPU_TENSOR_CAP)
        g, r = self.g[:k].cpu().numpy(), np.zeros(k, np.float32)
        pay, out = np.zeros(oracle.tbq_payload_bytes(k), np.uint8), np.empty(k, np.float32)

        def run(L):
            L.hpo_tbq_encode(_vp(g), _vp(r), k, _vp(pay), 0.05)
            L.hpo_tbq_decode(_vp(pay), _vp(out), k)

        return CpuJob(k, f"tbq encode+decode over the first {k:,} elements of the tensor", run)

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
    if name == "terngrad_seeded_vgg19":
        # no noise tensor: 4 bytes per element fewer for the encoder to read
        return SetWorkload(name, "terngrad", vgg, "vgg", {"bucket": 512}, 4.2578, 4.2578, 0, "terngrad_encode_kernel", 4.2578,
                           seeded=True)
    if name == "dgc_vgg19":
        return SetWorkload(name, "dgc", vgg, "vgg", {"momentum_factor": 0.9, "ratio": 0.001}, 20.0, 4.0, 0,
                           "sparse_accum_kernel", 20.0, nphases=7)
    if name == "graddrop_vgg19":
        return SetWorkload(name, "graddrop", vgg, "vgg", {"ratio": 0.01}, 12.0, 4.0, 0, "sparse_accum_kernel", 12.0, nphases=7)
    if name == "tbq_262144":
        # 128 buffer sets in turn (400 MB in all): one 3 MB set alone would be served from the caches
        return SetWorkload(name, "tbq", [262144], "n0.02", {"threshold": 0.05}, 12.25, 4.25, 0, "tbq_encode_kernel", 12.25,
                           rotate=128)
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
    if name == "tbq_vgg19_planned":
        return PlannedWorkload(name, "tbq", {"threshold": 0.05}, 12.25, 4.25, "tbq_encode_kernel")
    if name == "merge_tbq_vgg19":
        return MergeWorkload(name, "tbq", W.chunk_sizes(vgg))
    if name == "merge_dgc_vgg19":
        return MergeWorkload(name, "dgc", W.chunk_sizes(vgg))
    if name == "merge_terngrad_vgg19":  # the sum alone: TernGrad has no state to re-encode against
        return MergeWorkload(name, "terngrad", W.chunk_sizes(vgg))
    if name == "merge_tbq_vgg19_payload_only":
        return MergeWorkload(name, "tbq", W.chunk_sizes(vgg), aggregate=False)
    if name == "merge_dgc_vgg19_payload_only":
        return MergeWorkload(name, "dgc", W.chunk_sizes(vgg), aggregate=False)
    if name == "hop_tbq_vgg19":  # one hop of a ring: the payload that arrived + the node's own gradient -> the payload to send on
        return MergeWorkload(name, "tbq", W.chunk_sizes(vgg), npeers=1, aggregate=False, local=True)
    raise SystemExit(f"unknown workload {name}")


# the metric's configurations first (VGG19: TBQ, then DGC), then every other compressor / configuration
ALL_WORKLOADS = [
    "tbq_vgg19", "dgc_vgg19", "onebit_vgg19", "terngrad_vgg19", "graddrop_vgg19", "onebit_deferred_vgg19",
    "tbq_262144", "tbq_262144_x512", "terngrad_resnet50", "dgc_bert_large", "graddrop_bert_large",
    "merge_tbq_vgg19", "merge_dgc_vgg19", "compll_b2_fc6", "compll_generated_b2_fc6", "tbq_fc6", "tbq_generated_fc6",
    "merge_tbq_vgg19_payload_only", "merge_dgc_vgg19_payload_only", "tbq_vgg19_planned", "hop_tbq_vgg19",
    "terngrad_seeded_vgg19", "merge_terngrad_vgg19",
]
# any workload with the suffix _graph: the same step captured once into a HIP graph and replayed
EXTRA_WORKLOADS = [w + "_graph" for w in ALL_WORKLOADS]


def cpu_baseline(job, budget_s):
    """Times `job` (a CpuJob) with the scalar oracle for about budget_s seconds (at least one
    pass), then with the OpenMP build of the same source for about half of that."""
    import oracle

    def run(L, budget, max_passes=1000):
        passes, t0 = 0, time.perf_counter()
        while True:
            job.run(L)
            passes += 1
            el = time.perf_counter() - t0
            if el >= budget or passes >= max_passes:
                return passes, el

    passes, el = run(oracle.lib(), budget_s)
    out = {"value": 4.0 * job.elements * passes / el / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
           "sample": f"{job.sample}, {passes} passes, {el:.1f} s, scalar C oracle (gcc -O3, one thread)",
           "sample_short": f"front of the same tensors, {job.elements:,} elements/pass x {passes} passes, {el:.1f} s, scalar C oracle"}
    try:
        Lo = oracle.omp_lib()
        threads = int(Lo.hpo_threads())
        run(Lo, 0.0, 1)  # thread start-up
        p2, e2 = run(Lo, budget_s / 2)
        out["all_cores"] = {"value": 4.0 * job.elements * p2 / e2 / 1e9, "unit": "GB/s", "cores": threads,
                            "sample": f"same sample, same source built with -fopenmp, {p2} passes, {e2:.1f} s"}
    except Exception as exc:  # the OpenMP build is optional
        out["all_cores"] = {"error": str(exc)}
    return out


def c_level_latency():
    """encode+decode of one 262,144-element tensor timed by a small C program straight on the
    C ABI (no Python, no torch between the launches): separates the library's latency from
    the binding's.  Returns the program's JSON or an error note."""
    exe = os.path.join(ROOT, "hipress_amd", "hipress_latency")
    if not os.path.exists(exe):
        return {"error": "hipress_amd/hipress_latency is not built (python -m hipress_amd.build)"}
    try:
        r = subprocess.run([exe, "262144", "2000"], capture_output=True, text=True, timeout=120)
        return json.loads(r.stdout.strip().splitlines()[-1])
    except Exception as exc:
        return {"error": str(exc)}


def _warm_up(w, warmup, min_seconds):
    """At least `warmup` untimed steps, and as many more as it takes to keep the GPU busy for
    min_seconds: after set-up (or a CPU-baseline leg) the GPU has idled and its clocks take
    tens of milliseconds of work to come back, which a handful of sub-millisecond steps is not."""
    import torch

    done, t0 = 0, time.perf_counter()
    while done < warmup or time.perf_counter() - t0 < min_seconds:
        for _ in range(max(1, min(warmup, 10))):
            w.step()
            done += 1
        torch.cuda.synchronize()
    return done, time.perf_counter() - t0


def measure(name, steps, warmup, cpu_budget_s=0.0, min_warmup_s=0.25, min_timed_s=0.0):
    """One workload's record.  The timed region is exactly `steps` steps; with min_timed_s the
    number of steps is raised until the region lasts about that long (judged by the warm-up's
    rate), so that the two synchronisations around it, tens of microseconds, do not decide the
    figure of a workload whose step takes a few microseconds."""
    import torch

    dev = torch.device("cuda:0")
    graph = name.endswith("_graph")
    w = make_workload(name[: -len("_graph")] if graph else name)
    w.setup(dev)
    warm_steps, warm_s = _warm_up(w, warmup, min_warmup_s)
    if min_timed_s > 0 and warm_steps and warm_s > 0:
        steps = max(steps, min(5000, -(-int(min_timed_s * 1e6) // max(1, int(warm_s / warm_steps * 1e6)))))
    captured = None
    if graph:  # one step captured on a side stream; every later step is one graph launch
        side = torch.cuda.Stream()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            captured = torch.cuda.CUDAGraph()
            with torch.cuda.graph(captured, stream=side):
                w.step()
        torch.cuda.synchronize()
        eager_step = w.step
        w.step = lambda ev=None: captured.replay()
        for _ in range(warmup):
            w.step()
    # 1. exactly `steps` steps of the product calls between two synchronisations
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        w.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    # 2. the same steps one by one between events: the median step
    evs = _events(steps)
    for a, b in evs:
        a.record()
        w.step()
        b.record()
    torch.cuda.synchronize()
    median_ms = statistics.median(a.elapsed_time(b) for a, b in evs)
    # 3. the encode sequence launch by launch, the dominant kernel between events
    kev = _events(steps)
    for i in range(steps):
        w.step(kev[i])
    torch.cuda.synchronize()
    try:
        dom_ms = sum(a.elapsed_time(b) for a, b in kev) / steps
    except Exception:
        dom_ms = None  # the events were never recorded (no bracketed kernel for this workload)
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
    gbs = 4.0 * w.elements * steps / elapsed / 1e9
    alg_gbs = (enc_b + dec_b) * w.elements * steps / elapsed / 1e9
    res = {
        "workload": name,
        "steps": steps,
        "warmup_steps_run": warm_steps,
        "value": gbs,
        "ms_per_step": elapsed / steps * 1e3,
        "median_ms_per_step": median_ms,
        "value_at_median": 4.0 * w.elements / (median_ms * 1e-3) / 1e9,
        "elements": w.elements,
        "tensors": len(w.sizes),
        "algorithmic_bytes_per_element": enc_b + dec_b,
        "pct_of_hbm_roofline": 100.0 * alg_gbs / HBM_PEAK_GBS,
        **extra,
    }
    launches = launches_per_step(w)
    roof = roofline_of(name[: -len("_graph")] if graph else name, w.dominant_kernel,
                       dom_b * w.elements / launches, launches, dom_ms / launches if dom_ms else None)
    if roof:
        res["roofline"] = roof
    if name == "tbq_262144":
        res["c_level"] = c_level_latency()
    if cpu_budget_s > 0 and hasattr(w, "cpu_job") and not graph:
        job = w.cpu_job()
        torch.cuda.synchronize()
        res["cpu_baseline"] = cpu_baseline(job, cpu_budget_s)
        del job
    if graph:
        w.step = eager_step
        captured = None
    w.close()
    del w
    torch.cuda.empty_cache()
    return res


METRIC = "fp32 grad GB/s through encode+decode, % of HBM roofline; VGG19 TBQ, DGC"
DETAIL_PATH = os.path.join("gpurun_out", "bench_detail.json")
MAX_LINE_BYTES = 4096  # the final stdout line stays below this, whatever the number of workloads


def _sig(x, digits=4):
    """x rounded to `digits` significant digits (None stays None): keeps the line short."""
    if x is None or isinstance(x, (str, bool)):
        return x
    return float(f"{x:.{digits}g}")


def _short_roofline(r):
    keep = ("bound", "kernel", "achieved", "peak", "unit", "frac", "traffic", "traffic_ratio", "kernel_ms_source",
            "kernel_ms_profile", "kernel_ms_events", "frac_events", "launches_per_step", "algorithmic_bytes_per_launch")
    out = {k: r.get(k) for k in keep}
    for k in ("achieved", "frac", "traffic_ratio", "kernel_ms_profile", "kernel_ms_events", "frac_events"):
        out[k] = _sig(out[k])
    out["algorithmic_bytes_per_launch"] = int(out["algorithmic_bytes_per_launch"])
    return out


def _short_cpu(c):
    """cpu_baseline without prose beyond one short `sample` string."""
    out = {"value": _sig(c["value"]), "unit": c["unit"], "cores": c["cores"], "kind": c["kind"],
           "sample": c.get("sample_short", c["sample"])[:120]}
    ac = c.get("all_cores") or {}
    if "value" in ac:
        out["all_cores"] = {"value": _sig(ac["value"]), "cores": ac["cores"]}
    return out


def compact_line(main_res, others, steps, warmup):
    """The one JSON object bench.py prints on stdout: the headline workload in full (metric,
    value, timing, config, roofline, cpu_baseline) and every other workload reduced to
    {workload, value, ms_per_step, pct, frac, cpu1, cpuN}.  Stays below MAX_LINE_BYTES."""
    line = {
        "metric": METRIC,
        "value": _sig(main_res["value"], 6),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": _sig(main_res["ms_per_step"], 6),
        "median_ms_per_step": _sig(main_res["median_ms_per_step"], 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": main_res["workload"], "elements": main_res["elements"], "tensors": main_res["tensors"],
                   "algorithmic_bytes_per_element": _sig(main_res["algorithmic_bytes_per_element"], 6)},
        "pct_of_hbm_roofline": _sig(main_res["pct_of_hbm_roofline"]),
    }
    if main_res.get("roofline"):
        line["roofline"] = _short_roofline(main_res["roofline"])
    if "cpu_baseline" in main_res:
        line["cpu_baseline"] = _short_cpu(main_res["cpu_baseline"])
    if "density" in main_res:
        line["density"] = _sig(main_res["density"])
    line["detail"] = DETAIL_PATH
    if others:
        # cpu1 / cpuN of every entry: GB/s of the scalar oracle on one thread / on this many threads
        cores = [(r.get("cpu_baseline") or {}).get("all_cores", {}).get("cores") for r in others]
        line["others_cpu_cores"] = {"cpu1": 1, "cpuN": next((c for c in cores if c), None)}
        line["others"] = []
        for r in others:
            cpu = r.get("cpu_baseline") or {}
            line["others"].append({"workload": r["workload"], "value": _sig(r["value"]), "ms_per_step": _sig(r["ms_per_step"]),
                                   "pct": _sig(r["pct_of_hbm_roofline"], 3), "frac": _sig((r.get("roofline") or {}).get("frac"), 3),
                                   "cpu1": _sig(cpu.get("value"), 3), "cpuN": _sig((cpu.get("all_cores") or {}).get("value"), 3)})
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="tbq_vgg19", choices=ALL_WORKLOADS + EXTRA_WORKLOADS)
    ap.add_argument("--no-others", action="store_true", help="measure only --workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--others-steps", type=int, default=10)
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="one-thread CPU budget of the headline workload")
    ap.add_argument("--others-cpu-seconds", type=float, default=2.0, help="one-thread CPU budget of every other workload")
    ap.add_argument("--min-warmup-ms", type=float, default=250.0,
                    help="keep warming up (beyond --warmup steps) until the GPU has been busy this long")
    ap.add_argument("--others-min-timed-ms", type=float, default=2.0,
                    help="every other workload is timed over at least --others-steps steps and about this long "
                         "(the headline over exactly --steps)")
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

    def record(r):  # the full record of each workload goes to stderr as soon as it is measured
        sys.stderr.write(json.dumps(r) + "\n")
        sys.stderr.flush()
        return r

    main_res = record(measure(args.workload, args.steps, args.warmup, 0.0 if args.no_cpu else args.cpu_seconds,
                              args.min_warmup_ms * 1e-3))
    others = []
    if not args.no_others:
        for name in ALL_WORKLOADS:
            if name != args.workload:
                others.append(record(measure(name, args.others_steps, 3, 0.0 if args.no_cpu else args.others_cpu_seconds,
                                             args.min_warmup_ms * 1e-3, min_timed_s=args.others_min_timed_ms * 1e-3)))
    line = compact_line(main_res, others, args.steps, args.warmup)
    detail = {"headline": main_res, "others": others}
    try:  # the full records also go to a file next to the other run outputs
        os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
        with open(os.path.join(ROOT, DETAIL_PATH), "w") as f:
            json.dump(detail, f, indent=1)
    except OSError as exc:
        line["detail"] = f"not written: {exc}"
    print(json.dumps(line, separators=(",", ":")), flush=True)


if __name__ == "__main__":
    sys.path.insert(0, ROOT)
    main()
