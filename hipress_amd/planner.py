"""Selective compression and partitioning planner (SeCoPa).

For every gradient of a model the planner decides whether compressing it pays off
and into how many partitions it should be cut, from piecewise-linear cost models
of the synchronisation steps.  It restates the reference planner
(/root/reference/src/SeCoPa/SeCoPa.py:4-113) - same cost formulas, same
tie-breaking, same `name,size,y|n,K` plan lines (SeCoPa.py:139-151) - and adds what
the reference leaves to its users (/root/reference/src/SeCoPa/README.md:14-16):
fitting the encode / decode coefficients from measurements of this library's own
kernels on the GPU at hand.

    python -m hipress_amd.planner --input input.txt --output SeCoPaPlan.txt --topology PS --nnodes 4
    python -m hipress_amd.planner --calibrate tbq ...     # encode/decode/merge models measured on cuda:0
    python -m hipress_amd.planner --measured tbq ...      # the models measured on MI355X that ship with the package
    python -m hipress_amd.planner --calibrate-all out.json   # measure every algorithm, write such a file

Units.  The reference states no unit for its coefficients and no hardware
(SeCoPa.py:25-39; README.md:14 "measured in our local cluster").  Its encode model gives
0.054 for a small tensor and its 4-node gather 0.42 + 2.7e-6 per element: read as
milliseconds these are a 54 us kernel sequence and about 1.5 GB/s per peer, read as
seconds they would be a 54 ms encode of a few kilobytes, so milliseconds is the reading
taken here, and the models measured by `calibrate` are in milliseconds so that they can
stand beside the reference's gather / broadcast / ring-send models, which one GPU cannot
measure and which therefore stay the reference's.
"""
import argparse
import json
import os
from dataclasses import dataclass, field

MEASURED_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "models_mi355x.json")
# bytes on the wire per fp32 byte of gradient: 1 or 2 bits per element (+ one scale per 512
# for terngrad), 8-byte pairs for the kept fraction of the sparsifiers
COMP_RATIO = {"onebit": 1 / 32, "tbq": 1 / 16, "terngrad": 1 / 16 + 1 / 512, "dgc": 2 * 0.001, "graddrop": 2 * 0.01}


@dataclass(frozen=True)
class CostModel:
    """t(x) = overhead below the break-even size, weight * x + bias above it
    (SeCoPa.py:4-20).  The break-even size is where the line reaches the floor."""

    weight: float
    bias: float
    overhead: float

    @property
    def threshold(self):
        if self.weight == 0:
            return 0
        return max(0, (self.overhead - self.bias) / self.weight)

    def cost(self, x):
        return self.overhead if x < self.threshold else self.weight * x + self.bias


# Coefficients the reference ships (SeCoPa.py:25-39); their unit and hardware are not stated there.
REFERENCE_ENCODE = CostModel(1.4133e-8, 5.8938e-2, 0.05408)
REFERENCE_DECODE = CostModel(6.2041e-9, 1.3956e-1, 0.07287)
REFERENCE_RING_SEND = CostModel(8.5005e-7, 2.0337e-1, 0.09766)
REFERENCE_GATHER = {4: CostModel(2.7156e-6, 4.1930e-1, 0.15573), 8: CostModel(6.1167e-6, 8.0768e-1, 0.28778),
                    16: CostModel(1.2937e-5, 1.4406, 0.59503)}
REFERENCE_BROADCAST = {4: CostModel(2.7157e-6, 2.2156e-1, 0.14820), 8: CostModel(6.1172e-6, 2.7285e-1, 0.29666),
                       16: CostModel(1.2915e-5, 4.5538e-1, 0.58353)}


@dataclass
class Planner:
    """Cluster of `nodes` workers; every model can be replaced (e.g. by a fit from `calibrate`)."""

    nodes: int = 16
    comp_ratio: float = 1.0 / 16
    encode: CostModel = REFERENCE_ENCODE
    decode: CostModel = REFERENCE_DECODE
    aggregate: CostModel = CostModel(0, 0, 0)
    ring_send: CostModel = REFERENCE_RING_SEND
    gather: CostModel = field(default=None)
    broadcast: CostModel = field(default=None)
    # This library's aggregator decodes the peers' payloads, sums them and re-encodes the sum
    # in one launch sequence.  With a model of that step (a function of the uncompressed
    # partition size, for nodes - 1 peers) the PS cost counts it once in place of the
    # reference's nodes - 1 decodes, nodes - 1 aggregations and one encode at the server.
    merge: CostModel = field(default=None)

    @classmethod
    def from_measured(cls, alg, nodes, path=None, **kw):
        """Planner with the encode / decode / merge models of `alg` measured on MI355X
        (hipress_amd/models_mi355x.json, written by `--calibrate-all`); the merge model is the
        one measured for nodes - 1 peers when there is one.  Communication models stay the
        reference's."""
        with open(path or MEASURED_PATH) as f:
            data = json.load(f)
        model = lambda d: CostModel(d["weight"], d["bias"], d["overhead"])
        args = {"encode": model(data["encode"][alg]), "decode": model(data["decode"][alg]),
                "comp_ratio": data["comp_ratio"][alg]}
        merge = data.get("merge", {}).get(alg, {}).get(str(nodes - 1))
        if merge is not None:
            args["merge"] = model(merge)
        args.update(kw)
        return cls(nodes=nodes, **args)

    def __post_init__(self):
        if self.gather is None or self.broadcast is None:
            if self.nodes not in REFERENCE_GATHER:
                raise ValueError("reference gather/broadcast models exist for 4, 8 and 16 nodes only")
            self.gather = self.gather or REFERENCE_GATHER[self.nodes]
            self.broadcast = self.broadcast or REFERENCE_BROADCAST[self.nodes]

    # Each *_costs method returns the cost for K = 1..nodes partitions, terms added in the
    # reference's order so that ties fall the same way.
    def uncompressed_costs(self, size, topology="PS"):
        n = self.nodes
        out = []
        for k in range(1, n + 1):
            part = size / k
            agg = (n - 1) * self.aggregate.cost(part)
            if topology == "PS":  # co-located servers: gather, N-1 aggregations, broadcast (SeCoPa.py:46-59)
                out.append(self.gather.cost(part) + self.broadcast.cost(part) + agg)
            else:  # ring: 2(N-1) sends, N-1 aggregations (SeCoPa.py:61-71)
                out.append(2 * (n - 1) * self.ring_send.cost(part) + agg)
        return out

    def compressed_costs(self, size, topology="PS"):
        n, r = self.nodes, self.comp_ratio
        out = []
        for k in range(1, n + 1):
            part, cpart = size / k, size * r / k
            agg = (n - 1) * self.aggregate.cost(part)
            if topology == "PS" and self.merge is not None:
                enc = (min(k + 1, n) - 1) * self.encode.cost(part)
                dec = (min(n - 1 + k, 2 * (n - 1)) - (n - 1)) * self.decode.cost(cpart)
                out.append(self.gather.cost(cpart) + self.broadcast.cost(cpart) + enc + dec + self.merge.cost(part))
            elif topology == "PS":  # SeCoPa.py:75-88
                enc = min(k + 1, n) * self.encode.cost(part)
                dec = min(n - 1 + k, 2 * (n - 1)) * self.decode.cost(cpart)
                out.append(self.gather.cost(cpart) + self.broadcast.cost(cpart) + enc + dec + agg)
            else:  # SeCoPa.py:90-102
                send = 2 * (n - 1) * self.ring_send.cost(cpart)
                out.append(send + n * self.encode.cost(part) + n * self.decode.cost(cpart) + agg)
        return out

    @staticmethod
    def _best(costs):
        best = min(costs)
        return best, costs.index(best) + 1  # the smallest K among equals

    def decide(self, size, topology="PS"):
        """-> ('y' | 'n', partitions): compress only if strictly cheaper (SeCoPa.py:105-113)."""
        plain, plain_k = self._best(self.uncompressed_costs(size, topology))
        comp, comp_k = self._best(self.compressed_costs(size, topology))
        return ("y", comp_k) if plain > comp else ("n", plain_k)

    def plan(self, gradients, topology="PS"):
        """gradients: iterable of (name, size) -> plan lines `name,size,y|n,K`."""
        lines = []
        for name, size in gradients:
            flag, parts = self.decide(size, topology)
            lines.append(f"{name},{size},{flag},{parts}")
        return lines


def read_gradients(path):
    out = []
    with open(path) as f:
        for line in f:
            if line.strip():
                cols = line.split(",")
                out.append((str(cols[0]), int(cols[1])))
    return out


def read_plan(path):
    """Plan lines `name,size,y|n,K` (SeCoPa.py:147) -> [(name, size, compress, partitions)]."""
    out = []
    with open(path) as f:
        for line in f:
            if line.strip():
                out.append(parse_plan_line(line))
    return out


def parse_plan_line(line):
    cols = [c.strip() for c in line.split(",")]
    if len(cols) != 4 or cols[2] not in ("y", "n") or int(cols[3]) < 1 or int(cols[1]) < 0:
        raise ValueError(f"not a plan line (name,size,y|n,K): {line.strip()!r}")
    return str(cols[0]), int(cols[1]), cols[2] == "y", int(cols[3])


def partition_bounds(size, parts, align=4):
    """[(offset, length)] of the K partitions a plan cuts a gradient of `size` elements into.

    The planner prices K equal parts of size / K (SeCoPa.py:52-59); the code that cuts
    them is not in the reference checkout, so the rule is fixed here: parts of
    ceil(size / K) elements rounded up to `align` (4 floats = 16 bytes, which keeps every
    part on the operators' vector path when the gradient is), the last part taking what
    is left, parts that would be empty dropped."""
    if size < 0 or parts < 1 or align < 1:
        raise ValueError("size >= 0, parts >= 1 and align >= 1 are required")
    step = -(-size // parts)
    step = -(-step // align) * align
    out, off = [], 0
    while off < size:
        out.append((off, min(step, size - off)))
        off += step
    return out


# ---------------------------------------------------------------- fitting
def fit_cost_model(sizes, times):
    """Least-squares line through the measurements that rise above the floor; the floor
    (overhead) is the smallest time seen.  Returns a CostModel in the unit of `times`."""
    pts = sorted(zip(sizes, times))
    floor = min(t for _, t in pts)
    rising = [(x, t) for x, t in pts if t > 1.25 * floor] or pts[-2:]
    if len(rising) < 2:
        rising = pts[-2:]
    n = len(rising)
    sx = sum(x for x, _ in rising)
    st = sum(t for _, t in rising)
    sxx = sum(x * x for x, _ in rising)
    sxt = sum(x * t for x, t in rising)
    den = n * sxx - sx * sx
    weight = (n * sxt - sx * st) / den if den else 0.0
    bias = (st - weight * sx) / n
    return CostModel(weight, bias, floor)


def calibrate(alg="tbq", sizes=None, reps=20, comp_ratio=None):
    """Measures encode and decode of `alg` on cuda:0 over a range of tensor sizes (one tensor
    per launch sequence, as the planner's per-partition costs assume) and fits both models.
    Times are in milliseconds; encode is a function of the element count, decode of the
    compressed size in elements (count * ratio), the arguments the planner passes them."""
    import torch

    import hipress_amd as hp

    sizes = sizes or [1 << k for k in range(10, 28, 2)]
    ratio = comp_ratio if comp_ratio is not None else COMP_RATIO[alg]
    enc_t, dec_t = [], []
    for n in sizes:
        g = torch.randn(n, device="cuda") * 1e-2
        t = {"gradient": g, "out": torch.empty_like(g)}
        if alg in ("tbq", "onebit"):
            t["residual"] = torch.zeros_like(g)
            nb = hp.tbq_payload_bytes(n) if alg == "tbq" else hp.onebit_payload_bytes(n)
        elif alg == "terngrad":
            t["uniform"] = torch.rand(n, device="cuda")
            nb = hp.terngrad_payload_bytes(n, 512)
        elif alg == "dgc":
            t["momentum"], t["accumulator"] = torch.zeros_like(g), torch.zeros_like(g)
            nb = hp.dgc_payload_bytes(n, 0.001)
        else:
            t["accumulator"] = torch.zeros_like(g)
            nb = hp.graddrop_payload_bytes(n, 0.01)
        t["compressed"] = torch.zeros(nb, dtype=torch.uint8, device="cuda")
        b = hp.Batch(alg, [t], threshold=0.05, ratio=0.01 if alg == "graddrop" else 0.001)
        for fn, acc in ((b.encode, enc_t), (b.decode, dec_t)):
            for _ in range(3):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            acc.append(e0.elapsed_time(e1) / reps)
        b.close()
    return {"alg": alg, "unit": "ms", "sizes": sizes, "encode_ms": enc_t, "decode_ms": dec_t, "comp_ratio": ratio,
            "encode": fit_cost_model(sizes, enc_t), "decode": fit_cost_model([n * ratio for n in sizes], dec_t)}


def calibrate_merge(alg="tbq", npeers=3, sizes=None, reps=20):
    """Measures decode-and-merge of `npeers` payloads with the fused re-encode on cuda:0 over a
    range of partition sizes and fits the model (milliseconds as a function of the
    uncompressed partition size in elements).  alg: tbq, dgc or graddrop."""
    import torch

    import hipress_amd as hp

    sizes = sizes or [1 << k for k in range(10, 28, 2)]
    times = []
    for n in sizes:
        if alg == "tbq":
            nb, kw = hp.tbq_payload_bytes(n), {"threshold": 0.05}
            enc = lambda g, pay: hp.tbq_encode(g, torch.zeros_like(g), pay, 0.05)
        else:
            ratio = 0.01 if alg == "graddrop" else 0.001
            nb, kw = hp.sparse_payload_bytes(n, ratio), {"ratio": ratio}
            enc = lambda g, pay: hp.graddrop_encode(g, torch.zeros_like(g), pay, ratio)
        pays = []
        for p in range(npeers):
            pay = torch.zeros(nb, dtype=torch.uint8, device="cuda")
            enc(torch.randn(n, device="cuda") * 1e-2, pay)
            pays.append(pay)
        chunk = {"compressed": pays, "aggregate": torch.empty(n, device="cuda"), "state": torch.zeros(n, device="cuda"),
                 "out_compressed": torch.zeros(nb, dtype=torch.uint8, device="cuda")}
        mb = hp.MergeBatch("tbq" if alg == "tbq" else "dgc", [chunk], **kw)
        for _ in range(3):
            mb.run()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            mb.run()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) / reps)
        mb.close()
    return {"alg": alg, "npeers": npeers, "unit": "ms", "sizes": sizes, "merge_ms": times, "merge": fit_cost_model(sizes, times)}


def calibrate_all(reps=20, sizes=None):
    """Every model the planner can take from this library, measured on cuda:0: encode and
    decode of the five compressors, the fused decode-and-merge of tbq / dgc / graddrop for
    3, 7 and 15 peers (4, 8 and 16 nodes).  Returns the dictionary `from_measured` reads."""
    import torch

    as_dict = lambda m: {"weight": m.weight, "bias": m.bias, "overhead": m.overhead}
    props = torch.cuda.get_device_properties(0)
    out = {"device": f"{getattr(props, 'gcnArchName', '?').split(':')[0]} ({torch.cuda.get_device_name(0)})", "unit": "ms",
           "note": "t(x) = overhead below the break-even size, weight * x + bias above it; encode and merge take "
                   "fp32 elements, decode takes elements * comp_ratio",
           "encode": {}, "decode": {}, "comp_ratio": {}, "merge": {}, "raw": {}}
    for alg in ("onebit", "tbq", "terngrad", "dgc", "graddrop"):
        cal = calibrate(alg, sizes=sizes, reps=reps)
        out["encode"][alg], out["decode"][alg] = as_dict(cal["encode"]), as_dict(cal["decode"])
        out["comp_ratio"][alg] = cal["comp_ratio"]
        out["raw"][alg] = {"sizes": cal["sizes"], "encode_ms": cal["encode_ms"], "decode_ms": cal["decode_ms"]}
    for alg in ("tbq", "dgc", "graddrop"):
        out["merge"][alg] = {}
        for npeers in (3, 7, 15):
            mer = calibrate_merge(alg, npeers=npeers, sizes=sizes, reps=reps)
            out["merge"][alg][str(npeers)] = as_dict(mer["merge"])
            out["raw"][f"merge_{alg}_{npeers}"] = {"sizes": mer["sizes"], "merge_ms": mer["merge_ms"]}
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(description="SeCoPa: selective compression and partitioning plan")
    ap.add_argument("--measured", metavar="ALG", default=None,
                    help="plan with the models of ALG measured on MI355X that ship with the package")
    ap.add_argument("--calibrate-all", metavar="JSON", default=None,
                    help="measure every algorithm's models on cuda:0 and write them to JSON (no plan is made)")
    ap.add_argument("--input", default="input.txt", help="lines of name,size (fp32 elements)")
    ap.add_argument("--output", default="SeCoPaPlan.txt")
    ap.add_argument("--topology", default="PS", choices=["PS", "RING"])
    ap.add_argument("--nnodes", type=int, default=16)
    ap.add_argument("--calibrate", metavar="ALG", default=None,
                    help="measure ALG's encode/decode on cuda:0 and plan with the fitted models "
                         "(communication models stay the reference's)")
    args = ap.parse_args(argv)
    if args.calibrate_all:
        with open(args.calibrate_all, "w") as f:
            json.dump(calibrate_all(), f, indent=1)
        return
    kw = {}
    if args.measured:
        planner = Planner.from_measured(args.measured, args.nnodes)
        with open(args.output, "w") as f:
            for line in planner.plan(read_gradients(args.input), args.topology):
                f.write(line + "\n")
        return
    if args.calibrate:
        cal = calibrate(args.calibrate)
        kw = {"encode": cal["encode"], "decode": cal["decode"], "comp_ratio": cal["comp_ratio"]}
        print(json.dumps({k: (v.__dict__ if isinstance(v, CostModel) else v) for k, v in cal.items()}))
        if args.calibrate in ("tbq", "dgc", "graddrop") and args.topology == "PS":
            mer = calibrate_merge(args.calibrate, npeers=args.nnodes - 1)
            kw["merge"] = mer["merge"]
            print(json.dumps({k: (v.__dict__ if isinstance(v, CostModel) else v) for k, v in mer.items()}))
    planner = Planner(nodes=args.nnodes, **kw)
    with open(args.output, "w") as f:
        for line in planner.plan(read_gradients(args.input), args.topology):
            f.write(line + "\n")


if __name__ == "__main__":
    main()
