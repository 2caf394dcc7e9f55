"""The occupancy limit some streaming kernels set for themselves by claiming vector registers
(common.h: four_waves_per_simd) depends on how the compiler allocates registers, and results do
not: a compiler release that allocates differently would cost a few per cent without failing a
parity test.  This build-side test compiles the kernel files for gfx950 with the library's own
flags (device code only, nothing is run) and reads the compiler's resource-usage remarks: every
kernel that asks for the limit must come out at 97..128 vector registers, which is four
wavefronts per SIMD of the 512 registers a lane has, and the kernels that must stay unlimited
must not be caught by it."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "hipress_amd", "csrc")


def resource_usage(source):
    """{mangled kernel name: (vgprs, waves per SIMD)} from -Rpass-analysis=kernel-resource-usage."""
    from hipress_amd import build as hb

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    r = subprocess.run([hipcc, *hb.FLAGS, "--cuda-device-only", "-c", os.path.join(CSRC, source), "-o", os.devnull,
                        "-Rpass-analysis=kernel-resource-usage"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    out, name = {}, None
    for line in r.stderr.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            out[name] = [None, None]
        m = re.search(r"remark:\s+VGPRs: (\d+)", line)
        if m and name:
            out[name][0] = int(m.group(1))
        m = re.search(r"remark:\s+Occupancy \[waves/SIMD\]: (\d+)", line)
        if m and name:
            out[name][1] = int(m.group(1))
    return out


# source file -> (substrings of the mangled names that claim the limit, substrings of names that must not)
LIMITED = {
    "dense.hip": (["tbq_encode_kernel", "tbq_decode_kernel", "onebit_abs_kernel", "onebit_quant_kernel", "onebit_decode_kernel"],
                  ["terngrad_encode_kernel", "terngrad_decode_kernel", "onebit_deferred_kernel"]),
    "sparse.hip": (["sparse_accum_kernelINS_8BatchSrcELb0E", "sparse_accum_kernelINS_9SingleSrcELb0E"],
                   ["sparse_accum_kernelINS_8BatchSrcELb1E", "sparse_merge_kernel", "sparse_count_kernel", "sparse_emit_kernel"]),
    "compll.hip": (["compll_minmax_kernel"], ["compll_quant_kernel", "compll_decode_kernel"]),
}


@pytest.mark.parametrize("source", sorted(LIMITED))
def test_register_claimed_occupancy(source):
    usage = resource_usage(source)
    limited, free = LIMITED[source]
    for key in limited:
        hits = {k: v for k, v in usage.items() if key in k}
        assert hits, f"no kernel named like {key} in {source}"
        for name, (vgprs, waves) in hits.items():
            assert 97 <= vgprs <= 128 and waves == 4, (name, vgprs, waves)
    for key in free:
        hits = {k: v for k, v in usage.items() if key in k}
        assert hits, f"no kernel named like {key} in {source}"
        for name, (vgprs, waves) in hits.items():
            assert vgprs <= 128, (name, vgprs)  # nothing in the library runs below four wavefronts per SIMD
            assert waves >= 4, (name, waves)
