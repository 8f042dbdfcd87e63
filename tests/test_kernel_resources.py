"""The balanced kernel's stage loop is tuned down to the instruction: its 128 x 128 instantiations (the headline
4096^3 products) run at 95 % of the matrix peak with 201-203 vector registers, 64-66 accumulator registers and
no scratch, and the compiler's code for the loop has reacted to innocent edits before (folding its four unrolled
steps into one expression: 8 %; a fast path behind the loop: 12 %).  A source or compiler change that brings
spills or a visibly different allocation must fail here, not in a benchmark.

Reads the compiler's own report (-Rpass-analysis=kernel-resource-usage) that the build leaves beside the object;
compiles the device code itself (about two minutes) when that report is missing or older than the sources."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "dragon-alpha-v1.2_amd", "csrc")
REPORT = os.path.join(CSRC, "build", "gemm_mfma_streamk.resources.txt")
SOURCES = [os.path.join(CSRC, f) for f in ("gemm_mfma_streamk.hip", "gemm_mfma_kernel.h", "gemm_mfma.h", "build.sh")]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# the three headline kernels: A*B, A*B^T, A^T*B through 128 x 128 tiles, 32 k per stage, 4 stage buffers, one
# workgroup per unit; no bias, unsplit, no gather, no zero fill
HEADLINE = {
    "A*B": "gemm_f32_mfma_streamk<true, false, 2, 2, 2, 2, 32, 4, 1, false, false, false, false>",
    "A*B^T": "gemm_f32_mfma_streamk<true, true, 2, 2, 2, 2, 32, 4, 1, false, false, false, false>",
    "A^T*B": "gemm_f32_mfma_streamk<false, false, 2, 2, 2, 2, 32, 4, 1, false, false, false, false>",
}
VGPR_BUDGET = 208        # measured 201-203 where the kernels run at 95 % of the peak
AGPR_BUDGET = 72         # the accumulators of four blocks: 64, plus what the allocator parks there (66)


def report_text():
    if os.path.exists(REPORT) and all(os.path.getmtime(REPORT) >= os.path.getmtime(f) for f in SOURCES):
        return open(REPORT).read()
    if not os.path.exists(HIPCC):
        pytest.skip("no hipcc and no fresh compiler report")
    flags = ("--offload-arch=gfx950 -O3 -std=c++17 -fPIC -Wno-unused-function -Xclang -target-feature -Xclang "
             "-packed-fp32-ops --cuda-device-only -Rpass-analysis=kernel-resource-usage").split()
    r = subprocess.run([HIPCC] + flags + ["-c", os.path.join(CSRC, "gemm_mfma_streamk.hip"), "-o", os.devnull],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    return r.stderr


def kernels(text):
    """{demangled kernel name: {"vgpr": n, "agpr": n, "scratch": n, "occupancy": n}}"""
    blocks = re.split(r"remark: [^\n]*Function Name: ", text)[1:]
    mangled = [b.split("\n")[0].split(" [")[0].strip() for b in blocks]
    names = subprocess.run(["c++filt"], input="\n".join(mangled), capture_output=True, text=True, check=True).stdout.split("\n")
    out = {}
    for name, b in zip(names, blocks):
        name = name.replace("void dragon::(anonymous namespace)::", "").replace("(dragon::GemmParams)", "").strip()
        field = lambda pat: int(re.search(pat + r": (\d+)", b).group(1))
        out[name] = {"vgpr": field(r"VGPRs"), "agpr": field(r"AGPRs"), "scratch": field(r"ScratchSize \[bytes/lane\]"),
                     "occupancy": field(r"Occupancy \[waves/SIMD\]")}
    return out


@pytest.fixture(scope="module")
def usage():
    return kernels(report_text())


def test_the_headline_kernels_keep_their_registers_and_spill_nothing(usage):
    for product, name in HEADLINE.items():
        assert name in usage, "%s: no instantiation %s in the compiler's report" % (product, name)
        u = usage[name]
        assert u["scratch"] == 0, "%s spills: %s" % (product, u)
        assert u["vgpr"] <= VGPR_BUDGET and u["agpr"] <= AGPR_BUDGET, "%s left its register budget: %s" % (product, u)


def test_no_balanced_kernel_uses_scratch(usage):
    spilling = {n: u for n, u in usage.items() if n.startswith("gemm_f32_mfma_streamk<") and u["scratch"] != 0}
    assert not spilling, spilling
    assert sum(n.startswith("gemm_f32_mfma_streamk<") for n in usage) >= 60
