"""The JNI shim must export exactly the names the reference's Java classes bind.  No JVM
is available, so the names defined in csrc/jni/dragon_jni.cpp (macros expanded by hand
here) are compared with the names read from the reference's native sources
(tests/golden/jni_symbols.txt, produced by tests/golden/make_jni_symbols.py)."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIM = os.path.join(ROOT, "dragon-alpha-v1.2_amd", "csrc", "jni", "dragon_jni.cpp")
GOLDEN = os.path.join(ROOT, "tests", "golden", "jni_symbols.txt")

PREFIX = {"MM": "Java_z_dragon_engine_cuda_impl_math_Cuda_1matMul_",
          "BMM": "Java_z_dragon_engine_cuda_impl_math_Cuda_1batchMatMul_",
          "RT": "Java_z_dragon_engine_cuda_impl_Cuda_",
          "FN": "Java_z_dragon_engine_cuda_impl_math_Cuda_1function_",
          "EK": "Java_z_dragon_engine_cuda_impl_Cuda_1expk2_",
          "CV": "Java_z_dragon_engine_cuda_impl_math_Cuda_1conv3D_"}


def shim_names():
    text = open(SHIM).read()
    names = set()
    for macro, arg in re.findall(r"JNICALL\s+(MM|BMM|RT|FN|EK|CV)\((\w+)\)\s*\(", text):
        if arg != "jname":           # the macro bodies
            names.add(PREFIX[macro] + arg)
    for kind, arg in re.findall(r"^DEF_(MM2D|MMSK|BMM|BMM_MMA)\((\w+),", text, flags=re.M):
        names.add(PREFIX["MM" if kind.startswith("MM") else "BMM"] + arg)
    for arg in re.findall(r"^DEF_CV\w*\((\w+),", text, flags=re.M):
        names.add(PREFIX["CV"] + arg)
    return names


def golden():
    rows = [l.split() for l in open(GOLDEN).read().splitlines() if l.strip()]
    return {name: f for f, name in rows}


def test_every_matmul_native_of_the_reference_is_in_the_shim():
    g, s = golden(), shim_names()
    gemm = {n for n, f in g.items() if "Cuda_matMul" in f or "Cuda_batchMatMul" in f}
    assert len(gemm) == 12           # 7 in Cuda_matMul/A.cu, 5 in Cuda_batchMatMul/A.cu
    assert gemm <= s, sorted(gemm - s)


def test_bias_row_native_is_in_the_shim():
    g, s = golden(), shim_names()
    rows = {n for n, f in g.items() if "Cuda_function" in f}
    assert rows == {PREFIX["FN"] + "linear_1dual2D_1row", PREFIX["FN"] + "linear2D"}
    assert rows <= s


def test_every_convolution_native_of_the_reference_is_in_the_shim():
    g, s = golden(), shim_names()
    conv = {n for n, f in g.items() if "Cuda_conv3D" in f}
    assert len(conv) == 17           # kernel_remode, 5 plain, 7 with the re-ordered filter, 4 im2col-Winograd
    assert conv <= s, sorted(conv - s)
    assert {n for n in s if n.startswith(PREFIX["CV"])} - conv == {PREFIX["CV"] + "conv3D_1biased"}


def test_dimension_swap_natives_are_in_the_shim():
    g, s = golden(), shim_names()
    swaps = {n for n, f in g.items() if "Cuda_transpose" in f}
    assert swaps == {PREFIX["EK"] + n for n in ("transpose2D", "transpose3D", "transpose4D")}
    assert swaps <= s


def test_runtime_subset_names_exist_in_the_reference():
    g, s = golden(), shim_names()
    runtime = {n for n in s if n.startswith(PREFIX["RT"]) and not n.startswith(PREFIX["EK"])}
    assert len(runtime) >= 40
    unknown = sorted(n for n in runtime if n not in g)
    assert not unknown, "names the reference does not define: %s" % unknown
    # the natives the path calls (CudaFloat32EngineBase.java:649-694, 1008-1054, 1148-1260, 1519-1590)
    for must in ("malloc", "free", "memsetAsync", "newStream_1Blocking__", "deleteStream___3JI",
                 "streamSynchronize__J", "newEvent_1DisableTiming", "eventRecord__JJ",
                 "eventRecord__J_3JI", "eventSync_1Del", "deleteEvent", "streamWaitEvent_1default",
                 "deviceSynchronize", "set1D__JJ_3FI", "set2D__JJ_3FIII", "get1D", "get2D",
                 "get1D_1v2", "get2D_1v2", "set1D_1v2__JJ_3FJI", "set2D_1v2__JJ_3FJIII"):
        assert PREFIX["RT"] + must in s, must


def test_mma_names_follow_the_java_declarations():
    # the *_mma natives have no published native source; their names follow JNI mangling of
    # the Java declarations (Cuda_matMul.java:163,278,369; Cuda_batchMatMul.java:166,236,355)
    s = shim_names()
    for n in ("matMul_1mma", "matMulT1_1mma", "matMulT2_1mma"):
        assert PREFIX["MM"] + n in s
    for n in ("batchMatMul_1mma", "batchMatMulT1_1mma", "batchMatMulT2_1mma"):
        assert PREFIX["BMM"] + n in s
