"""The JNI shim must export exactly the names the reference's Java classes bind.  No JVM is available, so
the shim (csrc/jni/dragon_jni.cpp) is compiled here against a minimal test-only <jni.h>
(tests/jni_stub/jni.h), linked with the product library, and the dynamic symbols the compiler really
produced (nm -D) are compared with the names read from the reference's native sources
(tests/golden/jni_symbols.txt, written by tests/golden/make_jni_symbols.py)."""
import ctypes
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "dragon-alpha-v1.2_amd")
SHIM = os.path.join(PKG, "csrc", "jni", "dragon_jni.cpp")
STUB = os.path.join(ROOT, "tests", "jni_stub")
GOLDEN = os.path.join(ROOT, "tests", "golden", "jni_symbols.txt")

PREFIX = {"MM": "Java_z_dragon_engine_cuda_impl_math_Cuda_1matMul_",
          "BMM": "Java_z_dragon_engine_cuda_impl_math_Cuda_1batchMatMul_",
          "RT": "Java_z_dragon_engine_cuda_impl_Cuda_",
          "FN": "Java_z_dragon_engine_cuda_impl_math_Cuda_1function_",
          "EK": "Java_z_dragon_engine_cuda_impl_Cuda_1expk2_",
          "CV": "Java_z_dragon_engine_cuda_impl_math_Cuda_1conv3D_"}


@pytest.fixture(scope="module")
def shim_library(tmp_path_factory):
    """dragon_jni.cpp compiled with -Wall -Werror against the stand-in header and linked with libdragon_hip.so."""
    assert os.path.exists(os.path.join(PKG, "libdragon_hip.so")), "build the product library first"
    out = str(tmp_path_factory.mktemp("jni") / "libdragon_hip_jni.so")
    cmd = ["g++", "-O1", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Werror", "-I" + STUB, SHIM,
           "-L" + PKG, "-ldragon_hip", "-Wl,-rpath," + PKG, "-Wl,--no-undefined", "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    return out


@pytest.fixture(scope="module")
def shim_names(shim_library):
    out = subprocess.run(["nm", "-D", "--defined-only", shim_library], capture_output=True, text=True, check=True).stdout
    return {line.split()[-1] for line in out.splitlines() if line.split()[-1].startswith(("Java_", "JNI_"))}


def golden():
    rows = [l.split() for l in open(GOLDEN).read().splitlines() if l.strip()]
    return {name: f for f, name in rows}


def test_the_shim_compiles_links_and_loads(shim_library, shim_names):
    # every call it makes into the product library resolves (--no-undefined) and the JVM's entry hook answers
    lib = ctypes.CDLL(shim_library)
    lib.JNI_OnLoad.restype = ctypes.c_int32
    lib.JNI_OnLoad.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    assert lib.JNI_OnLoad(None, None) == 0x00010008          # JNI_VERSION_1_8
    assert "JNI_OnLoad" in shim_names and len([n for n in shim_names if n.startswith("Java_")]) >= 90


def test_every_exported_name_is_one_the_java_side_binds(shim_names):
    """Nothing misspelt: each Java_* export is a native of the reference (text of its sources), one of the
    *_mma natives (declared in Java, native source unpublished) or one of the documented additions."""
    g = golden()
    additions = {PREFIX["MM"] + "matMul_1biased", PREFIX["MM"] + "matMulSK_1static",
                 PREFIX["CV"] + "conv3D_1biased", PREFIX["BMM"] + "attention", PREFIX["BMM"] + "attention_1masked",
                 "Java_z_dragon_engine_cuda_impl_math_Cuda_1reduce_softmax2D"}
    mma = {PREFIX["MM"] + n for n in ("matMul_1mma", "matMulT1_1mma", "matMulT2_1mma")} | \
          {PREFIX["BMM"] + n for n in ("batchMatMul_1mma", "batchMatMulT1_1mma", "batchMatMulT2_1mma")}
    unknown = sorted(n for n in shim_names if n.startswith("Java_") and n not in g and n not in additions and n not in mma)
    assert not unknown, "exports the Java side has no native for: %s" % unknown


def test_every_matmul_native_of_the_reference_is_in_the_shim(shim_names):
    g = golden()
    gemm = {n for n, f in g.items() if "Cuda_matMul" in f or "Cuda_batchMatMul" in f}
    assert len(gemm) == 12           # 7 in Cuda_matMul/A.cu, 5 in Cuda_batchMatMul/A.cu
    assert gemm <= shim_names, sorted(gemm - shim_names)


def test_bias_row_native_is_in_the_shim(shim_names):
    g = golden()
    rows = {n for n, f in g.items() if "Cuda_function" in f}
    assert rows == {PREFIX["FN"] + "linear_1dual2D_1row", PREFIX["FN"] + "linear2D"}
    assert rows <= shim_names


def test_every_convolution_native_of_the_reference_is_in_the_shim(shim_names):
    g = golden()
    conv = {n for n, f in g.items() if "Cuda_conv3D" in f}
    assert len(conv) == 17           # kernel_remode, 5 plain, 7 with the re-ordered filter, 4 im2col-Winograd
    assert conv <= shim_names, sorted(conv - shim_names)
    assert {n for n in shim_names if n.startswith(PREFIX["CV"])} - conv == {PREFIX["CV"] + "conv3D_1biased"}


def test_dimension_swap_natives_are_in_the_shim(shim_names):
    g = golden()
    swaps = {n for n, f in g.items() if "Cuda_transpose" in f}
    assert swaps == {PREFIX["EK"] + n for n in ("transpose2D", "transpose3D", "transpose4D")}
    assert swaps <= shim_names


def test_runtime_subset_names_exist_in_the_reference(shim_names):
    g = golden()
    runtime = {n for n in shim_names if n.startswith(PREFIX["RT"]) and not n.startswith(PREFIX["EK"])}
    assert len(runtime) >= 40
    unknown = sorted(n for n in runtime if n not in g)
    assert not unknown, "names the reference does not define: %s" % unknown
    # the natives the path calls (CudaFloat32EngineBase.java:649-694, 1008-1054, 1148-1260, 1519-1590)
    for must in ("malloc", "free", "memsetAsync", "newStream_1Blocking__", "deleteStream___3JI",
                 "streamSynchronize__J", "newEvent_1DisableTiming", "eventRecord__JJ",
                 "eventRecord__J_3JI", "eventSync_1Del", "deleteEvent", "streamWaitEvent_1default",
                 "deviceSynchronize", "set1D__JJ_3FI", "set2D__JJ_3FIII", "get1D", "get2D",
                 "get1D_1v2", "get2D_1v2", "set1D_1v2__JJ_3FJI", "set2D_1v2__JJ_3FJIII"):
        assert PREFIX["RT"] + must in shim_names, must


def test_mma_names_follow_the_java_declarations(shim_names):
    # the *_mma natives have no published native source; their names follow JNI mangling of
    # the Java declarations (Cuda_matMul.java:163,278,369; Cuda_batchMatMul.java:166,236,355)
    for n in ("matMul_1mma", "matMulT1_1mma", "matMulT2_1mma"):
        assert PREFIX["MM"] + n in shim_names
    for n in ("batchMatMul_1mma", "batchMatMulT1_1mma", "batchMatMulT2_1mma"):
        assert PREFIX["BMM"] + n in shim_names
