"""Writes tests/golden/jni_symbols.txt: the JNI export names the reference's native
libraries define for the matrix-multiplication path and the runtime subset it uses,
read as text from the reference's source files (nothing is imported or run).

usage: python tests/golden/make_jni_symbols.py [/root/reference]
"""
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
CU = os.path.join(REF, "source", "engine-cuda-base")
FILES = [
    "Cuda_matMul/Cuda_matMul/A.cu",
    "Cuda_batchMatMul/Cuda_batchMatMul/A.cu",
    "Cuda/Cuda/Cuda_memory.cuh",
    "Cuda/Cuda/Cuda_Stream.cuh",
    "Cuda/Cuda/Cuda_Event.cuh",
    "Cuda/Cuda/Cuda_Device.cuh",
    "Cuda/Cuda/Cuda_Exception.cuh",
    "Cuda/Cuda/Cuda_float.cuh",
    "Cuda_function/Cuda_function/A.cu",
    "Cuda_expk2/Cuda_expk2/Cuda_transpose.cuh",
    "Cuda_conv3D/Cuda_conv3D/A.cu",
]
# of the element-wise library only the bias row and the scalar linear map belong to the path
ONLY = {"Cuda_function/Cuda_function/A.cu": {"Java_z_dragon_engine_cuda_impl_math_Cuda_1function_linear_1dual2D_1row",
                                             "Java_z_dragon_engine_cuda_impl_math_Cuda_1function_linear2D"}}
out = []
for f in FILES:
    text = open(os.path.join(CU, f), encoding="utf-8", errors="replace").read()
    for name in re.findall(r"\b(Java_z_dragon_engine_cuda_impl_\w+)\s*\(", text):
        if f in ONLY and name not in ONLY[f]:
            continue
        out.append("%s %s" % (f, name))
dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "jni_symbols.txt")
with open(dst, "w") as fh:
    fh.write("\n".join(out) + "\n")
print("wrote %d names to %s" % (len(out), dst))
