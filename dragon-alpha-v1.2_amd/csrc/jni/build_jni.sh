#!/bin/bash
# Builds libdragon_hip_jni.so where a JDK is installed (JAVA_HOME or javac on PATH).
# It links against ../../libdragon_hip.so; without a JDK there is nothing to build.
set -euo pipefail
cd "$(dirname "$0")"
JH=${JAVA_HOME:-}
if [ -z "$JH" ] && command -v javac >/dev/null 2>&1; then
  JH=$(dirname "$(dirname "$(readlink -f "$(command -v javac)")")")
fi
if [ -z "$JH" ] || [ ! -f "$JH/include/jni.h" ]; then
  echo "no JDK found (jni.h): the JNI shim is not built" >&2
  exit 0
fi
g++ -O2 -std=c++17 -fPIC -shared -I"$JH/include" -I"$JH/include/linux" dragon_jni.cpp \
    -L../.. -ldragon_hip -Wl,-rpath,'$ORIGIN' -o ../../libdragon_hip_jni.so
echo "built $(cd ../.. && pwd)/libdragon_hip_jni.so"
