#!/bin/bash
# Builds tensor_amd/lib/libotter_hip_host.so: the C++ host layer (Otter Layer / ConvolutionLayer / Net mirror) over
# the C ABI of libotter_hip_int8.so. Plain g++: no HIP headers are needed above the C ABI.
set -e
cd "$(dirname "$0")"
mkdir -p ../lib
g++ -std=c++17 -O2 -fPIC -shared -Wall -Wextra -Wno-unused-parameter otter_hip.cpp otter_file.cpp host_capi.cpp \
    -L../lib -lotter_hip_int8 -Wl,-rpath,'$ORIGIN' -o ../lib/libotter_hip_host.so
echo "built $(cd ../lib && pwd)/libotter_hip_host.so"
