#!/bin/bash
# Builds the C++ tests of the host-side operator mirror next to their sources.
set -e
cd "$(dirname "$0")"
ROOT=../..
g++ -std=c++17 -O1 -Wall -I$ROOT/include test_host_logic.cpp -o test_host_logic
/opt/rocm/bin/hipcc -std=c++17 -O1 -I$ROOT/include test_host_gpu.cpp -o test_host_gpu \
    -L$ROOT/ane-fieldfare_amd -lfieldfare_moe_hip -L$ROOT/oracle -lffmoe_oracle \
    -Wl,-rpath,'$ORIGIN/../../ane-fieldfare_amd' -Wl,-rpath,'$ORIGIN/../../oracle' 2> >(grep -v "packed-fp32-ops" >&2)
