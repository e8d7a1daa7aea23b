// Host-side basics of the PET operator layer on the MI355X backend.
// Mirrors the role of the reference's include/common.h (type aliases, guid and
// hash helpers at :127-162) without any CUDA / cuDNN / cuBLAS types: the device
// is reached only through the C ABI in pet_hip.h.
#pragma once

#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <iostream>
#include <map>
#include <memory>
#include <numeric>
#include <string>
#include <vector>

#include "pet_hip.h"

namespace tpm {

class Tensor;
class Operator;
class Graph;
class SubGraph;

using TensorVec = std::vector<Tensor *>;
using TensorMap = std::map<size_t, Tensor *>;
using OpVec = std::vector<Operator *>;
using OpMap = std::map<size_t, Operator *>;
// The reference computes in wrapping uint32 on the host (include/common.h:137);
// device tensors here are fp32, the type the kernels compute in.
using VType = float;
using SplittingPoints = std::vector<std::vector<int>>;

// Process-wide counters, as in the reference (not thread-safe there either).
inline size_t generateGuid() {
    static size_t next = 0;
    return next++;
}

inline uint64_t generateHash() {
    static uint64_t tag = 0;
    return std::hash<uint64_t>()(tag++);
}

// Same mixing constants as the reference so hashes of rebuilt graphs line up
// (include/common.h:151-155).
inline uint64_t hashAppend(uint64_t a, uint64_t b) {
    return (a * 10000019ull + b * 10000079ull) % 2147483647ull;
}
inline uint64_t hashPack(uint64_t x) { return (x * 10000103ull) % 2147483647ull; }

// Small integer helpers the mutators use (reference include/common.h:164-187).
inline int gcd(int a, int b) {
    while (b != 0) {
        int t = a % b;
        a = b;
        b = t;
    }
    return a;
}
inline int gcd(const std::vector<int> &v) {
    int g = v.empty() ? 1 : v[0];
    for (int x : v)
        g = gcd(g, x);
    return g;
}
inline int max(const std::vector<int> &v) {
    int m = 0;
    for (size_t i = 0; i < v.size(); ++i)
        m = i == 0 ? v[0] : std::max(m, v[i]);
    return m;
}

// Every C-ABI status goes through here: the reference exits on a CUDA error
// (include/common.h:30-38); this layer reports and lets the caller decide.
inline bool petOk(int status, const char *what) {
    if (status == PET_HIP_OK)
        return true;
    std::fprintf(stderr, "[pet] %s failed (status %d): %s\n", what, status, pet_hip_last_error());
    return false;
}

// PET_HOST_TRACE=1: say on stderr why an operator or graph did not compute.
inline bool hostTrace() {
    static const bool on = std::getenv("PET_HOST_TRACE") != nullptr;
    return on;
}

// One stream for the whole process (the reference uses the null stream).
pet_hip_stream_t petStream();
// Brings the backend up on device 0 once; returns false when no gfx950 device.
bool petInit();

} // namespace tpm
