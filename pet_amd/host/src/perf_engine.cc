#include "perf_engine.h"

namespace tpm {

PerfEngine::PerfEngine() { petInit(); }

PerfEngine::~PerfEngine() {
    for (auto &b : buf)
        if (b)
            pet_hip_free(b);
}

// Scratch operand `which`, at least `elems` floats, filled with uniform noise
// in [-1, 1) once per (re)allocation (the reference fills with cuRAND,
// src/Graph/perf_engine.cc:49-55).
float *PerfEngine::scratch(int which, size_t elems) {
    if (elems == 0)
        elems = 1;
    if (bufElems[which] >= elems)
        return buf[which];
    if (buf[which]) {
        pet_hip_stream_sync(petStream());
        pet_hip_free(buf[which]);
        buf[which] = nullptr;
        bufElems[which] = 0;
    }
    size_t want = elems + elems / 4; // head-room so that growing is rare
    void *p = nullptr;
    if (!petOk(pet_hip_malloc(&p, want * sizeof(float)), "pet_hip_malloc(scratch)"))
        return nullptr;
    buf[which] = (float *)p;
    bufElems[which] = want;
    petOk(pet_hip_rand_uniform_f32(buf[which], want, 0x9E3779B9u + which, -1.f, 1.f, petStream()),
          "pet_hip_rand_uniform_f32");
    return buf[which];
}

double PerfEngine::layoutBandwidthGiBs() {
    if (bandwidth > 0.0)
        return bandwidth;
    const size_t elems = (size_t)64 << 20; // 256 MiB each way
    float *src = scratch(0, elems), *dst = scratch(2, elems);
    if (!src || !dst)
        return 0.0;
    int dims[2] = {(int)(elems / 1024), 1024}, perm[2] = {0, 1};
    pet_hip_stream_t s = petStream();
    for (int i = 0; i < 2; ++i)
        pet_hip_transpose(src, dst, dims, perm, 2, s);
    pet_hip_event_t e0 = nullptr, e1 = nullptr;
    pet_hip_event_create(&e0);
    pet_hip_event_create(&e1);
    pet_hip_event_record(e0, s);
    const int reps = 5;
    for (int i = 0; i < reps; ++i)
        pet_hip_transpose(src, dst, dims, perm, 2, s);
    pet_hip_event_record(e1, s);
    pet_hip_event_sync(e1);
    float ms = 0.f;
    pet_hip_event_elapsed_ms(&ms, e0, e1);
    pet_hip_event_destroy(e0);
    pet_hip_event_destroy(e1);
    double bytes = 2.0 * elems * sizeof(float) * reps;
    bandwidth = bytes / (ms * 1e-3) / (1024.0 * 1024.0 * 1024.0);
    return bandwidth;
}

void PerfEngine::dumpPerfData() {
    for (auto &kv : convPerf) {
        int n, c, h, w, f, r, s, ph, pw, sh, sw, dh, dw, g, bi, ac;
        std::tie(n, c, h, w, f, r, s, ph, pw, sh, sw, dh, dw, g, bi, ac) = kv.first;
        std::printf("conv n%d c%d h%d w%d f%d r%d s%d p%d,%d s%d,%d d%d,%d g%d bias%d act%d: %.4f ms\n",
                    n, c, h, w, f, r, s, ph, pw, sh, sw, dh, dw, g, bi, ac, kv.second.time);
    }
    for (auto &kv : matmulPerf) {
        bool ta, tb;
        int b, m, n, k;
        std::tie(ta, tb, b, m, n, k) = kv.first;
        std::printf("matmul tA%d tB%d b%d m%d n%d k%d: %.4f ms\n", ta, tb, b, m, n, k,
                    kv.second.time);
    }
}

} // namespace tpm
