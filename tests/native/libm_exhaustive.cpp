// Exhaustive comparison of visualmesh_amd/csrc/libm_exact.h against the host C library, over every float
// of the ranges the lens projection can produce (and beyond). Built and run by tests/test_libm_exact.py.
// Prints one line per range: "<name> <mismatches>", exit status 0 iff all are zero.
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "libm_exact.h"

static float from_bits(uint32_t u) {
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
static uint32_t to_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}

template <class Mine, class Host>
static long sweep(const char* name, uint32_t lo, uint32_t hi, int threads, Mine mine, Host host) {
    std::atomic<long> bad(0);
    std::vector<std::thread> pool;
    for (int t = 0; t < threads; ++t)
        pool.emplace_back([&, t] {
            long b = 0;
            for (uint64_t u = uint64_t(lo) + t; u <= hi; u += threads) {
                const float x = from_bits(uint32_t(u));
                const float a = mine(x), r = host(x);
                if (to_bits(a) != to_bits(r) && !(a != a && r != r)) ++b;
            }
            bad += b;
        });
    for (auto& th : pool) th.join();
    std::printf("%s %ld\n", name, bad.load());
    return bad.load();
}

int main(int argc, char** argv) {
    const int threads = argc > 1 ? std::atoi(argv[1]) : 4;
    long bad = 0;
    bad += sweep("acosf[0,1]", 0x00000000u, 0x3f800000u, threads, vm_acosf, [](float x) { return acosf(x); });
    bad += sweep("acosf[-1,0]", 0x80000000u, 0xbf800000u, threads, vm_acosf, [](float x) { return acosf(x); });
    bad += sweep("sinf[0,pi]", 0x00000000u, 0x40490fdbu, threads, vm_sinf, [](float x) { return sinf(x); });
    bad += sweep("tanf[0,3pi/4)", 0x00000000u, 0x4016cbe3u, threads, vm_tanf, [](float x) { return tanf(x); });
    bad += sweep("sqrtf[0,4]", 0x00000000u, 0x40800000u, threads, vm_sqrtf, [](float x) { return sqrtf(x); });
    return bad == 0 ? 0 : 1;
}
