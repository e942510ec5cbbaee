// Random weights on the host: the same numbers, bit for bit, that the kernel of
// csrc/kernels/random_fill.hip makes on the GPU (both compile csrc/shared/random_normal.h).
// The reference has no random-weights mode; this one exists so that the engine can be tested
// against a plain implementation and measured without any file.
#include <algorithm>
#include <thread>
#include <vector>

#include "../shared/random_normal.h"

#define API extern "C" __attribute__((visibility("default")))

// out[i] = normal(key, first + i) * std + shift for i in [0, n); type 0: float32, 1: bfloat16.
API int lcu_random_fill_host(void *out, int type, long long n, unsigned long long key, long long first, float std,
                             float shift, int threads) {
    if (n < 0 || first < 0 || (type != 0 && type != 1) || (n > 0 && !out)) return -3;
    const int nt = (int)std::max<long long>(1, std::min<long long>(threads > 0 ? threads : 1, n / 65536));
    auto work = [=](long long a, long long b) {
        if (type == 0) {
            float *o = (float *)out;
            for (long long i = a; i < b; ++i) o[i] = lcu_random_weight(key, (uint64_t)(first + i), std, shift);
        } else {
            uint16_t *o = (uint16_t *)out;
            for (long long i = a; i < b; ++i) o[i] = lcu_bf16_bits(lcu_random_weight(key, (uint64_t)(first + i), std, shift));
        }
    };
    if (nt == 1) {
        work(0, n);
        return 0;
    }
    std::vector<std::thread> pool;
    for (int t = 0; t < nt; ++t) pool.emplace_back(work, n * t / nt, n * (t + 1) / nt);
    for (auto &t : pool) t.join();
    return 0;
}
