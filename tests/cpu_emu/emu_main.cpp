// Stand-alone driver of the CPU-emulated kernels, for sanitizer runs (AddressSanitizer needs an instrumented main):
//   emu_main <n> <sigma> <seed> [key_words]
// Sorts a random text through the emulated library and compares with the CPU oracle. Test infrastructure only.
#include "../../include/cascade_hip.h"
#include "../../oracle/cascade_oracle.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

int main(int argc, char** argv)
{
    const uint64_t n = argc > 1 ? strtoull(argv[1], 0, 10) : 8000;
    const unsigned sigma = argc > 2 ? atoi(argv[2]) : 3;
    uint64_t seed = argc > 3 ? strtoull(argv[3], 0, 10) : 1;
    const int key_words = argc > 4 ? atoi(argv[4]) : 1;
    std::vector<uint16_t> T(n);
    for (auto& x : T) {
        seed = seed * 6364136223846793005ull + 1442695040888963407ull;
        const unsigned r = (unsigned)(seed >> 33);
        x = (r % 50 == 0) ? 0xFFFF : (uint16_t)((r % sigma) * (65535u / (sigma > 1 ? sigma - 1 : 1)));
    }
    csa_handle* h = nullptr;
    if (csa_create(n, key_words, &h)) {
        printf("create failed: %s\n", csa_last_error());
        return 2;
    }
    std::vector<uint8_t> got(5 * n + 8), want(5 * n + ORC_SA_PAD_BYTES);
    csa_stats st;
    const int rc = csa_sort_partition_u16_dev(h, T.data(), n, 0, got.data(), nullptr, 0, &st);
    if (rc) {
        printf("sort failed: %s\n", csa_last_error());
        return 2;
    }
    orc_build_sa40_u16(T.data(), n, want.data());
    const bool ok = memcmp(got.data(), want.data(), 5 * n) == 0;
    printf("n=%llu sigma=%u kw=%d generations=%d", (unsigned long long)n, sigma, key_words, st.generations);
    for (int g = 0; g < st.generations; ++g)
        printf(" [%llu/%llu]", (unsigned long long)st.active[g], (unsigned long long)st.big[g]);
    printf(" %s\n", ok ? "OK" : "MISMATCH");
    csa_destroy(h);
    return ok ? 0 : 1;
}
