// Driver for tests/test_host_asan.py: the library's host-memory routines (templar_amd/csrc/tplr_host.cpp) on
// buffers of exactly the sizes their contract names, so that AddressSanitizer sees any byte read or written
// past them.  Exit status 0 and the line "ok <cases>" on success.
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <random>
#include <vector>

#include "tplr_hip.h"

#define CHECK(c)                                                   \
    do {                                                           \
        if (!(c)) {                                                \
            fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, #c); \
            return 1;                                              \
        }                                                          \
    } while (0)

int main() {
    std::mt19937_64 rng(12345);
    int cases = 0;
    // pack -> unpack round trips on exact-size heap buffers, sizes 0 .. a few thousand
    for (int rep = 0; rep < 300; ++rep) {
        const int64_t n = 2 * static_cast<int64_t>(rng() % 1500);
        int64_t* idx = static_cast<int64_t*>(malloc(n * 8 + 1));
        uint8_t* packed = static_cast<uint8_t*>(malloc(n / 2 * 3 + 1));
        int64_t* back = static_cast<int64_t*>(malloc(n * 8 + 1));
        for (int64_t i = 0; i < n; ++i) idx[i] = static_cast<int64_t>(rng() % 4096);
        int64_t bad = -1;
        CHECK(tplr_pack12_host(idx, n, packed, &bad) == 0);
        CHECK(n == 0 || bad == 0);
        CHECK(tplr_unpack12_host(packed, n, back) == 0);
        CHECK(memcmp(idx, back, n * 8) == 0);
        if (n) {  // an index past 12 bits is reported, not written past the buffer
            idx[n - 1] = 5000;
            CHECK(tplr_pack12_host(idx, n, packed, &bad) == 0 && bad == 5000);
        }
        CHECK(tplr_pack12_host(idx, n + 1, packed, &bad) == TPLR_E_ODD);
        free(idx); free(packed); free(back);
        ++cases;
    }
    CHECK(tplr_pack12_host(nullptr, 2, nullptr, nullptr) == TPLR_E_BADARG);
    CHECK(tplr_unpack12_host(nullptr, 2, nullptr) == TPLR_E_BADARG);
    CHECK(tplr_unpack12_host(nullptr, -2, nullptr) == TPLR_E_BADARG);
    // gather: random part sizes (zero-sized ones included), every thread count, small and large totals
    for (int rep = 0; rep < 120; ++rep) {
        const int64_t parts = 1 + static_cast<int64_t>(rng() % 40);
        const bool large = rep % 10 == 0;  // past the size where the copy is spread over threads
        std::vector<void*> src(parts);
        std::vector<int64_t> bytes(parts);
        int64_t total = 0;
        for (int64_t i = 0; i < parts; ++i) {
            bytes[i] = rng() % 5 == 0 ? 0 : static_cast<int64_t>(rng() % (large ? 300000 : 3000));
            src[i] = bytes[i] ? malloc(bytes[i]) : nullptr;
            for (int64_t b = 0; b < bytes[i]; ++b) static_cast<uint8_t*>(src[i])[b] = static_cast<uint8_t>(rng());
            total += bytes[i];
        }
        uint8_t* dst = static_cast<uint8_t*>(malloc(total + 1));
        const int threads = 1 + static_cast<int>(rng() % 64);
        CHECK(tplr_gather_host(src.data(), bytes.data(), parts, dst, threads) == 0);
        int64_t at = 0;
        for (int64_t i = 0; i < parts; ++i) {
            CHECK(bytes[i] == 0 || memcmp(dst + at, src[i], bytes[i]) == 0);
            at += bytes[i];
        }
        for (void* p : src) free(p);
        free(dst);
        ++cases;
    }
    int64_t one = 4;
    const void* null_part = nullptr;
    uint8_t sink[4];
    CHECK(tplr_gather_host(&null_part, &one, 1, sink, 1) == TPLR_E_BADARG);
    CHECK(tplr_gather_host(&null_part, &one, 1, sink, 65) == TPLR_E_BADARG);
    CHECK(tplr_gather_host(nullptr, nullptr, 0, nullptr, 1) == 0);
    printf("ok %d\n", cases);
    return 0;
}
