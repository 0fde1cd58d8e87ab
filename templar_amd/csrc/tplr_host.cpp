// The routines of libtplr_hip.so that touch host memory only (declared in include/tplr_hip.h): the 12-bit
// pack and unpack of downloaded payloads and the threaded concatenation into a pinned staging buffer.
// Plain C++ with no device code, so that it also builds with the host compiler alone (sanitizer runs).
#include <stdint.h>
#include <string.h>

#include <thread>
#include <vector>

#include "../../include/tplr_hip.h"

extern "C" {

int tplr_pack12_host(const int64_t* idx, int64_t n, uint8_t* packed, int64_t* bad) {
    if (n < 0) return TPLR_E_BADARG;
    if (n & 1) return TPLR_E_ODD;
    if (n == 0) return 0;
    if (!idx || !packed) return TPLR_E_BADARG;
    int64_t worst = 0;
    for (int64_t p = 0; p < n / 2; ++p) {
        const int64_t a = idx[2 * p], b = idx[2 * p + 1];
        worst = a > worst ? a : worst;
        worst = b > worst ? b : worst;
        const uint32_t w = (static_cast<uint32_t>(a) & 0xfffu) | ((static_cast<uint32_t>(b) & 0xfffu) << 12);
        packed[3 * p] = static_cast<uint8_t>(w);
        packed[3 * p + 1] = static_cast<uint8_t>(w >> 8);
        packed[3 * p + 2] = static_cast<uint8_t>(w >> 16);
    }
    if (bad) *bad = worst > 4095 ? worst : 0;
    return 0;
}

int tplr_gather_host(const void* const* h_src, const int64_t* h_bytes, int64_t n_parts, void* h_dst,
                     int n_threads) {
    if (n_parts < 0 || n_threads < 1 || n_threads > 64) return TPLR_E_BADARG;
    if (n_parts == 0) return 0;
    if (!h_src || !h_bytes || !h_dst) return TPLR_E_BADARG;
    int64_t total = 0;
    for (int64_t i = 0; i < n_parts; ++i) {
        if (h_bytes[i] < 0 || (h_bytes[i] > 0 && !h_src[i])) return TPLR_E_BADARG;
        total += h_bytes[i];
    }
    // every thread copies an equal share of the concatenated bytes, cutting parts where its share ends
    auto work = [=](int t) {
        const int64_t lo = total * t / n_threads, hi = total * (t + 1) / n_threads;
        int64_t at = 0;
        for (int64_t i = 0; i < n_parts && at < hi; at += h_bytes[i], ++i) {
            const int64_t b = at > lo ? at : lo, e = at + h_bytes[i] < hi ? at + h_bytes[i] : hi;
            if (b < e)
                memcpy(static_cast<char*>(h_dst) + b, static_cast<const char*>(h_src[i]) + (b - at),
                       static_cast<size_t>(e - b));
        }
    };
    if (n_threads == 1 || total < (1 << 20)) {
        for (int t = 0; t < n_threads; ++t) work(t);
        return 0;
    }
    std::vector<std::thread> pool;
    pool.reserve(n_threads - 1);
    for (int t = 1; t < n_threads; ++t) pool.emplace_back(work, t);
    work(0);
    for (auto& th : pool) th.join();
    return 0;
}

int tplr_unpack12_host(const uint8_t* packed, int64_t n, int64_t* idx) {
    if (n < 0) return TPLR_E_BADARG;
    if (n & 1) return TPLR_E_ODD;
    if (n == 0) return 0;
    if (!idx || !packed) return TPLR_E_BADARG;
    for (int64_t p = 0; p < n / 2; ++p) {
        const uint32_t w = packed[3 * p] | (static_cast<uint32_t>(packed[3 * p + 1]) << 8) |
                           (static_cast<uint32_t>(packed[3 * p + 2]) << 16);
        idx[2 * p] = w & 0xfffu;
        idx[2 * p + 1] = w >> 12;
    }
    return 0;
}

}  // extern "C"
