// Test infrastructure: drives the host-only part of the C ABI (csrc/tq_host.cpp: size arithmetic, decision thresholds,
// codec-table and QJL-table builders, table check, host-side quantiser) over every bit width and several head
// dimensions.  tests/test_host.py builds it together with tq_host.cpp under -fsanitize=address,undefined and runs it:
// an out-of-bounds write in a table builder would otherwise only show as a wrong code on the GPU.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../../include/tqamd.h"

static unsigned long long state = 0x2545f4914f6cdd1dull;
static float rnd() {
    state ^= state << 13; state ^= state >> 7; state ^= state << 17;
    return (float)((double)(state >> 11) / 9007199254740992.0 * 2.0 - 1.0);
}

int main() {
    if (tq_abi_version() <= 0 || !tq_status_string(0) || !tq_status_string(-3) || !tq_status_string(-99)) return 1;
    const int dims[] = {8, 32, 45, 64, 80, 96, 100, 128, 160, 255, 256};
    for (int D : dims) {
        std::vector<float> Pi((size_t)D * D), S((size_t)D * D);
        for (auto &v : Pi) v = rnd() / std::sqrt((float)D);
        for (auto &v : S) v = 3.f * rnd();
        for (int bits = 1; bits <= 8; ++bits) {
            const int levels = 1 << bits;
            std::vector<float> cent((size_t)levels), thr((size_t)levels);
            for (int i = 0; i < levels; ++i) cent[i] = (-1.f + 2.f * (i + 0.5f) / levels) * 3.f / std::sqrt((float)D);
            if (tq_decision_thresholds(cent.data(), levels, thr.data())) { std::fprintf(stderr, "thresholds D=%d b=%d\n", D, bits); return 1; }
            if (tq_bytes_per_vector(D, bits) <= 0) return 1;
            const long long n = tq_table_bytes(D, bits);
            if (n <= 0) { std::fprintf(stderr, "table_bytes D=%d b=%d -> %lld\n", D, bits, n); return 1; }
            std::vector<uint8_t> blob((size_t)n);      // exactly the size asked for: a write past it is caught
            int rc = tq_table_build(Pi.data(), cent.data(), D, bits, blob.data(), blob.size());
            if (rc) { std::fprintf(stderr, "table_build D=%d b=%d -> %d\n", D, bits, rc); return 1; }
            if (tq_table_check(blob.data(), blob.size(), D, bits)) return 1;
            if (!tq_table_check(blob.data(), blob.size(), D, bits == 8 ? 7 : bits + 1)) return 1;
            if (!tq_table_check(blob.data(), 100, D, bits)) return 1;
            std::vector<float> r(4096);
            std::vector<uint8_t> idx(r.size());
            for (auto &v : r) v = 1.2f * rnd();
            r[0] = 0.f; r[1] = 1.f; r[2] = -1.f; r[3] = INFINITY; r[4] = -INFINITY; r[5] = NAN; r[6] = 1e-30f;
            if (tq_table_quantize_host(blob.data(), r.data(), (long long)r.size(), idx.data())) return 1;
            for (size_t i = 0; i < r.size(); ++i) {        // against the definition: first nearest centroid
                if (!std::isfinite(r[i]) || std::fabs(r[i]) > 1.0f) continue;
                int best = 0;
                for (int j = 1; j < levels; ++j)
                    if (std::fabs(r[i] - cent[j]) < std::fabs(r[i] - cent[best])) best = j;
                if (idx[i] != best) { std::fprintf(stderr, "quantize D=%d b=%d r=%g: %d != %d\n", D, bits, r[i], idx[i], best); return 1; }
            }
            if (D == 128 && bits <= 7) {
                const long long nq = tq_qjl_table_bytes(D, bits);
                if (nq <= 0) return 1;
                std::vector<uint8_t> q((size_t)nq);
                rc = tq_qjl_table_build(Pi.data(), S.data(), cent.data(), D, bits, q.data(), q.size());
                if (rc) { std::fprintf(stderr, "qjl_table_build b=%d -> %d\n", bits, rc); return 1; }
            }
        }
    }
    if (tq_table_bytes(7, 4) >= 0 || tq_table_bytes(257, 4) >= 0 || tq_table_bytes(128, 9) >= 0 || tq_qjl_table_bytes(64, 3) >= 0) return 1;
    std::puts("ok");
    return 0;
}
