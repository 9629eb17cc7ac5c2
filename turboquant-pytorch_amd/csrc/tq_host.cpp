// Host side of the C ABI: status strings, size arithmetic, decision thresholds and the
// codec-table builder.  No device code here.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "../../include/tqamd.h"
#include "tq_table.h"

namespace {

// ---- float <-> 16-bit formats, round to nearest even ------------------------------------
inline uint32_t f32_bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float bits_f32(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

uint16_t to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
float from_bf16(uint16_t h) { return bits_f32((uint32_t)h << 16); }

uint16_t to_f16(float f) {
    const uint32_t x = f32_bits(f);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t ex = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (ex == 0xffu) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u | (man >> 13) : 0u));
    const int e = (int)ex - 112;  // rebias 127 -> 15
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        const uint32_t shift = (uint32_t)(14 - e);
        uint32_t h = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) ++h;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((uint32_t)e << 10) | (man >> 13);
    const uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;
    return (uint16_t)(sign | h);
}
float from_f16(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t ex = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (ex == 0) {
        if (!man) return bits_f32(sign);
        int s = 0;
        while (!(man & 0x400u)) { man <<= 1; ++s; }
        return bits_f32(sign | ((uint32_t)(113 - s) << 23) | ((man & 0x3ffu) << 13));
    }
    if (ex == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
    return bits_f32(sign | ((ex + 112u) << 23) | (man << 13));
}

// ---- totally ordered integer key of a float (for binary searches over float values) -----
inline int64_t fkey(float f) {
    const uint32_t u = f32_bits(f);
    return (u & 0x80000000u) ? -(int64_t)(u & 0x7fffffffu) : (int64_t)u;
}
inline float fkey_inv(int64_t k) {
    return k < 0 ? bits_f32(0x80000000u | (uint32_t)(-k)) : bits_f32((uint32_t)k);
}

inline uint32_t round_up(uint32_t v, uint32_t a) { return (v + a - 1) / a * a; }

bool valid_codebook(const float *c, int levels) {
    for (int i = 0; i < levels; ++i) {
        if (!std::isfinite(c[i])) return false;
        if (i && !(c[i] > c[i - 1])) return false;
    }
    return true;
}

// smallest float r in (lo, hi] for which the upper centroid is strictly nearer in float math
float threshold_between(float lo, float hi) {
    auto upper_wins = [&](float r) { return std::fabs(r - hi) < std::fabs(r - lo); };
    int64_t a = fkey(lo), b = fkey(hi);  // upper_wins(lo) is false, upper_wins(hi) is true
    while (b - a > 1) {
        const int64_t m = a + (b - a) / 2;
        if (upper_wins(fkey_inv(m))) b = m; else a = m;
    }
    return fkey_inv(b);
}

inline uint32_t grid_cell(float r, float scale, float bias) {
    return (f32_bits(std::fmaf(r, scale, bias)) & TQ_GRID_ADDR_MASK) >> 3;
}

struct Layout {
    uint32_t off_a_f16, off_a_bf16, off_grid, off_at_f16, off_lut, off_centroids, off_thresholds, total;
    uint32_t lut_entry_bytes;
    uint32_t off_pair_a_f16, off_pair_a_bf16, off_pair_at_f16;     // head_dim 64: room for the operands of diag(Pi, Pi)
};
// head dimensions the kernels take: 128 (the tuned kernels) and every other one from 8 to 256
bool supported_head_dim(int d) { return d >= TQ_ANYDIM_MIN && d <= TQ_ANYDIM_MAX; }

Layout layout_for(int head_dim, int bits) {
    const uint32_t levels = 1u << bits, ipb = 8u / (uint32_t)bits;
    const uint32_t operand = (uint32_t)TQ_OPERAND_BYTES_FOR(head_dim);
    Layout L{};
    uint32_t off = sizeof(TqTableHeader);
    L.off_a_f16 = off;      off += 2 * operand;
    L.off_a_bf16 = off;     off += 3 * operand;
    L.off_at_f16 = off;     off += 2 * operand;
    L.off_grid = off;       off += round_up(TQ_GRID_LDS_BYTES, 256);
    L.lut_entry_bytes = 2 * ipb;
    L.off_lut = off;        off += round_up(256 * L.lut_entry_bytes, 256);
    L.off_centroids = off;  off += round_up(levels * 4, 256);
    L.off_thresholds = off; off += round_up(levels * 4, 256);
    if (head_dim == TQ_HEAD_DIM / 2) {
        L.off_pair_a_f16 = off;  off += 2 * TQ_OPERAND_BYTES;
        L.off_pair_a_bf16 = off; off += 3 * TQ_OPERAND_BYTES;
        L.off_pair_at_f16 = off; off += 2 * TQ_OPERAND_BYTES;
    }
    L.total = off;
    return L;
}

}  // namespace

extern "C" {

int tq_abi_version(void) { return TQ_ABI_VERSION; }

const char *tq_status_string(int status) {
    switch (status) {
        case TQ_OK: return "ok";
        case TQ_ERR_NULL: return "null pointer argument";
        case TQ_ERR_BITS: return "bits must be in 1..8";
        case TQ_ERR_HEAD_DIM: return "unsupported head_dim (compress / decompress: 8 to 256; the other kernels: 128)";
        case TQ_ERR_DTYPE: return "unknown element type";
        case TQ_ERR_SIZE: return "invalid size or stride";
        case TQ_ERR_CODEBOOK: return "centroids must be finite and strictly ascending";
        case TQ_ERR_TABLE: return "malformed codec table";
        case TQ_ERR_ALIGN: return "pointer or stride not 16-byte aligned";
        case TQ_ERR_NO_DEVICE: return "no usable HIP device";
        case TQ_ERR_CAPACITY: return "request exceeds the fixed capacity of an entry point that allocates nothing";
        default: break;
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown status";
}

int tq_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

int tq_bytes_per_vector(int head_dim, int bits) {
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    if (head_dim < 1) return TQ_ERR_HEAD_DIM;
    const int ipb = 8 / bits;
    return (head_dim + ipb - 1) / ipb;
}

int tq_decision_thresholds(const float *centroids, int levels, float *thresholds) {
    if (!centroids || (levels > 1 && !thresholds)) return TQ_ERR_NULL;
    if (levels < 1 || levels > 256) return TQ_ERR_SIZE;
    if (!valid_codebook(centroids, levels)) return TQ_ERR_CODEBOOK;
    for (int i = 0; i + 1 < levels; ++i) thresholds[i] = threshold_between(centroids[i], centroids[i + 1]);
    return TQ_OK;
}

long long tq_table_bytes(int head_dim, int bits) {
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    if (!supported_head_dim(head_dim)) return TQ_ERR_HEAD_DIM;
    return layout_for(head_dim, bits).total;
}

int tq_table_build(const float *Pi, const float *centroids, int head_dim, int bits,
                   void *table_host, size_t table_bytes) {
    if (!Pi || !centroids || !table_host) return TQ_ERR_NULL;
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    if (!supported_head_dim(head_dim)) return TQ_ERR_HEAD_DIM;
    const Layout L = layout_for(head_dim, bits);
    if (table_bytes < L.total) return TQ_ERR_SIZE;
    const int levels = 1 << bits;
    const int D = head_dim;
    const bool tuned = D == TQ_HEAD_DIM;   // the 128-wide kernels have their own decompress tiling and keep shifted grid copies
    const bool tuned_grid = tuned || D == TQ_HEAD_DIM / 2;     // 64-wide vectors go through them in pairs: the same grid limit
    if (!valid_codebook(centroids, levels)) return TQ_ERR_CODEBOOK;
    for (int i = 0; i < D * D; ++i)
        if (!std::isfinite(Pi[i])) return TQ_ERR_SIZE;

    uint8_t *blob = static_cast<uint8_t *>(table_host);
    std::memset(blob, 0, L.total);

    // ---- thresholds ----
    std::vector<float> thr((size_t)levels);
    thr[levels - 1] = INFINITY;
    if (levels > 1) {
        const int rc = tq_decision_thresholds(centroids, levels, thr.data());
        if (rc) return rc;
    }
    std::memcpy(blob + L.off_centroids, centroids, (size_t)levels * 4);
    std::memcpy(blob + L.off_thresholds, thr.data(), (size_t)(levels - 1) * 4);

    // ---- quantiser grid: smallest power-of-two resolution with <= 1 threshold per cell ----
    // Cell k covers the reals [edge(k), edge(k+1)), edge(k) = (k - cells/2 - 1/16) / scale (see
    // tq_table.h); unit-sphere coordinates satisfy |rho| <= 1 + rounding, the grid spans +-1.0625.
    const double range = 1.0625;
    // Thresholds outside the span cannot be met by a coordinate of a unit vector (the codebooks of very small head
    // dimensions at 6 to 8 bits reach beyond +-1): those below count for every coordinate, those above for none.
    int t_first = 0, t_end = levels - 1;
    while (t_first < t_end && (double)thr[t_first] < -range) ++t_first;
    while (t_end > t_first && (double)thr[t_end - 1] > range) --t_end;
    float scale = 0.f, bias = 0.f;
    uint32_t cells = 0;
    std::vector<TqGridCell> grid;
    bool ok = false;
    for (int lg = 3; lg <= 12 && !ok; ++lg) {
        scale = (float)(1 << lg);
        cells = 2u * (uint32_t)std::ceil(range * scale);
        if (cells > (uint32_t)(tuned_grid ? TQ_GRID_MAX_CELLS(bits) : TQ_GRID_LDS_BYTES / 8)) break;
        bias = (float)(cells / 2) + TQ_GRID_MAGIC;
        grid.assign(cells, TqGridCell{INFINITY, 0});
        auto edge = [&](uint32_t k) { return ((double)k - (double)(cells / 2) - 0.0625) / (double)scale; };
        ok = true;
        int t = t_first;  // thresholds are ascending; walk them alongside the cells
        for (uint32_t q = 0; q < cells && ok; ++q) {
            const double lo = q == 0 ? -INFINITY : edge(q), hi = q + 1 == cells ? INFINITY : edge(q + 1);
            while (t < t_end && (double)thr[t] < lo) ++t;   // below the cell: counted for all of it
            grid[q].base = (uint32_t)t;
            int inside = 0;
            while (t + inside < t_end && (double)thr[t + inside] < hi) ++inside;
            if (inside > 1) { ok = false; break; }
            if (inside == 1) grid[q].threshold = thr[t];
        }
    }
    if (!ok) return TQ_ERR_CODEBOOK;  // levels too dense for the grid the kernels keep in LDS
    std::memcpy(blob + L.off_grid, grid.data(), (size_t)cells * sizeof(TqGridCell));

    // ---- rotation operands (of the rotation extended by zeros to a multiple of 32) ----
    const int DP = TQ_PADDED_DIM(D);
    const int tiles = DP / 32, steps = DP / 16;
    auto pi_at = [&](int row, int col) { return (row < D && col < D) ? Pi[row * D + col] : 0.0f; };
    auto operand_index = [steps](int t, int s, int l, int i) { return (((size_t)t * steps + s) * 64 + l) * 8 + i; };
    uint16_t *a_f16 = reinterpret_cast<uint16_t *>(blob + L.off_a_f16);
    uint16_t *a_bf16 = reinterpret_cast<uint16_t *>(blob + L.off_a_bf16);
    uint16_t *at_f16 = reinterpret_cast<uint16_t *>(blob + L.off_at_f16);
    const size_t term = (size_t)TQ_OPERAND_BYTES_FOR(D) / 2;  // halves per operand set
    const double pi_scale = (double)(1 << TQ_F16_PI_SHIFT);
    for (int t = 0; t < tiles; ++t)
        for (int s = 0; s < steps; ++s)
            for (int l = 0; l < 64; ++l) {
                const int m = l % 32, hk = l / 32;
                // MFMA row m = 8a + 4h + b  <->  accumulator register r = 4a + b of lane-half h
                const int a = m / 8, h = (m / 4) % 2, b = m % 4;
                const int out_c = 32 * t + 16 * h + 4 * a + b;                        // compress (see tq_table.h)
                const int out_d = tuned ? 64 * h + 16 * t + 4 * a + b : out_c;        // decompress
                for (int i = 0; i < 8; ++i) {
                    const size_t o = operand_index(t, s, l, i);
                    {   // compress: rotated[out] = sum_k x[k] * Pi[out][k],  k = 16s + 8hk + i
                        const int k = 16 * s + 8 * hk + i;
                        const float p = pi_at(out_c, k);
                        const double ps = (double)p * pi_scale;
                        const uint16_t hi = to_f16((float)ps);
                        const uint16_t lo = to_f16((float)(ps - (double)from_f16(hi)));
                        a_f16[o] = hi;
                        a_f16[term + o] = lo;
                        const uint16_t b0 = to_bf16(p);
                        const float r1 = p - from_bf16(b0);
                        const uint16_t b1 = to_bf16(r1);
                        const float r2 = r1 - from_bf16(b1);
                        a_bf16[o] = b0;
                        a_bf16[term + o] = b1;
                        a_bf16[2 * term + o] = to_bf16(r2);
                    }
                    {   // decompress: x[out] = sum_j y[j] * Pi[j][out],  j = 64hk + 8s + i
                        const int j = tuned ? 64 * hk + 8 * s + i : 16 * s + 8 * hk + i;
                        const float p = pi_at(j, out_d);
                        const uint16_t hi = to_f16(p);
                        at_f16[o] = hi;
                        at_f16[term + o] = to_f16((float)((double)p - (double)from_f16(hi)));
                    }
                }
            }

    // ---- head_dim 64: the same operand sets for diag(Pi, Pi) in the tilings of the 128-wide kernels ----
    const bool paired = D == TQ_HEAD_DIM / 2 && cells <= (uint32_t)TQ_GRID_MAX_CELLS(bits);
    if (paired) {
        const int W = TQ_HEAD_DIM;
        auto pp = [&](int row, int col) { return (row / D == col / D) ? Pi[(row % D) * D + (col % D)] : 0.0f; };   // diag(Pi, Pi)[row][col]
        uint16_t *pa_f16 = reinterpret_cast<uint16_t *>(blob + L.off_pair_a_f16);
        uint16_t *pa_bf16 = reinterpret_cast<uint16_t *>(blob + L.off_pair_a_bf16);
        uint16_t *pat_f16 = reinterpret_cast<uint16_t *>(blob + L.off_pair_at_f16);
        const size_t pterm = (size_t)TQ_OPERAND_BYTES / 2;
        for (int t = 0; t < TQ_TILES; ++t)
            for (int s = 0; s < TQ_STEPS; ++s)
                for (int l = 0; l < 64; ++l) {
                    const int m = l % 32, hk = l / 32;
                    const int a = m / 8, h = (m / 4) % 2, b = m % 4;
                    const int out_c = 32 * t + 16 * h + 4 * a + b;
                    const int out_d = 64 * h + 16 * t + 4 * a + b;
                    for (int i = 0; i < 8; ++i) {
                        const size_t o = (((size_t)t * TQ_STEPS + s) * 64 + l) * 8 + i;
                        {
                            const float p = pp(out_c, 16 * s + 8 * hk + i);
                            const double ps = (double)p * pi_scale;
                            const uint16_t hi = to_f16((float)ps);
                            pa_f16[o] = hi;
                            pa_f16[pterm + o] = to_f16((float)(ps - (double)from_f16(hi)));
                            const uint16_t b0 = to_bf16(p);
                            const float r1 = p - from_bf16(b0);
                            const uint16_t b1 = to_bf16(r1);
                            pa_bf16[o] = b0;
                            pa_bf16[pterm + o] = b1;
                            pa_bf16[2 * pterm + o] = to_bf16((r1 - from_bf16(b1)));
                        }
                        {
                            const float p = pp(64 * hk + 8 * s + i, out_d);
                            const uint16_t hi = to_f16(p);
                            pat_f16[o] = hi;
                            pat_f16[pterm + o] = to_f16((float)((double)p - (double)from_f16(hi)));
                        }
                    }
                }
        (void)W;
    }

    // ---- decode table: byte value -> the ipb centroids it holds (MSB-first), as fp16 ----
    const int ipb = 8 / bits;
    const unsigned mask = (1u << bits) - 1u;
    uint16_t *lut = reinterpret_cast<uint16_t *>(blob + L.off_lut);
    for (int v = 0; v < 256; ++v)
        for (int k = 0; k < ipb; ++k)
            lut[v * ipb + k] = to_f16(centroids[((unsigned)v >> (bits * (ipb - 1 - k))) & mask]);

    TqTableHeader hd{};
    hd.magic = TQ_TABLE_MAGIC;
    hd.version = TQ_TABLE_VERSION;
    hd.head_dim = (uint32_t)D;
    hd.bits = (uint32_t)bits;
    hd.levels = (uint32_t)levels;
    hd.ipb = (uint32_t)ipb;
    hd.bytes_per_vec = (uint32_t)((D + ipb - 1) / ipb);
    hd.grid_cells = cells;
    hd.grid_scale = scale;
    hd.grid_bias = bias;
    hd.total_bytes = L.total;
    hd.off_a_f16 = L.off_a_f16;
    hd.off_a_bf16 = L.off_a_bf16;
    hd.off_grid = L.off_grid;
    hd.off_at_f16 = L.off_at_f16;
    hd.off_lut = L.off_lut;
    hd.off_pair_a_f16 = paired ? L.off_pair_a_f16 : 0u;
    hd.off_pair_a_bf16 = paired ? L.off_pair_a_bf16 : 0u;
    hd.off_pair_at_f16 = paired ? L.off_pair_at_f16 : 0u;
    hd.padded_dim = (uint32_t)DP;
    hd.off_centroids = L.off_centroids;
    hd.off_thresholds = L.off_thresholds;
    hd.lut_entry_bytes = L.lut_entry_bytes;
    std::memcpy(blob, &hd, sizeof(hd));
    return TQ_OK;
}

long long tq_qjl_table_bytes(int head_dim, int mse_bits) {
    if (head_dim != TQ_HEAD_DIM) return TQ_ERR_HEAD_DIM;
    if (mse_bits < 1 || mse_bits > 7) return TQ_ERR_BITS;
    return (long long)sizeof(TqQjlHeader) + 6ll * TQ_OPERAND_BYTES + 2048;
}

int tq_qjl_table_build(const float *Pi, const float *S, const float *centroids, int head_dim, int mse_bits,
                       void *table_host, size_t table_bytes) {
    if (!Pi || !S || !centroids || !table_host) return TQ_ERR_NULL;
    const long long need = tq_qjl_table_bytes(head_dim, mse_bits);
    if (need < 0) return (int)need;
    if (table_bytes < (size_t)need) return TQ_ERR_SIZE;
    const int D = head_dim, levels = 1 << mse_bits;
    if (!valid_codebook(centroids, levels)) return TQ_ERR_CODEBOOK;
    for (int i = 0; i < D * D; ++i)
        if (!std::isfinite(Pi[i]) || !std::isfinite(S[i])) return TQ_ERR_SIZE;
    // power of two that puts the largest magnitude of v[0..n) into [2^13, 2^14) (all zeros: 1)
    auto shift_for = [](const float *v, size_t n) {
        float m = 0.f;
        for (size_t i = 0; i < n; ++i) m = std::fmax(m, std::fabs(v[i]));
        if (!(m > 0.f)) return 0;
        int e = 0;
        (void)std::frexp(m, &e);           // m = f * 2^e, f in [0.5, 1)
        const int sh = 14 - e;
        return sh < -100 ? -100 : sh > 100 ? 100 : sh;
    };
    const int sh_pit = shift_for(Pi, (size_t)D * D), sh_s = shift_for(S, (size_t)D * D), sh_c = shift_for(centroids, (size_t)levels);
    auto split = [](float v, int sh, uint16_t &hi, uint16_t &lo) {
        const double x = std::ldexp((double)v, sh);
        hi = to_f16((float)x);
        lo = to_f16((float)(x - (double)from_f16(hi)));
    };
    uint8_t *blob = static_cast<uint8_t *>(table_host);
    std::memset(blob, 0, (size_t)need);
    TqQjlHeader hd{};
    hd.magic = TQ_QJL_MAGIC;
    hd.version = TQ_QJL_VERSION;
    hd.head_dim = (uint32_t)D;
    hd.mse_bits = (uint32_t)mse_bits;
    hd.levels = (uint32_t)levels;
    hd.off_pit = sizeof(TqQjlHeader);
    hd.off_s = hd.off_pit + 2 * TQ_OPERAND_BYTES;
    hd.off_centroids = hd.off_s + 2 * TQ_OPERAND_BYTES;
    hd.off_m = hd.off_centroids + 1024;
    hd.off_cent_f32 = hd.off_m + 2 * TQ_OPERAND_BYTES;
    hd.total_bytes = (uint32_t)need;
    hd.k_scale = std::ldexp(1.0f, -(sh_pit + sh_c));
    uint16_t *pit = reinterpret_cast<uint16_t *>(blob + hd.off_pit);
    uint16_t *sm = reinterpret_cast<uint16_t *>(blob + hd.off_s);
    const size_t term = TQ_OPERAND_BYTES / 2;
    for (int t = 0; t < TQ_TILES; ++t)
        for (int s = 0; s < TQ_STEPS; ++s)
            for (int l = 0; l < 64; ++l) {
                const int m = l % 32, hk = l / 32;
                const int a = m / 8, h = (m / 4) % 2, b = m % 4;
                const int out = 32 * t + 16 * h + 4 * a + b;
                for (int i = 0; i < 8; ++i) {
                    const size_t o = (((size_t)t * TQ_STEPS + s) * 64 + l) * 8 + i;
                    const int k = 16 * s + 8 * hk + i;
                    split(Pi[k * D + out], sh_pit, pit[o], pit[term + o]);      // Pi^T[out][k]
                    split(S[out * D + k], sh_s, sm[o], sm[term + o]);
                }
            }
    uint32_t *pairs = reinterpret_cast<uint32_t *>(blob + hd.off_centroids);
    float *cent_f32 = reinterpret_cast<float *>(blob + hd.off_cent_f32);
    for (int i = 0; i < levels; ++i) {
        uint16_t hi, lo;
        split(centroids[i], sh_c, hi, lo);
        pairs[i] = (uint32_t)hi | ((uint32_t)lo << 16);
        cent_f32[i] = centroids[i];
    }
    {   // M = S Pi^T in double precision, then the same two-term tiles (only the sign of the projection is used: any scale does)
        std::vector<double> m((size_t)D * D);
        std::vector<float> mf((size_t)D * D);
        for (int out = 0; out < D; ++out)
            for (int k = 0; k < D; ++k) {
                double acc = 0.0;
                for (int j = 0; j < D; ++j) acc += (double)S[out * D + j] * (double)Pi[k * D + j];
                m[(size_t)out * D + k] = acc;
                mf[(size_t)out * D + k] = (float)acc;
            }
        const int sh_m = shift_for(mf.data(), (size_t)D * D);
        uint16_t *mm = reinterpret_cast<uint16_t *>(blob + hd.off_m);
        for (int t = 0; t < TQ_TILES; ++t)
            for (int s = 0; s < TQ_STEPS; ++s)
                for (int l = 0; l < 64; ++l) {
                    const int mrow = l % 32, hk = l / 32;
                    const int a = mrow / 8, h = (mrow / 4) % 2, b = mrow % 4;
                    const int out = 32 * t + 16 * h + 4 * a + b;
                    for (int i = 0; i < 8; ++i) {
                        const size_t o = (((size_t)t * TQ_STEPS + s) * 64 + l) * 8 + i;
                        const int k = 16 * s + 8 * hk + i;
                        const double x = std::ldexp(m[(size_t)out * D + k], sh_m);
                        mm[o] = to_f16((float)x);
                        mm[term + o] = to_f16((float)(x - (double)from_f16(mm[o])));
                    }
                }
    }
    std::memcpy(blob, &hd, sizeof(hd));
    return TQ_OK;
}

int tq_table_check(const void *table_host, size_t table_bytes, int head_dim, int bits) {
    if (!table_host) return TQ_ERR_NULL;
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    if (table_bytes < sizeof(TqTableHeader)) return TQ_ERR_TABLE;
    TqTableHeader hd;
    std::memcpy(&hd, table_host, sizeof(hd));
    if (hd.magic != TQ_TABLE_MAGIC || hd.version != TQ_TABLE_VERSION) return TQ_ERR_TABLE;
    if (hd.total_bytes > table_bytes || (long long)hd.total_bytes != tq_table_bytes((int)hd.head_dim, (int)hd.bits)) return TQ_ERR_TABLE;
    if ((int)hd.head_dim != head_dim || (int)hd.bits != bits) return TQ_ERR_TABLE;
    return TQ_OK;
}

int tq_table_quantize_host(const void *table_host, const float *r, long long n, uint8_t *idx) {
    if (!table_host || (n > 0 && (!r || !idx))) return TQ_ERR_NULL;
    TqTableHeader hd;
    std::memcpy(&hd, table_host, sizeof(hd));
    if (hd.magic != TQ_TABLE_MAGIC || hd.version != TQ_TABLE_VERSION) return TQ_ERR_TABLE;
    const TqGridCell *grid =
        reinterpret_cast<const TqGridCell *>(static_cast<const uint8_t *>(table_host) + hd.off_grid);
    for (long long i = 0; i < n; ++i) {
        const uint32_t q = grid_cell(r[i], hd.grid_scale, hd.grid_bias);
        const TqGridCell c = grid[q < hd.grid_cells ? q : 0];
        // the kernels evaluate fma(acc, inv, -threshold) >= 0; with acc = r, inv = 1 that is r - threshold
        idx[i] = (uint8_t)(c.base + (std::fmaf(r[i], 1.0f, -c.threshold) >= 0.0f ? 1u : 0u));
    }
    return TQ_OK;
}

}  // extern "C"
