// compress and decompress for head dimensions other than 128: any multiple of 32 from 32 to 256, taken at run
// time (upstream turboquant/compressors_v3.py:37-43 builds its rotation and codebook for whatever head_dim it
// is given; :46-81 compress, :84-105 decompress).  Same arithmetic as the 128-wide kernels (split rotation on the
// matrix cores, fp32 accumulation, norm applied after the rotation, threshold-grid code search, MSB-first packing,
// fp16 centroids on the way back), in a plain form: no register-resident rotation, no software pipeline.
//
// A block (four waves) works on groups of nt x 32 consecutive vectors (nt = 4, or fewer where that lets a second block
// share the compute unit's LDS).  The group is staged in LDS as 16-bit MFMA operands
// (compress: the input itself, fp32 inputs as three exact bf16 terms; decompress: the centroids of the codes as
// fp16); wave w then produces the row tiles w, w + waves, ... of the rotation (32 output coordinates each) for
// all NT column tiles, reading its A operands from the table in memory (they stay in L2: one 16-byte load per
// lane feeds NT matrix instructions per term) and the B operands from LDS.  Every lane ends up with 16
// consecutive coordinates of one vector per column tile, exactly as in the 128-wide compress kernel.
#include <mutex>
#include <type_traits>

#include "tq_anydim.h"

namespace {

constexpr int ROW_PAD = 8;      // halves appended to every staged row: rows stay 16-byte aligned and rotate over the banks
constexpr int MAX_WAVES = 4;

template <int DTYPE> struct AnyIn;
template <> struct AnyIn<TQ_F16> { static constexpr int ELEM = 2, XTERMS = 1, ATERMS = 2, NT = 4; };
template <> struct AnyIn<TQ_BF16> { static constexpr int ELEM = 2, XTERMS = 1, ATERMS = 2, NT = 4; };
template <> struct AnyIn<TQ_F32> { static constexpr int ELEM = 4, XTERMS = 3, ATERMS = 3, NT = 2; };

constexpr int DEC_NT = 4;       // column tiles per group of the decompress kernel

__host__ __device__ constexpr uint32_t align16(uint32_t v) { return (v + 15u) & ~15u; }

// LDS of the compress kernel: quantiser grid | per-piece sums of squares | per-vector sums | staged operand terms
template <int DTYPE>
__host__ __device__ constexpr uint32_t compress_lds_bytes(uint32_t d, uint32_t nt) {
    using T = AnyIn<DTYPE>;
    const uint32_t gv = nt * 32, pieces = d * T::ELEM / 16;
    return TQ_GRID_LDS_BYTES + align16(gv * pieces * 4) + gv * 4 + T::XTERMS * gv * (d + ROW_PAD) * 2;
}
// LDS of the decompress kernel: byte -> centroids table | per-vector norms | staged centroids
__host__ __device__ constexpr uint32_t decompress_lds_bytes(uint32_t d, uint32_t nt) {
    return 4096 + nt * 32 * 4 + nt * 32 * (d + ROW_PAD) * 2;
}

// A wave's share of a group's NT column tiles x d/32 row tiles.  With four or more row tiles every wave walks row tiles
// wave, wave + 4, ... over all column tiles (one operand load feeds NT matrix instructions); with fewer, the waves
// left over take a part of the column tiles each, so that all four work.
struct WaveShare {
    uint32_t rb0, rb_step;   // first row tile, stride
    uint32_t ct0, ct_n;      // column tiles [ct0, ct0 + ct_n); ct_n == 0: nothing to do
};
__device__ __forceinline__ WaveShare wave_share(uint32_t wave, uint32_t nwaves, uint32_t tiles, uint32_t nt) {
    WaveShare w;
    const uint32_t rb_waves = tiles < nwaves ? tiles : nwaves;
    uint32_t split = nwaves / rb_waves;          // waves per row tile: 4, 2, 1 (3 row tiles: 1, one wave rests)
    split = split < nt ? split : nt;
    const uint32_t part = wave / rb_waves;
    w.rb0 = wave % rb_waves;
    w.rb_step = rb_waves;
    w.ct_n = part < split ? nt / split : 0u;
    w.ct0 = part * (nt / split);
    return w;
}

template <int BITS>
struct PackAny {
    static constexpr int IPB = 8 / BITS;        // codes per byte
    static constexpr int NB = 16 / IPB;         // packed bytes of a lane's 16 codes: 2, 4, 8, 8, 16
    static constexpr int NW = NB < 4 ? 1 : NB / 4;
};

template <int DTYPE, int BITS>
__global__ __launch_bounds__(MAX_WAVES *TQ_WAVE, 2) void tq_anydim_compress_kernel(TqDevJob job0, const tq_job *jobs, uint32_t d, uint32_t nt) {
    using T = AnyIn<DTYPE>;
    using P = PackAny<BITS>;
    constexpr int ELEM = T::ELEM, NT = T::NT;      // NT: the most column tiles a group may have; nt <= NT: those it has
    constexpr int NB = P::NB, NW = P::NW, IPB = P::IPB;
    const uint32_t GV = nt * 32u;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const TqDevJob job = tq_load_job(job0, jobs, blockIdx.y, ELEM);
    const uint32_t tid = threadIdx.x, nthreads = blockDim.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6, nwaves = nthreads >> 6;
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const uint32_t n_groups = (job.n_vec + GV - 1u) / GV;
    if (blockIdx.x >= n_groups) return;   // also: an empty job of a batch, whose table may be NULL

    const uint32_t pieces = d * ELEM / 16u;          // 16-byte pieces per vector
    const uint32_t row_halves = d + ROW_PAD;
    const uint32_t tiles = d / 32u, steps = d / 16u;
    uint8_t *lds_grid = lds;
    float *part = reinterpret_cast<float *>(lds + TQ_GRID_LDS_BYTES);
    float *sumsq = reinterpret_cast<float *>(lds + TQ_GRID_LDS_BYTES + align16(GV * pieces * 4u));
    uint16_t *xs = reinterpret_cast<uint16_t *>(sumsq + GV);
    const uint32_t term_halves = GV * row_halves;    // one staged term

    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(job.table);
    const uint8_t *a_src = job.table + (DTYPE == TQ_F16 ? hd->off_a_f16 : hd->off_a_bf16);
    const uint32_t a_term = TQ_OPERAND_BYTES_FOR(d);
    tq_copy_to_lds(lds_grid, job.table + hd->off_grid, hd->grid_cells * 8u, tid, nthreads);
    const float grid_scale = hd->grid_scale, grid_bias = hd->grid_bias;
    const uint32_t g_bytes = d / IPB;                // packed bytes per vector

    auto load_a = [&](uint32_t rb, uint32_t s, tq_u4 (&a)[T::ATERMS]) {
        const uint8_t *p = a_src + (((size_t)rb * steps + s) * 64u + lane) * 16u;
#pragma unroll
        for (int t = 0; t < T::ATERMS; ++t) a[t] = tq_gload16(p + (size_t)t * a_term);
    };
    auto mfma = [&](tq_u4 a, tq_u4 b, tq_f16v c) { return DTYPE == TQ_F16 ? mfma_f16(a, b, c) : mfma_bf16(a, b, c); };

    for (uint32_t g = blockIdx.x; g < n_groups; g += gridDim.x) {
        __syncthreads();      // nobody still reads the previous group (first trip: the grid copy is published below)
        // ---- stage the group: 16-byte pieces, coalesced; vectors past the end re-read the last one (never stored)
        // (four fetches of a thread are in flight together)
        auto fetch = [&](uint32_t i) {
            const uint32_t v = i / pieces, p = i - v * pieces;
            uint32_t gv = g * GV + v;
            gv = gv < job.n_vec ? gv : job.n_vec - 1u;
            return tq_gload16(job.states + tq_vec_offset(job, gv) + p * 16u);
        };
        auto place = [&](uint32_t i, const tq_u4 q) {
            const uint32_t v = i / pieces, p = i - v * pieces;
            if constexpr (ELEM == 2) {
                *reinterpret_cast<tq_u4 *>(xs + v * row_halves + p * 8u) = q;
                part[i] = sumsq8<DTYPE>(q, 0.f);
            } else {
                float ss = 0.f;
                uint32_t t0[4], t1[4], t2[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {     // x = t0 + t1 + t2 exactly: every term a truncation, every remainder exact
                    const float x = __uint_as_float(q[k]);
                    ss = fmaf(x, x, ss);
                    const uint32_t xa = q[k] & 0xffff0000u;
                    const float r1 = x - __uint_as_float(xa);
                    const uint32_t xb = __float_as_uint(r1) & 0xffff0000u;
                    const float r2 = r1 - __uint_as_float(xb);
                    t0[k] = xa; t1[k] = xb; t2[k] = __float_as_uint(r2) & 0xffff0000u;
                }
                const tq_u2 w0 = {(t0[0] >> 16) | t0[1], (t0[2] >> 16) | t0[3]};
                const tq_u2 w1 = {(t1[0] >> 16) | t1[1], (t1[2] >> 16) | t1[3]};
                const tq_u2 w2 = {(t2[0] >> 16) | t2[1], (t2[2] >> 16) | t2[3]};
                uint16_t *dst = xs + v * row_halves + p * 4u;
                *reinterpret_cast<tq_u2 *>(dst) = w0;
                *reinterpret_cast<tq_u2 *>(dst + term_halves) = w1;
                *reinterpret_cast<tq_u2 *>(dst + 2u * term_halves) = w2;
                part[i] = ss;
            }
        };
        const uint32_t total = GV * pieces;
        for (uint32_t i0 = tid; i0 < total; i0 += 4u * nthreads) {
            tq_u4 q[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t i = i0 + u * nthreads;
                q[u] = fetch(i < total ? i : i0);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t i = i0 + u * nthreads;
                if (i < total) place(i, q[u]);
            }
        }
        __syncthreads();
        for (uint32_t v = tid; v < GV; v += nthreads) {   // pieces added in index order: the norm does not depend on the launch shape
            float s = 0.f;
            for (uint32_t p = 0; p < pieces; ++p) s += part[v * pieces + p];
            sumsq[v] = s;
        }
        __syncthreads();

        const WaveShare share = wave_share(wave, nwaves, tiles, nt);
        for (uint32_t rb = share.rb0; rb < tiles && share.ct_n; rb += share.rb_step) {
            tq_f16v acc[NT];
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) acc[ct] = tq_zero16();
            tq_u4 a_cur[2][T::ATERMS], a_nxt[2][T::ATERMS];
            load_a(rb, 0u, a_cur[0]);
            load_a(rb, 1u, a_cur[1]);
            for (uint32_t s = 0; s < steps; s += 2u) {      // steps is even; the operands of the next pair are fetched under this one
                const uint32_t sn = s + 2u < steps ? s + 2u : s;
                load_a(rb, sn, a_nxt[0]);
                load_a(rb, sn + 1u, a_nxt[1]);
#pragma unroll
                for (int u = 0; u < 2; ++u) {
#pragma unroll
                    for (int ct = 0; ct < NT; ++ct) {     // acc[ct] belongs to column tile share.ct0 + ct
                        if ((uint32_t)ct >= share.ct_n) break;
                        const uint16_t *row = xs + ((share.ct0 + ct) * 32u + n) * row_halves + 16u * (s + u) + 8u * hk;
#pragma unroll
                        for (int xt = 0; xt < T::XTERMS; ++xt) {
                            const tq_u4 b = *reinterpret_cast<const tq_u4 *>(row + xt * term_halves);
                            // all products whose weight is >= 2^-24 of the leading one (16-bit inputs: both rotation terms)
#pragma unroll
                            for (int at = 0; at + xt < (T::XTERMS == 1 ? T::ATERMS : 3); ++at) acc[ct] = mfma(a_cur[u][at], b, acc[ct]);
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int t = 0; t < T::ATERMS; ++t) a_cur[u][t] = a_nxt[u][t];
            }

            // ---- code search and packing: lane (n, hk) holds coordinates 32 rb + 16 hk + r of vector ct * 32 + n
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) {
                if ((uint32_t)ct >= share.ct_n) break;
                const float nrm = tq_norm_from_sumsq(sumsq[(share.ct0 + ct) * 32u + n]);
                float inv = __builtin_amdgcn_rcpf(nrm + 1e-8f);
                if (DTYPE == TQ_F16) inv *= 1.0f / (float)(1 << TQ_F16_PI_SHIFT);
                const float inv_cell = inv * grid_scale;
                uint32_t words[NW];
#pragma unroll
                for (int w = 0; w < NW; ++w) words[w] = 0u;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float a = acc[ct][r];
                    const uint32_t addr = __float_as_uint(fmaf(a, inv_cell, grid_bias)) & TQ_GRID_ADDR_MASK;
                    const tq_u2 cell = *reinterpret_cast<const tq_u2 *>(lds_grid + addr);
                    const float t = fmaf(a, inv, -__uint_as_float(cell[0]));
                    const uint32_t code = cell[1] + (~__float_as_uint(t) >> 31);      // base + !(rho < threshold)
                    const int byte = r / IPB, k = r % IPB;                            // most significant code of a byte first
                    words[byte / 4] |= code << (8 * (byte % 4) + BITS * (IPB - 1 - k));
                }
                const uint32_t v = g * GV + (share.ct0 + ct) * 32u + n;
                if (v < job.n_vec) {
                    const uint32_t slot = tq_packed_slot(job, v);
                    uint8_t *dst = job.idx_bytes + (size_t)slot * g_bytes + (2u * rb + hk) * NB;
                    if constexpr (NB == 2) {
                        tq_gstore2(reinterpret_cast<uint16_t *>(dst), (uint16_t)words[0]);
                    } else if constexpr (NB == 4) {
                        *reinterpret_cast<TQ_GLOBAL uint32_t *>((TQ_GLOBAL uint8_t *)dst) = words[0];
                    } else if constexpr (NB == 8) {
                        const tq_u2 o = {words[0], words[1]};
                        tq_gstore8(dst, o);
                    } else {
                        const tq_u4 o = {words[0], words[1], words[2], words[3]};
                        tq_gstore16(dst, o);
                    }
                    if (rb == 0u && hk == 0u) {
                        const _Float16 hn = (_Float16)nrm;
                        tq_gstore2(job.vec_norms + slot, __builtin_bit_cast(uint16_t, hn));
                    }
                }
            }
        }
    }
}

template <int DTYPE, int IPB>
__global__ __launch_bounds__(MAX_WAVES *TQ_WAVE, 2) void tq_anydim_decompress_kernel(TqDevJob job0, const tq_job *jobs, uint32_t d, uint32_t nt) {
    constexpr int ELEM = DTYPE == TQ_F32 ? 4 : 2;
    constexpr int NT = DEC_NT;
    const uint32_t GV = nt * 32u;
    constexpr int ENTRY = 2 * IPB;                 // bytes of a table entry: the fp16 centroids of one packed byte

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    const TqDevJob job = tq_load_job(job0, jobs, blockIdx.y, ELEM);
    uint8_t *out_base = const_cast<uint8_t *>(job.states);
    const uint32_t tid = threadIdx.x, nthreads = blockDim.x;
    const uint32_t lane = tid & 63u, wave = tid >> 6, nwaves = nthreads >> 6;
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const uint32_t n_groups = (job.n_vec + GV - 1u) / GV;
    if (blockIdx.x >= n_groups) return;

    const uint32_t row_halves = d + ROW_PAD;
    const uint32_t tiles = d / 32u, steps = d / 16u;
    const uint32_t g_bytes = d / IPB, g_words = g_bytes / 4u;
    uint8_t *lds_lut = lds;
    float *norms = reinterpret_cast<float *>(lds + 4096);
    uint16_t *ys = reinterpret_cast<uint16_t *>(norms + GV);

    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(job.table);
    const uint8_t *a_src = job.table + hd->off_at_f16;      // the leading fp16 term of Pi^T, as in the 128-wide kernel
    tq_copy_to_lds(lds_lut, job.table + hd->off_lut, 256u * ENTRY, tid, nthreads);

    auto load_a = [&](uint32_t rb, uint32_t s) { return tq_gload16(a_src + (((size_t)rb * steps + s) * 64u + lane) * 16u); };

    for (uint32_t g = blockIdx.x; g < n_groups; g += gridDim.x) {
        __syncthreads();
        // ---- stage: every packed byte becomes its IPB centroids (one table entry), in code order
        auto fetch = [&](uint32_t i) {
            const uint32_t v = i / g_words, w = i - v * g_words;
            uint32_t gv = g * GV + v;
            gv = gv < job.n_vec ? gv : job.n_vec - 1u;
            const uint32_t slot = tq_packed_slot(job, gv);
            return *reinterpret_cast<const TQ_GLOBAL uint32_t *>((const TQ_GLOBAL uint8_t *)job.idx_bytes + (size_t)slot * g_bytes + 4u * w);
        };
        auto place = [&](uint32_t i, uint32_t raw) {
            const uint32_t v = i / g_words, w = i - v * g_words;
            uint8_t *dst = reinterpret_cast<uint8_t *>(ys + v * row_halves) + 4u * w * ENTRY;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const uint8_t *e = lds_lut + ((raw >> (8 * b)) & 0xffu) * ENTRY;
                if constexpr (ENTRY == 2) *reinterpret_cast<uint16_t *>(dst + b * ENTRY) = *reinterpret_cast<const uint16_t *>(e);
                else if constexpr (ENTRY == 4) *reinterpret_cast<uint32_t *>(dst + b * ENTRY) = *reinterpret_cast<const uint32_t *>(e);
                else if constexpr (ENTRY == 8) *reinterpret_cast<tq_u2 *>(dst + b * ENTRY) = *reinterpret_cast<const tq_u2 *>(e);
                else *reinterpret_cast<tq_u4 *>(dst + b * ENTRY) = *reinterpret_cast<const tq_u4 *>(e);
            }
        };
        const uint32_t total = GV * g_words;
        for (uint32_t i0 = tid; i0 < total; i0 += 4u * nthreads) {     // four fetches of a thread in flight together
            uint32_t raw[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t i = i0 + u * nthreads;
                raw[u] = fetch(i < total ? i : i0);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t i = i0 + u * nthreads;
                if (i < total) place(i, raw[u]);
            }
        }
        for (uint32_t v = tid; v < GV; v += nthreads) {
            uint32_t gv = g * GV + v;
            gv = gv < job.n_vec ? gv : job.n_vec - 1u;
            norms[v] = (float)__builtin_bit_cast(_Float16, tq_gload2(job.vec_norms + tq_packed_slot(job, gv)));
        }
        __syncthreads();

        const WaveShare share = wave_share(wave, nwaves, tiles, nt);
        for (uint32_t rb = share.rb0; rb < tiles && share.ct_n; rb += share.rb_step) {
            tq_f16v acc[NT];
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) acc[ct] = tq_zero16();
            tq_u4 a_cur[2] = {load_a(rb, 0u), load_a(rb, 1u)};
            for (uint32_t s = 0; s < steps; s += 2u) {
                const uint32_t sn = s + 2u < steps ? s + 2u : s;
                const tq_u4 a_nxt[2] = {load_a(rb, sn), load_a(rb, sn + 1u)};
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int ct = 0; ct < NT; ++ct) {
                        if ((uint32_t)ct >= share.ct_n) break;
                        const tq_u4 b = *reinterpret_cast<const tq_u4 *>(ys + ((share.ct0 + ct) * 32u + n) * row_halves + 16u * (s + u) + 8u * hk);
                        acc[ct] = mfma_f16(a_cur[u], b, acc[ct]);
                    }
                a_cur[0] = a_nxt[0];
                a_cur[1] = a_nxt[1];
            }
            // ---- scale, cast, store: lane (n, hk) holds elements 32 rb + 16 hk + r of vector ct * 32 + n
#pragma unroll
            for (int ct = 0; ct < NT; ++ct) {
                if ((uint32_t)ct >= share.ct_n) break;
                const uint32_t v = g * GV + (share.ct0 + ct) * 32u + n;
                if (v >= job.n_vec) continue;
                const float nrm = norms[(share.ct0 + ct) * 32u + n];
                uint8_t *dst = out_base + tq_vec_offset(job, v) + (32u * rb + 16u * hk) * ELEM;
                if constexpr (ELEM == 2) {
#pragma unroll
                    for (int c = 0; c < 2; ++c) {
                        tq_u4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float x0 = acc[ct][8 * c + 2 * e] * nrm, x1 = acc[ct][8 * c + 2 * e + 1] * nrm;
                            if constexpr (DTYPE == TQ_F16) {
                                const tq_half2 h = {(_Float16)x0, (_Float16)x1};
                                o[e] = __builtin_bit_cast(uint32_t, h);
                            } else {
                                const tq_bf2 h = {(__bf16)x0, (__bf16)x1};
                                o[e] = __builtin_bit_cast(uint32_t, h);
                            }
                        }
                        tq_gstore16(dst + 16 * c, o);
                    }
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        tq_u4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = __float_as_uint(acc[ct][4 * c + e] * nrm);
                        tq_gstore16(dst + 16 * c, o);
                    }
                }
            }
        }
    }
}

// ---- host side --------------------------------------------------------------------------

constexpr int MAX_DEVICES = 64;
std::mutex host_state_mutex;

int device_cus(int &dev, int &cus) {
    static int cache[MAX_DEVICES] = {};
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return TQ_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(host_state_mutex);
    if (cache[dev] == 0) {
        int c = 0;
        e = hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return (int)e;
        cache[dev] = c > 0 ? c : 1;
    }
    cus = cache[dev];
    return 0;
}

// Launches `kernel` over (blocks per job) x n_jobs blocks of MAX_WAVES waves with `lds` bytes of
// dynamic LDS; `raised[dev]` remembers the largest LDS size the kernel has been allowed on each device.
template <typename K, typename L>
int launch(K kernel, uint32_t (&raised)[MAX_DEVICES], L lds_for, uint32_t nt_max, const TqDevJob &job,
           const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t d, hipStream_t stream) {
    // column tiles per group: as many as leave room for two blocks on a compute unit (the phases of a block do not
    // overlap one another; a second block fills the gaps), but at least half of the most
    uint32_t nt = nt_max;
    while (nt > 1u && nt > nt_max / 2u && lds_for(d, nt) > 80u * 1024u) nt /= 2u;
    const uint32_t lds = lds_for(d, nt), group_vectors = nt * 32u;
    int dev = 0, cus = 0;
    const int rc = device_cus(dev, cus);
    if (rc) return rc;
    {
        std::lock_guard<std::mutex> lock(host_state_mutex);
        if (raised[dev] < lds) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            raised[dev] = lds;
        }
    }
    const uint32_t groups = (max_vec + group_vectors - 1u) / group_vectors;
    const uint32_t waves = MAX_WAVES;
    const int resident = lds <= 53u * 1024u ? 3 : lds <= 80u * 1024u ? 2 : 1;     // blocks per compute unit (160 KiB of LDS, 168 registers)
    const uint32_t bx = tq_blocks_per_job(groups, cus * resident, n_jobs);
    hipLaunchKernelGGL(kernel, dim3(bx, (unsigned)n_jobs, 1), dim3(waves * TQ_WAVE, 1, 1), lds, stream, job, jobs_dev, d, nt);
    return (int)hipGetLastError();
}

template <int DTYPE, int BITS>
int launch_compress(const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t d, hipStream_t s) {
    static uint32_t raised[MAX_DEVICES] = {};
    return launch(&tq_anydim_compress_kernel<DTYPE, BITS>, raised, compress_lds_bytes<DTYPE>, AnyIn<DTYPE>::NT, job, jobs_dev,
                  n_jobs, max_vec, d, s);
}
template <int DTYPE>
int compress_bits(int bits, const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t d, hipStream_t s) {
    switch (bits) {
        case 1: return launch_compress<DTYPE, 1>(job, jobs_dev, n_jobs, max_vec, d, s);
        case 2: return launch_compress<DTYPE, 2>(job, jobs_dev, n_jobs, max_vec, d, s);
        case 3: return launch_compress<DTYPE, 3>(job, jobs_dev, n_jobs, max_vec, d, s);
        case 4: return launch_compress<DTYPE, 4>(job, jobs_dev, n_jobs, max_vec, d, s);
        case 5: case 6: case 7: case 8:  // one code per byte: identical packing
            return launch_compress<DTYPE, 8>(job, jobs_dev, n_jobs, max_vec, d, s);
        default: return TQ_ERR_BITS;
    }
}

template <int DTYPE, int IPB>
int launch_decompress(const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t d, hipStream_t s) {
    static uint32_t raised[MAX_DEVICES] = {};
    return launch(&tq_anydim_decompress_kernel<DTYPE, IPB>, raised, decompress_lds_bytes, DEC_NT, job, jobs_dev, n_jobs, max_vec, d, s);
}
template <int DTYPE>
int decompress_bits(int bits, const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t d, hipStream_t s) {
    switch (8 / bits) {
        case 8: return launch_decompress<DTYPE, 8>(job, jobs_dev, n_jobs, max_vec, d, s);
        case 4: return launch_decompress<DTYPE, 4>(job, jobs_dev, n_jobs, max_vec, d, s);
        case 2: return launch_decompress<DTYPE, 2>(job, jobs_dev, n_jobs, max_vec, d, s);
        case 1: return launch_decompress<DTYPE, 1>(job, jobs_dev, n_jobs, max_vec, d, s);
        default: return TQ_ERR_BITS;
    }
}

}  // namespace

bool tq_anydim_supported(int head_dim) {
    return head_dim >= TQ_ANYDIM_MIN && head_dim <= TQ_ANYDIM_MAX && head_dim % 32 == 0;
}

int tq_anydim_compress(int dtype, int bits, int head_dim, const TqDevJob &single, const tq_job *jobs_dev, int n_jobs,
                       uint32_t max_vec, hipStream_t stream) {
    if (!tq_anydim_supported(head_dim)) return TQ_ERR_HEAD_DIM;
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    const uint32_t d = (uint32_t)head_dim;
    switch (dtype) {
        case TQ_F32: return compress_bits<TQ_F32>(bits, single, jobs_dev, n_jobs, max_vec, d, stream);
        case TQ_F16: return compress_bits<TQ_F16>(bits, single, jobs_dev, n_jobs, max_vec, d, stream);
        case TQ_BF16: return compress_bits<TQ_BF16>(bits, single, jobs_dev, n_jobs, max_vec, d, stream);
        default: return TQ_ERR_DTYPE;
    }
}

int tq_anydim_decompress(int dtype, int bits, int head_dim, const TqDevJob &single, const tq_job *jobs_dev, int n_jobs,
                         uint32_t max_vec, hipStream_t stream) {
    if (!tq_anydim_supported(head_dim)) return TQ_ERR_HEAD_DIM;
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    const uint32_t d = (uint32_t)head_dim;
    switch (dtype) {
        case TQ_F32: return decompress_bits<TQ_F32>(bits, single, jobs_dev, n_jobs, max_vec, d, stream);
        case TQ_F16: return decompress_bits<TQ_F16>(bits, single, jobs_dev, n_jobs, max_vec, d, stream);
        case TQ_BF16: return decompress_bits<TQ_BF16>(bits, single, jobs_dev, n_jobs, max_vec, d, stream);
        default: return TQ_ERR_DTYPE;
    }
}
