// compress and decompress for head dimensions other than 128: 8 to 256, taken at run time (upstream
// turboquant/compressors_v3.py:37-43 builds its rotation and codebook for whatever head_dim it is given; :46-81
// compress, :84-105 decompress).  A dimension that is not a multiple of 32 is worked on as the next multiple (the
// RAGGED instantiations): the operand sets in the table are those of the rotation extended by zeros, the elements a
// vector does not have are staged as zeros, the coordinates it does not have get the code 0 (:64-68 pads the codes of
// a vector with zeros to a whole byte) and are neither decoded nor stored on the way back; input, packed codes and
// output are then moved element by element and byte by byte, since nothing about their alignment is known.  Same arithmetic as the 128-wide kernels (split rotation on the
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
#include "tq_wide.h"

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

// d: the dimension of the operand sets (a multiple of 32); dl: the head dimension itself (RAGGED: dl < d)
template <int DTYPE, int BITS, bool RAGGED>
__global__ __launch_bounds__(MAX_WAVES *TQ_WAVE, 2) void tq_anydim_compress_kernel(TqDevJob job0, const tq_job *jobs, uint32_t d, uint32_t dl, uint32_t nt) {
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
    const uint32_t g_bytes = (dl + IPB - 1u) / IPB;  // packed bytes per vector

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
            if constexpr (RAGGED) {      // what lies past the vector's end is zero
                constexpr uint32_t EPP = 16 / ELEM;
                const TQ_GLOBAL uint8_t *src = (const TQ_GLOBAL uint8_t *)job.states + tq_vec_offset(job, gv);
                if (p * EPP + EPP <= dl && (((uintptr_t)src + p * 16u) & 15u) == 0u)      // a whole piece at an aligned address
                    return *reinterpret_cast<const TQ_GLOBAL tq_u4 *>(src + p * 16u);
                if (p * EPP >= dl) return tq_u4{0u, 0u, 0u, 0u};
                tq_u4 q = {0u, 0u, 0u, 0u};      // element by element
#pragma unroll
                for (uint32_t k = 0; k < EPP; ++k) {
                    const uint32_t e = p * EPP + k;
                    if (e < dl) {
                        if constexpr (ELEM == 2) q[k / 2] |= (uint32_t)*reinterpret_cast<const TQ_GLOBAL uint16_t *>(src + 2u * e) << (16 * (k & 1));
                        else q[k] = *reinterpret_cast<const TQ_GLOBAL uint32_t *>(src + 4u * e);
                    }
                }
                return q;
            } else {
                return tq_gload16(job.states + tq_vec_offset(job, gv) + p * 16u);
            }
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
                    uint32_t code = cell[1] + (~__float_as_uint(t) >> 31);            // base + !(rho < threshold)
                    if constexpr (RAGGED) code = 32u * rb + 16u * hk + (uint32_t)r < dl ? code : 0u;
                    const int byte = r / IPB, k = r % IPB;                            // most significant code of a byte first
                    words[byte / 4] |= code << (8 * (byte % 4) + BITS * (IPB - 1 - k));
                }
                const uint32_t v = g * GV + (share.ct0 + ct) * 32u + n;
                if (v < job.n_vec) {
                    const uint32_t slot = tq_packed_slot(job, v);
                    uint8_t *dst = job.idx_bytes + (size_t)slot * g_bytes + (2u * rb + hk) * NB;
                    bool bytewise = false;
                    if constexpr (RAGGED) bytewise = (2u * rb + hk) * NB + NB > g_bytes || ((uintptr_t)dst & (uintptr_t)(NB - 1));
                    if (bytewise) {
#pragma unroll
                        for (int b = 0; b < NB; ++b)
                            if ((2u * rb + hk) * NB + (uint32_t)b < g_bytes)
                                *((TQ_GLOBAL uint8_t *)dst + b) = (uint8_t)(words[b / 4] >> (8 * (b % 4)));
                    } else if constexpr (NB == 2) {
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

template <int DTYPE, int IPB, bool RAGGED>
__global__ __launch_bounds__(MAX_WAVES *TQ_WAVE, 2) void tq_anydim_decompress_kernel(TqDevJob job0, const tq_job *jobs, uint32_t d, uint32_t dl, uint32_t nt) {
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
    const uint32_t g_words = d / IPB / 4u;               // staged words per vector (of the padded dimension)
    const uint32_t g_bytes = (dl + IPB - 1u) / IPB;      // packed bytes per vector in memory
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
            if constexpr (RAGGED) {      // byte by byte; past the vector's last byte: zero (never decoded)
                const TQ_GLOBAL uint8_t *src = (const TQ_GLOBAL uint8_t *)job.idx_bytes + (size_t)slot * g_bytes;
                if (4u * w + 4u <= g_bytes && (((uintptr_t)src + 4u * w) & 3u) == 0u)      // a whole word at an aligned address
                    return *reinterpret_cast<const TQ_GLOBAL uint32_t *>(src + 4u * w);
                uint32_t raw = 0u;
#pragma unroll
                for (uint32_t b = 0; b < 4u; ++b)
                    if (4u * w + b < g_bytes) raw |= (uint32_t)src[4u * w + b] << (8u * b);
                return raw;
            } else {
                return *reinterpret_cast<const TQ_GLOBAL uint32_t *>((const TQ_GLOBAL uint8_t *)job.idx_bytes + (size_t)slot * g_bytes + 4u * w);
            }
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
                if constexpr (RAGGED) {      // coordinates the vector does not have contribute nothing
                    const uint32_t c0 = (4u * w + (uint32_t)b) * IPB;
                    uint16_t *y = reinterpret_cast<uint16_t *>(dst + b * ENTRY);
#pragma unroll
                    for (uint32_t k = 0; k < (uint32_t)IPB; ++k)
                        if (c0 + k >= dl) y[k] = 0;
                }
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
                bool elementwise = false;
                if constexpr (RAGGED) elementwise = 32u * rb + 16u * hk + 16u > dl || ((uintptr_t)dst & 15u);
                if (elementwise) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        if (32u * rb + 16u * hk + (uint32_t)r >= dl) break;
                        const float x = acc[ct][r] * nrm;
                        if constexpr (DTYPE == TQ_F32) {
                            *reinterpret_cast<TQ_GLOBAL uint32_t *>((TQ_GLOBAL uint8_t *)dst + 4 * r) = __float_as_uint(x);
                        } else if constexpr (DTYPE == TQ_F16) {
                            const _Float16 h = (_Float16)x;
                            *reinterpret_cast<TQ_GLOBAL uint16_t *>((TQ_GLOBAL uint8_t *)dst + 2 * r) = __builtin_bit_cast(uint16_t, h);
                        } else {
                            const __bf16 h = (__bf16)x;
                            *reinterpret_cast<TQ_GLOBAL uint16_t *>((TQ_GLOBAL uint8_t *)dst + 2 * r) = __builtin_bit_cast(uint16_t, h);
                        }
                    }
                } else if constexpr (ELEM == 2) {
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

// ====================================================================================================================
// Head dimension 256 with 16-bit elements: the rotation resident in registers, as in the 128-wide kernels.
//
// compress: a block is eight waves that share tiles of 32 vectors (16 KiB); wave w keeps the 32 rows [32w, 32w+32) of
// Pi as MFMA A operands for all 16 steps of the contraction, two 16-bit terms (128 registers).  A tile is fetched with
// coalesced 16-byte loads one tile ahead, parked in a double-buffered XOR-swizzled LDS tile (one barrier per tile) and
// read back by every wave as the B operand of 32 matrix instructions.  The sum of squares of a vector is reduced over the
// 32 lanes that hold its 32 pieces while they park them (a butterfly: the same order for every vector, whatever the
// launch shape).  The code search of tile j-1 is written between the matrix instructions of tile j (one coordinate per
// step, from the other accumulator set), so that the vector work runs in their shadow.  65 536 x 4 flop per vector
// against 640 bytes puts this width on the matrix side of the roofline: the kernel is bound by the matrix rate the part
// sustains, not by memory.
template <int DTYPE, int BITS>
__global__ __launch_bounds__(512, 1) void tq_d256_compress_kernel(TqDevJob job0, const tq_job *jobs) {
    static_assert(DTYPE == TQ_F16 || DTYPE == TQ_BF16, "16-bit inputs");
    constexpr int D = 256, STEPS = D / 16, PIECES = D * 2 / 16;     // 32 pieces of 16 bytes per vector
    constexpr int IPB = 8 / BITS, NB = 16 / IPB, NW = NB < 4 ? 1 : NB / 4;
    constexpr int TILE_BYTES = 32 * D * 2;

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t *lds_grid = lds;                                                        // single copy, bases unshifted
    uint8_t (*lds_stage)[TILE_BYTES] = reinterpret_cast<uint8_t (*)[TILE_BYTES]>(lds + TQ_GRID_LDS_BYTES);
    float (*lds_ss)[32] = reinterpret_cast<float (*)[32]>(lds + TQ_GRID_LDS_BYTES + 2 * TILE_BYTES);     // [3][32]

    const TqDevJob job = tq_uniform_job(tq_load_job(job0, jobs, blockIdx.y, 2));
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = tq_uniform32(tid >> 6);
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const uint32_t n_tiles = (job.n_vec + 31u) / 32u;
    if (blockIdx.x >= n_tiles) return;        // also: an empty job of a batch, whose table may be NULL
    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(job.table);

    // loads of a tile: piece i = l * 512 + tid of the tile's 1024 is piece i % 32 of vector i / 32, so that the 32 pieces
    // of a vector sit in 32 consecutive lanes; vectors past the end re-read the job's last one (never stored)
    const uint32_t ld_vec = tid >> 5, ld_piece = tid & 31u;
    tq_u4 pre[2];
    auto issue_loads = [&](uint32_t tl) {
#pragma unroll
        for (int l = 0; l < 2; ++l) {
            uint32_t v = tl * 32u + l * 16u + ld_vec;
            v = v < job.n_vec ? v : job.n_vec - 1u;
            pre[l] = tq_gload16(job.states + tq_vec_offset(job, v) + ld_piece * 16u);
        }
    };
    issue_loads(blockIdx.x);

    tq_u4 areg[2][STEPS];
    {
        const uint8_t *src = job.table + (DTYPE == TQ_F16 ? hd->off_a_f16 : hd->off_a_bf16);
#pragma unroll
        for (int term = 0; term < 2; ++term)
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
                areg[term][s] = tq_gload16(src + (size_t)term * TQ_OPERAND_BYTES_FOR(D) + (((size_t)wave * STEPS + s) * 64 + lane) * 16);
    }
    tq_copy_to_lds(lds_grid, job.table + hd->off_grid, hd->grid_cells * 8u, tid, 512u);
    const float grid_scale = hd->grid_scale, grid_bias = hd->grid_bias;

    // park the prefetched tile in buffer b and leave the vectors' sums of squares in slot `slot`
    auto park = [&](uint32_t b, uint32_t slot) {
#pragma unroll
        for (int l = 0; l < 2; ++l) {
            const uint32_t v = l * 16u + ld_vec;
            *reinterpret_cast<tq_u4 *>(lds_stage[b] + v * (D * 2) + ((ld_piece ^ (v & 31u)) << 4)) = pre[l];
            float s = sumsq8<DTYPE>(pre[l], 0.f);
#pragma unroll
            for (int m = 1; m < 32; m <<= 1) s += __shfl_xor(s, m);
            if (ld_piece == 0u) lds_ss[slot][v] = s;
        }
    };
    // B operand of step s: piece (2 s + hk) ^ (n & 31) of row n = the piece of step 0 with 32 s toggled in its byte offset
    const uint32_t op_base = n * (D * 2) + ((hk ^ (n & 31u)) << 4);
    const uint32_t g_bytes = D / IPB;

    // iteration j: rotate tile j into acc_new, search tile j-1 from acc_old
    auto iteration = [&](auto rot_tag, auto search_tag, uint32_t j, tq_f16v &acc_new, const tq_f16v &acc_old) {
        constexpr bool ROT = decltype(rot_tag)::value, SEARCH = decltype(search_tag)::value;
        const uint8_t *stage = lds_stage[j & 1u];
        float nrm = 0.f, inv = 0.f, inv_cell = 0.f;
        if constexpr (SEARCH) {
            nrm = tq_norm_from_sumsq(lds_ss[(j + 2u) % 3u][n]);       // tile j-1 sits in slot (j-1) % 3
            inv = __builtin_amdgcn_rcpf(nrm + 1e-8f);
            if (DTYPE == TQ_F16) inv *= 1.0f / (float)(1 << TQ_F16_PI_SHIFT);
            inv_cell = inv * grid_scale;
        }
        if constexpr (ROT) acc_new = tq_zero16();
        uint32_t words[NW];
#pragma unroll
        for (int w = 0; w < NW; ++w) words[w] = 0u;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            if constexpr (ROT) {
                const tq_u4 bop = *reinterpret_cast<const tq_u4 *>(stage + (op_base ^ (32u * s)));
                acc_new = (DTYPE == TQ_F16) ? mfma_f16(areg[0][s], bop, acc_new) : mfma_bf16(areg[0][s], bop, acc_new);
                acc_new = (DTYPE == TQ_F16) ? mfma_f16(areg[1][s], bop, acc_new) : mfma_bf16(areg[1][s], bop, acc_new);
            }
            if constexpr (SEARCH) {     // coordinate 32 w + 16 hk + s of vector n
                const float a = acc_old[s];
                const uint32_t addr = __float_as_uint(fmaf(a, inv_cell, grid_bias)) & TQ_GRID_ADDR_MASK;
                const tq_u2 cell = *reinterpret_cast<const tq_u2 *>(lds_grid + addr);
                const float t = fmaf(a, inv, -__uint_as_float(cell[0]));
                const uint32_t code = cell[1] + (~__float_as_uint(t) >> 31);          // base + !(rho < threshold)
                const int byte = s / IPB, k = s % IPB;                                // most significant code of a byte first
                words[byte / 4] |= code << (8 * (byte % 4) + BITS * (IPB - 1 - k));
            }
            // keep the steps in this order: with all 16 operand reads and table lookups hoisted to the top the kernel
            // runs out of registers (the rotation alone holds 128)
            if (s % 2 == 1) __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (SEARCH) {
            const uint32_t v = (blockIdx.x + (j - 1u) * gridDim.x) * 32u + n;
            if (v < job.n_vec) {
                const uint32_t slot = tq_packed_slot(job, v);
                uint8_t *dst = job.idx_bytes + (size_t)slot * g_bytes + (2u * wave + hk) * NB;
                if constexpr (NB == 2) tq_gstore2(reinterpret_cast<uint16_t *>(dst), (uint16_t)words[0]);
                else if constexpr (NB == 4) *reinterpret_cast<TQ_GLOBAL uint32_t *>((TQ_GLOBAL uint8_t *)dst) = words[0];
                else if constexpr (NB == 8) { const tq_u2 o = {words[0], words[1]}; tq_gstore8(dst, o); }
                else { const tq_u4 o = {words[0], words[1], words[2], words[3]}; tq_gstore16(dst, o); }
                if (wave == 0u && hk == 0u) {
                    const _Float16 hn = (_Float16)nrm;
                    tq_gstore2(job.vec_norms + slot, __builtin_bit_cast(uint16_t, hn));
                }
            }
        }
    };

    const uint32_t m = (n_tiles - blockIdx.x + gridDim.x - 1u) / gridDim.x;     // this block's tiles
    // one trip: the tile after this one sets out while this one is rotated, and is parked behind the trip's work
    auto trip = [&](auto rot_tag, auto search_tag, uint32_t j, tq_f16v &acc_new, const tq_f16v &acc_old) {
        const bool more = j + 1u < m;
        if (more) issue_loads(blockIdx.x + (j + 1u) * gridDim.x);
        __syncthreads();        // tile j and its sums are parked, and nobody reads buffer (j + 1) & 1 any more
        iteration(rot_tag, search_tag, j, acc_new, acc_old);
        if (more) park((j + 1u) & 1u, (j + 1u) % 3u);
    };
    using T = std::true_type;
    using F = std::false_type;
    park(0u, 0u);
    tq_f16v acc_a, acc_b;       // tiles with an even index rotate into acc_a, the others into acc_b
    trip(T{}, F{}, 0u, acc_a, acc_a);
    uint32_t j = 1;
    for (; j + 1u < m; j += 2u) {
        trip(T{}, T{}, j, acc_b, acc_a);
        trip(T{}, T{}, j + 1u, acc_a, acc_b);
    }
    if (j < m) {
        trip(T{}, T{}, j, acc_b, acc_a);
        ++j;
    }
    if (m & 1u) trip(F{}, T{}, m, acc_b, acc_a);        // the last tile's codes
    else trip(F{}, T{}, m, acc_a, acc_b);
}

// decompress: a block is four waves that share tiles of 32 vectors; wave w keeps the rows [64w, 64w+64) of Pi^T as A
// operands for all 16 steps (the leading fp16 term: 128 registers).  The packed bytes of a tile are fetched one tile
// ahead (every thread the bytes of 32 codes), turned into fp16 centroids through the byte -> centroids table and parked
// in a double-buffered swizzled LDS tile that all four waves read as B operands; the scaled, rounded results go through
// a second LDS tile so that the stores are 512 contiguous bytes per vector.
template <int DTYPE, int IPB>
__global__ __launch_bounds__(256, 2) void tq_d256_decompress_kernel(TqDevJob job0, const tq_job *jobs) {
    static_assert(DTYPE == TQ_F16 || DTYPE == TQ_BF16, "16-bit outputs");
    constexpr int D = 256, STEPS = D / 16;
    constexpr int TILE_BYTES = 32 * D * 2;
    constexpr int ENTRY = 2 * IPB;                 // bytes of a table entry: the fp16 centroids of one packed byte
    constexpr int RAW = 32 / IPB;                  // packed bytes of a thread's 32 codes: 4, 8, 16, 32
    constexpr int RW = RAW / 4;                    // as dwords

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t *lds_lut = lds;
    uint8_t (*lds_y)[TILE_BYTES] = reinterpret_cast<uint8_t (*)[TILE_BYTES]>(lds + 4096);
    uint8_t *lds_out = lds + 4096 + 2 * TILE_BYTES;
    float (*lds_norm)[32] = reinterpret_cast<float (*)[32]>(lds + 4096 + 3 * TILE_BYTES);       // [2][32]

    const TqDevJob job = tq_uniform_job(tq_load_job(job0, jobs, blockIdx.y, 2));
    uint8_t *out_base = const_cast<uint8_t *>(job.states);
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = tq_uniform32(tid >> 6);
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const uint32_t n_tiles = (job.n_vec + 31u) / 32u;
    if (blockIdx.x >= n_tiles) return;
    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(job.table);
    const uint32_t g_bytes = D / IPB;

    // a thread's share of a tile: codes [32 c, 32 c + 32) of vector dv, c = tid % 8
    const uint32_t dv = tid >> 3, chunk = tid & 7u;
    uint32_t raw[RW];
    uint16_t norm_bits = 0;
    auto issue_loads = [&](uint32_t tl) {
        uint32_t v = tl * 32u + dv;
        v = v < job.n_vec ? v : job.n_vec - 1u;
        const uint32_t slot = tq_packed_slot(job, v);
        const uint8_t *src = job.idx_bytes + (size_t)slot * g_bytes + chunk * RAW;
        if constexpr (RW == 1) raw[0] = *reinterpret_cast<const TQ_GLOBAL uint32_t *>((const TQ_GLOBAL uint8_t *)src);
        else if constexpr (RW == 2) { const tq_u2 t = tq_gload8(src); raw[0] = t[0]; raw[1] = t[1]; }
        else {
#pragma unroll
            for (int q = 0; q < RW / 4; ++q) {
                const tq_u4 t = tq_gload16(src + 16 * q);
#pragma unroll
                for (int i = 0; i < 4; ++i) raw[4 * q + i] = t[i];
            }
        }
        if (chunk == 0u) norm_bits = tq_gload2(job.vec_norms + slot);
    };
    issue_loads(blockIdx.x);

    tq_u4 areg[2][STEPS];       // row tiles 2w, 2w + 1
    {
        const uint8_t *src = job.table + hd->off_at_f16;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
                areg[t][s] = tq_gload16(src + (((size_t)(2u * wave + t) * STEPS + s) * 64 + lane) * 16);
    }
    tq_copy_to_lds(lds_lut, job.table + hd->off_lut, 256u * ENTRY, tid, 256u);
    __syncthreads();

    // the prefetched bytes -> 32 fp16 centroids = pieces 4 chunk .. 4 chunk + 3 of row dv of buffer b
    auto decode = [&](uint32_t b) {
        uint32_t h[16];         // 32 halves
#pragma unroll
        for (int byte = 0; byte < RAW; ++byte) {
            const uint32_t v = (raw[byte / 4] >> (8 * (byte % 4))) & 0xffu;
            const uint8_t *e = lds_lut + v * ENTRY;
            if constexpr (IPB == 1) {
                const uint32_t c = *reinterpret_cast<const uint16_t *>(e);
                if (byte & 1) h[byte / 2] |= c << 16; else h[byte / 2] = c;
            } else if constexpr (IPB == 2) {
                h[byte] = *reinterpret_cast<const uint32_t *>(e);
            } else if constexpr (IPB == 4) {
                const tq_u2 c = *reinterpret_cast<const tq_u2 *>(e);
                h[2 * byte] = c[0]; h[2 * byte + 1] = c[1];
            } else {
                const tq_u4 c = *reinterpret_cast<const tq_u4 *>(e);
                h[4 * byte] = c[0]; h[4 * byte + 1] = c[1]; h[4 * byte + 2] = c[2]; h[4 * byte + 3] = c[3];
            }
        }
        // piece p = 4 chunk + q of a row sits at position ((q << 3) | chunk) ^ (row & 31): the eight threads that decode one
        // row write eight different bank groups at a time (with the pieces in place they would hit two), and the eight
        // rows an operand read touches still differ in the low three bits
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const tq_u4 o = {h[4 * q], h[4 * q + 1], h[4 * q + 2], h[4 * q + 3]};
            *reinterpret_cast<tq_u4 *>(lds_y[b] + dv * (D * 2) + (((((uint32_t)q << 3) | chunk) ^ (dv & 31u)) << 4)) = o;
        }
        if (chunk == 0u) lds_norm[b][dv] = (float)__builtin_bit_cast(_Float16, norm_bits);
    };
    // B operand of step s: piece 2 s + hk = 4 (s >> 1) + (2 (s & 1) + hk), i.e. position ((2 (s & 1) + hk) << 3 | s >> 1) ^ (n & 31)
    const uint32_t op_base = n * (D * 2) + (((hk << 3) ^ (n & 31u)) << 4);
    auto op_step = [](int s) { return (uint32_t)((((2 * (s & 1)) << 3) | (s >> 1)) << 4); };

    const uint32_t m = (n_tiles - blockIdx.x + gridDim.x - 1u) / gridDim.x;
    decode(0u);
    for (uint32_t j = 0; j < m; ++j) {
        const uint32_t tl = blockIdx.x + j * gridDim.x;
        if (j + 1u < m) issue_loads(tl + gridDim.x);
        __syncthreads();        // tile j is decoded; the output tile of the last iteration has been read
        const uint8_t *ys = lds_y[j & 1u];
        tq_f16v acc[2] = {tq_zero16(), tq_zero16()};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const tq_u4 b = *reinterpret_cast<const tq_u4 *>(ys + (op_base ^ op_step(s)));
            acc[0] = mfma_f16(areg[0][s], b, acc[0]);
            acc[1] = mfma_f16(areg[1][s], b, acc[1]);
        }
        // lane (n, hk) holds elements 32 t + 16 hk + r of vector n for its row tiles t = 2w, 2w + 1: pieces 4 t + 2 hk + c
        const float nrm = lds_norm[j & 1u][n];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                tq_u4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float x0 = acc[t][8 * c + 2 * e] * nrm, x1 = acc[t][8 * c + 2 * e + 1] * nrm;
                    if constexpr (DTYPE == TQ_F16) {
                        const tq_half2 hh = {(_Float16)x0, (_Float16)x1};
                        o[e] = __builtin_bit_cast(uint32_t, hh);
                    } else {
                        const tq_bf2 hh = {(__bf16)x0, (__bf16)x1};
                        o[e] = __builtin_bit_cast(uint32_t, hh);
                    }
                }
                const uint32_t piece = 4u * (2u * wave + t) + 2u * hk + c;
                *reinterpret_cast<tq_u4 *>(lds_out + n * (D * 2) + ((piece ^ (n & 31u)) << 4)) = o;
            }
        __syncthreads();        // the output tile is complete
#pragma unroll
        for (int k = 0; k < 4; ++k) {       // 1024 pieces, 256 threads: piece i % 32 of vector i / 32, 512 contiguous bytes per vector
            const uint32_t i = k * 256u + tid, vl = i >> 5, p = i & 31u;
            const tq_u4 val = *reinterpret_cast<const tq_u4 *>(lds_out + vl * (D * 2) + ((p ^ (vl & 31u)) << 4));
            const uint32_t v = tl * 32u + vl;
            if (v < job.n_vec) tq_gstore16_stream(out_base + tq_vec_offset(job, v) + p * 16u, val);
        }
        if (j + 1u < m) decode((j + 1u) & 1u);
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
           const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t d, uint32_t dl, hipStream_t stream) {
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
    hipLaunchKernelGGL(kernel, dim3(bx, (unsigned)n_jobs, 1), dim3(waves * TQ_WAVE, 1, 1), lds, stream, job, jobs_dev, d, dl, nt);
    return (int)hipGetLastError();
}

// Launch of one of the 256-wide kernels: `threads` per block, `resident` blocks per compute unit, `lds` bytes of dynamic LDS.
template <typename K>
int launch_d256(K kernel, bool (&raised)[MAX_DEVICES], uint32_t lds, uint32_t threads, int resident, const TqDevJob &job,
                const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, hipStream_t stream) {
    int dev = 0, cus = 0;
    const int rc = device_cus(dev, cus);
    if (rc) return rc;
    {
        std::lock_guard<std::mutex> lock(host_state_mutex);
        if (!raised[dev]) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            raised[dev] = true;
        }
    }
    const uint32_t tiles = (max_vec + 31u) / 32u;
    const uint32_t bx = tq_blocks_per_job(tiles, cus * resident, n_jobs);
    hipLaunchKernelGGL(kernel, dim3(bx, (unsigned)n_jobs, 1), dim3(threads, 1, 1), lds, stream, job, jobs_dev);
    return (int)hipGetLastError();
}

template <int DTYPE, int BITS>
int launch_compress(const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t d, hipStream_t s) {
    if constexpr (DTYPE != TQ_F32) {
        if (d == 256u) {
            static bool raised256[MAX_DEVICES] = {};
            constexpr uint32_t lds = TQ_GRID_LDS_BYTES + 2u * 32u * 256u * 2u + 3u * 32u * 4u;
            return launch_d256(&tq_d256_compress_kernel<DTYPE, BITS>, raised256, lds, 512u, 1, job, jobs_dev, n_jobs, max_vec, s);
        }
    }
    const uint32_t dp = TQ_PADDED_DIM(d);
    if (dp != d) {
        static uint32_t raised_ragged[MAX_DEVICES] = {};
        return launch(&tq_anydim_compress_kernel<DTYPE, BITS, true>, raised_ragged, compress_lds_bytes<DTYPE>, AnyIn<DTYPE>::NT, job,
                      jobs_dev, n_jobs, max_vec, dp, d, s);
    }
    static uint32_t raised[MAX_DEVICES] = {};
    return launch(&tq_anydim_compress_kernel<DTYPE, BITS, false>, raised, compress_lds_bytes<DTYPE>, AnyIn<DTYPE>::NT, job, jobs_dev,
                  n_jobs, max_vec, d, d, s);
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
    if constexpr (DTYPE != TQ_F32) {
        if (d == 256u) {
            static bool raised256[MAX_DEVICES] = {};
            constexpr uint32_t lds = 4096u + 3u * 32u * 256u * 2u + 2u * 32u * 4u;
            return launch_d256(&tq_d256_decompress_kernel<DTYPE, IPB>, raised256, lds, 256u, 2, job, jobs_dev, n_jobs, max_vec, s);
        }
    }
    const uint32_t dp = TQ_PADDED_DIM(d);
    if (dp != d) {
        static uint32_t raised_ragged[MAX_DEVICES] = {};
        return launch(&tq_anydim_decompress_kernel<DTYPE, IPB, true>, raised_ragged, decompress_lds_bytes, DEC_NT, job, jobs_dev, n_jobs,
                      max_vec, dp, d, s);
    }
    static uint32_t raised[MAX_DEVICES] = {};
    return launch(&tq_anydim_decompress_kernel<DTYPE, IPB, false>, raised, decompress_lds_bytes, DEC_NT, job, jobs_dev, n_jobs, max_vec, d, d, s);
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
    return head_dim >= TQ_ANYDIM_MIN && head_dim <= TQ_ANYDIM_MAX;
}

int tq_anydim_compress(int dtype, int bits, int head_dim, const TqDevJob &single, const tq_job *jobs_dev, int n_jobs,
                       uint32_t max_vec, hipStream_t stream) {
    if (!tq_anydim_supported(head_dim)) return TQ_ERR_HEAD_DIM;
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    if (tq_wide_supported(head_dim, dtype)) return tq_wide_compress(dtype, bits, head_dim, single, jobs_dev, n_jobs, max_vec, stream);
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
    if (tq_wide_supported(head_dim, dtype)) return tq_wide_decompress(dtype, bits, head_dim, single, jobs_dev, n_jobs, max_vec, stream);
    const uint32_t d = (uint32_t)head_dim;
    switch (dtype) {
        case TQ_F32: return decompress_bits<TQ_F32>(bits, single, jobs_dev, n_jobs, max_vec, d, stream);
        case TQ_F16: return decompress_bits<TQ_F16>(bits, single, jobs_dev, n_jobs, max_vec, d, stream);
        case TQ_BF16: return decompress_bits<TQ_BF16>(bits, single, jobs_dev, n_jobs, max_vec, d, stream);
        default: return TQ_ERR_DTYPE;
    }
}
