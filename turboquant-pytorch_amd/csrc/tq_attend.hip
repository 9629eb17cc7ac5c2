// Decode-time attention straight from the packed cache: scores against packed keys and the
// probability-weighted sum of packed values, without materialising de-quantised K / V.
//
// With k_hat = norm * (centroids[codes] @ Pi)  (upstream turboquant/compressors_v3.py:84-105)
//     q . k_hat      = norm * sum_j (Pi q)_j * centroids[code_j]
//     sum_t p_t v_hat_t = ( sum_t p_t * norm_t * centroids[codes_t] ) @ Pi
// so the query is rotated once (by the caller), every cached token costs its packed bytes only,
// and the value side is rotated back once per query head.  These kernels replace the pair
// "de-quantise the whole history (generation_test_v2.py:131-135), then let the model multiply by
// it" (score definition: validate_v3.py:87) for single-token decode steps.
#include "tq_device.h"

namespace {

constexpr int SC_WAVES = 4;
constexpr int WV_WAVES = 4;
constexpr int WV_MAX_GROUP = 8;

struct ScoreArgs {
    const uint8_t *idx_bytes;
    const uint16_t *vec_norms;
    const uint8_t *table;
    const float *q_rot;      // [rows, group, 128]
    float *scores;           // q head (row * group + g), token t at (row * group + g) * stride + t
    long long stride;
    uint32_t tokens, packed_row_stride, group;
};

// One wave per tile of 32 tokens of row blockIdx.y.  MFMA rows = query heads of the row's group
// (zero above `group`), MFMA columns = tokens; the B operand is the decompress kernel's.
// The queries are split into fp16 hi + lo of q * 2^(10 - e_row) (e_row: binary exponent of the
// row's largest magnitude), so the products carry ~22 bits whatever the scale of a head.
template <int IPB>
__global__ __launch_bounds__(SC_WAVES *TQ_WAVE) void tq_scores_kernel(ScoreArgs a) {
    constexpr int NB = 64 / IPB;   // packed bytes per lane (half a vector)
    constexpr int NW = NB / 4;
    __shared__ __attribute__((aligned(16))) uint8_t lds_lut[4096];
    __shared__ float lds_rowscale[32];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t row = blockIdx.y;
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(a.table);
    tq_copy_to_lds(lds_lut, a.table + hd->off_lut, 256u * 2u * IPB, tid, SC_WAVES * TQ_WAVE);

    // ---- A operand: query head m = n of this row, contraction slice (step s, half hk) = codes 64*hk + 8*s + i
    tq_u4 ahi[TQ_STEPS], alo[TQ_STEPS];
    {
        const bool live = n < a.group;
        const TQ_GLOBAL float *q = (const TQ_GLOBAL float *)a.q_rot + ((size_t)row * a.group + (live ? n : 0u)) * TQ_HEAD_DIM + 64u * hk;
        float big = 0.f;
        for (int i = 0; i < 64; ++i) big = fmaxf(big, fabsf(q[i]));
        big = fmaxf(big, __shfl_xor(big, 32));
        int e = 0;
        if (big > 0.f && big < __builtin_inff()) (void)frexpf(big, &e);
        e = e < -100 ? -100 : e;   // rows that small give zero scores either way; keeps 2^(10-e) finite
        const float up = ldexpf(1.f, TQ_F16_PI_SHIFT - e);
        if (hk == 0u) lds_rowscale[n] = live ? ldexpf(1.f, e - TQ_F16_PI_SHIFT) : 0.f;
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            tq_half8 h, l;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float x = live ? q[8 * s + i] * up : 0.f;
                const _Float16 xh = (_Float16)x;
                h[i] = xh;
                l[i] = (_Float16)(x - (float)xh);
            }
            ahi[s] = __builtin_bit_cast(tq_u4, h);
            alo[s] = __builtin_bit_cast(tq_u4, l);
        }
    }
    __syncthreads();
    // accumulator register r of lane (n, h = hk) belongs to query head 8*(r/4) + 4*h + r%4
    float rowscale[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) rowscale[r] = lds_rowscale[8 * (r / 4) + 4 * hk + (r % 4)];

    const uint32_t n_tiles = (a.tokens + 31u) / 32u;
    const uint32_t tile_stride = gridDim.x * SC_WAVES;
    uint32_t tile = blockIdx.x * SC_WAVES + wave;
    const size_t slot0 = (size_t)row * a.packed_row_stride;

    uint32_t raw[NW];
    uint16_t norm_bits = 0;
    auto issue_loads = [&](uint32_t tl) {
        const uint32_t t = tl * 32u + n;
        const bool ok = t < a.tokens;
        const size_t slot = slot0 + (ok ? t : 0u);
        const uint8_t *src = a.idx_bytes + slot * (2 * NB) + hk * NB;
        if constexpr (NW == 2) {
            tq_u2 v = {0u, 0u};
            if (ok) v = tq_gload8(src);
            raw[0] = v[0]; raw[1] = v[1];
        } else {
#pragma unroll
            for (int q = 0; q < NW / 4; ++q) {
                tq_u4 v = {0u, 0u, 0u, 0u};
                if (ok) v = tq_gload16(src + 16 * q);
#pragma unroll
                for (int i = 0; i < 4; ++i) raw[4 * q + i] = v[i];
            }
        }
        norm_bits = ok ? tq_gload2(a.vec_norms + slot) : (uint16_t)0;
    };
    if (tile < n_tiles) issue_loads(tile);
    while (tile < n_tiles) {
        uint32_t cur[NW];
#pragma unroll
        for (int i = 0; i < NW; ++i) cur[i] = raw[i];
        const float nrm = (float)__builtin_bit_cast(_Float16, norm_bits);
        const uint32_t next = tile + tile_stride;
        if (next < n_tiles) issue_loads(next);

        tq_f16v acc = tq_zero16();
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            const tq_u4 b = decode_step<IPB, NW>(cur, s, lds_lut);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(tq_half8, ahi[s]), __builtin_bit_cast(tq_half8, b), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(tq_half8, alo[s]), __builtin_bit_cast(tq_half8, b), acc, 0, 0, 0);
        }
        const uint32_t t = tile * 32u + n;
        if (t < a.tokens) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t m = 8u * (r / 4) + 4u * hk + (r % 4);
                if (m < a.group)
                    ((TQ_GLOBAL float *)a.scores)[((size_t)row * a.group + m) * a.stride + t] = acc[r] * rowscale[r] * nrm;
            }
        }
        tile = next;
    }
}

struct WvArgs {
    const uint8_t *idx_bytes;
    const uint16_t *vec_norms;
    const uint8_t *table;
    const float *weights;    // q head (row * group + g), token t at (row * group + g) * stride + t
    float *partial;          // [rows, splits, group, 128]
    long long stride;
    uint32_t tokens, packed_row_stride, group, chunk;   // chunk: tokens per split (multiple of 32)
};

// Block (split, row): sum over the split's tokens of  weight[g][t] * norm_t * centroids[codes_t]  for the
// row's `group` query heads, in the rotated space: a [group x tokens] x [tokens x 128] product whose
// contraction runs over tokens, on v_mfma_f32_32x32x16_f16.  A wave takes runs of up to 128 tokens (4 KiB of
// packed bytes, so that enough memory traffic is in flight per wave; loads run one run ahead):
//   * the run's packed bytes (contiguous in memory), norms and weights are staged in a wave-private LDS area;
//   * per tile of 32 tokens, lane (n, hk) owns coordinates 4n .. 4n+3 and, per MFMA step ks, tokens
//     16ks + 8hk + i (i < 8): for each of those tokens it reads the byte(s) holding its four codes and looks them
//     up in the byte -> centroids table, so every lookup is used in full; a token-pair byte permute inside the
//     lane turns the 8 x 4 values into four B operands (one per coordinate: MFMA column n of column tile c is
//     coordinate 4n + c), scaled by the tokens' norms in packed fp16;
//   * the A operand holds the weights (rows = query heads, zero above `group`) as fp16 hi + lo of
//     w * 2^14: weights are probabilities, so everything down to 2^-38 keeps at least a denormal.
// Accumulators (4 column tiles) live in registers across the split; the four waves' sums meet in LDS.
template <int IPB>
__global__ __launch_bounds__(WV_WAVES *TQ_WAVE) void tq_weighted_values_kernel(WvArgs a) {
    constexpr int GB = TQ_HEAD_DIM / IPB;                    // packed bytes per vector: 16 .. 128
    constexpr int SUB = GB >= 128 ? 1 : GB >= 64 ? 2 : 4;    // 32-token tiles per run
    constexpr int RUN = 32 * SUB;                            // tokens per run: 32, 64, 128
    constexpr int CODE_BYTES = RUN * GB;                     // <= 4096
    constexpr int CPIECES = CODE_BYTES / 16;                 // 16-byte pieces of packed bytes per run
    constexpr int NCP = (CPIECES + 63) / 64;
    constexpr int WROW = RUN / 4;                            // 16-byte pieces per weight row and run
    constexpr int WPIECES = WV_MAX_GROUP * WROW;
    constexpr int NWP = (WPIECES + 63) / 64;
    constexpr int W_SHIFT = 14;
    constexpr int AREA = 4096 + WV_MAX_GROUP * RUN * 4;      // per wave: staged codes + weights, later the wave's sums
    static_assert(CODE_BYTES <= 4096 && WV_MAX_GROUP * TQ_HEAD_DIM * 4 <= AREA, "wave area too small");
    __shared__ __attribute__((aligned(16))) uint8_t lds_lut[4096];
    __shared__ __attribute__((aligned(16))) uint8_t lds_area[WV_WAVES][AREA];
    __shared__ __attribute__((aligned(16))) uint16_t lds_norm[WV_WAVES][RUN];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t row = blockIdx.y, split = blockIdx.x;
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(a.table);
    tq_copy_to_lds(lds_lut, a.table + hd->off_lut, 256u * 2u * IPB, tid, WV_WAVES * TQ_WAVE);
    __syncthreads();

    const uint32_t t_begin = split * a.chunk;
    const uint32_t t_end = min(a.tokens, t_begin + a.chunk);
    const size_t slot0 = (size_t)row * a.packed_row_stride;
    const uint32_t G = a.group;
    const bool live = n < G;                                   // this lane's MFMA row is a query head
    const TQ_GLOBAL float *wbase = (const TQ_GLOBAL float *)a.weights + (size_t)row * G * a.stride;
    uint8_t *codes = lds_area[wave];
    float *wst = reinterpret_cast<float *>(lds_area[wave] + 4096);      // [query head][token of the run]
    // rows of the weight matrix start 16-byte aligned: four weights are one vector load
    const bool aligned_rows = (a.stride % 4 == 0) && (((uintptr_t)a.weights & 15u) == 0);

    tq_f16v acc[TQ_TILES];
#pragma unroll
    for (int c = 0; c < TQ_TILES; ++c) acc[c] = tq_zero16();

    // loads of a run, issued one run ahead of their use
    tq_u4 code_next[NCP];
    tq_u4 w_next[NWP];
    uint16_t norm_next[(RUN + 63) / 64];
    auto issue_loads = [&](uint32_t t0) {
        const uint32_t n_tok = min((uint32_t)RUN, t_end - t0);
        const uint8_t *src = a.idx_bytes + (slot0 + t0) * GB;
#pragma unroll
        for (int p = 0; p < NCP; ++p) {
            const uint32_t piece = p * 64u + lane;
            const bool ok = piece < CPIECES && piece * 16u < n_tok * GB;
            code_next[p] = tq_gload16(src + (ok ? piece : 0u) * 16u);
        }
#pragma unroll
        for (int p = 0; p < (RUN + 63) / 64; ++p) {
            const uint32_t tl = p * 64u + lane;
            norm_next[p] = (tl < n_tok) ? tq_gload2(a.vec_norms + slot0 + t0 + tl) : (uint16_t)0;   // tokens past the end weigh nothing
        }
#pragma unroll
        for (int p = 0; p < NWP; ++p) {
            const uint32_t piece = p * 64u + lane;
            const uint32_t g = piece / WROW, tl = (piece % WROW) * 4u;
            tq_u4 v = {0u, 0u, 0u, 0u};
            if (piece < WPIECES && g < G && tl < n_tok) {
                const TQ_GLOBAL float *wp = wbase + (size_t)g * a.stride + t0 + tl;
                if (aligned_rows && tl + 4u <= n_tok) {
                    v = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>(wp);
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[i] = (tl + i < n_tok) ? __float_as_uint(wp[i]) : 0u;
                }
            }
            w_next[p] = v;
        }
    };
    uint32_t t0 = t_begin + RUN * wave;
    if (t0 < t_end) issue_loads(t0);
    while (t0 < t_end) {
        // ---- stage the run: packed bytes [token][GB], norms [token], weights [head][token]
#pragma unroll
        for (int p = 0; p < NCP; ++p) {
            const uint32_t piece = p * 64u + lane;
            if (piece < CPIECES) *reinterpret_cast<tq_u4 *>(codes + piece * 16u) = code_next[p];
        }
#pragma unroll
        for (int p = 0; p < (RUN + 63) / 64; ++p) {
            const uint32_t tl = p * 64u + lane;
            if (tl < RUN) lds_norm[wave][tl] = norm_next[p];
        }
#pragma unroll
        for (int p = 0; p < NWP; ++p) {
            const uint32_t piece = p * 64u + lane;
            if (piece < WPIECES) *reinterpret_cast<tq_u4 *>(wst + piece * 4u) = w_next[p];
        }
        const uint32_t t_next = t0 + RUN * WV_WAVES;
        if (t_next < t_end) issue_loads(t_next);
        // staged as 16-byte vectors, read back in other units: no compiler reordering across this point
        // (the LDS itself serves a wave in order)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int u = 0; u < SUB; ++u) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const uint32_t tl0 = 32u * u + 16u * ks + 8u * hk;          // this lane's eight tokens of the step
                // weights of this lane's query head, fp16 hi + lo of w * 2^W_SHIFT
                tq_u4 whi = {0u, 0u, 0u, 0u}, wlo = {0u, 0u, 0u, 0u};
                if (live) {
                    const float4 w0 = *reinterpret_cast<const float4 *>(wst + n * RUN + tl0);
                    const float4 w1 = *reinterpret_cast<const float4 *>(wst + n * RUN + tl0 + 4);
                    const float x[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
                    tq_half8 h, l;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const float xs = x[i] * (float)(1 << W_SHIFT);
                        const _Float16 xh = (_Float16)xs;
                        h[i] = xh;
                        l[i] = (_Float16)(xs - (float)xh);
                    }
                    whi = __builtin_bit_cast(tq_u4, h);
                    wlo = __builtin_bit_cast(tq_u4, l);
                }
                const tq_u4 nrm = *reinterpret_cast<const tq_u4 *>(&lds_norm[wave][tl0]);   // fp16 norms of the eight tokens
                uint32_t lo[8], hi[8];   // per token: centroids of coordinates (4n, 4n+1) and (4n+2, 4n+3)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint8_t *tok = codes + (tl0 + i) * GB;
                    if constexpr (IPB == 8) {          // half a byte holds the lane's four codes
                        const uint32_t b = tok[n >> 1];
                        const tq_u2 v = *reinterpret_cast<const tq_u2 *>(lds_lut + b * 16u + (n & 1u) * 8u);
                        lo[i] = v[0]; hi[i] = v[1];
                    } else if constexpr (IPB == 4) {   // one byte
                        const uint32_t b = tok[n];
                        const tq_u2 v = *reinterpret_cast<const tq_u2 *>(lds_lut + b * 8u);
                        lo[i] = v[0]; hi[i] = v[1];
                    } else if constexpr (IPB == 2) {   // two bytes
                        const uint32_t two = *reinterpret_cast<const uint16_t *>(tok + 2u * n);
                        lo[i] = *reinterpret_cast<const uint32_t *>(lds_lut + (two & 0xffu) * 4u);
                        hi[i] = *reinterpret_cast<const uint32_t *>(lds_lut + (two >> 8) * 4u);
                    } else {                           // four bytes, one code each
                        const uint32_t four = *reinterpret_cast<const uint32_t *>(tok + 4u * n);
                        const uint32_t c0 = *reinterpret_cast<const uint16_t *>(lds_lut + (four & 0xffu) * 2u);
                        const uint32_t c1 = *reinterpret_cast<const uint16_t *>(lds_lut + ((four >> 8) & 0xffu) * 2u);
                        const uint32_t c2 = *reinterpret_cast<const uint16_t *>(lds_lut + ((four >> 16) & 0xffu) * 2u);
                        const uint32_t c3 = *reinterpret_cast<const uint16_t *>(lds_lut + (four >> 24) * 2u);
                        lo[i] = c0 | (c1 << 16); hi[i] = c2 | (c3 << 16);
                    }
                }
#pragma unroll
                for (int c = 0; c < TQ_TILES; ++c) {
                    // coordinate 4n + c of the eight tokens: token pairs (2d, 2d+1) side by side, times their norms
                    tq_u4 bt;
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const uint32_t even = c < 2 ? lo[2 * d] : hi[2 * d], odd = c < 2 ? lo[2 * d + 1] : hi[2 * d + 1];
                        bt[d] = __builtin_amdgcn_perm(odd, even, (c & 1) ? 0x07060302u : 0x05040100u);
                    }
                    const tq_half8 y = __builtin_bit_cast(tq_half8, bt) * __builtin_bit_cast(tq_half8, nrm);
                    acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(tq_half8, whi), y, acc[c], 0, 0, 0);
                    acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(tq_half8, wlo), y, acc[c], 0, 0, 0);
                }
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        t0 = t_next;
    }
    asm volatile("" ::: "memory");
    // accumulator register r of lane (n, hk), column tile c: query head 8*(r/4) + 4*hk + r%4, coordinate 4n + c
    float *sums = reinterpret_cast<float *>(lds_area[wave]);
#pragma unroll
    for (int c = 0; c < TQ_TILES; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t m = 8u * (r / 4) + 4u * hk + (r % 4);
            if (m < WV_MAX_GROUP) sums[m * TQ_HEAD_DIM + 4u * n + c] = acc[c][r] * (1.0f / (float)(1 << W_SHIFT));
        }
    __syncthreads();
    float *dst = a.partial + ((size_t)row * gridDim.x + split) * G * TQ_HEAD_DIM;
    for (uint32_t i = tid; i < G * TQ_HEAD_DIM; i += WV_WAVES * TQ_WAVE) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < WV_WAVES; ++w) s += reinterpret_cast<const float *>(lds_area[w])[i];
        ((TQ_GLOBAL float *)dst)[i] = s;
    }
}

// out[row][g][j] = sum over splits of partial[row][split][g][j], in split order (deterministic)
__global__ __launch_bounds__(256) void tq_reduce_splits_kernel(const float *partial, float *out, uint32_t per_row, uint32_t splits,
                                                               uint32_t total) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= total) return;
    const uint32_t row = i / per_row, k = i % per_row;
    const TQ_GLOBAL float *p = (const TQ_GLOBAL float *)partial + (size_t)row * splits * per_row + k;
    float s = 0.f;
    for (uint32_t sp = 0; sp < splits; ++sp) s += p[(size_t)sp * per_row];
    ((TQ_GLOBAL float *)out)[i] = s;
}

// ---- one pass over packed keys and values: scores, online softmax, weighted values ------------------------
struct AttendArgs {
    const uint8_t *k_idx, *v_idx;
    const uint16_t *k_norms, *v_norms;
    const uint8_t *table_k, *table_v;
    const float *q_rot;      // [rows, group, 128], softmax scale folded in
    float *partial;          // [rows, splits, group, 130]: largest score, sum of exp(score - largest), 128 weighted sums
    uint32_t tokens, packed_row_stride, group, chunk;
};
constexpr int AT_WAVES = 4;
constexpr int AT_RUN = 64;       // tokens per wave and trip
constexpr int AT_PART = TQ_HEAD_DIM + 2;

// Block (split, row), wave = runs of 64 tokens of the split, tile = 32 tokens.  Per tile:
//   S^T = K_dec * Q~^T on the matrix cores with the decoded keys as the A operand (rows = tokens, the natural
//     layout of the decode) and the rotated queries as B (columns = query heads), so that lane (g, h) ends up with
//     the scores of query head g against 16 tokens of the tile: the softmax statistics of a head stay inside two lanes;
//   online softmax in base 2 (running maximum m, sum l, both per lane; the two lanes of a head agree on m);
//   the probabilities, already in the lanes that own head g as an MFMA row, become the A operand of
//     P * V_dec (fp16 of p * 2^14); the tokens of a contraction slice are the ones the score registers hold,
//     16ks + 8(i/4) + 4h + i%4, and the B operand is built for exactly those tokens the way the weighted-values
//     kernel builds it (lane (n, h) owns coordinates 4n .. 4n+3, byte lookups + in-lane token-pair permutes, norms
//     folded in as packed fp16);
//   when a head's maximum moves, the value accumulators of its row are rescaled (factors passed through LDS).
// The four waves' (m, l, sums) are merged in LDS; splits and the uncompressed window are merged by the caller.
// Query heads per row: at most 8.
template <int IPBK, int IPBV>
__global__ __launch_bounds__(AT_WAVES *TQ_WAVE, 2) void tq_attend_kernel(AttendArgs a) {
    constexpr int NBK = 64 / IPBK, NWK = NBK / 4;        // key bytes / dwords per lane (half a vector)
    constexpr int GBV = TQ_HEAD_DIM / IPBV;              // value bytes per vector
    constexpr int SUB = AT_RUN / 32;
    constexpr int VBYTES = AT_RUN * GBV;                 // <= 8192
    constexpr int VPIECES = VBYTES / 16, NVP = (VPIECES + 63) / 64;
    constexpr int P_SHIFT = 14;
    constexpr int AREA = VBYTES > 8 * AT_PART * 4 ? VBYTES : 8 * AT_PART * 4;   // staged value codes, later the wave's result
    __shared__ __attribute__((aligned(16))) uint8_t lds_lut_k[4096];
    __shared__ __attribute__((aligned(16))) uint8_t lds_lut_v[4096];
    __shared__ __attribute__((aligned(16))) uint8_t lds_area[AT_WAVES][AREA];
    __shared__ __attribute__((aligned(16))) uint16_t lds_kn[AT_WAVES][AT_RUN];
    __shared__ __attribute__((aligned(16))) uint16_t lds_vn[AT_WAVES][AT_RUN];
    __shared__ __attribute__((aligned(16))) float lds_corr[AT_WAVES][8];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t row = blockIdx.y, split = blockIdx.x;
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const TqTableHeader *hk_hd = reinterpret_cast<const TqTableHeader *>(a.table_k);
    const TqTableHeader *hv_hd = reinterpret_cast<const TqTableHeader *>(a.table_v);
    tq_copy_to_lds(lds_lut_k, a.table_k + hk_hd->off_lut, 256u * 2u * IPBK, tid, AT_WAVES * TQ_WAVE);
    tq_copy_to_lds(lds_lut_v, a.table_v + hv_hd->off_lut, 256u * 2u * IPBV, tid, AT_WAVES * TQ_WAVE);

    const uint32_t G = a.group;
    const bool live = n < G;
    // ---- B operand of the score product: query head g = n, contraction slice (s, hk) = coordinates 64hk + 8s + i,
    //      fp16 hi + lo of q * 2^(10 - e) with e the binary exponent of the head's largest magnitude
    tq_u4 qhi[TQ_STEPS], qlo[TQ_STEPS];
    float c1;                // score in base-2 units = t * c1, t = accumulator * key norm
    float rowscale;          // natural score = t * rowscale
    {
        const TQ_GLOBAL float *q = (const TQ_GLOBAL float *)a.q_rot + ((size_t)row * G + (live ? n : 0u)) * TQ_HEAD_DIM + 64u * hk;
        float big = 0.f;
        for (int i = 0; i < 64; ++i) big = fmaxf(big, fabsf(q[i]));
        big = fmaxf(big, __shfl_xor(big, 32));
        int e = 0;
        if (big > 0.f && big < __builtin_inff()) (void)frexpf(big, &e);
        e = e < -100 ? -100 : e;
        const float up = ldexpf(1.f, TQ_F16_PI_SHIFT - e);
        rowscale = live ? ldexpf(1.f, e - TQ_F16_PI_SHIFT) : 0.f;
        c1 = rowscale * 1.44269504088896341f;
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            tq_half8 h, l;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float x = live ? q[8 * s + i] * up : 0.f;
                const _Float16 xh = (_Float16)x;
                h[i] = xh;
                l[i] = (_Float16)(x - (float)xh);
            }
            qhi[s] = __builtin_bit_cast(tq_u4, h);
            qlo[s] = __builtin_bit_cast(tq_u4, l);
        }
    }
    __syncthreads();

    const uint32_t t_begin = split * a.chunk;
    const uint32_t t_end = min(a.tokens, t_begin + a.chunk);
    const size_t slot0 = (size_t)row * a.packed_row_stride;
    uint8_t *vcodes = lds_area[wave];

    tq_f16v acc[TQ_TILES];   // weighted value sums: row = query head, column n of tile c = coordinate 4n + c
#pragma unroll
    for (int c = 0; c < TQ_TILES; ++c) acc[c] = tq_zero16();
    float m_run = -1e30f;    // running maximum of t for this lane's head
    float l_run = 0.f;       // running sum of p * 2^P_SHIFT over this lane's tokens

    // loads of a run, issued one run ahead
    uint32_t kraw_next[SUB][NWK];
    tq_u4 vpiece_next[NVP];
    uint16_t kn_next = 0, vn_next = 0;
    auto issue_loads = [&](uint32_t t0) {
        const uint32_t n_tok = min((uint32_t)AT_RUN, t_end - t0);
#pragma unroll
        for (int u = 0; u < SUB; ++u) {
            const uint32_t tl = 32u * u + n;
            const uint8_t *src = a.k_idx + (slot0 + t0 + (tl < n_tok ? tl : 0u)) * (2 * NBK) + hk * NBK;
            if constexpr (NWK == 2) {
                const tq_u2 v = tq_gload8(src);
                kraw_next[u][0] = v[0]; kraw_next[u][1] = v[1];
            } else {
#pragma unroll
                for (int q = 0; q < NWK / 4; ++q) {
                    const tq_u4 v = tq_gload16(src + 16 * q);
#pragma unroll
                    for (int i = 0; i < 4; ++i) kraw_next[u][4 * q + i] = v[i];
                }
            }
        }
        const uint8_t *vsrc = a.v_idx + (slot0 + t0) * GBV;
#pragma unroll
        for (int p = 0; p < NVP; ++p) {
            const uint32_t piece = p * 64u + lane;
            const bool ok = piece < VPIECES && piece * 16u < n_tok * GBV;
            vpiece_next[p] = tq_gload16(vsrc + (ok ? piece : 0u) * 16u);
        }
        kn_next = lane < n_tok ? tq_gload2(a.k_norms + slot0 + t0 + lane) : (uint16_t)0;
        vn_next = lane < n_tok ? tq_gload2(a.v_norms + slot0 + t0 + lane) : (uint16_t)0;   // tokens past the end weigh nothing
    };
    uint32_t t0 = t_begin + AT_RUN * wave;
    if (t0 < t_end) issue_loads(t0);
    while (t0 < t_end) {
        const uint32_t n_tok = min((uint32_t)AT_RUN, t_end - t0);
        uint32_t kraw[SUB][NWK];
#pragma unroll
        for (int u = 0; u < SUB; ++u)
#pragma unroll
            for (int i = 0; i < NWK; ++i) kraw[u][i] = kraw_next[u][i];
#pragma unroll
        for (int p = 0; p < NVP; ++p) {
            const uint32_t piece = p * 64u + lane;
            if (piece < VPIECES) *reinterpret_cast<tq_u4 *>(vcodes + piece * 16u) = vpiece_next[p];
        }
        lds_kn[wave][lane] = kn_next;
        lds_vn[wave][lane] = vn_next;
        const uint32_t t_next = t0 + AT_RUN * AT_WAVES;
        if (t_next < t_end) issue_loads(t_next);
        asm volatile("" ::: "memory");    // staged with one access width, read back with others (LDS serves a wave in order)
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int u = 0; u < SUB; ++u) {
            if (32u * u >= n_tok) break;  // uniform
            // ---- scores: lane (g, hk) gets tokens 8*(r/4) + 4*hk + r%4 of the tile in register r
            tq_f16v sc = tq_zero16();
#pragma unroll
            for (int s = 0; s < TQ_STEPS; ++s) {
                const tq_half8 kd = __builtin_bit_cast(tq_half8, decode_step<IPBK, NWK>(kraw[u], s, lds_lut_k));
                sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kd, __builtin_bit_cast(tq_half8, qhi[s]), sc, 0, 0, 0);
                sc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kd, __builtin_bit_cast(tq_half8, qlo[s]), sc, 0, 0, 0);
            }
            float t[16];
            float tmax = -1e30f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const tq_u2 kn4 = *reinterpret_cast<const tq_u2 *>(&lds_kn[wave][32u * u + 8u * j + 4u * hk]);
                // (whole-vector cast: casting single 32-bit elements of a vector to fp16 pairs miscompiles)
                typedef _Float16 half4 __attribute__((ext_vector_type(4)));
                const half4 k4 = __builtin_bit_cast(half4, kn4);
#pragma unroll
                for (int q = 0; q < 4; ++q) t[4 * j + q] = sc[4 * j + q] * (float)k4[q];
            }
            const bool partial_tile = 32u * u + 32u > n_tok;   // uniform
            if (partial_tile) {
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (32u * u + 8u * (r / 4) + 4u * hk + (r % 4) >= n_tok) t[r] = -1e30f;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, t[r]);
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
            const float m_new = fmaxf(m_run, tmax);
            const float corr = __builtin_amdgcn_exp2f((m_run - m_new) * c1);
            const float bias = P_SHIFT - m_new * c1;
            float ps[16];
            float lsum = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                ps[r] = __builtin_amdgcn_exp2f(fmaf(t[r], c1, bias));     // p * 2^P_SHIFT
                lsum += ps[r];
            }
            if (partial_tile) {       // a zero query makes every exponent 0: masked tokens need an explicit zero
                lsum = 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    if (32u * u + 8u * (r / 4) + 4u * hk + (r % 4) >= n_tok) ps[r] = 0.f;
                    lsum += ps[r];
                }
            }
            l_run = l_run * corr + lsum;
            // ---- the head's maximum moved: rescale the value sums of its row
            if (__any(m_new != m_run)) {
                if (hk == 0u && n < 8u) lds_corr[wave][n] = corr;
                asm volatile("" ::: "memory");
                __builtin_amdgcn_wave_barrier();
                const float4 c4 = *reinterpret_cast<const float4 *>(&lds_corr[wave][4u * hk]);
                asm volatile("" ::: "memory");
#pragma unroll
                for (int c = 0; c < TQ_TILES; ++c) {
                    acc[c][0] *= c4.x; acc[c][1] *= c4.y; acc[c][2] *= c4.z; acc[c][3] *= c4.w;
                }
            }
            m_run = m_new;
            // ---- P * V for the tile: contraction slices ks, tokens 16ks + 8(i/4) + 4hk + i%4
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                tq_half8 pa;
#pragma unroll
                for (int i = 0; i < 8; ++i) pa[i] = (_Float16)ps[8 * ks + i];
                const uint32_t tl0 = 32u * u + 16u * ks + 4u * hk;
                const tq_u2 vn_a = *reinterpret_cast<const tq_u2 *>(&lds_vn[wave][tl0]);        // tokens tl0 .. tl0+3
                const tq_u2 vn_b = *reinterpret_cast<const tq_u2 *>(&lds_vn[wave][tl0 + 8u]);   // tokens tl0+8 .. tl0+11
                const tq_u4 nrm = {vn_a[0], vn_a[1], vn_b[0], vn_b[1]};
                uint32_t lo[8], hi[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint8_t *tok = vcodes + (tl0 + 8u * (i / 4) + (i % 4)) * GBV;
                    if constexpr (IPBV == 8) {
                        const uint32_t b = tok[n >> 1];
                        const tq_u2 v = *reinterpret_cast<const tq_u2 *>(lds_lut_v + b * 16u + (n & 1u) * 8u);
                        lo[i] = v[0]; hi[i] = v[1];
                    } else if constexpr (IPBV == 4) {
                        const uint32_t b = tok[n];
                        const tq_u2 v = *reinterpret_cast<const tq_u2 *>(lds_lut_v + b * 8u);
                        lo[i] = v[0]; hi[i] = v[1];
                    } else if constexpr (IPBV == 2) {
                        const uint32_t two = *reinterpret_cast<const uint16_t *>(tok + 2u * n);
                        lo[i] = *reinterpret_cast<const uint32_t *>(lds_lut_v + (two & 0xffu) * 4u);
                        hi[i] = *reinterpret_cast<const uint32_t *>(lds_lut_v + (two >> 8) * 4u);
                    } else {
                        const uint32_t four = *reinterpret_cast<const uint32_t *>(tok + 4u * n);
                        const uint32_t c0 = *reinterpret_cast<const uint16_t *>(lds_lut_v + (four & 0xffu) * 2u);
                        const uint32_t c1v = *reinterpret_cast<const uint16_t *>(lds_lut_v + ((four >> 8) & 0xffu) * 2u);
                        const uint32_t c2 = *reinterpret_cast<const uint16_t *>(lds_lut_v + ((four >> 16) & 0xffu) * 2u);
                        const uint32_t c3 = *reinterpret_cast<const uint16_t *>(lds_lut_v + (four >> 24) * 2u);
                        lo[i] = c0 | (c1v << 16); hi[i] = c2 | (c3 << 16);
                    }
                }
#pragma unroll
                for (int c = 0; c < TQ_TILES; ++c) {
                    tq_u4 bt;
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const uint32_t even = c < 2 ? lo[2 * d] : hi[2 * d], odd = c < 2 ? lo[2 * d + 1] : hi[2 * d + 1];
                        bt[d] = __builtin_amdgcn_perm(odd, even, (c & 1) ? 0x07060302u : 0x05040100u);
                    }
                    const tq_half8 y = __builtin_bit_cast(tq_half8, bt) * __builtin_bit_cast(tq_half8, nrm);
                    acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(pa, y, acc[c], 0, 0, 0);
                }
            }
        }
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        t0 = t_next;
    }
    asm volatile("" ::: "memory");
    // ---- this wave's result for heads 0..7: [head][largest natural score, sum, 128 sums] in its LDS area
    float *res = reinterpret_cast<float *>(lds_area[wave]);
    {
        const float l_all = (l_run + __shfl_xor(l_run, 32)) * (1.0f / (float)(1 << P_SHIFT));
        if (hk == 0u && n < 8u) {
            res[n * AT_PART + 0] = m_run * rowscale;
            res[n * AT_PART + 1] = l_all;
        }
#pragma unroll
        for (int c = 0; c < TQ_TILES; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                res[(4u * hk + r) * AT_PART + 2 + 4u * n + c] = acc[c][r] * (1.0f / (float)(1 << P_SHIFT));
    }
    __syncthreads();
    // ---- merge the four waves
    float *dst = a.partial + ((size_t)row * gridDim.x + split) * G * AT_PART;
    for (uint32_t i = tid; i < G * AT_PART; i += AT_WAVES * TQ_WAVE) {
        const uint32_t g = i / AT_PART, j = i % AT_PART;
        float mw[AT_WAVES], mall = -3.0e38f;
#pragma unroll
        for (int w = 0; w < AT_WAVES; ++w) {
            mw[w] = reinterpret_cast<const float *>(lds_area[w])[g * AT_PART];
            mall = fmaxf(mall, mw[w]);
        }
        float out;
        if (j == 0) {
            out = mall;
        } else {
            out = 0.f;
#pragma unroll
            for (int w = 0; w < AT_WAVES; ++w)
                out += __expf(mw[w] - mall) * reinterpret_cast<const float *>(lds_area[w])[g * AT_PART + j];
        }
        ((TQ_GLOBAL float *)dst)[i] = out;
    }
}

// ---- the small ends of a decode step: query rotation + uncompressed window, and the final merge -----------
struct PrepareArgs {
    const void *queries;     // [rows, group, 128] elements of q_dtype (one query token), contiguous
    const float *pi_k_t;     // [128, 128] transposed rotation of the key codec: element [i][j] = Pi[j][i]
    const void *k_win, *v_win;   // window keys / values: row r, token t at element r * win_stride + t * 128
    float *q_rot;            // out: [rows, group, 128] = scale * Pi q
    float *part_w;           // out: [rows, group, 130]: largest window score, sum of exp, 128 weighted value sums
    long long win_stride;
    float scale;
    uint32_t group, n_win;
    int q_dtype, win_dtype;
};

__device__ __forceinline__ float tq_load_elem(const void *base, size_t i, int dtype) {
    if (dtype == TQ_F32) return ((const TQ_GLOBAL float *)base)[i];
    const uint16_t b = ((const TQ_GLOBAL uint16_t *)base)[i];
    if (dtype == TQ_F16) return (float)__builtin_bit_cast(_Float16, b);
    return __uint_as_float((uint32_t)b << 16);
}

// Eight consecutive window elements starting at element index i (a multiple of 8) as floats.
template <int WD>
__device__ __forceinline__ void tq_load8(const void *base, size_t i, float (&x)[8]) {
    if constexpr (WD == TQ_F32) {
        const tq_u4 lo = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>((const TQ_GLOBAL float *)base + i);
        const tq_u4 hi = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>((const TQ_GLOBAL float *)base + i + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) { x[e] = __uint_as_float(lo[e]); x[4 + e] = __uint_as_float(hi[e]); }
    } else {
        const tq_u4 u = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>((const TQ_GLOBAL uint16_t *)base + i);
        if constexpr (WD == TQ_F16) {
            const tq_half8 h = __builtin_bit_cast(tq_half8, u);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = (float)h[e];
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) { x[2 * e] = __uint_as_float(u[e] << 16); x[2 * e + 1] = __uint_as_float(u[e] & 0xffff0000u); }
        }
    }
}

// Two consecutive window elements starting at element index i (even).
template <int WD>
__device__ __forceinline__ void tq_load2(const void *base, size_t i, float &x0, float &x1) {
    if constexpr (WD == TQ_F32) {
        const tq_u2 u = *reinterpret_cast<const TQ_GLOBAL tq_u2 *>((const TQ_GLOBAL float *)base + i);
        x0 = __uint_as_float(u[0]); x1 = __uint_as_float(u[1]);
    } else {
        const uint32_t u = *reinterpret_cast<const TQ_GLOBAL uint32_t *>((const TQ_GLOBAL uint16_t *)base + i);
        if constexpr (WD == TQ_F16) {
            const tq_half2 h = __builtin_bit_cast(tq_half2, u);
            x0 = (float)h[0]; x1 = (float)h[1];
        } else {
            x0 = __uint_as_float(u << 16); x1 = __uint_as_float(u & 0xffff0000u);
        }
    }
}

// One block per packed row (batch x kv head), four waves.  Rotates the row's query heads for the packed keys and
// computes attention statistics over the uncompressed window tokens in fp32 (a few hundred tokens at most).
//   rotation   : thread (j, half) sums 64 of the 128 terms of every head's q_rot[j]; Pi^T is read once, coalesced
//   scores     : 16 lanes x 16 bytes cover one token, a wave takes four tokens per load; sums meet over 16 lanes
//   statistics : wave w owns heads w and w + 4
//   value sums : thread (column pair, wave) over every fourth token, the four waves' sums meet in LDS
template <int WD>
__global__ __launch_bounds__(256) void tq_attend_prepare_kernel(PrepareArgs a) {
    constexpr int MAXG = 8, MAXW = 512;
    __shared__ float q[MAXG][TQ_HEAD_DIM];
    __shared__ float sc[MAXG][MAXW];
    __shared__ float red[MAXG][2];
    __shared__ float part[4][MAXG][TQ_HEAD_DIM];
    const uint32_t row = blockIdx.x, tid = threadIdx.x, G = a.group, lane = tid & 63u, wave = tid >> 6;
    for (uint32_t i = tid; i < MAXG * TQ_HEAD_DIM; i += 256u)
        q[i / TQ_HEAD_DIM][i % TQ_HEAD_DIM] =
            i < G * TQ_HEAD_DIM ? tq_load_elem(a.queries, (size_t)row * G * TQ_HEAD_DIM + i, a.q_dtype) * a.scale : 0.f;
    __syncthreads();
    {   // rotated queries: q_rot[g][j] = sum_i Pi[j][i] * q[g][i]
        const uint32_t j = tid & 127u, half = tid >> 7;
        const TQ_GLOBAL float *pc = (const TQ_GLOBAL float *)a.pi_k_t + (size_t)half * 64u * TQ_HEAD_DIM + j;
        float s[MAXG];
#pragma unroll
        for (int g = 0; g < MAXG; ++g) s[g] = 0.f;
#pragma unroll 8
        for (int i = 0; i < 64; ++i) {
            const float p = pc[(size_t)i * TQ_HEAD_DIM];
#pragma unroll
            for (int g = 0; g < MAXG; ++g) s[g] = fmaf(p, q[g][half * 64u + i], s[g]);
        }
#pragma unroll
        for (int g = 0; g < MAXG; ++g) part[half][g][j] = s[g];
    }
    __syncthreads();
    for (uint32_t o = tid; o < G * TQ_HEAD_DIM; o += 256u)
        ((TQ_GLOBAL float *)a.q_rot)[(size_t)row * G * TQ_HEAD_DIM + o] =
            part[0][o / TQ_HEAD_DIM][o % TQ_HEAD_DIM] + part[1][o / TQ_HEAD_DIM][o % TQ_HEAD_DIM];
    if (!a.part_w) return;
    const uint32_t W = a.n_win;
    const size_t win_base = (size_t)row * a.win_stride;
    {   // scores of the window tokens
        const uint32_t sub = lane & 15u, tk = lane >> 4;
        float qq[MAXG][8];
#pragma unroll
        for (int g = 0; g < MAXG; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) qq[g][e] = q[g][8u * sub + e];
        for (uint32_t t0 = 4u * wave; t0 < W; t0 += 16u) {
            const uint32_t t = t0 + tk;
            float x[8];
            if (t < W) {
                tq_load8<WD>(a.k_win, win_base + (size_t)t * TQ_HEAD_DIM + 8u * sub, x);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = 0.f;
            }
#pragma unroll
            for (int g = 0; g < MAXG; ++g) {
                if ((uint32_t)g < G) {           // uniform over the block
                    float sg = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) sg = fmaf(x[e], qq[g][e], sg);
                    sg += __shfl_xor(sg, 1);
                    sg += __shfl_xor(sg, 2);
                    sg += __shfl_xor(sg, 4);
                    sg += __shfl_xor(sg, 8);
                    if (sub == 0u && t < W) sc[g][t] = sg;
                }
            }
        }
    }
    __syncthreads();                      // (the value sums below reuse `part`: every q_rot read of it is behind us)
    for (uint32_t g = wave; g < G; g += 4u) {
        float m = -3.0e38f;
        for (uint32_t t = lane; t < W; t += 64u) m = fmaxf(m, sc[g][t]);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d));
        float l = 0.f;
        for (uint32_t t = lane; t < W; t += 64u) {
            const float p = __expf(sc[g][t] - m);
            sc[g][t] = p;
            l += p;
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) l += __shfl_xor(l, d);
        if (lane == 0u) { red[g][0] = m; red[g][1] = l; }
    }
    __syncthreads();
    {   // weighted value sums: this thread's two columns over tokens wave, wave + 4, ...
        float acc[MAXG][2];
#pragma unroll
        for (int g = 0; g < MAXG; ++g) acc[g][0] = acc[g][1] = 0.f;
#pragma unroll 4
        for (uint32_t t = wave; t < W; t += 4u) {
            float x0, x1;
            tq_load2<WD>(a.v_win, win_base + (size_t)t * TQ_HEAD_DIM + 2u * lane, x0, x1);
#pragma unroll
            for (int g = 0; g < MAXG; ++g) {
                if ((uint32_t)g < G) {
                    const float p = sc[g][t];
                    acc[g][0] = fmaf(p, x0, acc[g][0]);
                    acc[g][1] = fmaf(p, x1, acc[g][1]);
                }
            }
        }
#pragma unroll
        for (int g = 0; g < MAXG; ++g) { part[wave][g][2u * lane] = acc[g][0]; part[wave][g][2u * lane + 1u] = acc[g][1]; }
    }
    __syncthreads();
    float *out = a.part_w + (size_t)row * G * AT_PART;
    for (uint32_t o = tid; o < G * AT_PART; o += 256u) {
        const uint32_t g = o / AT_PART, j = o % AT_PART;
        ((TQ_GLOBAL float *)out)[o] = j < 2u ? red[g][j] : part[0][g][j - 2u] + part[1][g][j - 2u] + part[2][g][j - 2u] + part[3][g][j - 2u];
    }
}

struct MergeArgs {
    const float *partial;    // [rows, splits, group, 130] from the packed history (rotated value space)
    const float *part_w;     // [rows, group, 130] from the window (plain space) or NULL
    const float *pi_v;       // [128, 128] rotation of the value codec
    void *out;               // [rows, group, 128] elements of out_dtype
    uint32_t group, splits;
    int out_dtype;
};

// One block per packed row: log-sum-exp merge of the splits, rotation of the value sums back (x = y @ Pi),
// the window's share, normalisation, cast.
__global__ __launch_bounds__(256) void tq_attend_merge_kernel(MergeArgs a) {
    constexpr int MAXG = 8;
    __shared__ float rot[MAXG][TQ_HEAD_DIM];
    __shared__ float den[MAXG], fw[MAXG];
    const uint32_t row = blockIdx.x, tid = threadIdx.x, G = a.group, S = a.splits;
    const TQ_GLOBAL float *part = (const TQ_GLOBAL float *)a.partial + (size_t)row * S * G * AT_PART;
    const TQ_GLOBAL float *pw = a.part_w ? (const TQ_GLOBAL float *)a.part_w + (size_t)row * G * AT_PART : nullptr;
    for (uint32_t o = tid; o < G * TQ_HEAD_DIM; o += 256u) {
        const uint32_t g = o / TQ_HEAD_DIM, j = o % TQ_HEAD_DIM;
        float m = pw ? pw[g * AT_PART] : -3.0e38f;
        for (uint32_t s = 0; s < S; ++s) m = fmaxf(m, part[(s * G + g) * AT_PART]);
        float acc = 0.f, l = 0.f;
        for (uint32_t s = 0; s < S; ++s) {
            const TQ_GLOBAL float *ps = part + (s * G + g) * AT_PART;
            const float f = __expf(ps[0] - m);
            acc = fmaf(f, ps[2 + j], acc);
            l = fmaf(f, ps[1], l);
        }
        rot[g][j] = acc;
        if (j == 0) {
            const float f = pw ? __expf(pw[g * AT_PART] - m) : 0.f;
            fw[g] = f;
            den[g] = l + (pw ? f * pw[g * AT_PART + 1] : 0.f);
        }
    }
    __syncthreads();
    for (uint32_t o = tid; o < G * TQ_HEAD_DIM; o += 256u) {
        const uint32_t g = o / TQ_HEAD_DIM, i = o % TQ_HEAD_DIM;
        float x = 0.f;
        for (int j = 0; j < TQ_HEAD_DIM; ++j) x = fmaf(rot[g][j], ((const TQ_GLOBAL float *)a.pi_v)[(size_t)j * TQ_HEAD_DIM + i], x);
        if (pw) x = fmaf(fw[g], pw[g * AT_PART + 2 + i], x);
        x /= den[g];
        const size_t idx = (size_t)row * G * TQ_HEAD_DIM + o;
        if (a.out_dtype == TQ_F32) {
            ((TQ_GLOBAL float *)a.out)[idx] = x;
        } else if (a.out_dtype == TQ_F16) {
            const _Float16 h = (_Float16)x;
            ((TQ_GLOBAL uint16_t *)a.out)[idx] = __builtin_bit_cast(uint16_t, h);
        } else {
            const __bf16 h = (__bf16)x;
            ((TQ_GLOBAL uint16_t *)a.out)[idx] = __builtin_bit_cast(uint16_t, h);
        }
    }
}

int device_cus(int &cus) {
    static int cache[64] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return TQ_ERR_NO_DEVICE;
    if (cache[dev] == 0) {
        int c = 0;
        e = hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return (int)e;
        cache[dev] = c > 0 ? c : 1;
    }
    cus = cache[dev];
    return 0;
}

int check_packed(const uint8_t *idx_bytes, const uint16_t *vec_norms, long long packed_row_stride, long long rows,
                 long long tokens, const void *table, int head_dim, int bits) {
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    if (head_dim != TQ_HEAD_DIM) return TQ_ERR_HEAD_DIM;
    if (rows < 0 || tokens < 0 || rows > 65535) return TQ_ERR_SIZE;
    if (rows == 0 || tokens == 0) return TQ_OK;
    if (!idx_bytes || !vec_norms || !table) return TQ_ERR_NULL;
    const long long prs = packed_row_stride ? packed_row_stride : tokens;
    if (prs < tokens || prs > (long long)0x7fffffff / rows) return TQ_ERR_SIZE;
    if (((uintptr_t)idx_bytes & 15u) || ((uintptr_t)vec_norms & 1u) || ((uintptr_t)table & 15u)) return TQ_ERR_ALIGN;
    return TQ_OK;
}

}  // namespace

extern "C" int tq_scores(const uint8_t *idx_bytes, const uint16_t *vec_norms, long long packed_row_stride,
                         long long rows, long long tokens, const void *table_dev, int head_dim, int bits,
                         const float *q_rot, int group, float *scores, long long scores_stride, void *stream) {
    int rc = check_packed(idx_bytes, vec_norms, packed_row_stride, rows, tokens, table_dev, head_dim, bits);
    if (rc) return rc;
    if (group < 1 || group > 32) return TQ_ERR_SIZE;
    if (rows == 0 || tokens == 0) return TQ_OK;
    if (!q_rot || !scores) return TQ_ERR_NULL;
    if (scores_stride < tokens) return TQ_ERR_SIZE;
    if (((uintptr_t)q_rot & 3u) || ((uintptr_t)scores & 3u)) return TQ_ERR_ALIGN;
    int cus = 0;
    rc = device_cus(cus);
    if (rc) return rc;
    ScoreArgs a;
    a.idx_bytes = idx_bytes;
    a.vec_norms = vec_norms;
    a.table = static_cast<const uint8_t *>(table_dev);
    a.q_rot = q_rot;
    a.scores = scores;
    a.stride = scores_stride;
    a.tokens = (uint32_t)tokens;
    a.packed_row_stride = (uint32_t)(packed_row_stride ? packed_row_stride : tokens);
    a.group = (uint32_t)group;
    const uint32_t tiles = (uint32_t)((tokens + 31) / 32);
    const uint32_t want = (tiles + SC_WAVES - 1) / SC_WAVES;
    uint32_t bx = (uint32_t)(((long long)cus * 8 + rows - 1) / rows);   // ~8 four-wave blocks per compute unit
    if (bx > want) bx = want;
    if (bx < 1) bx = 1;
    dim3 grid(bx, (unsigned)rows, 1), block(SC_WAVES * TQ_WAVE, 1, 1);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (8 / bits) {
        case 8: hipLaunchKernelGGL(tq_scores_kernel<8>, grid, block, 0, s, a); break;
        case 4: hipLaunchKernelGGL(tq_scores_kernel<4>, grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL(tq_scores_kernel<2>, grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL(tq_scores_kernel<1>, grid, block, 0, s, a); break;
    }
    return (int)hipGetLastError();
}

extern "C" int tq_weighted_values_splits(long long rows, long long tokens) {
    if (rows <= 0 || tokens <= 0) return 1;
    int cus = 0;
    if (device_cus(cus)) cus = 256;
    long long splits = ((long long)cus * 8 + rows - 1) / rows;       // ~8 four-wave blocks per compute unit
    const long long most = (tokens + 128 * WV_WAVES - 1) / (128 * WV_WAVES);
    if (splits > most) splits = most;
    if (splits > 4096) splits = 4096;
    return splits < 1 ? 1 : (int)splits;
}

extern "C" int tq_weighted_values(const uint8_t *idx_bytes, const uint16_t *vec_norms, long long packed_row_stride,
                                  long long rows, long long tokens, const void *table_dev, int head_dim, int bits,
                                  const float *weights, long long weights_stride, int group,
                                  float *partial, int splits, float *out_rot, void *stream) {
    int rc = check_packed(idx_bytes, vec_norms, packed_row_stride, rows, tokens, table_dev, head_dim, bits);
    if (rc) return rc;
    if (group < 1 || group > WV_MAX_GROUP || splits < 1 || splits > 65535) return TQ_ERR_SIZE;
    if (rows == 0) return TQ_OK;
    if (!out_rot) return TQ_ERR_NULL;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t per_row = (uint32_t)group * TQ_HEAD_DIM;
    const uint32_t total = (uint32_t)rows * per_row;
    if (tokens == 0) {   // empty sum
        hipLaunchKernelGGL(tq_reduce_splits_kernel, dim3((total + 255) / 256), dim3(256), 0, s, out_rot, out_rot, per_row, 0u, total);
        return (int)hipGetLastError();
    }
    if (!weights || !partial) return TQ_ERR_NULL;
    if (weights_stride < tokens) return TQ_ERR_SIZE;
    if (((uintptr_t)weights & 3u) || ((uintptr_t)partial & 3u) || ((uintptr_t)out_rot & 3u)) return TQ_ERR_ALIGN;
    WvArgs a;
    a.idx_bytes = idx_bytes;
    a.vec_norms = vec_norms;
    a.table = static_cast<const uint8_t *>(table_dev);
    a.weights = weights;
    a.partial = partial;
    a.stride = weights_stride;
    a.tokens = (uint32_t)tokens;
    a.packed_row_stride = (uint32_t)(packed_row_stride ? packed_row_stride : tokens);
    a.group = (uint32_t)group;
    const long long per_split = (tokens + splits - 1) / splits;
    a.chunk = (uint32_t)((per_split + 127) / 128 * 128);
    dim3 grid((unsigned)splits, (unsigned)rows, 1), block(WV_WAVES * TQ_WAVE, 1, 1);
    switch (8 / bits) {
        case 8: hipLaunchKernelGGL(tq_weighted_values_kernel<8>, grid, block, 0, s, a); break;
        case 4: hipLaunchKernelGGL(tq_weighted_values_kernel<4>, grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL(tq_weighted_values_kernel<2>, grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL(tq_weighted_values_kernel<1>, grid, block, 0, s, a); break;
    }
    rc = (int)hipGetLastError();
    if (rc) return rc;
    hipLaunchKernelGGL(tq_reduce_splits_kernel, dim3((total + 255) / 256), dim3(256), 0, s, partial, out_rot, per_row, (uint32_t)splits, total);
    return (int)hipGetLastError();
}

namespace {
template <int IPBK>
int launch_attend(int ipbv, dim3 grid, dim3 block, hipStream_t s, const AttendArgs &a) {
    switch (ipbv) {
        case 8: hipLaunchKernelGGL((tq_attend_kernel<IPBK, 8>), grid, block, 0, s, a); break;
        case 4: hipLaunchKernelGGL((tq_attend_kernel<IPBK, 4>), grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL((tq_attend_kernel<IPBK, 2>), grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL((tq_attend_kernel<IPBK, 1>), grid, block, 0, s, a); break;
    }
    return (int)hipGetLastError();
}
}  // namespace

extern "C" int tq_attend_splits(long long rows, long long tokens) {
    if (rows <= 0 || tokens <= 0) return 1;
    int cus = 0;
    if (device_cus(cus)) cus = 256;
    long long splits = ((long long)cus * 4 + rows - 1) / rows;       // two resident four-wave blocks per compute unit, twice over
    const long long most = (tokens + AT_RUN * AT_WAVES - 1) / (AT_RUN * AT_WAVES);
    if (splits > most) splits = most;
    if (splits > 4096) splits = 4096;
    return splits < 1 ? 1 : (int)splits;
}

extern "C" int tq_attend_partials(const uint8_t *k_idx, const uint16_t *k_norms, const uint8_t *v_idx, const uint16_t *v_norms,
                                  long long packed_row_stride, long long rows, long long tokens,
                                  const void *table_k, const void *table_v, int head_dim, int bits_k, int bits_v,
                                  const float *q_rot, int group, int splits, float *partial, void *stream) {
    int rc = check_packed(k_idx, k_norms, packed_row_stride, rows, tokens, table_k, head_dim, bits_k);
    if (rc) return rc;
    rc = check_packed(v_idx, v_norms, packed_row_stride, rows, tokens, table_v, head_dim, bits_v);
    if (rc) return rc;
    if (group < 1 || group > 8 || splits < 1 || splits > 65535) return TQ_ERR_SIZE;
    if (rows == 0 || tokens == 0) return TQ_ERR_SIZE;          // nothing to attend to: the caller handles it
    if (!q_rot || !partial) return TQ_ERR_NULL;
    if (((uintptr_t)q_rot & 3u) || ((uintptr_t)partial & 3u)) return TQ_ERR_ALIGN;
    AttendArgs a;
    a.k_idx = k_idx; a.v_idx = v_idx; a.k_norms = k_norms; a.v_norms = v_norms;
    a.table_k = static_cast<const uint8_t *>(table_k);
    a.table_v = static_cast<const uint8_t *>(table_v);
    a.q_rot = q_rot;
    a.partial = partial;
    a.tokens = (uint32_t)tokens;
    a.packed_row_stride = (uint32_t)(packed_row_stride ? packed_row_stride : tokens);
    a.group = (uint32_t)group;
    const long long per_split = (tokens + splits - 1) / splits;
    a.chunk = (uint32_t)((per_split + AT_RUN - 1) / AT_RUN * AT_RUN);
    dim3 grid((unsigned)splits, (unsigned)rows, 1), block(AT_WAVES * TQ_WAVE, 1, 1);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (8 / bits_k) {
        case 8: return launch_attend<8>(8 / bits_v, grid, block, s, a);
        case 4: return launch_attend<4>(8 / bits_v, grid, block, s, a);
        case 2: return launch_attend<2>(8 / bits_v, grid, block, s, a);
        default: return launch_attend<1>(8 / bits_v, grid, block, s, a);
    }
}

extern "C" int tq_attend_prepare(const void *queries, int q_dtype, long long rows, int group, float scale,
                                 const float *pi_k_t, const void *k_win, const void *v_win, int win_dtype,
                                 long long n_win, long long win_stride, float *q_rot, float *part_w, void *stream) {
    if (rows < 0 || rows > 0x7fffffff || group < 1 || group > 8 || n_win < 0 || n_win > 512) return TQ_ERR_SIZE;
    if ((q_dtype != TQ_F32 && q_dtype != TQ_F16 && q_dtype != TQ_BF16) ||
        (n_win && win_dtype != TQ_F32 && win_dtype != TQ_F16 && win_dtype != TQ_BF16)) return TQ_ERR_DTYPE;
    if (rows == 0) return TQ_OK;
    if (!queries || !pi_k_t || !q_rot) return TQ_ERR_NULL;
    if (n_win && (!k_win || !v_win || !part_w)) return TQ_ERR_NULL;
    if (n_win && win_stride < n_win * TQ_HEAD_DIM) return TQ_ERR_SIZE;
    // window tokens are read with 16-byte loads
    if (n_win && (((uintptr_t)k_win & 15u) || ((uintptr_t)v_win & 15u) || (win_stride & 7))) return TQ_ERR_ALIGN;
    PrepareArgs a;
    a.queries = queries; a.pi_k_t = pi_k_t; a.k_win = k_win; a.v_win = v_win;
    a.q_rot = q_rot; a.part_w = n_win ? part_w : nullptr;
    a.win_stride = win_stride; a.scale = scale;
    a.group = (uint32_t)group; a.n_win = (uint32_t)n_win;
    a.q_dtype = q_dtype; a.win_dtype = win_dtype;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    if (n_win && win_dtype == TQ_F32) hipLaunchKernelGGL(tq_attend_prepare_kernel<TQ_F32>, dim3((unsigned)rows), dim3(256), 0, st, a);
    else if (n_win && win_dtype == TQ_F16) hipLaunchKernelGGL(tq_attend_prepare_kernel<TQ_F16>, dim3((unsigned)rows), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(tq_attend_prepare_kernel<TQ_BF16>, dim3((unsigned)rows), dim3(256), 0, st, a);
    return (int)hipGetLastError();
}

extern "C" int tq_attend_merge(const float *partial, int splits, const float *part_w, const float *pi_v,
                               long long rows, int group, void *out, int out_dtype, void *stream) {
    if (rows < 0 || rows > 0x7fffffff || group < 1 || group > 8 || splits < 0) return TQ_ERR_SIZE;
    if (out_dtype != TQ_F32 && out_dtype != TQ_F16 && out_dtype != TQ_BF16) return TQ_ERR_DTYPE;
    if (rows == 0) return TQ_OK;
    if (!pi_v || !out || (splits && !partial) || (!splits && !part_w)) return TQ_ERR_NULL;
    MergeArgs a;
    a.partial = partial; a.part_w = part_w; a.pi_v = pi_v; a.out = out;
    a.group = (uint32_t)group; a.splits = (uint32_t)splits; a.out_dtype = out_dtype;
    hipLaunchKernelGGL(tq_attend_merge_kernel, dim3((unsigned)rows), dim3(256), 0, static_cast<hipStream_t>(stream), a);
    return (int)hipGetLastError();
}
