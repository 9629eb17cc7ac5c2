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
#include <atomic>

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

// ---- both terms of the V2 key estimate in one pass (upstream turboquant/compressors.py:124-158) ----------------------
//   score[row][q][t] = norm_t * (Pi q) . centroids[codes_t]  +  residual_norm_t * (c S q) . signs_t ,  c = sqrt(pi/2) / 128
// The first term is tq_scores_kernel's; the second reads the 16 sign bytes of a token as 1-bit codes over (-1, +1)
// (byte -> eight fp16 values from a table built here) against one fp16 term of the projected query (the term is a
// correction of the size of the quantisation residual: 2^-12 of it disappears under the tolerance of the first).
// Query tokens beyond 32 per row go to further blocks (blockIdx.z): one launch for any number of them.
struct QjlScoreArgs {
    const uint8_t *idx_bytes;
    const uint16_t *vec_norms;
    const uint8_t *sign_bytes;
    const uint16_t *residual_norm;
    const uint8_t *table;
    const float *q_rot;      // [rows, n_q, 128]
    const float *q_sign;     // [rows, n_q, 128]
    float *scores;           // [rows, n_q, tokens]
    uint32_t tokens, n_q;
};

template <int IPB>
__global__ __launch_bounds__(SC_WAVES *TQ_WAVE) void tq_qjl_scores_kernel(QjlScoreArgs a) {
    constexpr int NB = 64 / IPB;   // packed bytes per lane (half a vector)
    constexpr int NW = NB / 4;
    __shared__ __attribute__((aligned(16))) uint8_t lds_lut[4096];
    __shared__ __attribute__((aligned(16))) uint8_t lds_sign[4096];
    __shared__ float lds_rowscale[2][32];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t row = blockIdx.y, q0 = blockIdx.z * 32u;
    const uint32_t group = a.n_q - q0 < 32u ? a.n_q - q0 : 32u;      // query tokens of this block
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(a.table);
    tq_copy_to_lds(lds_lut, a.table + hd->off_lut, 256u * 2u * IPB, tid, SC_WAVES * TQ_WAVE);
    for (uint32_t v = tid; v < 256u; v += SC_WAVES * TQ_WAVE) {     // bit 7 - k of a sign byte belongs to coordinate k
        tq_half8 e;
#pragma unroll
        for (int k = 0; k < 8; ++k) e[k] = ((v >> (7 - k)) & 1u) ? (_Float16)1.0f : (_Float16)-1.0f;
        *reinterpret_cast<tq_u4 *>(lds_sign + 16u * v) = __builtin_bit_cast(tq_u4, e);
    }

    // ---- A operands: query n of this block, contraction slice (step s, half hk) = coordinates 64*hk + 8*s + i
    tq_u4 ahi[TQ_STEPS], alo[TQ_STEPS], shi[TQ_STEPS];
    {
        const bool live = n < group;
        const size_t qoff = ((size_t)row * a.n_q + q0 + (live ? n : 0u)) * TQ_HEAD_DIM + 64u * hk;
        auto exponent_of = [&](const TQ_GLOBAL float *q) {
            float big = 0.f;
            for (int i = 0; i < 64; ++i) big = fmaxf(big, fabsf(q[i]));
            big = fmaxf(big, __shfl_xor(big, 32));
            int e = 0;
            if (big > 0.f && big < __builtin_inff()) (void)frexpf(big, &e);
            return e < -100 ? -100 : e;   // rows that small give zero scores either way; keeps 2^(10-e) finite
        };
        const TQ_GLOBAL float *q = (const TQ_GLOBAL float *)a.q_rot + qoff;
        const TQ_GLOBAL float *qs = (const TQ_GLOBAL float *)a.q_sign + qoff;
        const int e1 = exponent_of(q), e2 = exponent_of(qs);
        const float up1 = ldexpf(1.f, TQ_F16_PI_SHIFT - e1), up2 = ldexpf(1.f, TQ_F16_PI_SHIFT - e2);
        if (hk == 0u) {
            lds_rowscale[0][n] = live ? ldexpf(1.f, e1 - TQ_F16_PI_SHIFT) : 0.f;
            lds_rowscale[1][n] = live ? ldexpf(1.f, e2 - TQ_F16_PI_SHIFT) : 0.f;
        }
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            tq_half8 h, l, g;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float x = live ? q[8 * s + i] * up1 : 0.f;
                const _Float16 xh = (_Float16)x;
                h[i] = xh;
                l[i] = (_Float16)(x - (float)xh);
                g[i] = (_Float16)(live ? qs[8 * s + i] * up2 : 0.f);
            }
            ahi[s] = __builtin_bit_cast(tq_u4, h);
            alo[s] = __builtin_bit_cast(tq_u4, l);
            shi[s] = __builtin_bit_cast(tq_u4, g);
        }
    }
    __syncthreads();
    // accumulator register r of lane (n, h = hk) belongs to query 8*(r/4) + 4*h + r%4
    float scale1[16], scale2[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        scale1[r] = lds_rowscale[0][8 * (r / 4) + 4 * hk + (r % 4)];
        scale2[r] = lds_rowscale[1][8 * (r / 4) + 4 * hk + (r % 4)];
    }

    const uint32_t n_tiles = (a.tokens + 31u) / 32u;
    const uint32_t tile_stride = gridDim.x * SC_WAVES;
    uint32_t tile = blockIdx.x * SC_WAVES + wave;
    const size_t slot0 = (size_t)row * a.tokens;

    uint32_t raw[NW], sraw[2];
    uint16_t norm_bits = 0, rnorm_bits = 0;
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
        tq_u2 sv = {0u, 0u};
        if (ok) sv = tq_gload8(a.sign_bytes + slot * 16u + hk * 8u);
        sraw[0] = sv[0]; sraw[1] = sv[1];
        norm_bits = ok ? tq_gload2(a.vec_norms + slot) : (uint16_t)0;
        rnorm_bits = ok ? tq_gload2(a.residual_norm + slot) : (uint16_t)0;
    };
    if (tile < n_tiles) issue_loads(tile);
    while (tile < n_tiles) {
        uint32_t cur[NW], scur[2];
#pragma unroll
        for (int i = 0; i < NW; ++i) cur[i] = raw[i];
        scur[0] = sraw[0]; scur[1] = sraw[1];
        const float nrm = (float)__builtin_bit_cast(_Float16, norm_bits);
        const float rnrm = (float)__builtin_bit_cast(_Float16, rnorm_bits);
        const uint32_t next = tile + tile_stride;
        if (next < n_tiles) issue_loads(next);

        tq_f16v acc = tq_zero16(), sacc = tq_zero16();
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            const tq_u4 b = decode_step<IPB, NW>(cur, s, lds_lut);
            const tq_u4 sb = decode_step<8, 2>(scur, s, lds_sign);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(tq_half8, ahi[s]), __builtin_bit_cast(tq_half8, b), acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(tq_half8, alo[s]), __builtin_bit_cast(tq_half8, b), acc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(tq_half8, shi[s]), __builtin_bit_cast(tq_half8, sb), sacc, 0, 0, 0);
        }
        const uint32_t t = tile * 32u + n;
        if (t < a.tokens) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t m = 8u * (r / 4) + 4u * hk + (r % 4);
                if (m < group)
                    ((TQ_GLOBAL float *)a.scores)[((size_t)row * a.n_q + q0 + m) * a.tokens + t] =
                        fmaf(sacc[r] * scale2[r], rnrm, acc[r] * scale1[r] * nrm);
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
    float *partial;          // [rows, splits, group, 130]: reference score m, sum of exp(score - m), 128 weighted sums
    uint32_t tokens, packed_row_stride, group, chunk;
};
constexpr int AT_RUN = 64;       // tokens per wave and trip (32 when keys or values use 8-bit codes)
constexpr int AT_PART = TQ_HEAD_DIM + 2;

// Block (split, row) of eight waves; a wave takes runs of 64 tokens of the split (staged one run ahead), a tile is 32
// tokens = two blocks of 16, all matrix work is v_mfma_f32_16x16x32_f16 with the row's query heads (at most 16) padded
// to 16 columns.  Lane (n16, q4) = (lane % 16, lane / 16).
//   scores  S^T[token][head]: A = decoded keys, lane (token n16 of the block, q4) holds the 32 coordinates
//     32 q4 .. 32 q4 + 31 of its token (KB contiguous packed bytes) and feeds 8 of them to each of 4 steps; B = rotated
//     queries in the same coordinate order (lane (head n16, q4), step s: coordinates 32 q4 + 8 s + j), one fp16 term;
//     result register r of lane (head n16, q4) = token 4 q4 + r of the block: a head's statistics live in four lanes;
//   softmax in base 2 against a per-head reference that follows the running maximum lazily (see m_ref below), so the
//     common tile needs no exchange between lanes;
//   P * V_dec: A = probabilities times value norms, lane (head n16, q4) slice j: token 4 q4 + j of block 0 (j < 4) or
//     block 1, which are the registers the lane already holds; B = decoded values for the same eight tokens, lane
//     (n16, q4) owns coordinates 8 n16 .. 8 n16 + 7 (8 / IPBV packed bytes per token, one decode), column block c =
//     coordinate 8 n16 + c; token pairs regrouped with v_perm;
//     accumulator register r of block c in lane (n16, q4) = head 4 q4 + r, coordinate 8 n16 + c.
// The waves' (m, l, sums) are merged in LDS; splits and the uncompressed window are merged by the caller.
typedef float tq_f4v __attribute__((ext_vector_type(4)));
constexpr int AT_WAVES = 8;      // one block per compute unit (two waves per SIMD): the table copies below are shared by its waves

template <int IPBK, int IPBV>
__global__ __launch_bounds__(AT_WAVES *TQ_WAVE, AT_WAVES / 4) void tq_attend_kernel(AttendArgs a) {
    constexpr int KB = TQ_HEAD_DIM / IPBK / 4;           // key bytes per lane and token (32 coordinates): 4, 8, 16, 32
    constexpr int NWK = KB / 4;
    constexpr int GBV = TQ_HEAD_DIM / IPBV;              // value bytes per vector
    constexpr int VB = 8 / IPBV;                         // value bytes per lane and token (8 coordinates): 1, 2, 4, 8
    constexpr int NWV = VB > 4 ? 2 : 1;
    constexpr int RUN = (IPBK == 1 || IPBV == 1) ? 32 : AT_RUN;   // tokens per wave and trip (8-bit codes: half, for registers)
    constexpr int SUB = RUN / 32;
    constexpr int VBYTES = RUN * GBV;                 // <= 8192
    constexpr int VPIECES = VBYTES / 16, NVP = (VPIECES + 63) / 64;
    constexpr int SLACK_LOG2 = 8;
    constexpr int P_SHIFT = 14 - SLACK_LOG2;             // p * 2^P_SHIFT * (value norm / 2^ev_ref < 2) <= 2^15 fits fp16
    constexpr int AREA = VBYTES > 16 * AT_PART * 4 ? VBYTES : 16 * AT_PART * 4;  // staged value codes, later the wave's result (16 heads)
    __shared__ __attribute__((aligned(16))) uint8_t lds_lut_k[32768];
    __shared__ __attribute__((aligned(16))) uint8_t lds_lut_v[32768];
    __shared__ __attribute__((aligned(16))) uint8_t lds_area[AT_WAVES][AREA];
    __shared__ __attribute__((aligned(16))) float lds_kn[AT_WAVES][RUN];        // key norms as fp32
    __shared__ __attribute__((aligned(16))) uint16_t lds_vn[AT_WAVES][RUN];     // value norms / 2^ev_ref as fp16
    __shared__ __attribute__((aligned(16))) float lds_corr[AT_WAVES][16];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t row = blockIdx.y, split = blockIdx.x;
    const uint32_t n16 = lane & 15u, q4 = lane >> 4;
    const TqTableHeader *hk_hd = reinterpret_cast<const TqTableHeader *>(a.table_k);
    const TqTableHeader *hv_hd = reinterpret_cast<const TqTableHeader *>(a.table_v);
    RepLut<IPBK>::stage(lds_lut_k, a.table_k + hk_hd->off_lut, tid, AT_WAVES * TQ_WAVE);
    RepLut<IPBV>::stage(lds_lut_v, a.table_v + hv_hd->off_lut, tid, AT_WAVES * TQ_WAVE);
    const uint8_t *lut_k = lds_lut_k + RepLut<IPBK>::lane_offset(lane);
    const uint8_t *lut_v = lds_lut_v + RepLut<IPBV>::lane_offset(lane);

    const uint32_t G = a.group;
    const bool live = n16 < G;
    // ---- B operand of the score product: fp16 of q * 2^(10 - e), e = binary exponent of the head's largest magnitude.
    //      One fp16 term for keys of up to 4 bits (its 2^-12 rounding per coordinate disappears under their
    //      quantisation error); hi + lo for wider keys, where that launch is bound by memory and the term costs 1 %.
    constexpr bool QLO = IPBK == 1;      // keys of 5 to 8 bits: a second term, the score then carries the keys' precision
    tq_u4 qb[4];
    tq_u4 ql[QLO ? 4 : 1];
    float c1;                // score in base-2 units = t * c1, t = accumulator * key norm
    float rowscale;          // natural score = t * rowscale
    {
        const TQ_GLOBAL float *q = (const TQ_GLOBAL float *)a.q_rot + ((size_t)row * G + (live ? n16 : 0u)) * TQ_HEAD_DIM + 32u * q4;
        float big = 0.f;
        for (int i = 0; i < 32; ++i) big = fmaxf(big, fabsf(q[i]));
        big = fmaxf(big, __shfl_xor(big, 16));
        big = fmaxf(big, __shfl_xor(big, 32));
        int e = 0;
        if (big > 0.f && big < __builtin_inff()) (void)frexpf(big, &e);
        e = e < -100 ? -100 : e;
        const float up = ldexpf(1.f, TQ_F16_PI_SHIFT - e);
        rowscale = live ? ldexpf(1.f, e - TQ_F16_PI_SHIFT) : 0.f;
        c1 = rowscale * 1.44269504088896341f;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            tq_half8 h, l;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float x = live ? q[8 * s + i] * up : 0.f;
                h[i] = (_Float16)x;
                l[i] = (_Float16)(x - (float)h[i]);
            }
            qb[s] = __builtin_bit_cast(tq_u4, h);
            if constexpr (QLO) ql[s] = __builtin_bit_cast(tq_u4, l);
        }
    }
    __syncthreads();

    const uint32_t t_begin = split * a.chunk;
    const uint32_t t_end = min(a.tokens, t_begin + a.chunk);
    const size_t slot0 = (size_t)row * a.packed_row_stride;
    uint8_t *vcodes = lds_area[wave];

    tq_f4v acc[8];           // weighted value sums: register r = query head 4 q4 + r, block c = coordinate 8 n16 + c
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = tq_f4v{0.f, 0.f, 0.f, 0.f};
    // Softmax reference of this lane's head, in units of t (the four lanes of a head agree).  It is not the exact
    // running maximum: it moves only when a score exceeds it by more than SLACK_LOG2 binary orders, so the common
    // tile needs no exchange between lanes; probabilities relative to it reach 2^SLACK_LOG2 at most.
    float m_ref = -1e30f;
    float l_run = 0.f;       // running sum of p * 2^P_SHIFT over this lane's tokens
    const float slack = live ? (float)SLACK_LOG2 / c1 : 3.0e38f;
    // Value norms are folded into the probabilities (A operand), relative to 2^ev_ref, ev_ref = the largest binary
    // exponent of a value norm seen by this wave so far (uniform over the wave); the sums are in units of 2^ev_ref.
    int ev_ref = -100;

    // loads of a run, issued one run ahead into the other of two register sets
    uint32_t kraw_buf[2][SUB][2][NWK];
    tq_u4 vpiece_buf[2][NVP];
    uint16_t kn_buf[2] = {0, 0}, vn_buf[2] = {0, 0};
    // FULL: the run has all its tokens, so no address is clamped and the arithmetic folds into constants
    auto issue_loads = [&](auto bsel, auto full_tag, uint32_t t0) __attribute__((always_inline)) {
        constexpr int B = decltype(bsel)::value;
        constexpr bool FULL = decltype(full_tag)::value;
        auto &kraw_next = kraw_buf[B];
        auto &vpiece_next = vpiece_buf[B];
        uint16_t &kn_next = kn_buf[B], &vn_next = vn_buf[B];
        const uint32_t n_tok = FULL ? (uint32_t)RUN : min((uint32_t)RUN, t_end - t0);
#pragma unroll
        for (int u = 0; u < SUB; ++u)
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const uint32_t tl = 32u * u + 16u * b + n16;
                const uint8_t *src = a.k_idx + (slot0 + t0 + ((FULL || tl < n_tok) ? tl : 0u)) * (4 * KB) + q4 * KB;
                if constexpr (KB == 4) {
                    kraw_next[u][b][0] = *reinterpret_cast<const TQ_GLOBAL uint32_t *>((const TQ_GLOBAL uint8_t *)src);
                } else if constexpr (KB == 8) {
                    const tq_u2 v = tq_gload8(src);
                    kraw_next[u][b][0] = v[0]; kraw_next[u][b][1] = v[1];
                } else {
#pragma unroll
                    for (int p = 0; p < KB / 16; ++p) {
                        const tq_u4 v = tq_gload16(src + 16 * p);
#pragma unroll
                        for (int i = 0; i < 4; ++i) kraw_next[u][b][4 * p + i] = v[i];
                    }
                }
            }
        const uint8_t *vsrc = a.v_idx + (slot0 + t0) * GBV;
#pragma unroll
        for (int p = 0; p < NVP; ++p) {
            const uint32_t piece = p * 64u + lane;
            const bool ok = piece < VPIECES && (FULL || piece * 16u < n_tok * GBV);
            vpiece_next[p] = tq_gload16(vsrc + (ok ? piece : 0u) * 16u);
        }
        kn_next = lane < n_tok ? tq_gload2(a.k_norms + slot0 + t0 + lane) : (uint16_t)0;
        vn_next = lane < n_tok ? tq_gload2(a.v_norms + slot0 + t0 + lane) : (uint16_t)0;   // tokens past the end weigh nothing
    };

    // one run of up to 64 staged tokens; FULL: all 64 exist (no per-token masks in the code).
    // The score products of both tiles are issued first, so that the second tile's matrix work runs under the
    // first tile's softmax arithmetic.
    auto run = [&](auto full_tag, const uint32_t (&kraw)[SUB][2][NWK], uint32_t n_tok) __attribute__((always_inline)) {
        constexpr bool FULL = decltype(full_tag)::value;
        tq_f4v sc[SUB][2];   // register r of block b = token 32 u + 16 b + 4 q4 + r
#pragma unroll
        for (int u = 0; u < SUB; ++u) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                sc[u][b] = tq_f4v{0.f, 0.f, 0.f, 0.f};
                if (!FULL && 32u * u >= n_tok) continue;   // uniform
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const tq_half8 kd = __builtin_bit_cast(tq_half8, decode_rep<IPBK, NWK>(kraw[u][b], s, lut_k));
                    sc[u][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kd, __builtin_bit_cast(tq_half8, qb[s]), sc[u][b], 0, 0, 0);
                    if constexpr (QLO)
                        sc[u][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kd, __builtin_bit_cast(tq_half8, ql[s]), sc[u][b], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < SUB; ++u) {
            if (!FULL && 32u * u >= n_tok) break;  // uniform
            float t[8];
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const float4 k4 = *reinterpret_cast<const float4 *>(&lds_kn[wave][32u * u + 16u * b + 4u * q4]);
                t[4 * b + 0] = sc[u][b][0] * k4.x; t[4 * b + 1] = sc[u][b][1] * k4.y;
                t[4 * b + 2] = sc[u][b][2] * k4.z; t[4 * b + 3] = sc[u][b][3] * k4.w;
            }
            if constexpr (!FULL) {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (32u * u + 16u * (j / 4) + 4u * q4 + (j % 4) >= n_tok) t[j] = -1e30f;
            }
            const float tmax = fmaxf(fmaxf(fmaxf(t[0], t[1]), fmaxf(t[2], t[3])), fmaxf(fmaxf(t[4], t[5]), fmaxf(t[6], t[7])));
            // ---- a score left the range the reference covers (rare after the first tiles): move the head's
            //      reference to the largest score seen and rescale its sums
            if (__any(tmax > m_ref + slack)) {
                float tm = fmaxf(tmax, __shfl_xor(tmax, 16));
                tm = fmaxf(tm, __shfl_xor(tm, 32));
                const float m_new = fmaxf(m_ref, tm);
                const float corr = __builtin_amdgcn_exp2f((m_ref - m_new) * c1);
                l_run *= corr;
                m_ref = m_new;
                if (q4 == 0u) lds_corr[wave][n16] = corr;
                asm volatile("" ::: "memory");
                __builtin_amdgcn_wave_barrier();
                const float4 c4 = *reinterpret_cast<const float4 *>(&lds_corr[wave][4u * q4]);
                asm volatile("" ::: "memory");
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    acc[c][0] *= c4.x; acc[c][1] *= c4.y; acc[c][2] *= c4.z; acc[c][3] *= c4.w;
                }
            }
            const float bias = P_SHIFT - m_ref * c1;
            float ps[8];
            float lsum = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                ps[j] = __builtin_amdgcn_exp2f(fmaf(t[j], c1, bias));     // p * 2^P_SHIFT, p <= 2^SLACK_LOG2
                if constexpr (!FULL) {   // a zero query makes every exponent 0: masked tokens need an explicit zero
                    if (32u * u + 16u * (j / 4) + 4u * q4 + (j % 4) >= n_tok) ps[j] = 0.f;
                }
                lsum += ps[j];
            }
            l_run += lsum;
            // ---- P * V: contraction slice j of lane (., q4) = token 32 u + 4 q4 + j (j < 4), 32 u + 16 + 4 q4 + j - 4
            tq_half8 pa;
#pragma unroll
            for (int j = 0; j < 8; ++j) pa[j] = (_Float16)ps[j];
            const uint32_t tok_a = 32u * u + 4u * q4, tok_b = tok_a + 16u;
            const tq_u2 vn_a = *reinterpret_cast<const tq_u2 *>(&lds_vn[wave][tok_a]);
            const tq_u2 vn_b = *reinterpret_cast<const tq_u2 *>(&lds_vn[wave][tok_b]);
            const tq_u4 nrm = {vn_a[0], vn_a[1], vn_b[0], vn_b[1]};
            pa = pa * __builtin_bit_cast(tq_half8, nrm);          // weight of token j = p_j * |v_j| / 2^ev_ref
            tq_u4 dec[8];        // per token: the lane's eight coordinates as fp16
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint8_t *src = vcodes + ((j < 4 ? tok_a : tok_b) + (uint32_t)(j % 4)) * GBV + n16 * VB;
                uint32_t raw[NWV];
                if constexpr (VB == 1) raw[0] = *src;
                else if constexpr (VB == 2) raw[0] = *reinterpret_cast<const uint16_t *>(src);
                else if constexpr (VB == 4) raw[0] = *reinterpret_cast<const uint32_t *>(src);
                else { const tq_u2 v = *reinterpret_cast<const tq_u2 *>(src); raw[0] = v[0]; raw[1] = v[1]; }
                dec[j] = decode_rep<IPBV, NWV>(raw, 0, lut_v);
            }
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                tq_u4 bt;
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    bt[d] = __builtin_amdgcn_perm(dec[2 * d + 1][c / 2], dec[2 * d][c / 2], (c & 1) ? 0x07060302u : 0x05040100u);
                acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, __builtin_bit_cast(tq_half8, bt), acc[c], 0, 0, 0);
            }
        }
    };

    // one trip: stage the run held in register set B, start the loads of the next run into the other set, compute
    auto trip = [&](auto bsel, uint32_t t0) __attribute__((always_inline)) {
        constexpr int B = decltype(bsel)::value;
        const uint32_t n_tok = min((uint32_t)RUN, t_end - t0);
#pragma unroll
        for (int p = 0; p < NVP; ++p) {
            const uint32_t piece = p * 64u + lane;
            if (piece < VPIECES) *reinterpret_cast<tq_u4 *>(vcodes + piece * 16u) = vpiece_buf[B][p];
        }
        {
            const _Float16 kh = __builtin_bit_cast(_Float16, kn_buf[B]);
            if (RUN == 64 || lane < (uint32_t)RUN) lds_kn[wave][lane] = (float)kh;     // one token per lane
            // does a value norm of this run exceed the reference exponent?  (a vote; a handful of times per wave)
            uint32_t e = ((uint32_t)vn_buf[B] >> 10) & 31u;
            if (__any((int)max(e, 1u) - 15 > ev_ref)) {
                // largest exponent field of the run: row-wise running maximum, then the four row ends
                e = max(e, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)e, 0x111, 0xf, 0xf, true));
                e = max(e, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)e, 0x112, 0xf, 0xf, true));
                e = max(e, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)e, 0x114, 0xf, 0xf, true));
                e = max(e, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)e, 0x118, 0xf, 0xf, true));
                const uint32_t emax = max(max((uint32_t)__builtin_amdgcn_readlane((int)e, 15), (uint32_t)__builtin_amdgcn_readlane((int)e, 31)),
                                          max((uint32_t)__builtin_amdgcn_readlane((int)e, 47), (uint32_t)__builtin_amdgcn_readlane((int)e, 63)));
                const int ev = (int)max(emax, 1u) - 15;
                const float f = ldexpf(1.f, ev_ref - ev);
#pragma unroll
                for (int c = 0; c < 8; ++c) acc[c] *= f;
                ev_ref = ev;
            }
            const _Float16 vh = __builtin_bit_cast(_Float16, vn_buf[B]);
            const _Float16 vs = (_Float16)ldexpf((float)vh, -ev_ref);
            if (RUN == 64 || lane < (uint32_t)RUN) lds_vn[wave][lane] = __builtin_bit_cast(uint16_t, vs);
        }
        const uint32_t t_next = t0 + RUN * AT_WAVES;
        if (t_next + RUN <= t_end) issue_loads(std::integral_constant<int, 1 - B>{}, std::true_type{}, t_next);
        else if (t_next < t_end) issue_loads(std::integral_constant<int, 1 - B>{}, std::false_type{}, t_next);
        asm volatile("" ::: "memory");    // staged with one access width, read back with others (LDS serves a wave in order)
        __builtin_amdgcn_wave_barrier();
        if (n_tok == RUN) run(std::true_type{}, kraw_buf[B], n_tok);
        else run(std::false_type{}, kraw_buf[B], n_tok);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        return t_next;
    };
    {
        uint32_t t0 = t_begin + RUN * wave;
        if (t0 < t_end) {
            issue_loads(std::integral_constant<int, 0>{}, std::false_type{}, t0);
            for (;;) {
                t0 = trip(std::integral_constant<int, 0>{}, t0);
                if (t0 >= t_end) break;
                t0 = trip(std::integral_constant<int, 1>{}, t0);
                if (t0 >= t_end) break;
            }
        }
    }
    asm volatile("" ::: "memory");
    // ---- this wave's result for heads 0..15: [head][largest natural score, sum, 128 sums] in its LDS area
    float *res = reinterpret_cast<float *>(lds_area[wave]);
    {
        float l_all = l_run + __shfl_xor(l_run, 16);
        l_all = (l_all + __shfl_xor(l_all, 32)) * (1.0f / (float)(1 << P_SHIFT));
        if (q4 == 0u) {
            res[n16 * AT_PART + 0] = m_ref * rowscale;
            res[n16 * AT_PART + 1] = l_all;
        }
        const float out_scale = ldexpf(1.f, ev_ref - P_SHIFT);
        {
#pragma unroll
            for (int c = 0; c < 8; ++c)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    res[(4u * q4 + r) * AT_PART + 2 + 8u * n16 + c] = acc[c][r] * out_scale;
        }
    }
    __syncthreads();
    // ---- merge the waves
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

// Eight consecutive window elements (element index i a multiple of 8): the load and the conversion apart, so that
// loads can be issued long before their use.
template <int WD> struct Raw8 { tq_u4 v[WD == TQ_F32 ? 2 : 1]; };

template <int WD>
__device__ __forceinline__ Raw8<WD> tq_load8_raw(const void *base, size_t i) {
    Raw8<WD> r;
    if constexpr (WD == TQ_F32) {
        r.v[0] = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>((const TQ_GLOBAL float *)base + i);
        r.v[1] = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>((const TQ_GLOBAL float *)base + i + 4);
    } else {
        r.v[0] = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>((const TQ_GLOBAL uint16_t *)base + i);
    }
    return r;
}

template <int WD>
__device__ __forceinline__ void tq_cvt8(const Raw8<WD> &r, float (&x)[8]) {
    if constexpr (WD == TQ_F32) {
#pragma unroll
        for (int e = 0; e < 4; ++e) { x[e] = __uint_as_float(r.v[0][e]); x[4 + e] = __uint_as_float(r.v[1][e]); }
    } else if constexpr (WD == TQ_F16) {
        const tq_half8 h = __builtin_bit_cast(tq_half8, r.v[0]);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = (float)h[e];
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) { x[2 * e] = __uint_as_float(r.v[0][e] << 16); x[2 * e + 1] = __uint_as_float(r.v[0][e] & 0xffff0000u); }
    }
}

// Sum over the 16 lanes of a DPP row; the total lands in lane 15 of the row.
__device__ __forceinline__ float tq_row_sum16(float x) {
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x111, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x112, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x114, 0xf, 0xf, true));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x118, 0xf, 0xf, true));
    return x;
}

// One block per packed row (batch x kv head), four waves.  Rotates the row's query heads for the packed keys and
// computes attention statistics over the uncompressed window tokens in fp32 (a few hundred tokens at most).
// GP = heads per row rounded up to 1, 2, 4, 8 or 16: the padding heads are zero queries, so no loop tests the head count.
// The loads of the first 128 window tokens, keys and values, are issued before anything else: the kernel waits for
// memory once.
//   rotation   : thread (j, half) sums 64 of the 128 terms of every head's q_rot[j]; Pi^T is read once, coalesced
//   scores     : 16 lanes x 8 elements cover a key, a wave takes 16 tokens per trip of 64; per token and head a dot
//                product summed over the DPP row of its 16 lanes
//   statistics : wave w owns heads w and w + 4
//   value sums : 32 lanes x 4 columns cover a value, a wave takes 8 tokens per trip of 32; the two token slots of a
//                wave meet through one exchange, the four waves in LDS
template <int WD, int GP>
__global__ __launch_bounds__(256) void tq_attend_prepare_kernel(PrepareArgs a) {
    constexpr int MAXG = 16, MAXW = 512;
    constexpr int PRE_K = 2;      // key trips (64 tokens each) loaded up front
    constexpr int PRE_V = 4;      // value trips (32 tokens each) loaded up front
    constexpr int VW = WD == TQ_F32 ? 4 : 2;             // dwords per four value elements
    __shared__ __attribute__((aligned(16))) float qt[TQ_HEAD_DIM][MAXG];     // scaled queries, head index fastest
    __shared__ float sc[MAXG][MAXW];
    __shared__ float red[MAXG][2];
    __shared__ float part[4][MAXG][TQ_HEAD_DIM];
    const uint32_t row = blockIdx.x, tid = threadIdx.x, G = a.group, lane = tid & 63u, wave = tid >> 6;
    const uint32_t sub = lane & 15u, tk = lane >> 4;          // key side: elements 8 sub .., token slot tk of 4
    const uint32_t sub5 = lane & 31u, tk5 = lane >> 5;        // value side: columns 4 sub5 .., token slot tk5 of 2
    // grid.y = 2 when there is a window: blocks (row, 0) rotate the queries, blocks (row, 1) take the window, side by side
    const bool do_rot = blockIdx.y == 0u, do_win = gridDim.y == 1u || blockIdx.y == 1u;
    const uint32_t W = (a.part_w && do_win) ? a.n_win : 0u;
    const size_t win_base = (size_t)row * a.win_stride;
    // past the end the last token is read again and not used
    auto ktoken = [&](uint32_t trip, int k) { return 64u * trip + 16u * wave + 4u * (uint32_t)k + tk; };
    auto vtoken = [&](uint32_t trip, int k) { return 32u * trip + 8u * wave + 2u * (uint32_t)k + tk5; };
    auto vload = [&](uint32_t t, uint32_t (&r)[VW]) __attribute__((always_inline)) {
        const size_t at = win_base + (size_t)min(t, W - 1u) * TQ_HEAD_DIM + 4u * sub5;
        if constexpr (WD == TQ_F32) {
            const tq_u4 v = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>((const TQ_GLOBAL float *)a.v_win + at);
            r[0] = v[0]; r[1] = v[1]; r[2] = v[2]; r[3] = v[3];
        } else {
            const tq_u2 v = *reinterpret_cast<const TQ_GLOBAL tq_u2 *>((const TQ_GLOBAL uint16_t *)a.v_win + at);
            r[0] = v[0]; r[1] = v[1];
        }
    };
    auto vcvt = [&](const uint32_t (&r)[VW], float (&x)[4]) __attribute__((always_inline)) {
        if constexpr (WD == TQ_F32) {
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = __uint_as_float(r[e]);
        } else if constexpr (WD == TQ_F16) {
            typedef _Float16 half4 __attribute__((ext_vector_type(4)));
            const tq_u2 v = {r[0], r[1]};
            const half4 h = __builtin_bit_cast(half4, v);
#pragma unroll
            for (int e = 0; e < 4; ++e) x[e] = (float)h[e];
        } else {
            x[0] = __uint_as_float(r[0] << 16); x[1] = __uint_as_float(r[0] & 0xffff0000u);
            x[2] = __uint_as_float(r[1] << 16); x[3] = __uint_as_float(r[1] & 0xffff0000u);
        }
    };
    Raw8<WD> kpre[PRE_K][4];
    uint32_t vpre[PRE_V][4][VW];
    if (W) {
#pragma unroll
        for (int tr = 0; tr < PRE_K; ++tr)
#pragma unroll
            for (int k = 0; k < 4; ++k)
                kpre[tr][k] = tq_load8_raw<WD>(a.k_win, win_base + (size_t)min(ktoken(tr, k), W - 1u) * TQ_HEAD_DIM + 8u * sub);
#pragma unroll
        for (int tr = 0; tr < PRE_V; ++tr)
#pragma unroll
            for (int k = 0; k < 4; ++k) vload(vtoken(tr, k), vpre[tr][k]);
    }
    {   // the row's queries, scaled, into `qt` (zeros for the padding heads): the element type is looked at once and
        // the loads of a thread are issued together
        constexpr int QG = GP < 4 ? 4 : GP;                  // heads written (the rotation reads four at a time)
        constexpr int NQ = QG * TQ_HEAD_DIM / 256;
        const size_t q0 = (size_t)row * G * TQ_HEAD_DIM;
        float qraw[NQ];
        auto load_all = [&](auto elem) __attribute__((always_inline)) {
#pragma unroll
            for (int n = 0; n < NQ; ++n) {
                const uint32_t i = tid + 256u * (uint32_t)n;
                qraw[n] = i < G * TQ_HEAD_DIM ? elem(q0 + i) : 0.f;
            }
        };
        if (a.q_dtype == TQ_F32) {
            load_all([&](size_t i) { return ((const TQ_GLOBAL float *)a.queries)[i]; });
        } else if (a.q_dtype == TQ_F16) {
            load_all([&](size_t i) { return (float)__builtin_bit_cast(_Float16, ((const TQ_GLOBAL uint16_t *)a.queries)[i]); });
        } else {
            load_all([&](size_t i) { return __uint_as_float((uint32_t)((const TQ_GLOBAL uint16_t *)a.queries)[i] << 16); });
        }
#pragma unroll
        for (int n = 0; n < NQ; ++n) {
            const uint32_t i = tid + 256u * (uint32_t)n;
            qt[i % TQ_HEAD_DIM][i / TQ_HEAD_DIM] = qraw[n] * a.scale;
        }
    }
    __syncthreads();
    if (do_rot) {   // rotated queries: q_rot[g][j] = sum_i Pi[j][i] * q[g][i]; all heads of a coordinate come with 16-byte reads
        const uint32_t j = tid & 127u, half = tid >> 7;
        const TQ_GLOBAL float *pc = (const TQ_GLOBAL float *)a.pi_k_t + (size_t)half * 64u * TQ_HEAD_DIM + j;
        float s[GP];
#pragma unroll
        for (int g = 0; g < GP; ++g) s[g] = 0.f;
#pragma unroll 16
        for (int i = 0; i < 64; ++i) {
            const float p = pc[(size_t)i * TQ_HEAD_DIM];
            float qv[MAXG];
#pragma unroll
            for (int h = 0; h < (GP + 3) / 4; ++h)
                *reinterpret_cast<float4 *>(&qv[4 * h]) = *reinterpret_cast<const float4 *>(&qt[half * 64u + i][4 * h]);
#pragma unroll
            for (int g = 0; g < GP; ++g) s[g] = fmaf(p, qv[g], s[g]);
        }
#pragma unroll
        for (int g = 0; g < GP; ++g) part[half][g][j] = s[g];
    }
    __syncthreads();
    if (do_rot)
        for (uint32_t o = tid; o < G * TQ_HEAD_DIM; o += 256u)
            ((TQ_GLOBAL float *)a.q_rot)[(size_t)row * G * TQ_HEAD_DIM + o] =
                part[0][o / TQ_HEAD_DIM][o % TQ_HEAD_DIM] + part[1][o / TQ_HEAD_DIM][o % TQ_HEAD_DIM];
    if (!W) return;
    {   // scores of the window tokens
        const uint32_t trips = (W + 63u) / 64u;
        float qq[GP][8];
#pragma unroll
        for (int g = 0; g < GP; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) qq[g][e] = qt[8u * sub + e][g];
        auto score4 = [&](uint32_t trip, const Raw8<WD> (&raw)[4]) __attribute__((always_inline)) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t t = ktoken(trip, k);
                float x[8];
                tq_cvt8<WD>(raw[k], x);
#pragma unroll
                for (int g = 0; g < GP; ++g) {
                    float sg = 0.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) sg = fmaf(x[e], qq[g][e], sg);
                    sg = tq_row_sum16(sg);
                    if (sub == 15u && t < W) sc[g][t] = sg;
                }
            }
        };
#pragma unroll
        for (int tr = 0; tr < PRE_K; ++tr)
            if ((uint32_t)tr < trips) score4(tr, kpre[tr]);      // uniform
        for (uint32_t trip = PRE_K; trip < trips; ++trip) {
            Raw8<WD> raw[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
                raw[k] = tq_load8_raw<WD>(a.k_win, win_base + (size_t)min(ktoken(trip, k), W - 1u) * TQ_HEAD_DIM + 8u * sub);
            score4(trip, raw);
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
    {   // weighted value sums: this lane's four columns over its tokens
        const uint32_t trips = (W + 31u) / 32u;
        float acc[GP][4];
#pragma unroll
        for (int g = 0; g < GP; ++g)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[g][e] = 0.f;
        auto sum4 = [&](uint32_t trip, const uint32_t (&raw)[4][VW]) __attribute__((always_inline)) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t t = vtoken(trip, k);
                float x[4];
                vcvt(raw[k], x);
#pragma unroll
                for (int g = 0; g < GP; ++g) {
                    const float p = (t < W && (uint32_t)g < G) ? sc[g][t] : 0.f;    // rows g >= G of sc are never written
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[g][e] = fmaf(p, x[e], acc[g][e]);
                }
            }
        };
#pragma unroll
        for (int tr = 0; tr < PRE_V; ++tr)
            if ((uint32_t)tr < trips) sum4(tr, vpre[tr]);        // uniform
        for (uint32_t trip = PRE_V; trip < trips; ++trip) {
            uint32_t raw[4][VW];
#pragma unroll
            for (int k = 0; k < 4; ++k) vload(vtoken(trip, k), raw[k]);
            sum4(trip, raw);
        }
#pragma unroll
        for (int g = 0; g < GP; ++g)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float v = acc[g][e] + __shfl_xor(acc[g][e], 32);
                if (tk5 == 0u) part[wave][g][4u * sub5 + e] = v;
            }
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

// One block per (packed row, GP query heads of it), 512 threads = (coordinate j, quarter q): log-sum-exp merge of the
// splits (each quarter takes every fourth split), rotation of the value sums back (x = y @ Pi_v; a quarter takes a
// fourth of the contraction and reads its part of Pi_v once for the block's heads), the window's share, normalisation,
// cast.  GP = the whole group (padded to 2, 4, 8, 16) when there are rows enough to fill the chip: Pi_v then crosses the
// L2 once per row instead of once per head (7.7 instead of 13.6 us for 512 rows x 4 heads).  GP = 1 for few rows, where
// the chain of a block that walks every head's splits is what takes the time (5.7 against 13.7 us for 8 rows x 32 splits).
template <int GP>
__global__ __launch_bounds__(512) void tq_attend_merge_kernel(MergeArgs a) {
    __shared__ float red_m[GP];
    __shared__ float acc_q[4][GP][TQ_HEAD_DIM];     // per quarter: sums of the splits, later partial rotations
    __shared__ float r_sum[GP][TQ_HEAD_DIM];
    __shared__ float l_q[4][GP];
    const uint32_t GA = a.group, S = a.splits;               // GA: all heads of a row (the stride of the records)
    const uint32_t per_row = (GA + GP - 1u) / GP;
    const uint32_t row = blockIdx.x / per_row, g0 = (blockIdx.x % per_row) * GP;
    const uint32_t G = min((uint32_t)GP, GA - g0);            // heads of this block: g0 .. g0 + G - 1
    const uint32_t tid = threadIdx.x, j = tid & 127u, q = tid >> 7, lane = tid & 63u, wave = tid >> 6;
    // record (s, g) of the block's heads at + (s * GA + g) * AT_PART
    const TQ_GLOBAL float *part = (const TQ_GLOBAL float *)a.partial + ((size_t)row * S * GA + g0) * AT_PART;
    const TQ_GLOBAL float *pw = a.part_w ? (const TQ_GLOBAL float *)a.part_w + ((size_t)row * GA + g0) * AT_PART : nullptr;
    // 1. per head, the largest of the records' references: wave w takes heads w, w + 8
    for (uint32_t g = wave; g < G; g += 8u) {
        float m = pw ? pw[g * AT_PART] : -3.0e38f;
        for (uint32_t s = lane; s < S; s += 64u) m = fmaxf(m, part[((size_t)s * GA + g) * AT_PART]);
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d));
        if (lane == 0u) red_m[g] = m;
    }
    __syncthreads();
    // 2. this quarter's splits, every head
    float acc[GP], l[GP], mg[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) { acc[g] = 0.f; l[g] = 0.f; mg[g] = (uint32_t)g < G ? red_m[g] : 0.f; }
    for (uint32_t s = q; s < S; s += 4u) {
#pragma unroll
        for (int g = 0; g < GP; ++g) {
            if ((uint32_t)g < G) {       // uniform
                const TQ_GLOBAL float *ps = part + ((size_t)s * GA + g) * AT_PART;
                const float f = __expf(ps[0] - mg[g]);
                acc[g] = fmaf(f, ps[2 + j], acc[g]);
                l[g] = fmaf(f, ps[1], l[g]);
            }
        }
    }
#pragma unroll
    for (int g = 0; g < GP; ++g) {
        acc_q[q][g][j] = acc[g];
        if (j == 0u) l_q[q][g] = l[g];
    }
    __syncthreads();
    // 3. sums over the quarters (thread (q, j) takes heads q, q + 4, ...; the padding heads hold zeros), then the rotation back
    for (uint32_t g = q; g < GP; g += 4u) r_sum[g][j] = acc_q[0][g][j] + acc_q[1][g][j] + acc_q[2][g][j] + acc_q[3][g][j];
    __syncthreads();
    float x[GP];
#pragma unroll
    for (int g = 0; g < GP; ++g) x[g] = 0.f;
#pragma unroll 8
    for (uint32_t k = 32u * q; k < 32u * q + 32u; ++k) {
        const float p = ((const TQ_GLOBAL float *)a.pi_v)[(size_t)k * TQ_HEAD_DIM + j];
#pragma unroll
        for (int g = 0; g < GP; ++g) x[g] = fmaf(r_sum[g][k], p, x[g]);
    }
#pragma unroll
    for (int g = 0; g < GP; ++g) acc_q[q][g][j] = x[g];        // every read of acc_q as split sums is behind the barrier above
    __syncthreads();
    // 4. the window's share, normalisation, cast: thread (q, j) finishes heads q, q + 4, ...
    for (uint32_t g = q; g < G; g += 4u) {
        float v = acc_q[0][g][j] + acc_q[1][g][j] + acc_q[2][g][j] + acc_q[3][g][j];
        float den = l_q[0][g] + l_q[1][g] + l_q[2][g] + l_q[3][g];
        if (pw) {
            const float f = __expf(pw[g * AT_PART] - red_m[g]);
            v = fmaf(f, pw[g * AT_PART + 2 + j], v);
            den = fmaf(f, pw[g * AT_PART + 1], den);
        }
        v /= den;
        const size_t idx = ((size_t)row * GA + g0 + g) * TQ_HEAD_DIM + j;
        if (a.out_dtype == TQ_F32) {
            ((TQ_GLOBAL float *)a.out)[idx] = v;
        } else if (a.out_dtype == TQ_F16) {
            const _Float16 h = (_Float16)v;
            ((TQ_GLOBAL uint16_t *)a.out)[idx] = __builtin_bit_cast(uint16_t, h);
        } else {
            const __bf16 h = (__bf16)v;
            ((TQ_GLOBAL uint16_t *)a.out)[idx] = __builtin_bit_cast(uint16_t, h);
        }
    }
}

int device_cus(int &cus) {
    static std::atomic<int> cache[64];   // per device; threads that race here store the same value
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return TQ_ERR_NO_DEVICE;
    int c = cache[dev].load(std::memory_order_relaxed);
    if (c == 0) {
        e = hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return (int)e;
        c = c > 0 ? c : 1;
        cache[dev].store(c, std::memory_order_relaxed);
    }
    cus = c;
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

extern "C" int tq_qjl_scores(const uint8_t *idx_bytes, const uint16_t *vec_norms, const uint8_t *sign_bytes, const uint16_t *residual_norm,
                             long long rows, long long tokens, const void *table_dev, int head_dim, int mse_bits,
                             const float *q_rot, const float *q_sign, long long n_queries, float *scores, void *stream) {
    int rc = check_packed(idx_bytes, vec_norms, 0, rows, tokens, table_dev, head_dim, mse_bits);
    if (rc) return rc;
    if (n_queries < 0 || n_queries > 32ll * 65535) return TQ_ERR_SIZE;
    if (rows == 0 || tokens == 0 || n_queries == 0) return TQ_OK;
    if (!sign_bytes || !residual_norm || !q_rot || !q_sign || !scores) return TQ_ERR_NULL;
    if (((uintptr_t)sign_bytes & 15u) || ((uintptr_t)residual_norm & 1u) || ((uintptr_t)q_rot & 3u) || ((uintptr_t)q_sign & 3u) ||
        ((uintptr_t)scores & 3u))
        return TQ_ERR_ALIGN;
    int cus = 0;
    rc = device_cus(cus);
    if (rc) return rc;
    QjlScoreArgs a;
    a.idx_bytes = idx_bytes;
    a.vec_norms = vec_norms;
    a.sign_bytes = sign_bytes;
    a.residual_norm = residual_norm;
    a.table = static_cast<const uint8_t *>(table_dev);
    a.q_rot = q_rot;
    a.q_sign = q_sign;
    a.scores = scores;
    a.tokens = (uint32_t)tokens;
    a.n_q = (uint32_t)n_queries;
    const uint32_t chunks = (uint32_t)((n_queries + 31) / 32);
    const uint32_t tiles = (uint32_t)((tokens + 31) / 32);
    const uint32_t want = (tiles + SC_WAVES - 1) / SC_WAVES;
    // about two four-wave blocks per compute unit: a block spends several microseconds on its query operands and
    // tables before its first tile, so it should have many tiles to walk
    uint32_t bx = (uint32_t)(((long long)cus * 2 + rows * chunks - 1) / (rows * chunks));
    if (bx > want) bx = want;
    if (bx < 1) bx = 1;
    dim3 grid(bx, (unsigned)rows, chunks), block(SC_WAVES * TQ_WAVE, 1, 1);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (8 / mse_bits) {
        case 8: hipLaunchKernelGGL(tq_qjl_scores_kernel<8>, grid, block, 0, s, a); break;
        case 4: hipLaunchKernelGGL(tq_qjl_scores_kernel<4>, grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL(tq_qjl_scores_kernel<2>, grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL(tq_qjl_scores_kernel<1>, grid, block, 0, s, a); break;
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
        case 8: hipLaunchKernelGGL((tq_attend_kernel<IPBK, 8>), grid, dim3(AT_WAVES * TQ_WAVE), 0, s, a); break;
        case 4: hipLaunchKernelGGL((tq_attend_kernel<IPBK, 4>), grid, dim3(AT_WAVES * TQ_WAVE), 0, s, a); break;
        case 2: hipLaunchKernelGGL((tq_attend_kernel<IPBK, 2>), grid, dim3(AT_WAVES * TQ_WAVE), 0, s, a); break;
        default: hipLaunchKernelGGL((tq_attend_kernel<IPBK, 1>), grid, dim3(AT_WAVES * TQ_WAVE), 0, s, a); break;
    }
    return (int)hipGetLastError();
}
}  // namespace

extern "C" int tq_attend_splits(long long rows, long long tokens) {
    if (rows <= 0 || tokens <= 0) return 1;
    int cus = 0;
    if (device_cus(cus)) cus = 256;
    // One eight-wave block is resident per compute unit.  Few rows: as many splits as fill the chip once (a
    // second generation of blocks would stage its tables again: 17 instead of 23 us for 8 rows x 32K tokens).
    // Many rows: two generations, which balances blocks of unequal speed better than one.
    long long splits = rows * 2 <= cus ? cus / rows : ((long long)cus * 2 + rows - 1) / rows;
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
    if (group < 1 || group > 16 || splits < 1 || splits > 65535) return TQ_ERR_SIZE;
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
    if (rows < 0 || rows > 0x7fffffff || group < 1 || group > 16 || n_win < 0 || n_win > 512) return TQ_ERR_SIZE;
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
    const int wd = n_win ? win_dtype : TQ_BF16;
    const int gp = group > 8 ? 16 : group > 4 ? 8 : group > 2 ? 4 : group;
    const dim3 grid((unsigned)rows, n_win ? 2u : 1u), block(256);
#define TQ_PREP_CASE(WD, GP) \
    if (wd == WD && gp == GP) hipLaunchKernelGGL((tq_attend_prepare_kernel<WD, GP>), grid, block, 0, st, a)
    TQ_PREP_CASE(TQ_F32, 1); TQ_PREP_CASE(TQ_F32, 2); TQ_PREP_CASE(TQ_F32, 4); TQ_PREP_CASE(TQ_F32, 8); TQ_PREP_CASE(TQ_F32, 16);
    TQ_PREP_CASE(TQ_F16, 1); TQ_PREP_CASE(TQ_F16, 2); TQ_PREP_CASE(TQ_F16, 4); TQ_PREP_CASE(TQ_F16, 8); TQ_PREP_CASE(TQ_F16, 16);
    TQ_PREP_CASE(TQ_BF16, 1); TQ_PREP_CASE(TQ_BF16, 2); TQ_PREP_CASE(TQ_BF16, 4); TQ_PREP_CASE(TQ_BF16, 8); TQ_PREP_CASE(TQ_BF16, 16);
#undef TQ_PREP_CASE
    return (int)hipGetLastError();
}

extern "C" int tq_attend_merge(const float *partial, int splits, const float *part_w, const float *pi_v,
                               long long rows, int group, void *out, int out_dtype, void *stream) {
    if (rows < 0 || rows > 0x7fffffff / 16 || group < 1 || group > 16 || splits < 0) return TQ_ERR_SIZE;
    if (out_dtype != TQ_F32 && out_dtype != TQ_F16 && out_dtype != TQ_BF16) return TQ_ERR_DTYPE;
    if (rows == 0) return TQ_OK;
    if (!pi_v || !out || (splits && !partial) || (!splits && !part_w)) return TQ_ERR_NULL;
    MergeArgs a;
    a.partial = partial; a.part_w = part_w; a.pi_v = pi_v; a.out = out;
    a.group = (uint32_t)group; a.splits = (uint32_t)splits; a.out_dtype = out_dtype;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    int cus = 0;
    if (device_cus(cus)) cus = 256;
    const dim3 block(512);
    if (group == 1 || rows * 2 <= cus) {                     // few rows: one block per (row, head)
        hipLaunchKernelGGL(tq_attend_merge_kernel<1>, dim3((unsigned)(rows * group)), block, 0, st, a);
    } else {
        const dim3 grid((unsigned)rows);
        if (group > 8) hipLaunchKernelGGL(tq_attend_merge_kernel<16>, grid, block, 0, st, a);
        else if (group > 4) hipLaunchKernelGGL(tq_attend_merge_kernel<8>, grid, block, 0, st, a);
        else if (group > 2) hipLaunchKernelGGL(tq_attend_merge_kernel<4>, grid, block, 0, st, a);
        else hipLaunchKernelGGL(tq_attend_merge_kernel<2>, grid, block, 0, st, a);
    }
    return (int)hipGetLastError();
}

// ---- one decode step of a streaming cache layer, as two calls -----------------------------------------
// Each call chains entry points declared above; a host that pays per call (an interpreter binding) makes two
// calls per layer and step instead of nine.

namespace {
// window slot `put` of every row <- the row's new key and value vector (16-byte pieces)
__global__ __launch_bounds__(256) void tq_window_put_kernel(const uint8_t *__restrict__ k_new, const uint8_t *__restrict__ v_new,
                                                            long long k_new_stride, long long v_new_stride,
                                                            uint8_t *__restrict__ k_win, uint8_t *__restrict__ v_win,
                                                            long long win_stride, uint32_t pieces, uint32_t rows) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;      // (row, tensor, piece)
    if (i >= rows * 2u * pieces) return;
    const uint32_t piece = i % pieces, tensor = (i / pieces) & 1u, row = i / (2u * pieces);
    const uint8_t *src = tensor ? v_new + (long long)row * v_new_stride : k_new + (long long)row * k_new_stride;
    uint8_t *dst = (tensor ? v_win : k_win) + (long long)row * win_stride;
    tq_gstore16(dst + piece * 16u, tq_gload16(src + piece * 16u));
}

inline int elem_size(int dtype) { return dtype == TQ_F32 ? 4 : (dtype == TQ_F16 || dtype == TQ_BF16) ? 2 : 0; }
}  // namespace

extern "C" int tq_append_token(const void *k_new, const void *v_new, int dtype, long long k_new_stride, long long v_new_stride,
                               void *k_win, void *v_win, long long win_stride, long long evict, long long put,
                               const void *table_k, const void *table_v, int head_dim, int bits_k, int bits_v,
                               uint8_t *k_idx, uint16_t *k_norms, uint8_t *v_idx, uint16_t *v_norms,
                               long long packed_row_stride, long long packed_slot, long long rows, void *stream) {
    const int eb = elem_size(dtype);
    if (!eb) return TQ_ERR_DTYPE;
    if (head_dim != TQ_HEAD_DIM) return TQ_ERR_HEAD_DIM;
    if (rows < 0 || rows > (1 << 24) || put < 0 || evict < -1 || packed_slot < 0) return TQ_ERR_SIZE;
    if (win_stride < (put + 1) * TQ_HEAD_DIM || win_stride < (evict + 1) * TQ_HEAD_DIM || evict == put) return TQ_ERR_SIZE;
    if (rows > 1 && (k_new_stride < TQ_HEAD_DIM || v_new_stride < TQ_HEAD_DIM)) return TQ_ERR_SIZE;
    if (rows == 0) return TQ_OK;
    if (!k_new || !v_new || !k_win || !v_win) return TQ_ERR_NULL;
    if (((uintptr_t)k_new & 15u) || ((uintptr_t)v_new & 15u) || ((uintptr_t)k_win & 15u) || ((uintptr_t)v_win & 15u) ||
        ((win_stride * eb) & 15) || (rows > 1 && (((k_new_stride * eb) & 15) || ((v_new_stride * eb) & 15))))
        return TQ_ERR_ALIGN;
    if (evict >= 0) {
        // the oldest window token of every row leaves the window: one vector per row, rows win_stride apart
        if (packed_slot >= (packed_row_stride ? packed_row_stride : 1)) return TQ_ERR_SIZE;
        const int gk = tq_bytes_per_vector(head_dim, bits_k), gv = tq_bytes_per_vector(head_dim, bits_v);
        if (gk < 0) return gk;
        if (gv < 0) return gv;
        if (!k_idx || !k_norms || !v_idx || !v_norms) return TQ_ERR_NULL;
        const uint8_t *kw = static_cast<const uint8_t *>(k_win) + evict * TQ_HEAD_DIM * eb;
        const uint8_t *vw = static_cast<const uint8_t *>(v_win) + evict * TQ_HEAD_DIM * eb;
        int rc = tq_compress(kw, dtype, rows, 1, win_stride, TQ_HEAD_DIM, table_k, head_dim, bits_k,
                             k_idx + packed_slot * gk, k_norms + packed_slot, packed_row_stride, nullptr, stream);
        if (rc) return rc;
        rc = tq_compress(vw, dtype, rows, 1, win_stride, TQ_HEAD_DIM, table_v, head_dim, bits_v,
                         v_idx + packed_slot * gv, v_norms + packed_slot, packed_row_stride, nullptr, stream);
        if (rc) return rc;
    }
    const uint32_t pieces = (uint32_t)(TQ_HEAD_DIM * eb / 16);
    const uint32_t n = (uint32_t)rows * 2u * pieces;
    hipLaunchKernelGGL(tq_window_put_kernel, dim3((n + 255u) / 256u), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint8_t *>(k_new), static_cast<const uint8_t *>(v_new),
                       k_new_stride * eb, v_new_stride * eb,
                       static_cast<uint8_t *>(k_win) + put * TQ_HEAD_DIM * eb, static_cast<uint8_t *>(v_win) + put * TQ_HEAD_DIM * eb,
                       win_stride * eb, pieces, (uint32_t)rows);
    return (int)hipGetLastError();
}

extern "C" int tq_attend_step(const void *queries, int q_dtype, long long rows, int group, float scale,
                              const float *pi_k_t, const float *pi_v,
                              const void *k_win, const void *v_win, int win_dtype, long long n_win, long long win_stride,
                              const uint8_t *k_idx, const uint16_t *k_norms, const uint8_t *v_idx, const uint16_t *v_norms,
                              long long packed_row_stride, long long tokens,
                              const void *table_k, const void *table_v, int head_dim, int bits_k, int bits_v,
                              float *q_rot, float *part_w, float *partial, int splits,
                              void *out, int out_dtype, void *stream) {
    if (tokens < 0 || n_win < 0 || (tokens == 0 && n_win == 0)) return TQ_ERR_SIZE;      // nothing to attend to
    if (out_dtype != TQ_F32 && out_dtype != TQ_F16 && out_dtype != TQ_BF16) return TQ_ERR_DTYPE;
    if (!out || !pi_v) return TQ_ERR_NULL;
    if (tokens && splits < 1) return TQ_ERR_SIZE;
    if (tokens && !partial) return TQ_ERR_NULL;
    int rc = tq_attend_prepare(queries, q_dtype, rows, group, scale, pi_k_t, k_win, v_win, win_dtype, n_win, win_stride,
                               q_rot, part_w, stream);
    if (rc || rows == 0) return rc;
    if (tokens) {
        rc = tq_attend_partials(k_idx, k_norms, v_idx, v_norms, packed_row_stride, rows, tokens, table_k, table_v,
                                head_dim, bits_k, bits_v, q_rot, group, splits, partial, stream);
        if (rc) return rc;
    }
    return tq_attend_merge(tokens ? partial : nullptr, tokens ? splits : 0, n_win ? part_w : nullptr, pi_v, rows, group,
                           out, out_dtype, stream);
}
