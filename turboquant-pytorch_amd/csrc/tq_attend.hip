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
// row's `group` query heads, in the rotated space.  A wave takes tiles of 32 tokens: the packed bytes and
// the norm-scaled weights go through a wave-private LDS area, then lane l accumulates coordinates 2l, 2l+1
// of every query head over the tile's tokens (the contraction runs over tokens, a few rows only: VALU work).
template <int IPB>
__global__ __launch_bounds__(WV_WAVES *TQ_WAVE) void tq_weighted_values_kernel(WvArgs a) {
    constexpr int GB = TQ_HEAD_DIM / IPB;            // packed bytes per vector
    constexpr int TILE_BYTES = 32 * GB;              // 512 .. 4096
    constexpr int PIECES = TILE_BYTES / 16;          // 16-byte pieces per tile: 32 .. 256
    __shared__ __attribute__((aligned(16))) uint8_t lds_lut[4096];
    __shared__ __attribute__((aligned(16))) uint8_t lds_codes[WV_WAVES][TILE_BYTES];
    __shared__ __attribute__((aligned(16))) float lds_w[WV_WAVES][32][WV_MAX_GROUP];
    __shared__ float lds_red[WV_WAVES][WV_MAX_GROUP][TQ_HEAD_DIM];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t row = blockIdx.y, split = blockIdx.x;
    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(a.table);
    tq_copy_to_lds(lds_lut, a.table + hd->off_lut, 256u * 2u * IPB, tid, WV_WAVES * TQ_WAVE);
    __syncthreads();

    const uint32_t t_begin = split * a.chunk;
    const uint32_t t_end = min(a.tokens, t_begin + a.chunk);
    const size_t slot0 = (size_t)row * a.packed_row_stride;
    const uint32_t G = a.group;

    // where this lane's two codes (coordinates 2l, 2l+1) sit: byte inside a vector, fp16 pair inside the table entry
    const uint32_t byte_in_vec = (2u * lane) / IPB;
    const uint32_t pair_off = ((2u * lane) % IPB) * 2u;

    float acc[WV_MAX_GROUP][2];
#pragma unroll
    for (int g = 0; g < WV_MAX_GROUP; ++g) acc[g][0] = acc[g][1] = 0.f;

    for (uint32_t t0 = t_begin + 32u * wave; t0 < t_end; t0 += 32u * WV_WAVES) {
        const uint32_t n_tok = min(32u, t_end - t0);
        // packed bytes of the tile: contiguous in memory (tokens of one row follow each other)
        const uint8_t *src = a.idx_bytes + (slot0 + t0) * GB;
#pragma unroll
        for (int p = 0; p < (PIECES + 63) / 64; ++p) {
            const uint32_t piece = p * 64u + lane;
            if (piece < PIECES && piece * 16u < n_tok * GB)
                *reinterpret_cast<tq_u4 *>(&lds_codes[wave][piece * 16u]) = tq_gload16(src + piece * 16u);
        }
        // weights times norms, [token][head]
        {
            const uint32_t tl = lane & 31u;
            const bool ok = tl < n_tok;
            const float nrm = ok ? (float)__builtin_bit_cast(_Float16, tq_gload2(a.vec_norms + slot0 + t0 + tl)) : 0.f;
            for (uint32_t g = lane >> 5; g < WV_MAX_GROUP; g += 2u) {
                float w = 0.f;
                if (ok && g < G) w = ((const TQ_GLOBAL float *)a.weights)[((size_t)row * G + g) * a.stride + t0 + tl] * nrm;
                lds_w[wave][tl][g] = w;
            }
        }
        __builtin_amdgcn_wave_barrier();
        for (uint32_t tl = 0; tl < n_tok; ++tl) {
            float c0, c1;
            if constexpr (IPB == 1) {
                const uint32_t two = *reinterpret_cast<const uint16_t *>(&lds_codes[wave][tl * GB + 2u * lane]);
                c0 = (float)__builtin_bit_cast(_Float16, *reinterpret_cast<const uint16_t *>(lds_lut + (two & 0xffu) * 2u));
                c1 = (float)__builtin_bit_cast(_Float16, *reinterpret_cast<const uint16_t *>(lds_lut + (two >> 8) * 2u));
            } else {
                const uint32_t b = lds_codes[wave][tl * GB + byte_in_vec];
                const tq_half2 c = __builtin_bit_cast(tq_half2, *reinterpret_cast<const uint32_t *>(lds_lut + b * (2u * IPB) + pair_off));
                c0 = (float)c[0];
                c1 = (float)c[1];
            }
            const float4 w03 = *reinterpret_cast<const float4 *>(&lds_w[wave][tl][0]);
            const float4 w47 = *reinterpret_cast<const float4 *>(&lds_w[wave][tl][4]);
            const float w[8] = {w03.x, w03.y, w03.z, w03.w, w47.x, w47.y, w47.z, w47.w};
#pragma unroll
            for (int g = 0; g < WV_MAX_GROUP; ++g) {
                acc[g][0] = fmaf(w[g], c0, acc[g][0]);
                acc[g][1] = fmaf(w[g], c1, acc[g][1]);
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int g = 0; g < WV_MAX_GROUP; ++g) {
        lds_red[wave][g][2 * lane] = acc[g][0];
        lds_red[wave][g][2 * lane + 1] = acc[g][1];
    }
    __syncthreads();
    float *dst = a.partial + ((size_t)row * gridDim.x + split) * G * TQ_HEAD_DIM;
    for (uint32_t i = tid; i < G * TQ_HEAD_DIM; i += WV_WAVES * TQ_WAVE) {
        const uint32_t g = i / TQ_HEAD_DIM, j = i % TQ_HEAD_DIM;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < WV_WAVES; ++w) s += lds_red[w][g][j];
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
    const long long most = (tokens + 32 * WV_WAVES - 1) / (32 * WV_WAVES);
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
    a.chunk = (uint32_t)((per_split + 31) / 32 * 32);
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
