// Second stage of the V2 key path: 1-bit QJL signs of the quantisation residual and its norm.
// Replaces, together with tq_compress for the first stage, TurboQuantCompressorV2.compress
// (upstream turboquant/compressors.py:84-122): given the input vectors and the MSE codes that tq_compress wrote,
//     k_mse    = (centroids[codes] @ Pi) * ||x||          (float32, :108-109)
//     residual = x - k_mse                                (:112)
//     residual_norm = ||residual||  -> fp16               (:113, :121)
//     signs    = (residual @ S^T >= 0)                    (:116-117), packed 8 per byte, coordinate 8b+k in bit 7-k
//
// Work decomposition (gfx950, wave64): a block is four waves that share tiles of 32 vectors; wave w keeps the rows
// [32w, 32w+32) of Pi^T and of S resident in registers as MFMA A operands, each as two fp16 terms (hi + lo: 22 bits)
// of the matrix times a power of two.  The B operands are two-term fp16 splits as well (the centroid of every code,
// from a table of ready-made pairs; then the residual, scaled per vector by a power of two taken from its norm's
// exponent), staged in LDS in the XOR-swizzled tile layout of the compress kernel.  The three products hi*hi, hi*lo,
// lo*hi are taken (the fourth weighs 2^-22), accumulation is fp32: both rotations agree with a float32 GEMM to a few
// 1e-7 of the vector's scale, the noise level of that GEMM's own rounding.  (The residual is a difference of nearly
// equal vectors, up to 70 times smaller than they are at 7 bits: this is the precision its signs need.)
#include <mutex>

#include "tq_device.h"

namespace {

constexpr int QTHREADS = 4 * TQ_WAVE;

struct QjlArgs {
    const uint8_t *states;      // input vectors, element type DTYPE
    long long token_stride;     // bytes between consecutive vectors
    const uint8_t *idx_bytes;   // MSE codes as tq_compress packs them, dense [n_vec, G]
    const uint8_t *table;       // blob of tq_qjl_table_build
    uint8_t *sign_bytes;        // out: [n_vec, 16]
    uint16_t *residual_norm;    // out: fp16 [n_vec]
    uint32_t n_vec;
    uint32_t mse_bits;
};

// Two floats -> their fp16 terms (hi: round toward zero, lo: the remainder, exact in fp32 before its own rounding).
struct TermPair { uint32_t hi, lo; };
__device__ __forceinline__ TermPair split_pair(float x0, float x1) {
    typedef __fp16 pk_half2 __attribute__((ext_vector_type(2)));
    const pk_half2 h = __builtin_amdgcn_cvt_pkrtz(x0, x1);
    const pk_half2 l = __builtin_amdgcn_cvt_pkrtz(x0 - (float)h[0], x1 - (float)h[1]);
    return {__builtin_bit_cast(uint32_t, h), __builtin_bit_cast(uint32_t, l)};
}

// BITS: packing class of the codes (1, 2, 3, 4, or 8 = one code per byte for 5..7 bits)
template <int DTYPE, int BITS>
__global__ __launch_bounds__(QTHREADS, 2) void tq_qjl_residual_kernel(QjlArgs a) {
    constexpr int ELEM = DTYPE == TQ_F32 ? 4 : 2;
    constexpr int IPB = 8 / BITS;
    constexpr int NB = 16 / IPB;           // packed bytes of 16 codes
    constexpr int G = 8 * NB;              // packed bytes per vector
    constexpr int TILE = 32 * TQ_HEAD_DIM * 2;   // one fp16 term of a 32-vector tile: 8 KiB

    __shared__ __attribute__((aligned(16))) uint8_t lds_terms[2][TILE];   // centroid terms, then residual terms
    __shared__ uint32_t lds_cent[256];     // code -> fp16 terms of its centroid (hi | lo << 16)
    __shared__ float lds_n2[4][32];        // shares of ||x||^2
    __shared__ float lds_r2[4][32];        // shares of ||residual||^2

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = tq_uniform32(tid >> 6);
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const TqQjlHeader *hd = reinterpret_cast<const TqQjlHeader *>(a.table);

    // ---- this wave's rows of Pi^T and S, resident for the whole kernel
    tq_u4 a_pit[2][TQ_STEPS], a_s[2][TQ_STEPS];
    {
        const uint8_t *pit = a.table + hd->off_pit, *sm = a.table + hd->off_s;
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            const size_t o = (((size_t)wave * TQ_STEPS + s) * 64 + lane) * 16;
#pragma unroll
            for (int q = 0; q < 2; ++q) a_pit[q][s] = tq_gload16(pit + (size_t)q * TQ_OPERAND_BYTES + o);
#pragma unroll
            for (int q = 0; q < 2; ++q) a_s[q][s] = tq_gload16(sm + (size_t)q * TQ_OPERAND_BYTES + o);
        }
    }
    for (uint32_t i = tid; i < 256u; i += QTHREADS)
        lds_cent[i] = i < hd->levels ? *reinterpret_cast<const TQ_GLOBAL uint32_t *>((const TQ_GLOBAL uint8_t *)(a.table + hd->off_centroids) + 4u * i) : 0u;
    const float k_scale = hd->k_scale;
    __syncthreads();

    const uint32_t n_tiles = (a.n_vec + 31u) / 32u;
    const uint32_t dv = tid >> 3, seg = tid & 7u;            // role in the decode: vector of the tile, 16-code segment
    const uint32_t code_mask = (1u << a.mse_bits) - 1u;
    // the lane's 16 coordinates [32w + 16hk, +16) of vector n are pieces 4w + 2hk and 4w + 2hk + 1 of its row
    const uint32_t my_piece = 4u * wave + 2u * hk;

    // What a thread reads of a tile: the packed bytes of 16 codes of vector dv (decode role) and the 16 input
    // coordinates [32w + 16hk, +16) of vector n (matrix role).  Fetched one tile ahead of the work on them.
    constexpr int XQ = 16 * ELEM / 16;     // 16-byte pieces of the lane's coordinates
    struct Fetched { uint32_t raw[4]; tq_u4 xq[XQ]; };
    auto fetch = [&](uint32_t tl) {
        Fetched f;
        uint32_t v = tl * 32u + dv;
        v = v < a.n_vec ? v : a.n_vec - 1u;              // tail: the last vector again, never stored
        const uint8_t *src = a.idx_bytes + (size_t)v * G + seg * NB;
        f.raw[0] = f.raw[1] = f.raw[2] = f.raw[3] = 0u;
        if constexpr (NB == 2) f.raw[0] = tq_gload2(reinterpret_cast<const uint16_t *>(src));
        else if constexpr (NB == 4) f.raw[0] = *reinterpret_cast<const TQ_GLOBAL uint32_t *>((const TQ_GLOBAL uint8_t *)src);
        else if constexpr (NB == 8) { const tq_u2 t = tq_gload8(src); f.raw[0] = t[0]; f.raw[1] = t[1]; }
        else { const tq_u4 t = tq_gload16(src); f.raw[0] = t[0]; f.raw[1] = t[1]; f.raw[2] = t[2]; f.raw[3] = t[3]; }
        uint32_t vx = tl * 32u + n;
        vx = vx < a.n_vec ? vx : a.n_vec - 1u;
        const uint8_t *xs = a.states + (long long)vx * a.token_stride + (32u * wave + 16u * hk) * ELEM;
#pragma unroll
        for (int q = 0; q < XQ; ++q) f.xq[q] = tq_gload16(xs + 16 * q);
        return f;
    };
    Fetched ahead = fetch(blockIdx.x < n_tiles ? blockIdx.x : 0u);

    for (uint32_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const Fetched cur = ahead;
        {
            const uint32_t next = tile + gridDim.x;
            ahead = fetch(next < n_tiles ? next : tile);     // past the end: the same tile again, never used
        }
        // ---- (1) codes -> the fp16 terms of their centroids in LDS (vector dv, codes [16 seg, 16 seg + 16))
        {
            const uint32_t (&raw)[4] = cur.raw;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                uint32_t c[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int k = 8 * half + i;                       // code number inside the segment
                    const int byte = k / IPB, pos = k % IPB;
                    const uint32_t bv = (raw[byte / 4] >> (8 * (byte % 4))) & 0xffu;
                    const uint32_t code = (bv >> (BITS * (IPB - 1 - pos))) & code_mask;
                    c[i] = lds_cent[code];
                }
                tq_u4 t0, t1;
#pragma unroll
                for (int d = 0; d < 4; ++d) {     // two codes per word: their hi terms, their lo terms
                    t0[d] = __builtin_amdgcn_perm(c[2 * d + 1], c[2 * d], 0x05040100u);
                    t1[d] = __builtin_amdgcn_perm(c[2 * d + 1], c[2 * d], 0x07060302u);
                }
                const uint32_t off = dv * 256u + (((2u * seg + half) ^ (dv & 15u)) << 4);
                *reinterpret_cast<tq_u4 *>(lds_terms[0] + off) = t0;
                *reinterpret_cast<tq_u4 *>(lds_terms[1] + off) = t1;
            }
        }
        // ---- the lane's 16 input coordinates, and its share of ||x||^2
        float x[16];
        {
            if constexpr (ELEM == 4) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const tq_u4 t = cur.xq[q];
#pragma unroll
                    for (int i = 0; i < 4; ++i) x[4 * q + i] = __uint_as_float(t[i]);
                }
            } else {
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const tq_u4 t = cur.xq[q];
                    if constexpr (DTYPE == TQ_BF16) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            x[8 * q + 2 * i] = __uint_as_float(t[i] << 16);
                            x[8 * q + 2 * i + 1] = __uint_as_float(t[i] & 0xffff0000u);
                        }
                    } else {
                        // (the halves are taken from a cast of the whole vector: casting one 32-bit element of `t` to a
                        // pair of halves made the compiler read element 0 four times)
                        const tq_half8 h8 = __builtin_bit_cast(tq_half8, t);
#pragma unroll
                        for (int i = 0; i < 8; ++i) x[8 * q + i] = (float)h8[i];
                    }
                }
            }
            float s2 = 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) s2 = fmaf(x[i], x[i], s2);
            s2 += __shfl_xor(s2, 32);
            lds_n2[wave][n] = s2;
        }
        __syncthreads();

        // ---- (2) k_unit = Pi^T c on the matrix cores
        tq_f16v acc = tq_zero16();
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            const uint32_t off = n * 256u + (((2u * s + hk) ^ (n & 15u)) << 4);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const tq_u4 bop = *reinterpret_cast<const tq_u4 *>(lds_terms[i] + off);
#pragma unroll
                for (int j = 0; i + j < 2; ++j) acc = mfma_f16(a_pit[j][s], bop, acc);
            }
        }
        const float nrm = sqrtf((lds_n2[0][n] + lds_n2[1][n]) + (lds_n2[2][n] + lds_n2[3][n]));
        // power of two that brings the residual (|r_i| <= 2 ||x||) into the fp16 range: 2^(10 - E), ||x|| = f * 2^E, f in [0.5, 1)
        uint32_t r_exp = 263u - ((__float_as_uint(nrm) >> 23) & 0xffu);
        r_exp = r_exp > 254u ? 254u : r_exp;
        const float r_scale = __uint_as_float(r_exp << 23);
        // ---- (3) residual, its norm, its two fp16 terms
        float r[16];
        float r2 = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float km = (acc[i] * k_scale) * nrm;
            r[i] = x[i] - km;
            r2 = fmaf(r[i], r[i], r2);
        }
        r2 += __shfl_xor(r2, 32);
        lds_r2[wave][n] = r2;
        __syncthreads();                   // everybody has read the centroid terms
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            tq_u4 t0, t1;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const TermPair t = split_pair(r[8 * half + 2 * d] * r_scale, r[8 * half + 2 * d + 1] * r_scale);
                t0[d] = t.hi;
                t1[d] = t.lo;
            }
            const uint32_t off = n * 256u + (((my_piece + half) ^ (n & 15u)) << 4);
            *reinterpret_cast<tq_u4 *>(lds_terms[0] + off) = t0;
            *reinterpret_cast<tq_u4 *>(lds_terms[1] + off) = t1;
        }
        __syncthreads();

        // ---- (4) projection by S, signs, stores
        tq_f16v prj = tq_zero16();
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            const uint32_t off = n * 256u + (((2u * s + hk) ^ (n & 15u)) << 4);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const tq_u4 bop = *reinterpret_cast<const tq_u4 *>(lds_terms[i] + off);
#pragma unroll
                for (int j = 0; i + j < 2; ++j) prj = mfma_f16(a_s[j][s], bop, prj);
            }
        }
        uint32_t word = 0;                 // byte 0: coordinates 0..7 of the lane, most significant bit first; byte 1: 8..15
#pragma unroll
        for (int i = 0; i < 16; ++i) word |= (prj[i] >= 0.f ? 1u : 0u) << (8 * (i / 8) + 7 - (i % 8));
        const uint32_t v = tile * 32u + n;
        if (v < a.n_vec) {
            tq_gstore2(reinterpret_cast<uint16_t *>(a.sign_bytes + (size_t)v * 16u + 4u * wave + 2u * hk), (uint16_t)word);
            if (wave == 0 && hk == 0) {
                const float rn = sqrtf((lds_r2[0][n] + lds_r2[1][n]) + (lds_r2[2][n] + lds_r2[3][n]));
                const _Float16 h = (_Float16)rn;
                tq_gstore2(a.residual_norm + v, __builtin_bit_cast(uint16_t, h));
            }
        }
        __syncthreads();                   // the residual terms and the shares are free again
    }
}

constexpr int MAX_DEVICES = 64;
std::mutex host_state_mutex;

template <int DTYPE, int BITS>
int launch(const QjlArgs &a, hipStream_t stream) {
    static int blocks[MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return TQ_ERR_NO_DEVICE;
    int resident;
    {
        std::lock_guard<std::mutex> lock(host_state_mutex);
        if (blocks[dev] == 0) {
            int cus = 0, per_cu = 0;
            e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e != hipSuccess) return (int)e;
            e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, tq_qjl_residual_kernel<DTYPE, BITS>, QTHREADS, 0);
            if (e != hipSuccess) return (int)e;
            blocks[dev] = (cus > 0 ? cus : 1) * (per_cu > 0 ? per_cu : 1);
        }
        resident = blocks[dev];
    }
    const uint32_t n_tiles = (a.n_vec + 31u) / 32u;
    const uint32_t bx = n_tiles < (uint32_t)resident ? n_tiles : (uint32_t)resident;
    hipLaunchKernelGGL((tq_qjl_residual_kernel<DTYPE, BITS>), dim3(bx), dim3(QTHREADS), 0, stream, a);
    return (int)hipGetLastError();
}

template <int DTYPE>
int dispatch_bits(int mse_bits, const QjlArgs &a, hipStream_t s) {
    switch (mse_bits) {
        case 1: return launch<DTYPE, 1>(a, s);
        case 2: return launch<DTYPE, 2>(a, s);
        case 3: return launch<DTYPE, 3>(a, s);
        case 4: return launch<DTYPE, 4>(a, s);
        case 5: case 6: case 7: return launch<DTYPE, 8>(a, s);
        default: return TQ_ERR_BITS;
    }
}

}  // namespace

extern "C" int tq_qjl_signs(const void *states, int dtype, long long n_vec, long long token_stride,
                            const uint8_t *idx_bytes, const void *qjl_table_dev, int head_dim, int mse_bits,
                            uint8_t *sign_bytes, uint16_t *residual_norm, void *stream) {
    if (mse_bits < 1 || mse_bits > 7) return TQ_ERR_BITS;
    if (head_dim != TQ_HEAD_DIM) return TQ_ERR_HEAD_DIM;
    const int eb = dtype == TQ_F32 ? 4 : (dtype == TQ_F16 || dtype == TQ_BF16) ? 2 : 0;
    if (!eb) return TQ_ERR_DTYPE;
    if (n_vec < 0 || n_vec > 0x7fffffffll) return TQ_ERR_SIZE;
    if (n_vec == 0) return TQ_OK;
    if (!states || !idx_bytes || !qjl_table_dev || !sign_bytes || !residual_norm) return TQ_ERR_NULL;
    if (token_stride < TQ_HEAD_DIM && n_vec > 1) return TQ_ERR_SIZE;
    if (((uintptr_t)states & 15u) || ((uintptr_t)idx_bytes & 15u) || ((uintptr_t)qjl_table_dev & 15u) ||
        ((uintptr_t)sign_bytes & 15u) || ((uintptr_t)residual_norm & 1u) || ((token_stride * eb) & 15))
        return TQ_ERR_ALIGN;
    QjlArgs a;
    a.states = static_cast<const uint8_t *>(states);
    a.token_stride = token_stride * eb;
    a.idx_bytes = idx_bytes;
    a.table = static_cast<const uint8_t *>(qjl_table_dev);
    a.sign_bytes = sign_bytes;
    a.residual_norm = residual_norm;
    a.n_vec = (uint32_t)n_vec;
    a.mse_bits = (uint32_t)mse_bits;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case TQ_F32: return dispatch_bits<TQ_F32>(mse_bits, a, s);
        case TQ_F16: return dispatch_bits<TQ_F16>(mse_bits, a, s);
        default: return dispatch_bits<TQ_BF16>(mse_bits, a, s);
    }
}
