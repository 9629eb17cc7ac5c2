// Second stage of the V2 key path: 1-bit QJL signs of the quantisation residual and its norm.
// Replaces, together with tq_compress for the first stage, TurboQuantCompressorV2.compress
// (upstream turboquant/compressors.py:84-122): given the input vectors and the MSE codes that tq_compress wrote,
//     k_mse    = (centroids[codes] @ Pi) * ||x||          (float32, :108-109)
//     residual = x - k_mse                                (:112)
//     residual_norm = ||residual||  -> fp16               (:113, :121)
//     signs    = (residual @ S^T >= 0)                    (:116-117), packed 8 per byte, coordinate 8b+k in bit 7-k
//
// Work decomposition (gfx950, wave64): a block is four waves that share tiles of 32 vectors; wave w keeps the rows
// [32w, 32w+32) of Pi^T (three bf16 terms) and of S (two bf16 terms) resident in registers as MFMA A operands.  The
// B operands are exact three-term bf16 splits of float32 data (the centroid of every code, then the residual),
// staged in LDS in the XOR-swizzled tile layout of the compress kernel; all products whose weight is at least
// 2^-24 of the leading one are taken, accumulation is fp32, so both rotations agree with a float32 GEMM to ~1e-6.
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

__device__ __forceinline__ tq_f16v qmfma(tq_u4 a, tq_u4 b, tq_f16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(tq_bf8, a), __builtin_bit_cast(tq_bf8, b), c, 0, 0, 0);
}

// Exact split of eight floats into three bf16 terms each (every term a truncation, every remainder exact in fp32).
__device__ __forceinline__ void qsplit8(const float (&x)[8], tq_u4 &t0, tq_u4 &t1, tq_u4 &t2) {
    uint32_t a[8], b[8], c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t xa = __float_as_uint(x[i]) & 0xffff0000u;
        const float r1 = x[i] - __uint_as_float(xa);
        const uint32_t xb = __float_as_uint(r1) & 0xffff0000u;
        const float r2 = r1 - __uint_as_float(xb);
        a[i] = xa; b[i] = xb; c[i] = __float_as_uint(r2) & 0xffff0000u;
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        t0[d] = (a[2 * d] >> 16) | a[2 * d + 1];
        t1[d] = (b[2 * d] >> 16) | b[2 * d + 1];
        t2[d] = (c[2 * d] >> 16) | c[2 * d + 1];
    }
}

// BITS: packing class of the codes (1, 2, 3, 4, or 8 = one code per byte for 5..7 bits)
template <int DTYPE, int BITS>
__global__ __launch_bounds__(QTHREADS, 2) void tq_qjl_residual_kernel(QjlArgs a) {
    constexpr int ELEM = DTYPE == TQ_F32 ? 4 : 2;
    constexpr int IPB = 8 / BITS;
    constexpr int NB = 16 / IPB;           // packed bytes of 16 codes
    constexpr int G = 8 * NB;              // packed bytes per vector
    constexpr int TILE = 32 * TQ_HEAD_DIM * 2;   // one bf16 term of a 32-vector tile: 8 KiB

    __shared__ __attribute__((aligned(16))) uint8_t lds_terms[3][TILE];   // centroid terms, then residual terms
    __shared__ float lds_cent[256];
    __shared__ float lds_n2[4][32];        // shares of ||x||^2
    __shared__ float lds_r2[4][32];        // shares of ||residual||^2

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = tq_uniform32(tid >> 6);
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const TqQjlHeader *hd = reinterpret_cast<const TqQjlHeader *>(a.table);

    // ---- this wave's rows of Pi^T and S, resident for the whole kernel
    tq_u4 a_pit[3][TQ_STEPS], a_s[2][TQ_STEPS];
    {
        const uint8_t *pit = a.table + hd->off_pit, *sm = a.table + hd->off_s;
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            const size_t o = (((size_t)wave * TQ_STEPS + s) * 64 + lane) * 16;
#pragma unroll
            for (int q = 0; q < 3; ++q) a_pit[q][s] = tq_gload16(pit + (size_t)q * TQ_OPERAND_BYTES + o);
#pragma unroll
            for (int q = 0; q < 2; ++q) a_s[q][s] = tq_gload16(sm + (size_t)q * TQ_OPERAND_BYTES + o);
        }
    }
    for (uint32_t i = tid; i < 256u; i += QTHREADS)
        lds_cent[i] = i < hd->levels ? *reinterpret_cast<const TQ_GLOBAL float *>((const TQ_GLOBAL uint8_t *)(a.table + hd->off_centroids) + 4u * i) : 0.f;
    __syncthreads();

    const uint32_t n_tiles = (a.n_vec + 31u) / 32u;
    const uint32_t dv = tid >> 3, seg = tid & 7u;            // role in the decode: vector of the tile, 16-code segment
    const uint32_t code_mask = (1u << a.mse_bits) - 1u;
    // the lane's 16 coordinates [32w + 16hk, +16) of vector n are pieces 4w + 2hk and 4w + 2hk + 1 of its row
    const uint32_t my_piece = 4u * wave + 2u * hk;

    for (uint32_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        // ---- (1) codes -> centroids -> three bf16 terms in LDS (vector dv, codes [16 seg, 16 seg + 16))
        {
            uint32_t v = tile * 32u + dv;
            v = v < a.n_vec ? v : a.n_vec - 1u;              // tail: the last vector again, never stored
            const uint8_t *src = a.idx_bytes + (size_t)v * G + seg * NB;
            uint32_t raw[4] = {0u, 0u, 0u, 0u};
            if constexpr (NB == 2) raw[0] = tq_gload2(reinterpret_cast<const uint16_t *>(src));
            else if constexpr (NB == 4) raw[0] = *reinterpret_cast<const TQ_GLOBAL uint32_t *>((const TQ_GLOBAL uint8_t *)src);
            else if constexpr (NB == 8) { const tq_u2 t = tq_gload8(src); raw[0] = t[0]; raw[1] = t[1]; }
            else { const tq_u4 t = tq_gload16(src); raw[0] = t[0]; raw[1] = t[1]; raw[2] = t[2]; raw[3] = t[3]; }
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                float c[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int k = 8 * half + i;                       // code number inside the segment
                    const int byte = k / IPB, pos = k % IPB;
                    const uint32_t bv = (raw[byte / 4] >> (8 * (byte % 4))) & 0xffu;
                    const uint32_t code = (bv >> (BITS * (IPB - 1 - pos))) & code_mask;
                    c[i] = lds_cent[code];
                }
                tq_u4 t0, t1, t2;
                qsplit8(c, t0, t1, t2);
                const uint32_t off = dv * 256u + (((2u * seg + half) ^ (dv & 15u)) << 4);
                *reinterpret_cast<tq_u4 *>(lds_terms[0] + off) = t0;
                *reinterpret_cast<tq_u4 *>(lds_terms[1] + off) = t1;
                *reinterpret_cast<tq_u4 *>(lds_terms[2] + off) = t2;
            }
        }
        // ---- the lane's 16 input coordinates, and its share of ||x||^2
        float x[16];
        {
            uint32_t v = tile * 32u + n;
            v = v < a.n_vec ? v : a.n_vec - 1u;
            const uint8_t *src = a.states + (long long)v * a.token_stride + (32u * wave + 16u * hk) * ELEM;
            if constexpr (ELEM == 4) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const tq_u4 t = tq_gload16(src + 16 * q);
#pragma unroll
                    for (int i = 0; i < 4; ++i) x[4 * q + i] = __uint_as_float(t[i]);
                }
            } else {
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const tq_u4 t = tq_gload16(src + 16 * q);
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
            for (int i = 0; i < 3; ++i) {
                const tq_u4 bop = *reinterpret_cast<const tq_u4 *>(lds_terms[i] + off);
#pragma unroll
                for (int j = 0; i + j < 3; ++j) acc = qmfma(a_pit[j][s], bop, acc);
            }
        }
        const float nrm = sqrtf((lds_n2[0][n] + lds_n2[1][n]) + (lds_n2[2][n] + lds_n2[3][n]));
        // ---- (3) residual, its norm, its three bf16 terms
        float r[16];
        float r2 = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float km = acc[i] * nrm;
            r[i] = x[i] - km;
            r2 = fmaf(r[i], r[i], r2);
        }
        r2 += __shfl_xor(r2, 32);
        lds_r2[wave][n] = r2;
        __syncthreads();                   // everybody has read the centroid terms
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float c[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) c[i] = r[8 * half + i];
            tq_u4 t0, t1, t2;
            qsplit8(c, t0, t1, t2);
            const uint32_t off = n * 256u + (((my_piece + half) ^ (n & 15u)) << 4);
            *reinterpret_cast<tq_u4 *>(lds_terms[0] + off) = t0;
            *reinterpret_cast<tq_u4 *>(lds_terms[1] + off) = t1;
            *reinterpret_cast<tq_u4 *>(lds_terms[2] + off) = t2;
        }
        __syncthreads();

        // ---- (4) projection by S, signs, stores
        tq_f16v prj = tq_zero16();
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            const uint32_t off = n * 256u + (((2u * s + hk) ^ (n & 15u)) << 4);
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                const tq_u4 bop = *reinterpret_cast<const tq_u4 *>(lds_terms[i] + off);
#pragma unroll
                for (int j = 0; j < 2 && i + j < 3; ++j) prj = qmfma(a_s[j][s], bop, prj);
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
