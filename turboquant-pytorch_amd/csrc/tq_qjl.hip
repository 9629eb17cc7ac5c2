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
#include <type_traits>

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
    // x - hi written as a fused multiply-add with the 16-bit operand widened inside the instruction (same value: one rounding)
    const pk_half2 l = __builtin_amdgcn_cvt_pkrtz(__builtin_fmaf((float)h[0], -1.0f, x0), __builtin_fmaf((float)h[1], -1.0f, x1));
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

// ====================================================================================================================
// One-pass form of the V2 key path for 16-bit inputs and MSE codes of up to 4 bits: codes, norms, residual signs and
// residual norms from a single read of the input (upstream turboquant/compressors.py:84-122 in one kernel).
//
// The kernel is the pipelined compress kernel (csrc/tq_compress.hip: tiles of 32 vectors shared by the four waves of
// a block, the rotation resident in registers, the input travelling straight into an LDS ring, code search through the
// threshold grid) with two more stages behind the search:
//   * the residual in ROTATED coordinates, which is an elementwise expression of what the search already holds:
//     (Pi residual)[k] = (Pi x)[k] - ||x|| * centroid(code_k)   (the centroids of a lane's packed bytes come from a
//     byte -> floats table in LDS, one lookup per byte), its squared norm, and its two fp16 terms (scaled by a power of
//     two taken from the norm's exponent) parked in LDS in the tile layout of the input;
//   * the projection by M = S Pi^T (resident in registers as two fp16 terms, like the rotation) of the residual tile
//     parked an iteration earlier: three matrix passes (hi*hi, lo*hi, hi*lo; the fourth weighs 2^-22), the signs of
//     the 16 projections of a lane packed into the two bytes it owns.
// Iteration j of a block therefore rotates tile j, searches tile j-1 and projects tile j-2, with one barrier.
// Against the float32 arithmetic of the reference the projections differ by the rotation's own error (2^-17 of the
// vector per coordinate for bf16 inputs, seen through the ratio ||x|| / ||residual||, which is why codes wider than
// 4 bits keep the two-kernel form) and by the rotation's departure from orthogonality (1e-7).
struct TqQjlDevJob {
    const uint8_t *states;
    uint8_t *idx_bytes;
    uint16_t *vec_norms;
    uint8_t *sign_bytes;
    uint16_t *residual_norm;
    const uint8_t *table;        // codec table of the MSE stage (tq_table_build)
    const uint8_t *qjl_table;    // tq_qjl_table_build
    uint32_t n_vec;
    long long token_stride;      // bytes
};

__device__ __forceinline__ TqQjlDevJob load_qjl_job(const TqQjlDevJob &single, const tq_qjl_job *jobs, uint32_t index, int elem_bytes) {
    TqQjlDevJob j = single;
    if (jobs) {
        const tq_qjl_job &s = jobs[index];
        j.states = static_cast<const uint8_t *>(s.states);
        j.idx_bytes = s.idx_bytes;
        j.vec_norms = s.vec_norms;
        j.sign_bytes = s.sign_bytes;
        j.residual_norm = s.residual_norm;
        j.table = static_cast<const uint8_t *>(s.table_dev);
        j.qjl_table = static_cast<const uint8_t *>(s.qjl_table_dev);
        j.n_vec = (uint32_t)s.n_vec;
        j.token_stride = s.token_stride * elem_bytes;
    }
    TqQjlDevJob u;
    u.states = reinterpret_cast<const uint8_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.states));
    u.idx_bytes = reinterpret_cast<uint8_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.idx_bytes));
    u.vec_norms = reinterpret_cast<uint16_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.vec_norms));
    u.sign_bytes = reinterpret_cast<uint8_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.sign_bytes));
    u.residual_norm = reinterpret_cast<uint16_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.residual_norm));
    u.table = reinterpret_cast<const uint8_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.table));
    u.qjl_table = reinterpret_cast<const uint8_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.qjl_table));
    u.n_vec = tq_uniform32(j.n_vec);
    u.token_stride = (long long)tq_uniform64((uint64_t)j.token_stride);
    return u;
}

template <int BITS>
struct FusedLds {
    static constexpr uint32_t TILE = 32 * TQ_HEAD_DIM * 2;
    static constexpr uint32_t STAGE_OFF = 0, RES_OFF = STAGE_OFF + 2 * TILE, GRID_OFF = RES_OFF + 4 * TILE;
    static constexpr uint32_t LUT_OFF = GRID_OFF + TQ_GRID_LDS_BYTES, PART_OFF = LUT_OFF + 256 * (8 / BITS) * 4;
    static constexpr uint32_t R2_OFF = PART_OFF + 2 * 32 * 4 * 4, UNSCALE_OFF = R2_OFF + 2 * 32 * 4 * 4, BYTES = UNSCALE_OFF + 2 * 32 * 4;
};

// BITS: packing class of the MSE codes: 1, 2, 3 or 4
template <int DTYPE, int BITS>
__global__ __launch_bounds__(QTHREADS, 2) void tq_qjl_fused_kernel(TqQjlDevJob job0, const tq_qjl_job *jobs) {
    using P = Pack<BITS>;
    static_assert(DTYPE == TQ_F16 || DTYPE == TQ_BF16, "16-bit inputs");
    static_assert(BITS >= 1 && BITS <= 4, "codes of up to 4 bits");
    constexpr int NB = P::NB, NW = P::NW, IPB = P::IPB;
    constexpr int VEC_BYTES = TQ_HEAD_DIM * 2;
    constexpr int STAGE = 32 * VEC_BYTES;       // one tile of 16-bit values: 8 KiB
    constexpr int NLOAD = 2;                    // direct-to-LDS loads per wave and tile

    // LDS (dynamic: more than the 64 KiB a kernel may declare statically): input ring | residual terms | grid | tables | shares
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds_all[];
    using L = FusedLds<BITS>;
    uint8_t (*lds_stage)[STAGE] = reinterpret_cast<uint8_t (*)[STAGE]>(lds_all + L::STAGE_OFF);
    uint8_t (*lds_res)[2][STAGE] = reinterpret_cast<uint8_t (*)[2][STAGE]>(lds_all + L::RES_OFF);            // [tile parity][term] of the residual
    uint8_t *lds_grid = lds_all + L::GRID_OFF;
    float *lds_lut = reinterpret_cast<float *>(lds_all + L::LUT_OFF);                                     // packed byte -> the centroids of its codes
    float (*lds_part)[32][4] = reinterpret_cast<float (*)[32][4]>(lds_all + L::PART_OFF);                 // shares of ||x||^2
    float (*lds_r2)[32][4] = reinterpret_cast<float (*)[32][4]>(lds_all + L::R2_OFF);                     // shares of ||scaled residual||^2
    float (*lds_unscale)[32] = reinterpret_cast<float (*)[32]>(lds_all + L::UNSCALE_OFF);                 // 1 / the residual's scale

    const TqQjlDevJob job = load_qjl_job(job0, jobs, blockIdx.y, 2);
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = tq_uniform32(tid >> 6);
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const uint32_t n_full = job.n_vec / 32u;        // the ragged end of a job is the caller's (two-kernel form)
    if (blockIdx.x >= n_full) return;
    const uint32_t m = (n_full - blockIdx.x + gridDim.x - 1u) / gridDim.x;     // this block's tiles: blockIdx.x + k * gridDim.x
    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(job.table);
    const TqQjlHeader *qh = reinterpret_cast<const TqQjlHeader *>(job.qjl_table);

    // ---- loads of a tile: lane i of load l fills bytes [16 i, 16 i + 16) of KiB (wave * NLOAD + l) of the slot, i.e.
    // vector vl = (wave * NLOAD + l) * 4 + i / 16, position i % 16, which has to hold piece (i % 16) ^ (vl & 15)
    uint32_t src_off[NLOAD];
#pragma unroll
    for (int l = 0; l < NLOAD; ++l) {
        const uint32_t vl = (wave * NLOAD + l) * 4u + (lane >> 4);
        src_off[l] = vl * (uint32_t)job.token_stride + (((lane & 15u) ^ (vl & 15u)) << 4);
    }
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)(lds_all + L::STAGE_OFF) + wave * (NLOAD * 1024u));
    auto tile_of = [&](uint32_t j) { return blockIdx.x + (j < m ? j : m - 1u) * gridDim.x; };      // past the end: the last tile again
    auto issue = [&](uint32_t slot, uint32_t tl) {
        const uint64_t a = (uint64_t)(uintptr_t)job.states + (uint64_t)tl * (uint64_t)(32 * job.token_stride);
        const uint32_t a_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
        const uint32_t a_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)a);
        const uint64_t base = ((uint64_t)a_hi << 32) | (uint64_t)a_lo;
#pragma unroll
        for (int l = 0; l < NLOAD; ++l) {
            const uint32_t dst = lds_wave + slot * (uint32_t)STAGE + l * 1024u;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         :: "s"(dst), "v"(src_off[l]), "s"(base) : "memory", "m0");
        }
    };
    issue(0u, tile_of(0u));

    // ---- resident operands: this wave's 32 rows of the rotation (walked in the step order 2w, 2w+1, ... of the
    // compress kernel, so that a vector gets the same norm from both) and of M, two 16-bit terms each
    const uint32_t step0 = 2u * wave;
    tq_u4 areg[2][TQ_STEPS], mreg[2][TQ_STEPS];
    {
        const uint8_t *src = job.table + (DTYPE == TQ_F16 ? hd->off_a_f16 : hd->off_a_bf16);
        const uint8_t *msrc = job.qjl_table + qh->off_m;
#pragma unroll
        for (int term = 0; term < 2; ++term)
#pragma unroll
            for (int s = 0; s < TQ_STEPS; ++s) {
                areg[term][s] = tq_gload16(src + (size_t)term * TQ_OPERAND_BYTES + (((size_t)wave * TQ_STEPS + ((s + step0) & 7u)) * 64 + lane) * 16);
                mreg[term][s] = tq_gload16(msrc + (size_t)term * TQ_OPERAND_BYTES + (((size_t)wave * TQ_STEPS + s) * 64 + lane) * 16);
            }
    }
    {   // quantiser grid: one copy per position of a code in a word, base pre-shifted (as in the compress kernel)
        const uint32_t cells = hd->grid_cells;
        const uint8_t *gsrc = job.table + hd->off_grid;
        for (uint32_t q = tid; q < cells; q += QTHREADS) {
            const tq_u2 cell = tq_gload8(gsrc + 8u * q);
#pragma unroll
            for (int c = 0; c < P::COPIES; ++c) {
                const tq_u2 e = {cell[0], cell[1] << copy_shift_rt<BITS>(c)};
                *reinterpret_cast<tq_u2 *>(lds_grid + c * P::COPY_STRIDE + 8u * q) = e;
            }
        }
        const float *cent = reinterpret_cast<const float *>(job.qjl_table + qh->off_cent_f32);
        constexpr uint32_t CODE_MASK = BITS == 3 ? 7u : (1u << BITS) - 1u;
        for (uint32_t e = tid; e < 256u * IPB; e += QTHREADS) {
            const uint32_t v = e / IPB, pos = e % IPB;
            const uint32_t code = (v >> (BITS * (IPB - 1 - pos))) & CODE_MASK;
            lds_lut[e] = *reinterpret_cast<const TQ_GLOBAL float *>((const TQ_GLOBAL uint8_t *)cent + 4u * code);
        }
    }
    const float grid_scale = hd->grid_scale, grid_bias = hd->grid_bias;

    // operand addresses inside a tile: rotation in this wave's step order, projection in the natural one
    uint32_t op_rot[TQ_STEPS], op_prj[TQ_STEPS];
#pragma unroll
    for (int i = 0; i < TQ_STEPS; ++i) {
        op_rot[i] = n * VEC_BYTES + (((2u * ((i + step0) & 7u) + hk) ^ (n & 15u)) << 4);
        op_prj[i] = n * VEC_BYTES + (((2u * i + hk) ^ (n & 15u)) << 4);
    }
    const uint32_t bperm_other_half = (lane ^ 32u) << 2;
    const uint32_t my_piece = 4u * wave + 2u * hk;      // the lane's 16 coordinates are pieces my_piece, my_piece + 1 of its row
    const uint32_t lane_slot = (2u * wave + hk) * NB;   // its bytes inside a vector's G = 8 * NB

    struct Scale { float nrm, inv, inv_cell; };
    auto scale_from_shares = [&](uint32_t par) {
        const float4 q = *reinterpret_cast<const float4 *>(&lds_part[par][n][0]);
        Scale sc;
        sc.nrm = tq_norm_from_sumsq((q.x + q.y) + (q.z + q.w));
        sc.inv = __builtin_amdgcn_rcpf(sc.nrm + 1e-8f);
        if (DTYPE == TQ_F16) sc.inv *= 1.0f / (float)(1 << TQ_F16_PI_SHIFT);
        sc.inv_cell = sc.inv * grid_scale;
        return sc;
    };

    // iteration j: ROT: tile j into `acc_new`; SEARCH: tile j-1 from `acc_old`; PROJECT: tile j-2.  par = j & 1.
    auto iteration = [&](auto rot_tag, auto search_tag, auto project_tag, auto par_tag, uint32_t j, tq_f16v &acc_new, const tq_f16v &acc_old) {
        constexpr bool ROT = decltype(rot_tag)::value, SEARCH = decltype(search_tag)::value, PROJECT = decltype(project_tag)::value;
        constexpr uint32_t PAR = decltype(par_tag)::value;
        // this wave's loads of tile j, issued at the start of the iteration before.  Younger than them are only that
        // iteration's stores (codes and norm of a searched tile, the signs of a projected one; the residual norm, which
        // wave 0 alone stores, comes last): two of them in iteration 1, three from then on, and they may stay in flight
        // (which measures the same as waiting for them: the kernel is bound by its matrix and vector instructions).
        // A third ring slot, which would let the loads run two iterations ahead, costs the second block of a compute
        // unit its LDS and a third of the rate.
        if (j >= 3u) wait_vmcnt<3>(); else if (j == 2u) wait_vmcnt<2>(); else wait_vmcnt<0>();
        __syncthreads();
        if constexpr (ROT) issue(PAR ^ 1u, tile_of(j + 1u));
        const uint8_t *stage = lds_stage[PAR];
        const uint8_t *res_hi = lds_res[PAR][0], *res_lo = lds_res[PAR][1];       // tile j-2 has the parity of j
        tq_f16v prj = tq_zero16();
        if constexpr (ROT) acc_new = tq_zero16();
        uint32_t lt[NW], lo[NW];
#pragma unroll
        for (int w = 0; w < NW; ++w) lt[w] = lo[w] = 0u;
        Scale sc{};
        if constexpr (SEARCH) sc = scale_from_shares(PAR ^ 1u);
        float share = 0.f;
#pragma unroll
        for (int i = 0; i < TQ_STEPS; ++i) {
            if constexpr (ROT) {
                const tq_u4 bop = *reinterpret_cast<const tq_u4 *>(stage + op_rot[i]);
                acc_new = (DTYPE == TQ_F16) ? mfma_f16(areg[0][i], bop, acc_new) : mfma_bf16(areg[0][i], bop, acc_new);
                if (i < 2) share = sumsq8<DTYPE>(bop, share);
                acc_new = (DTYPE == TQ_F16) ? mfma_f16(areg[1][i], bop, acc_new) : mfma_bf16(areg[1][i], bop, acc_new);
                if (i == 1) {
                    share += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((int)bperm_other_half, __builtin_bit_cast(int, share)));
                    lds_part[PAR][n][wave] = share;
                }
            }
            if constexpr (SEARCH) {
#pragma unroll
                for (int q = 2 * i; q < 2 * i + 2; ++q) {      // coordinates in the order (word, position in word)
                    const int w = q / P::CPW, c = q % P::CPW;
                    const float a = acc_old[P::local_code(w, c)];
                    const uint32_t addr = __float_as_uint(fmaf(a, sc.inv_cell, grid_bias)) & TQ_GRID_ADDR_MASK;
                    const tq_u2 cell = *reinterpret_cast<const tq_u2 *>(lds_grid + P::copy_of(c) * P::COPY_STRIDE + addr);
                    const float t = fmaf(a, sc.inv, -__uint_as_float(cell[0]));
                    const int cursor = c == 0 ? 8 * P::WB : P::shift_of(c - 1);
                    const int gap = cursor - (P::shift_of(c) + P::FIELD);
                    if (gap > 0) lt[w] = __builtin_amdgcn_alignbit(lt[w], 0u, 32 - gap);
                    lt[w] = __builtin_amdgcn_alignbit(lt[w], __float_as_uint(t), 32 - P::FIELD);
                    lo[w] |= cell[1];
                }
            }
            if constexpr (PROJECT) {
                const tq_u4 bh = *reinterpret_cast<const tq_u4 *>(res_hi + op_prj[i]);
                const tq_u4 bl = *reinterpret_cast<const tq_u4 *>(res_lo + op_prj[i]);
                prj = mfma_f16(mreg[0][i], bh, prj);
                prj = mfma_f16(mreg[1][i], bh, prj);
                prj = mfma_f16(mreg[0][i], bl, prj);
            }
        }
        if constexpr (SEARCH) {
            const uint32_t tl = tile_of(j - 1u);
            uint32_t words[NW];
#pragma unroll
            for (int w = 0; w < NW; ++w) words[w] = lo[w] + ((~lt[w] & P::sign_mask()) >> (P::FIELD - 1));
            uint8_t *dst = job.idx_bytes + ((size_t)tl * 32u + n) * (8 * NB) + lane_slot;
            if constexpr (NB == 2) tq_gstore2(reinterpret_cast<uint16_t *>(dst), (uint16_t)words[0]);
            else if constexpr (NB == 4) *reinterpret_cast<TQ_GLOBAL uint32_t *>((TQ_GLOBAL uint8_t *)dst) = words[0];
            else { const tq_u2 o = {words[0], words[1]}; tq_gstore8(dst, o); }
            const _Float16 hn = (_Float16)sc.nrm;
            tq_gstore2(job.vec_norms + (size_t)tl * 32u + n, __builtin_bit_cast(uint16_t, hn));

            // ---- the residual in rotated coordinates.  Scale: 2^(10 - E) for ||x|| = f * 2^E, f in [0.5, 1): the scaled
            // residual (|r_k| <= 2 ||x||) stays inside the fp16 range, and ||x|| times the scale is below 2^10.
            uint32_t r_exp = 263u - ((__float_as_uint(sc.nrm) >> 23) & 0xffu);
            r_exp = r_exp > 254u ? 254u : r_exp;
            const float r_scale = __uint_as_float(r_exp << 23);
            const float a_scale = DTYPE == TQ_F16 ? r_scale * (1.0f / (float)(1 << TQ_F16_PI_SHIFT)) : r_scale;
            const float n_scaled = sc.nrm * r_scale;
            float r[16];
#pragma unroll
            for (int b = 0; b < NB; ++b) {      // byte b of the lane: its codes are coordinates b * IPB ...
                const uint32_t v = (words[b / 4] >> (8 * (b % 4))) & 0xffu;
                const float *e = lds_lut + v * IPB;
                if constexpr (IPB == 8) {
                    const float4 c0 = *reinterpret_cast<const float4 *>(e), c1 = *reinterpret_cast<const float4 *>(e + 4);
                    const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
#pragma unroll
                    for (int p = 0; p < 8; ++p) r[8 * b + p] = fmaf(acc_old[8 * b + p], a_scale, -(c[p] * n_scaled));
                } else if constexpr (IPB == 4) {
                    const float4 c0 = *reinterpret_cast<const float4 *>(e);
                    const float c[4] = {c0.x, c0.y, c0.z, c0.w};
#pragma unroll
                    for (int p = 0; p < 4; ++p) r[4 * b + p] = fmaf(acc_old[4 * b + p], a_scale, -(c[p] * n_scaled));
                } else {
                    const float2 c0 = *reinterpret_cast<const float2 *>(e);
                    r[2 * b] = fmaf(acc_old[2 * b], a_scale, -(c0.x * n_scaled));
                    r[2 * b + 1] = fmaf(acc_old[2 * b + 1], a_scale, -(c0.y * n_scaled));
                }
            }
            float r2 = 0.f;
#pragma unroll
            for (int k = 0; k < 16; ++k) r2 = fmaf(r[k], r[k], r2);
            r2 += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((int)bperm_other_half, __builtin_bit_cast(int, r2)));
            lds_r2[PAR ^ 1u][n][wave] = r2;
            if (wave == 0) lds_unscale[PAR ^ 1u][n] = __uint_as_float((254u - r_exp) << 23);
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                tq_u4 t0, t1;
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const TermPair t = split_pair(r[8 * half + 2 * d], r[8 * half + 2 * d + 1]);
                    t0[d] = t.hi;
                    t1[d] = t.lo;
                }
                const uint32_t off = n * VEC_BYTES + (((my_piece + half) ^ (n & 15u)) << 4);
                *reinterpret_cast<tq_u4 *>(lds_res[PAR ^ 1u][0] + off) = t0;
                *reinterpret_cast<tq_u4 *>(lds_res[PAR ^ 1u][1] + off) = t1;
            }
        }
        if constexpr (PROJECT) {
            const uint32_t tl = tile_of(j - 2u);
            // byte 0: coordinates 0..7 of the lane, most significant bit first; byte 1: 8..15.  The sign bits are shifted
            // in one instruction each (8..15 first, so that they end up in the upper byte) and inverted at the end: a
            // sum that starts from +0 is never -0, so "sign bit clear" is ">= 0".
            uint32_t neg = 0;
#pragma unroll
            for (int k = 0; k < 16; ++k) neg = __builtin_amdgcn_alignbit(neg, __float_as_uint(prj[(k + 8) & 15]), 31);
            const uint32_t word = ~neg;
            const size_t v = (size_t)tl * 32u + n;
            tq_gstore2(reinterpret_cast<uint16_t *>(job.sign_bytes + v * 16u + 4u * wave + 2u * hk), (uint16_t)word);
            if (wave == 0) {
                const float4 q = *reinterpret_cast<const float4 *>(&lds_r2[PAR][n][0]);
                const float rn = sqrtf((q.x + q.y) + (q.z + q.w)) * lds_unscale[PAR][n];
                const _Float16 h = (_Float16)rn;
                tq_gstore2(job.residual_norm + v, __builtin_bit_cast(uint16_t, h));
            }
        }
    };

    using T = std::true_type;
    using F = std::false_type;
    using P0 = std::integral_constant<uint32_t, 0>;
    using P1 = std::integral_constant<uint32_t, 1>;
    tq_f16v acc_a, acc_b;
    // iteration j rotates while j < m, searches while 1 <= j <= m, projects while 2 <= j <= m + 1
    iteration(T{}, F{}, F{}, P0{}, 0u, acc_a, acc_a);
    if (m > 1u) iteration(T{}, T{}, F{}, P1{}, 1u, acc_b, acc_a);
    else iteration(F{}, T{}, F{}, P1{}, 1u, acc_b, acc_a);
    uint32_t j = 2;
    for (; j + 1u < m; j += 2u) {
        iteration(T{}, T{}, T{}, P0{}, j, acc_a, acc_b);
        iteration(T{}, T{}, T{}, P1{}, j + 1u, acc_b, acc_a);
    }
    // what is left: j == m - 1 (one more tile to rotate), then the two iterations that only finish tiles
    if (j < m) {
        iteration(T{}, T{}, T{}, P0{}, j, acc_a, acc_b);
        ++j;
    }
    if (m > 1u) {       // j == m: search tile m - 1, project tile m - 2
        if (j & 1u) iteration(F{}, T{}, T{}, P1{}, j, acc_b, acc_a);
        else iteration(F{}, T{}, T{}, P0{}, j, acc_a, acc_b);
        ++j;
    }
    if (j & 1u) iteration(F{}, F{}, T{}, P1{}, j, acc_b, acc_a);          // j == m + 1: project tile m - 1
    else iteration(F{}, F{}, T{}, P0{}, j, acc_a, acc_b);
    wait_vmcnt<0>();       // the re-read past the last tile may still be on its way into the ring
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

// ---- the one-pass form: host side ------------------------------------------------------------------------------------
namespace {

template <int DTYPE, int BITS>
int launch_fused(const TqQjlDevJob &job, const tq_qjl_job *jobs_dev, int n_jobs, uint32_t max_tiles, hipStream_t stream) {
    static int slots[MAX_DEVICES] = {};     // blocks the device holds at once (0: not asked yet)
    constexpr uint32_t lds = FusedLds<BITS>::BYTES;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return TQ_ERR_NO_DEVICE;
    int resident;
    {
        std::lock_guard<std::mutex> lock(host_state_mutex);
        if (slots[dev] == 0) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(&tq_qjl_fused_kernel<DTYPE, BITS>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            int cus = 0, per_cu = 0;
            e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e != hipSuccess) return (int)e;
            e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, tq_qjl_fused_kernel<DTYPE, BITS>, QTHREADS, lds);
            if (e != hipSuccess) return (int)e;
            slots[dev] = (cus > 0 ? cus : 1) * (per_cu > 0 ? per_cu : 1);
        }
        resident = slots[dev];
    }
    const uint32_t bx = tq_blocks_per_job(max_tiles, resident, n_jobs);
    hipLaunchKernelGGL((tq_qjl_fused_kernel<DTYPE, BITS>), dim3(bx, (unsigned)n_jobs, 1), dim3(QTHREADS), lds, stream, job, jobs_dev);
    return (int)hipGetLastError();
}

template <int DTYPE>
int fused_bits(int mse_bits, const TqQjlDevJob &job, const tq_qjl_job *jobs_dev, int n_jobs, uint32_t max_tiles, hipStream_t s) {
    switch (mse_bits) {
        case 1: return launch_fused<DTYPE, 1>(job, jobs_dev, n_jobs, max_tiles, s);
        case 2: return launch_fused<DTYPE, 2>(job, jobs_dev, n_jobs, max_tiles, s);
        case 3: return launch_fused<DTYPE, 3>(job, jobs_dev, n_jobs, max_tiles, s);
        case 4: return launch_fused<DTYPE, 4>(job, jobs_dev, n_jobs, max_tiles, s);
        default: return TQ_ERR_BITS;
    }
}

bool one_pass_takes(int dtype, int mse_bits) {
    return (dtype == TQ_F16 || dtype == TQ_BF16) && mse_bits >= 1 && mse_bits <= TQ_QJL_ONE_PASS_MAX_BITS;
}

int check_qjl_job(const tq_qjl_job &j, int head_dim) {
    if (j.mse_bits < 1 || j.mse_bits > 7) return TQ_ERR_BITS;
    if (head_dim != TQ_HEAD_DIM) return TQ_ERR_HEAD_DIM;
    const int eb = j.dtype == TQ_F32 ? 4 : (j.dtype == TQ_F16 || j.dtype == TQ_BF16) ? 2 : 0;
    if (!eb) return TQ_ERR_DTYPE;
    if (j.n_vec < 0 || j.n_vec > 0x7fffffffll) return TQ_ERR_SIZE;
    if (j.n_vec == 0) return TQ_OK;
    if (!j.states || !j.idx_bytes || !j.vec_norms || !j.sign_bytes || !j.residual_norm || !j.table_dev || !j.qjl_table_dev) return TQ_ERR_NULL;
    if (j.token_stride < TQ_HEAD_DIM && j.n_vec > 1) return TQ_ERR_SIZE;
    if (j.token_stride * eb >= (1ll << 26)) return TQ_ERR_SIZE;
    if (((uintptr_t)j.states & 15u) || ((uintptr_t)j.idx_bytes & 15u) || ((uintptr_t)j.table_dev & 15u) || ((uintptr_t)j.qjl_table_dev & 15u) ||
        ((uintptr_t)j.sign_bytes & 15u) || ((uintptr_t)j.vec_norms & 1u) || ((uintptr_t)j.residual_norm & 1u) || ((j.token_stride * eb) & 15))
        return TQ_ERR_ALIGN;
    return TQ_OK;
}

// the two-kernel form on vectors [first, n_vec) of a job
int two_kernels(const tq_qjl_job &j, long long first, int head_dim, void *stream) {
    const long long n = j.n_vec - first;
    if (n <= 0) return TQ_OK;
    const int eb = j.dtype == TQ_F32 ? 4 : 2;
    const int g = tq_bytes_per_vector(head_dim, j.mse_bits);
    if (g < 0) return g;
    const uint8_t *x = static_cast<const uint8_t *>(j.states) + first * j.token_stride * eb;
    uint8_t *idx = j.idx_bytes + first * g;
    int rc = tq_compress(x, j.dtype, 1, n, 0, j.token_stride, j.table_dev, head_dim, j.mse_bits, idx, j.vec_norms + first, 0, nullptr, stream);
    if (rc) return rc;
    return tq_qjl_signs(x, j.dtype, n, j.token_stride, idx, j.qjl_table_dev, head_dim, j.mse_bits,
                        j.sign_bytes + first * 16, j.residual_norm + first, stream);
}

}  // namespace

extern "C" int tq_qjl_compress_batched(const tq_qjl_job *jobs_host, const tq_qjl_job *jobs_dev, int n_jobs, int head_dim, void *stream) {
    if (n_jobs == 0) return TQ_OK;
    if (!jobs_host) return TQ_ERR_NULL;
    if (n_jobs < 0 || n_jobs > TQ_MAX_JOBS) return TQ_ERR_SIZE;
    long long max_vec = 0;
    for (int i = 0; i < n_jobs; ++i) {
        if (jobs_host[i].mse_bits != jobs_host[0].mse_bits) return TQ_ERR_BITS;
        if (jobs_host[i].dtype != jobs_host[0].dtype) return TQ_ERR_DTYPE;
        const int rc = check_qjl_job(jobs_host[i], head_dim);
        if (rc) return rc;
        if (jobs_host[i].n_vec > max_vec) max_vec = jobs_host[i].n_vec;
    }
    if (max_vec == 0) return TQ_OK;
    const bool one_pass = one_pass_takes(jobs_host[0].dtype, jobs_host[0].mse_bits);
    if (one_pass && max_vec >= 32) {
        if (!jobs_dev) return TQ_ERR_NULL;
        TqQjlDevJob none{};
        const uint32_t tiles = (uint32_t)(max_vec / 32);
        const hipStream_t s = static_cast<hipStream_t>(stream);
        const int rc = jobs_host[0].dtype == TQ_F16 ? fused_bits<TQ_F16>(jobs_host[0].mse_bits, none, jobs_dev, n_jobs, tiles, s)
                                                    : fused_bits<TQ_BF16>(jobs_host[0].mse_bits, none, jobs_dev, n_jobs, tiles, s);
        if (rc) return rc;
    }
    // what the one-pass kernel leaves: the ragged end of every job (fewer than 32 vectors), or everything
    for (int i = 0; i < n_jobs; ++i) {
        const long long done = one_pass ? jobs_host[i].n_vec / 32 * 32 : 0;
        const int rc = two_kernels(jobs_host[i], done, head_dim, stream);
        if (rc) return rc;
    }
    return TQ_OK;
}

extern "C" int tq_qjl_compress(const void *states, int dtype, long long n_vec, long long token_stride, const void *table_dev,
                               const void *qjl_table_dev, int head_dim, int mse_bits, uint8_t *idx_bytes, uint16_t *vec_norms,
                               uint8_t *sign_bytes, uint16_t *residual_norm, void *stream) {
    tq_qjl_job j{};
    j.states = states;
    j.idx_bytes = idx_bytes;
    j.vec_norms = vec_norms;
    j.sign_bytes = sign_bytes;
    j.residual_norm = residual_norm;
    j.table_dev = table_dev;
    j.qjl_table_dev = qjl_table_dev;
    j.n_vec = n_vec;
    j.token_stride = token_stride;
    j.mse_bits = mse_bits;
    j.dtype = dtype;
    const int rc = check_qjl_job(j, head_dim);
    if (rc || n_vec == 0) return rc;
    long long done = 0;
    if (one_pass_takes(dtype, mse_bits) && n_vec >= 32) {
        TqQjlDevJob d;
        d.states = static_cast<const uint8_t *>(states);
        d.idx_bytes = idx_bytes;
        d.vec_norms = vec_norms;
        d.sign_bytes = sign_bytes;
        d.residual_norm = residual_norm;
        d.table = static_cast<const uint8_t *>(table_dev);
        d.qjl_table = static_cast<const uint8_t *>(qjl_table_dev);
        d.n_vec = (uint32_t)n_vec;
        d.token_stride = token_stride * 2;
        const hipStream_t s = static_cast<hipStream_t>(stream);
        const uint32_t tiles = (uint32_t)(n_vec / 32);
        const int r = dtype == TQ_F16 ? fused_bits<TQ_F16>(mse_bits, d, nullptr, 1, tiles, s) : fused_bits<TQ_BF16>(mse_bits, d, nullptr, 1, tiles, s);
        if (r) return r;
        done = n_vec / 32 * 32;
    }
    return two_kernels(j, done, head_dim, stream);
}
