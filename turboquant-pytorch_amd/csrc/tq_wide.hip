// compress and decompress for the head dimensions 96, 160, 192 and 224 with 16-bit elements: the structure of the
// 256-wide kernels (csrc/tq_anydim.hip) with the dimension as a template argument.  Upstream
// turboquant/compressors_v3.py:37-43 builds rotation and codebook for whatever head_dim it is given; :46-81
// compress, :84-105 decompress.
//
// A block is D/32 waves that share tiles of 32 vectors; wave w keeps the rows [32w, 32w+32) of the rotation (compress:
// two 16-bit terms of Pi; decompress: the leading fp16 term of Pi^T) resident in registers as MFMA A operands for all
// D/16 steps of the contraction, so nothing of the table is read again after a block's first tile.  Tiles are fetched
// one ahead with coalesced loads, parked in a double-buffered LDS tile (one barrier per tile) and read back by every
// wave as B operands.  A row of such a tile is D*2 bytes, an odd multiple of 64: rows are rotated by their index
// (piece p of row v sits at position (p + v) mod D/8), which spreads the eight rows a 16-byte LDS access touches over all
// banks.  Same arithmetic, in the same order, as the run-time-dimension kernels: a vector gets the same bytes whichever
// of the two compresses it (fp32 elements go there).  The RAGGED instantiations take a head dimension dl that is not a
// multiple of 32 as the next multiple D, the way the run-time-dimension kernels do: the table holds the rotation extended
// by zeros, elements a vector does not have are staged as zeros, coordinates it does not have get the code 0 and are
// neither decoded nor stored; whole 16-byte pieces at aligned addresses take the wide loads and stores, the rest moves
// element by element.
#include <mutex>
#include <type_traits>

#include "tq_wide.h"

namespace {

template <int D>
struct Wide {
    static_assert(D % 32 == 0 && D > 64 && D < 256 && D != 128, "96, 160, 192, 224");
    static constexpr int WAVES = D / 32, THREADS = 64 * WAVES, STEPS = D / 16, PIECES = D / 8;
    static constexpr int ROW = D * 2, TILE_BYTES = 32 * ROW;
    // waves per SIMD the compress kernel is compiled for: three (168 registers) at 96, where a compute unit's LDS holds
    // four blocks of three waves; from 160 on the resident rotation takes D/2 registers and the kernel 228 to 256 (held
    // to 168 it spills 60 to 80 of them and runs at half the rate), so one block of D/32 waves is resident per unit
    static constexpr int COMPRESS_WAVES_PER_SIMD = D == 96 ? 3 : 2;
    // compress: quantiser grid | two tiles | per-piece sums of squares of three tiles
    static constexpr uint32_t COMPRESS_LDS = TQ_GRID_LDS_BYTES + 2 * TILE_BYTES + 3 * 32 * PIECES * 4;
    // decompress: byte -> centroids table | two tiles of centroids | output tile | norms of two tiles
    static constexpr uint32_t DECOMPRESS_LDS = 4096 + 3 * TILE_BYTES + 2 * 32 * 4;
};

// position of piece p in row v of a tile
template <int D>
__device__ __forceinline__ uint32_t rotated_piece(uint32_t p, uint32_t v) {
    return (p + v) % (uint32_t)Wide<D>::PIECES;
}

template <int DTYPE, int BITS, int D, bool RAGGED>
__global__ __launch_bounds__(Wide<D>::THREADS, Wide<D>::COMPRESS_WAVES_PER_SIMD) void tq_wide_compress_kernel(TqDevJob job0, const tq_job *jobs, uint32_t dl) {
    static_assert(DTYPE == TQ_F16 || DTYPE == TQ_BF16, "16-bit inputs");
    using W = Wide<D>;
    constexpr int STEPS = W::STEPS, PIECES = W::PIECES, ROW = W::ROW, THREADS = W::THREADS;
    constexpr int IPB = 8 / BITS, NB = 16 / IPB, NW = NB < 4 ? 1 : NB / 4;
    constexpr int CPS = (16 + STEPS - 1) / STEPS;      // coordinates searched per step of the contraction

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t *lds_grid = lds;                                                        // single copy, bases unshifted
    uint8_t (*lds_stage)[W::TILE_BYTES] = reinterpret_cast<uint8_t (*)[W::TILE_BYTES]>(lds + TQ_GRID_LDS_BYTES);
    float (*lds_part)[32][PIECES] = reinterpret_cast<float (*)[32][PIECES]>(lds + TQ_GRID_LDS_BYTES + 2 * W::TILE_BYTES);   // [3]

    const TqDevJob job = tq_uniform_job(tq_load_job(job0, jobs, blockIdx.y, 2));
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = tq_uniform32(tid >> 6);
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const uint32_t n_tiles = (job.n_vec + 31u) / 32u;
    if (blockIdx.x >= n_tiles) return;        // also: an empty job of a batch, whose table may be NULL
    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(job.table);

    // loads of a tile: piece i = l * THREADS + tid of the tile's 32 * PIECES is piece i % PIECES of vector i / PIECES;
    // vectors past the end re-read the job's last one (never stored)
    uint32_t ld_vec[2], ld_piece[2];
#pragma unroll
    for (int l = 0; l < 2; ++l) {
        const uint32_t i = l * THREADS + tid;
        ld_vec[l] = i / PIECES;
        ld_piece[l] = i % PIECES;
    }
    tq_u4 pre[2];
    auto issue_loads = [&](uint32_t tl) {
#pragma unroll
        for (int l = 0; l < 2; ++l) {
            uint32_t v = tl * 32u + ld_vec[l];
            v = v < job.n_vec ? v : job.n_vec - 1u;
            if constexpr (RAGGED) {
                const TQ_GLOBAL uint8_t *src = (const TQ_GLOBAL uint8_t *)job.states + tq_vec_offset(job, v);
                const uint32_t e0 = ld_piece[l] * 8u;
                if (e0 + 8u <= dl && (((uintptr_t)src + 2u * e0) & 15u) == 0u) {      // a whole piece at an aligned address
                    pre[l] = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>(src + 2u * e0);
                } else {                                                              // element by element; past the end: zero
                    tq_u4 q = {0u, 0u, 0u, 0u};
#pragma unroll
                    for (uint32_t k = 0; k < 8u; ++k)
                        if (e0 + k < dl) q[k / 2] |= (uint32_t)*reinterpret_cast<const TQ_GLOBAL uint16_t *>(src + 2u * (e0 + k)) << (16 * (k & 1));
                    pre[l] = q;
                }
            } else {
                pre[l] = tq_gload16(job.states + tq_vec_offset(job, v) + ld_piece[l] * 16u);
            }
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
    tq_copy_to_lds(lds_grid, job.table + hd->off_grid, hd->grid_cells * 8u, tid, (uint32_t)THREADS);
    const float grid_scale = hd->grid_scale, grid_bias = hd->grid_bias;

    // park the prefetched tile in buffer b and leave the pieces' sums of squares in slot `slot`
    uint32_t park_off[2];
#pragma unroll
    for (int l = 0; l < 2; ++l) park_off[l] = ld_vec[l] * ROW + (rotated_piece<D>(ld_piece[l], ld_vec[l]) << 4);
    auto park = [&](uint32_t b, uint32_t slot) {
#pragma unroll
        for (int l = 0; l < 2; ++l) {
            *reinterpret_cast<tq_u4 *>(lds_stage[b] + park_off[l]) = pre[l];
            lds_part[slot][ld_vec[l]][ld_piece[l]] = sumsq8<DTYPE>(pre[l], 0.f);
        }
    };
    // B operand of step s: piece 2 s + hk of row n
    uint32_t op_off[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) op_off[s] = n * ROW + (rotated_piece<D>(2u * s + hk, n) << 4);
    const uint32_t g_bytes = RAGGED ? (dl + IPB - 1u) / IPB : (uint32_t)(D / IPB);      // packed bytes per vector

    // iteration j: rotate tile j into acc_new, search tile j-1 from acc_old
    auto iteration = [&](auto rot_tag, auto search_tag, uint32_t j, tq_f16v &acc_new, const tq_f16v &acc_old) {
        constexpr bool ROT = decltype(rot_tag)::value, SEARCH = decltype(search_tag)::value;
        const uint8_t *stage = lds_stage[j & 1u];
        float nrm = 0.f, inv = 0.f, inv_cell = 0.f;
        if constexpr (SEARCH) {
            // pieces added in index order, as the run-time-dimension kernel adds them: tile j-1 sits in slot (j-1) % 3
            const float4 *pp = reinterpret_cast<const float4 *>(&lds_part[(j + 2u) % 3u][n][0]);
            float ss = 0.f;
#pragma unroll
            for (int q = 0; q < PIECES / 4; ++q) {
                const float4 f = pp[q];
                ss += f.x; ss += f.y; ss += f.z; ss += f.w;
            }
            nrm = tq_norm_from_sumsq(ss);
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
                const tq_u4 bop = *reinterpret_cast<const tq_u4 *>(stage + op_off[s]);
                acc_new = (DTYPE == TQ_F16) ? mfma_f16(areg[0][s], bop, acc_new) : mfma_bf16(areg[0][s], bop, acc_new);
                acc_new = (DTYPE == TQ_F16) ? mfma_f16(areg[1][s], bop, acc_new) : mfma_bf16(areg[1][s], bop, acc_new);
            }
            if constexpr (SEARCH) {     // coordinates 32 w + 16 hk + c of vector n, CPS of them behind every step
#pragma unroll
                for (int c = s * CPS; c < (s + 1) * CPS && c < 16; ++c) {
                    const float a = acc_old[c];
                    const uint32_t addr = __float_as_uint(fmaf(a, inv_cell, grid_bias)) & TQ_GRID_ADDR_MASK;
                    const tq_u2 cell = *reinterpret_cast<const tq_u2 *>(lds_grid + addr);
                    const float t = fmaf(a, inv, -__uint_as_float(cell[0]));
                    uint32_t code = cell[1] + (~__float_as_uint(t) >> 31);                // base + !(rho < threshold)
                    if constexpr (RAGGED) code = 32u * wave + 16u * hk + (uint32_t)c < dl ? code : 0u;
                    const int byte = c / IPB, k = c % IPB;                                // most significant code of a byte first
                    words[byte / 4] |= code << (8 * (byte % 4) + BITS * (IPB - 1 - k));
                }
            }
            if (s % 2 == 1) __builtin_amdgcn_sched_barrier(0);      // keep the steps in this order (register pressure)
        }
        if constexpr (SEARCH) {
            const uint32_t v = (blockIdx.x + (j - 1u) * gridDim.x) * 32u + n;
            if (v < job.n_vec) {
                const uint32_t slot = tq_packed_slot(job, v);
                uint8_t *dst = job.idx_bytes + (size_t)slot * g_bytes + (2u * wave + hk) * NB;
                bool bytewise = false;
                if constexpr (RAGGED) bytewise = (2u * wave + hk) * NB + NB > g_bytes || ((uintptr_t)dst & (uintptr_t)(NB - 1));
                if (bytewise) {
#pragma unroll
                    for (int b = 0; b < NB; ++b)
                        if ((2u * wave + hk) * NB + (uint32_t)b < g_bytes)
                            *((TQ_GLOBAL uint8_t *)dst + b) = (uint8_t)(words[b / 4] >> (8 * (b % 4)));
                } else if constexpr (NB == 2) tq_gstore2(reinterpret_cast<uint16_t *>(dst), (uint16_t)words[0]);
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

// decompress: wave w keeps the rows [32w, 32w+32) of Pi^T (leading fp16 term).  The packed bytes of a tile are fetched
// one tile ahead (every thread the bytes of 16 codes), turned into fp16 centroids through the byte -> centroids table and
// parked in a double-buffered LDS tile that all waves read as B operands; the scaled, rounded results go through a
// second LDS tile so that the stores are D*2 contiguous bytes per vector.
template <int DTYPE, int IPB, int D, bool RAGGED>
__global__ __launch_bounds__(Wide<D>::THREADS) void tq_wide_decompress_kernel(TqDevJob job0, const tq_job *jobs, uint32_t dl) {
    static_assert(DTYPE == TQ_F16 || DTYPE == TQ_BF16, "16-bit outputs");
    using W = Wide<D>;
    constexpr int STEPS = W::STEPS, PIECES = W::PIECES, ROW = W::ROW, THREADS = W::THREADS, WAVES = W::WAVES;
    constexpr int ENTRY = 2 * IPB;                 // bytes of a table entry: the fp16 centroids of one packed byte
    constexpr int RAW = 16 / IPB;                  // packed bytes of a thread's 16 codes: 2, 4, 8, 16

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t *lds_lut = lds;
    uint8_t (*lds_y)[W::TILE_BYTES] = reinterpret_cast<uint8_t (*)[W::TILE_BYTES]>(lds + 4096);
    uint8_t *lds_out = lds + 4096 + 2 * W::TILE_BYTES;
    float (*lds_norm)[32] = reinterpret_cast<float (*)[32]>(lds + 4096 + 3 * W::TILE_BYTES);       // [2][32]

    const TqDevJob job = tq_uniform_job(tq_load_job(job0, jobs, blockIdx.y, 2));
    uint8_t *out_base = const_cast<uint8_t *>(job.states);
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = tq_uniform32(tid >> 6);
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const uint32_t n_tiles = (job.n_vec + 31u) / 32u;
    if (blockIdx.x >= n_tiles) return;
    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(job.table);
    const uint32_t g_bytes = RAGGED ? (dl + IPB - 1u) / IPB : (uint32_t)(D / IPB);      // packed bytes per vector in memory

    // a thread's share of a tile: codes [16 c, 16 c + 16) of vector dv, c = tid % (2 WAVES)
    const uint32_t dv = tid / (2u * WAVES), chunk = tid % (2u * WAVES);
    uint32_t raw[4] = {0u, 0u, 0u, 0u};
    uint16_t norm_bits = 0;
    auto issue_loads = [&](uint32_t tl) {
        uint32_t v = tl * 32u + dv;
        v = v < job.n_vec ? v : job.n_vec - 1u;
        const uint32_t slot = tq_packed_slot(job, v);
        const uint8_t *src = job.idx_bytes + (size_t)slot * g_bytes + chunk * RAW;
        bool bytewise = false;
        if constexpr (RAGGED) bytewise = chunk * RAW + RAW > g_bytes || ((uintptr_t)src & (uintptr_t)(RAW - 1));
        if (bytewise) {     // byte by byte; past the vector's last byte: zero (never decoded)
#pragma unroll
            for (int q = 0; q < 4; ++q) raw[q] = 0u;
#pragma unroll
            for (int b = 0; b < RAW; ++b)
                if (chunk * RAW + (uint32_t)b < g_bytes) raw[b / 4] |= (uint32_t)*((const TQ_GLOBAL uint8_t *)src + b) << (8 * (b % 4));
        } else if constexpr (RAW == 2) raw[0] = tq_gload2(reinterpret_cast<const uint16_t *>(src));
        else if constexpr (RAW == 4) raw[0] = *reinterpret_cast<const TQ_GLOBAL uint32_t *>((const TQ_GLOBAL uint8_t *)src);
        else if constexpr (RAW == 8) { const tq_u2 t = tq_gload8(src); raw[0] = t[0]; raw[1] = t[1]; }
        else { const tq_u4 t = tq_gload16(src); raw[0] = t[0]; raw[1] = t[1]; raw[2] = t[2]; raw[3] = t[3]; }
        if (chunk == 0u) norm_bits = tq_gload2(job.vec_norms + slot);
    };
    issue_loads(blockIdx.x);

    tq_u4 areg[STEPS];
    {
        const uint8_t *src = job.table + hd->off_at_f16;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) areg[s] = tq_gload16(src + (((size_t)wave * STEPS + s) * 64 + lane) * 16);
    }
    tq_copy_to_lds(lds_lut, job.table + hd->off_lut, 256u * ENTRY, tid, (uint32_t)THREADS);
    __syncthreads();

    // the prefetched bytes -> 16 fp16 centroids = pieces 2 chunk, 2 chunk + 1 of row dv of buffer b.  In this tile the even
    // pieces of a row come first and the odd ones after them (piece 2 c + q at index q * PIECES/2 + c, then rotated by the
    // row like everywhere else): the threads that decode a row write neighbouring bank groups at a time instead of every
    // second one.
    const uint32_t y_off[2] = {dv * ROW + (rotated_piece<D>(chunk, dv) << 4), dv * ROW + (rotated_piece<D>(PIECES / 2 + chunk, dv) << 4)};
    auto decode = [&](uint32_t b) {
        uint32_t h[8];          // 16 halves
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
        if constexpr (RAGGED) {     // coordinates the vector does not have contribute nothing
#pragma unroll
            for (int k = 0; k < 16; ++k)
                if (16u * chunk + (uint32_t)k >= dl) h[k / 2] &= (k & 1) ? 0x0000ffffu : 0xffff0000u;
        }
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const tq_u4 o = {h[4 * q], h[4 * q + 1], h[4 * q + 2], h[4 * q + 3]};
            *reinterpret_cast<tq_u4 *>(lds_y[b] + y_off[q]) = o;
        }
        if (chunk == 0u) lds_norm[b][dv] = (float)__builtin_bit_cast(_Float16, norm_bits);
    };
    uint32_t op_off[STEPS];     // B operand of step s: piece 2 s + hk of row n, at index hk * PIECES/2 + s
#pragma unroll
    for (int s = 0; s < STEPS; ++s) op_off[s] = n * ROW + (rotated_piece<D>(hk * (PIECES / 2) + s, n) << 4);
    // lane (n, hk) ends up with elements 32 w + 16 hk + r of vector n: pieces 4 w + 2 hk + c of its output row
    const uint32_t out_off[2] = {n * ROW + (rotated_piece<D>(4u * wave + 2u * hk, n) << 4), n * ROW + (rotated_piece<D>(4u * wave + 2u * hk + 1u, n) << 4)};
    // the stores of a tile: piece i = k * THREADS + tid is piece i % PIECES of vector i / PIECES
    uint32_t st_vec[2], st_piece[2], st_off[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const uint32_t i = k * THREADS + tid;
        st_vec[k] = i / PIECES;
        st_piece[k] = i % PIECES;
        st_off[k] = st_vec[k] * ROW + (rotated_piece<D>(st_piece[k], st_vec[k]) << 4);
    }

    const uint32_t m = (n_tiles - blockIdx.x + gridDim.x - 1u) / gridDim.x;
    decode(0u);
    for (uint32_t j = 0; j < m; ++j) {
        const uint32_t tl = blockIdx.x + j * gridDim.x;
        if (j + 1u < m) issue_loads(tl + gridDim.x);
        __syncthreads();        // tile j is decoded; the output tile of the last iteration has been read
        const uint8_t *ys = lds_y[j & 1u];
        tq_f16v acc = tq_zero16();
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const tq_u4 b = *reinterpret_cast<const tq_u4 *>(ys + op_off[s]);
            acc = mfma_f16(areg[s], b, acc);
        }
        const float nrm = lds_norm[j & 1u][n];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            tq_u4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float x0 = acc[8 * c + 2 * e] * nrm, x1 = acc[8 * c + 2 * e + 1] * nrm;
                if constexpr (DTYPE == TQ_F16) {
                    const tq_half2 hh = {(_Float16)x0, (_Float16)x1};
                    o[e] = __builtin_bit_cast(uint32_t, hh);
                } else {
                    const tq_bf2 hh = {(__bf16)x0, (__bf16)x1};
                    o[e] = __builtin_bit_cast(uint32_t, hh);
                }
            }
            *reinterpret_cast<tq_u4 *>(lds_out + out_off[c]) = o;
        }
        __syncthreads();        // the output tile is complete
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const tq_u4 val = *reinterpret_cast<const tq_u4 *>(lds_out + st_off[k]);
            const uint32_t v = tl * 32u + st_vec[k];
            if (v >= job.n_vec) continue;
            uint8_t *dst = out_base + tq_vec_offset(job, v) + st_piece[k] * 16u;
            if constexpr (RAGGED) {
                const uint32_t e0 = st_piece[k] * 8u;
                if (e0 >= dl) continue;
                if (e0 + 8u > dl || ((uintptr_t)dst & 15u)) {       // element by element
#pragma unroll
                    for (uint32_t e = 0; e < 8u; ++e)
                        if (e0 + e < dl) *reinterpret_cast<TQ_GLOBAL uint16_t *>((TQ_GLOBAL uint8_t *)dst + 2u * e) = (uint16_t)(val[e / 2] >> (16 * (e & 1)));
                    continue;
                }
            }
            tq_gstore16_stream(dst, val);
        }
        if (j + 1u < m) decode((j + 1u) & 1u);
    }
}

// ---- host side --------------------------------------------------------------------------

constexpr int MAX_DEVICES = 64;
std::mutex host_state_mutex;

// Launch of one kernel: blocks of `threads` threads with `lds` bytes of dynamic LDS, as many per compute unit as the
// runtime says fit (remembered per device in `slots`).
template <typename K>
int launch(K kernel, int (&slots)[MAX_DEVICES], uint32_t lds, uint32_t threads, const TqDevJob &job, const tq_job *jobs_dev,
           int n_jobs, uint32_t max_vec, uint32_t dl, hipStream_t stream) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return TQ_ERR_NO_DEVICE;
    int resident;
    {
        std::lock_guard<std::mutex> lock(host_state_mutex);
        if (slots[dev] == 0) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            int cus = 0, per_cu = 0;
            e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e != hipSuccess) return (int)e;
            e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, (int)threads, lds);
            if (e != hipSuccess) return (int)e;
            slots[dev] = (cus > 0 ? cus : 1) * (per_cu > 0 ? per_cu : 1);
        }
        resident = slots[dev];
    }
    const uint32_t tiles = (max_vec + 31u) / 32u;
    const uint32_t bx = tq_blocks_per_job(tiles, resident, n_jobs);
    hipLaunchKernelGGL(kernel, dim3(bx, (unsigned)n_jobs, 1), dim3(threads, 1, 1), lds, stream, job, jobs_dev, dl);
    return (int)hipGetLastError();
}

template <int DTYPE, int BITS, int D>
int launch_compress(const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t dl, hipStream_t s) {
    if (dl != (uint32_t)D) {
        static int slots_ragged[MAX_DEVICES] = {};
        return launch(&tq_wide_compress_kernel<DTYPE, BITS, D, true>, slots_ragged, Wide<D>::COMPRESS_LDS, Wide<D>::THREADS, job, jobs_dev, n_jobs, max_vec, dl, s);
    }
    static int slots[MAX_DEVICES] = {};
    return launch(&tq_wide_compress_kernel<DTYPE, BITS, D, false>, slots, Wide<D>::COMPRESS_LDS, Wide<D>::THREADS, job, jobs_dev, n_jobs, max_vec, dl, s);
}
template <int DTYPE, int D>
int compress_bits(int bits, const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t dl, hipStream_t s) {
    switch (bits) {
        case 1: return launch_compress<DTYPE, 1, D>(job, jobs_dev, n_jobs, max_vec, dl, s);
        case 2: return launch_compress<DTYPE, 2, D>(job, jobs_dev, n_jobs, max_vec, dl, s);
        case 3: return launch_compress<DTYPE, 3, D>(job, jobs_dev, n_jobs, max_vec, dl, s);
        case 4: return launch_compress<DTYPE, 4, D>(job, jobs_dev, n_jobs, max_vec, dl, s);
        case 5: case 6: case 7: case 8:  // one code per byte: identical packing
            return launch_compress<DTYPE, 8, D>(job, jobs_dev, n_jobs, max_vec, dl, s);
        default: return TQ_ERR_BITS;
    }
}
template <int DTYPE>
int compress_dim(int head_dim, int bits, const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, hipStream_t s) {
    const uint32_t dl = (uint32_t)head_dim;
    switch (TQ_PADDED_DIM(head_dim)) {
        case 96: return compress_bits<DTYPE, 96>(bits, job, jobs_dev, n_jobs, max_vec, dl, s);
        case 160: return compress_bits<DTYPE, 160>(bits, job, jobs_dev, n_jobs, max_vec, dl, s);
        case 192: return compress_bits<DTYPE, 192>(bits, job, jobs_dev, n_jobs, max_vec, dl, s);
        case 224: return compress_bits<DTYPE, 224>(bits, job, jobs_dev, n_jobs, max_vec, dl, s);
        default: return TQ_ERR_HEAD_DIM;
    }
}

template <int DTYPE, int IPB, int D>
int launch_decompress(const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t dl, hipStream_t s) {
    if (dl != (uint32_t)D) {
        static int slots_ragged[MAX_DEVICES] = {};
        return launch(&tq_wide_decompress_kernel<DTYPE, IPB, D, true>, slots_ragged, Wide<D>::DECOMPRESS_LDS, Wide<D>::THREADS, job, jobs_dev, n_jobs, max_vec, dl, s);
    }
    static int slots[MAX_DEVICES] = {};
    return launch(&tq_wide_decompress_kernel<DTYPE, IPB, D, false>, slots, Wide<D>::DECOMPRESS_LDS, Wide<D>::THREADS, job, jobs_dev, n_jobs, max_vec, dl, s);
}
template <int DTYPE, int D>
int decompress_bits(int bits, const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, uint32_t dl, hipStream_t s) {
    switch (8 / bits) {
        case 8: return launch_decompress<DTYPE, 8, D>(job, jobs_dev, n_jobs, max_vec, dl, s);
        case 4: return launch_decompress<DTYPE, 4, D>(job, jobs_dev, n_jobs, max_vec, dl, s);
        case 2: return launch_decompress<DTYPE, 2, D>(job, jobs_dev, n_jobs, max_vec, dl, s);
        case 1: return launch_decompress<DTYPE, 1, D>(job, jobs_dev, n_jobs, max_vec, dl, s);
        default: return TQ_ERR_BITS;
    }
}
template <int DTYPE>
int decompress_dim(int head_dim, int bits, const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_vec, hipStream_t s) {
    const uint32_t dl = (uint32_t)head_dim;
    switch (TQ_PADDED_DIM(head_dim)) {
        case 96: return decompress_bits<DTYPE, 96>(bits, job, jobs_dev, n_jobs, max_vec, dl, s);
        case 160: return decompress_bits<DTYPE, 160>(bits, job, jobs_dev, n_jobs, max_vec, dl, s);
        case 192: return decompress_bits<DTYPE, 192>(bits, job, jobs_dev, n_jobs, max_vec, dl, s);
        case 224: return decompress_bits<DTYPE, 224>(bits, job, jobs_dev, n_jobs, max_vec, dl, s);
        default: return TQ_ERR_HEAD_DIM;
    }
}

}  // namespace

bool tq_wide_supported(int head_dim, int dtype) {
    const int padded = TQ_PADDED_DIM(head_dim);      // 65 ... 96, 129 ... 224
    return (dtype == TQ_F16 || dtype == TQ_BF16) && head_dim >= 8 && (padded == 96 || padded == 160 || padded == 192 || padded == 224);
}

int tq_wide_compress(int dtype, int bits, int head_dim, const TqDevJob &single, const tq_job *jobs_dev, int n_jobs,
                     uint32_t max_vec, hipStream_t stream) {
    if (!tq_wide_supported(head_dim, dtype)) return TQ_ERR_HEAD_DIM;
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    return dtype == TQ_F16 ? compress_dim<TQ_F16>(head_dim, bits, single, jobs_dev, n_jobs, max_vec, stream)
                           : compress_dim<TQ_BF16>(head_dim, bits, single, jobs_dev, n_jobs, max_vec, stream);
}

int tq_wide_decompress(int dtype, int bits, int head_dim, const TqDevJob &single, const tq_job *jobs_dev, int n_jobs,
                       uint32_t max_vec, hipStream_t stream) {
    if (!tq_wide_supported(head_dim, dtype)) return TQ_ERR_HEAD_DIM;
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    return dtype == TQ_F16 ? decompress_dim<TQ_F16>(head_dim, bits, single, jobs_dev, n_jobs, max_vec, stream)
                           : decompress_dim<TQ_BF16>(head_dim, bits, single, jobs_dev, n_jobs, max_vec, stream);
}
