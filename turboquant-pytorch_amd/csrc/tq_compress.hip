// compress: per-vector L2 norm, rotation on the matrix cores, Lloyd-Max code search, bit packing.
// Replaces MSECompressor.compress (upstream turboquant/compressors_v3.py:46-81) with one kernel.
//
// Work decomposition (gfx950, wave64):
//   * a block is four waves that share tiles of 32 consecutive vectors; wave w keeps the quarter
//     of the rotation that produces coordinates [32w, 32w+32) resident in registers as MFMA A
//     operands (all 16-bit terms of the split: 64 registers), so the matrix pipe never waits for
//     operand loads and several waves fit on a SIMD;
//   * the tile is fetched with fully coalesced 16-byte loads (one instruction = 1 KiB of
//     consecutive memory, a quarter of them by each wave), parked in a double-buffered,
//     XOR-swizzled LDS buffer (one barrier per tile) and read back as the B operand of
//     v_mfma_f32_32x32x16 (vector n on MFMA column n);
//   * the rotation is pre-split on the host into 16-bit terms whose sum is Pi to ~2^-22 (fp16
//     path) / 2^-17 (bf16 path); inputs are exact in the MFMA input type (fp32 inputs are split
//     into three exact bf16 terms and use three Pi terms), accumulation is fp32, so the rotated
//     coordinates agree with an fp32 GEMM to ~1e-6 or better;
//   * the rotation is applied to the raw vector and scaled by 1 / (norm + 1e-8) afterwards
//     (linearity), so the norm reduction overlaps the MFMAs;
//   * every lane ends up with 16 consecutive rotated coordinates of one vector: the code search
//     is two fused multiply-adds, one 8-byte LDS lookup and a funnel shift per coordinate, and
//     the packed bytes of a lane are contiguous in memory;
//   * tiles whose 32 vectors all exist take a path without per-lane predicates: a fixed number
//     of loads and stores per iteration lets the compiler wait for the prefetched loads alone
//     (s_waitcnt vmcnt(n)) instead of draining the previous tile's stores on every iteration.
#include <mutex>
#include <type_traits>

#include "tq_anydim.h"
#include "tq_device.h"

namespace {

#ifndef TQ_C16_WAVES
#define TQ_C16_WAVES 3
#endif
// tiles of 16-bit input that a block keeps in LDS or on their way there (direct-to-LDS loads)
#ifndef TQ_RING
#define TQ_RING 4
#endif
#ifndef TQ_PIN_SCHEDULE
#define TQ_PIN_SCHEDULE 1
#endif
// log2 of the iterations a block keeps one issue priority before it moves to the next (0: priorities stay untouched)
#ifndef TQ_PRIO_SHIFT
#define TQ_PRIO_SHIFT 3
#endif
// Measurement build (never the shipped library): the pipelined path keeps its loads, LDS traffic, barriers, norm
// arithmetic and stores, and leaves out the matrix instructions and the code search (1), the matrix instructions only
// (2) or the code search only (3).  What it writes is garbage; its time is what the rest of the kernel costs on its own.
#ifndef TQ_SKELETON
#define TQ_SKELETON 0
#endif
#define TQ_SKEL_NO_MFMA (TQ_SKELETON == 1 || TQ_SKELETON == 2)
#define TQ_SKEL_NO_SEARCH (TQ_SKELETON == 1 || TQ_SKELETON == 3)
template <int DTYPE> struct InTraits;
template <> struct InTraits<TQ_F16> { static constexpr int ELEM = 2, TERMS = 2, MIN_WAVES = TQ_C16_WAVES; };
template <> struct InTraits<TQ_BF16> { static constexpr int ELEM = 2, TERMS = 2, MIN_WAVES = TQ_C16_WAVES; };
// fp32 input keeps three rotation terms resident and stages 16 KiB tiles
template <> struct InTraits<TQ_F32> { static constexpr int ELEM = 4, TERMS = 3, MIN_WAVES = 2; };

constexpr int CWAVES = TQ_TILES;        // waves per block = MFMA row tiles
constexpr int CTHREADS = CWAVES * TQ_WAVE;

// calls step(k) for k = FROM .. TO-1 until one of them reports the end; true = ended
template <uint32_t FROM, uint32_t TO, typename F>
__device__ __forceinline__ bool run_tail(F &step) {
    if constexpr (FROM >= TO) {
        return false;
    } else {
        if (step(std::integral_constant<uint32_t, FROM>{})) return true;
        return run_tail<FROM + 1, TO>(step);
    }
}

template <int DTYPE, int BITS>
__global__ __launch_bounds__(CTHREADS, InTraits<DTYPE>::MIN_WAVES) void tq_compress_kernel(TqDevJob job0, const tq_job *jobs, uint32_t *workspace,
                                                                                          uint32_t tshift, uint32_t paired) {
    using T = InTraits<DTYPE>;
    using P = Pack<BITS>;
    constexpr int ELEM = T::ELEM;
    constexpr int VEC_BYTES = TQ_HEAD_DIM * ELEM;      // 256 or 512
    constexpr int STAGE = 32 * VEC_BYTES;              // one tile
    constexpr int NLOAD = STAGE / 1024 / CWAVES;       // 16-byte loads per lane per tile (this wave's quarter)
    constexpr int PIECES = VEC_BYTES / 16;             // 16-byte pieces per vector
    constexpr int VEC_PER_LOAD = 64 / PIECES;          // vectors covered by one load instruction
    constexpr int NB = P::NB, NW = P::NW;

    // grid copies first, so that their LDS addresses are small compile-time immediates
    constexpr int RING = ELEM == 2 ? TQ_RING : 2;     // staged tiles
    __shared__ __attribute__((aligned(16))) uint8_t lds_grid[TQ_GRID_LDS_BYTES];
    __shared__ __attribute__((aligned(1024))) uint8_t lds_stage[RING][STAGE];
    __shared__ float lds_ss[2][32];   // sum of squares of the tile's vectors (16-bit inputs)
    __shared__ float lds_ssh[2][32][2];   // the same per half of a row (rows that are pairs of 64-wide vectors)
    __shared__ __attribute__((aligned(16))) float lds_part[2][32][4];   // the same, one share per wave (pipelined path)

    // paired: the job's vectors are 64 wide and the kernel works on pairs of them as 128-wide rows (diag(Pi, Pi) from the
    // table's pair sections).  Everything is as for 128-wide vectors except the norm: one per half of a row; the
    // coordinates of wave w belong to half w / 2.
    const TqDevJob job = tq_uniform_job(tq_pair_job(tq_load_job(job0, jobs, blockIdx.y, ELEM), paired != 0u));

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t n_tiles = (job.n_vec + 31u) / 32u;
    if (n_tiles == 0u) return;    // an empty job of a batch: its table may be NULL, and its counters stay untouched (zero)
    const uint32_t n_full = job.n_vec / 32u;
    const bool one_row = job.tokens >= job.n_vec;
    // Which tiles a block works on.  Single-row jobs of 16-bit elements (the pipelined path below) hand their tiles out
    // as tickets of 2^tshift consecutive tiles: block b starts with ticket b; its later tickets are b + grid, b + 2 grid, ...
    // (fixed assignment) or, with a workspace, come from a counter in device memory in the order in which the blocks
    // ask, so that compute units that run slower than others (the dies of this part do not all run at one pace) take
    // fewer tiles and all blocks of a job end together.  counter[0] = tiles handed out beyond every block's first ticket,
    // counter[1] = blocks of the job that are done; the last block to finish sets both back to zero, so a workspace
    // that was zero before a launch is zero after it (the contract of the decompress kernel's counters).
    // Every other job walks single tiles blockIdx.x, blockIdx.x + grid, ...
    const bool ticket_job = ELEM == 2 && one_row && job.token_stride < (1ll << 26);
    // (a ticket has to outlast the pipeline's depth: the first drawn ticket is published one iteration after the start)
    uint32_t *counter = workspace && (1u << tshift) > (uint32_t)TQ_RING ? workspace + blockIdx.y * (TQ_WORKSPACE_BYTES_PER_JOB / 4) : nullptr;
    auto report_done = [&]() {      // once per block of a non-empty job, after its last draw has been answered
        if (counter && tid == 0) {
            if (atomicAdd(counter + 1, 1u) == gridDim.x - 1u) {
                atomicExch(counter, 0u);
                atomicExch(counter + 1, 0u);
            }
        }
    };
    uint32_t tile = ticket_job ? blockIdx.x << tshift : blockIdx.x;
    if (tile >= n_tiles) {        // whole block idle (uniform)
        report_done();
        return;
    }
    const uint32_t tile_stride = gridDim.x;

    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(job.table);

    // ---- this wave's quarter of the rotation, resident for the whole kernel.  Wave w walks the 16-input
    // steps of the contraction in the order 2w, 2w+1, ... (mod 8): its first two steps then cover inputs
    // [32w, 32w+32), the share of the vector whose squares it sums in the pipelined path.
    // (fp32 inputs sum their squares while they walk the steps, every wave over the whole vector: same order in all waves)
    const uint32_t step0 = ELEM == 2 ? 2u * wave : 0u;
    tq_u4 areg[T::TERMS][TQ_STEPS];
    // Rotation operands into registers and the quantiser grid into LDS (one copy per code position, base pre-shifted).
    // Every cell is fetched once and written to all its copies; the fetches of a thread are issued together.
    // Called once per block: behind the first tile loads on the pipelined path, so that their latencies overlap.
    auto load_tables = [&]() {
        const uint8_t *src = job.table + (paired ? (DTYPE == TQ_F16 ? hd->off_pair_a_f16 : hd->off_pair_a_bf16)
                                                 : (DTYPE == TQ_F16 ? hd->off_a_f16 : hd->off_a_bf16));
#pragma unroll
        for (int term = 0; term < T::TERMS; ++term)
#pragma unroll
            for (int s = 0; s < TQ_STEPS; ++s)
                areg[term][s] = tq_gload16(src + (size_t)term * TQ_OPERAND_BYTES +
                                           (((size_t)wave * TQ_STEPS + ((s + step0) & 7u)) * 64 + lane) * 16);
        constexpr int CELL_TRIPS = (TQ_GRID_MAX_CELLS(BITS) + CTHREADS - 1) / CTHREADS;
        const uint32_t cells = hd->grid_cells;
        const uint8_t *gsrc = job.table + hd->off_grid;
        tq_u2 cell[CELL_TRIPS];
#pragma unroll
        for (int k = 0; k < CELL_TRIPS; ++k) {
            const uint32_t q = tid + k * CTHREADS;
            cell[k] = tq_gload8(gsrc + 8u * (q < cells ? q : 0u));
        }
#pragma unroll
        for (int k = 0; k < CELL_TRIPS; ++k) {
            const uint32_t q = tid + k * CTHREADS;
            if (q < cells) {
#pragma unroll
                for (int c = 0; c < P::COPIES; ++c) {
                    const tq_u2 e = {cell[k][0], cell[k][1] << copy_shift_rt<BITS>(c)};
                    *reinterpret_cast<tq_u2 *>(lds_grid + c * P::COPY_STRIDE + 8u * q) = e;
                }
            }
        }
    };
    const float grid_scale = hd->grid_scale, grid_bias = hd->grid_bias;

    const uint32_t ld_vec = lane / PIECES, ld_piece = lane % PIECES;  // role in the coalesced loads
    const uint32_t n = lane & 31u, hk = lane >> 5;                    // role in the MFMA: column, half
    const uint32_t half = wave >> 1;                                  // paired rows: the 64-wide vector this wave's coordinates belong to

    // LDS offset of this lane's piece of load j (computed where it is used: these paths are not the hot one)
    auto st_off = [&](int j) {
        const uint32_t vl = (wave * NLOAD + j) * VEC_PER_LOAD + ld_vec;
        const uint32_t swz = (ELEM == 2) ? (vl & 15u) : ((vl & 15u) << 1);
        return vl * VEC_BYTES + ((ld_piece ^ swz) << 4);
    };

    tq_u4 pre[NLOAD];
    // loads of this wave's quarter of tile `tl`, generic addressing (any strides, tail clamped)
    auto issue_loads = [&](auto full_tag, uint32_t tl) {
        constexpr bool FULL = decltype(full_tag)::value;
        const uint32_t v0 = tl * 32u + (wave * NLOAD) * VEC_PER_LOAD + ld_vec;
#pragma unroll
        for (int j = 0; j < NLOAD; ++j) {
            uint32_t v = v0 + j * VEC_PER_LOAD;
            if (!FULL) v = v < job.n_vec ? v : job.n_vec - 1u;   // tail: re-read the last vector, never stored
            pre[j] = tq_gload16(job.states + tq_vec_offset(job, v) + ld_piece * 16u);
        }
    };

    // Park this wave's quarter of the prefetched tile in LDS (swizzled: the operand reads are conflict
    // free).  For 16-bit inputs the squares are summed here, where every element is touched once: the 16
    // lanes of a DPP row hold the 16 pieces of one vector.  The order of the additions is the one of the
    // pipelined path below (pieces 4w + h and 4w + 2 + h as one chain, the two chains of a wave's share
    // added, the shares added pairwise), so that a vector gets the same norm whichever path compresses it.
    auto row_shr = [](float v, auto n_tag) {
        constexpr int N = decltype(n_tag)::value;
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x110 + N, 0xf, 0xf, true));
    };
    auto park = [&](uint32_t b, const tq_u4 (&src)[NLOAD]) {
        uint8_t *stage = lds_stage[b];
#pragma unroll
        for (int j = 0; j < NLOAD; ++j) *reinterpret_cast<tq_u4 *>(stage + st_off(j)) = src[j];
        if constexpr (ELEM == 2) {
#pragma unroll
            for (int j = 0; j < NLOAD; ++j) {
                const float own = sumsq8<DTYPE>(src[j], 0.f);
                const float chain = sumsq8<DTYPE>(src[j], row_shr(own, std::integral_constant<int, 2>{}));   // pieces p - 2, p
                const float share = chain + row_shr(chain, std::integral_constant<int, 1>{});               // at p % 4 == 3
                const float pair = share + row_shr(share, std::integral_constant<int, 4>{});                // at p == 7, 15
                const float total = pair + row_shr(pair, std::integral_constant<int, 8>{});                 // at p == 15
                if ((lane & 15u) == 15u) lds_ss[b][(wave * NLOAD + j) * VEC_PER_LOAD + ld_vec] = total;
                if ((lane & 7u) == 7u) lds_ssh[b][(wave * NLOAD + j) * VEC_PER_LOAD + ld_vec][(lane >> 3) & 1u] = pair;   // pieces 0..7, 8..15
            }
        }
    };

    // ---- the three stages of a tile ---------------------------------------------------------
    // (1) rotation step s of the tile parked in `stage`: acc[r] += sum over 16 inputs of
    //     Pi[32w + 16h + r][k] * x_n[k]  (raw, unnormalised); fp32 inputs also sum their squares here
    auto rotate_step = [&](const uint8_t *stage, int s, tq_f16v &acc, float &ss0, float &ss1) {
        const uint32_t sg = ((uint32_t)s + step0) & 7u;   // the step of the contraction that areg[.][s] belongs to
        if constexpr (ELEM == 2) {
            const uint32_t piece = 2u * sg + hk;
            const tq_u4 bop = *reinterpret_cast<const tq_u4 *>(stage + n * VEC_BYTES + ((piece ^ (n & 15u)) << 4));
#pragma unroll
            for (int term = 0; term < T::TERMS; ++term)
                acc = (DTYPE == TQ_F16) ? mfma_f16(areg[term][s], bop, acc) : mfma_bf16(areg[term][s], bop, acc);
        } else {
            const uint32_t piece = 2u * (2u * sg + hk);
            const uint32_t swz = (n & 15u) << 1;
            const uint8_t *row = stage + n * VEC_BYTES;
            const tq_u4 q0 = *reinterpret_cast<const tq_u4 *>(row + ((piece ^ swz) << 4));
            const tq_u4 q1 = *reinterpret_cast<const tq_u4 *>(row + (((piece + 1u) ^ swz) << 4));
            float x[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) { x[i] = __uint_as_float(q0[i]); x[4 + i] = __uint_as_float(q1[i]); }
            if (!paired || (sg >> 2) == half) {      // (a half row: the four steps that cover it)
#pragma unroll
                for (int i = 0; i < 8; ++i) { if (i & 1) ss1 = fmaf(x[i], x[i], ss1); else ss0 = fmaf(x[i], x[i], ss0); }
            }
            tq_u4 xt[3];
            split_f32x8(x, xt[0], xt[1], xt[2]);
            // all products whose weight is >= 2^-24 of the leading one: (x term i, Pi term j), i + j <= 2
#pragma unroll
            for (int i = 0; i < 3; ++i)
#pragma unroll
                for (int term = 0; term + i < 3; ++term) acc = mfma_bf16(areg[term][s], xt[i], acc);
        }
    };

    // (2) norm of the lane's vector and the two scale factors of the code search
    struct Scale { float nrm, inv, inv_cell; };
    auto scale_from_ss = [&](float ss) {
        Scale sc;
        sc.nrm = tq_norm_from_sumsq(ss);
        // 1 / (norm + 1e-8): the reciprocal only scales the coordinates, one ulp is irrelevant
        sc.inv = __builtin_amdgcn_rcpf(sc.nrm + 1e-8f);
        if (DTYPE == TQ_F16) sc.inv *= 1.0f / (float)(1 << TQ_F16_PI_SHIFT);
        sc.inv_cell = sc.inv * grid_scale;   // grid_scale is a power of two: exact
        return sc;
    };
    auto scale_of = [&](uint32_t b, float ss0, float ss1) {
        float ss;
        if constexpr (ELEM == 2) {
            ss = paired ? lds_ssh[b][n][half] : lds_ss[b][n];
        } else {
            ss = ss0 + ss1;                 // both lanes of a vector hold half of the squares
            ss += __shfl_xor(ss, 32);
        }
        return scale_from_ss(ss);
    };

    // (3) code search + packing.  Lane (n, hk) of wave w holds coordinates 32w + 16hk + r.
    // Per coordinate: cell address (fma, and), one 8-byte LDS lookup from the grid copy whose base
    // is pre-shifted to the code's bit position, exact comparison by fma, sign bit funnelled
    // into `lt`, bases OR-ed together.  code = base + !(rho < threshold).
    // The 16 coordinates of a lane are visited in the order q = 0..15 = (word, position in word).
    struct Search { uint32_t lt[NW], lo[NW], hi[NW]; };
    auto search_begin = [&](Search &z) {
#pragma unroll
        for (int w = 0; w < NW; ++w) z.lt[w] = z.lo[w] = z.hi[w] = 0u;
    };
    auto search_lookup = [&](int q, const tq_f16v &acc, const Scale &sc) {
        const int w = q / P::CPW, i = q % P::CPW;
        const float a = acc[P::local_code(w, i)];
        const uint32_t addr = __float_as_uint(fmaf(a, sc.inv_cell, grid_bias)) & TQ_GRID_ADDR_MASK;
        return *reinterpret_cast<const tq_u2 *>(lds_grid + P::copy_of(i) * P::COPY_STRIDE + addr);
    };
    auto search_apply = [&](Search &z, int q, const tq_f16v &acc, const Scale &sc, tq_u2 cell) {
        const int w = q / P::CPW, i = q % P::CPW;
        const float a = acc[P::local_code(w, i)];
        const float t = fmaf(a, sc.inv, -__uint_as_float(cell[0]));
        const int cursor = i == 0 ? 8 * P::WB : P::shift_of(i - 1);
        const int gap = cursor - (P::shift_of(i) + P::FIELD);
        if (gap > 0) z.lt[w] = __builtin_amdgcn_alignbit(z.lt[w], 0u, 32 - gap);
        z.lt[w] = __builtin_amdgcn_alignbit(z.lt[w], __float_as_uint(t), 32 - P::FIELD);
        if (P::IPB == 1 && P::byte_of(i) >= 2) z.hi[w] |= cell[1]; else z.lo[w] |= cell[1];
    };
    auto search_coord = [&](Search &z, int q, const tq_f16v &acc, const Scale &sc) {
        search_apply(z, q, acc, sc, search_lookup(q, acc, sc));
    };
    auto search_end = [&](const Search &z, uint32_t (&words)[NW]) {
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const uint32_t bases = P::IPB == 1 ? (z.lo[w] | (z.hi[w] << 16)) : z.lo[w];
            const uint32_t ge = (~z.lt[w] & P::sign_mask()) >> (P::FIELD - 1);
            words[w] = bases + ge;
        }
    };

    // One tile, parked in buffer `b` and published by a barrier: rotate, then search.
    // Leaves the lane's packed words in `words` and the vector's norm in `nrm`.
    auto compute = [&](uint32_t b, uint32_t (&words)[NW], float &nrm) {
        tq_f16v acc = tq_zero16();
        float ss0 = 0.f, ss1 = 0.f;
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) rotate_step(lds_stage[b], s, acc, ss0, ss1);
        const Scale sc = scale_of(b, ss0, ss1);
        Search z;
        search_begin(z);
#pragma unroll
        for (int q = 0; q < 16; ++q) search_coord(z, q, acc, sc);
        search_end(z, words);
        nrm = sc.nrm;
    };

    // the lane's NB packed bytes and (identical in all lanes of a vector) the fp16 norm
    auto store = [&](uint8_t *dst, uint16_t *ndst, const uint32_t (&words)[NW], float nrm) {
        if constexpr (NB == 2) {
            tq_gstore2(reinterpret_cast<uint16_t *>(dst), (uint16_t)words[0]);
        } else if constexpr (NB == 4) {
            *reinterpret_cast<TQ_GLOBAL uint32_t *>((TQ_GLOBAL uint8_t *)dst) = words[0];
        } else if constexpr (NB == 8) {
            tq_u2 o = {words[0], words[1]};
            tq_gstore8(dst, o);
        } else {
            tq_u4 o = {words[0], words[1], words[2], words[3]};
            tq_gstore16(dst, o);
        }
        // every lane of every wave holds the same norm for vector n: all store it (identical values
        // to one address) rather than predicating the store on a fraction of the lanes
        const _Float16 hn = (_Float16)nrm;
        tq_gstore2(ndst, __builtin_bit_cast(uint16_t, hn));
    };
    const uint32_t lane_slot = (2u * wave + hk) * NB;   // this lane's bytes inside a vector's G = 8 * NB
    auto norm_slot = [&](size_t slot) { return paired ? 2u * slot + half : slot; };     // where the norm of this wave's half of row `slot` goes

    uint32_t buf = 0;
    uint32_t words[NW];
    float nrm;
    // (the pipelined path addresses a tile's vectors with 32-bit offsets from a scalar base: the stride limit of ticket_job)
    const bool pipelined = ticket_job && tile < n_full;
    if (!pipelined) load_tables();
    if (pipelined) {
        if constexpr (ELEM == 2) {
            // Single-row jobs with 16-bit elements (the KV-cache case): a software pipeline over this block's full
            // tiles t_0 .. t_{m-1}.  Tiles travel from memory straight into a ring of RING LDS slots
            // (global_load_lds_dwordx4: no registers, no LDS write instructions); iteration j
            //   waits for its own loads of t_j (issued RING-1 iterations ago) and passes the barrier: t_j is complete
            //   in slot j % RING, and everybody has finished reading t_{j-1};
            //   starts the loads of t_{j+RING-1} into the slot that t_{j-1} has just left;
            //   rotates t_j on the matrix cores while it searches and packs the codes of t_{j-1}, whose rotated
            //   coordinates wait in the other accumulator set (two independent instruction streams: the VALU work
            //   fills the issue slots under the MFMAs); the scale of t_{j-1} comes from the four waves' shares of
            //   its sum of squares, written an iteration ago;
            //   sums the squares of its own share of t_j from the first two operands it feeds to the matrix cores;
            //   stores t_{j-1}.
            // The loads are invisible to the compiler (inline assembly), so it never waits for them; the explicit
            // s_waitcnt counts the younger vector-memory operations of the wave, which is fixed: 2 loads and
            // 2 stores per iteration.
            constexpr int P = RING;
            static_assert(NLOAD == 2 && P >= 2 && P <= 6, "the wait counts below assume two loads per wave and tile");
            // lane i of load j fills bytes [16 i, 16 i + 16) of KiB (wave * NLOAD + j) of the slot: vector
            // vl = (wave * NLOAD + j) * 4 + i / 16, position i % 16, which has to hold piece (i % 16) ^ (vl & 15)
            uint32_t src_off[NLOAD];
#pragma unroll
            for (int j = 0; j < NLOAD; ++j) {
                const uint32_t vl = (wave * NLOAD + j) * VEC_PER_LOAD + ld_vec;
                src_off[j] = vl * (uint32_t)job.token_stride + ((ld_piece ^ (vl & 15u)) << 4);
            }
            const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(
                (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)&lds_stage[0][0] + wave * (NLOAD * 1024u));

            // ---- the block's sequence of tiles.  q[i] = the tile of iteration j - 1 + i while iteration j runs: q[0] is
            // searched and stored, q[1] rotated, q[P] loaded.  All of it lives in scalar registers.  A value >= n_full
            // marks the end (the sequence of a block only grows); loads past the end re-read the job's last full tile.
            __shared__ uint32_t tk[4];          // ticket k of the block sits in slot k % 4 (counter mode only)
            const uint32_t per_ticket = 1u << tshift;
            const uint32_t drawn_origin = gridDim.x << tshift;
            uint32_t q[P + 1];
            uint32_t left = per_ticket - 1u;    // tiles of the head's ticket beyond the head
            uint32_t kt = 0;                    // tickets the head has entered beyond the first
            uint32_t drawn = 0;                 // thread 0: what the atomic of this iteration's draw returned, not yet looked at
            bool have_drawn = false;
            auto draw = [&]() {                 // counter mode; the value is taken by thread 0 alone
                // (the returned value stays untouched until publish(): arithmetic on it here would put a wait for all of
                // the wave's memory operations right behind the atomic)
                if (tid == 0) drawn = atomicAdd(counter, per_ticket);
                have_drawn = true;
            };
            auto publish = [&]() {              // at the end of an iteration: the draw's latency hides behind the tile's work
                if (have_drawn) {
                    if (tid == 0) tk[(kt + 1u) & 3u] = drawn_origin + drawn;
                    have_drawn = false;
                }
            };
            auto advance = [&](uint32_t head) -> uint32_t {    // the tile after `head` in this block's sequence
                if (left) {
                    --left;
                    return head + 1u;
                }
                left = per_ticket - 1u;
                ++kt;
                if (counter) {
                    // ticket kt was drawn when the head entered ticket kt - 1, at least four iterations (one barrier) ago
                    const uint32_t base = (uint32_t)__builtin_amdgcn_readfirstlane(tk[kt & 3u]);
                    draw();
                    return base;
                }
                return (blockIdx.x + kt * gridDim.x) << tshift;
            };
            q[0] = 0xffffffffu;
            q[1] = tile;
#pragma unroll
            for (int i = 2; i <= P; ++i) q[i] = advance(q[i - 1]);     // (counter mode: tickets hold more than P tiles, no draw here)
            if (counter) draw();                // ticket 1: in LDS at the end of the first iteration, read per_ticket - P iterations later
            auto issue = [&](uint32_t slot, uint32_t tl) {
                tl = tl < n_full ? tl : n_full - 1u;
                const uint64_t a = (uint64_t)(uintptr_t)job.states + (uint64_t)tl * (uint64_t)(32 * job.token_stride);
                // (the builtin returns int: widen through uint32_t, or the low half is sign-extended into the high one)
                const uint32_t a_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
                const uint32_t a_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)a);
                const uint64_t base = ((uint64_t)a_hi << 32) | (uint64_t)a_lo;
#pragma unroll
                for (int j = 0; j < NLOAD; ++j) {
                    const uint32_t dst = lds_wave + slot * (uint32_t)STAGE + j * 1024u;
                    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                                 :: "s"(dst), "v"(src_off[j]), "s"(base) : "memory", "m0");
                }
            };
            // operand addresses inside a slot, in this wave's step order
            uint32_t op_off[TQ_STEPS];
#pragma unroll
            for (int i = 0; i < TQ_STEPS; ++i) {
                const uint32_t piece = 2u * ((i + step0) & 7u) + hk;
                op_off[i] = n * VEC_BYTES + ((piece ^ (n & 15u)) << 4);
            }
            const uint32_t bperm_other_half = (lane ^ 32u) << 2;

            // output addresses: a base per tile that is the same in every lane, plus a per-lane constant
            const uint32_t cd_lane = n * (8 * NB) + lane_slot, nd_lane = n;
            auto store_tile = [&](uint32_t tl, const uint32_t (&w)[NW], float nrm_of_tile) {
                store(job.idx_bytes + (size_t)tl * (32u * (8 * NB)) + cd_lane, job.vec_norms + norm_slot((size_t)tl * 32u + nd_lane), w, nrm_of_tile);
            };

            auto scale_from_shares = [&](uint32_t par) {
                const float4 q = *reinterpret_cast<const float4 *>(&lds_part[par][n][0]);
                const float lo_half = q.x + q.y, hi_half = q.z + q.w;
                return scale_from_ss(paired ? (half ? hi_half : lo_half) : lo_half + hi_half);
            };
            // iteration j: slot = j % P; `acc_new` receives t_j, `acc_old` holds t_{j-1}
            auto iteration = [&](auto with_search, auto slot_tag, bool warm, uint32_t par, tq_f16v &acc_new, const tq_f16v &acc_old) {
                constexpr bool SEARCH = decltype(with_search)::value;
                constexpr uint32_t SLOT = decltype(slot_tag)::value;
                // younger than the loads of t_j: the loads of P-2 tiles and, once the pipeline is full, the stores of P-1
                if (warm) wait_vmcnt<2 * (P - 2) + 2 * (P - 1)>(); else wait_vmcnt<2 * (P - 2)>();
                __syncthreads();
                issue((SLOT + P - 1u) % P, q[P]);
                const uint32_t head_next = advance(q[P]);
                const uint8_t *stage = lds_stage[SLOT];
                auto operand = [&](int i) { return *reinterpret_cast<const tq_u4 *>(stage + op_off[i]); };
                auto mfma = [&](int term, int i, tq_u4 bop) {
#if TQ_SKEL_NO_MFMA
                    if (term == 0) acc_new[i] = __uint_as_float(bop[0] ^ bop[1] ^ bop[2] ^ bop[3]);     // the operand read stays alive
#else
                    acc_new = (DTYPE == TQ_F16) ? mfma_f16(areg[term][i], bop, acc_new) : mfma_bf16(areg[term][i], bop, acc_new);
#endif
                };
                acc_new = tq_zero16();
                Search z;
                search_begin(z);
                Scale sc_old{};
                float share = 0.f;
                // Order of the instruction stream: the first step's MFMAs come before anything that depends on the
                // scale of t_{j-1} (an LDS read, a reciprocal square root); the search runs one step behind:
                // coordinates 2i-2, 2i-1 are looked up in step i-1 and applied in step i.
                tq_u4 bop = operand(0);
                tq_u2 c0 = {0u, 0u}, c1 = {0u, 0u};
#pragma unroll
                for (int i = 0; i < TQ_STEPS; ++i) {
                    tq_u4 bop_next = bop;
                    tq_u2 n0 = c0, n1 = c1;
                    if (i + 1 < TQ_STEPS) bop_next = operand(i + 1);
                    if constexpr (SEARCH && !TQ_SKEL_NO_SEARCH) {
                        if (i >= 1) { n0 = search_lookup(2 * i - 2, acc_old, sc_old); n1 = search_lookup(2 * i - 1, acc_old, sc_old); }
                    }
                    mfma(0, i, bop);
                    if (i < 2) share = sumsq8<DTYPE>(bop, share);
                    if constexpr (SEARCH) {
                        if (i == 0) sc_old = scale_from_shares(par ^ 1u);
                        if (i >= 2 && !TQ_SKEL_NO_SEARCH) search_apply(z, 2 * i - 4, acc_old, sc_old, c0);
                    }
                    mfma(1, i, bop);
                    if constexpr (SEARCH && !TQ_SKEL_NO_SEARCH) {
                        if (i >= 2) search_apply(z, 2 * i - 3, acc_old, sc_old, c1);
                    }
                    if (i == 1) {
                        share += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((int)bperm_other_half, __builtin_bit_cast(int, share)));
                        lds_part[par][n][wave] = share;
                    }
#if TQ_PIN_SCHEDULE && !TQ_SKELETON
                    if constexpr (SEARCH) {
                        // pin the order: address arithmetic, the step's LDS reads, then each MFMA followed by the
                        // VALU work that fills its shadow
                        if (i == 0) {
                            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // DS read: next operand, shares
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
                            __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);  // VALU: squares, scale
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);
                        } else if (i == 1) {
                            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        } else {
                            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);   // VALU
                            __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);   // DS read
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
                            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                        }
                    }
#endif
                    bop = bop_next; c0 = n0; c1 = n1;
                }
                if constexpr (SEARCH) {
#if TQ_SKEL_NO_SEARCH
#pragma unroll
                    for (int w = 0; w < NW; ++w) words[w] = __float_as_uint(acc_old[w] * sc_old.inv);
#else
                    search_apply(z, 12, acc_old, sc_old, c0);
                    search_apply(z, 13, acc_old, sc_old, c1);
                    search_coord(z, 14, acc_old, sc_old);
                    search_coord(z, 15, acc_old, sc_old);
                    search_end(z, words);
#endif
                    store_tile(q[0], words, sc_old.nrm);
                }
                publish();
#pragma unroll
                for (int i = 0; i < P; ++i) q[i] = q[i + 1];
                q[P] = head_next;
            };
            auto drain = [&](uint32_t par, const tq_f16v &acc_old) {    // par: parity of the iteration that would come next
                __syncthreads();    // the last tile's shares of the sum of squares are complete
                const Scale sc_old = scale_from_shares(par ^ 1u);
                Search z;
                search_begin(z);
#pragma unroll
                for (int q = 0; q < 16; ++q) search_coord(z, q, acc_old, sc_old);
                search_end(z, words);
                store_tile(q[0], words, sc_old.nrm);
            };

#pragma unroll
            for (int p = 0; p < P - 1; ++p) issue((uint32_t)p, q[1 + p]);
            load_tables();      // (the waits for these loads also cover the older tile loads: harmless, once per block)
            tq_f16v acc_a, acc_b;
            uint32_t done = 0;     // iterations finished
            iteration(std::false_type{}, std::integral_constant<uint32_t, 0>{}, false, 0u, acc_a, acc_a);
            ++done;
            // unrolled by U = lcm(2 accumulator sets, P slots); iteration j runs variant j % U
            constexpr uint32_t U = (P % 2 == 0) ? P : 2 * P;
            // The blocks that share a compute unit do not advance at the same pace: the instruction arbiter prefers the
            // oldest wave, so the block dispatched first finishes its tiles well before the one dispatched last, and the
            // unit then runs under-occupied until that one is done.  Every block therefore walks through the issue
            // priorities 0 .. RES-1, a few iterations each, starting from its place in the dispatch order: over time each
            // of the co-resident blocks is preferred equally often, and they finish together.
            constexpr uint32_t RES = T::MIN_WAVES;
            const uint32_t age = ((blockIdx.y * gridDim.x + blockIdx.x) * RES) / (gridDim.x * gridDim.y);
            auto step = [&](auto k_tag) -> bool {    // true = all tiles rotated
                constexpr uint32_t K = decltype(k_tag)::value;
                if (q[1] >= n_full) return true;
                if constexpr (K == 0 && TQ_PRIO_SHIFT > 0) {
                    if ((done & ((1u << TQ_PRIO_SHIFT) - 1u)) == 0u) {
                        const uint32_t prio = (age + (done >> TQ_PRIO_SHIFT)) % RES;
                        if (prio == 0u) __builtin_amdgcn_s_setprio(0);
                        else if (prio == 1u) __builtin_amdgcn_s_setprio(1);
                        else __builtin_amdgcn_s_setprio(2);
                    }
                }
                if constexpr (K & 1u) iteration(std::true_type{}, std::integral_constant<uint32_t, K % P>{}, done >= (uint32_t)P, 1u, acc_b, acc_a);
                else iteration(std::true_type{}, std::integral_constant<uint32_t, K % P>{}, done >= (uint32_t)P, 0u, acc_a, acc_b);
                ++done;
                return false;
            };
            bool fin = run_tail<1, U>(step);         // the first trip starts at iteration 1
            while (!fin) fin = run_tail<0, U>(step);
            // the accumulator set filled last belongs to iteration done - 1
            if (done & 1u) drain(1u, acc_a); else drain(0u, acc_b);
            wait_vmcnt<0>();       // re-reads past the last tile may still be on their way into the ring
            __syncthreads();
            tile = q[1];           // where the sequence left the full tiles: n_full itself in the one block whose turn the partial tile is
            buf = 0u;
        }
    } else if (!ticket_job && tile < n_full) {
        // General case (several rows with their own stride, fp32 elements).  Iteration k: start the
        // loads of tile k+1, barrier (publishes buffer k, and everyone has finished reading buffer
        // k-1), compute and store tile k, then park tile k+1 into the other buffer.  Loads, stores
        // and the wait for the loads sit in one straight line, unpredicated: s_waitcnt vmcnt(#stores).
        issue_loads(std::true_type{}, tile);
        park(0, pre);
        while (tile < n_full) {
            const uint32_t next = tile + tile_stride;
            issue_loads(std::true_type{}, next < n_full ? next : tile);
            __syncthreads();
            compute(buf, words, nrm);
            const uint32_t slot = tq_packed_slot(job, tile * 32u + n);
            store(job.idx_bytes + (size_t)slot * (8 * NB) + lane_slot, job.vec_norms + norm_slot(slot), words, nrm);
            buf ^= 1u;
            park(buf, pre);
            tile = next;
        }
    }
    // the partial last tile of the job, if this block is the one whose turn it is
    if (tile == n_full && n_full < n_tiles) {
        issue_loads(std::false_type{}, tile);
        park(buf, pre);
        __syncthreads();
        compute(buf, words, nrm);
        const uint32_t v = tile * 32u + n;
        if (v < job.n_vec) {
            const uint32_t slot = tq_packed_slot(job, v);
            store(job.idx_bytes + (size_t)slot * (8 * NB) + lane_slot, job.vec_norms + norm_slot(slot), words, nrm);
        }
    }
    report_done();
}

// ---- host side --------------------------------------------------------------------------

constexpr int MAX_DEVICES = 64;
std::mutex host_state_mutex;   // guards the per-device tables below (filled once per device, read often)

struct DeviceInfo {
    int dev = 0;
    int cus = 0;
    int lds_optin = 0;
};
int query_device(DeviceInfo &info) {
    static DeviceInfo cache[MAX_DEVICES];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return TQ_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(host_state_mutex);
    if (cache[dev].cus == 0) {
        int cus = 0, lds = 0;
        e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return (int)e;
        e = hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
        if (e != hipSuccess) return (int)e;
        cache[dev].dev = dev;
        cache[dev].lds_optin = lds;
        cache[dev].cus = cus > 0 ? cus : 1;
    }
    info = cache[dev];
    return 0;
}

#ifndef TQ_COMPRESS_TICKET_SHIFT
#define TQ_COMPRESS_TICKET_SHIFT 3
#endif

template <int DTYPE, int BITS>
int launch_compress(const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_tiles, void *workspace, bool paired, hipStream_t stream) {
    DeviceInfo info;
    int rc = query_device(info);
    if (rc) return rc;
    // blocks resident per compute unit for this instantiation (registers and LDS decide): the grid
    // is that many blocks per unit, each walking its share of the tiles.  Asked once per device.
    int resident;
    {
        static int resident_on[MAX_DEVICES] = {};
        std::lock_guard<std::mutex> lock(host_state_mutex);
        if (resident_on[info.dev] == 0) {
            int nb = 0;
            hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, tq_compress_kernel<DTYPE, BITS>, CTHREADS, 0);
            if (e != hipSuccess) return (int)e;
            resident_on[info.dev] = nb > 0 ? nb : 1;
        }
        resident = resident_on[info.dev];
    }
    // Tickets from a counter pay off once every block has several to draw; below that (and without a workspace) the
    // blocks walk single tiles b, b + grid, ..., which splits a small job most evenly.
    uint32_t bx = tq_blocks_per_job(max_tiles, info.cus * resident, n_jobs);
    uint32_t tshift = 0;
    uint32_t *counters = nullptr;
    if (workspace && InTraits<DTYPE>::ELEM == 2 && TQ_COMPRESS_TICKET_SHIFT > 0) {
        const uint32_t tickets = (max_tiles + (1u << TQ_COMPRESS_TICKET_SHIFT) - 1u) >> TQ_COMPRESS_TICKET_SHIFT;
        const uint32_t bt = tq_blocks_per_job(tickets, info.cus * resident, n_jobs);
        if (tickets >= 4u * bt) {
            bx = bt;
            tshift = TQ_COMPRESS_TICKET_SHIFT;
            counters = static_cast<uint32_t *>(workspace);
        }
    }
    dim3 grid(bx, (unsigned)n_jobs, 1), block(CTHREADS, 1, 1);
    hipLaunchKernelGGL((tq_compress_kernel<DTYPE, BITS>), grid, block, 0, stream, job, jobs_dev, counters, tshift, paired ? 1u : 0u);
    return (int)hipGetLastError();
}

template <int DTYPE>
int dispatch_bits(int bits, const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_tiles, void *ws, bool paired, hipStream_t s) {
    switch (bits) {
        case 1: return launch_compress<DTYPE, 1>(job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        case 2: return launch_compress<DTYPE, 2>(job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        case 3: return launch_compress<DTYPE, 3>(job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        case 4: return launch_compress<DTYPE, 4>(job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        case 5: case 6: case 7: case 8:  // one code per byte: identical packing
            return launch_compress<DTYPE, 8>(job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        default: return TQ_ERR_BITS;
    }
}

int dispatch(int dtype, int bits, const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_tiles, void *ws, bool paired, hipStream_t s) {
    switch (dtype) {
        case TQ_F32: return dispatch_bits<TQ_F32>(bits, job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        case TQ_F16: return dispatch_bits<TQ_F16>(bits, job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        case TQ_BF16: return dispatch_bits<TQ_BF16>(bits, job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        default: return TQ_ERR_DTYPE;
    }
}

int elem_bytes(int dtype) { return dtype == TQ_F32 ? 4 : (dtype == TQ_F16 || dtype == TQ_BF16) ? 2 : 0; }

// Shared argument checks of one job; fills n_vec.
int check_job(const void *states, int dtype, long long rows, long long tokens, long long row_stride,
              long long token_stride, const void *table, int head_dim, int bits, const void *idx_bytes,
              const void *vec_norms, long long packed_row_stride, long long *n_vec) {
    if (bits < 1 || bits > 8) return TQ_ERR_BITS;
    if (head_dim != TQ_HEAD_DIM && !tq_anydim_supported(head_dim)) return TQ_ERR_HEAD_DIM;
    const int eb = elem_bytes(dtype);
    if (!eb) return TQ_ERR_DTYPE;
    if (rows < 0 || tokens < 0) return TQ_ERR_SIZE;
    if (rows != 0 && tokens > (long long)0x7fffffff / rows) return TQ_ERR_SIZE;
    *n_vec = rows * tokens;
    if (*n_vec == 0) return TQ_OK;
    if (!states || !table || !idx_bytes || !vec_norms) return TQ_ERR_NULL;
    if (token_stride < head_dim && tokens > 1) return TQ_ERR_SIZE;
    if (rows > 1 && row_stride < 0) return TQ_ERR_SIZE;
    if (packed_row_stride != 0 && (packed_row_stride < tokens || packed_row_stride > (long long)0x7fffffff / rows)) return TQ_ERR_SIZE;
    const uintptr_t va = tq_vector_alignment(head_dim, eb) - 1u;
    if (((uintptr_t)states & va) || ((uintptr_t)table & 15u) || ((uintptr_t)idx_bytes & (tq_packed_alignment(head_dim, bits) - 1u)) || ((uintptr_t)vec_norms & 1u))
        return TQ_ERR_ALIGN;
    if (((uintptr_t)(token_stride * eb) & va) || (rows > 1 && ((uintptr_t)(row_stride * eb) & va))) return TQ_ERR_ALIGN;
    return TQ_OK;
}

}  // namespace

extern "C" int tq_compress(const void *states, int dtype, long long rows, long long tokens,
                           long long row_stride, long long token_stride, const void *table_dev,
                           int head_dim, int bits, uint8_t *idx_bytes, uint16_t *vec_norms,
                           long long packed_row_stride, void *workspace, void *stream) {
    long long n_vec = 0;
    const int rc = check_job(states, dtype, rows, tokens, row_stride, token_stride, table_dev, head_dim, bits,
                             idx_bytes, vec_norms, packed_row_stride, &n_vec);
    if (rc) return rc;
    if ((uintptr_t)workspace & 63u) return TQ_ERR_ALIGN;
    if (n_vec == 0) return TQ_OK;
    TqDevJob job;
    job.states = static_cast<const uint8_t *>(states);
    job.idx_bytes = idx_bytes;
    job.vec_norms = vec_norms;
    job.table = static_cast<const uint8_t *>(table_dev);
    job.n_vec = (uint32_t)n_vec;
    job.tokens = (uint32_t)tokens;
    job.packed_row_stride = (uint32_t)(packed_row_stride ? packed_row_stride : tokens);
    job.row_stride = row_stride * elem_bytes(dtype);
    job.token_stride = token_stride * elem_bytes(dtype);
    if (head_dim == TQ_HEAD_DIM / 2 && tq_pairable(rows, tokens, token_stride, packed_row_stride, head_dim, idx_bytes))
        return dispatch(dtype, bits, job, nullptr, 1, (uint32_t)((n_vec / 2 + 31) / 32), workspace, true, static_cast<hipStream_t>(stream));
    if (head_dim != TQ_HEAD_DIM)
        return tq_anydim_compress(dtype, bits, head_dim, job, nullptr, 1, (uint32_t)n_vec, static_cast<hipStream_t>(stream));
    return dispatch(dtype, bits, job, nullptr, 1, (uint32_t)((n_vec + 31) / 32), workspace, false, static_cast<hipStream_t>(stream));
}

extern "C" int tq_compress_batched(const tq_job *jobs_host, const tq_job *jobs_dev, int n_jobs,
                                   int head_dim, void *workspace, void *stream) {
    if (n_jobs == 0) return TQ_OK;
    if (!jobs_host || !jobs_dev) return TQ_ERR_NULL;
    if (n_jobs < 0 || n_jobs > TQ_MAX_JOBS) return TQ_ERR_SIZE;
    if ((uintptr_t)workspace & 63u) return TQ_ERR_ALIGN;
    long long max_vec = 0;
    bool paired = head_dim == TQ_HEAD_DIM / 2;     // 64-wide vectors in pairs, if every job of the launch allows it
    for (int i = 0; i < n_jobs; ++i) {
        const tq_job &j = jobs_host[i];
        if (j.bits != jobs_host[0].bits) return TQ_ERR_BITS;
        if (j.dtype != jobs_host[0].dtype) return TQ_ERR_DTYPE;
        long long n_vec = 0;
        const int rc = check_job(j.states, j.dtype, j.rows, j.tokens, j.row_stride, j.token_stride, j.table_dev,
                                 head_dim, j.bits, j.idx_bytes, j.vec_norms, j.packed_row_stride, &n_vec);
        if (rc) return rc;
        if (n_vec > max_vec) max_vec = n_vec;
        if (n_vec && !tq_pairable(j.rows, j.tokens, j.token_stride, j.packed_row_stride, head_dim, j.idx_bytes)) paired = false;
    }
    if (max_vec == 0) return TQ_OK;
    TqDevJob none{};
    if (paired)
        return dispatch(jobs_host[0].dtype, jobs_host[0].bits, none, jobs_dev, n_jobs, (uint32_t)((max_vec / 2 + 31) / 32),
                        workspace, true, static_cast<hipStream_t>(stream));
    if (head_dim != TQ_HEAD_DIM)
        return tq_anydim_compress(jobs_host[0].dtype, jobs_host[0].bits, head_dim, none, jobs_dev, n_jobs, (uint32_t)max_vec,
                                  static_cast<hipStream_t>(stream));
    return dispatch(jobs_host[0].dtype, jobs_host[0].bits, none, jobs_dev, n_jobs, (uint32_t)((max_vec + 31) / 32),
                    workspace, false, static_cast<hipStream_t>(stream));
}
