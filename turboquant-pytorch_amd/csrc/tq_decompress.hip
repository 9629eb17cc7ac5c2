// decompress: unpack codes, centroid lookup, inverse rotation on the matrix cores, norm rescale,
// cast to the output type, coalesced store (optionally straight into a strided slice of the
// full-length K/V buffer).  Replaces MSECompressor.decompress (upstream
// turboquant/compressors_v3.py:84-105) and the cast + concatenation of
// TurboQuantV3.decompress_kv (:226-232) with one kernel.
//
// A wave owns 32 consecutive vectors.  Lane (n, hk) reads the packed bytes of codes
// [64*hk, 64*hk+64) of vector n, turns every byte into the fp16 centroids it holds with one
// LDS table lookup (the table is indexed by the whole byte, so 2-, 4- and 8-per-byte widths
// cost 1/2, 1/4, 1/8 lookup per code) and feeds them as the B operand of
// v_mfma_f32_32x32x16_f16; the A operand is Pi^T in fp16, fp32 accumulate.  The 32x128 result
// tile is transposed through a wave-private, XOR-swizzled LDS buffer so that every store
// instruction writes 1 KiB of consecutive memory.
//
// Which tiles a block works on.  A block draws "tickets": one ticket = WAVES consecutive tiles,
// one per wave.  A block's first ticket is fixed (block b: tiles b * WAVES ...), so its loads start before the tables
// are staged; with a workspace the later tickets of a job come from a counter in device memory
// (atomicAdd), so the blocks walk through the job in the order in which they become free and the
// addresses being written at any moment stay within a few MiB of each other; on this part that
// write pattern reaches 10-15 % more bandwidth than a fixed assignment (block b takes tickets
// b, b + grid, ...), under which fast and slow blocks drift apart.  Without a workspace, and for
// jobs too small to matter, the fixed assignment is used.  Thread 0 draws one ticket ahead and
// hands it to the block through LDS; one barrier per ticket.  The last block of a job to finish
// sets the job's counters back to zero, so a workspace that was zero before a launch is zero after it.
#include <mutex>
#include <type_traits>

#include "tq_anydim.h"
#include "tq_device.h"

// Ticket counters of tq_decompress_batched_noalloc: the workspace that tq_decompress_batched takes from its
// caller, held by the library instead (TQ_NOALLOC_MAX_JOBS jobs x TQ_WORKSPACE_BYTES_PER_JOB bytes on every
// device the library runs on, until the process ends).  In host code this name is only a handle for
// hipGetSymbolAddress; launches receive the per-device address kept by static_counters().
static __device__ __align__(256) uint32_t scratch[TQ_NOALLOC_MAX_JOBS * (TQ_WORKSPACE_BYTES_PER_JOB / 4)];

// Measurement build (never the shipped library): full tiles keep their loads, the scale / cast / transposition through
// LDS and their stores, and leave out the decode, the matrix instructions and their operand reads.  What it writes is
// garbage; its time is what the kernel's memory pattern costs on its own.
#ifndef TQ_SKELETON
#define TQ_SKELETON 0
#endif

namespace {

template <int DTYPE> struct OutTraits;
template <> struct OutTraits<TQ_F16> { static constexpr int ELEM = 2, WAVES = 8; };
template <> struct OutTraits<TQ_BF16> { static constexpr int ELEM = 2, WAVES = 8; };
template <> struct OutTraits<TQ_F32> { static constexpr int ELEM = 4, WAVES = 4; };

constexpr int LUT_LDS_BYTES = 4096;

template <int DTYPE>
constexpr size_t decompress_lds_bytes() {
    using T = OutTraits<DTYPE>;
    return (size_t)TQ_OPERAND_BYTES + LUT_LDS_BYTES + (size_t)T::WAVES * 32 * TQ_HEAD_DIM * T::ELEM;
}

__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

template <int DTYPE, int IPB>
__global__ __launch_bounds__(OutTraits<DTYPE>::WAVES *TQ_WAVE) void tq_decompress_kernel(TqDevJob job0, const tq_job *jobs, uint32_t *workspace, uint32_t paired) {
    using T = OutTraits<DTYPE>;
    constexpr int ELEM = T::ELEM;
    constexpr int VEC_BYTES = TQ_HEAD_DIM * ELEM;   // 256 or 512
    constexpr int STAGE = 32 * VEC_BYTES;
    constexpr int NSTORE = STAGE / 1024;            // 16-byte stores per lane per tile
    constexpr int PIECES = VEC_BYTES / 16;          // 16-byte pieces per vector: 16 or 32
    constexpr int VEC_PER_STORE = 64 / PIECES;
    constexpr int NB = 64 / IPB;                    // packed bytes per lane
    constexpr int NW = NB / 4;                      // dwords per lane: 2, 4, 8, 16

    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

    // paired: the job's vectors are 64 wide; two neighbours are one 128-wide row here (diag(Pi, Pi)^T from the table's pair
    // section).  Lane half hk decodes and produces the second vector of the pair; only its norm is its own.
    const TqDevJob job = tq_pair_job(tq_load_job(job0, jobs, blockIdx.y, ELEM), paired != 0u);
    uint8_t *out_base = const_cast<uint8_t *>(job.states);

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t n_tiles = (job.n_vec + 31u) / 32u;
    if (n_tiles == 0u) return;   // an empty job of a batch: its table may be NULL, and its counters stay untouched (zero)

    const TqTableHeader *hd = reinterpret_cast<const TqTableHeader *>(job.table);
    uint8_t *lds_a = lds;
    uint8_t *lds_lut = lds + TQ_OPERAND_BYTES;
    uint8_t *stage = lds_lut + LUT_LDS_BYTES + wave * STAGE;

    // tickets: counter[0] = tiles handed out beyond every block's first ticket, counter[1] = blocks of this job that are done.
    // The first ticket of a block is fixed (block b: tiles b * WAVES ...), so its loads can start before anything else.
    __shared__ uint32_t tk[3];         // ticket k of the block sits in slot k % 3
    uint32_t *counter = workspace ? workspace + blockIdx.y * (TQ_WORKSPACE_BYTES_PER_JOB / 4) : nullptr;
    const uint32_t first = blockIdx.x * T::WAVES;
    const uint32_t drawn_origin = gridDim.x * T::WAVES;
    uint32_t fixed_next = first + drawn_origin;
    // thread 0 only.  The ticket is computed from the atomic's result on the spot, which makes the drawing wave wait for
    // its own outstanding loads and stores once per ticket.  Measured against a form that leaves the result untouched
    // until it is published a tile later (no wait at the draw): the launches of the Llama-3-8B 32K workload take
    // 318 / 382 / 300 us this way and 339 / 388 / 305 us that way (2-, 4-, 8-bit), so the wait stays.
    auto draw = [&]() -> uint32_t {
        if (counter) {
            const uint32_t t = drawn_origin + atomicAdd(counter, (uint32_t)T::WAVES);
            return t < n_tiles ? t : n_tiles;
        }
        const uint32_t t = fixed_next < n_tiles ? fixed_next : n_tiles;   // saturates: no wrap-around on huge grids
        fixed_next = t + drawn_origin;
        return t;
    };
    // Everything a block needs besides its first tile: Pi^T and the byte -> centroids table into LDS (all fetches
    // of a thread issued together), the second ticket, one barrier.  Called behind the first tile's loads.
    auto stage_tables = [&]() {
        constexpr int NT = T::WAVES * TQ_WAVE;
        constexpr int A_TRIPS = TQ_OPERAND_BYTES / 16 / NT;
        static_assert(A_TRIPS * NT * 16 == TQ_OPERAND_BYTES, "whole trips");
        const uint8_t *a_src = job.table + (paired ? hd->off_pair_at_f16 : hd->off_at_f16);
        tq_u4 v[A_TRIPS];
#pragma unroll
        for (int k = 0; k < A_TRIPS; ++k) v[k] = tq_gload16(a_src + 16u * (tid + k * NT));
        if (tid == 0) tk[1] = draw();
#pragma unroll
        for (int k = 0; k < A_TRIPS; ++k) reinterpret_cast<tq_u4 *>(lds_a)[tid + k * NT] = v[k];
        tq_copy_to_lds(lds_lut, job.table + hd->off_lut, 256u * 2u * IPB, tid, NT);
        __syncthreads();
    };

    uint32_t base = first;             // first tile of the block's current ticket (the same in every wave)
    uint32_t tile = base + wave;
    const uint32_t n = lane & 31u, hk = lane >> 5;
    const uint32_t st_vec = lane / PIECES, st_piece = lane % PIECES;

    // Addressing of a tile.  The tile index is the same for the whole wave, so the split of its first
    // vector into (row, token) is one scalar division per tile; the other vectors follow by adding
    // per-lane constants, plus one fixed correction for those past the end of the row (rows hold at
    // least 32 tokens on this path, so a tile crosses at most one row boundary).
    const bool one_row = job.tokens >= job.n_vec;
    const bool fast = (one_row || job.tokens >= 32u) && job.token_stride < (1ll << 24);
    struct Origin {
        long long out_base;   // byte offset of the tile's first vector in the output tensor
        uint32_t slot_base;   // its packed slot
        uint32_t in_row;      // vectors of the tile that still belong to that row
    };
    auto origin_of = [&](uint32_t tl) {
        Origin o;
        const uint32_t v0 = __builtin_amdgcn_readfirstlane(tl) * 32u;
        const uint32_t row = one_row ? 0u : v0 / job.tokens;
        const uint32_t tok = v0 - row * job.tokens;
        o.out_base = (long long)row * job.row_stride + (long long)tok * job.token_stride;
        o.slot_base = one_row ? tok : row * job.packed_row_stride + tok;
        o.in_row = one_row ? 32u : job.tokens - tok;
        return o;
    };
    // jump of the output offset / packed slot from the last vector of a row to the first of the next
    const long long row_wrap = job.row_stride - (long long)job.tokens * job.token_stride;
    const uint32_t slot_wrap = job.packed_row_stride - job.tokens;
    uint32_t st_off[NSTORE];   // byte offset of this lane's piece of store j relative to the tile's first vector
#pragma unroll
    for (int j = 0; j < NSTORE; ++j) st_off[j] = (j * VEC_PER_STORE + st_vec) * (uint32_t)job.token_stride + st_piece * 16u;

    uint32_t raw[NW];
    uint16_t norm_bits = 0;
    // this lane's half vector of tile `tl` (FULL: all 32 vectors of the tile exist, nothing is predicated)
    auto issue_loads = [&](auto full_tag, auto fast_tag, uint32_t tl) {
        constexpr bool FULL = decltype(full_tag)::value;
        constexpr bool FAST = decltype(fast_tag)::value;
        const bool ok = FULL || tl * 32u + n < job.n_vec;
        const uint32_t vl = ok ? n : 0u;
        uint32_t slot;
        if constexpr (FAST) {
            const Origin o = origin_of(tl);
            slot = o.slot_base + vl + (vl >= o.in_row ? slot_wrap : 0u);
        } else {   // rows shorter than a tile: the general formula
            slot = tq_packed_slot(job, tl * 32u + vl);
        }
        const uint8_t *src = job.idx_bytes + (size_t)slot * (2 * NB) + hk * NB;
        if constexpr (NW == 2) {
            const tq_u2 t = tq_gload8(src);
            raw[0] = t[0]; raw[1] = t[1];
        } else {
#pragma unroll
            for (int q = 0; q < NW / 4; ++q) {
                const tq_u4 t = tq_gload16(src + 16 * q);
#pragma unroll
                for (int i = 0; i < 4; ++i) raw[4 * q + i] = t[i];
            }
        }
        norm_bits = tq_gload2(job.vec_norms + (paired ? 2u * (size_t)slot + hk : (size_t)slot));
    };

    // one tile: decode + rotate + scale + transpose + store
    auto process = [&](auto full_tag, auto fast_tag, uint32_t tl, const uint32_t (&cur)[NW], float nrm) {
        constexpr bool FULL = decltype(full_tag)::value;
        constexpr bool FAST = decltype(fast_tag)::value;
        // ---- x_hat[64h + 16t + r] = sum_j y[j] * Pi[j][.]   (un-scaled)
        tq_f16v acc[TQ_TILES];
#pragma unroll
        for (int t = 0; t < TQ_TILES; ++t) acc[t] = tq_zero16();
#if TQ_SKELETON
#pragma unroll
        for (int t = 0; t < TQ_TILES; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][r] = __uint_as_float(cur[(4 * t + r) % NW] + (uint32_t)r);
#else
#pragma unroll
        for (int s = 0; s < TQ_STEPS; ++s) {
            const tq_u4 b = decode_step<IPB, NW>(cur, s, lds_lut);
            const tq_u4 *a_base = reinterpret_cast<const tq_u4 *>(lds_a) + (size_t)s * 64 + lane;
#pragma unroll
            for (int t = 0; t < TQ_TILES; ++t) {
                const tq_u4 a = a_base[t * TQ_STEPS * 64];
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(tq_half8, a),
                                                                __builtin_bit_cast(tq_half8, b), acc[t], 0, 0, 0);
            }
        }
#endif

        // ---- scale, cast, transpose through LDS.  Lane (n, hk) holds elements 64*hk + 16*t + r.
        if constexpr (ELEM == 2) {
#pragma unroll
            for (int t = 0; t < TQ_TILES; ++t)
#pragma unroll
                for (int c = 0; c < 2; ++c) {  // two 16-byte pieces of 8 elements per MFMA tile
                    tq_u4 o;
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const float x0 = acc[t][8 * c + 2 * d] * nrm, x1 = acc[t][8 * c + 2 * d + 1] * nrm;
                        if constexpr (DTYPE == TQ_F16) {
                            const tq_half2 h = {(_Float16)x0, (_Float16)x1};
                            o[d] = __builtin_bit_cast(uint32_t, h);
                        } else {
                            const tq_bf2 h = {(__bf16)x0, (__bf16)x1};
                            o[d] = __builtin_bit_cast(uint32_t, h);
                        }
                    }
                    const uint32_t piece = 8u * hk + 2u * t + c;
                    *reinterpret_cast<tq_u4 *>(stage + n * VEC_BYTES + ((piece ^ (n & 15u)) << 4)) = o;
                }
        } else {
#pragma unroll
            for (int t = 0; t < TQ_TILES; ++t)
#pragma unroll
                for (int c = 0; c < 4; ++c) {  // four 16-byte pieces of 4 floats per MFMA tile
                    tq_u4 o;
#pragma unroll
                    for (int d = 0; d < 4; ++d) o[d] = __float_as_uint(acc[t][4 * c + d] * nrm);
                    const uint32_t piece = 16u * hk + 4u * t + c;
                    *reinterpret_cast<tq_u4 *>(stage + n * VEC_BYTES + ((piece ^ n) << 4)) = o;
                }
        }
        tq_u4 val[NSTORE];
#pragma unroll
        for (int j = 0; j < NSTORE; ++j) {
            const uint32_t vl = j * VEC_PER_STORE + st_vec;
            const uint32_t swz = (ELEM == 2) ? (vl & 15u) : vl;
            val[j] = *reinterpret_cast<const tq_u4 *>(stage + vl * VEC_BYTES + ((st_piece ^ swz) << 4));
        }
        if constexpr (FAST) {
            const Origin o = origin_of(tl);
            uint8_t *base = out_base + o.out_base;
#pragma unroll
            for (int j = 0; j < NSTORE; ++j) {
                const uint32_t vl = j * VEC_PER_STORE + st_vec;
                if (FULL || tl * 32u + vl < job.n_vec)
                    tq_gstore16_stream(base + st_off[j] + (vl >= o.in_row ? row_wrap : 0ll), val[j]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < NSTORE; ++j) {
                const uint32_t vl = j * VEC_PER_STORE + st_vec;
                if (FULL || tl * 32u + vl < job.n_vec)
                    tq_gstore16_stream(out_base + tq_vec_offset(job, tl * 32u + vl) + st_piece * 16u, val[j]);
            }
        }
    };

    // Tiles whose 32 vectors all exist: the loads of the next tile are always issued (past the end: the
    // current tile again, never used) and nothing is predicated, so loads -> stores -> wait for the loads
    // leaves the stores in flight (s_waitcnt vmcnt(#stores)) instead of draining them every iteration.
    // The loop runs once per ticket of the block, the same number of times in every wave (the barrier).
    const uint32_t n_full = job.n_vec / 32u;
    auto run = [&](auto fast_tag) {
        uint32_t cur[NW];
        float nrm = 0.f;
        if (tile < n_full) issue_loads(std::true_type{}, fast_tag, tile);
        stage_tables();
        if (tile < n_full) {
#pragma unroll
            for (int i = 0; i < NW; ++i) cur[i] = raw[i];
            nrm = half_bits_to_float(norm_bits);
        }
        uint32_t s_next = 1u, s_fresh = 2u;                // slots of the next ticket and of the one drawn now
        while (base < n_tiles) {
            uint32_t fresh = 0;
            if (tid == 0) fresh = draw();                 // the ticket after next; its latency hides behind the tile
            const uint32_t nbase = tk[s_next];             // written before the previous barrier
            const uint32_t next = nbase + wave;
            if (tile < n_full) {
                issue_loads(std::true_type{}, fast_tag, next < n_full ? next : tile);
                asm volatile("" ::: "memory");          // the prefetch stays ahead of the tile's work
                process(std::true_type{}, fast_tag, tile, cur, nrm);
                // take the prefetched registers here, behind the stores: the wait for them then sits inside
                // the loop body, where the number of younger stores is known
#pragma unroll
                for (int i = 0; i < NW; ++i) {
                    asm volatile("" : "+v"(raw[i]));
                    cur[i] = raw[i];
                }
                uint32_t nb = norm_bits;
                asm volatile("" : "+v"(nb));
                nrm = half_bits_to_float((uint16_t)nb);
            } else if (tile == n_full && n_full < n_tiles) {   // the partial last tile of the job
                issue_loads(std::false_type{}, fast_tag, tile);
                uint32_t part[NW];
#pragma unroll
                for (int i = 0; i < NW; ++i) part[i] = raw[i];
                process(std::false_type{}, fast_tag, tile, part, half_bits_to_float(norm_bits));
            }
            if (tid == 0) tk[s_fresh] = fresh;             // last read two barriers ago (three slots, not two: the first
            __syncthreads();                               // ticket is read after a barrier that this write could overtake)
            base = nbase;
            tile = next;
            s_next = s_fresh;
            s_fresh = s_fresh == 2u ? 0u : s_fresh + 1u;
        }
    };
    if (fast) run(std::true_type{}); else run(std::false_type{});

    // Every ticket this block drew has been answered (the values went through LDS) before it reports itself
    // done, so the block that finds all others done knows that nobody touches the counters again in this
    // launch.  All accesses to the counters are device-scope atomics, which are performed in one place;
    // no fence is needed, and a release fence here would write back the L2's share of the output first.
    if (counter && tid == 0) {
        if (atomicAdd(counter + 1, 1u) == gridDim.x - 1u) {
            atomicExch(counter, 0u);
            atomicExch(counter + 1, 0u);
        }
    }
}

// Sets n 32-bit words to zero.  A kernel rather than hipMemsetAsync, so that a caller may record the launch
// into a HIP graph.
__global__ void tq_clear_words_kernel(uint32_t *p, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// ---- host side --------------------------------------------------------------------------

constexpr int MAX_DEVICES = 64;
std::mutex host_state_mutex;   // guards the per-device tables below (filled once per device, read often)

int device_cus(int &cus) {
    static int cache[MAX_DEVICES] = {};
    int dev = 0;
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

// Address of `scratch` on the current device.  Every device holds its own copy of the array at its own
// address, so the address is looked up once per device, with that device current, and kept.
int static_counters(uint32_t **out) {
    static uint32_t *address[MAX_DEVICES] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return TQ_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(host_state_mutex);
    if (!address[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return TQ_ERR_NO_DEVICE;
        address[dev] = static_cast<uint32_t *>(p);
    }
    *out = address[dev];
    return 0;
}

template <int DTYPE, int IPB>
int launch_decompress(const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_tiles, void *workspace, bool paired,
                      hipStream_t stream) {
    using T = OutTraits<DTYPE>;
    int cus = 0;
    int rc = device_cus(cus);
    if (rc) return rc;
    constexpr size_t lds = decompress_lds_bytes<DTYPE>();
    {   // the kernel's LDS limit is raised once per device (one flag table per instantiation)
        static bool configured[MAX_DEVICES] = {};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return (int)e;
        if (dev < 0 || dev >= MAX_DEVICES) return TQ_ERR_NO_DEVICE;
        std::lock_guard<std::mutex> lock(host_state_mutex);
        if (!configured[dev]) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(&tq_decompress_kernel<DTYPE, IPB>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            configured[dev] = true;
        }
    }
    const uint32_t want = (max_tiles + T::WAVES - 1) / T::WAVES;
    const uint32_t bx = tq_blocks_per_job(want, cus, n_jobs);
    dim3 grid(bx, (unsigned)n_jobs, 1), block(T::WAVES * TQ_WAVE, 1, 1);
    // tickets pay off once every block has several to draw; below that the fixed assignment starts sooner
    uint32_t *counters = want >= 4u * bx ? static_cast<uint32_t *>(workspace) : nullptr;
    hipLaunchKernelGGL((tq_decompress_kernel<DTYPE, IPB>), grid, block, lds, stream, job, jobs_dev, counters, paired ? 1u : 0u);
    return (int)hipGetLastError();
}

template <int DTYPE>
int dispatch_bits(int bits, const TqDevJob &job, const tq_job *jobs_dev, int n_jobs, uint32_t max_tiles, void *ws, bool paired, hipStream_t s) {
    switch (8 / bits) {
        case 8: return launch_decompress<DTYPE, 8>(job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        case 4: return launch_decompress<DTYPE, 4>(job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        case 2: return launch_decompress<DTYPE, 2>(job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
        case 1: return launch_decompress<DTYPE, 1>(job, jobs_dev, n_jobs, max_tiles, ws, paired, s);
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

int check_job(const void *out, int dtype, long long rows, long long tokens, long long row_stride,
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
    if (!out || !table || !idx_bytes || !vec_norms) return TQ_ERR_NULL;
    if (token_stride < head_dim && tokens > 1) return TQ_ERR_SIZE;
    if (rows > 1 && row_stride < 0) return TQ_ERR_SIZE;
    if (packed_row_stride != 0 && (packed_row_stride < tokens || packed_row_stride > (long long)0x7fffffff / rows)) return TQ_ERR_SIZE;
    const uintptr_t va = tq_vector_alignment(head_dim, eb) - 1u;
    if (((uintptr_t)out & va) || ((uintptr_t)table & 15u) || ((uintptr_t)idx_bytes & (tq_packed_alignment(head_dim, bits) - 1u)) || ((uintptr_t)vec_norms & 1u))
        return TQ_ERR_ALIGN;
    if (((uintptr_t)(token_stride * eb) & va) || (rows > 1 && ((uintptr_t)(row_stride * eb) & va))) return TQ_ERR_ALIGN;
    return TQ_OK;
}

}  // namespace

extern "C" int tq_decompress(const uint8_t *idx_bytes, const uint16_t *vec_norms, long long packed_row_stride,
                             long long rows, long long tokens,
                             const void *table_dev, int head_dim, int bits, void *out, int out_dtype,
                             long long row_stride, long long token_stride, void *workspace, void *stream) {
    long long n_vec = 0;
    const int rc = check_job(out, out_dtype, rows, tokens, row_stride, token_stride, table_dev, head_dim, bits,
                             idx_bytes, vec_norms, packed_row_stride, &n_vec);
    if (rc) return rc;
    if ((uintptr_t)workspace & 63u) return TQ_ERR_ALIGN;
    if (n_vec == 0) return TQ_OK;
    TqDevJob job;
    job.states = static_cast<const uint8_t *>(out);
    job.idx_bytes = const_cast<uint8_t *>(idx_bytes);
    job.vec_norms = const_cast<uint16_t *>(vec_norms);
    job.table = static_cast<const uint8_t *>(table_dev);
    job.n_vec = (uint32_t)n_vec;
    job.tokens = (uint32_t)tokens;
    job.packed_row_stride = (uint32_t)(packed_row_stride ? packed_row_stride : tokens);
    job.row_stride = row_stride * elem_bytes(out_dtype);
    job.token_stride = token_stride * elem_bytes(out_dtype);
    if (head_dim == TQ_HEAD_DIM / 2 && tq_pairable(rows, tokens, token_stride, packed_row_stride, head_dim, idx_bytes))
        return dispatch(out_dtype, bits, job, nullptr, 1, (uint32_t)((n_vec / 2 + 31) / 32), workspace, true, static_cast<hipStream_t>(stream));
    if (head_dim != TQ_HEAD_DIM)     // the run-time-dimension kernel assigns its tiles statically: no counters
        return tq_anydim_decompress(out_dtype, bits, head_dim, job, nullptr, 1, (uint32_t)n_vec, static_cast<hipStream_t>(stream));
    return dispatch(out_dtype, bits, job, nullptr, 1, (uint32_t)((n_vec + 31) / 32), workspace, false, static_cast<hipStream_t>(stream));
}

extern "C" long long tq_workspace_bytes(int n_jobs) {
    if (n_jobs < 0 || n_jobs > TQ_MAX_JOBS) return TQ_ERR_SIZE;
    return (long long)TQ_WORKSPACE_BYTES_PER_JOB * (n_jobs > 0 ? n_jobs : 1);
}

namespace {
// Argument checks of a batch; max_vec = vectors of its largest job (0: nothing to launch).
int check_batch(const tq_job *jobs_host, int n_jobs, int head_dim, long long *max_vec, bool *paired) {
    *max_vec = 0;
    *paired = head_dim == TQ_HEAD_DIM / 2;       // 64-wide vectors in pairs, if every job of the launch allows it
    for (int i = 0; i < n_jobs; ++i) {
        const tq_job &j = jobs_host[i];
        if (8 / (j.bits < 1 || j.bits > 8 ? 1 : j.bits) != 8 / (jobs_host[0].bits < 1 || jobs_host[0].bits > 8 ? 1 : jobs_host[0].bits))
            return TQ_ERR_BITS;
        if (j.dtype != jobs_host[0].dtype) return TQ_ERR_DTYPE;
        long long n_vec = 0;
        const int rc = check_job(j.states, j.dtype, j.rows, j.tokens, j.row_stride, j.token_stride, j.table_dev,
                                 head_dim, j.bits, j.idx_bytes, j.vec_norms, j.packed_row_stride, &n_vec);
        if (rc) return rc;
        if (n_vec > *max_vec) *max_vec = n_vec;
        if (n_vec && !tq_pairable(j.rows, j.tokens, j.token_stride, j.packed_row_stride, head_dim, j.idx_bytes)) *paired = false;
    }
    return TQ_OK;
}

int launch_batch(const tq_job *jobs_host, const tq_job *jobs_dev, int n_jobs, int head_dim, long long max_vec, bool paired,
                 void *workspace, void *stream) {
    TqDevJob none{};
    if (paired)
        return dispatch(jobs_host[0].dtype, jobs_host[0].bits, none, jobs_dev, n_jobs, (uint32_t)((max_vec / 2 + 31) / 32),
                        workspace, true, static_cast<hipStream_t>(stream));
    if (head_dim != TQ_HEAD_DIM)
        return tq_anydim_decompress(jobs_host[0].dtype, jobs_host[0].bits, head_dim, none, jobs_dev, n_jobs, (uint32_t)max_vec,
                                    static_cast<hipStream_t>(stream));
    return dispatch(jobs_host[0].dtype, jobs_host[0].bits, none, jobs_dev, n_jobs, (uint32_t)((max_vec + 31) / 32),
                    workspace, false, static_cast<hipStream_t>(stream));
}
}  // namespace

extern "C" int tq_decompress_batched(const tq_job *jobs_host, const tq_job *jobs_dev, int n_jobs,
                                     int head_dim, void *workspace, void *stream) {
    if (n_jobs == 0) return TQ_OK;
    if (!jobs_host || !jobs_dev) return TQ_ERR_NULL;
    if (n_jobs < 0 || n_jobs > TQ_MAX_JOBS) return TQ_ERR_SIZE;
    if ((uintptr_t)workspace & 63u) return TQ_ERR_ALIGN;
    long long max_vec = 0;
    bool paired = false;
    const int rc = check_batch(jobs_host, n_jobs, head_dim, &max_vec, &paired);
    if (rc || max_vec == 0) return rc;
    return launch_batch(jobs_host, jobs_dev, n_jobs, head_dim, max_vec, paired, workspace, stream);
}

extern "C" int tq_decompress_batched_noalloc(const tq_job *jobs_host, const tq_job *jobs_dev, int n_jobs,
                                             int head_dim, void *stream) {
    if (n_jobs == 0) return TQ_OK;
    if (!jobs_host || !jobs_dev) return TQ_ERR_NULL;
    if (n_jobs < 0) return TQ_ERR_SIZE;
    if (n_jobs > TQ_NOALLOC_MAX_JOBS) return TQ_ERR_CAPACITY;
    // every argument is checked before anything is launched: an argument error leaves the stream untouched
    long long max_vec = 0;
    bool paired = false;
    int rc = check_batch(jobs_host, n_jobs, head_dim, &max_vec, &paired);
    if (rc || max_vec == 0) return rc;
    uint32_t *counters = nullptr;
    rc = static_counters(&counters);
    if (rc) return rc;
    // The array keeps what the last call left.  A launch that completed left zeros, one that failed half-way
    // may not have: the words this call uses are cleared first, on the same stream.
    const uint32_t words = (uint32_t)n_jobs * (TQ_WORKSPACE_BYTES_PER_JOB / 4);
    hipLaunchKernelGGL(tq_clear_words_kernel, dim3((words + 255u) / 256u), dim3(256), 0, static_cast<hipStream_t>(stream),
                       counters, words);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    return launch_batch(jobs_host, jobs_dev, n_jobs, head_dim, max_vec, paired, counters, stream);
}
