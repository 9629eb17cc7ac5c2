// Device-side helpers shared by the compress and decompress kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tqamd.h"
#include "tq_table.h"

typedef _Float16 tq_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 tq_half2 __attribute__((ext_vector_type(2)));
typedef __bf16 tq_bf8 __attribute__((ext_vector_type(8)));
typedef __bf16 tq_bf2 __attribute__((ext_vector_type(2)));
typedef float tq_f16v __attribute__((ext_vector_type(16)));
typedef uint32_t tq_u4 __attribute__((ext_vector_type(4)));
typedef uint32_t tq_u2 __attribute__((ext_vector_type(2)));

#define TQ_WAVE 64
#define TQ_GLOBAL __attribute__((address_space(1)))

// Launch-time job descriptor (device view of tq_job, plus derived fields).
struct TqDevJob {
    const uint8_t *states;   // compress input / decompress output, byte pointer
    uint8_t *idx_bytes;
    uint16_t *vec_norms;
    const uint8_t *table;
    uint32_t n_vec;          // rows * tokens  (< 2^31)
    uint32_t tokens;
    uint32_t packed_row_stride;  // packed slots per row (>= tokens)
    long long row_stride;    // bytes
    long long token_stride;  // bytes
};

__device__ __forceinline__ TqDevJob tq_load_job(const TqDevJob &single, const tq_job *jobs, uint32_t index, int elem_bytes) {
    if (!jobs) return single;
    const tq_job &j = jobs[index];
    TqDevJob job;
    job.states = static_cast<const uint8_t *>(j.states);
    job.idx_bytes = j.idx_bytes;
    job.vec_norms = j.vec_norms;
    job.table = static_cast<const uint8_t *>(j.table_dev);
    job.n_vec = (uint32_t)(j.rows * j.tokens);
    job.tokens = (uint32_t)j.tokens;
    job.packed_row_stride = (uint32_t)(j.packed_row_stride ? j.packed_row_stride : j.tokens);
    job.row_stride = j.row_stride * elem_bytes;
    job.token_stride = j.token_stride * elem_bytes;
    return job;
}

// Two 64-wide vectors that lie next to each other are one 128-wide row to the 128-wide kernels (rotated by diag(Pi, Pi)):
// the job seen that way.  The host has checked that every row holds an even number of tokens, 64 elements apart.
__device__ __forceinline__ TqDevJob tq_pair_job(TqDevJob j, bool paired) {
    if (paired) {
        j.n_vec >>= 1;
        j.tokens >>= 1;
        j.packed_row_stride >>= 1;
        j.token_stride <<= 1;
    }
    return j;
}

// The job's fields are the same in every lane of a block, but a record fetched from the job array arrives in vector
// registers (the compiler cannot prove that nobody writes the array).  Moving every field into scalar registers keeps
// them out of the vector register budget and lets the address arithmetic on them run on the scalar unit.
__device__ __forceinline__ uint32_t tq_uniform32(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint64_t tq_uniform64(uint64_t v) {
    return ((uint64_t)tq_uniform32((uint32_t)(v >> 32)) << 32) | (uint64_t)tq_uniform32((uint32_t)v);
}
__device__ __forceinline__ TqDevJob tq_uniform_job(const TqDevJob &j) {
    TqDevJob u;
    u.states = reinterpret_cast<const uint8_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.states));
    u.idx_bytes = reinterpret_cast<uint8_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.idx_bytes));
    u.vec_norms = reinterpret_cast<uint16_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.vec_norms));
    u.table = reinterpret_cast<const uint8_t *>((uintptr_t)tq_uniform64((uint64_t)(uintptr_t)j.table));
    u.n_vec = tq_uniform32(j.n_vec);
    u.tokens = tq_uniform32(j.tokens);
    u.packed_row_stride = tq_uniform32(j.packed_row_stride);
    u.row_stride = (long long)tq_uniform64((uint64_t)j.row_stride);
    u.token_stride = (long long)tq_uniform64((uint64_t)j.token_stride);
    return u;
}

// Byte offset of vector v inside `states`.
__device__ __forceinline__ long long tq_vec_offset(const TqDevJob &job, uint32_t v) {
    if (job.tokens >= job.n_vec) return (long long)v * job.token_stride;  // one row
    const uint32_t row = v / job.tokens;
    const uint32_t tok = v - row * job.tokens;
    return (long long)row * job.row_stride + (long long)tok * job.token_stride;
}

// Packed slot (index into idx_bytes rows and vec_norms) of vector v.
__device__ __forceinline__ uint32_t tq_packed_slot(const TqDevJob &job, uint32_t v) {
    if (job.tokens >= job.n_vec) return v;  // one row
    const uint32_t row = v / job.tokens;
    return row * job.packed_row_stride + (v - row * job.tokens);
}

// Global-memory accessors (explicit address space: plain pointers read from a descriptor
// would otherwise be accessed with flat instructions, which also occupy the LDS counter).
__device__ __forceinline__ tq_u4 tq_gload16(const uint8_t *p) {
    return *reinterpret_cast<const TQ_GLOBAL tq_u4 *>((const TQ_GLOBAL uint8_t *)p);
}
__device__ __forceinline__ tq_u2 tq_gload8(const uint8_t *p) {
    return *reinterpret_cast<const TQ_GLOBAL tq_u2 *>((const TQ_GLOBAL uint8_t *)p);
}
__device__ __forceinline__ uint16_t tq_gload2(const uint16_t *p) {
    return *((const TQ_GLOBAL uint16_t *)p);
}
// Streaming store for bulk output that this launch does not read again (the de-quantised tensors): the
// non-temporal hint keeps it out of the last-level cache.  Measured on the Llama-3-8B 32K workload: the 4- and
// 8-bit decompress launches 4-5 % faster (436 -> 413 us, 340 -> 327 us), and packed codes that fit the
// last-level cache stay there across launches.  The same hint on the compress kernel's loads changed nothing;
// on its packed-code stores it cost 45 % on the 8-bit launch.
__device__ __forceinline__ void tq_gstore16_stream(uint8_t *p, tq_u4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<TQ_GLOBAL tq_u4 *>((TQ_GLOBAL uint8_t *)p));
}
__device__ __forceinline__ void tq_gstore16(uint8_t *p, tq_u4 v) {
    *reinterpret_cast<TQ_GLOBAL tq_u4 *>((TQ_GLOBAL uint8_t *)p) = v;
}
__device__ __forceinline__ void tq_gstore8(uint8_t *p, tq_u2 v) {
    *reinterpret_cast<TQ_GLOBAL tq_u2 *>((TQ_GLOBAL uint8_t *)p) = v;
}
__device__ __forceinline__ void tq_gstore2(uint16_t *p, uint16_t v) {
    *((TQ_GLOBAL uint16_t *)p) = v;
}

// Cooperative copy global -> LDS, 16 bytes per thread per trip.
__device__ __forceinline__ void tq_copy_to_lds(uint8_t *dst, const uint8_t *src, uint32_t bytes,
                                               uint32_t tid, uint32_t nthreads) {
    tq_u4 *d = reinterpret_cast<tq_u4 *>(dst);
    for (uint32_t i = tid; i < bytes / 16; i += nthreads) d[i] = tq_gload16(src + 16u * i);
}

__device__ __forceinline__ tq_f16v tq_zero16() {
    tq_f16v z;
#pragma unroll
    for (int i = 0; i < 16; ++i) z[i] = 0.f;
    return z;
}

// ---- matrix-core and input helpers of the compress-side kernels -----------------------------------
static __device__ __forceinline__ tq_f16v mfma_f16(tq_u4 a, tq_u4 b, tq_f16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(tq_half8, a), __builtin_bit_cast(tq_half8, b), c, 0, 0, 0);
}
static __device__ __forceinline__ tq_f16v mfma_bf16(tq_u4 a, tq_u4 b, tq_f16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(tq_bf8, a), __builtin_bit_cast(tq_bf8, b), c, 0, 0, 0);
}

// sum of squares of the eight 16-bit values in v, added to acc (fp32).
// (Pairs are taken from the whole-vector cast: casting one 32-bit element of `v` to a 16-bit
// pair made the compiler read element 0 four times.)
template <int DTYPE>
static __device__ __forceinline__ float sumsq8(tq_u4 v, float acc) {
    if constexpr (DTYPE == TQ_F16) {
        const tq_half8 h8 = __builtin_bit_cast(tq_half8, v);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const tq_half2 h = {h8[2 * d], h8[2 * d + 1]};
            acc = __builtin_amdgcn_fdot2(h, h, acc, false);
        }
    } else {
        const tq_bf8 b8 = __builtin_bit_cast(tq_bf8, v);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const tq_bf2 b = {b8[2 * d], b8[2 * d + 1]};
            acc = __builtin_amdgcn_fdot2_f32_bf16(b, b, acc, false);
        }
    }
    return acc;
}

// Exact split of eight floats into three bf16 terms each (x = t0 + t1 + t2, every term a
// truncation, every remainder exact in fp32).  Output: packed bf16 operands.
static __device__ __forceinline__ void split_f32x8(const float (&x)[8], tq_u4 &t0, tq_u4 &t1, tq_u4 &t2) {
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

// ---- packing geometry -------------------------------------------------------------------
// A lane owns 16 consecutive codes = NB packed bytes, handled as NW words of WB bytes (a full
// dword, or the lane's 2 bytes for 1-bit codes).  Inside a word, code number i (in the order
// "highest byte first, most significant code of the byte first") sits at bit shift_of(i);
// FIELD is the spacing the sign-collecting funnel shift uses.
template <int BITS> struct Pack {
    static constexpr int IPB = 8 / BITS;                 // codes per byte
    static constexpr int NB = 16 / IPB;                  // bytes per lane: 2, 4, 8, 8, 16
    static constexpr int WB = NB < 4 ? NB : 4;           // bytes per word
    static constexpr int NW = NB / WB;                   // words per lane
    static constexpr int CPW = WB * IPB;                 // codes per word
    static constexpr int FIELD = IPB == 1 ? 8 : BITS;    // bits the funnel shift advances per code
    static constexpr int COPIES = TQ_GRID_COPIES(BITS);
    static constexpr int COPY_STRIDE = TQ_GRID_COPY_STRIDE(BITS);
    static constexpr int byte_of(int i) { return WB - 1 - i / IPB; }
    static constexpr int k_of(int i) { return i % IPB; }
    static constexpr int shift_of(int i) { return 8 * byte_of(i) + BITS * (IPB - 1 - k_of(i)); }
    static constexpr int local_code(int w, int i) { return w * CPW + byte_of(i) * IPB + k_of(i); }
    // grid copy used for the i-th code: its base is pre-shifted to the code's bit position
    // (one-code-per-byte widths use two copies, shifts 0 and 8, and merge halves with one shift)
    static constexpr int copy_of(int i) {
        return IPB == 1 ? (byte_of(i) & 1) : byte_of(i) * IPB + (IPB - 1 - k_of(i));
    }
    static constexpr uint32_t sign_mask() {
        uint32_t m = 0;
        for (int i = 0; i < CPW; ++i) m |= 1u << (shift_of(i) + FIELD - 1);
        return m;
    }
};

template <int BITS>
__device__ __forceinline__ uint32_t copy_shift_rt(uint32_t c) {
    constexpr int IPB = 8 / BITS;
    return IPB == 1 ? 8u * c : 8u * (c / IPB) + (uint32_t)BITS * (c % IPB);
}

// s_waitcnt vmcnt(N) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, expcnt 6:4 and lgkmcnt 11:8 left at their maxima)
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Norm of a vector from the fp32 sum of its squares.  Reciprocal square root plus one Newton step is correctly
// rounded except for a vanishing fraction of inputs.  Sums below 1e-35 (norm < 1e-17: it vanishes both in
// norm + 1e-8 and in fp16) count as zero; infinite and NaN sums pass through.
static __device__ __forceinline__ float tq_norm_from_sumsq(float ss) {
    const float r = __builtin_amdgcn_rsqf(ss);
    const float g = ss * r, h = 0.5f * r;
    float nrm = fmaf(fmaf(-g, g, ss), h, g);
    nrm = ss < 1e-35f ? 0.f : nrm;
    return ss < __builtin_inff() ? nrm : ss;
}

// Decode the eight codes of MFMA step s held by this lane (codes 64*hk + 8*s .. + 7 of its vector)
// into a packed fp16x8 operand, through the byte -> centroids table `lut` in LDS.
// raw[] holds the lane's 64/IPB packed bytes, little-endian dwords.
template <int IPB, int NW>
__device__ __forceinline__ tq_u4 decode_step(const uint32_t (&raw)[NW], int s, const uint8_t *lut) {
    tq_u4 out;
    if constexpr (IPB == 1) {  // 8 bytes, one code each -> 8 two-byte lookups
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t b0 = (raw[2 * s + (2 * d) / 4] >> (8 * ((2 * d) % 4))) & 0xffu;
            const uint32_t b1 = (raw[2 * s + (2 * d + 1) / 4] >> (8 * ((2 * d + 1) % 4))) & 0xffu;
            const uint32_t lo = *reinterpret_cast<const uint16_t *>(lut + b0 * 2u);
            const uint32_t hi = *reinterpret_cast<const uint16_t *>(lut + b1 * 2u);
            out[d] = lo | (hi << 16);
        }
    } else if constexpr (IPB == 2) {  // 4 bytes, two codes each -> 4 four-byte lookups
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t b = (raw[s] >> (8 * d)) & 0xffu;
            out[d] = *reinterpret_cast<const uint32_t *>(lut + b * 4u);
        }
    } else if constexpr (IPB == 4) {  // 2 bytes, four codes each -> 2 eight-byte lookups
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t b = (raw[s / 2] >> (16 * (s % 2) + 8 * q)) & 0xffu;
            const tq_u2 v = *reinterpret_cast<const tq_u2 *>(lut + b * 8u);
            out[2 * q] = v[0];
            out[2 * q + 1] = v[1];
        }
    } else {  // IPB == 8: 1 byte, eight codes -> 1 sixteen-byte lookup
        const uint32_t b = (raw[s / 4] >> (8 * (s % 4))) & 0xffu;
        out = *reinterpret_cast<const tq_u4 *>(lut + b * 16u);
    }
    return out;
}

// The byte -> centroids tables are read with data-dependent addresses by every lane.  With one copy, 64 random
// addresses over 32 banks serialise several times over (measured: the LDS pipe was busy 70 % of the kernel).  Here
// every table entry is spread over 128 bytes = one slot per bank group, and a lane always reads the slot of its own
// banks: entries of 2 or 4 bytes have 32 slots of 4 bytes (lane % 32), 8-byte entries 16 slots (lane % 16: a 64-bit
// read serves 16 lanes per clock), 16-byte entries 8 slots.  256 entries x 128 bytes = 32 KiB per table.
template <int IPB>
struct RepLut {
    static constexpr int ES = 2 * IPB;                    // bytes per entry
    static constexpr int SL = ES < 4 ? 4 : ES;            // slot size
    static constexpr int NC = 128 / SL;                   // copies
    static __device__ __forceinline__ uint32_t lane_offset(uint32_t lane) { return (lane & (NC - 1)) * SL; }
    static __device__ __forceinline__ void stage(uint8_t *lds, const uint8_t *src, uint32_t tid, uint32_t nthreads) {
        for (uint32_t i = tid; i < 256u * NC; i += nthreads) {
            const uint32_t e = i / NC, c = i % NC;
            uint8_t *dst = lds + e * 128u + c * SL;
            const TQ_GLOBAL uint8_t *g = (const TQ_GLOBAL uint8_t *)src + e * ES;
            if constexpr (ES == 2) *reinterpret_cast<uint16_t *>(dst) = *reinterpret_cast<const TQ_GLOBAL uint16_t *>(g);
            else if constexpr (ES == 4) *reinterpret_cast<uint32_t *>(dst) = *reinterpret_cast<const TQ_GLOBAL uint32_t *>(g);
            else if constexpr (ES == 8) *reinterpret_cast<tq_u2 *>(dst) = *reinterpret_cast<const TQ_GLOBAL tq_u2 *>(g);
            else *reinterpret_cast<tq_u4 *>(dst) = *reinterpret_cast<const TQ_GLOBAL tq_u4 *>(g);
        }
    }
};

// decode_step against a replicated table; `lut` already points at the lane's slot of entry 0
template <int IPB, int NW>
__device__ __forceinline__ tq_u4 decode_rep(const uint32_t (&raw)[NW], int s, const uint8_t *lut) {
    tq_u4 out;
    if constexpr (IPB == 1) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t b0 = (raw[2 * s + (2 * d) / 4] >> (8 * ((2 * d) % 4))) & 0xffu;
            const uint32_t b1 = (raw[2 * s + (2 * d + 1) / 4] >> (8 * ((2 * d + 1) % 4))) & 0xffu;
            const uint32_t lo = *reinterpret_cast<const uint16_t *>(lut + (b0 << 7));
            const uint32_t hi = *reinterpret_cast<const uint16_t *>(lut + (b1 << 7));
            out[d] = lo | (hi << 16);
        }
    } else if constexpr (IPB == 2) {
#pragma unroll
        for (int d = 0; d < 4; ++d) out[d] = *reinterpret_cast<const uint32_t *>(lut + (((raw[s] >> (8 * d)) & 0xffu) << 7));
    } else if constexpr (IPB == 4) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t b = (raw[s / 2] >> (16 * (s % 2) + 8 * q)) & 0xffu;
            const tq_u2 v = *reinterpret_cast<const tq_u2 *>(lut + (b << 7));
            out[2 * q] = v[0];
            out[2 * q + 1] = v[1];
        }
    } else {
        const uint32_t b = (raw[s / 4] >> (8 * (s % 4))) & 0xffu;
        out = *reinterpret_cast<const tq_u4 *>(lut + (b << 7));
    }
    return out;
}

// 64-wide vectors can go through the 128-wide kernels two at a time when the two vectors of every pair are neighbours in
// memory and in the packed store, and no pair straddles two rows: an even number of tokens per row, 64 elements apart,
// an even packed row stride.
static inline bool tq_pairable(long long rows, long long tokens, long long token_stride, long long packed_row_stride, int head_dim,
                               const void *idx_bytes) {
    (void)rows;
    return head_dim == TQ_HEAD_DIM / 2 && tokens > 0 && (tokens & 1) == 0 && token_stride == head_dim && (packed_row_stride & 1) == 0 &&
           ((uintptr_t)idx_bytes & 15u) == 0;      // (the 128-wide kernels move packed bytes 16 at a time)
}

// Alignment the packed codes need: 16 bytes for the 128-wide kernels; the kernels of the other head dimensions move them
// in pieces no larger than the largest power of two that divides a vector's packed bytes (a token slice of a store of
// 24-byte vectors starts on a multiple of 8).
static inline uintptr_t tq_packed_alignment(int head_dim, int bits) {
    if (head_dim == TQ_HEAD_DIM) return 16;
    if (head_dim % 32) return 1;        // moved byte by byte
    const uintptr_t g = (uintptr_t)((head_dim + (8 / bits) - 1) / (8 / bits));
    const uintptr_t low = g & (~g + 1);
    return low < 16 ? low : 16;
}

// Alignment of the vectors themselves (pointer and strides, in bytes): 16, except for head dimensions that are not a
// multiple of 32, whose vectors are moved element by element.
static inline uintptr_t tq_vector_alignment(int head_dim, int elem_bytes) {
    return head_dim % 32 ? (uintptr_t)elem_bytes : 16;
}

// Blocks per job for a (blocks_per_job x n_jobs) grid of equal-cost blocks on `cus` compute units
// that hold one block each.  Every block pays a set-up (rotation operands, tables), so the fewest
// device-wide rounds win as long as the last round is nearly full (at most 3 % of the slots idle);
// failing that, the round count with the fullest last round.
static inline uint32_t tq_blocks_per_job(uint32_t want, int cus, int n_jobs) {
    if (n_jobs <= 1) return want < (uint32_t)cus ? (want ? want : 1u) : (uint32_t)cus;
    uint32_t best = 1;
    double best_waste = 1e30;
    for (int rounds = 1; rounds <= 8; ++rounds) {
        uint32_t per_job = (uint32_t)((long long)cus * rounds / n_jobs);
        if (per_job == 0) continue;
        if (per_job > want) per_job = want ? want : 1u;
        const long long total = (long long)per_job * n_jobs;
        const long long padded = (total + cus - 1) / cus * cus;
        const double waste = (double)(padded - total) / (double)padded;
        if (waste < best_waste - 1e-9) { best_waste = waste; best = per_job; }
        if (waste <= 0.03 || per_job >= want) break;
    }
    return best;
}
