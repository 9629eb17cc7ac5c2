// Layout of the codec table blob shared by the host-side builder and the gfx950 kernels.
//
// One blob per compressor instance (rotation + codebook).  All section offsets are from the
// start of the blob and 256-byte aligned.
#pragma once
#include <stdint.h>

#define TQ_TABLE_MAGIC 0x54514d49u /* "TQMI" */
#define TQ_TABLE_VERSION 8u
#define TQ_HEAD_DIM 128

// --- MFMA operand tiling (v_mfma_f32_32x32x16_{f16,bf16}) --------------------------------
// A-operand tile (t, s): 64 lanes x 8 halves.  Lane l supplies row  m = l % 32  and the
// contraction slice  (hk = l / 32, i = 0..7).  The accumulator register r (0..15) of lane
// (n = l % 32, h = l / 32) holds row  m = 8*(r/4) + 4*h + (r%4)  of column n.
//
// Both kernels put the vectors on the MFMA columns (one vector per lane, two lanes per
// vector) and keep the rotation resident in registers as the A operand.
//
// compress: a tile of 32 vectors is shared by the four waves of a block; wave w owns MFMA tile w
// and the row order is chosen so that lane-half h of wave w ends up with 16 consecutive rotated
// coordinates:
//     output(tile = w, h, r) = 32*w + 16*h + r
//     input(s, hk, i)        = 16*s + 8*hk + i               (element of x)
// decompress: one wave owns all four MFMA tiles, lane-half h gets 64 consecutive elements:
//     output(tile t, h, r)        = 64*h + 16*t + r
//     input(s, hk, i)             = 64*hk + 8*s + i          (code index)
#define TQ_TILES 4  /* 128 outputs / 32 rows  */
#define TQ_STEPS 8  /* 128 inputs  / 16 deep  */
#define TQ_OPERAND_BYTES (TQ_TILES * TQ_STEPS * 64 * 16) /* one 128x128 16-bit operand set: 32 KiB */

// Other head dimensions (TQ_ANYDIM_MIN to TQ_ANYDIM_MAX) go through one pair of kernels that takes the dimension at run
// time.  Their tables hold d/32 row tiles x d/16 steps per operand set, compress AND decompress operands in the compress
// tiling above (out = 32t + 16h + r, in = 16s + 8hk + i), and a quantiser grid of up to TQ_GRID_LDS_BYTES / 8 cells
// whatever the width (those kernels keep a single, unshifted copy).
// A head dimension that is not a multiple of 32 is worked on as the next multiple: the operand sets are those of the
// rotation extended by zero rows and columns, the kernels read the missing input elements as zeros, give the missing
// coordinates the code 0 (upstream turboquant/compressors_v3.py:64-68 pads the codes of a vector with zeros up to a
// whole byte) and neither decode nor store them on the way back.
#define TQ_ANYDIM_MIN 8
#define TQ_ANYDIM_MAX 256
#define TQ_PADDED_DIM(d) ((((d) + 31) / 32) * 32)
#define TQ_OPERAND_BYTES_FOR(d) ((TQ_PADDED_DIM(d) / 32) * (TQ_PADDED_DIM(d) / 16) * 64 * 16)

// The fp16 split of Pi is stored multiplied by 2^TQ_F16_PI_SHIFT so that the low term stays
// in the fp16 normal range; the kernels fold 2^-shift into the per-vector scale.
#define TQ_F16_PI_SHIFT 10

// Quantiser grid.  With rho = acc * inv (the exact real product; acc = raw rotated coordinate,
// inv = 1 / (norm + 1e-8)) the kernels compute
//     cell(rho) = (bits(fma(acc, inv * grid_scale, grid_bias)) & TQ_GRID_ADDR_MASK) / 8
//     code      = base[cell] + (fma(acc, inv, -threshold[cell]) >= 0)
// Both fused multiply-adds see the same exact product, so cell edges are the exact reals
// (k - cells/2 - 1/16) / grid_scale (grid_bias carries 1.5 * 2^20, one ulp = 1/8) and the
// comparison is exact.  entry = { float threshold; uint32 base }, at most one threshold per cell.
//
// In LDS the kernels keep one copy of the grid per position of a code inside a 32-bit word,
// with `base` pre-shifted to that position, at a fixed stride so that the copy is selected by
// the immediate offset of the LDS read.
#define TQ_GRID_ADDR_MASK 0x7ff8u
#define TQ_GRID_LDS_BYTES 18432
#define TQ_GRID_MAGIC 1572864.0f /* 1.5 * 2^20: one ulp = 1/8 */
// copies: one per code position in a dword (32 / bits), two for the one-code-per-byte widths
#define TQ_GRID_COPIES(bits) ((bits) >= 5 ? 2 : (bits) == 3 ? 8 : 32 / (bits))
#define TQ_GRID_COPY_STRIDE(bits) (TQ_GRID_LDS_BYTES / TQ_GRID_COPIES(bits))
#define TQ_GRID_MAX_CELLS(bits) (TQ_GRID_COPY_STRIDE(bits) / 8)

struct TqGridCell {
    float threshold;
    uint32_t base;
};

struct TqTableHeader {
    uint32_t magic;
    uint32_t version;
    uint32_t head_dim;
    uint32_t bits;
    uint32_t levels;
    uint32_t ipb;            // indices per byte = 8 / bits
    uint32_t bytes_per_vec;  // ceil(head_dim / ipb)
    uint32_t grid_cells;
    float grid_scale;        // cells per unit of r (power of two)
    float grid_bias;         // grid_cells/2 + TQ_GRID_MAGIC
    uint32_t total_bytes;
    uint32_t off_a_f16;      // compress operand, Pi * 2^shift as fp16 hi, lo     (2 x 32 KiB)
    uint32_t off_a_bf16;     // compress operand, Pi as bf16 hi, mid, lo          (3 x 32 KiB)
    uint32_t off_grid;       // TqGridCell[grid_cells]
    uint32_t off_at_f16;     // decompress operand, Pi^T as fp16 hi, lo           (2 x 32 KiB)
    uint32_t off_lut;        // decode table: 256 entries of ipb fp16 centroids (byte -> values)
    uint32_t off_centroids;  // float[levels]
    uint32_t off_thresholds; // float[levels - 1]
    uint32_t lut_entry_bytes; // 2 * ipb
    // head_dim 64 only, and only when the quantiser grid fits the shifted copies of the 128-wide kernels (0 otherwise):
    // operand sets of the 128 x 128 block-diagonal matrix diag(Pi, Pi) in the tilings of those kernels.  Two consecutive
    // 64-wide vectors that lie next to each other in memory are one 128-wide row to them; rotated by diag(Pi, Pi), searched
    // and packed per coordinate, they come out as the two vectors' codes one after the other, which is the packed layout
    // of two 64-wide vectors.  Only the norm is per half.
    uint32_t off_pair_a_f16;  // compress operand of diag(Pi, Pi) * 2^shift as fp16 hi, lo     (2 x 32 KiB)
    uint32_t off_pair_a_bf16; // compress operand of diag(Pi, Pi) as bf16 hi, mid, lo          (3 x 32 KiB)
    uint32_t off_pair_at_f16; // decompress operand of diag(Pi, Pi)^T as fp16 hi, lo           (2 x 32 KiB)
    uint32_t padded_dim;      // TQ_PADDED_DIM(head_dim): the dimension of the operand sets
    uint32_t reserved[41];
};
static_assert(sizeof(TqTableHeader) == 256, "header is one 256-byte block");

// --- table of the V2 key path (MSE codes + 1-bit QJL signs of the residual) ---------------------------------------
// Operand tiles in the compress tiling above (tile = wave, out = 32w + 16h + r, input = 16s + 8hk + i), as fp16 terms
// (hi, lo: 22 bits, 2^-22 of the largest entry) of the matrices times a power of two that puts their largest entry
// into [2^13, 2^14), so that the low terms stay in the fp16 normal range:
//   Pi^T : k_unit[out] = sum_j centroid(code_j) * Pi[j][out]
//   S    : projected[out] = sum_k residual[k] * S[out][k]      (only its sign is used: any positive scale does)
// The centroids come as pairs of fp16 terms of centroid * 2^cent_shift, one 32-bit word per code (hi | lo << 16);
// k_scale = 2^-(pit_shift + cent_shift) takes the product back.
// For the one-pass kernel (codes, norms, signs and residual norms from a single read of the input) the table also holds
//   M = S Pi^T : projected[out] = sum_k (Pi residual)[k] * M[out][k]
// in the same tiling and term format: with the rotated input y = Pi x that the code search works on anyway, the residual
// in rotated coordinates is y - norm * centroid(code), coordinate by coordinate (Pi (centroids @ Pi) = centroids up to the
// rotation's departure from orthogonality, 1e-6 of the residual's own projection), so the inverse rotation never
// has to be formed.  M is computed in double precision from Pi and S.  The centroids are there as plain floats as well.
#define TQ_QJL_MAGIC 0x54514a4cu /* "TQJL" */
#define TQ_QJL_VERSION 3u
struct TqQjlHeader {
    uint32_t magic;
    uint32_t version;
    uint32_t head_dim;
    uint32_t mse_bits;
    uint32_t levels;
    uint32_t off_pit;        // 2 x TQ_OPERAND_BYTES
    uint32_t off_s;          // 2 x TQ_OPERAND_BYTES
    uint32_t off_centroids;  // uint32[256], the first `levels` used
    uint32_t total_bytes;
    float k_scale;
    uint32_t off_m;          // 2 x TQ_OPERAND_BYTES
    uint32_t off_cent_f32;   // float[256], the first `levels` used
    uint32_t reserved[52];
};
static_assert(sizeof(TqQjlHeader) == 256, "header is one 256-byte block");
