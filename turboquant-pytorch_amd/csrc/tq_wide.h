// Entry points of the codec kernels for the head dimensions 96, 160, 192 and 224 with 16-bit elements
// (tq_wide.hip), called by the dispatchers of tq_anydim.hip.  Arguments as there: `single` describes the one job of a
// plain call (jobs_dev NULL), `jobs_dev` the device copy of a batch.
#pragma once
#include "tq_device.h"

bool tq_wide_supported(int head_dim, int dtype);
int tq_wide_compress(int dtype, int bits, int head_dim, const TqDevJob &single, const tq_job *jobs_dev, int n_jobs,
                     uint32_t max_vec, hipStream_t stream);
int tq_wide_decompress(int dtype, int bits, int head_dim, const TqDevJob &single, const tq_job *jobs_dev, int n_jobs,
                       uint32_t max_vec, hipStream_t stream);
