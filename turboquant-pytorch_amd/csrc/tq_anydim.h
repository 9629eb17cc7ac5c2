// Entry points of the run-time-dimension codec kernels (tq_anydim.hip), called by the C ABI functions of
// tq_compress.hip / tq_decompress.hip for head dimensions other than 128.  Arguments as in their own dispatchers:
// `single` describes the one job of a plain call (jobs_dev NULL), `jobs_dev` the device copy of a batch.
#pragma once
#include "tq_device.h"

bool tq_anydim_supported(int head_dim);
int tq_anydim_compress(int dtype, int bits, int head_dim, const TqDevJob &single, const tq_job *jobs_dev, int n_jobs,
                       uint32_t max_vec, hipStream_t stream);
int tq_anydim_decompress(int dtype, int bits, int head_dim, const TqDevJob &single, const tq_job *jobs_dev, int n_jobs,
                         uint32_t max_vec, hipStream_t stream);
