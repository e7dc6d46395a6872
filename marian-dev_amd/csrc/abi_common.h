// Shared by the translation units of the library: the per-thread HIP error behind
// marian_hip_last_hip_error().
#pragma once

namespace marian_hip {

// Remembers hipError_t `e` for the calling thread and returns MARIAN_HIP_ERR_HIP.
int record_hip_error(int e);

// Launches the abs-max pass over n floats (n % 4 == 0) on `stream`: partials (at least 4 KB of
// workspace) receives *n_partials values whose maximum is max|A|.  Returns a status code.
int launch_absmax_partials(const float* A, unsigned long n, float* partials, int* n_partials, void* stream);

}  // namespace marian_hip
