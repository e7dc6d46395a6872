// Shared by the translation units of the library: the per-thread HIP error behind
// marian_hip_last_hip_error().
#pragma once

namespace marian_hip {

// Remembers hipError_t `e` for the calling thread and returns MARIAN_HIP_ERR_HIP.
int record_hip_error(int e);

}  // namespace marian_hip
