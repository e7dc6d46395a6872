// How marian_hip_nbest_beams splits the row of a batch entry over workgroups (host code, no HIP).
#pragma once

#include <stdint.h>

namespace marian_hip {

// The row of a batch entry is the beam's `beam` segments of `vocab` scores.  Each segment is cut
// into perSeg slices of sliceLen scores (the last one may be shorter, never empty); one workgroup
// per slice leaves its N best, and the N best of the beam * perSeg * N candidates are the result.
struct NbestPlan {
  int perSeg;
  long long sliceLen;
  int parts;   // beam * perSeg workgroups per batch entry
};

// Enough workgroups for every CU (256 and up) as long as a slice keeps 4096 scores; at most 1024
// candidates per entry (what the merge draws from); sliceLen a multiple of four so that slices
// start 16-byte aligned when the rows do.
inline NbestPlan nbest_plan(int64_t beam, int64_t dimBatch, int64_t vocab, int64_t N) {
  long long perSeg = (256 + beam * dimBatch - 1) / (beam * dimBatch);
  const long long most = vocab / 4096 > 0 ? vocab / 4096 : 1;
  if(perSeg > most) perSeg = most;
  while(perSeg > 1 && beam * perSeg * N > 1024) --perSeg;
  long long sliceLen = ((vocab + perSeg - 1) / perSeg + 3) / 4 * 4;
  perSeg = (vocab + sliceLen - 1) / sliceLen;
  return NbestPlan{(int)perSeg, sliceLen, (int)(beam * perSeg)};
}

}  // namespace marian_hip
