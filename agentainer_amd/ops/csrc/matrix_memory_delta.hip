// Instantiations of the matrix-memory recurrence kernel: delta.
#include "matrix_memory_kernel.h"

namespace mm {
void launch_delta(const ScanArgs& a, int B, int lanes, bool bf16,
                hipStream_t stream) {
  if (bf16) launch_scan<KIND_DELTA, short>(a, B, lanes, stream);
  else launch_scan<KIND_DELTA, float>(a, B, lanes, stream);
}
}  // namespace mm
