// Instantiations of the matrix-memory recurrence kernel: mlstm.
#include "matrix_memory_kernel.h"

namespace mm {
void launch_mlstm(const ScanArgs& a, int B, int lanes, bool bf16,
                hipStream_t stream) {
  if (bf16) launch_scan<KIND_MLSTM, short>(a, B, lanes, stream);
  else launch_scan<KIND_MLSTM, float>(a, B, lanes, stream);
}
}  // namespace mm
