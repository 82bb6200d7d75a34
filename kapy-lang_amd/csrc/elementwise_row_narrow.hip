// elementwise_row_narrow.hip — the row machine's kernels with the general step: 16-bit operands and results, any op.
#include "ew_row_machine.hpp"

namespace kapy {
int launch_row_narrow(const StackProgram &P, int ns, hipStream_t s) { return launch_row_kernel<kModeNarrow>(P, ns, s); }
}  // namespace kapy
