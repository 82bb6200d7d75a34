// elementwise_row_any.hip — the row machine's kernels with the general step: any operand and result type.
#include "ew_row_machine.hpp"

namespace kapy {
int launch_row_any(const StackProgram &P, int ns, hipStream_t s) { return launch_row_kernel<kModeAny>(P, ns, s); }
}  // namespace kapy
