// One flavour of the interpreter kernel: compute type, log domain and feature mode come from the command line
// (-DSPN_INST_REAL=float -DSPN_INST_LOG2=true -DSPN_INST_FEAT=1 -DSPN_INST_NAME=interpKernel_f32_log2_staged).
#include "interp_kernel_impl.h"

namespace spnc_hip {
const void* SPN_INST_NAME(int mode) { return kernelPtr<SPN_INST_REAL, SPN_INST_LOG2, SPN_INST_FEAT>(mode); }
}  // namespace spnc_hip
