// libiris_hip: the MFMA kernel builds for fp8 inputs (all tile shapes and operand layouts).
#include "fused_kernel.h"

template int dispatch_mfma_in<IN_FP8>(FusedParams&, int, bool, int, int, hipStream_t);
