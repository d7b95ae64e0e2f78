// libiris_hip: the MFMA kernel builds for bf16 inputs (all tile shapes and operand layouts).
#include "fused_kernel.h"

template int dispatch_mfma_in<IN_BF16>(FusedParams&, int, bool, int, int, hipStream_t);
