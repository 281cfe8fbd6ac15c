// The staged form of the column-splitting skinny kernel for bf16 activations (gemv_cs_staged.h).
#include "gemv_cs_staged.h"

hipError_t turq_launch_gemv_cs_staged_bf16(TURQ_STAGED_LAUNCH_ARGS) { return staged_launch<TURQ_ACT_BF16>(TURQ_STAGED_LAUNCH_PASS); }
hipError_t turq_launch_gemv_cs_staged_gateup_bf16(TURQ_STAGED_GATEUP_ARGS) { return staged_gateup_launch<TURQ_ACT_BF16>(TURQ_STAGED_GATEUP_PASS); }

TURQ_NONFINITE_READER(turq_nonfinite_gemv_cs_staged_bf16)
