#define CK_INST_DT f16_tag
#define CK_INST_FN launch_gemm_fused_f16
#include "gemm_fused_inst.inc"
