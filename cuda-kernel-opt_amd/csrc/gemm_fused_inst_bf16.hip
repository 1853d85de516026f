#define CK_INST_DT bf16_tag
#define CK_INST_FN launch_gemm_fused_bf16
#include "gemm_fused_inst.inc"
