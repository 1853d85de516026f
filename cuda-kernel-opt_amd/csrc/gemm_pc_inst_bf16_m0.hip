#define CK_INST_DT bf16_tag
#define CK_INST_MODE 0
#define CK_INST_FN launch_gemm_pc_bf16_m0
#include "gemm_pc_inst.inc"
