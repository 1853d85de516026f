#define CK_INST_DT bf16_tag
#define CK_INST_MODE 1
#define CK_INST_FN launch_gemm_pc_bf16_m1
#include "gemm_pc_inst.inc"
