#define CK_INST_DT bf16_tag
#define CK_INST_MODE 2
#define CK_INST_FN launch_gemm_pc_bf16_m2
#include "gemm_pc_inst.inc"
