#define CK_INST_DT f16_tag
#define CK_INST_MODE 1
#define CK_INST_FN launch_gemm_pc_f16_m1
#include "gemm_pc_inst.inc"
