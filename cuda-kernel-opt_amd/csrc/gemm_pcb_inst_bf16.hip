#define CK_INST_DT bf16_tag
#define CK_INST_FN launch_gemm_pcb_bf16
#include "gemm_pcb_inst.inc"
