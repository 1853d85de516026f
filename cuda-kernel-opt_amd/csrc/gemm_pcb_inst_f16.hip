#define CK_INST_DT f16_tag
#define CK_INST_FN launch_gemm_pcb_f16
#include "gemm_pcb_inst.inc"
