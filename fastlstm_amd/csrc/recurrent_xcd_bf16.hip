// XCD-local forward kernels, element type __bf16.
#define REC_T __bf16
#define REC_SUF bf16
#include "recurrent_xcd_inst.inc"
