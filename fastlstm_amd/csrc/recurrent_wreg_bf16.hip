// Forward kernels with register-resident W_h, element type __bf16.
#define REC_T __bf16
#define REC_SUF bf16
#include "recurrent_wreg_inst.inc"
