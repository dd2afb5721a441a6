// Forward kernels with register-resident W_h, element type _Float16.
#define REC_T _Float16
#define REC_SUF f16
#include "recurrent_wreg_inst.inc"
