// Forward kernels with register-resident W_h, element type float.
#define REC_T float
#define REC_SUF f32
#include "recurrent_wreg_inst.inc"
