// XCD-local forward kernels, element type float.
#define REC_T float
#define REC_SUF f32
#include "recurrent_xcd_inst.inc"
