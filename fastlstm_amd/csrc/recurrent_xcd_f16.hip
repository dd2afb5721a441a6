// XCD-local forward kernels, element type _Float16.
#define REC_T _Float16
#define REC_SUF f16
#include "recurrent_xcd_inst.inc"
