// Persistent forward / reverse kernels, element type __bf16.
#define REC_T __bf16
#define REC_SUF bf16
#include "recurrent_inst.inc"
