// Reverse kernel of H = 1280 ... 2048 with the product split over K among team members, element type __bf16.
#define REC_T __bf16
#define REC_SUF bf16
#include "recurrent_wsplit_inst.inc"
