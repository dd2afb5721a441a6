// Reverse kernel of H = 1280 ... 2048 with the product split over K among team members, element type _Float16.
#define REC_T _Float16
#define REC_SUF f16
#include "recurrent_wsplit_inst.inc"
