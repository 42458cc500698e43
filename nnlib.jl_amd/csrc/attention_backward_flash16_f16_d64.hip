// Instantiation of the MFMA attention backward for f16, head dim 64.
#define BWD_T F16
#define BWD_D 64
#define BWD_ENTRY launch_bwd_flash16_f16_d64
#include "attention_backward_flash16.inc"
