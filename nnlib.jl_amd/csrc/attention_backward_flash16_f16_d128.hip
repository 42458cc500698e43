// Instantiation of the MFMA attention backward for f16, head dim 128.
#define BWD_T F16
#define BWD_D 128
#define BWD_ENTRY launch_bwd_flash16_f16_d128
#include "attention_backward_flash16.inc"
