// Instantiation of the MFMA attention backward for bf16, head dim 64.
#define BWD_T BF16
#define BWD_D 64
#define BWD_ENTRY launch_bwd_flash16_bf16_d64
#include "attention_backward_flash16.inc"
