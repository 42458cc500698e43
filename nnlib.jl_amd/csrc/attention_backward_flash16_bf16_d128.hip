// Instantiation of the MFMA attention backward for bf16, head dim 128.
#define BWD_T BF16
#define BWD_D 128
#define BWD_ENTRY launch_bwd_flash16_bf16_d128
#include "attention_backward_flash16.inc"
