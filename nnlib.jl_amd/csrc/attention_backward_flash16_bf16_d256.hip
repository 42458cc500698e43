// Instantiation of the MFMA attention backward for bf16, head dims above 128 up to 256.
#define BWD_T BF16
#define BWD_D 256
#define BWD_ENTRY launch_bwd_flash16_bf16_d256
#include "attention_backward_flash16.inc"
