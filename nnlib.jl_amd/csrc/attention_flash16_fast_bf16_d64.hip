// Instantiation of the software-pipelined flash forward kernel for bf16, head dim 64.
#define FAST_T BF16
#define FAST_D 64
#define FAST_ENTRY launch_flash16_fast_bf16_d64
#define FAST_SUPPORTS flash16_fast_supports_bf16_d64
#include "attention_flash16_fast.inc"
