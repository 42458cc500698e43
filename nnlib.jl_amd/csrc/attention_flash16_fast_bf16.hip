// Instantiation of the software-pipelined flash forward kernel (head dim 128) for bf16.
#define FAST_T BF16
#define FAST_ENTRY launch_flash16_fast_bf16
#define FAST_SUPPORTS flash16_fast_supports_bf16
#include "attention_flash16_fast.inc"
