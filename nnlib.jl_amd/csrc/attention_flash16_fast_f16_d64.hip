// Instantiation of the software-pipelined flash forward kernel for f16, head dim 64.
#define FAST_T F16
#define FAST_D 64
#define FAST_ENTRY launch_flash16_fast_f16_d64
#define FAST_SUPPORTS flash16_fast_supports_f16_d64
#include "attention_flash16_fast.inc"
