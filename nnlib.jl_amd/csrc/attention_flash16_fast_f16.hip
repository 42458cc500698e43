// Instantiation of the software-pipelined flash forward kernel (head dim 128) for f16.
#define FAST_T F16
#define FAST_ENTRY launch_flash16_fast_f16
#define FAST_SUPPORTS flash16_fast_supports_f16
#include "attention_flash16_fast.inc"
