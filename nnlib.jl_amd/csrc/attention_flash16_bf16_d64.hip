// Instantiation of the 16-bit MFMA flash forward kernel: bf16, head dim 64.
#define FLASH_T BF16
#define FLASH_D 64
#define FLASH_QB 1
#define FLASH_ENTRY launch_flash16_bf16_d64
#include "attention_flash16.inc"
