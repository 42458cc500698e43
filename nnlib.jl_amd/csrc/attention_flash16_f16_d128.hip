// Instantiation of the 16-bit MFMA flash forward kernel: f16, head dim 128.
#define FLASH_T F16
#define FLASH_D 128
#define FLASH_QB 1
#define FLASH_ENTRY launch_flash16_f16_d128
#include "attention_flash16.inc"
