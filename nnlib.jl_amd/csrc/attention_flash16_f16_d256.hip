// Instantiation of the 16-bit MFMA flash forward kernel: f16, head dims above 128 up to 256.
#define FLASH_T F16
#define FLASH_D 256
#define FLASH_QB 1
#define FLASH_ENTRY launch_flash16_f16_d256
#include "attention_flash16.inc"
