// bf16 instances of the block-sparse prefill kernel.
#define BR_LAUNCH_PREFILL br_launch_prefill_bf16
#include "br_prefill_mfma_launch.h"
