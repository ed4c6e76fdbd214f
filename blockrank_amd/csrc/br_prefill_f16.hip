// fp16 instances of the block-sparse prefill kernel: the same templates with _Float16 elements, v_mfma_f32_32x32x16_f16
// and v_dot2_f32_f16 (fp32 softmax and accumulation as for bf16; the probabilities stay below 2^8, well inside fp16).
#define BR_E16 _Float16
#define BR_E16_IS_F16 1
#define BR_LAUNCH_PREFILL br_launch_prefill_f16
#include "br_prefill_mfma_launch.h"
