// The bfloat16 instantiations of the any-shape attention (attention_generic_kernel.h), in a source
// file of their own so that they compile beside the float ones.
#include "attention_generic_kernel.h"

void tl_attention_generic_bf16(const AgLaunch& a) { ag_launch_all<bf16_t>(a); }
