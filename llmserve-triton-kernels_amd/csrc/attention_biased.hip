// The prompt attention of attention_mfma.hip with a learned bias per head and distance on the scaled scores and a sigmoid
// gate on the result, as a library of its own (the plain attention's library holds none of these variants): the same
// kernel, built with BIAS, for heads of 32, 64, 96 and 128 numbers.  Entry point: llms_attention_prompt_biased.
#define LLMS_ATTENTION_BIASED 1
#include "attention_mfma.hip"
