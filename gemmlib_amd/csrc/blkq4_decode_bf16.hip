// The decode kernel for bf16 activations, scales and outputs: the same source as for fp16, with the element type
// switched (conversion of the weights, MFMA instruction, rounding of the outputs, bias).
#define BLKQ4_DECODE_BF16 1
#include "blkq4_decode.hip"
