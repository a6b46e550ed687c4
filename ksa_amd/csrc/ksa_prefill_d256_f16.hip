// Translation unit of ksa_prefill.hip that holds the fp16 kernels of head_dim 256.
#define KSA_PREFILL_UNIT 2
#include "ksa_prefill.hip"
