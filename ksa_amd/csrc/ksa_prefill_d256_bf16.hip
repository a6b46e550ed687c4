// Translation unit of ksa_prefill.hip that holds the bf16 kernels of head_dim 256 (compiled next to
// the main unit instead of inside it: these instantiations take minutes to compile).
#define KSA_PREFILL_UNIT 1
#include "ksa_prefill.hip"
