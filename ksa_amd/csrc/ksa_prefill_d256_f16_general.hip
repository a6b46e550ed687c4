// Translation unit of ksa_prefill.hip that holds the fp16 kernel of head_dim 256 with general tile addressing
// (compiled next to the main unit instead of inside it: each of these instantiations takes over a minute).
#define KSA_PREFILL_UNIT 4
#include "ksa_prefill.hip"
