// One compilation of ep_reduce_quant.hip.h: bf16 rows, no tile readiness flags.
#define TILEXR_REDUCE_BF16 true
#define TILEXR_REDUCE_FLAGS 0
#define TILEXR_REDUCE_ENTRY LaunchReduceQuantBf16
#include "ep_reduce_quant.hip.h"
