// One compilation of ep_reduce_quant.hip.h: bf16 rows, without tile readiness flags.
#define TILEXR_REDUCE_BF16 true
#define TILEXR_REDUCE_FLAGS false
#define TILEXR_REDUCE_ENTRY LaunchReduceQuantBf16
#include "ep_reduce_quant.hip.h"
