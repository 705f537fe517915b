// One compilation of ep_reduce_quant.hip.h: bf16 rows, tile readiness flags that may still be pending.
#define TILEXR_REDUCE_BF16 true
#define TILEXR_REDUCE_FLAGS 1
#define TILEXR_REDUCE_ENTRY LaunchReduceQuantBf16Flags
#include "ep_reduce_quant.hip.h"
