// One compilation of ep_reduce_quant.hip.h: fp16 rows, tile readiness flags that may still be pending.
#define TILEXR_REDUCE_BF16 false
#define TILEXR_REDUCE_FLAGS 1
#define TILEXR_REDUCE_ENTRY LaunchReduceQuantFp16Flags
#include "ep_reduce_quant.hip.h"
