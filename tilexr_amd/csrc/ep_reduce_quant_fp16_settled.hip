// One compilation of ep_reduce_quant.hip.h: fp16 rows, tile readiness flags that were published before the launch began.
#define TILEXR_REDUCE_BF16 false
#define TILEXR_REDUCE_FLAGS 2
#define TILEXR_REDUCE_ENTRY LaunchReduceQuantFp16Settled
#include "ep_reduce_quant.hip.h"
