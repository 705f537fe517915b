// One compilation of ep_reduce_quant.hip.h: fp16 rows, no tile readiness flags.
#define TILEXR_REDUCE_BF16 false
#define TILEXR_REDUCE_FLAGS 0
#define TILEXR_REDUCE_ENTRY LaunchReduceQuantFp16
#include "ep_reduce_quant.hip.h"
