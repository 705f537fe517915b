// One compilation of ep_reduce_vec.hip.h: fp16 rows, with tile readiness flags.
#define TILEXR_REDUCE_BF16 false
#define TILEXR_REDUCE_FLAGS true
#define TILEXR_REDUCE_ENTRY LaunchReduceVecFp16Flags
#include "ep_reduce_vec.hip.h"
