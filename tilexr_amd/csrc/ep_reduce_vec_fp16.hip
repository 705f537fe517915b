// One compilation of ep_reduce_vec.hip.h: fp16 rows, without tile readiness flags.
#define TILEXR_REDUCE_BF16 false
#define TILEXR_REDUCE_FLAGS false
#define TILEXR_REDUCE_ENTRY LaunchReduceVecFp16
#include "ep_reduce_vec.hip.h"
