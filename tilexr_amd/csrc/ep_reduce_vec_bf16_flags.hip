// One compilation of ep_reduce_vec.hip.h: bf16 rows, with tile readiness flags.
#define TILEXR_REDUCE_BF16 true
#define TILEXR_REDUCE_FLAGS true
#define TILEXR_REDUCE_ENTRY LaunchReduceVecBf16Flags
#include "ep_reduce_vec.hip.h"
