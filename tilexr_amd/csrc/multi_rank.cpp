// Dispatch / combine across several logical ranks that share the device (rankSize > 1).
#include "ep_context.h"
#include "ep_host.h"
#include "ep_launch.h"

namespace TileXREp {

int RunDispatchMulti(EpComm *, const EpDispatchParams &, bool, int64_t)
{
    return TileXR::TILEXR_ERROR_NOT_SUPPORT;
}

int RunCombineMulti(EpComm *, const EpCombineParams &, bool, int64_t)
{
    return TileXR::TILEXR_ERROR_NOT_SUPPORT;
}

} // namespace TileXREp
