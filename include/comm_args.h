// Communicator description handed to EP kernels and returned by TileXRGetCommArgsHost / TileXRGetCommArgsDev.
//
// Field order, types and array extents follow the reference's struct (src/include/comm_args.h:122-147) so that a
// caller compiled against the reference header reads the same offsets.  On one MI355X every logical rank lives on
// the same device: peerMems[r] points into one HBM allocation owned by the communicator's world, localRankSize ==
// rankSize, and the transport-specific members (credit memory, UDMA / SDMA pointers, dump address) stay null.
#ifndef TILEXR_COMM_ARGS_H
#define TILEXR_COMM_ARGS_H

#include <cstdint>

#ifndef GM_ADDR
using GM_ADDR = uint8_t *;
#endif

namespace TileXR {

constexpr int TILEXR_MAX_RANK_SIZE = 128;                       // src/include/comm_args.h:38
constexpr int64_t IPC_BUFF_MAX_SIZE = 512LL * 1024 * 1024;      // :40  capacity the reference's window checks use
constexpr int64_t IPC_DATA_OFFSET = 2 * 1024 * 1024;            // :58  flag area in front of each peer window
constexpr int DFX_COUNT = 50;                                   // :85

struct ExtraFlag {                                              // :104-120 (bits the EP host logic tests)
    static constexpr uint32_t UDMA = 1u << 10;
    static constexpr uint32_t SDMA = 1u << 11;
    static constexpr uint32_t MEMORY_ONLY = 1u << 18;
};

struct CommArgs {
    int rank = 0;
    int localRank = -1;
    int rankSize = 0;
    int localRankSize = -1;
    uint32_t extraFlag = 0;
    GM_ADDR peerMems[TILEXR_MAX_RANK_SIZE] = {};
    GM_ADDR creditMems[TILEXR_MAX_RANK_SIZE] = {};
    int64_t sendCountMatrix[TILEXR_MAX_RANK_SIZE * TILEXR_MAX_RANK_SIZE] = {};
    int64_t dfx[DFX_COUNT] = {};
    GM_ADDR dumpAddr = nullptr;
    int32_t magics[TILEXR_MAX_RANK_SIZE] = {0};
    uint64_t fftsVal = 0;
    GM_ADDR udmaInfoPtr = nullptr;
    GM_ADDR udmaRegistryPtr = nullptr;
    GM_ADDR sdmaWorkspacePtr = nullptr;
    GM_ADDR udmaFullmeshPtr = nullptr;
    uint64_t udmaRegistrationGeneration = 0U;
    uint64_t peerMemBytes = 0U;
    int32_t commDomain = 0;
    uint32_t reserved0 = 0U;
};

} // namespace TileXR

#endif // TILEXR_COMM_ARGS_H
