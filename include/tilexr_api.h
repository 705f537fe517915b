// Communicator calls libtilexr-ep needs from the communication runtime, for ranks that share one MI355X.
//
// The reference's EP library sits on libtile-comm (src/include/tilexr_api.h:44-48, 86): the caller obtains a
// communicator with TileXRCommInitRankLocal, the EP host code fetches CommArgs from it and draws one "magic"
// (epoch) per launch.  This header declares the five calls the EP path uses, with the reference's names and
// signatures, implemented here for logical ranks that all live on the current HIP device of one process:
//
//   * Communicators created with the same rankSize join one "world" until every rank of it exists; a further
//     call with that rankSize starts the next world.  All ranks of a world must be created on the same device.
//   * A world owns a small per-rank flag area in HBM (CommArgs::peerMems[r]) and the staging buffers that
//     multi-rank dispatch / combine exchange rows through; they are released when its last communicator is
//     destroyed.
//   * The magic counter starts at 1 and is advanced atomically (reference: src/comm/tilexr_comm.h:101,
//     src/comm/tilexr_comm.cpp:1235-1238).
//   * Without a usable HIP device the communicator is still created, with null peerMems; EP entry points then
//     return TILEXR_ERROR_NOT_INITIALIZED after argument validation.
#ifndef TILEXR_API_H
#define TILEXR_API_H

#include <cstddef>
#include <cstdint>

#include "comm_args.h"

extern "C" {
#pragma GCC visibility push(default)   // the entry points below are what the shared library exports

typedef void *TileXRCommPtr;

// reference: src/include/tilexr_api.h:29
int TileXRCommInitRankLocal(int rankSize, int rank, TileXRCommPtr *comm);

// reference: src/include/tilexr_api.h:86
int TileXRCommDestroy(TileXRCommPtr comm);

// reference: src/include/tilexr_api.h:44 -- device-resident copy of CommArgs
int TileXRGetCommArgsDev(TileXRCommPtr comm, GM_ADDR &commArgsPtr);

// reference: src/include/tilexr_api.h:46 -- host copy, owned by the communicator
int TileXRGetCommArgsHost(TileXRCommPtr comm, TileXR::CommArgs *&commArgsPtr);

// reference: src/include/tilexr_api.h:48
int TileXRCommNextMagic(TileXRCommPtr comm, int64_t *magic);

#pragma GCC visibility pop
}

#endif // TILEXR_API_H
