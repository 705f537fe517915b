// Destination row of one route, shared by the stand-alone place kernel and the scatter kernels (which resolve the
// rows of their own token when no separate place launch is needed).
//   row   = keyOffset[key] + (rank of the route within its key), routes at or beyond `capacity` get none
//   tuple = {srcRank, token, k, expert id} (reference: src/ep/common/ep_window.h:47-52,
//           src/ep/kernels/tilexr_ep_dispatch_memory_kernel.h:1240-1258)
#ifndef TILEXR_AMD_EP_PLACE_HIP_H
#define TILEXR_AMD_EP_PLACE_HIP_H

#include <cstdint>

#include <hip/hip_runtime.h>

#include "ep_launch.h"

namespace TileXREp {

struct PlaceArgs {
    const int32_t *ids;          // nullptr: rows are read from rowOf instead of being resolved
    const int32_t *localRank;    // [n] rank within (chunk, key), -1 = not live
    const int32_t *chunkBase;    // [chunks, numKeys] routes of the key in earlier chunks
    const int32_t *keyOffset;    // [numKeys + 1]
    int chunkShift;
    int n;
    int topK;
    int keyDiv;
    int numKeys;
    int capacity;
    int32_t srcRank;
    int32_t expertIdBias;
    int32_t sharedNum;           // leading shared routes per token (see RoutePlaceLaunch)
    const int32_t *tupleExperts; // optional [n]: expert id reported by the tuple
    int32_t *rowOf;              // optional out [n]
    int32_t *assist;             // out [rows, 4]
};

inline PlaceArgs MakePlaceArgs(const RoutePlaceLaunch &l)
{
    PlaceArgs a {};
    a.ids = l.ids;
    a.localRank = l.scratch.localRank;
    a.chunkBase = l.scratch.chunkHist;
    a.keyOffset = l.scratch.keyOffset;
    a.chunkShift = l.scratch.chunkShift;
    a.n = static_cast<int>(l.bs * l.topK);
    a.topK = static_cast<int>(l.topK);
    a.keyDiv = static_cast<int>(l.keyDiv);
    a.numKeys = static_cast<int>(l.numKeys);
    a.capacity = static_cast<int>(l.capacity);
    a.srcRank = l.srcRank;
    a.expertIdBias = l.expertIdBias;
    a.sharedNum = l.sharedNum;
    a.tupleExperts = l.tupleExperts;
    a.rowOf = l.rowOf;
    a.assist = l.assist;
    return a;
}

// Resolves route i (< a.n), writes its assist tuple and rowOf entry, returns the row or -1.
__device__ __forceinline__ int PlaceRoute(const PlaceArgs &a, int i)
{
    // both loads at once: the id is there for every route, whether it is live or not
    const int lr = a.localRank[i];
    const int e = a.ids[i];
    int row = -1;
    if (lr >= 0) {
        const int key = a.keyDiv == 1 ? e : e / a.keyDiv;
        const int within = a.chunkBase[static_cast<int64_t>(i >> a.chunkShift) * a.numKeys + key] + lr;
        if (a.capacity <= 0 || within < a.capacity) {
            row = a.keyOffset[key] + within;
            int32_t *tuple = a.assist + static_cast<int64_t>(row) * 4;
            const int pos = i % a.topK;
            tuple[0] = a.srcRank;
            tuple[1] = i / a.topK;
            // shared routes come first in a token's row and report the slots after the routed ones
            // (reference: src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:536-568)
            tuple[2] = pos < a.sharedNum ? a.topK - a.sharedNum + pos : pos - a.sharedNum;
            tuple[3] = a.tupleExperts != nullptr ? a.tupleExperts[i] : e + a.expertIdBias;
        }
    }
    if (a.rowOf != nullptr) {
        a.rowOf[i] = row;
    }
    return row;
}

} // namespace TileXREp

#endif // TILEXR_AMD_EP_PLACE_HIP_H
