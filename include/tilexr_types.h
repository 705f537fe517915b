// Status codes and element-type codes shared by the tilexr-ep C ABI.
//
// Values are the ones the reference publishes in src/include/tilexr_types.h:17-25 (status) and :60-79
// (TileXRDataType); only the members the EP dispatch / combine path can see are listed.
#ifndef TILEXR_TYPES_H
#define TILEXR_TYPES_H

#include <cstdint>

namespace TileXR {

constexpr int TILEXR_SUCCESS = 0;
constexpr int TILEXR_ERROR_NOT_INITIALIZED = -1;   // communicator has no peer memory / unknown communicator
constexpr int TILEXR_ERROR_MKIRT = -2;             // a kernel launch was refused by the runtime
constexpr int TILEXR_ERROR_PARA_CHECK_FAIL = -3;   // argument or shape rejected
constexpr int TILEXR_ERROR_INTERNAL = -4;
constexpr int TILEXR_ERROR_TIMEOUT = -5;           // a bounded device-side wait expired
constexpr int TILEXR_ERROR_NOT_SUPPORT = -6;       // legal request outside the implemented feature set
constexpr int TILEXR_ERROR_NOT_FOUND = -7;
constexpr int64_t TILEXR_INVALID_VALUE = -1;

enum TileXRDataType {
    TILEXR_DATA_TYPE_INT8 = 0,
    TILEXR_DATA_TYPE_INT16 = 1,
    TILEXR_DATA_TYPE_INT32 = 2,
    TILEXR_DATA_TYPE_FP16 = 3,
    TILEXR_DATA_TYPE_FP32 = 4,
    TILEXR_DATA_TYPE_INT64 = 5,
    TILEXR_DATA_TYPE_UINT64 = 6,
    TILEXR_DATA_TYPE_UINT8 = 7,
    TILEXR_DATA_TYPE_UINT16 = 8,
    TILEXR_DATA_TYPE_UINT32 = 9,
    TILEXR_DATA_TYPE_FP64 = 10,
    TILEXR_DATA_TYPE_BFP16 = 11,
    TILEXR_DATA_TYPE_INT128 = 12,
    TILEXR_DATA_TYPE_HIF8 = 14,
    TILEXR_DATA_TYPE_FP8E4M3 = 15,
    TILEXR_DATA_TYPE_FP8E5M2 = 16,
    TILEXR_DATA_TYPE_FP8E8M0 = 17,
    TILEXR_DATA_TYPE_RESERVED = 255
};

} // namespace TileXR

#endif // TILEXR_TYPES_H
