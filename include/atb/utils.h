// atb::Utils - tensor size helpers and log-level control
// (reference include/atb/utils.h:37-98, src/atb/utils/utils.cpp:28-150).
#ifndef ATB_UTILS_H
#define ATB_UTILS_H
#include <cstdint>
#include <string>
#include "atb/types.h"

namespace atb {
class Utils {
public:
    static std::string GetAtbVersion();

    // Bytes = numel * element size; 0 for an empty shape, a non-positive
    // extent, an unknown dtype or an overflow.
    static uint64_t GetTensorSize(const Tensor &tensor);
    static uint64_t GetTensorSize(const TensorDesc &tensorDesc);

    static uint64_t GetTensorNumel(const Tensor &tensor);
    static uint64_t GetTensorNumel(const TensorDesc &tensorDesc);

    // Packs each float's bit pattern into the low 32 bits of a uint64.
    static void QuantParamConvert(const float *src, uint64_t *dest, uint64_t itemCount);

    static Status SetLogLevel(const atb::LogLevel atbLogLevel);
    static Status ResetLogLevel();
};
} // namespace atb
#endif
