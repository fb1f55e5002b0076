// atb::Utils (reference src/atb/utils/utils.cpp:20-175).
#include "atb/utils.h"
#include <complex>
#include <cstring>
#include <limits>
#include "log.h"

namespace atb {
namespace {
// Bytes per element; 0 = dtype this library cannot size.
uint64_t ElementSize(aclDataType dtype)
{
    switch (dtype) {
        case ACL_DT_UNDEFINED:
        case ACL_BOOL:
        case ACL_INT8:
        case ACL_UINT8:
            return 1;
        case ACL_FLOAT16:
        case ACL_BF16:
        case ACL_INT16:
        case ACL_UINT16:
            return 2;
        case ACL_FLOAT:
        case ACL_INT32:
        case ACL_UINT32:
            return 4;
        case ACL_INT64:
        case ACL_UINT64:
        case ACL_DOUBLE:
        case ACL_COMPLEX64:
            return 8;
        case ACL_COMPLEX128:
            return 16;
        case ACL_STRING:
            return sizeof(std::string);
        default:
            return 0;
    }
}
} // namespace

std::string Utils::GetAtbVersion()
{
    return "8.5.0-mi355x";
}

uint64_t Utils::GetTensorNumel(const Tensor &tensor)
{
    return GetTensorNumel(tensor.desc);
}

uint64_t Utils::GetTensorNumel(const TensorDesc &desc)
{
    if (desc.shape.dimNum == 0 || desc.shape.dimNum > MAX_DIM) {
        return 0;
    }
    uint64_t n = 1;
    for (uint64_t i = 0; i < desc.shape.dimNum; ++i) {
        const int64_t d = desc.shape.dims[i];
        if (d <= 0) {
            ATB_LOG(ERROR) << "dims[" << i << "] is <= 0";
            return 0;
        }
        if (std::numeric_limits<uint64_t>::max() / static_cast<uint64_t>(d) < n) {
            ATB_LOG(ERROR) << "GetTensorNumel overflow";
            return 0;
        }
        n *= static_cast<uint64_t>(d);
    }
    return n;
}

uint64_t Utils::GetTensorSize(const Tensor &tensor)
{
    return GetTensorSize(tensor.desc);
}

uint64_t Utils::GetTensorSize(const TensorDesc &desc)
{
    if (desc.shape.dimNum == 0) {
        return 0;
    }
    const uint64_t item = ElementSize(desc.dtype);
    if (item == 0) {
        ATB_LOG(ERROR) << "GetTensorSize: unsupported dtype " << static_cast<int>(desc.dtype);
        return 0;
    }
    const uint64_t n = GetTensorNumel(desc);
    if (n == 0 || std::numeric_limits<uint64_t>::max() / n < item) {
        return 0;
    }
    return n * item;
}

void Utils::QuantParamConvert(const float *src, uint64_t *dest, uint64_t itemCount)
{
    if (!src || !dest) {
        return;
    }
    for (uint64_t i = 0; i < itemCount; ++i) {
        uint32_t bits = 0;
        memcpy(&bits, &src[i], sizeof(bits));
        dest[i] = bits;
    }
}

Status Utils::SetLogLevel(const atb::LogLevel atbLogLevel)
{
    if (atbLogLevel < LogLevel::DEBUG || atbLogLevel > LogLevel::NONE) {
        return ERROR_INVALID_PARAM;
    }
    logging::SetLevel(atbLogLevel);
    return NO_ERROR;
}

Status Utils::ResetLogLevel()
{
    logging::ResetLevel();
    return NO_ERROR;
}
} // namespace atb
