// dlprim type vocabulary for the HIP-backed convolution path.
//
// Same names and meanings as dlprimitives' include/dlprim/definitions.hpp for the
// items this path uses (DataType :78-94, exceptions :38-75, StandardActivations
// :278-284, Convolution2DConfigBase :313-321), so code written against
// dlprim::core::Conv2DForward / IPForward compiles unchanged.
#pragma once
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

#include "../dlprim_hip.h"

namespace dlprim {

class Error : public std::runtime_error {
public:
    explicit Error(std::string const &v) : std::runtime_error(v) {}
};
class NotImplementedError : public Error {
public:
    explicit NotImplementedError(std::string const &v) : Error(v) {}
};
class ValidationError : public Error {
public:
    explicit ValidationError(std::string const &v) : Error(v) {}
};

#define DLPRIM_CHECK(x)                                                                                            \
    do {                                                                                                           \
        if (!(x))                                                                                                  \
            throw ::dlprim::ValidationError(std::string("Failed " #x " at " __FILE__ ":") + std::to_string(__LINE__)); \
    } while (0)

// numeric values are part of the ABI (they are passed through dlprim_hip.h as ints)
enum DataType {
    double_data = 4 + (0 << 3),
    int64_data = 4 + (2 << 3),
    uint64_data = 4 + (3 << 3),
    float_data = 3 + (0 << 3),
    int32_data = 3 + (2 << 3),
    uint32_data = 3 + (3 << 3),
    half_data = 2 + (0 << 3),
    bfloat16_data = 2 + (1 << 3),
    int16_data = 2 + (2 << 3),
    uint16_data = 2 + (3 << 3),
    int8_data = 1 + (2 << 3),
    uint8_data = 1 + (3 << 3),
};

inline int size_of_data_type(DataType d) { return 1 << ((d & 7) - 1); }

enum class StandardActivations : int {
    identity = 0,
    relu = 1,
    tanh = 2,
    sigmoid = 3,
    relu6 = 4,
};

inline StandardActivations activation_from_name(std::string const &name)
{
    if (name == "identity")
        return StandardActivations::identity;
    if (name == "relu")
        return StandardActivations::relu;
    if (name == "tanh")
        return StandardActivations::tanh;
    if (name == "sigmoid")
        return StandardActivations::sigmoid;
    if (name == "relu6")
        return StandardActivations::relu6;
    throw ValidationError("unknown activation \"" + name + "\" (identity, relu, tanh, sigmoid, relu6)");
}

struct Convolution2DConfigBase {
    int channels_in = -1;
    int channels_out = -1;
    int kernel[2] = {1, 1};
    int stride[2] = {1, 1};
    int dilate[2] = {1, 1};
    int pad[2] = {0, 0};
    int groups = 1;
};

namespace details {
// turn a dlprim_hip.h status into the exception the reference would have thrown
inline void check_status(int rc)
{
    if (rc == DLP_OK)
        return;
    std::string msg = dlp_last_error();
    if (rc == DLP_ERR_VALIDATION)
        throw ValidationError(msg);
    if (rc == DLP_ERR_NOT_IMPLEMENTED)
        throw NotImplementedError(msg);
    throw Error(msg);
}
} // namespace details

} // namespace dlprim
