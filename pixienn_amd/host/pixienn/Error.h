// Host-side error type of the MI355X layer kernels: every C-ABI status other than PXH_OK and
// every failed HIP runtime call becomes a px::Error, the exception the engine's layers throw
// (reference: include/Error.h:27-65, include/CudaError.h:27-47).
#pragma once

#include <hip/hip_runtime_api.h>

#include <sstream>
#include <stdexcept>
#include <string>

#include "pixienn_hip.h"

namespace px {

class Error : public std::runtime_error
{
public:
    Error(const char* file, unsigned line, const char* function, const std::string& message)
            : std::runtime_error(compose(file, line, function, message)), file_(file), line_(line),
              function_(function), message_(message) {}

    const std::string& file() const noexcept { return file_; }
    unsigned line() const noexcept { return line_; }
    const std::string& function() const noexcept { return function_; }
    const std::string& message() const noexcept { return message_; }

private:
    static std::string compose(const char* file, unsigned line, const char* function, const std::string& message)
    {
        std::ostringstream ss;
        ss << file << ":" << line << " (" << function << "): " << message;
        return ss.str();
    }

    std::string file_;
    unsigned line_;
    std::string function_;
    std::string message_;
};

namespace hip {

// Status of a pxh_* call -> exception.  Negative: the call was rejected before any launch;
// positive: the hipError_t of a failed launch.
inline void checkStatus(int status, const char* file, unsigned line, const char* function)
{
    if (status == PXH_OK) return;
    std::string message = pxh_last_error();
    if (status > 0) {
        message += " [";
        message += hipGetErrorName(static_cast<hipError_t>(status));
        message += "]";
    }
    throw Error(file, line, function, message);
}

inline void checkHip(hipError_t status, const char* file, unsigned line, const char* function)
{
    if (status == hipSuccess) return;
    throw Error(file, line, function, std::string(hipGetErrorName(status)) + ": " + hipGetErrorString(status));
}

}   // hip
}   // px

#define PX_HIP_CHECK(call) ::px::hip::checkStatus((call), __FILE__, __LINE__, __func__)
#define PX_HIP_RUNTIME_CHECK(call) ::px::hip::checkHip((call), __FILE__, __LINE__, __func__)
#define PX_CHECK(cond, msg) \
    do { if (!(cond)) throw ::px::Error(__FILE__, __LINE__, __func__, (msg)); } while (0)
