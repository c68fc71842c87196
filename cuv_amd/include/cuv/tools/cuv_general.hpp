// Error conventions of the DIA path, re-expressed for HIP.
//
// Mirrors src/cuv/tools/cuv_general.hpp:19-56 and cuv_general.cu:45-80 of the
// reference: a violated precondition throws std::runtime_error carrying the
// stringified condition, a failed runtime call throws with the call text and
// the runtime's error string.  The function names (initCUDA, exitCUDA,
// safeThreadSync) are kept so that code written against CUV still compiles.
#ifndef __CUV_GENERAL_HPP__
#define __CUV_GENERAL_HPP__

#include <hip/hip_runtime_api.h>

#include <stdexcept>
#include <string>

#include "cuvdia.h"

#ifndef CUDA_TEST_DEVICE
#  define CUDA_TEST_DEVICE 0
#endif

namespace cuv {

inline void cuvAssertFailed(const char *msg) { throw std::runtime_error(std::string(msg)); }

#define cuvAssert(X) \
    if (__builtin_expect(!(X), 0)) { cuv::cuvAssertFailed(#X); }

inline void checkHipError(hipError_t err, const char *msg)
{
    if (err != hipSuccess) {
        (void)hipGetLastError();
        throw std::runtime_error(std::string(msg) + ": " + hipGetErrorString(err));
    }
}

#define cuvSafeCall(X) cuv::checkHipError((X), #X)

// A negative code from the C ABI becomes the same kind of exception.
inline void checkDiaCall(int code, const char *what)
{
    if (code < 0) {
        std::string m = std::string(what) + ": " + cuvdia_strerror(code);
        if (code == CUVDIA_EHIP) m += std::string(" (") + cuvdia_last_hip_error() + ")";
        throw std::runtime_error(m);
    }
}

inline void initCUDA(int dev = 0)
{
    if (dev < 0) return;
    cuvSafeCall(hipSetDevice(dev));
}
inline void exitCUDA() { (void)hipDeviceSynchronize(); }
inline void safeThreadSync() { cuvSafeCall(hipDeviceSynchronize()); }

}  // namespace cuv
#endif
