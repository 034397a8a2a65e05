// Error-checking macros with the reference's names (src/utils/macro.h): CHECK for runtime API calls
// (prints and exits, macro.h:10-25 there), LLM_CHECK / LLM_CHECK_WITH_INFO for argument checks
// (throw std::runtime_error with the "[oneLLM][ERROR] ... Assertion fail: file:line" text,
// macro.h:92-110 there).  The runtime underneath is HIP.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>

#define CHECK(call)                                                              \
    do {                                                                         \
        const hipError_t isp_check_status_ = (call);                             \
        if (isp_check_status_ != hipSuccess) {                                   \
            std::printf("HIP Error:\n    File:       %s\n    Line:       %d\n"   \
                        "    Error code: %d\n    Error text: %s\n",              \
                        __FILE__, __LINE__, (int)isp_check_status_,              \
                        hipGetErrorString(isp_check_status_));                   \
            std::exit(1);                                                        \
        }                                                                        \
    } while (0)

[[noreturn]] inline void throwRuntimeError(const char* const file, int const line,
                                           std::string const& info = "") {
    throw std::runtime_error(std::string("[oneLLM][ERROR] ") + info + " Assertion fail: " + file +
                             ":" + std::to_string(line) + " \n");
}

inline void llmAssert(bool result, const char* const file, int const line,
                      std::string const& info = "") {
    if (!result) throwRuntimeError(file, line, info);
}

inline void syncAndCheck(const char* const file, int const line) {
    (void)hipDeviceSynchronize();
    const hipError_t status = hipGetLastError();
    if (status != hipSuccess) {
        throw std::runtime_error(std::string("[oneLLM][ERROR] HIP runtime error: ") +
                                 hipGetErrorString(status) + " " + file + ":" +
                                 std::to_string(line) + " \n");
    }
}

#define DeviceSyncAndCheckCudaError() syncAndCheck(__FILE__, __LINE__)
#define LLM_CHECK(val) llmAssert((val), __FILE__, __LINE__)
#define LLM_CHECK_WITH_INFO(val, info)                                   \
    do {                                                                 \
        const bool isp_check_ok_ = (val);                                \
        if (!isp_check_ok_) llmAssert(false, __FILE__, __LINE__, (info)); \
    } while (0)
