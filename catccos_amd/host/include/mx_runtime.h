// Device-runtime glue of the host plugin layer: everything the operators need from the GPU runtime
// goes through the C ABI of libcatccos_mx (cmx_rt_*), so this layer has no HIP types of its own.
#pragma once

#include <cstddef>
#include <cstdint>
#include <iostream>
#include <stdexcept>
#include <string>

#include "catccos_mx.h"

// Logs a failed runtime call and carries on, which is what the operators' callers expect of
// allocation and copy helpers (mains that must stop on the first failure use MxCheckOrThrow).
#define MX_CHECK(call)                                                                                   \
    do {                                                                                                 \
        int mx_status_ = (call);                                                                         \
        if (mx_status_ != CMX_OK) {                                                                      \
            std::cerr << __FILE__ << ":" << __LINE__ << " mxError:" << mx_status_ << " " << cmx_last_error() \
                      << std::endl;                                                                      \
        }                                                                                                \
    } while (0)

inline void MxCheckOrThrow(int status, const char* what)
{
    if (status != CMX_OK) {
        throw std::runtime_error(std::string(what) + " failed: " + cmx_last_error());
    }
}

namespace mxrt {

inline uint8_t* DeviceAlloc(size_t bytes)
{
    void* p = nullptr;
    MX_CHECK(cmx_rt_malloc(&p, bytes));
    return static_cast<uint8_t*>(p);
}

inline uint8_t* HostAlloc(size_t bytes)
{
    void* p = nullptr;
    MX_CHECK(cmx_rt_malloc_host(&p, bytes));
    return static_cast<uint8_t*>(p);
}

}  // namespace mxrt
