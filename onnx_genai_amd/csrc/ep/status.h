// NxrtStatus / NxmemStatus construction helpers and the exception fence used at every extern "C" entry.
#pragma once

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <exception>
#include <string>

#include "../../../include/nxrt_ep_rocm.h"
#include "../hip_ffi.h"

namespace nxrt_rocm {

inline NxrtStatus make_status(uint32_t code, const std::string& message = std::string())
{
    NxrtStatus s;
    std::memset(&s, 0, sizeof(s));
    s.code = code;
    size_t len = message.size();
    const size_t nul = message.find('\0');
    if (nul != std::string::npos) len = nul;
    if (len > NXRT_STATUS_MESSAGE_MAX) len = NXRT_STATUS_MESSAGE_MAX;
    std::memcpy(s.message, message.data(), len);
    s.message_len = static_cast<uint32_t>(len);
    return s;
}

inline NxrtStatus ok() { return make_status(NXRT_OK); }

inline NxrtStatus hip_status(int err, const char* what)
{
    if (err == 0) return ok();
    if (err >= 10000) return make_status(NXRT_DEVICE_ERROR, std::string(what) + ": hipBLASLt status " + std::to_string(err - 10000));
    const uint32_t code = err == 2 /* hipErrorOutOfMemory */ ? NXRT_OUT_OF_MEMORY : NXRT_DEVICE_ERROR;
    return make_status(code, std::string(what) + ": " + rocm_ffi_error_string(err));
}

inline NxmemStatus make_mem_status(uint32_t code, const std::string& message = std::string())
{
    NxmemStatus s;
    std::memset(&s, 0, sizeof(s));
    s.code = code;
    size_t len = message.size();
    if (len > NXMEM_STATUS_MESSAGE_MAX) len = NXMEM_STATUS_MESSAGE_MAX;
    std::memcpy(s.message, message.data(), len);
    s.message_len = static_cast<uint32_t>(len);
    return s;
}

// Nothing may unwind across the C boundary (the reference catches panics at every entry:
// crates/onnx-runtime-ep-nxrt-abi/src/status.rs:198-).
template <typename F>
NxrtStatus fenced(F&& f) noexcept
{
    try {
        return f();
    } catch (const std::bad_alloc&) {
        return make_status(NXRT_OUT_OF_MEMORY, "host allocation failed");
    } catch (const std::exception& e) {
        return make_status(NXRT_INTERNAL_ERROR, e.what());
    } catch (...) {
        return make_status(NXRT_INTERNAL_ERROR, "unknown exception (fail-closed)");
    }
}

}  // namespace nxrt_rocm
