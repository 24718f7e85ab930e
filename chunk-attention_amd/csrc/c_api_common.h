// What both halves of the C-ABI share: the calling thread's last error message and the
// translation of C++ exceptions into error codes at the boundary.  No HIP types here: the
// host-only half (c_api_host.cpp) compiles with a plain C++ compiler.
#pragma once

#include <exception>
#include <new>
#include <stdexcept>
#include <string>

#include "chunk_attn_hip.h"

namespace ca {
namespace abi {

// Sets the calling thread's message (what ca_last_error returns) and hands `code` back.
int fail(int code, const std::string& msg);
const char* last_error();

// Translates C++ exceptions of the manager into error codes at the ABI boundary.
template <typename F>
int guarded(F&& f) {
    try {
        return f();
    } catch (const std::bad_alloc&) {
        return fail(CA_ERR_RUNTIME, "out of host memory");
    } catch (const std::invalid_argument& e) {
        return fail(CA_ERR_INVALID, e.what());
    } catch (const std::out_of_range& e) {
        return fail(CA_ERR_INVALID, e.what());
    } catch (const std::exception& e) {
        const std::string msg = e.what();
        return fail(msg.find("capacity reached") != std::string::npos ? CA_ERR_CAPACITY
                                                                       : CA_ERR_RUNTIME,
                    msg);
    }
}

}  // namespace abi
}  // namespace ca
