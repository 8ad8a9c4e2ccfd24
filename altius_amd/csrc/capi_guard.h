// What an exception becomes at the C boundary.  Nothing may unwind through an extern "C" function: the frames above it
// belong to a caller that is not C++ (Rust, Python's ctypes), and an exception that escapes ends the process.  Every
// entry point that can allocate is a function-try-block whose handler returns caught_at_boundary(its name):
// std::bad_alloc and std::length_error (a container asked to grow past what exists) read AHIP_ERR_OOM, anything else
// AHIP_ERR_UNSUPPORTED, with the exception's text as the error message.
#pragma once

#include <exception>
#include <new>
#include <stdexcept>
#include <string>

#include "../../include/altius_hip.h"
#include "device/ctx.h"

namespace altius {

inline int caught_at_boundary(const char *where) noexcept {
    int code = AHIP_ERR_UNSUPPORTED;
    try {
        try {
            throw;
        } catch (const std::bad_alloc &) {
            code = AHIP_ERR_OOM;
            set_global_error(std::string(where) + ": out of host memory");
        } catch (const std::length_error &e) {
            code = AHIP_ERR_OOM;
            set_global_error(std::string(where) + ": " + e.what());
        } catch (const std::exception &e) {
            set_global_error(std::string(where) + ": " + e.what());
        } catch (...) {
            set_global_error(std::string(where) + ": unknown failure");
        }
    } catch (...) {
        // not even the message could be stored: the code alone goes back
    }
    return code;
}

}  // namespace altius
