// Maps C-ABI status codes to the error behaviour callers of the reference expect:
// argument problems throw std::invalid_argument / std::overflow_error before anything is
// launched; runtime failures print the message and end the process
// (reference: include/core/cuda_check.h:19-38; the operator tests assert the exception types).
#pragma once

#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>

#include "cgptx.h"

namespace cgptx_detail {

// A stream capture that would have needed new scratch memory is reported as std::runtime_error so
// that the caller can end the capture, run once eagerly and capture again.
inline void check(const int status) {
    if (status == CGPTX_OK) return;
    const std::string message = cgptx_last_error();
    if (status == CGPTX_INVALID_ARGUMENT) throw std::invalid_argument(message);
    if (status == CGPTX_OVERFLOW) throw std::overflow_error(message);
    if (status == CGPTX_CAPTURE_ALLOC) throw std::runtime_error(message);
    std::fprintf(stderr, "%s\n", message.c_str());
    std::exit(EXIT_FAILURE);
}

}  // namespace cgptx_detail
