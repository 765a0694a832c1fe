// include/motifcl/core/error.hpp:13-29 of MotifCL (the OpenCL helpers are dropped).
#pragma once

#include <stdexcept>
#include <string>

namespace motifcl {

class Error : public std::runtime_error {
public:
    explicit Error(const std::string& message) : std::runtime_error(message) {}
};

}  // namespace motifcl

#define MCL_CHECK(cond, msg)                                                                  \
    do {                                                                                      \
        if (!(cond)) {                                                                        \
            throw ::motifcl::Error(std::string("MotifCL check failed: ") + (msg) + " at " +   \
                                   __FILE__ + ":" + std::to_string(__LINE__));                \
        }                                                                                     \
    } while (0)
