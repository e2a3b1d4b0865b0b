// API version this header library stands in for: the reference configures the same three macros and
// rocwmma_get_version() from its build (library/include/rocwmma/internal/rocwmma-version.hpp.in,
// CMakeLists.txt:80-85 there, version 1.6.0); its test logger prints them (test/rocwmma_logging.hpp:81).
#ifndef ROCWMMA_API_VERSION_HPP
#define ROCWMMA_API_VERSION_HPP

#include <string>

#define ROCWMMA_VERSION_MAJOR 1
#define ROCWMMA_VERSION_MINOR 6
#define ROCWMMA_VERSION_PATCH 0

inline std::string rocwmma_get_version()
{
    return std::to_string(ROCWMMA_VERSION_MAJOR) + "." + std::to_string(ROCWMMA_VERSION_MINOR) + "."
           + std::to_string(ROCWMMA_VERSION_PATCH);
}

#endif // ROCWMMA_API_VERSION_HPP
