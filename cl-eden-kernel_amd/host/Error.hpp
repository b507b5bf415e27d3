// Status-returning checks in the style of the reference's
// src/userdriver/common/operator_interfaces/common/Error.hpp:20-27: log and return, no exceptions.
#pragma once

#include <cstdio>

#include "Common.hpp"

#define ERROR_PRINT(...)              \
    do {                              \
        std::fprintf(stderr, __VA_ARGS__); \
    } while (0)

#define CHECK_EXPR_RETURN_FAILURE(expr, ...) \
    do {                                     \
        if (!(expr)) {                       \
            ERROR_PRINT(__VA_ARGS__);        \
            ERROR_PRINT("\n");               \
            return Status::FAILURE;          \
        }                                    \
    } while (0)
