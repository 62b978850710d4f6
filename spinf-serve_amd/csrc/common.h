// Shared helpers of the library's translation units (error reporting; HIP call checking in the .hip files).
#pragma once
#include <cstdarg>
#include <cstdio>

int spinf_fail(int code, const char* fmt, ...);   // records a thread-local message, returns code
