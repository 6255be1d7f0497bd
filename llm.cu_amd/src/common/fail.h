// Error convention of the host layer: print a message and exit(1), as the
// reference does everywhere (src/safetensor/safetensor.cu:20-23,125-128,
// src/llama3/llama3.cu:12-15, src/inference/inference.cu:13-21,267-270).
// A test can install a handler that throws instead (llama3_set_error_handler).
#pragma once
#include <cstdarg>

[[noreturn]] void llama3_fail(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

// Checks a status returned by the HIP C-ABI layer.
void llama3_check(int status, const char *what);
