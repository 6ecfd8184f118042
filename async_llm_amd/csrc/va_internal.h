// Declarations shared by the translation units of libviewattn.so.
#pragma once
#include <stdint.h>

#include "../../include/viewattn.h"

// Record a formatted message for va_last_error() and return `code`.
int va_fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Matrix-core path eligibility and tile limits (defined next to the kernels).
bool va_mfma_supported(int dtype, int head_dim, int gqa);
int va_mfma_max_q_tile(int gqa);
int va_mfma_default_q_tile(int gqa, bool has_chain);
int va_mfma_wide_q_tile(int gqa, int head_dim);  // query rows of a wide tile

// Scratch for `n_partials` partial softmax states: fp32 accumulator rows plus
// (max, sum) pairs, per q head.
int64_t va_workspace_bytes_for(int64_t n_partials, int num_q_heads, int head_dim);
