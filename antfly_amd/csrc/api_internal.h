// Shared between the two halves of the C ABI implementation.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "antfly_hip_qmatmul.h"

namespace afhip {

struct LaunchCounters {
    uint64_t mmv = 0, small_batch = 0, mm = 0, f32_route = 0, activation_quant = 0, prepare = 0;
};

bool checked_mul(size_t a, size_t b, size_t* out);
size_t block_bytes(int tensor_type);

// The op behind every linear launcher.  dots.ptr != 0 switches to "write the
// int32 block dots instead of Y".
// weight_b.ptr != 0 adds a second matrix of the same shape and layout that shares the
// input (result in dst_b; not together with dots).
afhip_status linear_impl(void* stream, int tensor_type, int layout, afhip_buffer dst, afhip_buffer input,
                         afhip_buffer weight, size_t rows, size_t in_dim, size_t out_dim, afhip_buffer workspace,
                         int dispatch, afhip_buffer dots, LaunchCounters* counters,
                         afhip_buffer dst_b = afhip_buffer{0, 0}, afhip_buffer weight_b = afhip_buffer{0, 0});

}  // namespace afhip
