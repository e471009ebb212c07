// Shared between the two halves of the C ABI implementation.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "antfly_hip_qmatmul.h"

namespace afhip {

struct LaunchCounters {
    uint64_t mmv = 0, small_batch = 0, mm = 0, f32_route = 0, activation_quant = 0, prepare = 0;
    // Opt-in phase timing (the engine's QuantExecutionTimingStats, ops/ops.zig:649-713): when
    // `phase_events` is set, the op records phase_events[0] before its first kernel, [1] behind the
    // stand-alone activation quantizer (or at once, when the kernel quantizes in its own prologue)
    // and [2] behind its last kernel, all on the op's stream.  They are hipEvent_t.
    void** phase_events = nullptr;
};

bool checked_mul(size_t a, size_t b, size_t* out);
size_t block_bytes(int tensor_type);

// The op behind every linear launcher.  dots.ptr != 0 switches to "write the
// int32 block dots instead of Y".
// weight_b.ptr != 0 adds a second matrix of the same shape and layout that shares the
// input (result in dst_b; not together with dots).
// extras: what the kernel that writes Y adds to the plain product (not together with dots).
struct LinearExtras {
    afhip_buffer bias{0, 0};      // f32 [out_dim], added to every row of dst
    afhip_buffer bias_b{0, 0};    // the same for dst_b
    afhip_buffer residual{0, 0};  // f32 [rows][out_dim], added last (one matrix only)
    int activation = AFHIP_ACTIVATION_NONE;  // applied after the bias (one matrix only)
};
afhip_status linear_impl(void* stream, int tensor_type, int layout, afhip_buffer dst, afhip_buffer input,
                         afhip_buffer weight, size_t rows, size_t in_dim, size_t out_dim, afhip_buffer workspace,
                         int dispatch, afhip_buffer dots, LaunchCounters* counters,
                         afhip_buffer dst_b = afhip_buffer{0, 0}, afhip_buffer weight_b = afhip_buffer{0, 0},
                         const LinearExtras& extras = LinearExtras{});

// argmax over the last row of f32 [rows, dim]; `workspace` (optional) lets several workgroups scan a long row.
afhip_status argmax_last_row_impl(void* stream, afhip_buffer token_u32, afhip_buffer token_f32, afhip_buffer input,
                                  size_t rows, size_t dim, afhip_buffer workspace);

// argmax(X[rows-1] * W^T): one GEMV over the last row whose workgroups keep the best of their
// columns (repacked weights), or logits into `workspace` and the argmax kernels.
afhip_status linear_argmax_impl(void* stream, int tensor_type, int layout, afhip_buffer token_u32,
                                afhip_buffer token_f32, afhip_buffer input, afhip_buffer weight, size_t rows,
                                size_t in_dim, size_t out_dim, afhip_buffer workspace, LaunchCounters* counters);

}  // namespace afhip
