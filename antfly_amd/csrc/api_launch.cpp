// C ABI, part 1: dispatch vocabulary (graph/quant_matmul.zig) and the
// stream-ordered launchers (ops/cuda/kernels.zig:1221-1289).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <limits>

#include "antfly_hip_qmatmul.h"
#include "api_internal.h"
#include "qmatmul_launch.h"

// Scratch of afhip_launch_linear_f32_static: one copy per GPU, at its own address on each.
// In host code the name below is only a handle for hipGetSymbolAddress; kernels and copies
// get the address that call returned.
static __device__ __align__(256) unsigned char scratch[AFHIP_STATIC_SCRATCH_BYTES];

namespace afhip {

namespace {
constexpr int kMaxDevices = 64;
std::atomic<unsigned char*> g_static_scratch[kMaxDevices];

// The array's address on the current device, resolved once per device.
afhip_status static_scratch_address(unsigned char** out) {
    int dev = -1;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return static_cast<afhip_status>(e);
    if (dev < 0 || dev >= kMaxDevices) return AFHIP_ERR_INVALID_STATE;
    unsigned char* p = g_static_scratch[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        void* addr = nullptr;
        if (hipError_t e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)); e != hipSuccess) return static_cast<afhip_status>(e);
        if (addr == nullptr) return AFHIP_ERR_INVALID_STATE;
        p = static_cast<unsigned char*>(addr);
        g_static_scratch[dev].store(p, std::memory_order_release);  // (two threads may both resolve it: same value)
    }
    *out = p;
    return AFHIP_OK;
}
}  // namespace

bool checked_mul(size_t a, size_t b, size_t* out) { return !__builtin_mul_overflow(a, b, out); }

// Records phase event `i` of an op that is being timed (see LaunchCounters).
static void mark_phase(LaunchCounters* counters, int i, hipStream_t stream) {
    if (counters && counters->phase_events) (void)hipEventRecord(static_cast<hipEvent_t>(counters->phase_events[i]), stream);
}

size_t block_bytes(int tensor_type) {
    if (tensor_type == AFHIP_TYPE_Q4_0) return 18;
    if (tensor_type == AFHIP_TYPE_Q8_0) return 34;
    return 0;
}

static bool fits_u32(size_t v) { return v <= std::numeric_limits<uint32_t>::max(); }  // toU32, kernels.zig:2558-2563

// Scratch layout: [qx int8 rows*in_dim | pad to 256][sx f32 rows*kb][sums i32 rows*kb]
struct WorkspaceView {
    int8_t* qx;
    float* sx;
    int* sums;
    size_t bytes;
};
static WorkspaceView workspace_view(uint64_t base, size_t rows, size_t in_dim) {
    const size_t kb = in_dim / 32;
    const size_t q_bytes = (rows * in_dim + 255) / 256 * 256;
    WorkspaceView v;
    v.qx = reinterpret_cast<int8_t*>(base);
    v.sx = reinterpret_cast<float*>(base + q_bytes);
    v.sums = reinterpret_cast<int*>(base + q_bytes + rows * kb * 4);
    v.bytes = q_bytes + rows * kb * 8;
    return v;
}

// The GEMV quantizes X in its own prologue (every workgroup repeats that work) for one or
// two rows of any length, and for three or four rows of Q4_0 up to this many 32-value
// blocks of X; beyond, a separate kernel quantizes X once.
constexpr size_t kGemvFusedQuantBlocks = 512;
// fewest rows served by the single-shot MFMA kernel (batch_mfma_kernels.hip)
constexpr size_t kBatchMfmaMinRows = 5;

// LDS the GEMV may use per workgroup; gfx950 has 160 KiB per CU.  The larger figure is
// for up to eight rows of a long K (8 x 14336): one workgroup per CU then, but the
// weights are read once instead of once per slice of rows.
constexpr size_t kGemvLdsBudget = 96 * 1024;
constexpr size_t kGemvLdsBudgetFewRows = 152 * 1024;

// Rows one GEMV launch takes: as many as fit the LDS budget.
constexpr int kGemvMaxRowsPerLaunch = 16;
static int gemv_row_chunk(size_t rows, size_t in_dim) {
    if (rows <= 8 && gemv_fused_lds_bytes(static_cast<int>(rows), static_cast<int>(in_dim)) <= kGemvLdsBudgetFewRows)
        return static_cast<int>(rows);
    int chunk = rows < kGemvMaxRowsPerLaunch ? static_cast<int>(rows) : kGemvMaxRowsPerLaunch;
    while (chunk > 0 && gemv_fused_lds_bytes(chunk, static_cast<int>(in_dim)) > kGemvLdsBudget) --chunk;
    return chunk;
}

// Launch geometry of the fused GEMV.  AFHIP_GEMV_THREADS overrides it for tuning runs (the CPU engine exposes TERMITE_QUANT_* knobs the
// same way, ops/native_compute.zig:2902-2945).
static int env_int(const char* name) {
    const char* v = std::getenv(name);
    return v && *v ? std::atoi(v) : 0;
}

// Whether the single-shot MFMA kernel serves this shape (measured against the kernels it replaces;
// AFHIP_BATCH_MFMA_MIN_ROWS overrides the lower row bound for tuning runs, 0 switches the kernel off):
// from five rows on (six on a K longer than 4096, where the split-K GEMV still wins at five) up to 64
// (128 on wide Q4_0 matrices), and for Q8_0, whose K shares are half as long, only while all workgroups
// of the launch are resident at once.  Five to eight rows (Q8_0: sixteen) on a K of whole 256-value runs always:
// the eight-row kernel requests weights as it goes and needs neither condition.  Two to four rows where measured
// faster than the decode kernels (the rules below).
static bool batch_mfma_preferred(int tensor_type, size_t rows, size_t in_dim, size_t out_dim, bool pair) {
    static const char* v = std::getenv("AFHIP_BATCH_MFMA_MIN_ROWS");
    static const long forced = v && *v ? std::atol(v) : -1;
    // up to 64 rows everywhere; up to 128 on a Q4_0 matrix wide enough to give every compute unit a
    // column tile (there the tiled GEMM, whose 64 x 128 workgroup tiles re-read X per tile, is slower)
    // ... and where the tiled GEMM's grid of 32 x 64 tiles would not fit the compute units in one round while its
    // 64 x 128 tiles leave most of them idle (65 .. 128 rows on 4608 .. 8160 columns: 128 rows x 4608 columns 31.5 -> 24.1 us,
    // 65 rows x 6144 columns 31.0 -> 19.9, 100 rows of K = 8192 x 6144 columns 56.6 -> 43.8; one round of the GEMM stays
    // faster: 128 rows x 4096 columns 17.8 against 21.2, 96 rows x 5120 columns 17.7 against 20.1)
    const size_t units = static_cast<size_t>(gemv_compute_units());
    const bool wide = (out_dim + 31) / 32 >= units || (rows + 31) / 32 * ((out_dim + 63) / 64) > units;
    const size_t max_rows = tensor_type == AFHIP_TYPE_Q4_0 && wide ? 128 : 64;
    if (forced == 0 || rows > max_rows || !batch_mfma_supports(tensor_type, rows, in_dim, out_dim)) return false;
    if (forced > 0) return rows >= static_cast<size_t>(forced);
    if (rows >= kBatchMfmaMinRows && batch_mfma_eight_rows(tensor_type, rows, in_dim, out_dim)) return true;
    // Three and four rows of Q4_0 on more columns than one round of the decode kernel's workgroups takes (64 columns a
    // compute unit; both matrices of a pair count): the decode kernel's block dots, on the vector ALU, grow with rows
    // and columns, the eight-row kernel's time does not.  Four rows: a pair of 14336 columns 18.3 -> 16.7 us, 28672
    // columns 18.5 -> 16.9, 128256 columns 64.6 -> 50.8 (three rows 55.9 -> 49.8); on one round the decode kernel wins
    // (14336 columns 9.9 against 10.9, a pair of 8192 10.2 against 11.3), and three rows on two rounds are even.
    // (Four rows of 4096 values -- eight quantizing wavefronts, which then request their weights behind their
    // quantization -- hold out for two rounds as well: 20480 columns 13.3 against 16.1, a pair of 11008 14.0 against 15.1,
    // 28672 columns 16.5 against 17.0; 128256 columns 65.3 against 52.1.)
    if (tensor_type == AFHIP_TYPE_Q4_0 && in_dim <= 4096 && (rows == 3 || rows == 4)) {
        const size_t round = static_cast<size_t>(gemv_compute_units()) * 64, columns = out_dim * (pair ? 2 : 1);
        const size_t rounds = rows == 4 && rows * in_dim < 16384 ? 1 : 2;
        if (columns > rounds * round && batch_mfma_eight_rows(tensor_type, rows, in_dim, out_dim)) return true;
    }
    // Q8_0, K of 2048 to 4096 (one K share of the eight-row kernel in one round on a wide matrix): four rows from 11008
    // columns on (11008 14.2 -> 12.3 us, 14336 16.0 -> 14.4, 28672 29.1 -> 23.8, a pair of 14336 30.1 -> 23.2; 8192 9.3
    // against 10.0 stays), three rows beyond 14336 (28672 25.9 -> 23.5, K = 2048 x 16384 10.9 -> 9.9; 14336 is even);
    // two rows stay on the decode kernel everywhere (14336 12.6 against 14.4).  One matrix's columns, also for a pair.
    if (tensor_type == AFHIP_TYPE_Q8_0 && in_dim >= 2048 && in_dim <= 4096 &&
        ((rows == 4 && out_dim >= 11008) || (rows == 3 && out_dim > 14336)) && batch_mfma_eight_rows(tensor_type, rows, in_dim, out_dim))
        return true;
    // Two to four rows on a K beyond 4096, against the kernel that shares K out over workgroups and its reduce launch
    // (us, that kernel first): Q4_0 four rows 6144 x 4096 columns 9.9 / 8.4, 8192 x 8192 12.5 / 11.3, 14336 x 4096
    // 12.7 / 11.7, 14336 x 8192 21.0 / 16.5; three rows 6144 x 2048 8.6 / 6.7, 8192 x 4096 8.9 / 9.0, 14336 x 8192
    // 18.9 / 16.5, but 11008 x 4096 10.7 / 11.4 and 14336 x 2048 8.9 / 9.7; two rows stay (8192 x 8192 8.4 / 11.3).
    // Q8_0 three and four rows everywhere (8192 x 8192 20.0 / 15.0, 6144 x 2048 7.7 / 6.9); two rows on a long K or
    // a wide matrix (14336 x 4096 15.7 / 14.3, 6144 x 16384 25.1 / 21.1, but 8192 x 4096 8.2 / 10.0).  (One matrix's
    // columns also for a pair: both halves take the kernel the single op takes.)
    if (in_dim > 4096 && rows >= 2 && rows <= 4 && batch_mfma_eight_rows(tensor_type, rows, in_dim, out_dim)) {
        if (tensor_type == AFHIP_TYPE_Q4_0) {
            if (rows == 4) return true;
            if (rows == 3) return in_dim <= 8192 || out_dim >= 8192;
        } else {
            if (rows >= 3) return true;
            return (in_dim > 11008 && out_dim >= 4096) || out_dim > 8192;
        }
    }
    if (rows < (in_dim > 4096 ? kBatchMfmaMinRows + 1 : kBatchMfmaMinRows)) return false;
    if (tensor_type == AFHIP_TYPE_Q8_0) {
        const size_t shares = (in_dim / 32 + 63) / 64, tiles = (out_dim + 31) / 32;
        return shares == 1 || tiles * shares <= 2 * static_cast<size_t>(gemv_compute_units());
    }
    return true;
}

static GemvTuning gemv_tuning(int tensor_type, int rows, size_t in_dim, size_t out_dim) {
    (void)tensor_type;
    (void)out_dim;
    static const int env_threads = env_int("AFHIP_GEMV_THREADS");
    GemvTuning t;
    // every workgroup quantizes all of X, so large workgroups share that work best
    t.threads = 1024;
    if (env_threads >= 64 && env_threads <= 1024 && env_threads % 64 == 0) {
        t.threads = env_threads;
        t.exact = true;
    }
    return t;
}

// Q4_K: f32 activations against the dequantized weights, one kernel family for any row count;
// on the CPU engine's gated short-K shapes, Q8_K-quantized activations and integer sub-block dots.
static afhip_status linear_q4k_impl(hipStream_t stream, int layout, afhip_buffer dst, afhip_buffer input, afhip_buffer weight,
                                    size_t rows, size_t in_dim, size_t out_dim, afhip_buffer workspace, int dispatch,
                                    bool want_dots,
                                    LaunchCounters* counters, afhip_buffer dst_b, afhip_buffer weight_b,
                                    const Epilogue& ep, const Epilogue& ep_b) {
    const bool pair = weight_b.ptr != 0 || dst_b.ptr != 0;
    if (want_dots) return AFHIP_ERR_INVALID_ARGUMENT;  // the block-dot output exists for the 32-value formats only
    if (dispatch < AFHIP_DISPATCH_AUTO_F32_ACTIVATIONS || dispatch > AFHIP_DISPATCH_MM) return AFHIP_ERR_INVALID_ARGUMENT;
    // f32 activations everywhere (what the engine's accelerator backends compute), also on the CPU engine's gated shapes
    const bool f32_everywhere = dispatch == AFHIP_DISPATCH_AUTO_F32_ACTIVATIONS;
    if (f32_everywhere) dispatch = AFHIP_DISPATCH_AUTO;
    if (layout != AFHIP_LAYOUT_RAW && layout != AFHIP_LAYOUT_PREPARED) return AFHIP_ERR_INVALID_ARGUMENT;
    if (in_dim == 0 || in_dim % 256 != 0) return AFHIP_ERR_INVALID_STATE;
    const bool tiled = layout == AFHIP_LAYOUT_PREPARED;
    size_t out_count, in_count, w_blocks, w_bytes, bytes;
    if (!checked_mul(rows, out_dim, &out_count) || !checked_mul(rows, in_dim, &in_count) ||
        !checked_mul(out_dim + (tiled ? 31 : 0), in_dim / 256, &w_blocks) || !checked_mul(w_blocks, 144, &w_bytes))
        return AFHIP_ERR_INVALID_STATE;
    if (tiled) w_bytes = q4k_tiled_bytes(out_dim, in_dim);
    if (!checked_mul(out_count, 4, &bytes) || bytes > dst.len || (pair && bytes > dst_b.len)) return AFHIP_ERR_INVALID_STATE;
    if (!checked_mul(in_count, 4, &bytes) || bytes > input.len) return AFHIP_ERR_INVALID_STATE;
    if (w_bytes > weight.len || (pair && w_bytes > weight_b.len)) return AFHIP_ERR_INVALID_STATE;
    if (out_count == 0) return AFHIP_OK;
    if (rows > 0x7fffffff || out_dim > 0x7fffffff) return AFHIP_ERR_INVALID_STATE;
    if (in_dim > static_cast<size_t>(gemv_q4k_max_in_dim())) return AFHIP_ERR_OP_UNSUPPORTED;
    if (dst.ptr == 0 || input.ptr == 0 || weight.ptr == 0 || dst.ptr % 4 != 0 || input.ptr % 16 != 0 || weight.ptr % 16 != 0)
        return AFHIP_ERR_INVALID_STATE;
    if (pair && (dst_b.ptr == 0 || weight_b.ptr == 0 || dst_b.ptr % 4 != 0 || weight_b.ptr % 16 != 0))
        return AFHIP_ERR_INVALID_STATE;
    const int kind = dispatch >= 0 ? dispatch : afhip_quant_matmul_select(rows, in_dim, out_dim, AFHIP_FORMAT_Q4_K);
    if (!f32_everywhere && afhip_uses_q8k_activation_quant(AFHIP_TYPE_Q4_K, rows, in_dim, out_dim)) {
        // the CPU engine's gated shapes: activations quantized to Q8_K, integer sub-block dots
        const bool fused = linear_q4k_q8k_fuses_quantizer(tiled, rows, in_dim);  // decode: the quantizer inside the matmul launch
        // (which reads no workspace; the stand-alone quantizer writes the Q8_K rows there)
        if (!fused && (workspace.ptr == 0 || workspace.ptr % 16 != 0 || workspace.len < q4k_q8k_workspace_bytes(rows, in_dim)))
            return AFHIP_ERR_INVALID_STATE;
        if (counters) counters->activation_quant++;
        hipError_t e = fused ? hipSuccess
                             : launch_quantize_q8k(stream, reinterpret_cast<const float*>(input.ptr), static_cast<int>(rows),
                                                   static_cast<int>(in_dim), reinterpret_cast<void*>(workspace.ptr));
        for (int i = 0; e == hipSuccess && i < (pair ? 2 : 1); ++i) {
            if (counters) {
                if (kind == AFHIP_DISPATCH_MMV) counters->mmv++;
                else if (kind == AFHIP_DISPATCH_SMALL_BATCH) counters->small_batch++;
                else counters->mm++;
            }
            if (fused) {  // a pair: both matrices in one launch
                if (i == 0)
                    e = launch_linear_q4k_q8k_fused(stream, reinterpret_cast<float*>(dst.ptr), reinterpret_cast<const float*>(input.ptr),
                                                    reinterpret_cast<const uint8_t*>(weight.ptr), static_cast<int>(rows),
                                                    static_cast<int>(in_dim), static_cast<int>(out_dim), ep,
                                                    pair ? reinterpret_cast<float*>(dst_b.ptr) : nullptr,
                                                    pair ? reinterpret_cast<const uint8_t*>(weight_b.ptr) : nullptr, ep_b);
                continue;
            }
            e = launch_linear_q4k_q8k(stream, reinterpret_cast<float*>(i ? dst_b.ptr : dst.ptr),
                                      reinterpret_cast<const void*>(workspace.ptr),
                                      reinterpret_cast<const uint8_t*>(i ? weight_b.ptr : weight.ptr), tiled,
                                      static_cast<int>(rows), static_cast<int>(in_dim), static_cast<int>(out_dim), i ? ep_b : ep);
        }
        return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
    }
    // three to eight rows with scratch: X as fixed-point digit planes once, then the int8 kernel on each matrix
    static const int env_no_planes = env_int("AFHIP_Q4K_NO_DIGIT_PLANES");
    if (tiled && env_no_planes == 0 && q4k_i8_rows_supports(rows, in_dim) && workspace.ptr != 0 && workspace.ptr % 16 == 0 &&
        workspace.len >= q4k_i8_rows_workspace_bytes(in_dim)) {
        // (few column tiles: two workgroups a tile with half of K each add to the results, which the planes' launch clears)
        const bool two_shares = q4k_i8_rows_two_shares(rows, in_dim, out_dim, pair, ep, ep_b);
        hipError_t e = launch_q4k_digit_planes(stream, reinterpret_cast<const float*>(input.ptr), static_cast<int>(rows),
                                               static_cast<int>(in_dim), reinterpret_cast<void*>(workspace.ptr),
                                               two_shares ? reinterpret_cast<float*>(dst.ptr) : nullptr,
                                               two_shares && pair ? reinterpret_cast<float*>(dst_b.ptr) : nullptr, rows * out_dim);
        if (counters) {
            for (int i = 0; i < (pair ? 2 : 1); ++i) {
                if (kind == AFHIP_DISPATCH_MMV) counters->mmv++;
                else if (kind == AFHIP_DISPATCH_SMALL_BATCH) counters->small_batch++;
                else counters->mm++;
            }
        }
        if (e == hipSuccess)  // a pair: both matrices in one launch
            e = launch_gemv_q4k_i8_rows(stream, reinterpret_cast<float*>(dst.ptr), reinterpret_cast<const void*>(workspace.ptr),
                                        reinterpret_cast<const uint8_t*>(weight.ptr), static_cast<int>(rows), static_cast<int>(in_dim),
                                        static_cast<int>(out_dim), ep, pair ? reinterpret_cast<float*>(dst_b.ptr) : nullptr,
                                        pair ? reinterpret_cast<const uint8_t*>(weight_b.ptr) : nullptr, ep_b, two_shares);
        return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
    }
    // more rows than one GEMV launch holds: X split once into the caller's scratch, then the
    // GEMM (without scratch the GEMV serves them a launch at a time)
    const size_t gemm_rows = static_cast<size_t>(gemm_q4k_min_rows(static_cast<int>(in_dim)));
    const bool gemm = tiled && rows >= gemm_rows && workspace.ptr != 0 && workspace.ptr % 16 == 0 && workspace.len >= gemm_q4k_workspace_bytes(rows, in_dim, out_dim);
    for (int i = 0; i < (pair ? 2 : 1); ++i) {
        if (counters) {
            if (kind == AFHIP_DISPATCH_MMV) counters->mmv++;
            else if (kind == AFHIP_DISPATCH_SMALL_BATCH) counters->small_batch++;
            else counters->mm++;
        }
        if (gemm) {
            hipError_t e = launch_gemm_q4k_tiled(stream, reinterpret_cast<float*>(i ? dst_b.ptr : dst.ptr),
                                                 reinterpret_cast<const float*>(input.ptr),
                                                 reinterpret_cast<const uint8_t*>(i ? weight_b.ptr : weight.ptr),
                                                 reinterpret_cast<void*>(workspace.ptr), static_cast<int>(rows),
                                                 static_cast<int>(in_dim), static_cast<int>(out_dim), i ? ep_b : ep, i == 0);
            if (e != hipSuccess) return static_cast<afhip_status>(e);
            continue;
        }
        if (tiled) {  // a pair goes down together: one launch for both where the int8 kernel serves the rows
            if (i == 1) continue;
            hipError_t e = launch_gemv_q4k_tiled(stream, reinterpret_cast<float*>(dst.ptr), reinterpret_cast<const float*>(input.ptr),
                                                 reinterpret_cast<const uint8_t*>(weight.ptr), static_cast<int>(rows), static_cast<int>(in_dim),
                                                 static_cast<int>(out_dim), ep, pair ? reinterpret_cast<float*>(dst_b.ptr) : nullptr,
                                                 pair ? reinterpret_cast<const uint8_t*>(weight_b.ptr) : nullptr, ep_b);
            if (e != hipSuccess) return static_cast<afhip_status>(e);
            continue;
        }
        hipError_t e = launch_gemv_q4k(stream, reinterpret_cast<float*>(i ? dst_b.ptr : dst.ptr), reinterpret_cast<const float*>(input.ptr),
                                       reinterpret_cast<const uint8_t*>(i ? weight_b.ptr : weight.ptr), static_cast<int>(rows),
                                       static_cast<int>(in_dim), static_cast<int>(out_dim), i ? ep_b : ep);
        if (e != hipSuccess) return static_cast<afhip_status>(e);
    }
    return AFHIP_OK;
}

static afhip_status linear_impl_body(void* stream_v, int tensor_type, int layout, afhip_buffer dst, afhip_buffer input,
                                     afhip_buffer weight, size_t rows, size_t in_dim, size_t out_dim, afhip_buffer workspace,
                                     int dispatch, afhip_buffer dots, LaunchCounters* counters, afhip_buffer dst_b,
                                     afhip_buffer weight_b, const LinearExtras& extras, bool* quantizer_marked);

afhip_status linear_impl(void* stream_v, int tensor_type, int layout, afhip_buffer dst, afhip_buffer input,
                         afhip_buffer weight, size_t rows, size_t in_dim, size_t out_dim, afhip_buffer workspace,
                         int dispatch, afhip_buffer dots, LaunchCounters* counters, afhip_buffer dst_b,
                         afhip_buffer weight_b, const LinearExtras& extras) {
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    bool quantizer_marked = false;
    mark_phase(counters, 0, stream);
    const afhip_status s = linear_impl_body(stream_v, tensor_type, layout, dst, input, weight, rows, in_dim, out_dim, workspace,
                                            dispatch, dots, counters, dst_b, weight_b, extras, &quantizer_marked);
    if (!quantizer_marked) mark_phase(counters, 1, stream);  // no stand-alone quantizer ran (or nothing ran): an empty phase
    mark_phase(counters, 2, stream);
    return s;
}

static afhip_status linear_impl_body(void* stream_v, int tensor_type, int layout, afhip_buffer dst, afhip_buffer input,
                                     afhip_buffer weight, size_t rows, size_t in_dim, size_t out_dim, afhip_buffer workspace,
                                     int dispatch, afhip_buffer dots, LaunchCounters* counters, afhip_buffer dst_b,
                                     afhip_buffer weight_b, const LinearExtras& extras, bool* quantizer_marked) {
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    const bool pair = weight_b.ptr != 0 || dst_b.ptr != 0;
    // biases: f32 [out_dim], the second one only with a second matrix; activation and residual
    // (f32 [rows][out_dim]) only with one matrix; none of them with the block dots
    const bool any_extra = extras.bias.ptr != 0 || extras.bias_b.ptr != 0 || extras.residual.ptr != 0 ||
                           extras.activation != AFHIP_ACTIVATION_NONE;
    if ((extras.bias_b.ptr != 0 && !pair) || (any_extra && dots.ptr != 0)) return AFHIP_ERR_INVALID_ARGUMENT;
    if (pair && (extras.residual.ptr != 0 || extras.activation != AFHIP_ACTIVATION_NONE)) return AFHIP_ERR_INVALID_ARGUMENT;
    if (extras.activation < AFHIP_ACTIVATION_NONE || extras.activation > AFHIP_ACTIVATION_GELU) return AFHIP_ERR_INVALID_ARGUMENT;
    for (const afhip_buffer& b : {extras.bias, extras.bias_b}) {
        size_t need;
        if (b.ptr == 0) continue;
        if (b.ptr % 4 != 0 || !checked_mul(out_dim, 4, &need) || b.len < need) return AFHIP_ERR_INVALID_STATE;
    }
    if (extras.residual.ptr != 0) {
        size_t count, need;
        if (extras.residual.ptr % 4 != 0 || !checked_mul(rows, out_dim, &count) || !checked_mul(count, 4, &need) ||
            extras.residual.len < need)
            return AFHIP_ERR_INVALID_STATE;
    }
    Epilogue ep, ep_b;
    ep.bias = reinterpret_cast<const float*>(extras.bias.ptr);
    ep.residual = reinterpret_cast<const float*>(extras.residual.ptr);
    ep.activation = extras.activation;  // AFHIP_ACTIVATION_* and kAct* share their values
    ep_b.bias = reinterpret_cast<const float*>(extras.bias_b.ptr);
    if (tensor_type == AFHIP_TYPE_Q4_K)
        return linear_q4k_impl(stream, layout, dst, input, weight, rows, in_dim, out_dim, workspace, dispatch, dots.ptr != 0,
                               counters, dst_b, weight_b, ep, ep_b);
    const size_t bb = block_bytes(tensor_type);
    if (bb == 0) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    if (layout != AFHIP_LAYOUT_RAW && layout != AFHIP_LAYOUT_PREPARED) return AFHIP_ERR_INVALID_ARGUMENT;
    if (dispatch < AFHIP_DISPATCH_AUTO_F32_ACTIVATIONS || dispatch > AFHIP_DISPATCH_MM) return AFHIP_ERR_INVALID_ARGUMENT;
    if (dispatch == AFHIP_DISPATCH_AUTO_F32_ACTIVATIONS) dispatch = AFHIP_DISPATCH_AUTO;  // a Q4_K matter: the same as auto here
    if (in_dim == 0 || in_dim % 32 != 0) return AFHIP_ERR_INVALID_STATE;
    const size_t kb = in_dim / 32;
    size_t out_count, in_count, w_blocks, w_bytes, bytes;
    if (!checked_mul(rows, out_dim, &out_count) || !checked_mul(rows, in_dim, &in_count) ||
        !checked_mul(out_dim, kb, &w_blocks) || !checked_mul(w_blocks, bb, &w_bytes))
        return AFHIP_ERR_INVALID_STATE;
    const bool want_dots = dots.ptr != 0;
    if (!want_dots) {
        if (!checked_mul(out_count, 4, &bytes) || bytes > dst.len) return AFHIP_ERR_INVALID_STATE;
    } else {
        size_t n;
        if (!checked_mul(out_count, kb, &n) || !checked_mul(n, 4, &bytes) || bytes > dots.len) return AFHIP_ERR_INVALID_STATE;
    }
    if (!checked_mul(in_count, 4, &bytes) || bytes > input.len) return AFHIP_ERR_INVALID_STATE;
    if (layout == AFHIP_LAYOUT_PREPARED) {  // quant bytes, scales, and the scales in tile order
        w_bytes = afhip_prepared_weight_bytes(tensor_type, out_dim, in_dim);
        if (w_bytes == 0 && w_blocks != 0) return AFHIP_ERR_INVALID_STATE;
    }
    if (w_bytes > weight.len) return AFHIP_ERR_INVALID_STATE;
    if (pair) {
        if (want_dots) return AFHIP_ERR_INVALID_ARGUMENT;
        if (!checked_mul(out_count, 4, &bytes) || bytes > dst_b.len || w_bytes > weight_b.len) return AFHIP_ERR_INVALID_STATE;
    }
    if (out_count == 0) return AFHIP_OK;
    if (!fits_u32(rows) || !fits_u32(in_dim) || !fits_u32(out_dim) || in_dim > 0x7fffffff || out_dim > 0x7fffffff ||
        rows > 0x7fffffff)
        return AFHIP_ERR_INVALID_STATE;
    if ((!want_dots && dst.ptr == 0) || input.ptr == 0 || weight.ptr == 0) return AFHIP_ERR_INVALID_STATE;
    // 128-bit activation loads; prepared weights are read with 128-bit loads, raw GGUF bytes with 16-bit loads
    if (input.ptr % 16 != 0 || dst.ptr % 4 != 0 || dots.ptr % 4 != 0) return AFHIP_ERR_INVALID_STATE;
    if (weight.ptr % (layout == AFHIP_LAYOUT_PREPARED ? 16 : 2) != 0) return AFHIP_ERR_INVALID_STATE;
    if (pair && (dst_b.ptr == 0 || weight_b.ptr == 0 || dst_b.ptr % 4 != 0 ||
                 weight_b.ptr % (layout == AFHIP_LAYOUT_PREPARED ? 16 : 2) != 0))
        return AFHIP_ERR_INVALID_STATE;

    float* y = reinterpret_cast<float*>(dst.ptr);
    float* y_b = reinterpret_cast<float*>(dst_b.ptr);
    const uint8_t* w_b = reinterpret_cast<const uint8_t*>(weight_b.ptr);
    int* dot_out = reinterpret_cast<int*>(dots.ptr);
    const float* x = reinterpret_cast<const float*>(input.ptr);
    const uint8_t* w = reinterpret_cast<const uint8_t*>(weight.ptr);

    // The block dots only exist on the activation-quantized route.
    const bool route_a = want_dots || afhip_uses_activation_quant(rows, in_dim, out_dim);
    if (!route_a) {
        if (counters) counters->f32_route++;
        hipError_t e = launch_linear_generic(stream, tensor_type, layout, false, y, nullptr, x, nullptr, nullptr, w,
                                             static_cast<int>(rows), static_cast<int>(in_dim), static_cast<int>(out_dim), ep);
        if (e == hipSuccess && pair) {
            if (counters) counters->f32_route++;
            e = launch_linear_generic(stream, tensor_type, layout, false, y_b, nullptr, x, nullptr, nullptr, w_b,
                                      static_cast<int>(rows), static_cast<int>(in_dim), static_cast<int>(out_dim), ep_b);
        }
        return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
    }

    int kind = dispatch >= 0 ? dispatch : afhip_quant_matmul_select(rows, in_dim, out_dim,
                                                                    afhip_quant_format_from_tensor_type(tensor_type));
    const int chunk = gemv_row_chunk(rows, in_dim);
    const bool fused_ok = layout == AFHIP_LAYOUT_PREPARED && chunk > 0 && kind != AFHIP_DISPATCH_SCALAR &&
                          in_dim <= static_cast<size_t>(gemv_fused_max_in_dim());
    // Five to 64 (128) rows: the weights are read once, so the single-shot MFMA kernel (X quantized into
    // MFMA operand order first) beats both the row-by-row GEMV and the tiled GEMM.
    if (layout == AFHIP_LAYOUT_PREPARED && !want_dots && kind != AFHIP_DISPATCH_SCALAR &&
        batch_mfma_preferred(tensor_type, rows, in_dim, out_dim, pair) &&
        // (below five rows the decode kernel, which needs no workspace, remains for a caller that lends none)
        (rows >= kBatchMfmaMinRows || (workspace.ptr != 0 && workspace.ptr % 16 == 0 &&
                                       workspace.len >= batch_mfma_workspace_bytes(tensor_type, rows, in_dim, out_dim)))) {
        const size_t need = batch_mfma_workspace_bytes(tensor_type, rows, in_dim, out_dim);
        if (workspace.ptr == 0 || workspace.len < need || workspace.ptr % 16 != 0) return AFHIP_ERR_INVALID_STATE;
        if (counters) {
            if (kind == AFHIP_DISPATCH_MMV) counters->mmv++;
            else if (kind == AFHIP_DISPATCH_SMALL_BATCH) counters->small_batch++;
            else counters->mm++;
            if (pair) {
                if (kind == AFHIP_DISPATCH_MM) counters->mm++;
            }
            counters->activation_quant++;
        }
        // (the launcher records the end of its quantizer launch for an op that is being timed)
        void* quantizer_done = counters && counters->phase_events ? counters->phase_events[1] : nullptr;
        if (quantizer_done) *quantizer_marked = true;
        hipError_t e = launch_batch_mfma(stream, tensor_type, y, x, w, static_cast<int>(rows), static_cast<int>(in_dim),
                                         static_cast<int>(out_dim), reinterpret_cast<uint8_t*>(workspace.ptr), pair ? y_b : nullptr,
                                         pair ? w_b : nullptr, ep, ep_b, quantizer_done);
        return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
    }
    if (layout == AFHIP_LAYOUT_PREPARED && kind == AFHIP_DISPATCH_MM) {
        // rows >= 9 (or a plan that asks for mul_mm): quantize X once, then the int8-MFMA GEMM
        const WorkspaceView ws = workspace_view(workspace.ptr, rows, in_dim);
        if (workspace.ptr == 0 || workspace.len < ws.bytes || workspace.ptr % 16 != 0) return AFHIP_ERR_INVALID_STATE;
        if (counters) {
            counters->mm++;
            counters->activation_quant++;
        }
        hipError_t e = launch_quantize_activations(stream, x, static_cast<int>(rows), static_cast<int>(in_dim), ws.qx,
                                                   ws.sx, ws.sums);
        if (e == hipSuccess) {
            mark_phase(counters, 1, stream);
            *quantizer_marked = true;
        }
        if (e != hipSuccess) return static_cast<afhip_status>(e);
        // room behind the quantized activations for the partial sums of K shares (small grids): optional
        const size_t partial_at = (ws.bytes + 255) / 256 * 256;
        const size_t partial_bytes = gemm_i8_partial_bytes(rows, in_dim, out_dim);
        float* partial = partial_bytes != 0 && workspace.len >= partial_at + partial_bytes
                             ? reinterpret_cast<float*>(workspace.ptr + partial_at) : nullptr;
        e = launch_gemm_i8(stream, tensor_type, want_dots ? nullptr : y, dot_out, ws.qx, ws.sx, w, static_cast<int>(rows),
                           static_cast<int>(in_dim), static_cast<int>(out_dim), ep, partial);
        if (e == hipSuccess && pair) {  // the second matrix reuses the quantized activations (and the partial sums' room)
            if (counters) counters->mm++;
            e = launch_gemm_i8(stream, tensor_type, y_b, nullptr, ws.qx, ws.sx, w_b, static_cast<int>(rows),
                               static_cast<int>(in_dim), static_cast<int>(out_dim), ep_b, partial);
        }
        return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
    }
    // (Two rows up to K = 11008 stay on the decode kernel below: one launch, the K slices of a column group meet inside the
    // workgroup.  Measured against this path's kernel + reduce launch: K = 6144 x N = 4096 6.0 against 7.2 us, K = N = 8192
    // 8.7 against 10.5, a pair of K = 8192 x N = 4096 8.7 against 12.2, K = 11008 8.4 against 9.0, Q8_0 K = N = 8192 14.7
    // against 19.2; from K = 12288 on this path wins -- 9.3 against 9.5, N = 8192 15.0 against 17.0 -- and with three and
    // four rows it does from K = 6144 on.)
    if (fused_ok && rows >= 2 && in_dim > 4096 && !(rows == 2 && in_dim <= 11008)) {
        // small batches on a K longer than 4096 (also when a plan forces them on more rows: slices
        // of eight rows): K is shared out over workgroups, each of which stages and quantizes only
        // its 4096-value slice of X; the slices' sums meet in the caller's scratch.
        if (counters) {
            if (kind == AFHIP_DISPATCH_MMV) counters->mmv++;
            else if (kind == AFHIP_DISPATCH_SMALL_BATCH) counters->small_batch++;
            else counters->mm++;
        }
        constexpr size_t kBatchRows = 8;
        const size_t partial_bytes = want_dots ? 0 : gemv_batch_partial_bytes(rows < kBatchRows ? rows : kBatchRows, in_dim, out_dim, pair);
        if (partial_bytes != 0 && (workspace.ptr == 0 || workspace.len < partial_bytes || workspace.ptr % 16 != 0))
            return AFHIP_ERR_INVALID_STATE;
        for (size_t r0 = 0; r0 < rows; r0 += kBatchRows) {
            const int nr = static_cast<int>(rows - r0 < kBatchRows ? rows - r0 : kBatchRows);
            Epilogue ep_rows = ep;
            if (ep_rows.residual) ep_rows.residual += r0 * out_dim;
            hipError_t e = launch_gemv_batch(stream, tensor_type, want_dots ? nullptr : y + r0 * out_dim,
                                             want_dots ? dot_out + r0 * out_dim * kb : nullptr, x + r0 * in_dim, w, nr,
                                             static_cast<int>(in_dim), static_cast<int>(out_dim),
                                             partial_bytes ? reinterpret_cast<float*>(workspace.ptr) : nullptr,
                                             pair ? y_b + r0 * out_dim : nullptr, pair ? w_b : nullptr, ep_rows, ep_b);
            if (e != hipSuccess) return static_cast<afhip_status>(e);
        }
        return AFHIP_OK;
    }

    if (fused_ok) {
        // mmv / small_batch (also when a plan forces them on more rows: 16-row slices).
        // Few rows: the GEMV quantizes X in its own prologue, one launch.  More: every
        // workgroup would repeat too much of that work, so X is quantized once by its own
        // kernel into the caller's scratch.  (AFHIP_GEMV_FUSED_ROWS caps the rows for tuning runs.)
        static const int env_fused_rows = env_int("AFHIP_GEMV_FUSED_ROWS");
        const size_t type_rows = 4;  // both formats
        const size_t fused_rows = env_fused_rows >= 1 && env_fused_rows <= 4 ? size_t(env_fused_rows) : type_rows;
        const bool prequantize = rows > fused_rows || (rows > 2 && rows * kb > kGemvFusedQuantBlocks);
        const WorkspaceView ws = workspace_view(workspace.ptr, rows, in_dim);
        if (prequantize && (workspace.ptr == 0 || workspace.len < ws.bytes || workspace.ptr % 16 != 0))
            return AFHIP_ERR_INVALID_STATE;
        if (counters) {
            if (kind == AFHIP_DISPATCH_MMV) counters->mmv++;
            else if (kind == AFHIP_DISPATCH_SMALL_BATCH) counters->small_batch++;
            else counters->mm++;
            if (prequantize) counters->activation_quant++;
        }
        if (prequantize) {
            hipError_t e = launch_quantize_activations(stream, x, static_cast<int>(rows), static_cast<int>(in_dim), ws.qx,
                                                       ws.sx, ws.sums);
            if (e == hipSuccess) {
                mark_phase(counters, 1, stream);
                *quantizer_marked = true;
            }
            if (e != hipSuccess) return static_cast<afhip_status>(e);
        }
        for (size_t r0 = 0; r0 < rows; r0 += static_cast<size_t>(chunk)) {
            const int nr = rows - r0 < static_cast<size_t>(chunk) ? static_cast<int>(rows - r0) : chunk;
            const GemvTuning tune = gemv_tuning(tensor_type, nr, in_dim, out_dim);
            GemvActivations pre;
            if (prequantize) {
                pre.q = ws.qx + r0 * in_dim;
                pre.scale = ws.sx + r0 * kb;
                pre.sum = ws.sums + r0 * kb;
            }
            // a pair is one launch over the columns of both matrices
            Epilogue ep_rows = ep;
            if (ep_rows.residual) ep_rows.residual += r0 * out_dim;
            hipError_t e = launch_gemv_fused(stream, tensor_type, want_dots ? nullptr : y + r0 * out_dim,
                                             want_dots ? dot_out + r0 * out_dim * kb : nullptr, x + r0 * in_dim, pre, w,
                                             nr, static_cast<int>(in_dim), static_cast<int>(out_dim), tune,
                                             pair ? y_b + r0 * out_dim : nullptr, pair ? w_b : nullptr, ep_rows, ep_b);
            if (e != hipSuccess) return static_cast<afhip_status>(e);
        }
        return AFHIP_OK;
    }

    // Generic activation-quantized path: quantize into the caller's scratch first.
    const WorkspaceView ws = workspace_view(workspace.ptr, rows, in_dim);
    if (workspace.ptr == 0 || workspace.len < ws.bytes || workspace.ptr % 16 != 0) return AFHIP_ERR_INVALID_STATE;
    if (counters) {
        counters->activation_quant++;
        if (kind == AFHIP_DISPATCH_MMV) counters->mmv++;
        else if (kind == AFHIP_DISPATCH_SMALL_BATCH) counters->small_batch++;
        else counters->mm++;
    }
    hipError_t e = launch_quantize_activations(stream, x, static_cast<int>(rows), static_cast<int>(in_dim), ws.qx, ws.sx,
                                               ws.sums);
    if (e == hipSuccess) {
        mark_phase(counters, 1, stream);
        *quantizer_marked = true;
    }
    if (e != hipSuccess) return static_cast<afhip_status>(e);
    e = launch_linear_generic(stream, tensor_type, layout, true, want_dots ? nullptr : y, dot_out, nullptr, ws.qx, ws.sx,
                              w, static_cast<int>(rows), static_cast<int>(in_dim), static_cast<int>(out_dim), ep);
    if (e == hipSuccess && pair)
        e = launch_linear_generic(stream, tensor_type, layout, true, y_b, nullptr, nullptr, ws.qx, ws.sx, w_b,
                                  static_cast<int>(rows), static_cast<int>(in_dim), static_cast<int>(out_dim), ep_b);
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

static size_t argmax_logits_bytes(size_t out_dim) { return (out_dim * 4 + 255) / 256 * 256; }
// scratch of the one-row linear inside the fused lm_head (Q4_K: none, or the Q8_K activations on its gated shapes)
static size_t argmax_linear_bytes(int tensor_type, size_t in_dim, size_t out_dim) {
    if (tensor_type != AFHIP_TYPE_Q4_K) return workspace_view(0, 1, in_dim).bytes;
    const size_t q8k = afhip_uses_q8k_activation_quant(tensor_type, 1, in_dim, out_dim) ? q4k_q8k_workspace_bytes(1, in_dim) : 0;
    return q8k > 256 ? q8k : 256;
}
static size_t argmax_keys_bytes(size_t dim) {
    if (dim > 0x7fffffff) return 0;
    const int groups = argmax_row_workgroups(static_cast<int>(dim));
    return groups > 1 ? (static_cast<size_t>(groups) * 8 + 255) / 256 * 256 : 0;
}

afhip_status argmax_last_row_impl(void* stream, afhip_buffer token_u32, afhip_buffer token_f32, afhip_buffer input,
                                  size_t rows, size_t dim, afhip_buffer workspace) {
    if (rows == 0 || dim == 0) return AFHIP_ERR_INVALID_SHAPE;  // error.InvalidTensorShape, native_compute.zig:37903
    size_t count, bytes;
    if (!checked_mul(rows, dim, &count) || !checked_mul(count, 4, &bytes)) return AFHIP_ERR_INVALID_SHAPE;
    if (bytes > input.len) return AFHIP_ERR_INVALID_SHAPE;
    if (dim > 0x7fffffff || input.ptr == 0 || input.ptr % 4 != 0) return AFHIP_ERR_INVALID_STATE;
    if (token_u32.ptr == 0 && token_f32.ptr == 0) return AFHIP_ERR_INVALID_STATE;
    if ((token_u32.ptr != 0 && (token_u32.len < 4 || token_u32.ptr % 4 != 0)) ||
        (token_f32.ptr != 0 && (token_f32.len < 4 || token_f32.ptr % 4 != 0)))
        return AFHIP_ERR_INVALID_STATE;
    // a long row is scanned by several workgroups when the caller lends room for their keys
    unsigned long long* keys = nullptr;
    if (workspace.ptr != 0 && workspace.ptr % 8 == 0 && argmax_keys_bytes(dim) != 0 && workspace.len >= argmax_keys_bytes(dim))
        keys = reinterpret_cast<unsigned long long*>(workspace.ptr);
    hipError_t e = launch_argmax_row(static_cast<hipStream_t>(stream),
                                     reinterpret_cast<const float*>(input.ptr) + (rows - 1) * dim, static_cast<int>(dim),
                                     keys, reinterpret_cast<uint32_t*>(token_u32.ptr),
                                     reinterpret_cast<float*>(token_f32.ptr));
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

// Workspace: [keys or logits: out_dim f32, padded to 256][scratch of a one-row linear][keys of the argmax over logits]
afhip_status linear_argmax_impl(void* stream, int tensor_type, int layout, afhip_buffer token_u32,
                                afhip_buffer token_f32, afhip_buffer input, afhip_buffer weight, size_t rows,
                                size_t in_dim, size_t out_dim, afhip_buffer workspace, LaunchCounters* counters) {
    const bool q4k = tensor_type == AFHIP_TYPE_Q4_K;
    const size_t bb = q4k ? 144 : block_bytes(tensor_type);
    const size_t block_values = q4k ? 256 : 32;
    if (bb == 0) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    if (layout != AFHIP_LAYOUT_RAW && layout != AFHIP_LAYOUT_PREPARED) return AFHIP_ERR_INVALID_ARGUMENT;
    if (rows == 0 || in_dim == 0 || out_dim == 0) return AFHIP_ERR_INVALID_SHAPE;
    if (in_dim % block_values != 0) return AFHIP_ERR_INVALID_STATE;
    size_t count, bytes, w_blocks, w_bytes;
    if (!checked_mul(rows, in_dim, &count) || !checked_mul(count, 4, &bytes) || bytes > input.len)
        return AFHIP_ERR_INVALID_STATE;
    if (!checked_mul(out_dim, in_dim / block_values, &w_blocks) || !checked_mul(w_blocks, bb, &w_bytes)) return AFHIP_ERR_INVALID_STATE;
    if (q4k && layout == AFHIP_LAYOUT_PREPARED) {
        if (!checked_mul(out_dim + 31, in_dim / block_values, &w_blocks) || !checked_mul(w_blocks, bb, &w_bytes))
            return AFHIP_ERR_INVALID_STATE;
        w_bytes = q4k_tiled_bytes(out_dim, in_dim);
    } else if (!q4k && layout == AFHIP_LAYOUT_PREPARED) {
        w_bytes = afhip_prepared_weight_bytes(tensor_type, out_dim, in_dim);
        if (w_bytes == 0) return AFHIP_ERR_INVALID_STATE;
    }
    if (w_bytes > weight.len) return AFHIP_ERR_INVALID_STATE;
    if (in_dim > 0x7fffffff || out_dim > 0x7fffffff || input.ptr == 0 || input.ptr % 16 != 0 || weight.ptr == 0)
        return AFHIP_ERR_INVALID_STATE;
    if ((token_u32.ptr == 0 && token_f32.ptr == 0) ||
        (token_u32.ptr != 0 && (token_u32.len < 4 || token_u32.ptr % 4 != 0)) ||
        (token_f32.ptr != 0 && (token_f32.len < 4 || token_f32.ptr % 4 != 0)))
        return AFHIP_ERR_INVALID_STATE;
    const size_t logits_bytes = argmax_logits_bytes(out_dim);
    if (workspace.ptr == 0 || workspace.ptr % 256 != 0 ||
        workspace.len < afhip_linear_argmax_workspace_bytes(tensor_type, in_dim, out_dim))
        return AFHIP_ERR_INVALID_STATE;
    // only the last row's logits matter: one GEMV whatever `rows` is
    const afhip_buffer last_row{input.ptr + (rows - 1) * in_dim * 4, in_dim * 4};

    if (!q4k && layout == AFHIP_LAYOUT_PREPARED && weight.ptr % 16 == 0 && afhip_uses_activation_quant(1, in_dim, out_dim) &&
        in_dim <= static_cast<size_t>(gemv_fused_max_in_dim()) && gemv_row_chunk(1, in_dim) > 0) {
        // the GEMV's workgroups keep the best of their own columns; no logits are written
        unsigned long long* keys = reinterpret_cast<unsigned long long*>(workspace.ptr);  // at most (out_dim + 1) / 2 of them
        int key_count = 0;
        if (counters) counters->mmv++;
        hipError_t e = launch_gemv_argmax_keys(static_cast<hipStream_t>(stream), tensor_type, keys, &key_count,
                                               reinterpret_cast<const float*>(last_row.ptr),
                                               reinterpret_cast<const uint8_t*>(weight.ptr), static_cast<int>(in_dim),
                                               static_cast<int>(out_dim), gemv_tuning(tensor_type, 1, in_dim, out_dim));
        if (e == hipSuccess)
            e = launch_argmax_keys(static_cast<hipStream_t>(stream), keys, key_count,
                                   reinterpret_cast<uint32_t*>(token_u32.ptr), reinterpret_cast<float*>(token_f32.ptr));
        return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
    }

    const afhip_buffer logits{workspace.ptr, out_dim * 4};
    const size_t linear_bytes = argmax_linear_bytes(tensor_type, in_dim, out_dim);
    const afhip_buffer linear_ws{workspace.ptr + logits_bytes, linear_bytes};
    const size_t keys_offset = logits_bytes + (linear_bytes + 255) / 256 * 256;
    const afhip_buffer keys_ws{workspace.ptr + keys_offset, workspace.len - keys_offset};
    afhip_status s = linear_impl(stream, tensor_type, layout, logits, last_row, weight, 1, in_dim, out_dim, linear_ws,
                                 -1, afhip_buffer{0, 0}, counters);
    if (s != AFHIP_OK) return s;
    return argmax_last_row_impl(stream, token_u32, token_f32, logits, 1, out_dim, keys_ws);
}

}  // namespace afhip

using namespace afhip;

extern "C" {

const char* afhip_status_string(afhip_status status) {
    switch (status) {
        case AFHIP_OK: return "ok";
        case AFHIP_ERR_INVALID_STATE: return "InvalidHipState";
        case AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE: return "UnsupportedTensorType";
        case AFHIP_ERR_INVALID_SHAPE: return "InvalidShape";
        case AFHIP_ERR_WEIGHT_NOT_FOUND: return "WeightNotFound";
        case AFHIP_ERR_OP_UNSUPPORTED: return "HipOpUnsupported";
        case AFHIP_ERR_INVALID_PARTITION_PLAN: return "InvalidPartitionPlan";
        case AFHIP_ERR_UNAVAILABLE: return "HipUnavailable";
        case AFHIP_ERR_NO_DEVICES: return "NoHipDevices";
        case AFHIP_ERR_OUT_OF_MEMORY: return "OutOfMemory";
        case AFHIP_ERR_INVALID_ARGUMENT: return "InvalidArgument";
        case AFHIP_ERR_SMOKE_MISMATCH: return "HipSmokeMismatch";
        case AFHIP_ERR_INVALID_TOKEN_ID: return "InvalidTokenId";
        case AFHIP_ERR_GGUF_INVALID_MAGIC: return "InvalidGgufMagic";
        case AFHIP_ERR_GGUF_UNEXPECTED_EOF: return "UnexpectedEndOfFile";
        case AFHIP_ERR_GGUF_UNSUPPORTED_METADATA: return "UnsupportedMetadataType";
        case AFHIP_ERR_GGUF_NESTED_ARRAY: return "UnsupportedNestedMetadataArray";
        case AFHIP_ERR_TENSOR_NOT_FOUND: return "TensorNotFound";
        case AFHIP_ERR_IO: return "FileNotAccessible";
        default: break;
    }
    if (status > 0) return hipGetErrorName(static_cast<hipError_t>(status));
    return "unknown";
}

// ---- graph/quant_matmul.zig

static size_t format_values_per_block(int format) {
    switch (format) {  // Format.valuesPerBlock, :84-117
        case AFHIP_FORMAT_Q4_0:
        case AFHIP_FORMAT_Q8_0: return 32;
        case AFHIP_FORMAT_Q4_K: return 256;
        case AFHIP_FORMAT_F32: return 1;
        default: return 0;
    }
}

static bool valid_shape(size_t rows, size_t in_dim, size_t out_dim, int format) {  // validShape, :566-576
    if (rows == 0 || in_dim == 0 || out_dim == 0) return false;
    const size_t vpb = format_values_per_block(format);
    if (vpb == 0) return false;
    return in_dim % vpb == 0;
}

int afhip_quant_matmul_select(size_t rows, size_t in_dim, size_t out_dim, int format) {  // select, :263-268
    if (!valid_shape(rows, in_dim, out_dim, format)) return AFHIP_DISPATCH_SCALAR;
    if (rows >= 2 && rows <= 8) return AFHIP_DISPATCH_SMALL_BATCH;
    if (rows >= 9) return AFHIP_DISPATCH_MM;
    return AFHIP_DISPATCH_MMV;
}

int afhip_quant_row_bucket(size_t rows) {  // rowBucket, :558-564
    if (rows == 0) return AFHIP_ROWS_0;
    if (rows == 1) return AFHIP_ROWS_1;
    if (rows <= 8) return AFHIP_ROWS_2_8;
    if (rows <= 64) return AFHIP_ROWS_9_64;
    return AFHIP_ROWS_65_PLUS;
}

void afhip_quant_matmul_plan(size_t rows, size_t in_dim, size_t out_dim, int format, afhip_quant_plan* out) {
    if (!out) return;
    const int d = afhip_quant_matmul_select(rows, in_dim, out_dim, format);
    out->dispatch = static_cast<uint8_t>(d);
    // primitiveForDispatch, :270-277
    static const uint8_t prim[4] = {AFHIP_PRIM_SCALAR, AFHIP_PRIM_MAT_VEC, AFHIP_PRIM_MAT_VEC_EXT, AFHIP_PRIM_MAT_MAT};
    out->primitive = prim[d];
    // operatorForDispatch, :279-287: every format known here supports mul_mv / mul_mv_ext / mul_mm
    const bool known = format == AFHIP_FORMAT_Q4_0 || format == AFHIP_FORMAT_Q8_0 || format == AFHIP_FORMAT_Q4_K ||
                       format == AFHIP_FORMAT_F32;
    static const uint8_t op[4] = {AFHIP_OP_FALLBACK, AFHIP_OP_MUL_MV, AFHIP_OP_MUL_MV_EXT, AFHIP_OP_MUL_MM};
    out->op = known ? op[d] : static_cast<uint8_t>(AFHIP_OP_FALLBACK);
    out->row_bucket = static_cast<uint8_t>(afhip_quant_row_bucket(rows));
    out->format = static_cast<uint16_t>(format);
    out->rows = rows;
    out->in_dim = in_dim;
    out->out_dim = out_dim;
}

int afhip_quant_format_from_tensor_type(int tensor_type) {  // backend_contracts.zig:199-236
    switch (tensor_type) {
        case AFHIP_TYPE_Q4_0: return AFHIP_FORMAT_Q4_0;
        case AFHIP_TYPE_Q8_0: return AFHIP_FORMAT_Q8_0;
        case AFHIP_TYPE_Q4_K: return AFHIP_FORMAT_Q4_K;
        case AFHIP_TYPE_F32: return AFHIP_FORMAT_F32;
        default: return AFHIP_FORMAT_UNKNOWN;
    }
}

int afhip_uses_activation_quant(size_t rows, size_t in_dim, size_t out_dim) {
    (void)rows;
    return out_dim >= 512 && in_dim / 32 >= 3;
}

int afhip_uses_q8k_activation_quant(int tensor_type, size_t rows, size_t in_dim, size_t out_dim) {
    if (tensor_type != AFHIP_TYPE_Q4_K || in_dim % 256 != 0 || out_dim < 512) return 0;
    const size_t row_blocks = in_dim / 256;
    if (!(row_blocks == 2 || row_blocks == 3 || row_blocks == 6 || row_blocks == 8 || row_blocks == 12)) return 0;
    if (rows == 1 || rows == 2 || rows == 4 || rows == 9) return 1;
    if (rows == 50 || rows == 64 || rows == 77 || rows == 197 || rows == 257 || rows == 308 || rows == 514) return 1;
    return rows > 0 && rows <= 308 && rows % 77 == 0;
}

// ---- launchers

size_t afhip_linear_workspace_bytes(int tensor_type, size_t rows, size_t in_dim, size_t out_dim) {
    if (tensor_type == AFHIP_TYPE_Q4_K) {  // the split of X for the prefill GEMM; decode rows need none
        size_t count, bytes;
        if (in_dim == 0 || in_dim % 256 != 0 || in_dim > 0x7fffffff || out_dim == 0 || !checked_mul(rows, in_dim, &count) ||
            !checked_mul(count, 8, &bytes))
            return 0;
        if (afhip_uses_q8k_activation_quant(tensor_type, rows, in_dim, out_dim)) return q4k_q8k_workspace_bytes(rows, in_dim);
        const size_t gemm_rows = static_cast<size_t>(gemm_q4k_min_rows(static_cast<int>(in_dim)));
        const size_t gemm_bytes = rows >= gemm_rows ? gemm_q4k_workspace_bytes(rows, in_dim, out_dim) : 0;
        const size_t planes_bytes = q4k_i8_rows_supports(rows, in_dim) ? q4k_i8_rows_workspace_bytes(in_dim) : 0;  // 3 .. 8 rows
        return gemm_bytes > planes_bytes ? gemm_bytes : planes_bytes;
    }
    if (block_bytes(tensor_type) == 0 || in_dim % 32 != 0 || rows == 0 || out_dim == 0) return 0;
    size_t guard;  // the sizes below are sums of a few such products: refuse shapes whose products wrap
    if (!checked_mul(rows, in_dim, &guard) || !checked_mul(guard, 16, &guard) || !checked_mul(rows, out_dim, &guard) ||
        !checked_mul(guard, 256, &guard))
        return 0;
    const size_t base = workspace_view(0, rows, in_dim).bytes;
    // nine rows and more (the MFMA GEMM): room for the partial sums of K shares when the grid is small
    const size_t partial = rows >= 9 ? gemm_i8_partial_bytes(rows, in_dim, out_dim) : 0;
    const size_t gemm_bytes = partial != 0 ? (base + 255) / 256 * 256 + partial : base;
    // small batches on a long K (also slices of eight rows of a forced plan): the K slices' sums, for a pair of matrices
    const size_t batch_bytes = gemv_batch_partial_bytes(rows < 8 ? rows : 8, in_dim, out_dim, true);
    // up to 128 rows: X in MFMA operand order and the partial sums of K shares of the single-shot MFMA kernel
    const size_t mfma_bytes = rows <= 128 ? batch_mfma_workspace_bytes(tensor_type, rows, in_dim, out_dim) : 0;
    size_t need = gemm_bytes > batch_bytes ? gemm_bytes : batch_bytes;
    return need > mfma_bytes ? need : mfma_bytes;
}

afhip_status afhip_launch_linear_f32(void* stream, int tensor_type, int layout, afhip_buffer dst, afhip_buffer input,
                                     afhip_buffer weight, size_t rows, size_t in_dim, size_t out_dim,
                                     afhip_buffer workspace, int dispatch) {
    return linear_impl(stream, tensor_type, layout, dst, input, weight, rows, in_dim, out_dim, workspace, dispatch,
                       afhip_buffer{0, 0}, nullptr);
}

afhip_status afhip_static_scratch_init(void) {
    unsigned char* p = nullptr;
    return static_scratch_address(&p);
}

afhip_status afhip_launch_linear_f32_static(void* stream, int tensor_type, int layout, afhip_buffer dst, afhip_buffer input,
                                            afhip_buffer weight, size_t rows, size_t in_dim, size_t out_dim, int dispatch) {
    // what the call would ask a caller to lend: beyond the array is refused, not truncated
    if (afhip_linear_workspace_bytes(tensor_type, rows, in_dim, out_dim) > AFHIP_STATIC_SCRATCH_BYTES)
        return AFHIP_ERR_OP_UNSUPPORTED;
    unsigned char* p = nullptr;
    if (afhip_status s = static_scratch_address(&p); s != AFHIP_OK) return s;
    const afhip_buffer workspace{reinterpret_cast<uint64_t>(p), AFHIP_STATIC_SCRATCH_BYTES};
    return linear_impl(stream, tensor_type, layout, dst, input, weight, rows, in_dim, out_dim, workspace, dispatch,
                       afhip_buffer{0, 0}, nullptr);
}

afhip_status afhip_launch_linear_pair_f32(void* stream, int tensor_type, int layout, afhip_buffer dst_a,
                                          afhip_buffer dst_b, afhip_buffer input, afhip_buffer weight_a,
                                          afhip_buffer weight_b, size_t rows, size_t in_dim, size_t out_dim,
                                          afhip_buffer workspace, int dispatch) {
    if (weight_b.ptr == 0 || (dst_b.ptr == 0 && rows != 0 && out_dim != 0)) return AFHIP_ERR_INVALID_STATE;
    return linear_impl(stream, tensor_type, layout, dst_a, input, weight_a, rows, in_dim, out_dim, workspace, dispatch,
                       afhip_buffer{0, 0}, nullptr, dst_b, weight_b);
}

afhip_status afhip_launch_linear_bias_f32(void* stream, int tensor_type, int layout, afhip_buffer dst, afhip_buffer input,
                                          afhip_buffer weight, afhip_buffer bias, size_t rows, size_t in_dim,
                                          size_t out_dim, afhip_buffer workspace, int dispatch) {
    if (bias.ptr == 0 && out_dim != 0) return AFHIP_ERR_INVALID_STATE;
    LinearExtras extras;
    extras.bias = bias;
    return linear_impl(stream, tensor_type, layout, dst, input, weight, rows, in_dim, out_dim, workspace, dispatch,
                       afhip_buffer{0, 0}, nullptr, afhip_buffer{0, 0}, afhip_buffer{0, 0}, extras);
}

afhip_status afhip_launch_linear_epilogue_f32(void* stream, int tensor_type, int layout, afhip_buffer dst,
                                              afhip_buffer input, afhip_buffer weight, afhip_buffer bias,
                                              afhip_buffer residual, int activation, size_t rows, size_t in_dim,
                                              size_t out_dim, afhip_buffer workspace, int dispatch) {
    LinearExtras extras;
    extras.bias = bias;
    extras.residual = residual;
    extras.activation = activation;
    return linear_impl(stream, tensor_type, layout, dst, input, weight, rows, in_dim, out_dim, workspace, dispatch,
                       afhip_buffer{0, 0}, nullptr, afhip_buffer{0, 0}, afhip_buffer{0, 0}, extras);
}

afhip_status afhip_launch_linear_pair_bias_f32(void* stream, int tensor_type, int layout, afhip_buffer dst_a,
                                               afhip_buffer dst_b, afhip_buffer input, afhip_buffer weight_a,
                                               afhip_buffer bias_a, afhip_buffer weight_b, afhip_buffer bias_b,
                                               size_t rows, size_t in_dim, size_t out_dim, afhip_buffer workspace,
                                               int dispatch) {
    if (weight_b.ptr == 0 || (dst_b.ptr == 0 && rows != 0 && out_dim != 0)) return AFHIP_ERR_INVALID_STATE;
    if ((bias_a.ptr == 0 || bias_b.ptr == 0) && out_dim != 0) return AFHIP_ERR_INVALID_STATE;
    LinearExtras extras;
    extras.bias = bias_a;
    extras.bias_b = bias_b;
    return linear_impl(stream, tensor_type, layout, dst_a, input, weight_a, rows, in_dim, out_dim, workspace, dispatch,
                       afhip_buffer{0, 0}, nullptr, dst_b, weight_b, extras);
}

afhip_status afhip_launch_linear_q8_0_f32(void* stream, afhip_buffer dst, afhip_buffer input, afhip_buffer weight_raw,
                                          size_t rows, size_t in_dim, size_t out_dim, afhip_buffer workspace) {
    return linear_impl(stream, AFHIP_TYPE_Q8_0, AFHIP_LAYOUT_RAW, dst, input, weight_raw, rows, in_dim, out_dim,
                       workspace, -1, afhip_buffer{0, 0}, nullptr);
}

afhip_status afhip_launch_linear_q4_0_f32(void* stream, afhip_buffer dst, afhip_buffer input, afhip_buffer weight_raw,
                                          size_t rows, size_t in_dim, size_t out_dim, afhip_buffer workspace) {
    return linear_impl(stream, AFHIP_TYPE_Q4_0, AFHIP_LAYOUT_RAW, dst, input, weight_raw, rows, in_dim, out_dim,
                       workspace, -1, afhip_buffer{0, 0}, nullptr);
}

afhip_status afhip_launch_block_dots(void* stream, int tensor_type, int layout, afhip_buffer dots, afhip_buffer input,
                                     afhip_buffer weight, size_t rows, size_t in_dim, size_t out_dim,
                                     afhip_buffer workspace, int dispatch) {
    if (dots.ptr == 0) return AFHIP_ERR_INVALID_STATE;
    return linear_impl(stream, tensor_type, layout, afhip_buffer{0, 0}, input, weight, rows, in_dim, out_dim, workspace,
                       dispatch, dots, nullptr);
}

size_t afhip_prepared_weight_bytes(int tensor_type, size_t out_dim, size_t in_dim) {
    size_t blocks, bytes;
    if (tensor_type == AFHIP_TYPE_Q4_K) {
        if (in_dim % 256 != 0 || !checked_mul(out_dim + 31, in_dim / 256, &blocks) || !checked_mul(blocks, 144, &bytes)) return 0;
        return q4k_tiled_bytes(out_dim, in_dim);
    }
    const size_t bb = block_bytes(tensor_type);
    if (bb == 0 || in_dim % 32 != 0 || !checked_mul(out_dim, in_dim / 32, &blocks) || !checked_mul(blocks, bb, &bytes)) return 0;
    // the scales once more in wavefront-tile order (padded to whole tiles): at most the raw size again
    size_t padded;
    if (!checked_mul(out_dim + 3, in_dim / 32 + kTileSliceBlocks, &padded) || !checked_mul(padded, 8, &padded)) return 0;
    return prepared_bytes_q(tensor_type, out_dim, in_dim / 32);
}

size_t afhip_weight_layout_bytes(int tensor_type, int layout, size_t out_dim, size_t in_dim) {
    size_t blocks, bytes;
    if (layout == AFHIP_LAYOUT_PREPARED) return afhip_prepared_weight_bytes(tensor_type, out_dim, in_dim);
    if (layout != AFHIP_LAYOUT_RAW) return 0;
    const size_t bb = tensor_type == AFHIP_TYPE_Q4_K ? 144 : block_bytes(tensor_type);
    const size_t values = tensor_type == AFHIP_TYPE_Q4_K ? 256 : 32;
    if (bb == 0 || in_dim % values != 0 || !checked_mul(out_dim, in_dim / values, &blocks) || !checked_mul(blocks, bb, &bytes))
        return 0;
    return bytes;
}

afhip_status afhip_launch_prepare_weight(void* stream, int tensor_type, afhip_buffer dst, afhip_buffer src,
                                         size_t out_dim, size_t in_dim) {
    if (tensor_type == AFHIP_TYPE_Q4_K) {  // tile-major layout for the MFMA kernel
        if (in_dim == 0 || in_dim % 256 != 0) return AFHIP_ERR_INVALID_STATE;
        size_t raw_blocks, raw_bytes;
        if (!checked_mul(out_dim, in_dim / 256, &raw_blocks) || !checked_mul(raw_blocks, 144, &raw_bytes))
            return AFHIP_ERR_INVALID_STATE;
        const size_t tiled_bytes = afhip_prepared_weight_bytes(tensor_type, out_dim, in_dim);
        if (out_dim != 0 && tiled_bytes == 0) return AFHIP_ERR_INVALID_STATE;
        if (raw_bytes > src.len || tiled_bytes > dst.len) return AFHIP_ERR_INVALID_STATE;
        if (raw_blocks == 0) return AFHIP_OK;
        if (out_dim > 0x7fffffff || in_dim > 0x7fffffff || dst.ptr == 0 || src.ptr == 0 || dst.ptr % 16 != 0 ||
            src.ptr % 16 != 0)
            return AFHIP_ERR_INVALID_STATE;
        hipError_t e = launch_q4k_tile_repack(static_cast<hipStream_t>(stream), reinterpret_cast<uint8_t*>(dst.ptr),
                                              reinterpret_cast<const uint8_t*>(src.ptr), static_cast<int>(out_dim),
                                              static_cast<int>(in_dim));
        return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
    }
    const size_t bb = block_bytes(tensor_type);
    if (bb == 0) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    if (in_dim == 0 || in_dim % 32 != 0) return AFHIP_ERR_INVALID_STATE;
    size_t blocks, bytes;
    if (!checked_mul(out_dim, in_dim / 32, &blocks) || !checked_mul(blocks, bb, &bytes)) return AFHIP_ERR_INVALID_STATE;
    const size_t prepared = afhip_prepared_weight_bytes(tensor_type, out_dim, in_dim);
    if (bytes > src.len || (blocks != 0 && prepared == 0) || prepared > dst.len) return AFHIP_ERR_INVALID_STATE;
    if (blocks == 0) return AFHIP_OK;
    if (dst.ptr == 0 || src.ptr == 0 || dst.ptr % 16 != 0 || src.ptr % 2 != 0) return AFHIP_ERR_INVALID_STATE;
    hipError_t e = launch_prepare_weight(static_cast<hipStream_t>(stream), tensor_type,
                                         reinterpret_cast<uint8_t*>(dst.ptr), reinterpret_cast<const uint8_t*>(src.ptr),
                                         out_dim, in_dim / 32);
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_quantize_activations(void* stream, afhip_buffer input, size_t rows, size_t in_dim,
                                               afhip_buffer q, afhip_buffer scales, afhip_buffer sums) {
    if (in_dim == 0 || in_dim % 32 != 0) return AFHIP_ERR_INVALID_STATE;
    size_t count, bytes;
    if (!checked_mul(rows, in_dim, &count) || !checked_mul(count, 4, &bytes)) return AFHIP_ERR_INVALID_STATE;
    const size_t nb = count / 32;  // (count * 4 did not overflow: nb * 4 cannot)
    if (bytes > input.len || count > q.len || nb * 4 > scales.len) return AFHIP_ERR_INVALID_STATE;
    if (sums.ptr != 0 && nb * 4 > sums.len) return AFHIP_ERR_INVALID_STATE;
    if (count == 0) return AFHIP_OK;
    if (rows > 0x7fffffff || in_dim > 0x7fffffff || input.ptr == 0 || q.ptr == 0 || scales.ptr == 0 ||
        input.ptr % 16 != 0 || q.ptr % 4 != 0)
        return AFHIP_ERR_INVALID_STATE;
    hipError_t e = launch_quantize_activations(static_cast<hipStream_t>(stream),
                                               reinterpret_cast<const float*>(input.ptr), static_cast<int>(rows),
                                               static_cast<int>(in_dim), reinterpret_cast<int8_t*>(q.ptr),
                                               reinterpret_cast<float*>(scales.ptr), reinterpret_cast<int*>(sums.ptr));
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_stream_read(void* stream, afhip_buffer src, afhip_buffer sink) {
    if (src.len / 16 > 0xffffffffull * 256) return AFHIP_ERR_INVALID_STATE;
    if (src.len < 16) return AFHIP_OK;
    if (src.ptr == 0 || src.ptr % 16 != 0 || sink.ptr == 0 || sink.len < 4) return AFHIP_ERR_INVALID_STATE;
    hipError_t e = launch_stream_read(static_cast<hipStream_t>(stream), reinterpret_cast<const uint8_t*>(src.ptr),
                                      reinterpret_cast<uint32_t*>(sink.ptr), src.len);
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_stream_read_shaped(void* stream, afhip_buffer src, afhip_buffer sink, int threads, int loads_per_lane,
                                            int nontemporal) {
    if (src.len < 16) return AFHIP_OK;
    if (src.ptr == 0 || src.ptr % 16 != 0 || sink.ptr == 0 || sink.len < 4) return AFHIP_ERR_INVALID_STATE;
    hipError_t e = launch_stream_read_shaped(static_cast<hipStream_t>(stream), reinterpret_cast<const uint8_t*>(src.ptr),
                                             reinterpret_cast<uint32_t*>(sink.ptr), src.len, threads, loads_per_lane, nontemporal);
    if (e == hipErrorInvalidValue) return AFHIP_ERR_INVALID_ARGUMENT;
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_stream_copy(void* stream, afhip_buffer src, afhip_buffer dst) {
    if (src.len / 16 > 0xffffffffull * 256 || dst.len < src.len / 16 * 16) return AFHIP_ERR_INVALID_STATE;
    if (src.len < 16) return AFHIP_OK;
    if (src.ptr == 0 || src.ptr % 16 != 0 || dst.ptr == 0 || dst.ptr % 16 != 0) return AFHIP_ERR_INVALID_STATE;
    hipError_t e = launch_stream_copy(static_cast<hipStream_t>(stream), reinterpret_cast<uint8_t*>(dst.ptr),
                                      reinterpret_cast<const uint8_t*>(src.ptr), src.len);
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_gemv_probe_rows(void* stream, int probe, size_t rows, afhip_buffer dst, afhip_buffer input,
                                          afhip_buffer weight, size_t in_dim, size_t out_dim) {
    if (probe < 0 || probe > 7 || (rows != 1 && rows != 2 && rows != 4)) return AFHIP_ERR_INVALID_ARGUMENT;
    if (in_dim == 0 || in_dim % 32 != 0 || in_dim > 4096 || out_dim == 0 || out_dim > 0x7fffffff) return AFHIP_ERR_INVALID_STATE;
    const size_t need = afhip_prepared_weight_bytes(AFHIP_TYPE_Q4_0, out_dim, in_dim);
    if (need == 0 || weight.len < need || input.len < rows * in_dim * 4 || dst.len < rows * out_dim * 4) return AFHIP_ERR_INVALID_STATE;
    if (dst.ptr == 0 || input.ptr == 0 || weight.ptr == 0 || dst.ptr % 4 != 0 || input.ptr % 16 != 0 || weight.ptr % 16 != 0)
        return AFHIP_ERR_INVALID_STATE;
    hipError_t e = launch_gemv_probe(static_cast<hipStream_t>(stream), probe, static_cast<int>(rows),
                                     reinterpret_cast<float*>(dst.ptr), reinterpret_cast<const float*>(input.ptr),
                                     reinterpret_cast<const uint8_t*>(weight.ptr), static_cast<int>(in_dim),
                                     static_cast<int>(out_dim));
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_gemv_timeline(void* stream, size_t rows, afhip_buffer stamps, afhip_buffer input, afhip_buffer weight,
                                        size_t in_dim, size_t out_dim, size_t* workgroups, size_t* wavefronts_per_workgroup) {
    if (rows != 1 && rows != 2 && rows != 4) return AFHIP_ERR_INVALID_ARGUMENT;
    // (one row also on a K of several slices, as the decode kernel takes it)
    if (in_dim == 0 || in_dim % 32 != 0 || in_dim > (rows == 1 ? static_cast<size_t>(gemv_fused_max_in_dim()) : 4096) || out_dim == 0 ||
        out_dim > 0x7fffffff)
        return AFHIP_ERR_INVALID_STATE;
    const size_t need = afhip_prepared_weight_bytes(AFHIP_TYPE_Q4_0, out_dim, in_dim);
    if (need == 0 || weight.len < need || input.len < rows * in_dim * 4) return AFHIP_ERR_INVALID_STATE;
    if (stamps.ptr == 0 || stamps.ptr % 4 != 0 || input.ptr == 0 || weight.ptr == 0 || input.ptr % 16 != 0 || weight.ptr % 16 != 0)
        return AFHIP_ERR_INVALID_STATE;
    int grid = 0, waves = 0;
    hipError_t e = launch_gemv_probe(static_cast<hipStream_t>(stream), 8, static_cast<int>(rows), nullptr,
                                     reinterpret_cast<const float*>(input.ptr), reinterpret_cast<const uint8_t*>(weight.ptr),
                                     static_cast<int>(in_dim), static_cast<int>(out_dim), reinterpret_cast<uint32_t*>(stamps.ptr),
                                     stamps.len, &grid, &waves);
    if (workgroups) *workgroups = static_cast<size_t>(grid);
    if (wavefronts_per_workgroup) *wavefronts_per_workgroup = static_cast<size_t>(waves);
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_rows8_timeline(void* stream, size_t rows, afhip_buffer stamps, afhip_buffer input, afhip_buffer weight,
                                         size_t in_dim, size_t out_dim, afhip_buffer workspace, size_t* workgroups,
                                         size_t* columns_per_workgroup) {
    if (rows < 1 || rows > 8) return AFHIP_ERR_INVALID_ARGUMENT;
    if (in_dim == 0 || in_dim % 256 != 0 || in_dim > 4096 || out_dim == 0 || out_dim > 0x7fffffff) return AFHIP_ERR_INVALID_STATE;
    const size_t need = afhip_prepared_weight_bytes(AFHIP_TYPE_Q4_0, out_dim, in_dim);
    const size_t ws = batch_mfma_workspace_bytes(AFHIP_TYPE_Q4_0, rows, in_dim, out_dim);
    if (need == 0 || weight.len < need || input.len < rows * in_dim * 4 || ws == 0 || workspace.len < ws) return AFHIP_ERR_INVALID_STATE;
    if (stamps.ptr == 0 || stamps.ptr % 4 != 0 || input.ptr == 0 || weight.ptr == 0 || workspace.ptr == 0 || input.ptr % 16 != 0 ||
        weight.ptr % 16 != 0 || workspace.ptr % 16 != 0)
        return AFHIP_ERR_INVALID_STATE;
    int groups = 0, cols = 0;
    hipError_t e = launch_batch8_timeline(static_cast<hipStream_t>(stream), reinterpret_cast<uint32_t*>(stamps.ptr), stamps.len,
                                          reinterpret_cast<const float*>(input.ptr), reinterpret_cast<const uint8_t*>(weight.ptr),
                                          static_cast<int>(rows), static_cast<int>(in_dim), static_cast<int>(out_dim),
                                          reinterpret_cast<uint8_t*>(workspace.ptr), &groups, &cols);
    if (workgroups) *workgroups = static_cast<size_t>(groups);
    if (columns_per_workgroup) *columns_per_workgroup = static_cast<size_t>(cols);
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_gemv_probe(void* stream, int probe, afhip_buffer dst, afhip_buffer input, afhip_buffer weight,
                                     size_t in_dim, size_t out_dim) {
    return afhip_launch_gemv_probe_rows(stream, probe, 1, dst, input, weight, in_dim, out_dim);
}

afhip_status afhip_tune_batch32_max_workgroups(long bound) {
    set_batch32_max_workgroups(bound);
    return AFHIP_OK;
}

afhip_status afhip_launch_gemm_stamps(void* stream, afhip_buffer stamps, afhip_buffer q, afhip_buffer scales,
                                      afhip_buffer weight_prepared, size_t rows, size_t in_dim, size_t out_dim) {
    if (rows == 0 || rows > 0x7fffffff || in_dim == 0 || in_dim % 32 != 0 || in_dim > 0x7fffffff || out_dim == 0 ||
        out_dim > 0x7fffffff)
        return AFHIP_ERR_INVALID_STATE;
    const size_t need = afhip_prepared_weight_bytes(AFHIP_TYPE_Q8_0, out_dim, in_dim);
    if (need == 0 || weight_prepared.len < need || q.len < rows * in_dim || scales.len < rows * (in_dim / 32) * 4 ||
        stamps.len < rows * out_dim * 4)
        return AFHIP_ERR_INVALID_STATE;
    if (stamps.ptr == 0 || q.ptr == 0 || scales.ptr == 0 || weight_prepared.ptr == 0 || stamps.ptr % 4 != 0 ||
        q.ptr % 16 != 0 || scales.ptr % 4 != 0 || weight_prepared.ptr % 16 != 0)
        return AFHIP_ERR_INVALID_STATE;
    hipError_t e = launch_gemm_i8_stamps(static_cast<hipStream_t>(stream), reinterpret_cast<float*>(stamps.ptr),
                                         reinterpret_cast<const int8_t*>(q.ptr), reinterpret_cast<const float*>(scales.ptr),
                                         reinterpret_cast<const uint8_t*>(weight_prepared.ptr), static_cast<int>(rows),
                                         static_cast<int>(in_dim), static_cast<int>(out_dim));
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_rate_probe(void* stream, int pattern, int wavefronts_per_simd, int iterations, afhip_buffer sink,
                                     afhip_buffer stamps) {
    if (pattern < 0 || pattern > 23 || (wavefronts_per_simd != 1 && wavefronts_per_simd != 2 && wavefronts_per_simd != 4) ||
        iterations < 1 || iterations > (1 << 20))
        return AFHIP_ERR_INVALID_ARGUMENT;
    if (sink.ptr == 0 || sink.ptr % 16 != 0 || sink.len < 65536 * 4 + (2u << 20) + 8192) return AFHIP_ERR_INVALID_STATE;
    if (stamps.ptr == 0 || stamps.ptr % 4 != 0 || stamps.len < afhip_rate_probe_wavefronts(wavefronts_per_simd) * 16)
        return AFHIP_ERR_INVALID_STATE;
    hipError_t e = launch_rate_probe(static_cast<hipStream_t>(stream), pattern, wavefronts_per_simd, iterations,
                                     reinterpret_cast<int*>(sink.ptr), reinterpret_cast<uint32_t*>(stamps.ptr));
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

size_t afhip_rate_probe_wavefronts(int wavefronts_per_simd) {
    return wavefronts_per_simd < 1 ? 0 : static_cast<size_t>(rate_probe_wavefronts(wavefronts_per_simd));
}

afhip_status afhip_launch_decode_fp16(void* stream, afhip_buffer dst, afhip_buffer src, size_t n) {
    size_t dst_bytes, src_bytes;
    if (!checked_mul(n, 4, &dst_bytes) || !checked_mul(n, 2, &src_bytes) || dst_bytes > dst.len || src_bytes > src.len)
        return AFHIP_ERR_INVALID_STATE;
    if (n == 0) return AFHIP_OK;
    if (dst.ptr == 0 || src.ptr == 0) return AFHIP_ERR_INVALID_STATE;
    hipError_t e = launch_decode_fp16(static_cast<hipStream_t>(stream), reinterpret_cast<float*>(dst.ptr),
                                      reinterpret_cast<const uint16_t*>(src.ptr), n);
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

// ---- lm_head: argmax over the last row

size_t afhip_argmax_workspace_bytes(size_t dim) { return argmax_keys_bytes(dim); }

afhip_status afhip_launch_argmax_last_row_f32(void* stream, afhip_buffer token_u32, afhip_buffer token_f32,
                                              afhip_buffer input, size_t rows, size_t dim, afhip_buffer workspace) {
    return argmax_last_row_impl(stream, token_u32, token_f32, input, rows, dim, workspace);
}

size_t afhip_linear_argmax_workspace_bytes(int tensor_type, size_t in_dim, size_t out_dim) {
    if (tensor_type == AFHIP_TYPE_Q4_K)
        return in_dim == 0 || in_dim % 256 != 0 || out_dim == 0
                   ? 0
                   : argmax_logits_bytes(out_dim) + (argmax_linear_bytes(tensor_type, in_dim, out_dim) + 255) / 256 * 256 +
                         argmax_keys_bytes(out_dim);
    if (block_bytes(tensor_type) == 0 || in_dim % 32 != 0 || in_dim == 0 || out_dim == 0) return 0;
    return argmax_logits_bytes(out_dim) + (workspace_view(0, 1, in_dim).bytes + 255) / 256 * 256 + argmax_keys_bytes(out_dim);
}

afhip_status afhip_launch_linear_argmax_last_row_f32(void* stream, int tensor_type, int layout, afhip_buffer token_u32,
                                                     afhip_buffer token_f32, afhip_buffer input, afhip_buffer weight,
                                                     size_t rows, size_t in_dim, size_t out_dim,
                                                     afhip_buffer workspace) {
    return linear_argmax_impl(stream, tensor_type, layout, token_u32, token_f32, input, weight, rows, in_dim, out_dim,
                              workspace, nullptr);
}

// ---- row operators: get_rows / cpy_q_to_f32 / cpy_f32_to_q / set_rows

static afhip_status dequantize_rows(void* stream, int tensor_type, int layout, afhip_buffer dst, afhip_buffer weight,
                                    afhip_buffer ids, bool gather, size_t rows, size_t dim, size_t weight_rows) {
    const bool dense = tensor_type == AFHIP_TYPE_F32;
    const bool q4k = tensor_type == AFHIP_TYPE_Q4_K;
    const size_t bb = q4k ? 144 : block_bytes(tensor_type);
    const size_t block_values = q4k ? 256 : 32;
    if (!dense && bb == 0) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    if (layout != AFHIP_LAYOUT_RAW && layout != AFHIP_LAYOUT_PREPARED) return AFHIP_ERR_INVALID_ARGUMENT;
    if (dim == 0 || (!dense && dim % block_values != 0) || (dense && !gather)) return AFHIP_ERR_INVALID_STATE;
    size_t out_count, out_bytes, w_count, w_bytes, id_bytes;
    if (!checked_mul(rows, dim, &out_count) || !checked_mul(out_count, 4, &out_bytes) ||
        !checked_mul(weight_rows, dim, &w_count) || !checked_mul(rows, 8, &id_bytes))
        return AFHIP_ERR_INVALID_STATE;
    if (dense) {
        if (!checked_mul(w_count, 4, &w_bytes)) return AFHIP_ERR_INVALID_STATE;
    } else if (!checked_mul(w_count / block_values, bb, &w_bytes)) {
        return AFHIP_ERR_INVALID_STATE;
    }
    const bool q4k_tiled = q4k && layout == AFHIP_LAYOUT_PREPARED;
    if (q4k_tiled) {
        size_t padded;
        if (!checked_mul(weight_rows + 31, dim / block_values, &padded) || !checked_mul(padded, bb, &padded))
            return AFHIP_ERR_INVALID_STATE;
        w_bytes = q4k_tiled_bytes(weight_rows, dim);
    }
    if (out_bytes > dst.len || w_bytes > weight.len || (gather && id_bytes > ids.len)) return AFHIP_ERR_INVALID_STATE;
    if (out_count == 0) return AFHIP_OK;
    if (dim > 0x7fffffff || dst.ptr == 0 || weight.ptr == 0 || dst.ptr % 16 != 0 ||
        weight.ptr % (dense ? 4 : (q4k || layout == AFHIP_LAYOUT_PREPARED ? 16 : 2)) != 0 ||
        (gather && (ids.ptr == 0 || ids.ptr % 8 != 0)))
        return AFHIP_ERR_INVALID_STATE;
    if (q4k) {
        hipError_t e = (q4k_tiled ? launch_dequantize_q4k_tiled_rows : launch_dequantize_q4k_rows)(
            static_cast<hipStream_t>(stream), reinterpret_cast<float*>(dst.ptr), reinterpret_cast<const uint8_t*>(weight.ptr),
            gather ? reinterpret_cast<const long long*>(ids.ptr) : nullptr, rows, static_cast<int>(dim), weight_rows);
        return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
    }
    hipError_t e = launch_dequantize_rows(static_cast<hipStream_t>(stream), tensor_type, layout,
                                          reinterpret_cast<float*>(dst.ptr), reinterpret_cast<const uint8_t*>(weight.ptr),
                                          gather ? reinterpret_cast<const long long*>(ids.ptr) : nullptr, rows,
                                          static_cast<int>(dim), weight_rows);
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

afhip_status afhip_launch_embedding_lookup_f32(void* stream, int tensor_type, int layout, afhip_buffer dst,
                                               afhip_buffer weight, afhip_buffer ids_i64, size_t total, size_t dim,
                                               size_t vocab) {
    return dequantize_rows(stream, tensor_type, layout, dst, weight, ids_i64, true, total, dim, vocab);
}

afhip_status afhip_launch_dequantize_f32(void* stream, int tensor_type, int layout, afhip_buffer dst,
                                         afhip_buffer weight, size_t rows, size_t dim) {
    return dequantize_rows(stream, tensor_type, layout, dst, weight, afhip_buffer{0, 0}, false, rows, dim, rows);
}

afhip_status afhip_launch_quantize_rows(void* stream, int tensor_type, afhip_buffer dst_raw, afhip_buffer input,
                                        afhip_buffer row_ids_i64, size_t rows, size_t dim, size_t dst_rows) {
    const bool q4k = tensor_type == AFHIP_TYPE_Q4_K;
    const size_t bb = q4k ? 144 : block_bytes(tensor_type);
    if (bb == 0) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    const size_t block_values = q4k ? 256 : 32;
    if (dim == 0 || dim % block_values != 0) return AFHIP_ERR_INVALID_STATE;
    const bool scatter = row_ids_i64.ptr != 0;
    if (!scatter && dst_rows != rows) return AFHIP_ERR_INVALID_STATE;
    size_t in_count, in_bytes, d_count, d_bytes, id_bytes;
    if (!checked_mul(rows, dim, &in_count) || !checked_mul(in_count, 4, &in_bytes) ||
        !checked_mul(dst_rows, dim, &d_count) || !checked_mul(d_count / block_values, bb, &d_bytes) ||
        !checked_mul(rows, 8, &id_bytes))
        return AFHIP_ERR_INVALID_STATE;
    if (in_bytes > input.len || d_bytes > dst_raw.len || (scatter && id_bytes > row_ids_i64.len)) return AFHIP_ERR_INVALID_STATE;
    if (in_count == 0) return AFHIP_OK;
    if (dim > 0x7fffffff || input.ptr == 0 || input.ptr % 16 != 0 || dst_raw.ptr == 0 || dst_raw.ptr % (q4k ? 16 : 2) != 0 ||
        (scatter && row_ids_i64.ptr % 8 != 0))
        return AFHIP_ERR_INVALID_STATE;
    if (q4k) {
        hipError_t e = launch_quantize_q4k_rows(static_cast<hipStream_t>(stream), reinterpret_cast<uint8_t*>(dst_raw.ptr),
                                                reinterpret_cast<const float*>(input.ptr),
                                                scatter ? reinterpret_cast<const long long*>(row_ids_i64.ptr) : nullptr, rows,
                                                static_cast<int>(dim), dst_rows);
        return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
    }
    hipError_t e = launch_quantize_rows(static_cast<hipStream_t>(stream), tensor_type,
                                        reinterpret_cast<uint8_t*>(dst_raw.ptr), reinterpret_cast<const float*>(input.ptr),
                                        scatter ? reinterpret_cast<const long long*>(row_ids_i64.ptr) : nullptr, rows,
                                        static_cast<int>(dim), dst_rows);
    return e == hipSuccess ? AFHIP_OK : static_cast<afhip_status>(e);
}

}  // extern "C"
