// C ABI, part 2: the backend object.  Mirrors ops/cuda/cuda_compute.zig
// (CudaCompute, CudaTensor and the ComputeBackend vtable entries on the
// quantized-linear path), ops/cuda/context.zig (one device, one stream),
// ops/cuda/buffer.zig (DeviceBuffer) and ops/cuda/scratch.zig (grow-only scratch).
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstring>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

#include "antfly_hip_qmatmul.h"
#include "api_internal.h"

using namespace afhip;

struct afhip_tensor {  // CudaTensor, cuda_compute.zig:29-38
    afhip_buffer buffer{0, 0};
    int dtype = AFHIP_DTYPE_F32;
    std::vector<int64_t> shape;
    size_t elem_count = 0;
    int quant_type = -1;  // GGUF tensor type, -1 = not quantized
    int layout = AFHIP_LAYOUT_RAW;
    bool owns_buffer = true;
    bool owned_by_tensor = true;
};

struct afhip_compute {
    int device = 0;
    hipStream_t stream = nullptr;
    std::unordered_map<std::string, afhip_tensor> resident_weights;
    std::vector<afhip_buffer> temp_buffers;  // freed buffers, best-fit reuse (cuda_compute.zig:193-223)
    afhip_buffer scratch{0, 0};              // DeviceScratch, scratch.zig
    afhip_debug_stats stats{};
    LaunchCounters counters;
    hipEvent_t phase_events[3] = {nullptr, nullptr, nullptr};  // created by afhip_compute_set_phase_timing
    bool phase_timing = false;
    bool q4k_f32_activations = false;  // afhip_compute_set_q4k_f32_activations
};

namespace {

constexpr size_t kMaxTempBuffers = 256;

afhip_status from_hip(hipError_t e) {
    if (e == hipSuccess) return AFHIP_OK;
    if (e == hipErrorOutOfMemory) return AFHIP_ERR_OUT_OF_MEMORY;
    return static_cast<afhip_status>(e);
}

afhip_status make_current(afhip_compute* self) { return from_hip(hipSetDevice(self->device)); }  // context.zig:100

afhip_status alloc_device_buffer(afhip_compute* self, size_t len, afhip_buffer* out) {
    *out = afhip_buffer{0, 0};
    if (len == 0) return AFHIP_OK;
    size_t best = SIZE_MAX, best_len = SIZE_MAX;
    for (size_t i = 0; i < self->temp_buffers.size(); ++i) {
        const afhip_buffer& b = self->temp_buffers[i];
        if (b.len >= len && b.len < best_len) {
            best = i;
            best_len = b.len;
        }
    }
    if (best != SIZE_MAX) {
        *out = self->temp_buffers[best];
        self->temp_buffers[best] = self->temp_buffers.back();  // swapRemove
        self->temp_buffers.pop_back();
        return AFHIP_OK;
    }
    void* p = nullptr;
    afhip_status s = from_hip(hipMalloc(&p, len));
    if (s != AFHIP_OK) return s;
    self->stats.device_allocs++;
    *out = afhip_buffer{reinterpret_cast<uint64_t>(p), len};
    return AFHIP_OK;
}

void free_device_buffer(afhip_buffer* b) {
    if (b->ptr != 0) (void)hipFree(reinterpret_cast<void*>(b->ptr));
    *b = afhip_buffer{0, 0};
}

void release_device_buffer(afhip_compute* self, afhip_buffer* b) {
    if (b->ptr == 0) return;
    if (self->temp_buffers.size() < kMaxTempBuffers) {
        self->temp_buffers.push_back(*b);
        *b = afhip_buffer{0, 0};
        return;
    }
    // hipFree synchronizes with outstanding work on the device
    free_device_buffer(b);
}

afhip_status acquire_scratch(afhip_compute* self, size_t len, afhip_buffer* out) {  // DeviceScratch.acquire
    *out = afhip_buffer{0, 0};
    if (len == 0) return AFHIP_OK;
    if (self->scratch.len < len) {
        if (self->scratch.ptr != 0) {
            afhip_status s = from_hip(hipStreamSynchronize(self->stream));
            if (s != AFHIP_OK) return s;
            free_device_buffer(&self->scratch);
        }
        void* p = nullptr;
        afhip_status s = from_hip(hipMalloc(&p, len));
        if (s != AFHIP_OK) return s;
        self->stats.device_allocs++;
        self->scratch = afhip_buffer{reinterpret_cast<uint64_t>(p), len};
    }
    *out = afhip_buffer{self->scratch.ptr, len};
    return AFHIP_OK;
}

afhip_status copy_from_host(afhip_compute* self, afhip_buffer dst, const void* src, size_t len) {
    if (len > dst.len) return AFHIP_ERR_INVALID_STATE;
    if (len == 0) return AFHIP_OK;
    self->stats.h2d_bytes += len;
    return from_hip(hipMemcpyHtoDAsync(reinterpret_cast<hipDeviceptr_t>(dst.ptr), const_cast<void*>(src), len,
                                       self->stream));
}

afhip_status copy_to_host(afhip_compute* self, void* dst, afhip_buffer src, size_t len) {
    if (len > src.len) return AFHIP_ERR_INVALID_STATE;
    if (len == 0) return AFHIP_OK;
    self->stats.d2h_bytes += len;
    return from_hip(hipMemcpyDtoHAsync(dst, reinterpret_cast<hipDeviceptr_t>(src.ptr), len, self->stream));
}

bool element_count(const int64_t* shape, size_t n, size_t* out) {
    size_t count = 1;
    for (size_t i = 0; i < n; ++i) {
        if (shape[i] < 0) return false;
        if (!checked_mul(count, static_cast<size_t>(shape[i]), &count)) return false;
    }
    *out = count;
    return true;
}

void free_tensor_storage(afhip_compute* self, afhip_tensor* t) {
    if (t->owns_buffer) release_device_buffer(self, &t->buffer);
}

bool is_f32(const afhip_tensor* t) { return t->dtype == AFHIP_DTYPE_F32 && t->quant_type < 0; }  // ensureF32

afhip_status make_f32_result(afhip_compute* self, afhip_buffer device, size_t rows, size_t out_dim, size_t out_count,
                             afhip_tensor** out) {
    afhip_tensor* t = new (std::nothrow) afhip_tensor();
    if (!t) {
        release_device_buffer(self, &device);
        return AFHIP_ERR_OUT_OF_MEMORY;
    }
    t->buffer = device;
    t->dtype = AFHIP_DTYPE_F32;
    t->shape = {static_cast<int64_t>(rows), static_cast<int64_t>(out_dim)};
    t->elem_count = out_count;
    *out = t;
    return AFHIP_OK;
}

// weight_b / out_b null: one linear; otherwise two linears of the same shape that share
// the input (the weights must have the same format and layout to share one launch).
afhip_status linear_no_bias_impl(afhip_compute* self, const afhip_tensor* input, const afhip_tensor* weight,
                                 size_t rows, size_t in_dim, size_t out_dim, int dispatch, afhip_tensor** out,
                                 const afhip_tensor* weight_b = nullptr, afhip_tensor** out_b = nullptr,
                                 const afhip_tensor* bias = nullptr, const afhip_tensor* bias_b = nullptr,
                                 const afhip_tensor* residual = nullptr, int activation = AFHIP_ACTIVATION_NONE) {
    // cuda_compute.zig:689-717; with biases (f32 [out_dim], added to every row): linear :544-575, linearPair :799-815
    const bool pair = weight_b != nullptr || out_b != nullptr;
    if (!self || !input || !weight || !out || (pair && (!weight_b || !out_b)) || (bias_b && !pair))
        return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    if (pair) *out_b = nullptr;
    if (!is_f32(input)) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    for (const afhip_tensor* b : {bias, bias_b}) {
        if (!b) continue;
        if (!is_f32(b)) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
        if (b->elem_count != out_dim) return AFHIP_ERR_INVALID_SHAPE;
    }
    if (pair && (residual || activation != AFHIP_ACTIVATION_NONE)) return AFHIP_ERR_INVALID_ARGUMENT;
    if (residual && !is_f32(residual)) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    const afhip_tensor* ws[2] = {weight, weight_b};
    size_t in_count, w_count, out_count, out_bytes;
    if (!checked_mul(rows, in_dim, &in_count) || !checked_mul(out_dim, in_dim, &w_count) ||
        !checked_mul(rows, out_dim, &out_count) || !checked_mul(out_count, 4, &out_bytes))
        return AFHIP_ERR_INVALID_SHAPE;
    if (input->elem_count != in_count) return AFHIP_ERR_INVALID_SHAPE;
    if (residual && residual->elem_count != out_count) return AFHIP_ERR_INVALID_SHAPE;
    for (int i = 0; i < (pair ? 2 : 1); ++i) {
        const afhip_tensor* w = ws[i];
        if (w->quant_type < 0 && !is_f32(w)) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
        if (w->elem_count != w_count) return AFHIP_ERR_INVALID_SHAPE;
        if (w->quant_type < 0) return AFHIP_ERR_OP_UNSUPPORTED;  // dense f32 linear is another operator
        if (w->quant_type != AFHIP_TYPE_Q4_0 && w->quant_type != AFHIP_TYPE_Q8_0 && w->quant_type != AFHIP_TYPE_Q4_K)
            return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    }
    if (pair && (weight_b->quant_type != weight->quant_type || weight_b->layout != weight->layout)) {
        // nothing to share: two independent ops, as the engine's wrapper does (ops/ops.zig:1828-1849)
        afhip_status s = linear_no_bias_impl(self, input, weight, rows, in_dim, out_dim, dispatch, out, nullptr, nullptr, bias);
        if (s != AFHIP_OK) return s;
        s = linear_no_bias_impl(self, input, weight_b, rows, in_dim, out_dim, dispatch, out_b, nullptr, nullptr, bias_b);
        if (s != AFHIP_OK) {
            free_tensor_storage(self, *out);
            delete *out;
            *out = nullptr;
        }
        return s;
    }

    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;
    afhip_buffer device, device_b{0, 0};
    s = alloc_device_buffer(self, out_bytes, &device);
    if (s != AFHIP_OK) return s;
    if (pair) {
        s = alloc_device_buffer(self, out_bytes, &device_b);
        if (s != AFHIP_OK) {
            release_device_buffer(self, &device);
            return s;
        }
    }
    afhip_buffer scratch{0, 0};
    if (weight->quant_type == AFHIP_TYPE_Q4_K) {
        // scratch for the digit planes of three to eight rows and for the split of X when the prefill GEMM serves the
        // rows (repacked tensors), or for the Q8_K activations on the gated short-K shapes (either layout)
        const bool needs = weight->layout == AFHIP_LAYOUT_PREPARED || afhip_uses_q8k_activation_quant(AFHIP_TYPE_Q4_K, rows, in_dim, out_dim);
        const size_t need = needs ? afhip_linear_workspace_bytes(AFHIP_TYPE_Q4_K, rows, in_dim, out_dim) : 0;
        if (need) s = acquire_scratch(self, need, &scratch);
    } else if (afhip_uses_activation_quant(rows, in_dim, out_dim)) {  // scratch for separately quantized activations
        s = acquire_scratch(self, afhip_linear_workspace_bytes(weight->quant_type, rows, in_dim, out_dim), &scratch);
    }
    if (s == AFHIP_OK) {
        LinearExtras extras;
        if (bias) extras.bias = bias->buffer;
        if (bias_b) extras.bias_b = bias_b->buffer;
        if (residual) extras.residual = residual->buffer;
        extras.activation = activation;
        self->counters.phase_events = self->phase_timing ? reinterpret_cast<void**>(self->phase_events) : nullptr;
        const int launch_dispatch =
            dispatch == AFHIP_DISPATCH_AUTO && self->q4k_f32_activations ? AFHIP_DISPATCH_AUTO_F32_ACTIVATIONS : dispatch;
        s = linear_impl(self->stream, weight->quant_type, weight->layout, device, input->buffer, weight->buffer, rows,
                        in_dim, out_dim, scratch, launch_dispatch, afhip_buffer{0, 0}, &self->counters, device_b,
                        pair ? weight_b->buffer : afhip_buffer{0, 0}, extras);
        self->counters.phase_events = nullptr;
        if (s == AFHIP_OK && self->phase_timing && hipEventSynchronize(self->phase_events[2]) == hipSuccess) {
            float quant_ms = 0.0f, compute_ms = 0.0f;
            if (hipEventElapsedTime(&quant_ms, self->phase_events[0], self->phase_events[1]) == hipSuccess &&
                hipEventElapsedTime(&compute_ms, self->phase_events[1], self->phase_events[2]) == hipSuccess) {
                self->stats.activation_quant_ns += static_cast<uint64_t>(quant_ms * 1e6f);
                self->stats.compute_ns += static_cast<uint64_t>(compute_ms * 1e6f);
                self->stats.timed_ops++;
            }
        }
    }
    if (s != AFHIP_OK) {
        release_device_buffer(self, &device);
        if (pair) release_device_buffer(self, &device_b);
        return s;
    }
    s = make_f32_result(self, device, rows, out_dim, out_count, out);
    if (s != AFHIP_OK) {
        if (pair) release_device_buffer(self, &device_b);
        return s;
    }
    if (pair) {
        s = make_f32_result(self, device_b, rows, out_dim, out_count, out_b);
        if (s != AFHIP_OK) {
            free_tensor_storage(self, *out);
            delete *out;
            *out = nullptr;
        }
    }
    return s;
}

}  // namespace

extern "C" {

afhip_status afhip_compute_create(afhip_compute** out) {
    // CudaContext.initDefault (context.zig:44-82): init, device 0, one stream.
    if (!out) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess) return AFHIP_ERR_UNAVAILABLE;
    if (count <= 0) return AFHIP_ERR_NO_DEVICES;
    afhip_compute* self = new (std::nothrow) afhip_compute();
    if (!self) return AFHIP_ERR_OUT_OF_MEMORY;
    self->device = 0;
    afhip_status s = from_hip(hipSetDevice(0));
    if (s == AFHIP_OK) s = from_hip(hipStreamCreate(&self->stream));
    if (s != AFHIP_OK) {
        delete self;
        return s;
    }
    *out = self;
    return AFHIP_OK;
}

void afhip_compute_destroy(afhip_compute* self) {
    if (!self) return;
    (void)hipSetDevice(self->device);
    if (self->stream) (void)hipStreamSynchronize(self->stream);
    for (auto& kv : self->resident_weights) free_device_buffer(&kv.second.buffer);
    for (auto& b : self->temp_buffers) free_device_buffer(&b);
    free_device_buffer(&self->scratch);
    for (hipEvent_t e : self->phase_events)
        if (e) (void)hipEventDestroy(e);
    if (self->stream) (void)hipStreamDestroy(self->stream);
    delete self;
}

int afhip_compute_backend_kind(const afhip_compute*) { return AFHIP_BACKEND_HIP; }

void* afhip_compute_stream(afhip_compute* self) { return self ? self->stream : nullptr; }

afhip_status afhip_compute_synchronize(afhip_compute* self) {
    if (!self) return AFHIP_ERR_INVALID_ARGUMENT;
    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;
    return from_hip(hipStreamSynchronize(self->stream));
}

afhip_status afhip_compute_device_name(afhip_compute* self, char* out, size_t out_len) {
    if (!self || !out || out_len == 0) return AFHIP_ERR_INVALID_ARGUMENT;
    hipDeviceProp_t prop;
    afhip_status s = from_hip(hipGetDeviceProperties(&prop, self->device));
    if (s != AFHIP_OK) return s;
    std::string name = std::string(prop.name) + " (" + prop.gcnArchName + ")";
    std::strncpy(out, name.c_str(), out_len - 1);
    out[out_len - 1] = '\0';
    return AFHIP_OK;
}

afhip_status afhip_compute_insert_weight_from_loaded(afhip_compute* self, const char* key, int tensor_type,
                                                     const void* raw_bytes, size_t raw_len, const int64_t* shape,
                                                     size_t shape_len, int keep_raw_layout) {
    if (!self || !key || (!raw_bytes && raw_len) || (!shape && shape_len)) return AFHIP_ERR_INVALID_ARGUMENT;
    if (tensor_type == AFHIP_TYPE_F32) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;  // f32 goes through insert_weight_f32
    size_t elem_count;
    if (!element_count(shape, shape_len, &elem_count)) return AFHIP_ERR_INVALID_SHAPE;
    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;

    afhip_tensor t;
    t.dtype = AFHIP_DTYPE_U8;
    t.shape.assign(shape, shape + shape_len);
    t.elem_count = elem_count;
    t.quant_type = tensor_type;
    t.layout = AFHIP_LAYOUT_RAW;
    t.owns_buffer = false;
    t.owned_by_tensor = false;
    s = alloc_device_buffer(self, raw_len, &t.buffer);
    if (s != AFHIP_OK) return s;
    s = copy_from_host(self, t.buffer, raw_bytes, raw_len);
    if (s == AFHIP_OK) s = from_hip(hipStreamSynchronize(self->stream));
    if (s != AFHIP_OK) {
        free_device_buffer(&t.buffer);
        return s;
    }
    // Device-side repack for the formats this backend has kernels for; any other
    // quantized type stays resident as raw bytes and is rejected at the op, like
    // the reference backend does (cuda_compute.zig:703-712).
    const bool q4k = tensor_type == AFHIP_TYPE_Q4_K;
    const size_t bb = q4k ? 144 : block_bytes(tensor_type);
    const int64_t block_values = q4k ? 256 : 32;
    if (!keep_raw_layout && bb != 0 && shape_len == 2 && shape[1] > 0 && shape[1] % block_values == 0 &&
        raw_len == static_cast<size_t>(shape[0]) * static_cast<size_t>(shape[1] / block_values) * bb && raw_len > 0) {
        afhip_buffer prepared;
        const size_t prepared_len = afhip_prepared_weight_bytes(tensor_type, static_cast<size_t>(shape[0]), static_cast<size_t>(shape[1]));
        s = alloc_device_buffer(self, prepared_len, &prepared);
        if (s == AFHIP_OK) {
            prepared.len = prepared_len;  // (a pooled buffer may be longer: the weight's own size is what the counters report)
            s = afhip_launch_prepare_weight(self->stream, tensor_type, prepared, t.buffer, static_cast<size_t>(shape[0]),
                                            static_cast<size_t>(shape[1]));
            if (s == AFHIP_OK) s = from_hip(hipStreamSynchronize(self->stream));
            if (s != AFHIP_OK) {
                free_device_buffer(&prepared);
                free_device_buffer(&t.buffer);
                return s;
            }
            self->counters.prepare++;
            free_device_buffer(&t.buffer);  // weight-sized staging copy of the raw bytes: freed, not pooled
            t.buffer = prepared;
            t.layout = AFHIP_LAYOUT_PREPARED;
        } else {
            free_device_buffer(&t.buffer);
            return s;
        }
    }
    auto it = self->resident_weights.find(key);
    if (it != self->resident_weights.end()) {
        self->stats.resident_weight_bytes -= it->second.buffer.len;
        // a replaced weight goes back to the driver, not into the pool of temporaries (queued
        // kernels may still read it: wait for them first)
        (void)hipStreamSynchronize(self->stream);
        free_device_buffer(&it->second.buffer);
        self->resident_weights.erase(it);
    }
    self->stats.resident_weight_bytes += t.buffer.len;
    self->resident_weights.emplace(key, std::move(t));
    return AFHIP_OK;
}

afhip_status afhip_compute_insert_weight_f32(afhip_compute* self, const char* key, const float* data,
                                             const int64_t* shape, size_t shape_len) {
    // insertWeightFromTensor, cuda_compute.zig:140-160
    if (!self || !key || (!shape && shape_len)) return AFHIP_ERR_INVALID_ARGUMENT;
    size_t elem_count, bytes;
    if (!element_count(shape, shape_len, &elem_count) || !checked_mul(elem_count, 4, &bytes)) return AFHIP_ERR_INVALID_SHAPE;
    if (!data && elem_count) return AFHIP_ERR_INVALID_ARGUMENT;
    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;
    afhip_tensor t;
    t.dtype = AFHIP_DTYPE_F32;
    t.shape.assign(shape, shape + shape_len);
    t.elem_count = elem_count;
    t.owns_buffer = false;
    t.owned_by_tensor = false;
    s = alloc_device_buffer(self, bytes, &t.buffer);
    if (s != AFHIP_OK) return s;
    s = copy_from_host(self, t.buffer, data, bytes);
    if (s == AFHIP_OK) s = from_hip(hipStreamSynchronize(self->stream));
    if (s != AFHIP_OK) {
        free_device_buffer(&t.buffer);
        return s;
    }
    auto it = self->resident_weights.find(key);
    if (it != self->resident_weights.end()) {
        self->stats.resident_weight_bytes -= it->second.buffer.len;
        // a replaced weight goes back to the driver, not into the pool of temporaries (queued
        // kernels may still read it: wait for them first)
        (void)hipStreamSynchronize(self->stream);
        free_device_buffer(&it->second.buffer);
        self->resident_weights.erase(it);
    }
    self->stats.resident_weight_bytes += t.buffer.len;
    self->resident_weights.emplace(key, std::move(t));
    return AFHIP_OK;
}

afhip_status afhip_compute_get_weight(afhip_compute* self, const char* key, afhip_tensor** out) {
    if (!self || !key || !out) return AFHIP_ERR_INVALID_ARGUMENT;
    auto it = self->resident_weights.find(key);
    if (it == self->resident_weights.end()) {
        *out = nullptr;
        return AFHIP_ERR_WEIGHT_NOT_FOUND;
    }
    *out = &it->second;  // borrowed; unordered_map never moves its nodes
    return AFHIP_OK;
}

afhip_status afhip_compute_from_float32(afhip_compute* self, const float* data, size_t data_len, const int32_t* shape,
                                        size_t shape_len, afhip_tensor** out) {
    if (!self || !out || (!shape && shape_len)) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    size_t elem_count = 1;
    for (size_t i = 0; i < shape_len; ++i) {
        if (shape[i] < 0) return AFHIP_ERR_INVALID_SHAPE;
        if (!checked_mul(elem_count, static_cast<size_t>(shape[i]), &elem_count)) return AFHIP_ERR_INVALID_SHAPE;
    }
    size_t bytes;
    if (elem_count != data_len || !checked_mul(elem_count, 4, &bytes)) return AFHIP_ERR_INVALID_SHAPE;
    if (!data && elem_count) return AFHIP_ERR_INVALID_ARGUMENT;
    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;
    afhip_buffer device;
    s = alloc_device_buffer(self, bytes, &device);
    if (s != AFHIP_OK) return s;
    s = copy_from_host(self, device, data, bytes);
    if (s == AFHIP_OK) s = from_hip(hipStreamSynchronize(self->stream));
    if (s != AFHIP_OK) {
        free_device_buffer(&device);
        return s;
    }
    afhip_tensor* t = new (std::nothrow) afhip_tensor();
    if (!t) {
        release_device_buffer(self, &device);
        return AFHIP_ERR_OUT_OF_MEMORY;
    }
    t->buffer = device;
    t->shape.assign(shape, shape + shape_len);
    t->elem_count = elem_count;
    *out = t;
    return AFHIP_OK;
}

afhip_status afhip_compute_wrap_device_f32(afhip_compute* self, uint64_t device_ptr, const int64_t* shape,
                                           size_t shape_len, afhip_tensor** out) {
    if (!self || !out || (!shape && shape_len)) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    size_t elem_count, bytes;
    if (!element_count(shape, shape_len, &elem_count) || !checked_mul(elem_count, 4, &bytes)) return AFHIP_ERR_INVALID_SHAPE;
    if (device_ptr == 0 && elem_count) return AFHIP_ERR_INVALID_ARGUMENT;
    afhip_tensor* t = new (std::nothrow) afhip_tensor();
    if (!t) return AFHIP_ERR_OUT_OF_MEMORY;
    t->buffer = afhip_buffer{device_ptr, bytes};
    t->shape.assign(shape, shape + shape_len);
    t->elem_count = elem_count;
    t->owns_buffer = false;
    *out = t;
    return AFHIP_OK;
}

afhip_status afhip_compute_to_float32(afhip_compute* self, const afhip_tensor* tensor, float* out, size_t out_count) {
    if (!self || !tensor || (!out && out_count)) return AFHIP_ERR_INVALID_ARGUMENT;
    if (tensor->dtype != AFHIP_DTYPE_F32) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    if (out_count != tensor->elem_count) return AFHIP_ERR_INVALID_SHAPE;
    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;
    s = copy_to_host(self, out, tensor->buffer, out_count * 4);
    if (s != AFHIP_OK) return s;
    return from_hip(hipStreamSynchronize(self->stream));
}

void afhip_compute_free_tensor(afhip_compute* self, afhip_tensor* tensor) {
    if (!self || !tensor) return;
    if (!tensor->owned_by_tensor) return;  // resident weights are borrowed
    free_tensor_storage(self, tensor);
    delete tensor;
}

afhip_status afhip_compute_eval_tensor(afhip_compute* self, const afhip_tensor*) { return afhip_compute_synchronize(self); }

int afhip_tensor_dtype(const afhip_tensor* t) { return t ? t->dtype : -1; }
int afhip_tensor_quant_type(const afhip_tensor* t) { return t ? t->quant_type : -1; }
int afhip_tensor_layout(const afhip_tensor* t) { return t ? t->layout : -1; }
size_t afhip_tensor_elem_count(const afhip_tensor* t) { return t ? t->elem_count : 0; }
size_t afhip_tensor_rank(const afhip_tensor* t) { return t ? t->shape.size() : 0; }
afhip_status afhip_tensor_shape(const afhip_tensor* t, int64_t* out, size_t out_len) {
    if (!t || (!out && out_len)) return AFHIP_ERR_INVALID_ARGUMENT;
    if (out_len < t->shape.size()) return AFHIP_ERR_INVALID_SHAPE;
    for (size_t i = 0; i < t->shape.size(); ++i) out[i] = t->shape[i];
    return AFHIP_OK;
}
uint64_t afhip_tensor_device_ptr(const afhip_tensor* t) { return t ? t->buffer.ptr : 0; }
size_t afhip_tensor_byte_len(const afhip_tensor* t) { return t ? t->buffer.len : 0; }

afhip_status afhip_compute_embedding_lookup(afhip_compute* self, const afhip_tensor* weight, const int64_t* ids,
                                            size_t ids_len, size_t total, size_t dim, afhip_tensor** out) {
    // cuda_compute.zig:405-435
    if (!self || !weight || !out || (!ids && ids_len != 0)) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    if (weight->quant_type < 0 && !is_f32(weight)) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    if (ids_len != total) return AFHIP_ERR_INVALID_SHAPE;
    if (dim == 0 || weight->elem_count % dim != 0) return AFHIP_ERR_INVALID_SHAPE;
    const size_t vocab = weight->elem_count / dim;
    for (size_t i = 0; i < total; ++i)
        if (ids[i] < 0 || static_cast<uint64_t>(ids[i]) >= vocab) return AFHIP_ERR_INVALID_TOKEN_ID;
    if (weight->quant_type >= 0 && weight->quant_type != AFHIP_TYPE_Q4_0 && weight->quant_type != AFHIP_TYPE_Q8_0 &&
        weight->quant_type != AFHIP_TYPE_Q4_K)
        return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    size_t out_count, out_bytes;
    if (!checked_mul(total, dim, &out_count) || !checked_mul(out_count, 4, &out_bytes)) return AFHIP_ERR_INVALID_SHAPE;
    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;
    afhip_buffer ids_device, device;
    s = alloc_device_buffer(self, total * 8, &ids_device);  // uploadTempI64
    if (s != AFHIP_OK) return s;
    s = alloc_device_buffer(self, out_bytes, &device);
    if (s == AFHIP_OK) s = copy_from_host(self, ids_device, ids, total * 8);
    if (s == AFHIP_OK)
        s = afhip_launch_embedding_lookup_f32(self->stream, weight->quant_type < 0 ? AFHIP_TYPE_F32 : weight->quant_type,
                                              weight->layout, device, weight->buffer, ids_device, total, dim, vocab);
    // the ids were read from pageable host memory: the copy has completed on return, and the
    // kernel that reads the device copy is ordered before any later use of the pooled buffer
    release_device_buffer(self, &ids_device);
    if (s != AFHIP_OK) {
        release_device_buffer(self, &device);
        return s;
    }
    return make_f32_result(self, device, total, dim, out_count, out);
}

afhip_status afhip_compute_linear_no_bias(afhip_compute* self, const afhip_tensor* input, const afhip_tensor* weight,
                                          size_t rows, size_t in_dim, size_t out_dim, afhip_tensor** out) {
    return linear_no_bias_impl(self, input, weight, rows, in_dim, out_dim, -1, out);
}

afhip_status afhip_compute_linear_no_bias_pair(afhip_compute* self, const afhip_tensor* input,
                                               const afhip_tensor* weight_a, const afhip_tensor* weight_b, size_t rows,
                                               size_t in_dim, size_t out_dim, afhip_tensor** out_first,
                                               afhip_tensor** out_second) {
    if (!weight_b || !out_second) return AFHIP_ERR_INVALID_ARGUMENT;
    return linear_no_bias_impl(self, input, weight_a, rows, in_dim, out_dim, -1, out_first, weight_b, out_second);
}

afhip_status afhip_compute_linear(afhip_compute* self, const afhip_tensor* input, const afhip_tensor* weight,
                                  const afhip_tensor* bias, size_t rows, size_t in_dim, size_t out_dim,
                                  afhip_tensor** out) {
    if (!bias) return AFHIP_ERR_INVALID_ARGUMENT;
    return linear_no_bias_impl(self, input, weight, rows, in_dim, out_dim, -1, out, nullptr, nullptr, bias);
}

afhip_status afhip_compute_linear_activation(afhip_compute* self, const afhip_tensor* input, const afhip_tensor* weight,
                                             const afhip_tensor* bias, int activation, size_t rows, size_t in_dim,
                                             size_t out_dim, afhip_tensor** out) {
    if (!bias || activation < AFHIP_ACTIVATION_NONE || activation > AFHIP_ACTIVATION_GELU) return AFHIP_ERR_INVALID_ARGUMENT;
    return linear_no_bias_impl(self, input, weight, rows, in_dim, out_dim, -1, out, nullptr, nullptr, bias, nullptr, nullptr,
                               activation);
}

afhip_status afhip_compute_linear_add(afhip_compute* self, const afhip_tensor* input, const afhip_tensor* weight,
                                      const afhip_tensor* bias, const afhip_tensor* residual, size_t rows, size_t in_dim,
                                      size_t out_dim, afhip_tensor** out) {
    if (!bias || !residual) return AFHIP_ERR_INVALID_ARGUMENT;
    return linear_no_bias_impl(self, input, weight, rows, in_dim, out_dim, -1, out, nullptr, nullptr, bias, nullptr, residual);
}

afhip_status afhip_compute_linear_pair(afhip_compute* self, const afhip_tensor* input, const afhip_tensor* weight_a,
                                       const afhip_tensor* bias_a, const afhip_tensor* weight_b,
                                       const afhip_tensor* bias_b, size_t rows, size_t in_dim, size_t out_dim,
                                       afhip_tensor** out_first, afhip_tensor** out_second) {
    if (!weight_b || !out_second || !bias_a || !bias_b) return AFHIP_ERR_INVALID_ARGUMENT;
    return linear_no_bias_impl(self, input, weight_a, rows, in_dim, out_dim, -1, out_first, weight_b, out_second, bias_a,
                               bias_b);
}

afhip_status afhip_compute_linear_triple(afhip_compute* self, const afhip_tensor* input, const afhip_tensor* weight_a,
                                         const afhip_tensor* bias_a, const afhip_tensor* weight_b,
                                         const afhip_tensor* bias_b, const afhip_tensor* weight_c,
                                         const afhip_tensor* bias_c, size_t rows, size_t in_dim, size_t out_dim,
                                         afhip_tensor** out_first, afhip_tensor** out_second,
                                         afhip_tensor** out_third) {
    // Q/K/V with separate weights: the first two share one launch where a pair does, the third follows
    if (!out_third || !weight_c || !bias_c) return AFHIP_ERR_INVALID_ARGUMENT;
    *out_third = nullptr;
    afhip_status s = afhip_compute_linear_pair(self, input, weight_a, bias_a, weight_b, bias_b, rows, in_dim, out_dim,
                                               out_first, out_second);
    if (s != AFHIP_OK) return s;
    s = afhip_compute_linear(self, input, weight_c, bias_c, rows, in_dim, out_dim, out_third);
    if (s != AFHIP_OK) {
        for (afhip_tensor** t : {out_first, out_second}) {
            free_tensor_storage(self, *t);
            delete *t;
            *t = nullptr;
        }
    }
    return s;
}

afhip_status afhip_compute_linear_no_bias_grouped(afhip_compute* self, const afhip_tensor* input,
                                                  const afhip_tensor* weight, size_t rows, size_t in_dim, size_t out_dim,
                                                  const uint32_t* projection_out_dims, size_t num_projections,
                                                  afhip_tensor** out) {
    if (!out) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    if (num_projections == 0 || !projection_out_dims) return AFHIP_ERR_INVALID_SHAPE;
    size_t total = 0;
    for (size_t i = 0; i < num_projections; ++i) {
        if (projection_out_dims[i] == 0) return AFHIP_ERR_INVALID_SHAPE;
        total += projection_out_dims[i];
    }
    if (total != out_dim) return AFHIP_ERR_INVALID_SHAPE;
    // the projections are rows [o0, o1) of one concatenated matrix: one linear serves them all
    return linear_no_bias_impl(self, input, weight, rows, in_dim, out_dim, -1, out);
}

afhip_status afhip_compute_argmax_last_row(afhip_compute* self, const afhip_tensor* tensor, size_t rows, size_t dim,
                                           uint32_t* token) {
    if (!self || !tensor || !token) return AFHIP_ERR_INVALID_ARGUMENT;
    if (!is_f32(tensor)) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    size_t count;
    if (rows == 0 || dim == 0 || !checked_mul(rows, dim, &count) || tensor->elem_count != count)
        return AFHIP_ERR_INVALID_SHAPE;
    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;
    afhip_buffer id;
    s = alloc_device_buffer(self, 4, &id);
    if (s != AFHIP_OK) return s;
    afhip_buffer scratch{0, 0};
    s = acquire_scratch(self, afhip_argmax_workspace_bytes(dim), &scratch);
    if (s == AFHIP_OK)
        s = afhip_launch_argmax_last_row_f32(self->stream, id, afhip_buffer{0, 0}, tensor->buffer, rows, dim, scratch);
    if (s == AFHIP_OK) s = copy_to_host(self, token, id, 4);
    if (s == AFHIP_OK) s = from_hip(hipStreamSynchronize(self->stream));
    release_device_buffer(self, &id);
    return s;
}

namespace {

// token_host: the id is copied back and the stream synchronized; token_tensor: a new f32 [1] tensor.
afhip_status linear_argmax(afhip_compute* self, const afhip_tensor* input, const afhip_tensor* weight, size_t rows,
                           size_t in_dim, size_t out_dim, uint32_t* token_host, afhip_tensor** token_tensor) {
    if (!self || !input || !weight) return AFHIP_ERR_INVALID_ARGUMENT;
    if (!is_f32(input)) return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    size_t in_count, w_count;
    if (rows == 0 || in_dim == 0 || out_dim == 0 || !checked_mul(rows, in_dim, &in_count) ||
        !checked_mul(out_dim, in_dim, &w_count) || input->elem_count != in_count || weight->elem_count != w_count)
        return AFHIP_ERR_INVALID_SHAPE;
    if (weight->quant_type < 0) return is_f32(weight) ? AFHIP_ERR_OP_UNSUPPORTED : AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    if (weight->quant_type != AFHIP_TYPE_Q4_0 && weight->quant_type != AFHIP_TYPE_Q8_0 && weight->quant_type != AFHIP_TYPE_Q4_K)
        return AFHIP_ERR_UNSUPPORTED_TENSOR_TYPE;
    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;
    afhip_buffer id;  // [f32 id][u32 id]
    s = alloc_device_buffer(self, 8, &id);
    if (s != AFHIP_OK) return s;
    afhip_buffer scratch{0, 0};
    s = acquire_scratch(self, afhip_linear_argmax_workspace_bytes(weight->quant_type, in_dim, out_dim), &scratch);
    const afhip_buffer id_f32{id.ptr, 4};
    const afhip_buffer id_u32{id.ptr + 4, 4};
    if (s == AFHIP_OK)
        s = linear_argmax_impl(self->stream, weight->quant_type, weight->layout, id_u32, id_f32, input->buffer,
                               weight->buffer, rows, in_dim, out_dim, scratch, &self->counters);
    if (s == AFHIP_OK && token_host) {
        s = copy_to_host(self, token_host, id_u32, 4);
        if (s == AFHIP_OK) s = from_hip(hipStreamSynchronize(self->stream));
    }
    if (s != AFHIP_OK || !token_tensor) {
        release_device_buffer(self, &id);
        return s;
    }
    // the f32 copy of the id (first word) is the tensor's one element; the buffer goes with the tensor
    afhip_tensor* t = new (std::nothrow) afhip_tensor();
    if (!t) {
        release_device_buffer(self, &id);
        return AFHIP_ERR_OUT_OF_MEMORY;
    }
    t->buffer = id;
    t->dtype = AFHIP_DTYPE_F32;
    t->shape = {1};
    t->elem_count = 1;
    *token_tensor = t;
    return AFHIP_OK;
}

}  // namespace

afhip_status afhip_compute_linear_no_bias_argmax_last_row(afhip_compute* self, const afhip_tensor* input,
                                                          const afhip_tensor* weight, size_t rows, size_t in_dim,
                                                          size_t out_dim, uint32_t* token) {
    if (!token) return AFHIP_ERR_INVALID_ARGUMENT;
    return linear_argmax(self, input, weight, rows, in_dim, out_dim, token, nullptr);
}

afhip_status afhip_compute_linear_no_bias_argmax_last_row_tensor(afhip_compute* self, const afhip_tensor* input,
                                                                 const afhip_tensor* weight, size_t rows, size_t in_dim,
                                                                 size_t out_dim, afhip_tensor** out) {
    if (!out) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    return linear_argmax(self, input, weight, rows, in_dim, out_dim, nullptr, out);
}

afhip_status afhip_compute_linear_no_bias_planned(afhip_compute* self,
                                                  const afhip_linear_no_bias_planned_request* request,
                                                  afhip_tensor** out) {
    if (!self || !request || !out) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = nullptr;
    if (!request->weight || !request->input) return AFHIP_ERR_INVALID_ARGUMENT;
    // validateQuantLinearPlan, ops/native_compute.zig:5039-5050
    const afhip_operator_plan& plan = request->operator_plan;
    if (plan.kind != AFHIP_PLAN_QUANT_MATMUL) return AFHIP_ERR_INVALID_PARTITION_PLAN;
    const afhip_quant_plan& q = plan.quant_matmul;
    if (q.op == AFHIP_OP_FALLBACK || q.rows != request->rows || q.in_dim != request->in_dim ||
        q.out_dim != request->out_dim)
        return AFHIP_ERR_INVALID_PARTITION_PLAN;
    const int expected = afhip_quant_format_from_tensor_type(request->weight->quant_type);
    if (request->weight->quant_type < 0 || expected == AFHIP_FORMAT_UNKNOWN || q.format != expected)
        return AFHIP_ERR_INVALID_PARTITION_PLAN;
    if (q.dispatch > AFHIP_DISPATCH_MM) return AFHIP_ERR_INVALID_PARTITION_PLAN;
    return linear_no_bias_impl(self, request->input, request->weight, request->rows, request->in_dim, request->out_dim,
                               q.dispatch, out);
}

afhip_status afhip_compute_set_q4k_f32_activations(afhip_compute* self, int enabled) {
    if (!self) return AFHIP_ERR_INVALID_ARGUMENT;
    self->q4k_f32_activations = enabled != 0;
    return AFHIP_OK;
}

afhip_status afhip_compute_set_phase_timing(afhip_compute* self, int enabled) {
    if (!self) return AFHIP_ERR_INVALID_ARGUMENT;
    afhip_status s = make_current(self);
    if (s != AFHIP_OK) return s;
    if (enabled && self->phase_events[0] == nullptr) {
        for (hipEvent_t& e : self->phase_events) {
            s = from_hip(hipEventCreate(&e));
            if (s != AFHIP_OK) {
                // all three or none: a later call starts over
                for (hipEvent_t& made : self->phase_events) {
                    if (made != nullptr) (void)hipEventDestroy(made);
                    made = nullptr;
                }
                return s;
            }
        }
    }
    self->phase_timing = enabled != 0;
    return AFHIP_OK;
}

afhip_status afhip_compute_debug_stats(const afhip_compute* self, afhip_debug_stats* out) {
    if (!self || !out) return AFHIP_ERR_INVALID_ARGUMENT;
    *out = self->stats;
    out->pooled_buffers = self->temp_buffers.size();
    out->launches_mmv = self->counters.mmv;
    out->launches_small_batch = self->counters.small_batch;
    out->launches_mm = self->counters.mm;
    out->launches_f32_route = self->counters.f32_route;
    out->launches_activation_quant = self->counters.activation_quant;
    out->launches_prepare = self->counters.prepare;
    out->scratch_bytes = self->scratch.len;
    return AFHIP_OK;
}

// ---- smokes, ops/cuda/kernels.zig:2309-2399

static afhip_status run_smoke(int tensor_type) {
    const size_t rows = 2, in_dim = 32, out_dim = 3;
    float input[64];
    for (int i = 0; i < 32; ++i) {
        input[i] = static_cast<float>(i + 1);
        input[32 + i] = -static_cast<float>(i + 1);
    }
    const size_t bb = block_bytes(tensor_type);
    uint8_t weight[3 * 34] = {0};
    const uint16_t scale_bits[3] = {0x3C00, 0x3800, 0x4000};  // 1.0, 0.5, 2.0
    const int values[3] = {1, 2, -1};
    for (int r = 0; r < 3; ++r) {
        uint8_t* blk = weight + r * bb;
        blk[0] = static_cast<uint8_t>(scale_bits[r] & 0xff);
        blk[1] = static_cast<uint8_t>(scale_bits[r] >> 8);
        if (tensor_type == AFHIP_TYPE_Q8_0) {
            for (int i = 0; i < 32; ++i) blk[2 + i] = static_cast<uint8_t>(static_cast<int8_t>(values[r]));
        } else {
            const uint8_t nib = static_cast<uint8_t>(values[r] + 8);
            for (int i = 0; i < 16; ++i) blk[2 + i] = static_cast<uint8_t>(nib | (nib << 4));
        }
    }
    afhip_compute* c = nullptr;
    afhip_status s = afhip_compute_create(&c);
    if (s != AFHIP_OK) return s;
    const int64_t wshape[2] = {static_cast<int64_t>(out_dim), static_cast<int64_t>(in_dim)};
    const int32_t xshape[2] = {static_cast<int32_t>(rows), static_cast<int32_t>(in_dim)};
    afhip_tensor *x = nullptr, *w = nullptr, *y = nullptr;
    float out[6] = {0};
    s = afhip_compute_insert_weight_from_loaded(c, "smoke.weight", tensor_type, weight, out_dim * bb, wshape, 2, 0);
    if (s == AFHIP_OK) s = afhip_compute_get_weight(c, "smoke.weight", &w);
    if (s == AFHIP_OK) s = afhip_compute_from_float32(c, input, 64, xshape, 2, &x);
    if (s == AFHIP_OK) s = afhip_compute_linear_no_bias(c, x, w, rows, in_dim, out_dim, &y);
    if (s == AFHIP_OK) s = afhip_compute_to_float32(c, y, out, 6);
    if (s == AFHIP_OK) {
        const float expected[6] = {528, 528, -1056, -528, -528, 1056};
        for (int i = 0; i < 6; ++i)
            if (!(std::fabs(out[i] - expected[i]) <= 0.01f)) s = AFHIP_ERR_SMOKE_MISMATCH;
    }
    afhip_compute_free_tensor(c, y);
    afhip_compute_free_tensor(c, x);
    afhip_compute_destroy(c);
    return s;
}

afhip_status afhip_smoke_q8_0(void) { return run_smoke(AFHIP_TYPE_Q8_0); }
afhip_status afhip_smoke_q4_0(void) { return run_smoke(AFHIP_TYPE_Q4_0); }

}  // extern "C"
