// The forward-only fp32 C API (include/flashlstm/lstm_api.h) on top of the device-resident core.
// Behaviour follows the reference entry points: lstm_create_buffers (src/lstm.cu:675-857),
// lstm_destroy_buffers (:859-866), lstm_set_execution_mode (:868-884), lstm_pack_weights (:886-931)
// and lstm_forward (:1897-2148): same validation order, same error value (1) for bad arguments,
// blocking semantics, a private non-blocking stream per handle, and sequence lengths that may
// shrink or grow between calls.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <new>

#include "../../include/flashlstm/lstm_api.h"
#include "../../include/flashlstm/lstm_core.h"
#include "instrument.h"

namespace {

struct V1Impl {
    lstm_compute_precision_t precision;
    size_t batch, input_size, hidden_size;
    int proj_chunk;
    lstm_execution_mode_t mode;
    flstm_core_plan* plan;   // null when any dimension is zero
    hipStream_t stream;
    bool weights_packed;
    size_t cached_T;         // sequence length of the forward pass whose caches the plan holds (0 = none)
};

constexpr int kInvalid = int(hipErrorInvalidValue);

void destroy_impl(V1Impl* impl) {
    if (!impl) return;
    if (impl->plan) flstm_core_destroy(impl->plan);
    if (impl->stream) (void)hipStreamDestroy(impl->stream);
    delete impl;
}

}  // namespace

extern "C" int lstm_create_buffers(lstm_compute_precision_t precision, size_t seq_len, size_t batch,
                                   size_t input_size, size_t hidden_size, int input_proj_chunk_size,
                                   lstm_buffers* buffers) {
    (void)seq_len;  // buffers are sized by the first forward and grow on demand
    if (!buffers) return kInvalid;
    buffers->impl = nullptr;
    if (precision != LSTM_COMPUTE_PRECISION_FP16_ACC32 && precision != LSTM_COMPUTE_PRECISION_FP16_ACC16)
        return kInvalid;
    auto* impl = new (std::nothrow) V1Impl();
    if (!impl) return int(hipErrorOutOfMemory);
    impl->precision = precision;
    impl->batch = batch;
    impl->input_size = input_size;
    impl->hidden_size = hidden_size;
    impl->proj_chunk = input_proj_chunk_size;
    impl->mode = LSTM_EXECUTION_MODE_IMMEDIATE;
    impl->plan = nullptr;
    impl->stream = nullptr;
    impl->cached_T = 0;
    const bool empty = (batch == 0 || input_size == 0 || hidden_size == 0);
    impl->weights_packed = (hidden_size == 0 || input_size + hidden_size == 0);
    if (!empty) {
        int rc = flstm_core_create(batch, input_size, hidden_size, &impl->plan);
        if (rc) { destroy_impl(impl); return rc; }
        flstm_core_set_option(impl->plan, "proj_chunk", input_proj_chunk_size);
    }
    hipError_t e = hipStreamCreateWithFlags(&impl->stream, hipStreamNonBlocking);
    if (e != hipSuccess) { destroy_impl(impl); return int(e); }
    buffers->impl = impl;
    return 0;
}

extern "C" int lstm_destroy_buffers(lstm_buffers* buffers) {
    if (!buffers) return kInvalid;
    destroy_impl(static_cast<V1Impl*>(buffers->impl));
    buffers->impl = nullptr;
    return 0;
}

extern "C" int lstm_set_execution_mode(lstm_buffers* buffers, lstm_execution_mode_t mode) {
    if (!buffers || !buffers->impl) return kInvalid;
    if (mode != LSTM_EXECUTION_MODE_IMMEDIATE && mode != LSTM_EXECUTION_MODE_GRAPH) return kInvalid;
    auto* impl = static_cast<V1Impl*>(buffers->impl);
    if (impl->mode == mode) return 0;
    impl->mode = mode;
    return 0;
}

extern "C" int lstm_pack_weights(lstm_compute_precision_t precision, const float* weight_ih,
                                 const float* weight_hh, size_t input_size, size_t hidden_size,
                                 lstm_buffers* buffers) {
    if (!buffers || !buffers->impl) return kInvalid;
    auto* impl = static_cast<V1Impl*>(buffers->impl);
    if (impl->precision != precision) {
        std::fprintf(stderr, "Precision mismatch in lstm_pack_weights\n");
        return kInvalid;
    }
    if (impl->input_size != input_size || impl->hidden_size != hidden_size) {
        std::fprintf(stderr, "Dimension mismatch in lstm_pack_weights\n");
        return kInvalid;
    }
    if (impl->plan) {
        int rc = flstm_core_pack_weights(impl->plan, weight_ih, weight_hh, impl->stream);
        if (rc) return rc;
    }
    impl->weights_packed = true;
    return 0;
}

extern "C" int lstm_forward(const float* x, const float* b_ih, const float* b_hh, const float* h0,
                            const float* c0, float* output, float* hn, float* cn, size_t seq_len,
                            size_t batch, size_t input_size, size_t hidden_size, const lstm_buffers* buffers,
                            lstm_compute_precision_t precision) {
    flstm_hip::RangeGuard range("FlashLSTM::lstm_forward");
    if (!buffers || !buffers->impl) return kInvalid;
    auto* impl = static_cast<V1Impl*>(buffers->impl);
    if (impl->precision != precision) return kInvalid;
    if (impl->batch != batch || impl->input_size != input_size || impl->hidden_size != hidden_size) return kInvalid;
    if (!impl->weights_packed) return kInvalid;
    if (!impl->stream) return kInvalid;
    if (!impl->plan) return 0;
    const size_t state_bytes = batch * hidden_size * sizeof(float);
    if (seq_len == 0) {
        // no steps: the final state is the initial state
        if (hn && h0) { hipError_t e = hipMemcpyAsync(hn, h0, state_bytes, hipMemcpyDeviceToDevice, impl->stream); if (e != hipSuccess) return int(e); }
        if (cn && c0) { hipError_t e = hipMemcpyAsync(cn, c0, state_bytes, hipMemcpyDeviceToDevice, impl->stream); if (e != hipSuccess) return int(e); }
        return int(hipStreamSynchronize(impl->stream));
    }
    // GRAPH selects the persistent recurrence, IMMEDIATE the step-by-step launches.  Like the
    // reference (which forces its graph path, src/lstm.cu:23,1922-1924) the persistent path is used
    // unless FLASHLSTM_V1_HONOR_IMMEDIATE is set in the environment.
    static const bool honor_immediate = (getenv("FLASHLSTM_V1_HONOR_IMMEDIATE") != nullptr);
    flstm_core_set_option(impl->plan, "stepwise",
                          (honor_immediate && impl->mode == LSTM_EXECUTION_MODE_IMMEDIATE) ? 1 : 0);
    int rc = flstm_core_pack_bias(impl->plan, b_ih, b_hh, impl->stream);
    if (rc) return rc;
    flstm_hip::RangeGuard compute("FlashLSTM::lstm_forward::compute");
    impl->cached_T = 0;
    rc = flstm_core_forward(impl->plan, seq_len, x, FLSTM_F32, h0, c0, FLSTM_F32, output, FLSTM_F32, hn, cn,
                            FLSTM_F32, 1, impl->stream);
    if (rc == 0) impl->cached_T = seq_len;
    return rc;
}

extern "C" int lstm_get_cache(const lstm_buffers* buffers, int which, const void** ptr, size_t* ld, size_t* seq_len) {
    if (!buffers || !buffers->impl || !ptr || !ld) return kInvalid;
    auto* impl = static_cast<V1Impl*>(buffers->impl);
    if (!impl->plan || impl->cached_T == 0) return kInvalid;
    if (seq_len) *seq_len = impl->cached_T;
    return flstm_core_cache_ptr(impl->plan, which, ptr, ld);
}

extern "C" int lstm_backward(const float* x, const float* d_output, const float* d_hn, const float* d_cn,
                             float* dx, float* dW_ih, float* dW_hh, float* db, float* dh0, float* dc0,
                             size_t seq_len, size_t batch, size_t input_size, size_t hidden_size,
                             const lstm_buffers* buffers) {
    flstm_hip::RangeGuard range("FlashLSTM::lstm_backward");
    if (!buffers || !buffers->impl) return kInvalid;
    auto* impl = static_cast<V1Impl*>(buffers->impl);
    if (impl->batch != batch || impl->input_size != input_size || impl->hidden_size != hidden_size) return kInvalid;
    if (!impl->plan || seq_len == 0) return 0;
    return flstm_core_backward(impl->plan, seq_len, x, FLSTM_F32, d_output, FLSTM_F32, d_hn, d_cn, FLSTM_F32, 1.f,
                               dx, FLSTM_F32, dW_ih, dW_hh, db, nullptr, dh0, dc0, impl->stream);
}
