// Streaming LSTM forward / backward: host-resident sequences, device-resident weights and states.
//
// Drop-in for the reference's flashlstm_v2/include/lstm.hpp:7-213 with HIP types in place of the
// CUDA ones (__half from <hip/hip_fp16.h>, hipStream_t): same namespace, struct layouts, enum
// values, argument order (note that `options` is the LAST argument of flstm_StreamingLstmBackward
// but sits before hy/cy in flstm_StreamingLstmForward) and the same failure behaviour -- the C++
// overloads throw std::runtime_error, the C entry points print the message and abort().
//
// Tensors:
//   host (pinned preferred, pageable accepted), fp16:  x (T,B,I)  y (T,B,H)  dY (T,B,H)  dx (T,B,I)
//   host caches: h and c checkpoints (ceil(T/R), B, H); entry k is the state BEFORE step k*R
//                (entry 0 = h0/c0); element type per cache from StreamingLstmOptions
//   device fp16: h0, c0, hy, cy, d_hn, d_cn (B,H)      device fp32: W_ih (4H,I) W_hh (4H,H) b (4H)
//   device fp32 outputs of backward (overwritten): dW_ih, dW_hh, db_ih (== db_hh), dh0, dc0
// The three streams must be pairwise distinct; all are synchronised before the calls return.
// Calls are not re-entrant.
#pragma once

#include <cstddef>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

namespace flstm {

enum class GateCacheDType : int {
    kFloat32 = 0,
    kFloat16 = 1,
};

struct GateCacheHost {
    void *h_ptr;
    void *c_ptr;
};

struct StreamingLstmOptions {
    GateCacheDType h_dtype = GateCacheDType::kFloat32;
    GateCacheDType c_dtype = GateCacheDType::kFloat32;
};

void StreamingLstmForward(
    size_t time_steps, size_t batch_size, size_t input_size, size_t hidden_size,
    size_t recompute_interval,
    const __half *x_tensor_host, const __half *h0_device, const __half *c0_device,
    const float *weights_ih, const float *weights_hh, const float *bias_ih, const float *bias_hh,
    __half *y_tensor_host,
    GateCacheHost gate_cache_host, StreamingLstmOptions options,
    __half *hy_device, __half *cy_device,
    hipStream_t compute_stream, hipStream_t h2d_stream, hipStream_t d2h_stream);

void StreamingLstmBackward(
    size_t time_steps, size_t batch_size, size_t input_size, size_t hidden_size,
    size_t recompute_interval,
    const __half *x_tensor_host, const __half *y_tensor_host,
    GateCacheHost gate_cache_host, StreamingLstmOptions options,
    const __half *dY_tensor_host, const __half *d_hn_device, const __half *d_cn_device,
    const __half *h0_device, const __half *c0_device,
    const float *weights_ih, const float *weights_hh, const float *bias_ih, const float *bias_hh,
    __half *dx_tensor_host,
    float *dW_ih, float *dW_hh, float *db_ih, float *db_hh, float *dh0_out, float *dc0_out,
    hipStream_t compute_stream, hipStream_t h2d_stream, hipStream_t d2h_stream);

} // namespace flstm

extern "C" {

typedef enum {
    FLSTM_GATE_CACHE_FLOAT32 = 0,
    FLSTM_GATE_CACHE_FLOAT16 = 1,
} flstm_GateCacheDType;

typedef struct {
    void *h_ptr;
    void *c_ptr;
} flstm_GateCacheHost;

typedef struct {
    flstm_GateCacheDType h_dtype;
    flstm_GateCacheDType c_dtype;
} flstm_StreamingLstmOptions;

void flstm_StreamingLstmForward(
    size_t time_steps, size_t batch_size, size_t input_size, size_t hidden_size,
    size_t recompute_interval,
    const __half *x_tensor_host, const __half *h0_device, const __half *c0_device,
    const float *weights_ih, const float *weights_hh, const float *bias_ih, const float *bias_hh,
    __half *y_tensor_host,
    flstm_GateCacheHost gate_cache_host, const flstm_StreamingLstmOptions *options,
    __half *hy_device, __half *cy_device,
    hipStream_t compute_stream, hipStream_t h2d_stream, hipStream_t d2h_stream);

void flstm_StreamingLstmBackward(
    size_t time_steps, size_t batch_size, size_t input_size, size_t hidden_size,
    size_t recompute_interval,
    const __half *x_tensor_host, const __half *y_tensor_host,
    flstm_GateCacheHost gate_cache_host,
    const __half *dY_tensor_host, const __half *d_hn_device, const __half *d_cn_device,
    const __half *h0_device, const __half *c0_device,
    const float *weights_ih, const float *weights_hh, const float *bias_ih, const float *bias_hh,
    __half *dx_tensor_host,
    float *dW_ih, float *dW_hh, float *db_ih, float *db_hh, float *dh0_out, float *dc0_out,
    hipStream_t compute_stream, hipStream_t h2d_stream, hipStream_t d2h_stream,
    const flstm_StreamingLstmOptions *options);

// Addition (not in the reference): frees every plan and device staging buffer the two entry points
// keep between calls.
void flstm_ReleaseStreamingCaches(void);

} // extern "C"
