/* C API of the device-resident forward LSTM (fp32 tensors in and out, fp16 MFMA arithmetic inside).
 *
 * Binary-compatible with the reference's include/flashlstm/lstm_api.h:9-56: same five entry points,
 * enum values and opaque handle, so its ctypes and C++ callers (python/test_lstm.py:44-84,
 * src/run_lstm.cu:209-256) bind to this library unchanged.  Implemented for MI355X (gfx950).
 *
 * Contract (all tensor pointers are device memory, fp32, contiguous):
 *   x (T,B,I)   W_ih (4H,I)   W_hh (4H,H)   b_ih,b_hh (4H)   h0,c0,hn,cn (B,H)   output (T,B,H)
 * Gate order i,f,g,o.  Every function returns 0 on success and a hipError_t value otherwise
 * (invalid arguments: 1).  lstm_forward blocks until the results are in place; seq_len may differ
 * from the one given at creation, batch/input/hidden may not.  A handle must not be used from two
 * threads at once.
 *
 * Additions over the reference are at the end of this file (lstm_backward and friends); they do not
 * change the layout or meaning of anything above them.
 */
#ifndef FLASHLSTM_LSTM_API_H_
#define FLASHLSTM_LSTM_API_H_

#ifdef __cplusplus
#include <cstddef>
extern "C" {
#else
#include <stddef.h>
#endif

/* Both values compute with fp16 operands.  CDNA4 MFMA always accumulates in fp32, so
 * ..._FP16_ACC16 is accepted and runs with fp32 accumulation (a strictly tighter result). */
typedef enum {
    LSTM_COMPUTE_PRECISION_FP16_ACC32 = 0,
    LSTM_COMPUTE_PRECISION_FP16_ACC16 = 1,
} lstm_compute_precision_t;

/* IMMEDIATE: one kernel launch per time step.  GRAPH: the whole recurrence in one persistent
 * launch (the role CUDA graphs play in the reference).  Results are identical. */
typedef enum {
    LSTM_EXECUTION_MODE_IMMEDIATE = 0,
    LSTM_EXECUTION_MODE_GRAPH = 1,
} lstm_execution_mode_t;

typedef struct lstm_buffers {
    void* impl;
} lstm_buffers;

/* input_proj_chunk_size: time steps per input-projection GEMM; <= 0 means the whole sequence. */
int lstm_create_buffers(lstm_compute_precision_t precision,
                        size_t seq_len,
                        size_t batch,
                        size_t input_size,
                        size_t hidden_size,
                        int input_proj_chunk_size,
                        lstm_buffers* buffers);

int lstm_destroy_buffers(lstm_buffers* buffers);

int lstm_set_execution_mode(lstm_buffers* buffers, lstm_execution_mode_t mode);

int lstm_pack_weights(lstm_compute_precision_t precision,
                      const float* weight_ih,
                      const float* weight_hh,
                      size_t input_size,
                      size_t hidden_size,
                      lstm_buffers* buffers);

int lstm_forward(const float* x,
                 const float* b_ih,
                 const float* b_hh,
                 const float* h0,
                 const float* c0,
                 float* output,
                 float* hn,
                 float* cn,
                 size_t seq_len,
                 size_t batch,
                 size_t input_size,
                 size_t hidden_size,
                 const lstm_buffers* buffers,
                 lstm_compute_precision_t precision);

/* ---- additions (no counterpart in the reference, whose v1 API is forward-only) ---------------- */

/* BPTT for the most recent lstm_forward on this handle (which keeps its fp16 gate cache and fp32
 * cell states).  d_output (T,B,H); d_hn, d_cn (B,H) may be null.  Outputs (any may be null):
 * dx (T,B,I), dW_ih (4H,I), dW_hh (4H,H), db (4H, the gradient of both b_ih and b_hh),
 * dh0, dc0 (B,H).  All fp32 device memory. */
int lstm_backward(const float* x,
                  const float* d_output,
                  const float* d_hn,
                  const float* d_cn,
                  float* dx,
                  float* dW_ih,
                  float* dW_hh,
                  float* db,
                  float* dh0,
                  float* dc0,
                  size_t seq_len,
                  size_t batch,
                  size_t input_size,
                  size_t hidden_size,
                  const lstm_buffers* buffers);

/* Read access to what the most recent lstm_forward on this handle cached for lstm_backward (device pointers,
 * valid until the next lstm_forward or lstm_destroy_buffers on the handle; the reference keeps no such cache:
 * its pointwise kernel overwrites the pre-activations every step, src/lstm.cu:1330).  `which`:
 *   LSTM_CACHE_HIDDEN (0): h states, fp16 [(T+1)*B][ld], row t*B+b = h before step t (row block 0 = h0)
 *   LSTM_CACHE_CELL   (1): c states, fp32 [(T+1)*B][ld], row block t = c before step t
 *   LSTM_CACHE_GATES  (2): activated gates, fp16 [T*B][ld], column 4*unit + gate with gates i, f, g, o
 * *ld receives the row pitch in elements (hidden size rounded up to a multiple of 32, times 4 for the gates),
 * *seq_len the length of the cached sequence.  Returns 1 when nothing is cached. */
enum { LSTM_CACHE_HIDDEN = 0, LSTM_CACHE_CELL = 1, LSTM_CACHE_GATES = 2 };
int lstm_get_cache(const lstm_buffers* buffers, int which, const void** ptr, size_t* ld, size_t* seq_len);

#ifdef __cplusplus
}  /* extern "C" */
#endif
#endif  /* FLASHLSTM_LSTM_API_H_ */
