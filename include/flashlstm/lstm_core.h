/* Device-resident LSTM forward + BPTT core for MI355X (gfx950): the C-ABI under both public
 * surfaces of this library (lstm_api.h and lstm_v2.h).
 *
 * It has no single counterpart in the reference: it is the device-side work of
 *   - lstm_forward / lstm_pack_weights               (reference src/lstm.cu:886-931, 1897-2148)
 *   - flstm::StreamingLstmForward                    (reference flashlstm_v2/src/lstm_forward.cu:464-966)
 *   - flstm::StreamingLstmBackward                   (reference flashlstm_v2/src/lstm_backward.cu:643-1250)
 * with every tensor already in HBM, so that host streaming (the v2 surface) and fp32 marshalling
 * (the v1 surface) stay outside the timed hot path.
 *
 * All pointers are device pointers unless noted; tensors are contiguous:
 *   x (T,B,I)   h0,c0,hy,cy (B,H)   y,dY (T,B,H)   W_ih (4H,I)   W_hh (4H,H)   b (4H)
 * Gate order i,f,g,o (PyTorch).  Element types are selected per argument with flstm_dtype.
 * Every function returns 0 on success, a hipError_t value on a HIP failure, or a FLSTM_E_* code.
 * A plan is not thread-safe; distinct plans are independent.  Calls are synchronous with respect
 * to `stream` (they return after the enqueued work has finished and its status was checked).
 */
#ifndef FLASHLSTM_LSTM_CORE_H_
#define FLASHLSTM_LSTM_CORE_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct flstm_core_plan flstm_core_plan;

typedef enum { FLSTM_F32 = 0, FLSTM_F16 = 1 } flstm_dtype;

enum {
    FLSTM_E_INVALID = 1,        /* same value as hipErrorInvalidValue */
    FLSTM_E_NOT_PACKED = 2001,  /* forward before weights were packed */
    FLSTM_E_NO_CACHE = 2002,    /* backward without a matching forward(save_for_backward=1) */
    FLSTM_E_STALLED = 2003,     /* recurrence kernels gave up waiting even in step-wise mode */
    FLSTM_E_TOO_LARGE = 2004    /* flstm_core_forward_static: the pass needs more scratch memory than the fixed array holds */
};

/* Creates a plan for fixed (batch, input, hidden); sequence length may vary per call. */
int flstm_core_create(size_t batch, size_t input_size, size_t hidden_size, flstm_core_plan** plan);
int flstm_core_destroy(flstm_core_plan* plan);

/* Options: "stepwise" (1 = one launch per time step instead of the persistent kernels),
 * "proj_chunk" (time steps per input-projection GEMM, <=0 = whole sequence; results do not depend
 * on it), "spin_limit" / "spin_ms" (reloads of a not-yet-written operand, and milliseconds spent on them, before a
 * waiting workgroup of a persistent launch gives up; default 2^30 reloads / 250 ms; 0 reloads = give up at the first
 * operand found unwritten), "dw_splits" (split-K slices of
 * the weight-gradient GEMM, 0 = automatic), "accumulate_grads" (1 = the backward pass adds dW_ih, dW_hh, db_ih
 * and db_hh to what the caller's buffers hold instead of overwriting them: a sequence processed as several
 * consecutive segments, last segment first, each segment's dh0 / dc0 fed to the next call as d_hn / d_cn),
 * "row_tiles_fwd" / "row_tiles_bwd" (16-row tiles per row block of that recurrence: 1, 2, or 0 = automatic),
 * "cooperative" (1: persistent launches are cooperative launches, so that co-residency of the whole grid is a
 * condition of the launch; 0: plain launches; default 1, but 0 when a rocprofiler-sdk tool is attached -- a process
 * that made a cooperative launch faults inside that tool at exit -- and FLASHLSTM_COOPERATIVE_LAUNCH overrides),
 * "step_graphs" (1, the default: where a pass runs as one launch per time step -- weights that do not fit on chip, a
 * demoted direction, "stepwise" -- the launches of a range of steps are captured into a hipGraph on first use and
 * replayed afterwards, when the stream allows capture; 0 = plain launches; FLASHLSTM_STEP_GRAPHS sets the default),
 * "bwd_two_d" (backward recurrence on a 256-CU device: the layout that splits the product over output columns and
 * over the contraction and sums partial products through a second ring, for 2048 padded hidden units and at most 128
 * batch rows or 1024 and at most 256; 0 = never, 1 = where it measured faster than the one-way layout
 * (2048 units with at most 32 or with 65..128 batch rows), 2 = wherever it can run; default 1, FLASHLSTM_BWD_TWO_D sets
 * the default),
 * "inject_stall" (test hook: the next N passes that use a persistent kernel are treated as if that launch had
 * given up, which exercises the step-wise repeat and the demotion rule without making any kernel wait). */
int flstm_core_set_option(flstm_core_plan* plan, const char* name, long value);
/* Reads back facts about the plan: "persistent_fwd", "persistent_bwd", "xcd_local_fwd", "xcd_local_bwd",
 * "fallbacks" (persistent launches that had to be redone step-wise), "demotions_fwd", "demotions_bwd" (how often a
 * direction was demoted to step-wise launches after such a give-up), "hold_fwd", "hold_bwd" (passes a demoted
 * direction still runs step-wise before the persistent kernel is tried again; 0 = not demoted), "slice_fwd", "slice_bwd" (hidden units
 * per workgroup of the recurrence kernels), "row_tiles" (16-row tiles of a 32-row batch block that the
 * recurrence fetches and multiplies: 1 for batches of at most 16 rows, else 2), "hidden_padded",
 * "input_padded", "device_bytes" (device memory the plan holds), "static_scratch_bytes" (size of the fixed scratch
 * array of flstm_core_forward_static), "num_cus" and "clock_khz" (compute units and
 * maximum engine clock of the plan's device).
 * Unknown names give -1. */
long flstm_core_get_info(const flstm_core_plan* plan, const char* name);

/* fp32 PyTorch-layout weights -> fp16 MFMA operand layouts held by the plan. */
int flstm_core_pack_weights(flstm_core_plan* plan, const float* w_ih, const float* w_hh, void* stream);
/* bias = b_ih + b_hh, kept in fp32. Either pointer may be null (treated as zeros). */
int flstm_core_pack_bias(flstm_core_plan* plan, const float* b_ih, const float* b_hh, void* stream);

/* Forward over T steps.  h0/c0 may be null (zeros).  y, hy, cy may be null (not written).
 * With save_for_backward != 0 the plan keeps the fp16 gate cache (activated i,f,g,o), the fp32
 * cell states and the fp16 outputs of this call for flstm_core_backward. */
int flstm_core_forward(flstm_core_plan* plan, size_t seq_len,
                       const void* x, flstm_dtype x_dtype,
                       const void* h0, const void* c0, flstm_dtype state_dtype,
                       void* y, flstm_dtype y_dtype,
                       void* hy, void* cy, flstm_dtype out_state_dtype,
                       int save_for_backward, void* stream);

/* flstm_core_forward for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc, the host code around a HIP graph).  It has no counterpart in the reference.  Same arguments, results
 * and kernels as flstm_core_forward with save_for_backward = 0, but everything the kernels need beyond the caller's
 * tensors and the plan's packed weights -- status word, converted x rows, x-projection / gate rows, state rows,
 * exchange ring -- lives in one fixed 64 MiB array in the library's device image instead of buffers grown by the
 * plan: the call allocates and frees nothing, also not when a persistent launch gives up and the pass is repeated
 * with one launch per step (those are plain launches here, never a captured graph).  Like flstm_core_forward it is
 * SYNCHRONOUS -- it waits for its stream and reads the status of the pass on the host -- so it cannot itself be
 * recorded into a graph that is being captured.  A pass that needs more (about T*B*(14*Hp + 2*Ip) bytes; the limit
 * is flstm_core_get_info(plan, "static_scratch_bytes")) is rejected with FLSTM_E_TOO_LARGE before any work is
 * enqueued.  Nothing is kept for a backward pass, and a cache that an earlier flstm_core_forward left in the plan
 * stays valid.  Every call on a GPU uses that GPU's one array, whichever plan it comes from: calls that overlap
 * on one GPU (two threads, two streams) race; calls on different GPUs do not.  The plan's device must be current. */
int flstm_core_forward_static(flstm_core_plan* plan, size_t seq_len,
                              const void* x, flstm_dtype x_dtype,
                              const void* h0, const void* c0, flstm_dtype state_dtype,
                              void* y, flstm_dtype y_dtype,
                              void* hy, void* cy, flstm_dtype out_state_dtype, void* stream);

/* BPTT for the last forward of this plan.  d_hn/d_cn may be null (zeros).  Any output may be null.
 * grad_scale (a power of two, 1 if <= 0) multiplies dY on load and is divided out of every
 * output; use it when dY is too small for fp16 pre-activation gradients.
 * db_ih and db_hh receive the same values. */
int flstm_core_backward(flstm_core_plan* plan, size_t seq_len,
                        const void* x, flstm_dtype x_dtype,
                        const void* dY, flstm_dtype dy_dtype,
                        const void* d_hn, const void* d_cn, flstm_dtype dstate_dtype,
                        float grad_scale,
                        void* dx, flstm_dtype dx_dtype,
                        float* dW_ih, float* dW_hh, float* db_ih, float* db_hh,
                        float* dh0, float* dc0, void* stream);

/* The same two passes fed in ranges of time steps, for callers that stream a sequence through the device
 * while it is being processed.  (No counterpart in the reference, which walks 32-step chunks inside
 * flashlstm_v2/src/lstm_forward.cu:646-940 and lstm_backward.cu:897-1213; this is the hook its replacement
 * uses to overlap host transfers with compute.)  x / dY / dx name whole-sequence device buffers; only the
 * rows of a range have to be valid (x, dY) or are written (h rows of the state cache, dx) when the range runs.
 * _steps calls only enqueue work.  forward ranges go from step 0 upwards and must cover [0, T) in order;
 * backward ranges go from step T-1 downwards.  _end waits, returns FLSTM_E_STALLED if a persistent launch
 * gave up (repeat the pass with flstm_core_forward / flstm_core_backward, which fall back to step-wise
 * launches), and otherwise finishes the pass (final states; weight and bias gradients). */
int flstm_core_forward_begin(flstm_core_plan* plan, size_t seq_len, const void* x, flstm_dtype x_dtype,
                             const void* h0, const void* c0, flstm_dtype state_dtype, void* stream);
int flstm_core_forward_steps(flstm_core_plan* plan, size_t t0, size_t nsteps, void* stream);
int flstm_core_forward_end(flstm_core_plan* plan, void* hy, void* cy, flstm_dtype out_state_dtype,
                           int save_for_backward, void* stream);
int flstm_core_backward_begin(flstm_core_plan* plan, size_t seq_len, const void* dY, flstm_dtype dy_dtype,
                              const void* d_hn, const void* d_cn, flstm_dtype dstate_dtype, float grad_scale,
                              void* dx, flstm_dtype dx_dtype, void* stream);
int flstm_core_backward_steps(flstm_core_plan* plan, size_t t_hi, size_t nsteps, void* stream);
int flstm_core_backward_end(flstm_core_plan* plan, const void* x, flstm_dtype x_dtype, float* dW_ih, float* dW_hh,
                            float* db_ih, float* db_hh, float* dh0, float* dc0, void* stream);

/* Read access to what forward cached (device pointers, valid until the next forward/destroy):
 *   which = 0: h states fp16 [(T+1)*B][Hp], row t*B+b = h before step t   (ld = *ld)
 *   which = 1: c states fp32 [(T+1)*B][Hp]
 *   which = 2: activated gates fp16 [T*B][4Hp], column 4 * unit + gate (gates i, f, g, o) */
int flstm_core_cache_ptr(const flstm_core_plan* plan, int which, const void** ptr, size_t* ld);

/* Average device time in milliseconds of the phases of the most recent forward / backward,
 * measured with events on the call's stream: names "fwd_proj", "fwd_rec", "fwd_total",
 * "bwd_rec", "bwd_dx", "bwd_dw", "bwd_total".  Negative when not available. */
double flstm_core_last_ms(const flstm_core_plan* plan, const char* phase);

/* Tuner (the counterpart of the reference's projection-chunk tuner, src/tune_projchunksz.cu:56-226, and of the
 * autotune loop of python/benchmark_lstm.py:203-301, for the launch choices that matter in this library).  For
 * sequence length seq_len it times, on synthetic data of varied values (the matrix cores run slower on those than
 * on constants) in the plan's own buffers, `repeats` passes of every candidate: 16- or 32-row blocks for each
 * recurrence (where both fit), persistent or -- with try_stepwise -- one launch per step, the layout of the
 * backward recurrence where the two-way split can run (option "bwd_two_d" 0 / 1 / 2, unless that option was set
 * explicitly), and the split-K count of the weight-gradient GEMM around the rule of thumb; the fastest choice
 * per phase is cached in the plan and used by every later pass whose length is within a factor of two of a tuned
 * one (explicit options "stepwise", "row_tiles_fwd", "row_tiles_bwd", "dw_splits" still win; option "clear_tuned"
 * forgets everything).  Read back with flstm_core_get_info: "tuned_entries", and for the entry in force for the
 * last pass "tuned_T", "tuned_row_tiles_fwd", "tuned_row_tiles_bwd", "tuned_stepwise_fwd", "tuned_stepwise_bwd",
 * "tuned_dw_splits" (0 = rule of thumb), "tuned_bwd_two_d" (-1 = not tuned); flstm_core_tuned_ms gives the best time
 * found per phase ("fwd_rec", "bwd_rec", "bwd_dw").  The plan's forward cache is invalidated.  Allocates temporary
 * device buffers. */
int flstm_core_tune(flstm_core_plan* plan, size_t seq_len, int repeats, int try_stepwise, void* stream);
double flstm_core_tuned_ms(const flstm_core_plan* plan, size_t seq_len, const char* phase);

/* The tuned entries of a plan, read out and written back: what a tuning run found can be kept by the caller (the
 * reference's tuner prints its table for exactly that reuse, src/tune_projchunksz.cu:200-226) and a fresh process
 * starts tuned.  get: entry `index` of flstm_core_get_info(plan, "tuned_entries"); any output pointer may be null.
 * set: replaces the entry of that sequence length; row_tiles 0 / 1 / 2 (0 = rule of thumb), dw_splits 0..64
 * (0 = rule of thumb), bwd_two_d -1 (not tuned) / 0 / 1 / 2.  Values that do not fit the plan's sizes are ignored by
 * the planner exactly as the corresponding options are. */
int flstm_core_get_tuned(const flstm_core_plan* plan, size_t index, size_t* seq_len, int* row_tiles_fwd, int* row_tiles_bwd,
                         int* stepwise_fwd, int* stepwise_bwd, int* dw_splits, int* bwd_two_d);
int flstm_core_set_tuned(flstm_core_plan* plan, size_t seq_len, int row_tiles_fwd, int row_tiles_bwd, int stepwise_fwd,
                         int stepwise_bwd, int dw_splits, int bwd_two_d);

/* The fp16 x fp16 -> fp32-accumulate MFMA GEMMs the passes are built from, callable on their own (the counterpart
 * of flstm::GemmTN / GemmNN / GemmNT, reference flashlstm_v2/src/gemm.h:8-51; device pointers, work is enqueued on
 * `stream` and not waited for).
 *
 * flstm_gemm_nt:  C[M][N] = alpha * A[M][K] * B[N][K]^T (+ bias[n]); A, B fp16 row-major with K contiguous (this
 *   is the input projection X * W_ih^T and, with the transposed weights, dX = dG * W_ih).  K must be a multiple
 *   of 64, lda and ldb multiples of 8 and below 2^22; C is fp16 or fp32 with any ldc >= N; bias (fp32, 16-byte aligned)
 *   may be null.
 * flstm_gemm_tn:  C[M][N] = alpha * sum_k A[k][m] * B[k][n]; A is [K][lda], B is [K][ldb] fp16 (the weight gradients
 *   dG^T * X).  M and N must be multiples of 8, K is arbitrary; A and B are 16-byte aligned, lda and ldb multiples of 8
 *   and below 2^22; C is fp32, 16-byte aligned.  splits > 1 cuts K
 *   into that many slices (at most: every slice gets whole 64-row slabs) whose partial products go to `workspace`
 *   (flstm_gemm_tn_workspace_bytes() bytes of device memory, 16-byte aligned) and are then summed into C.
 * flstm_gemm_tn_auto_splits:  the split count flstm_gemm_tn runs fastest with on a 256-CU part, at most max_splits
 *   (the rule flstm_core_backward applies to the weight gradients; a pure function of the sizes, no device needed). */
int flstm_gemm_nt(const void* A, size_t lda, const void* B, size_t ldb, size_t M, size_t N, size_t K,
                  void* C, flstm_dtype c_dtype, size_t ldc, float alpha, const float* bias, void* stream);
size_t flstm_gemm_tn_workspace_bytes(size_t M, size_t N, size_t K, int splits);
int flstm_gemm_tn_auto_splits(size_t M, size_t N, size_t K, int max_splits);
int flstm_gemm_tn(const void* A, size_t lda, const void* B, size_t ldb, size_t M, size_t N, size_t K,
                  float* C, size_t ldc, float alpha, int splits, void* workspace, void* stream);

#ifdef __cplusplus
}
#endif
#endif  /* FLASHLSTM_LSTM_CORE_H_ */
