// Layout kernels around the GEMMs and the recurrence: weight packing, dtype conversion with
// padding, transposes, and the reductions that turn scaled/padded internals into caller tensors.
#pragma once
#include "common.h"

namespace flstm_hip {

// Packed gate order of the gate arrays (x-projection / gate cache, dG) and of everything indexed like them (rows
// of the packed W_ih, bias, contraction index of the backward products): the four gates of a hidden unit are
// neighbours, q = 4 * j + gate.   PyTorch row of (gate, j) is gate*H + j.
struct Dims {
    int B, I, H;     // caller sizes
    int Ip, Hp;      // I rounded up to 64, H rounded up to 32
};

// Replaces src/kernels.cu:57-84 (pack_weights_kernel) and :45-55 (combine_bias_kernel): fp32
// PyTorch-layout weights -> the fp16 operand layouts of the kernels in this library.
hipError_t pack_weights(const Dims& d, const float* w_ih, const float* w_hh, half_t* wih_p /*[4Hp][Ip]*/,
                        half_t* wih_t /*[Ip][4Hp]*/, half8* wfrag_fwd, int ks_fwd, int nt_fwd, int rot_div_fwd, int nw_fwd,
                        half8* wfrag_bwd, int ks_bwd, int nt_bwd, int rot_div_bwd, int nw_bwd, hipStream_t s);
// W_hh in the layout of the backward recurrence that splits its product two ways (2048 padded hidden units only);
// kq = 8 or 4 contraction slices.
hipError_t pack_wfrag_bwd2d(const Dims& d, const float* w_hh, half8* out, int kq, hipStream_t s);
hipError_t pack_bias(const Dims& d, const float* b_ih, const float* b_hh, float* bias_p, hipStream_t s);

// rows x cols (ld_in, fp32 when in_f32 else fp16) -> fp16 [rows_out][ld_out], zero padded.
// Replaces src/kernels.cu:5-43 (populate_activations_kernel).
hipError_t convert_pad(const void* in, int in_f32, size_t rows, int cols, size_t ld_in, float scale,
                       half_t* out, size_t rows_out, size_t ld_out, hipStream_t s);
// fp16/fp32 (rows x cols) -> fp32 [rows][ld_out] zero padded, scaled; null input -> zeros.
hipError_t convert_pad_f32(const void* in, int in_f32, size_t rows, int cols, float scale, float* out,
                           size_t ld_out, hipStream_t s);
// padded internals -> caller tensors: out[r][c] = scale * in[r][c], c < cols.
hipError_t unpad_from_half(const half_t* in, size_t ld_in, size_t rows, int cols, void* out, int out_f32,
                           hipStream_t s);
hipError_t unpad_from_float(const float* in, size_t ld_in, size_t rows, int cols, float scale, void* out,
                            int out_f32, hipStream_t s);

// Row-block gather: output row r is input row (r / rows_per_block) * block_stride + r % rows_per_block.
// Used to pull the pre-step states at every R-th step out of the state arrays (the h/c checkpoints
// of flashlstm_v2/src/lstm_forward.cu:727-783).
hipError_t gather_from_half(const half_t* in, size_t ld_in, size_t rows, int cols, void* out, int out_f32,
                            size_t rows_per_block, size_t block_stride, hipStream_t s);
hipError_t gather_from_float(const float* in, size_t ld_in, size_t rows, int cols, float scale, void* out,
                             int out_f32, size_t rows_per_block, size_t block_stride, hipStream_t s);

// out[c][r] = in[r][c] for r < rows, c < cols; out rows are ld_out long, columns [rows, ld_out) are
// zeroed; output rows [cols, cols_out) are zeroed as well.
hipError_t transpose_pad(const void* in, int in_f32, size_t rows, int cols, size_t ld_in, half_t* out,
                         int cols_out, size_t ld_out, hipStream_t s);

// Sums columns [col0, col0 + ncols) of the split-K partials [splits][4Hp][ld] (packed gate rows) into dst
// [4H][out_cols] (PyTorch row order, the first out_cols of those columns), times `scale`; `accumulate` adds to dst
// instead of overwriting it (the beta=1 accumulation over chunks of flashlstm_v2/src/lstm_backward.cu:1112-1142).
hipError_t reduce_dw(const Dims& d, const float* partial, int splits, size_t ld, int col0, int ncols, int out_cols,
                     float scale, bool accumulate, float* dst, hipStream_t s);
// db_part [ng][4Hp] packed -> db_ih == db_hh (4H), times scale (flashlstm_v2/src/lstm_backward.cu:1218-1231).
hipError_t reduce_db(const Dims& d, const float* db_part, int ng, float scale, bool accumulate, float* db_ih,
                     float* db_hh, hipStream_t s);

// dst[r][c] (pitch ldc) = sum over z < splits of partial[z * per + r * cols + c]: split-K partials of a plain GEMM.
hipError_t reduce_partials(const float* partial, int splits, size_t per, int rows, int cols, size_t ldc, float* dst,
                           hipStream_t s);

// *out += a position-weighted 64-bit sum over the 16-bit units of a device buffer (`salt` tells buffers apart when
// several are folded into one sum); null or empty buffers add nothing.  Evidence that device tensors still hold what
// an earlier call saw.
hipError_t checksum_add(const void* p, size_t bytes, u64 salt, u64* out, hipStream_t s);

hipError_t fill_zero(void* p, size_t bytes, hipStream_t s);

// Up to ten of the small operations above in ONE launch: a pass starts with half a dozen of them (state rows, rings,
// counters), each a few microseconds of kernel plus a launch gap of its own when issued one by one.
struct PrepOp {
    enum Kind : int { kNone = 0, kFill = 1, kToHalf = 2, kToFloat = 3, kUnpad = 4 };
    int kind = kNone;
    int in_f32 = 0, out_f32 = 0;
    void* dst = nullptr;
    const void* src = nullptr;   // kToHalf / kToFloat: null reads as zeros
    size_t n = 0;                // kFill: 32-bit words; kToHalf / kToFloat: rows_out * ld_out elements; kUnpad: rows * cols
    unsigned word = 0;           // kFill
    size_t rows = 0, ld_in = 0, ld_out = 1;
    int cols = 0;
    float scale = 1.f;
};
struct PrepList {
    int count = 0;
    PrepOp op[10];
    void fill(void* p, size_t bytes, unsigned word) {
        if (bytes == 0) return;
        PrepOp& o = op[count++];
        o.kind = PrepOp::kFill; o.dst = p; o.n = bytes / 4; o.word = word;
    }
    // the operations of convert_pad() and convert_pad_f32()
    void to_half(const void* in, int in_f32, size_t rows, int cols, size_t ld_in, float scale, half_t* out, size_t rows_out, size_t ld_out) {
        if (rows_out * ld_out == 0) return;
        PrepOp& o = op[count++];
        o.kind = PrepOp::kToHalf; o.in_f32 = in_f32; o.dst = out; o.src = in; o.n = rows_out * ld_out;
        o.rows = rows; o.cols = cols; o.ld_in = ld_in; o.ld_out = ld_out; o.scale = scale;
    }
    void to_float(const void* in, int in_f32, size_t rows, int cols, float scale, float* out, size_t ld_out) {
        if (rows * ld_out == 0) return;
        PrepOp& o = op[count++];
        o.kind = PrepOp::kToFloat; o.in_f32 = in_f32; o.dst = out; o.src = in; o.n = rows * ld_out;
        o.rows = rows; o.cols = cols; o.ld_in = size_t(cols); o.ld_out = ld_out; o.scale = scale;
    }
    // the operation of unpad_from_half() / unpad_from_float(): out[r][c] = scale * in[r][c], c < cols; a null `out` adds nothing
    void unpad(const void* in, int in_f32, size_t ld_in, size_t rows, int cols, float scale, void* out, int out_f32) {
        if (out == nullptr || rows * size_t(cols) == 0) return;
        PrepOp& o = op[count++];
        o.kind = PrepOp::kUnpad; o.in_f32 = in_f32; o.out_f32 = out_f32; o.dst = out; o.src = in; o.n = rows * size_t(cols);
        o.rows = rows; o.cols = cols; o.ld_in = ld_in; o.ld_out = size_t(cols); o.scale = scale;
    }
};
hipError_t run_prep(const PrepList& list, hipStream_t s);
// fp16 values spread over (-amp, amp) from a hash of the index (operands for timing runs)
hipError_t fill_noise(half_t* p, size_t n, unsigned seed, float amp, hipStream_t s);
// Fills a buffer (multiple of 4 bytes) with one 32-bit pattern; a kernel, so it may be captured in a graph.
hipError_t fill_words(void* p, size_t bytes, unsigned value, hipStream_t s);

}  // namespace flstm_hip
