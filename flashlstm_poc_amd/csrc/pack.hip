// Layout kernels: weight packing, padded dtype conversion, transposes and output reductions.
// All are pure HBM-bandwidth work; each thread moves a few elements with coalesced accesses.
#include "pack.h"
#include "recurrent.h"

namespace flstm_hip {
namespace {

constexpr int kT = 256;

__host__ __device__ inline int grid_for(size_t n) { return int((n + kT - 1) / kT); }

// Column q of the gate arrays (x-projection / gate cache, dG, and with them the rows of the packed W_ih, the bias
// and the contraction index of the backward products) -> PyTorch weight row, or -1 for a padding unit.  The four
// gates of a hidden unit are neighbours, q = 4 * unit + gate, so a thread that owns a few consecutive units moves
// all of their gate values with one 16-byte access.
__device__ __forceinline__ int torch_row(int q, int H) {
    const int j = q / 4, gate = q % 4;
    return j < H ? gate * H + j : -1;
}

__global__ void pack_wih_kernel(Dims d, const float* __restrict__ w_ih, half_t* __restrict__ wih_p,
                                half_t* __restrict__ wih_t) {
    const size_t idx = size_t(blockIdx.x) * kT + threadIdx.x;
    const size_t total = size_t(4) * d.Hp * d.Ip;
    if (idx >= total) return;
    const int q = int(idx / d.Ip), i = int(idx % d.Ip);
    const int row = torch_row(q, d.H);
    const float v = (row >= 0 && i < d.I) ? w_ih[size_t(row) * d.I + i] : 0.f;
    wih_p[idx] = (half_t)v;
    wih_t[size_t(i) * 4 * d.Hp + q] = (half_t)v;
}

// Forward fragments: B operand of  gates[b][c] += h[b][k] * W_hh[row(c)][k].  The product's columns are local to
// a workgroup (they only meet the pointwise stage through LDS) and stay gate-major within the slice of JB = 4*NT
// units: column c = gate * JB + unit.  With eight waves per workgroup (rec_fwd_il_kernel) they are unit-major,
// column c = 4 * unit + gate: the four accumulation registers of a lane are then the four gates of one unit.
// fragment (hs, wave, ks, n): lane l holds column c = n*16 + l%16 of slice hs,
// k = (ks*nw + wave)*32 + 8*(l/16) + e, e = 0..7 (nw = wavefronts per workgroup, 4 or 8).
__global__ void pack_wfrag_fwd_kernel(Dims d, const float* __restrict__ w_hh, half_t* __restrict__ out,
                                      int ks_wave, int nt, int rot_div, int nw) {
    const size_t idx = size_t(blockIdx.x) * kT + threadIdx.x;  // one half element
    const int nh = d.Hp / (4 * nt);
    const size_t total = size_t(nh) * nw * ks_wave * nt * kWave * 8;
    if (idx >= total) return;
    size_t r = idx;
    const int e = int(r % 8); r /= 8;
    const int lane = int(r % kWave); r /= kWave;
    const int n = int(r % nt); r /= nt;
    const int ks = int(r % ks_wave); r /= ks_wave;
    const int wave = int(r % nw); r /= nw;
    const int hs = int(r);
    const int jb = 4 * nt, c = n * 16 + lane % 16;
    const int gate = (nw == 8) ? c % 4 : c / jb, unit = hs * jb + ((nw == 8) ? c / 4 : c % jb);
    // (slot ks of slice hs holds a rotated k-step: recurrent.h, rec_kstep_rotation)
    const int kstep = rec_kstep_of_slot(ks, rec_kstep_rotation(hs, nh, ks_wave, rot_div), ks_wave);
    const int k = (kstep * nw + wave) * 32 + 8 * (lane / 16) + e;
    out[idx] = (half_t)((unit < d.H && k < d.H) ? w_hh[size_t(gate * d.H + unit) * d.H + k] : 0.f);
}

// Backward fragments: B operand of  dh[b][k] += dG[b][q] * W_hh[row(q)][k].
// fragment (hs, wave, ks, n): lane l holds output column k = hs*16*NT + n*16 + l%16,
// contraction index q = (ks*nw + wave)*32 + 8*(l/16) + e.
__global__ void pack_wfrag_bwd_kernel(Dims d, const float* __restrict__ w_hh, half_t* __restrict__ out,
                                      int ks_wave, int nt, int rot_div, int nw) {
    const size_t idx = size_t(blockIdx.x) * kT + threadIdx.x;
    const int nh = d.Hp / (16 * nt);
    const size_t total = size_t(nh) * nw * ks_wave * nt * kWave * 8;
    if (idx >= total) return;
    size_t r = idx;
    const int e = int(r % 8); r /= 8;
    const int lane = int(r % kWave); r /= kWave;
    const int n = int(r % nt); r /= nt;
    const int ks = int(r % ks_wave); r /= ks_wave;
    const int wave = int(r % nw); r /= nw;
    const int hs = int(r);
    const int k = hs * 16 * nt + n * 16 + lane % 16;
    const int kstep = rec_kstep_of_slot(ks, rec_kstep_rotation(hs, nh, ks_wave, rot_div), ks_wave);
    const int q = (kstep * nw + wave) * 32 + 8 * (lane / 16) + e;
    float v = 0.f;
    if (q < 4 * d.Hp && k < d.H) {
        const int row = torch_row(q, d.H);
        if (row >= 0) v = w_hh[size_t(row) * d.H + k];
    }
    out[idx] = (half_t)v;
}

// Two-dimensional backward layout: [Hp / 64 column slices s][kq contraction slices q][4 waves][ks k-steps][4 tiles][64 lanes][8],
// ks = Hp / (32 kq): lane l of tile n holds column 64 s + 16 n + l % 16 of W_hh (hidden unit k of dh = dG * W_hh^T-packed)
// and the eight packed gate rows (4 Hp / kq) q + 32 (4 ks + wave) + 8 (l / 16) .. +7.
__global__ void pack_wfrag_bwd2d_kernel(Dims d, const float* __restrict__ w_hh, half_t* __restrict__ out, int kq) {
    const size_t idx = size_t(blockIdx.x) * kT + threadIdx.x;
    const size_t total = size_t(4) * d.Hp * d.Hp;
    if (idx >= total) return;
    const int ksn = d.Hp / (32 * kq);   // k-steps per wave: 4 waves * ksn * 32 = 4 Hp / kq packed gate rows
    size_t r = idx;
    const int e = int(r % 8); r /= 8;
    const int lane = int(r % kWave); r /= kWave;
    const int n = int(r % 4); r /= 4;
    const int ks = int(r % ksn); r /= ksn;
    const int wave = int(r % 4); r /= 4;
    const int qs = int(r % kq); r /= kq;
    const int sl = int(r);
    const int k = sl * 64 + n * 16 + lane % 16;
    // (slot ks of a wave holds the k-step the kernel fetches there: rotated per column slice)
    const int kstep = rec_kstep_of_slot(ks, rec_bwd2d_rotation(sl, ksn, kq), ksn);
    const int q = qs * (4 * d.Hp / kq) + (kstep * 4 + wave) * 32 + 8 * (lane / 16) + e;
    float v = 0.f;
    if (q < 4 * d.Hp && k < d.H) {
        const int row = torch_row(q, d.H);
        if (row >= 0) v = w_hh[size_t(row) * d.H + k];
    }
    out[idx] = (half_t)v;
}

__global__ void pack_bias_kernel(Dims d, const float* __restrict__ b_ih, const float* __restrict__ b_hh,
                                 float* __restrict__ out) {
    const int q = blockIdx.x * kT + threadIdx.x;
    if (q >= 4 * d.Hp) return;
    const int row = torch_row(q, d.H);
    out[q] = row >= 0 ? b_ih[row] + b_hh[row] : 0.f;
}

template <typename TIn>
__global__ void convert_pad_kernel(const TIn* __restrict__ in, size_t rows, int cols, size_t ld_in,
                                   float scale, half_t* __restrict__ out, size_t rows_out, size_t ld_out) {
    const size_t idx = size_t(blockIdx.x) * kT + threadIdx.x;
    if (idx >= rows_out * ld_out) return;
    const size_t r = idx / ld_out;
    const int c = int(idx % ld_out);
    float v = 0.f;
    if (r < rows && c < cols) v = scale * (float)in[r * ld_in + c];
    out[idx] = (half_t)v;
}

template <typename TIn>
__global__ void convert_pad_f32_kernel(const TIn* __restrict__ in, size_t rows, int cols, float scale,
                                       float* __restrict__ out, size_t ld_out) {
    const size_t idx = size_t(blockIdx.x) * kT + threadIdx.x;
    if (idx >= rows * ld_out) return;
    const size_t r = idx / ld_out;
    const int c = int(idx % ld_out);
    float v = 0.f;
    if (in != nullptr && c < cols) v = scale * (float)in[r * cols + c];
    out[idx] = v;
}

// Output row r comes from input row (r / rows_per_block) * block_stride + r % rows_per_block.
template <typename TIn, typename TOut>
__global__ void unpad_kernel(const TIn* __restrict__ in, size_t ld_in, size_t rows, int cols, float scale,
                             TOut* __restrict__ out, size_t rows_per_block, size_t block_stride) {
    const size_t idx = size_t(blockIdx.x) * kT + threadIdx.x;
    if (idx >= rows * size_t(cols)) return;
    const size_t r = idx / cols;
    const int c = int(idx % cols);
    const size_t rin = (r / rows_per_block) * block_stride + r % rows_per_block;
    out[idx] = (TOut)(scale * (float)in[rin * ld_in + c]);
}

// 64x64 tile transpose through LDS.
template <typename TIn>
__global__ void transpose_pad_kernel(const TIn* __restrict__ in, size_t rows, int cols, size_t ld_in,
                                     half_t* __restrict__ out, int cols_out, size_t ld_out) {
    __shared__ half_t tile[64][66];
    const size_t r0 = size_t(blockIdx.x) * 64;
    const int c0 = blockIdx.y * 64;
    const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;  // 4 rows of 64 threads
    for (int i = ty; i < 64; i += 4) {
        const size_t r = r0 + i;
        const int c = c0 + tx;
        float v = 0.f;
        if (r < rows && c < cols) v = (float)in[r * ld_in + c];
        tile[i][tx] = (half_t)v;
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
        const int c = c0 + i;       // output row
        const size_t r = r0 + tx;   // output column
        if (c < cols_out && r < ld_out) out[size_t(c) * ld_out + r] = tile[tx][i];
    }
}

// columns [col0, col0 + ncols) of partial [splits][4Hp][ld] with packed gate rows -> dst [4H][out_cols] in PyTorch
// row order
__global__ void reduce_dw_kernel(Dims d, const float* __restrict__ partial, int splits, size_t ld, int col0, int ncols,
                                 int out_cols, float scale, int accumulate, float* __restrict__ dst) {
    const size_t idx = size_t(blockIdx.x) * kT + threadIdx.x;
    if (idx >= size_t(4) * d.Hp * ncols) return;
    const int q = int(idx / ncols), n = int(idx % ncols);
    const int row = torch_row(q, d.H);
    if (row < 0 || n >= out_cols) return;
    const size_t per = size_t(4) * d.Hp * ld, src = size_t(q) * ld + col0 + n;
    float s = 0.f;
    for (int z = 0; z < splits; ++z) s += partial[size_t(z) * per + src];
    float* out = dst + size_t(row) * out_cols + n;
    *out = accumulate ? *out + scale * s : scale * s;
}

__global__ void reduce_db_kernel(Dims d, const float* __restrict__ db_part, int ng, float scale, int accumulate,
                                 float* __restrict__ db_ih, float* __restrict__ db_hh) {
    const int q = blockIdx.x * kT + threadIdx.x;
    if (q >= 4 * d.Hp) return;
    const int row = torch_row(q, d.H);
    if (row < 0) return;
    float s = 0.f;
    for (int g = 0; g < ng; ++g) s += db_part[size_t(g) * 4 * d.Hp + q];
    s *= scale;
    if (db_ih) db_ih[row] = accumulate ? db_ih[row] + s : s;
    if (db_hh && db_hh != db_ih) db_hh[row] = accumulate ? db_hh[row] + s : s;
}

// flat 16-byte copy (both ends 16-byte aligned, n16 chunks)
__global__ void copy16_kernel(const uint4* __restrict__ in, uint4* __restrict__ out, size_t n16) {
    const size_t stride = size_t(gridDim.x) * kT;
    for (size_t i = size_t(blockIdx.x) * kT + threadIdx.x; i < n16; i += stride) out[i] = in[i];
}

__global__ void fill_words_kernel(unsigned* p, size_t words, unsigned value) {
    const size_t stride = size_t(gridDim.x) * kT;
    for (size_t i = size_t(blockIdx.x) * kT + threadIdx.x; i < words; i += stride) p[i] = value;
}

// blockIdx.y selects the operation, the blocks of a row walk it with a grid stride
__global__ void prep_kernel(PrepList list) {
    const PrepOp& o = list.op[blockIdx.y];
    const size_t stride = size_t(gridDim.x) * kT;
    const size_t first = size_t(blockIdx.x) * kT + threadIdx.x;
    if (o.kind == PrepOp::kFill) {
        unsigned* p = static_cast<unsigned*>(o.dst);
        for (size_t i = first; i < o.n; i += stride) p[i] = o.word;
    } else if (o.kind == PrepOp::kToHalf || o.kind == PrepOp::kToFloat) {
        for (size_t i = first; i < o.n; i += stride) {
            const size_t r = i / o.ld_out;
            const int c = int(i % o.ld_out);
            float v = 0.f;
            if (o.src != nullptr && r < o.rows && c < o.cols) {
                const size_t at = r * o.ld_in + c;
                v = o.scale * (o.in_f32 ? static_cast<const float*>(o.src)[at] : (float)static_cast<const half_t*>(o.src)[at]);
            }
            if (o.kind == PrepOp::kToHalf) static_cast<half_t*>(o.dst)[i] = (half_t)v;
            else static_cast<float*>(o.dst)[i] = v;
        }
    } else if (o.kind == PrepOp::kUnpad) {
        for (size_t i = first; i < o.n; i += stride) {
            const size_t at = (i / o.cols) * o.ld_in + i % o.cols;
            const float v = o.scale * (o.in_f32 ? static_cast<const float*>(o.src)[at] : (float)static_cast<const half_t*>(o.src)[at]);
            if (o.out_f32) static_cast<float*>(o.dst)[i] = v;
            else static_cast<half_t*>(o.dst)[i] = (half_t)v;
        }
    }
}

}  // namespace

hipError_t pack_weights(const Dims& d, const float* w_ih, const float* w_hh, half_t* wih_p, half_t* wih_t,
                        half8* wfrag_fwd, int ks_fwd, int nt_fwd, int rot_div_fwd, int nw_fwd, half8* wfrag_bwd, int ks_bwd,
                        int nt_bwd, int rot_div_bwd, int nw_bwd, hipStream_t s) {
    const size_t n1 = size_t(4) * d.Hp * d.Ip;
    hipLaunchKernelGGL(pack_wih_kernel, dim3(grid_for(n1)), dim3(kT), 0, s, d, w_ih, wih_p, wih_t);
    const size_t n2 = size_t(d.Hp / (4 * nt_fwd)) * nw_fwd * ks_fwd * nt_fwd * kWave * 8;
    hipLaunchKernelGGL(pack_wfrag_fwd_kernel, dim3(grid_for(n2)), dim3(kT), 0, s, d, w_hh,
                       reinterpret_cast<half_t*>(wfrag_fwd), ks_fwd, nt_fwd, rot_div_fwd, nw_fwd);
    const size_t n3 = size_t(d.Hp / (16 * nt_bwd)) * nw_bwd * ks_bwd * nt_bwd * kWave * 8;
    hipLaunchKernelGGL(pack_wfrag_bwd_kernel, dim3(grid_for(n3)), dim3(kT), 0, s, d, w_hh,
                       reinterpret_cast<half_t*>(wfrag_bwd), ks_bwd, nt_bwd, rot_div_bwd, nw_bwd);
    return hipGetLastError();
}

hipError_t pack_wfrag_bwd2d(const Dims& d, const float* w_hh, half8* out, int kq, hipStream_t s) {
    // Hp / 64 slices of 64 columns, kq slices of 4 Hp / kq packed gate rows, 8 or 16 k-steps per wave
    if (!((d.Hp == 2048 && (kq == 4 || kq == 8)) || (d.Hp == 1024 && kq == 2))) return hipErrorInvalidValue;
    const size_t n = size_t(4) * d.Hp * d.Hp;
    hipLaunchKernelGGL(pack_wfrag_bwd2d_kernel, dim3(grid_for(n)), dim3(kT), 0, s, d, w_hh, reinterpret_cast<half_t*>(out), kq);
    return hipGetLastError();
}

hipError_t pack_bias(const Dims& d, const float* b_ih, const float* b_hh, float* bias_p, hipStream_t s) {
    hipLaunchKernelGGL(pack_bias_kernel, dim3(grid_for(size_t(4) * d.Hp)), dim3(kT), 0, s, d, b_ih, b_hh, bias_p);
    return hipGetLastError();
}

hipError_t convert_pad(const void* in, int in_f32, size_t rows, int cols, size_t ld_in, float scale,
                       half_t* out, size_t rows_out, size_t ld_out, hipStream_t s) {
    const size_t n = rows_out * ld_out;
    if (n == 0) return hipSuccess;
    if (in_f32)
        hipLaunchKernelGGL(convert_pad_kernel<float>, dim3(grid_for(n)), dim3(kT), 0, s,
                           static_cast<const float*>(in), rows, cols, ld_in, scale, out, rows_out, ld_out);
    else
        hipLaunchKernelGGL(convert_pad_kernel<half_t>, dim3(grid_for(n)), dim3(kT), 0, s,
                           static_cast<const half_t*>(in), rows, cols, ld_in, scale, out, rows_out, ld_out);
    return hipGetLastError();
}

hipError_t convert_pad_f32(const void* in, int in_f32, size_t rows, int cols, float scale, float* out,
                           size_t ld_out, hipStream_t s) {
    const size_t n = rows * ld_out;
    if (n == 0) return hipSuccess;
    if (in_f32)
        hipLaunchKernelGGL(convert_pad_f32_kernel<float>, dim3(grid_for(n)), dim3(kT), 0, s,
                           static_cast<const float*>(in), rows, cols, scale, out, ld_out);
    else
        hipLaunchKernelGGL(convert_pad_f32_kernel<half_t>, dim3(grid_for(n)), dim3(kT), 0, s,
                           static_cast<const half_t*>(in), rows, cols, scale, out, ld_out);
    return hipGetLastError();
}

hipError_t gather_from_half(const half_t* in, size_t ld_in, size_t rows, int cols, void* out, int out_f32,
                            size_t rows_per_block, size_t block_stride, hipStream_t s) {
    const size_t n = rows * size_t(cols);
    if (n == 0 || out == nullptr) return hipSuccess;
    // unpadded fp16 rows that are contiguous on both sides: a flat vector copy
    if (!out_f32 && size_t(cols) == ld_in && rows_per_block >= rows && (n * sizeof(half_t)) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
        const size_t n16 = n * sizeof(half_t) / 16;
        size_t blocks = (n16 + kT - 1) / kT;
        if (blocks > 8192) blocks = 8192;
        hipLaunchKernelGGL(copy16_kernel, dim3(unsigned(blocks)), dim3(kT), 0, s, reinterpret_cast<const uint4*>(in),
                           static_cast<uint4*>(out), n16);
        return hipGetLastError();
    }
    if (out_f32)
        hipLaunchKernelGGL((unpad_kernel<half_t, float>), dim3(grid_for(n)), dim3(kT), 0, s, in, ld_in, rows,
                           cols, 1.f, static_cast<float*>(out), rows_per_block, block_stride);
    else
        hipLaunchKernelGGL((unpad_kernel<half_t, half_t>), dim3(grid_for(n)), dim3(kT), 0, s, in, ld_in, rows,
                           cols, 1.f, static_cast<half_t*>(out), rows_per_block, block_stride);
    return hipGetLastError();
}

hipError_t gather_from_float(const float* in, size_t ld_in, size_t rows, int cols, float scale, void* out,
                             int out_f32, size_t rows_per_block, size_t block_stride, hipStream_t s) {
    const size_t n = rows * size_t(cols);
    if (n == 0 || out == nullptr) return hipSuccess;
    if (out_f32)
        hipLaunchKernelGGL((unpad_kernel<float, float>), dim3(grid_for(n)), dim3(kT), 0, s, in, ld_in, rows,
                           cols, scale, static_cast<float*>(out), rows_per_block, block_stride);
    else
        hipLaunchKernelGGL((unpad_kernel<float, half_t>), dim3(grid_for(n)), dim3(kT), 0, s, in, ld_in, rows,
                           cols, scale, static_cast<half_t*>(out), rows_per_block, block_stride);
    return hipGetLastError();
}

hipError_t unpad_from_half(const half_t* in, size_t ld_in, size_t rows, int cols, void* out, int out_f32,
                           hipStream_t s) {
    return gather_from_half(in, ld_in, rows, cols, out, out_f32, rows ? rows : 1, 0, s);
}

hipError_t unpad_from_float(const float* in, size_t ld_in, size_t rows, int cols, float scale, void* out,
                            int out_f32, hipStream_t s) {
    return gather_from_float(in, ld_in, rows, cols, scale, out, out_f32, rows ? rows : 1, 0, s);
}

hipError_t transpose_pad(const void* in, int in_f32, size_t rows, int cols, size_t ld_in, half_t* out,
                         int cols_out, size_t ld_out, hipStream_t s) {
    if (cols_out == 0 || ld_out == 0) return hipSuccess;
    dim3 grid(unsigned(ceil_div(ld_out, 64)), unsigned(ceil_div(size_t(cols_out), 64)));
    if (in_f32)
        hipLaunchKernelGGL(transpose_pad_kernel<float>, grid, dim3(kT), 0, s, static_cast<const float*>(in),
                           rows, cols, ld_in, out, cols_out, ld_out);
    else
        hipLaunchKernelGGL(transpose_pad_kernel<half_t>, grid, dim3(kT), 0, s, static_cast<const half_t*>(in),
                           rows, cols, ld_in, out, cols_out, ld_out);
    return hipGetLastError();
}

hipError_t reduce_dw(const Dims& d, const float* partial, int splits, size_t ld, int col0, int ncols, int out_cols,
                     float scale, bool accumulate, float* dst, hipStream_t s) {
    if (dst == nullptr) return hipSuccess;
    const size_t n = size_t(4) * d.Hp * ncols;
    hipLaunchKernelGGL(reduce_dw_kernel, dim3(grid_for(n)), dim3(kT), 0, s, d, partial, splits, ld, col0, ncols,
                       out_cols, scale, int(accumulate), dst);
    return hipGetLastError();
}

hipError_t reduce_db(const Dims& d, const float* db_part, int ng, float scale, bool accumulate, float* db_ih,
                     float* db_hh, hipStream_t s) {
    hipLaunchKernelGGL(reduce_db_kernel, dim3(grid_for(size_t(4) * d.Hp)), dim3(kT), 0, s, d, db_part, ng,
                       scale, int(accumulate), db_ih, db_hh);
    return hipGetLastError();
}

__global__ void reduce_partials_kernel(const float* __restrict__ partial, int splits, size_t per, int rows, int cols,
                                       size_t ldc, float* __restrict__ dst) {
    const size_t idx = size_t(blockIdx.x) * kT + threadIdx.x;
    if (idx >= size_t(rows) * cols) return;
    float s = 0.f;
    for (int z = 0; z < splits; ++z) s += partial[size_t(z) * per + idx];
    dst[(idx / cols) * ldc + idx % cols] = s;
}

hipError_t reduce_partials(const float* partial, int splits, size_t per, int rows, int cols, size_t ldc, float* dst,
                           hipStream_t s) {
    if (rows <= 0 || cols <= 0) return hipSuccess;
    hipLaunchKernelGGL(reduce_partials_kernel, dim3(grid_for(size_t(rows) * cols)), dim3(kT), 0, s, partial, splits, per,
                       rows, cols, ldc, dst);
    return hipGetLastError();
}

// Position-weighted sum of the 16-bit units of a buffer, added to *out: any changed, moved or swapped element
// changes the sum (up to a 2^-64 accident); the order of the additions does not matter, so atomics may be used.
__global__ void checksum_kernel(const unsigned short* __restrict__ p, size_t n, u64 salt, u64* out) {
    u64 acc = 0;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        u64 v = (u64(p[i]) + 1u) * (2 * (i + salt) + 1) * 0x9E3779B97F4A7C15ull;
        v ^= v >> 29;
        acc += v * 0xBF58476D1CE4E5B9ull;
    }
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    if (threadIdx.x % 64 == 0 && acc != 0) atomicAdd(reinterpret_cast<unsigned long long*>(out), acc);
}

hipError_t checksum_add(const void* p, size_t bytes, u64 salt, u64* out, hipStream_t s) {
    if (p == nullptr || bytes < 2) return hipSuccess;
    const size_t n = bytes / 2;   // every tensor of this library is made of 2- or 4-byte elements
    int blocks = grid_for(n);
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(checksum_kernel, dim3(blocks), dim3(kT), 0, s, static_cast<const unsigned short*>(p), n, salt, out);
    return hipGetLastError();
}

hipError_t fill_words(void* p, size_t bytes, unsigned value, hipStream_t s) {
    if (bytes == 0) return hipSuccess;
    const size_t words = bytes / 4;  // all buffers of this library are multiples of 4 bytes
    int blocks = grid_for(words);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_words_kernel, dim3(blocks), dim3(kT), 0, s, static_cast<unsigned*>(p), words, value);
    return hipGetLastError();
}

hipError_t run_prep(const PrepList& list, hipStream_t s) {
    if (list.count <= 0) return hipSuccess;
    size_t most = 0;
    for (int i = 0; i < list.count; ++i) most = list.op[i].n > most ? list.op[i].n : most;
    size_t blocks = (most + kT - 1) / kT;
    if (blocks > 256) blocks = 256;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(prep_kernel, dim3(unsigned(blocks), unsigned(list.count)), dim3(kT), 0, s, list);
    return hipGetLastError();
}

hipError_t fill_zero(void* p, size_t bytes, hipStream_t s) { return fill_words(p, bytes, 0u, s); }

// n fp16 values spread over (-amp, amp) from a hash of the index: operands for timing runs (the matrix cores draw
// more power, and run slower, on varied operands than on constant ones)
__global__ void fill_noise_kernel(half_t* p, size_t n, unsigned seed, float amp) {
    const size_t stride = size_t(gridDim.x) * kT;
    for (size_t i = size_t(blockIdx.x) * kT + threadIdx.x; i < n; i += stride) {
        unsigned h = unsigned(i) * 0x9E3779B1u + unsigned(i >> 32) * 0x85EBCA77u + seed;
        h ^= h >> 15; h *= 0x2C1B3C6Du; h ^= h >> 12; h *= 0x297A2D39u; h ^= h >> 15;
        p[i] = (half_t)(amp * (float(h >> 8) * (2.f / 16777216.f) - 1.f));
    }
}

hipError_t fill_noise(half_t* p, size_t n, unsigned seed, float amp, hipStream_t s) {
    if (n == 0) return hipSuccess;
    int blocks = grid_for(n);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_noise_kernel, dim3(blocks), dim3(kT), 0, s, p, n, seed, amp);
    return hipGetLastError();
}

}  // namespace flstm_hip
