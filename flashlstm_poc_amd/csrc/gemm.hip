// LDS-staged fp16 MFMA GEMM for gfx950 (CDNA4), NT form: C[M][N] = A[M][K] * B[N][K]^T.
//
// This is the dense contraction behind the hoisted input projection X*W_ih^T (the reference does it
// with a CUTLASS 128x128x32 tensor-op GEMM, src/lstm.cu:1204-1239, src/lstm_internal.h:48-68), the
// input gradient dX = dG*W_ih and the weight gradients dW = dG^T*[X;H] (reference:
// flashlstm_v2/src/lstm_backward.cu:1112-1172 through flashlstm_v2/src/gemm.cu:222-330).
//
// Tiling: one 256-thread workgroup (4 wavefronts, 2x2, one per SIMD) owns a 256x256 tile of C; every
// wavefront owns 128x128 as a 4x4 grid of v_mfma_f32_32x32x16_f16 tiles (256 accumulator registers).
// K is walked in slabs of 64: global -> registers -> LDS (row pitch padded to 72 halfs so that the
// 16-byte fragment reads of 8 consecutive lanes fall in distinct banks), double buffered, one
// workgroup barrier per slab.  The MFMA operands are swapped (D = B_tile * A_tile^T) so that a lane ends
// up with four consecutive columns of one row of C and stores them as one 8- or 16-byte access.
// Workgroups are numbered so that the 32 that share an XCD (block id mod 8) work on neighbouring tiles
// and reuse each other's operand slabs in that XCD's L2.
#include "gemm.h"

namespace flstm_hip {
namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int LDS_LD = 72;  // halfs per LDS row (64 + 8 pad)
constexpr int kWavesN = 4;                 // wavefronts along N (2 along M): wave tile 128 x (256 / kWavesN)
constexpr int kThreads = 128 * kWavesN;
constexpr int kTN = 8 / kWavesN;            // 32-wide MFMA tiles per wave along N
constexpr int kLd = 2048 / kThreads;        // 16-byte chunks per thread, operand and slab
constexpr size_t kLdsBytes = size_t(2) * (BM + BN) * LDS_LD * sizeof(half_t);

// Work list: items are (K-split z, tile) pairs ordered z-major, tiles row-major.  The hardware deals
// workgroups round-robin over the 8 XCDs in dispatch order (x fastest), so the 32 workgroups that run
// together on one XCD are given 32 CONSECUTIVE items: one K range and a compact block of tiles, whose
// operand slabs they then share through that XCD's L2.
__device__ __forceinline__ bool work_item(int tiles_m, int tiles_n, int splits, int& tm, int& tn, int& z) {
    const int ntiles = tiles_m * tiles_n;
    const int items = ntiles * splits;
    const int lin = blockIdx.y * gridDim.x + blockIdx.x;   // dispatch order
    const int xcd = lin % 8, s = lin / 8;
    const int item = ((s / 32) * 8 + xcd) * 32 + s % 32;
    if (item >= items) return false;
    z = item / ntiles;
    const int tile = item % ntiles;
    tm = tile / tiles_n;
    tn = tile % tiles_n;
    return true;
}

// Epilogue shared by both kernels.  With swapped MFMA operands register r of tile (i, j) holds row
// (i*32 + lane%32) of the wave's 128 x 64 block and column j*32 + 8*(r/4) + 4*(lane/32) + r%4: four
// consecutive columns per group of four registers, stored as one 8-byte (fp16) or 16-byte (fp32) access.
__device__ __forceinline__ void store_tile(const GemmNT& g, floatx16 (&acc)[4][kTN], int m0, int n0, int wm,
                                           int wn, int lane, int z) {
    const int row = m0 + wm * 128 + lane % 32;
    const int colb = n0 + wn * 32 * kTN + 4 * (lane / 32);
    float* c32 = g.C32 ? g.C32 + size_t(z) * g.split_stride : nullptr;
    const bool full = (m0 + BM <= g.M) && (n0 + BN <= g.N) && (g.ldc % 4 == 0);
    if (full) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const size_t rowoff = size_t(row + i * 32) * g.ldc + colb;
#pragma unroll
            for (int j = 0; j < kTN; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const size_t off = rowoff + j * 32 + 8 * q;
                    if (c32) {
                        floatx4 v;
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = g.alpha * acc[i][j][4 * q + e];
                        *reinterpret_cast<floatx4*>(c32 + off) = v;
                    } else {
                        half4 v;
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = (half_t)(g.alpha * acc[i][j][4 * q + e]);
                        *reinterpret_cast<half4*>(g.C16 + off) = v;
                    }
                }
                __builtin_amdgcn_sched_barrier(0);   // one 32x32 tile at a time: keeps register use flat
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r_ = row + i * 32;
            if (r_ >= g.M) continue;
#pragma unroll
            for (int j = 0; j < kTN; ++j) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int col = colb + j * 32 + 8 * (r / 4) + (r % 4);
                    if (col >= g.N) continue;
                    const size_t off = size_t(r_) * g.ldc + col;
                    const float v = g.alpha * acc[i][j][r];
                    if (c32) c32[off] = v;
                    else g.C16[off] = (half_t)v;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
}


__global__ __launch_bounds__(kThreads) void gemm_nt_256x256(GemmNT g, int tiles_m, int tiles_n,
                                                             int k_per_split) {
    extern __shared__ __attribute__((aligned(16))) half_t smem[];
    half_t* As = smem;                      // [2][BM][LDS_LD]
    half_t* Bs = smem + 2 * BM * LDS_LD;    // [2][BN][LDS_LD]

    int tm, tn, z;
    if (!work_item(tiles_m, tiles_n, gridDim.y, tm, tn, z)) return;
    const int m0 = tm * BM, n0 = tn * BN;
    const int k_begin = z * k_per_split;
    const int k_end = min(g.K, k_begin + k_per_split);
    const int nslab = (k_end - k_begin) / BK;

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int wm = wave / kWavesN, wn = wave % kWavesN;

    // Global->LDS staging: 16-byte chunk c = tid + 256*i covers row c/8, halfs [8*(c%8), +8).
    const int ld_row = tid / 8, ld_kc = (tid % 8) * 8;
    const half_t* a_src[kLd];
    const half_t* b_src[kLd];
    constexpr int kRowStep = kThreads / 8;
#pragma unroll
    for (int i = 0; i < kLd; ++i) {
        const int ra = min(m0 + ld_row + kRowStep * i, g.M - 1);
        const int rb = min(n0 + ld_row + kRowStep * i, g.N - 1);
        a_src[i] = g.A + size_t(ra) * g.lda + k_begin + ld_kc;
        b_src[i] = g.B + size_t(rb) * g.ldb + k_begin + ld_kc;
    }
    const int st_off = ld_row * LDS_LD + ld_kc;

    floatx16 acc[4][kTN];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < kTN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    half8 ra[kLd], rb[kLd];
    if (nslab > 0) {
#pragma unroll
        for (int i = 0; i < kLd; ++i) { ra[i] = ld_half8(a_src[i]); rb[i] = ld_half8(b_src[i]); }
#pragma unroll
        for (int i = 0; i < kLd; ++i) {
            st_half8(As + st_off + kRowStep * i * LDS_LD, ra[i]);
            st_half8(Bs + st_off + kRowStep * i * LDS_LD, rb[i]);
        }
    }
    __syncthreads();

    const int a_frag_off = (wm * 128 + lane % 32) * LDS_LD + 8 * (lane / 32);
    const int b_frag_off = (wn * 32 * kTN + lane % 32) * LDS_LD + 8 * (lane / 32);

    for (int s = 0; s < nslab; ++s) {
        const int cur = s & 1;
        const bool more = (s + 1 < nslab);
        if (more) {
            const int koff = (s + 1) * BK;
#pragma unroll
            for (int i = 0; i < kLd; ++i) {
                ra[i] = ld_half8(a_src[i] + koff);
                rb[i] = ld_half8(b_src[i] + koff);
            }
        }
        const half_t* Ac = As + cur * BM * LDS_LD + a_frag_off;
        const half_t* Bc = Bs + cur * BN * LDS_LD + b_frag_off;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            half8 af[4], bf[kTN];
#pragma unroll
            for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const half8*>(Ac + i * 32 * LDS_LD + kk * 16);
#pragma unroll
            for (int j = 0; j < kTN; ++j) bf[j] = *reinterpret_cast<const half8*>(Bc + j * 32 * LDS_LD + kk * 16);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < kTN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
        }
        if (more) {
            half_t* An = As + (cur ^ 1) * BM * LDS_LD + st_off;
            half_t* Bn = Bs + (cur ^ 1) * BN * LDS_LD + st_off;
#pragma unroll
            for (int i = 0; i < kLd; ++i) {
                st_half8(An + kRowStep * i * LDS_LD, ra[i]);
                st_half8(Bn + kRowStep * i * LDS_LD, rb[i]);
            }
        }
        __syncthreads();
    }

    store_tile(g, acc, m0, n0, wm, wn, lane, z);
}

// TN form: C[M][N] = alpha * sum_k A[k][m] * B[k][n] with both operands stored k-major ([K][M] and
// [K][N], m / n contiguous) -- the shape of the weight gradients dW = dG^T * X, whose operands come out
// of the recurrence as [time*batch][features].  Slabs are staged in LDS exactly as they sit in memory
// (coalesced 16-byte rows along m / n) and the MFMA fragments, which need 8 consecutive k per lane,
// are read with the gfx950 transposing LDS load ds_read_b64_tr_b16: in every group of 16 lanes, lane j
// supplies 4 halfs of row j/4 and receives the k-column for its own m, so no transposed copy of the
// operands ever exists in HBM.  Rows k >= K read as zero.
constexpr int kPitchT = 256 + 16;   // halfs per LDS row: 4 consecutive k rows fall in distinct banks
constexpr size_t kLdsBytesTN = size_t(2) * 2 * BK * kPitchT * sizeof(half_t);

typedef short short4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v lds_short4;

__device__ __forceinline__ half8 read_frag_tr(const half_t* lds_lane) {
    union { short4v s[2]; half8 h; } u;
    u.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(lds_lane));
    u.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(lds_lane + 4 * kPitchT));
    return u.h;
}

__global__ __launch_bounds__(kThreads) void gemm_tn_256x256(GemmNT g, int tiles_m, int tiles_n,
                                                             int slabs_per_split) {
    extern __shared__ __attribute__((aligned(16))) half_t smem[];
    half_t* As = smem;                        // [2][BK][kPitchT]
    half_t* Bs = smem + 2 * BK * kPitchT;     // [2][BK][kPitchT]

    int tm, tn, z;
    if (!work_item(tiles_m, tiles_n, gridDim.y, tm, tn, z)) return;
    const int m0 = tm * BM, n0 = tn * BN;
    const int nslab_total = (g.K + BK - 1) / BK;
    const int slab_begin = z * slabs_per_split;
    const int nslab = min(nslab_total - slab_begin, slabs_per_split);
    const int k_begin = slab_begin * BK;

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int wm = wave / kWavesN, wn = wave % kWavesN;

    // Global->LDS staging: 16-byte chunk c = tid + kThreads*i is k-row c/32, columns [8*(c%32), +8).
    const int ld_k = tid / 32, ld_c = (tid % 32) * 8;
    constexpr int kRowStep = kThreads / 32;
    const bool a_ok = (m0 + ld_c) < g.M, b_ok = (n0 + ld_c) < g.N;
    const half_t* a_src = g.A + min(m0 + ld_c, g.M - 8);
    const half_t* b_src = g.B + min(n0 + ld_c, g.N - 8);
    const int st_off = ld_k * kPitchT + ld_c;
    half8 ra[kLd], rb[kLd];
    // per-thread row pointers advance by one slab per fetch; only the slab that crosses K (always the
    // last one of the matrix) needs per-row masking
    const half_t* a_ptr = a_src + size_t(k_begin + ld_k) * g.lda;
    const half_t* b_ptr = b_src + size_t(k_begin + ld_k) * g.ldb;
    const size_t a_step = size_t(kRowStep) * g.lda, b_step = size_t(kRowStep) * g.ldb;
    auto fetch = [&](int slab) {
        const int k0 = k_begin + slab * BK;
        if (a_ok && b_ok && k0 + BK <= g.K) {
#pragma unroll
            for (int i = 0; i < kLd; ++i) {
                ra[i] = ld_half8(a_ptr + i * a_step);
                rb[i] = ld_half8(b_ptr + i * b_step);
            }
        } else {
#pragma unroll
            for (int i = 0; i < kLd; ++i) {
                const int k = k0 + ld_k + kRowStep * i;
                const int kc = min(k, g.K - 1);
                ra[i] = ld_half8(a_src + size_t(kc) * g.lda);
                rb[i] = ld_half8(b_src + size_t(kc) * g.ldb);
                if (!(a_ok && k < g.K)) ra[i] = half8{};
                if (!(b_ok && k < g.K)) rb[i] = half8{};
            }
        }
        a_ptr += size_t(BK) * g.lda;
        b_ptr += size_t(BK) * g.ldb;
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < kLd; ++i) {
            st_half8(As + buf * BK * kPitchT + st_off + kRowStep * i * kPitchT, ra[i]);
            st_half8(Bs + buf * BK * kPitchT + st_off + kRowStep * i * kPitchT, rb[i]);
        }
    };
    // transposing fragment read: lane (group gq = lane/16, j = lane%16) addresses k-row 8*(gq/2) + j/4,
    // column 16*(gq%2) + 4*(j%4) of a 32-wide tile; it receives k = 8*(lane/32) .. +7 for column lane%32.
    const int gq = lane / 16, jq = lane % 16;
    const int frag_off = (8 * (gq / 2) + jq / 4) * kPitchT + 16 * (gq % 2) + 4 * (jq % 4);
    const int a_frag_off = frag_off + wm * 128;
    const int b_frag_off = frag_off + wn * 32 * kTN;

    floatx16 acc[4][kTN];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < kTN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    if (nslab > 0) {
        fetch(0);
        stage(0);
    }
    __syncthreads();

    for (int s = 0; s < nslab; ++s) {
        const int cur = s & 1;
        const bool more = (s + 1 < nslab);
        if (more) fetch(s + 1);
        const half_t* Ac = As + cur * BK * kPitchT + a_frag_off;
        const half_t* Bc = Bs + cur * BK * kPitchT + b_frag_off;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            half8 af[4], bf[kTN];
#pragma unroll
            for (int i = 0; i < 4; ++i) af[i] = read_frag_tr(Ac + kk * 16 * kPitchT + i * 32);
#pragma unroll
            for (int j = 0; j < kTN; ++j) bf[j] = read_frag_tr(Bc + kk * 16 * kPitchT + j * 32);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < kTN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
        }
        if (more) stage(cur ^ 1);
        __syncthreads();
    }
    store_tile(g, acc, m0, n0, wm, wn, lane, z);
}

}  // namespace

hipError_t launch_gemm_nt(const GemmNT& g, hipStream_t stream) {
    if (g.M <= 0 || g.N <= 0 || g.K <= 0) return hipSuccess;
    if (g.K % BK != 0 || g.lda % 8 != 0 || g.ldb % 8 != 0) return hipErrorInvalidValue;
    if ((g.C16 == nullptr) == (g.C32 == nullptr)) return hipErrorInvalidValue;
    // the vector stores of full tiles need an aligned base (rows are covered by the ldc % 4 test in the kernel)
    if (g.C32 && (reinterpret_cast<uintptr_t>(g.C32) % 16 != 0 || g.split_stride % 4 != 0)) return hipErrorInvalidValue;
    if (g.C16 && (reinterpret_cast<uintptr_t>(g.C16) % 8 != 0)) return hipErrorInvalidValue;
    int splits = g.splits < 1 ? 1 : g.splits;
    if (splits > 1 && g.C32 == nullptr) return hipErrorInvalidValue;
    const int nslab = g.K / BK;
    if (splits > nslab) splits = nslab;
    const int slabs_per_split = (nslab + splits - 1) / splits;
    splits = (nslab + slabs_per_split - 1) / slabs_per_split;
    if (splits != (g.splits < 1 ? 1 : g.splits) && g.splits > 1) {
        // The caller sized its partial buffer for g.splits slices; fewer are produced, so the unused
        // ones must read as zero.  Callers use gemm_effective_splits() to avoid this path.
        return hipErrorInvalidValue;
    }
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_nt_256x256),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(kLdsBytes));
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    // gridDim.y carries the split count; x is padded so that x*y is a whole number of 256-workgroup rounds
    const int items = tiles_m * tiles_n * splits;
    const int rounded = (items + 255) / 256 * 256;
    dim3 grid((rounded + splits - 1) / splits, splits, 1);
    hipLaunchKernelGGL(gemm_nt_256x256, grid, dim3(kThreads), kLdsBytes, stream, g, tiles_m, tiles_n,
                       slabs_per_split * BK);
    return hipGetLastError();
}

hipError_t launch_gemm_tn(const GemmNT& g, hipStream_t stream) {
    if (g.M <= 0 || g.N <= 0 || g.K <= 0) return hipSuccess;
    if (g.M % 8 != 0 || g.N % 8 != 0 || g.lda % 8 != 0 || g.ldb % 8 != 0) return hipErrorInvalidValue;
    if ((g.C16 == nullptr) == (g.C32 == nullptr)) return hipErrorInvalidValue;
    if (g.C32 && (reinterpret_cast<uintptr_t>(g.C32) % 16 != 0 || g.split_stride % 4 != 0)) return hipErrorInvalidValue;
    if (g.C16 && (reinterpret_cast<uintptr_t>(g.C16) % 8 != 0)) return hipErrorInvalidValue;
    const int splits = g.splits < 1 ? 1 : g.splits;
    if (splits > 1 && g.C32 == nullptr) return hipErrorInvalidValue;
    if (gemm_effective_splits(g.K, splits) != splits) return hipErrorInvalidValue;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tn_256x256),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(kLdsBytesTN));
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int nslab = (g.K + BK - 1) / BK;
    const int slabs_per_split = (nslab + splits - 1) / splits;
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    const int items = tiles_m * tiles_n * splits;
    const int rounded = (items + 255) / 256 * 256;
    dim3 grid((rounded + splits - 1) / splits, splits, 1);
    hipLaunchKernelGGL(gemm_tn_256x256, grid, dim3(kThreads), kLdsBytesTN, stream, g, tiles_m, tiles_n,
                       slabs_per_split);
    return hipGetLastError();
}

int gemm_effective_splits(int K, int wanted) {
    const int nslab = (K + BK - 1) / BK;
    if (wanted < 1) wanted = 1;
    if (wanted > nslab) wanted = nslab;
    if (wanted < 1) wanted = 1;
    const int per = (nslab + wanted - 1) / wanted;
    return (nslab + per - 1) / per;
}

}  // namespace flstm_hip
