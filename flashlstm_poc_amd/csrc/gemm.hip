// fp16 MFMA GEMMs for gfx950 (CDNA4), fp32 accumulation.
//
// These are the dense contractions around the recurrence: the hoisted input projection X*W_ih^T (the
// reference does it with a CUTLASS 128x128x32 tensor-op GEMM, src/lstm.cu:1204-1239,
// src/lstm_internal.h:48-68), the input gradient dX = dG*W_ih (both "NT": operands K-contiguous) and the
// weight gradients dW = dG^T*[X;H] ("TN": operands k-major; reference:
// flashlstm_v2/src/lstm_backward.cu:1112-1172 through flashlstm_v2/src/gemm.cu:222-330).
//
// Common tiling: one 512-thread workgroup (8 wavefronts, 2 along M x 4 along N, two per SIMD) owns a
// 256x256 tile of C; every wavefront owns 128x64 as a 4x2 grid of v_mfma_f32_32x32x16_f16 tiles (128
// accumulator registers).  K is walked in slabs of 64 through double-buffered LDS.  The MFMA operands are
// swapped (D = B_tile * A_tile^T) so that a lane ends up with four consecutive columns of one row of C;
// full tiles are then turned through a little LDS so that every store instruction writes whole 128-byte
// lines.  The work order gives the 32 workgroups that share an XCD one compact block of tiles.
#include "gemm.h"

namespace flstm_hip {
namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kWavesN = 4;                 // wavefronts along N (2 along M): wave tile 128 x (256 / kWavesN)
constexpr int kThreads = 128 * kWavesN;
constexpr int kTN = 8 / kWavesN;            // 32-wide MFMA tiles per wave along N

// Work order.  The hardware deals workgroups round-robin over the 8 XCDs in dispatch order, so the 32
// workgroups with the same (dispatch index mod 8) that run together share one XCD and its 4 MiB L2.  They
// are given one SUPER-TILE: a compact sm x sn block of tiles (sm * sn = 32, normally 8 x 4, i.e.
// 2048 x 1024 of C) of one K split, for which they fetch sm + sn operand panels instead of up to 33.
// Consecutive super-tiles of an XCD walk down M inside one column group, so the B panels of that group
// stay in its L2 from one round to the next.
struct TileOrder {
    int tiles_m, tiles_n, splits;
    int sm, sn;        // super-tile shape in tiles
    int nsm, nsn;      // super-tiles along M and N
    int per_xcd;       // super-tiles (= rounds) per XCD
};

__device__ __forceinline__ bool work_item(const TileOrder& o, int lin, int& tm, int& tn, int& z) {
    const int xcd = lin % 8, s = lin / 8;
    const int slot = s % 32, round = s / 32;
    const int nst = o.nsm * o.nsn * o.splits;
    const int st = xcd * o.per_xcd + round;
    if (round >= o.per_xcd || st >= nst) return false;
    z = st / (o.nsm * o.nsn);
    const int r = st % (o.nsm * o.nsn);
    tm = (r % o.nsm) * o.sm + slot / o.sn;
    tn = (r / o.nsm) * o.sn + slot % o.sn;
    return tm < o.tiles_m && tn < o.tiles_n;
}

// Epilogue shared by both kernels.  With swapped MFMA operands register r of tile (i, j) holds row
// (i*32 + lane%32) of the wave's 128 x 64 block and column j*32 + 8*(r/4) + 4*(lane/32) + r%4: four
// consecutive columns per group of four registers, stored as one 8-byte (fp16) or 16-byte (fp32) access.
// bias[col .. col+3] of a full tile (col % 4 == 0), zeros when the GEMM has no bias.  Every epilogue forms
// fma(alpha, acc, bias) explicitly in fp32 and only then rounds to fp16 (out16 keeps the compiler from
// merging the two into one mixed-precision instruction with a single rounding), so an element gets the
// same bits whichever path stores its tile.
__device__ __forceinline__ half_t out16(float alpha, float acc, float bias) {
    float v = __builtin_fmaf(alpha, acc, bias);
    asm volatile("" : "+v"(v));
    return (half_t)v;
}

// Vector stores of full tiles need rows of a multiple of 4 elements that start on 8 (fp16) / 16 (fp32) bytes;
// any other output (odd row length, a sub-matrix that starts at an odd row) takes the element-wise path.
__device__ __forceinline__ bool vector_output(const GemmNT& g) {
    if (g.ldc % 4 != 0) return false;
    if (g.C16) return reinterpret_cast<uintptr_t>(g.C16) % 8 == 0;
    return reinterpret_cast<uintptr_t>(g.C32) % 16 == 0 && g.split_stride % 4 == 0;
}

__device__ __forceinline__ floatx4 bias4(const GemmNT& g, int col) {
    return g.bias ? *reinterpret_cast<const floatx4*>(g.bias + col) : floatx4{0.f, 0.f, 0.f, 0.f};
}

__device__ __forceinline__ void store_tile(const GemmNT& g, floatx16 (&acc)[4][kTN], int m0, int n0, int wm,
                                           int wn, int lane, int z) {
    const int row = m0 + wm * 128 + lane % 32;
    const int colb = n0 + wn * 32 * kTN + 4 * (lane / 32);
    float* c32 = g.C32 ? g.C32 + size_t(z) * g.split_stride : nullptr;
    const bool full = (m0 + BM <= g.M) && (n0 + BN <= g.N) && vector_output(g);
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
                        for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf(g.alpha, acc[i][j][4 * q + e], bias4(g, colb + j * 32 + 8 * q)[e]);
                        *reinterpret_cast<floatx4*>(c32 + off) = v;
                    } else {
                        half4 v;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            v[e] = out16(g.alpha, acc[i][j][4 * q + e], bias4(g, colb + j * 32 + 8 * q)[e]);
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
                    const float bv = g.bias ? g.bias[col] : 0.f;
                    if (c32) c32[off] = __builtin_fmaf(g.alpha, acc[i][j][r], bv);
                    else g.C16[off] = out16(g.alpha, acc[i][j][r], bv);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
}


// ------------------------------------------------------------------------------------- NT kernel
// C[M][N] = alpha * A[M][K] * B[N][K]^T (+ bias[n]).  Operand slabs go from global memory straight into
// LDS (global_load_lds_dwordx4: no staging registers, no LDS store instructions), double buffered in
// slabs of 64 k.  Every wave copies 8 KiB of a slab with eight 1 KiB copies, each addressed as a scalar base
// plus a per-lane offset that is fixed for the tile, and issues them behind the MFMAs of the last k-step
// of the slab before, right after the barrier that frees the buffer: a slab is requested one slab ahead and
// a slab boundary costs no wave a wait with nothing to multiply.  (The copies used to carry 64-bit address
// arithmetic per lane: ~15 instructions each in the shadow of two MFMAs, which made instruction issue,
// not the matrix cores, the limit while they ran.)
// The kernel is persistent: each workgroup walks its list of work items and the copies keep running
// across item boundaries, so the first slabs of the next tile arrive during the last MFMAs and the
// output stores of this one.
//
// LDS rows are 128 bytes (8 chunks of 16).  The LDS has 64 banks of 4 bytes and serves a 16-byte read
// for 16 lanes per clock, so the 16 rows read together must land in 16 different 16-byte bank groups of
// the 256-byte bank row; two rows share a bank row, hence chunk c of row r sits at position c ^ (r/2)%8.
constexpr int kSlabBytes = (BM + BN) * BK * 2;               // 64 KiB: A rows then B rows
constexpr int kEpiBytesPerWave = 32 * 64 * 2;                 // one 32 x 64 fp16 block of the wave's output
constexpr size_t kLdsBytesStream = size_t(2) * kSlabBytes + 8 * kEpiBytesPerWave;   // 160 KiB
constexpr int kCopiesPerWave = 8;                            // 8 waves x 8 KiB = one slab

typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void global_void;

__device__ __forceinline__ void copy_1k_to_lds(const char* src_lane, char* lds_block) {
    __builtin_amdgcn_global_load_lds((global_void*)(src_lane), (lds_void*)(lds_block), 16, 0, 0);
}

// The same copy issued by hand: scalar base + 32-bit offset per lane, LDS destination in M0.  The compiler
// does not know that it writes LDS, so it places no wait for it in front of LDS reads (it cannot tell that
// the transposing reads of gemm_tn_stream never touch the buffer being filled, and would wait for every
// copy right after it was issued); the kernel's own s_waitcnt vmcnt(0) + barrier order copies and reads.
// Counted waits that the compiler places for its own loads and stores only become stricter by the extra
// operations in flight.
typedef __attribute__((address_space(3))) char lds_char;
__device__ __forceinline__ void copy_1k_to_lds_unseen(const char* base, unsigned lane_off, char* lds_block) {
    const unsigned m = unsigned(reinterpret_cast<unsigned long>((lds_char*)(lds_block)));
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_off), "s"(base), "s"(m) : "m0", "memory");
}

template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// fp16 epilogue of a full tile with whole-line stores.  In the accumulators one row of the wave's 128 x 64
// block is spread over two lanes in 8-byte pieces, which makes 32 partial-line writes per store instruction.
// Each 32 x 64 block is therefore turned through a private 4 KiB of LDS (16-byte chunks XOR-swizzled by
// row / 2, so the 16-byte reads are conflict free): 8 lanes then hold one 128-byte row segment and a store
// instruction writes 8 complete lines.  16 stores per wave instead of 32.
__device__ __forceinline__ void store_tile_lines(const GemmNT& g, floatx16 (&acc)[4][kTN], int m0, int n0, int wm,
                                                 int wn, int lane, char* stage) {
    static_assert(kTN == 2, "the staging block is 64 columns wide");
    const int wr = lane % 32;                              // row written by this lane
    const int wsw = (wr >> 1) & 7;
    const int rr = lane / 8, rc = lane % 8;                // row (+ 8p) and 16-byte chunk read by this lane
    half_t* cbase = g.C16 + size_t(m0 + wm * 128) * g.ldc + n0 + wn * 64 + rc * 8;
    floatx4 bv[kTN][4];   // bias of this lane's 32 columns
#pragma unroll
    for (int j = 0; j < kTN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) bv[j][q] = bias4(g, n0 + wn * 64 + j * 32 + 8 * q + 4 * (lane / 32));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < kTN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                half4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = out16(g.alpha, acc[i][j][4 * q + e], bv[j][q][e]);
                const int chunk = 4 * j + q;
                *reinterpret_cast<half4*>(stage + wr * 128 + ((chunk ^ wsw) * 16) + 8 * (lane / 32)) = v;
            }
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int row = rr + 8 * p;
            const half8 v = *reinterpret_cast<const half8*>(stage + row * 128 + ((rc ^ ((row >> 1) & 7)) * 16));
            *reinterpret_cast<half8*>(cbase + size_t(i * 32 + row) * g.ldc) = v;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

__global__ __launch_bounds__(kThreads) void gemm_nt_stream(GemmNT g, TileOrder order, int k_per_split) {
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wm = wave / kWavesN, wn = wave % kWavesN;
    const int rounds = order.per_xcd;

    // ordinal n of this workgroup -> (tile, split) in the order of work_item().  Ordinals that fall on a
    // tile outside the matrix are skipped, by the copy sequence and the consumer alike.
    auto decode = [&](int n, int& m0, int& n0, int& z, int& kb, int& nk) -> bool {
        int tm, tn;
        if (!work_item(order, n * int(gridDim.x) + blockIdx.x, tm, tn, z)) return false;
        m0 = tm * BM;
        n0 = tn * BN;
        kb = z * k_per_split;
        nk = (min(g.K, kb + k_per_split) - kb) / BK;
        return nk > 0;
    };

    // ---- copier state: the slab copied next is slab ld_k of item ordinal ld_n.  Copy c of a slab
    // (operand c % 2, row block i = c / 2) fills rows [64q + 8i, +8) of the tile, q = wave % 4; lane l
    // lands at row l / 8, chunk position l % 8 and therefore fetches chunk (l % 8) ^ swizzle(row).
    // A copy is addressed as a wave-uniform base (the slab's first row and column, kept in scalar
    // registers and advanced by 128 bytes per slab) plus a 32-bit byte offset per lane that is fixed for
    // the whole tile: one instruction per copy, no address arithmetic in the shadow of the MFMAs.
    int ld_n = 0, ld_k = 0, ld_nk = 0;
    bool ld_live = false;
    const char* ld_a = reinterpret_cast<const char*>(g.A);
    const char* ld_b = reinterpret_cast<const char*>(g.B);
    unsigned voff_a[4], voff_b[4];
    const int cp_row = wave * 32 + lane / 8;
    auto loader_open = [&]() {
        int z, m0 = 0, n0 = 0, kb = 0;
        bool valid = false;
        while (ld_n < rounds && !(valid = decode(ld_n, m0, n0, z, kb, ld_nk))) ++ld_n;
        // past the last item the copies go on, of the first slab of the operands (the copier no longer
        // advances) into a buffer nobody reads any more: cheaper than a branch around every copy
        if (!valid) m0 = n0 = kb = 0;
        ld_live = valid;
        ld_k = 0;
        ld_a = reinterpret_cast<const char*>(g.A + size_t(m0) * g.lda + kb);
        ld_b = reinterpret_cast<const char*>(g.B + size_t(n0) * g.ldb + kb);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int rt = cp_row + 8 * i;
            const unsigned chunk = unsigned((lane % 8) ^ ((rt >> 1) & 7)) * 16u;
            voff_a[i] = unsigned(min(m0 + rt, g.M - 1) - m0) * unsigned(g.lda * 2) + chunk;
            voff_b[i] = unsigned(min(n0 + rt, g.N - 1) - n0) * unsigned(g.ldb * 2) + chunk;
        }
    };
    auto issue_copy = [&](int slot, int c) {
        const int i = c / 2;
        char* dst = lds + slot * kSlabBytes + wave * 4096 + i * 1024;
        if (c % 2 == 0) copy_1k_to_lds(ld_a + voff_a[i], dst);
        else copy_1k_to_lds(ld_b + voff_b[i], dst + BM * BK * 2);
    };
    auto loader_advance = [&]() {
        if (!ld_live) return;
        ld_a += BK * 2;
        ld_b += BK * 2;
        if (++ld_k == ld_nk) {
            ++ld_n;
            loader_open();
        }
    };

    // ---- consumer: fragment addresses inside a slab (tile rows of one lane are multiples of 32 apart,
    // so the swizzle depends on the lane only)
    const int a_frag = (wm * 128 + lane % 32) * (BK * 2);
    const int b_frag = BM * BK * 2 + (wn * 32 * kTN + lane % 32) * (BK * 2);
    int pos[BK / 16];
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) pos[kk] = ((2 * kk + lane / 32) ^ ((lane % 32) >> 1 & 7)) * 16;

    constexpr int KK = BK / 16;
    constexpr int kPerStep = 4 * kTN;   // MFMAs per k-step
    static_assert(kPerStep == kCopiesPerWave, "one copy behind every MFMA of a slab's last k-step");
    half8 af[2][4], bf[2][kTN];
    // fragment f of a k-step: 0..3 the A rows, 4.. the B rows
    auto read_frag = [&](const char* st, int kk, int set, int f) {
        if (f < 4) af[set][f] = *reinterpret_cast<const half8*>(st + a_frag + f * 32 * BK * 2 + pos[kk]);
        else bf[set][f - 4] = *reinterpret_cast<const half8*>(st + b_frag + (f - 4) * 32 * BK * 2 + pos[kk]);
    };
    auto read_frags = [&](const char* st, int kk, int set) {
#pragma unroll
        for (int f = 0; f < 4 + kTN; ++f) read_frag(st, kk, set, f);
    };

    // Prologue: the first two slabs are requested, the first one awaited (copies complete in the order
    // they were issued, so at most the second slab's 8 may be outstanding) and its first fragments read.
    loader_open();
#pragma unroll
    for (int c = 0; c < kCopiesPerWave; ++c) issue_copy(0, c);
    loader_advance();
#pragma unroll
    for (int c = 0; c < kCopiesPerWave; ++c) issue_copy(1, c);
    loader_advance();
    wait_vm<kCopiesPerWave>();
    __builtin_amdgcn_s_barrier();
    read_frags(lds, 0, 0);

    int slot = 0;            // LDS buffer of the slab being multiplied
    for (int n = 0; n < rounds; ++n) {
        int m0, n0, z, kb, nk;
        if (!decode(n, m0, n0, z, kb, nk)) continue;
        floatx16 acc[4][kTN];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < kTN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

        for (int ks = 0; ks < nk; ++ks) {
            const char* st = lds + slot * kSlabBytes;
            const char* st_next = lds + (slot ^ 1) * kSlabBytes;
            // Source order below is the schedule (pinned by sched_barrier): the fragments of the next
            // 16-wide k-step are read one by one behind the first MFMAs of this one, so that a wave never
            // stands at a wait for fragments it has only just asked for.
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const int cur = kk & 1;
                if (kk + 1 < KK) {
#pragma unroll
                    for (int m = 0; m < kPerStep; ++m) {
                        const int i = m / kTN, j = m % kTN;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[cur][j], af[cur][i], acc[i][j], 0, 0, 0);
                        __builtin_amdgcn_sched_barrier(0);
                        if (m < 4 + kTN) read_frag(st, kk + 1, cur ^ 1, m);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
                    // The slab's last fragments have been requested.  Once they are in registers nothing of
                    // this wave reads the buffer again, and the copies this wave made of the next slab, issued
                    // one slab ago, are awaited here too: behind the barrier the next slab is complete and
                    // this buffer is free.  The next slab's first fragments are then read, and the slab after
                    // it requested, under the MFMAs of this last k-step, so no wave ever waits at a slab
                    // boundary with nothing to multiply.  (The wait is for everything: loads complete in issue
                    // order among themselves, but the output stores of the previous tile may be acknowledged
                    // out of order with them and would spoil a count.)
                    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    const bool more = ks + 1 < nk;   // (a tile's last slab: fragments after its epilogue)
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int m = 0; m < kPerStep; ++m) {
                        const int i = m / kTN, j = m % kTN;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[cur][j], af[cur][i], acc[i][j], 0, 0, 0);
                        __builtin_amdgcn_sched_barrier(0);
                        if (more && m < 4 + kTN) read_frag(st_next, 0, cur ^ 1, m);
                        issue_copy(slot, m);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            loader_advance();
            slot ^= 1;
        }
        const bool full = (m0 + BM <= g.M) && (n0 + BN <= g.N) && vector_output(g);
        if (full && g.C16 && g.ldc % 8 == 0 && reinterpret_cast<uintptr_t>(g.C16) % 16 == 0) {
            store_tile_lines(g, acc, m0, n0, wm, wn, lane, lds + 2 * kSlabBytes + wave * kEpiBytesPerWave);
        } else {
            store_tile(g, acc, m0, n0, wm, wn, lane, z);
        }
        read_frags(lds + slot * kSlabBytes, 0, 0);
    }
    wait_vm<0>();   // no copy may still be heading for LDS when the workgroup retires
}

// TN form: C[M][N] = alpha * sum_k A[k][m] * B[k][n] with both operands stored k-major ([K][M] and
// [K][N], m / n contiguous) -- the shape of the weight gradients dW = dG^T * X, whose operands come out
// of the recurrence as [time*batch][features].  Slabs sit in LDS as they sit in memory (64 k-rows of
// 256 halfs per operand) and the MFMA fragments, which need 8 consecutive k per lane, are read with the
// gfx950 transposing LDS load ds_read_b64_tr_b16: in every group of 16 lanes, lane j supplies 4 halfs of
// row j/4 and receives the k-column for its own m, so no transposed copy of the operands ever exists in
// HBM.  Rows k >= K read as zero.
//
// The kernel has the structure of gemm_nt_stream: persistent, slabs copied from global memory straight
// into LDS one slab ahead (a copy instruction fills two 512-byte k-rows), the barrier of a slab boundary
// taken under the last k-step's MFMAs.  LDS rows are 512 bytes without padding; the four k-rows that 32
// lanes read together (64 bytes each) are kept in different quarters of the 256-byte bank row by
// exchanging the 64-byte chunks of a row: chunk c of k-row r sits at position c ^ (r % 4).

typedef short short4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v lds_short4;

// one MFMA operand fragment: 8 consecutive k for this lane's column, as two transposing reads 4 k-rows apart
__device__ __forceinline__ half8 read_frag_tr(const char* lds_lane) {
    union { short4v s[2]; half8 h; } u;
    u.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(lds_lane));
    u.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(lds_lane + 4 * 512));
    return u.h;
}

// fp32 epilogue of a full tile with whole-line stores (split-K partials): every 32 x 32 accumulator tile
// is one 128-byte line per row; it is turned through a private 4 KiB of LDS so that 8 lanes hold one row
// and a store instruction writes 8 complete lines instead of 32 quarter lines.
__device__ __forceinline__ void store_tile_lines_f32(const GemmNT& g, floatx16 (&acc)[4][kTN], int m0, int n0,
                                                     int wm, int wn, int lane, int z, char* stage) {
    const int wr = lane % 32;
    const int wsw = (wr >> 1) & 7;
    const int rr = lane / 8, rc = lane % 8;
    float* cbase = g.C32 + size_t(z) * g.split_stride + size_t(m0 + wm * 128) * g.ldc + n0 + wn * 32 * kTN + rc * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < kTN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                floatx4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = g.alpha * acc[i][j][4 * q + e];
                const int chunk = 2 * q + lane / 32;
                *reinterpret_cast<floatx4*>(stage + wr * 128 + ((chunk ^ wsw) * 16)) = v;
            }
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int row = rr + 8 * p;
                const floatx4 v = *reinterpret_cast<const floatx4*>(stage + row * 128 + ((rc ^ ((row >> 1) & 7)) * 16));
                *reinterpret_cast<floatx4*>(cbase + size_t(i * 32 + row) * g.ldc + j * 32) = v;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

__global__ __launch_bounds__(kThreads) void gemm_tn_stream(GemmNT g, TileOrder order, int slabs_per_split) {
    extern __shared__ __attribute__((aligned(1024))) char lds[];

    const int tid = threadIdx.x, lane = tid % 64;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wm = wave / kWavesN, wn = wave % kWavesN;
    const int rounds = order.per_xcd;
    const int nslab_total = (g.K + BK - 1) / BK;
    const int tiles_n1 = g.B2 ? (g.N1 + BN - 1) / BN : (1 << 30);

    // ordinal n of this workgroup -> (tile, split).  With two B operands side by side each side has its
    // own tiles, so a tile reads one operand only: side 1 is B2 and columns [N1, N) of C.
    struct Item { int m0, n0, side, z, slab0, nk; };
    auto decode = [&](int n, Item& it) -> bool {
        int tm, tn;
        if (!work_item(order, n * int(gridDim.x) + blockIdx.x, tm, tn, it.z)) return false;
        it.side = tn >= tiles_n1 ? 1 : 0;
        it.m0 = tm * BM;
        it.n0 = (tn - (it.side ? tiles_n1 : 0)) * BN;
        it.slab0 = it.z * slabs_per_split;
        it.nk = min(nslab_total - it.slab0, slabs_per_split);
        return it.nk > 0;
    };

    // ---- copier.  Copy c of a slab (operand c % 2, row pair i = c / 2) fills k-rows 8*wave + 2i, +1; lane l
    // lands in row l / 32 of the pair at 16-byte position l % 32, i.e. in 64-byte position p = (l % 32) / 4,
    // and therefore fetches chunk p ^ (row % 4).  Addressing as in gemm_nt_stream: scalar base (the slab's
    // first k-row) + a per-lane byte offset fixed for the item; only a slab that crosses K computes clamped
    // row addresses (rows >= K are then cleared in LDS by the wave that copied them).
    int ld_n = 0, ld_k = 0, ld_nk = 0, ld_rows = BK, ld_slab = 0;
    bool ld_live = false;
    const char* ld_a = reinterpret_cast<const char*>(g.A);
    const char* ld_b = reinterpret_cast<const char*>(g.B);
    unsigned ld_pa = 0, ld_pb = 0;          // bytes per k-row of the operands of the item being copied
    unsigned col_a[2], col_b[2], voff_a[2], voff_b[2];   // [row pair % 2]: the chunk exchange depends on row % 4
    const int cp_row = 8 * wave + lane / 32;
    auto loader_open = [&]() {
        Item it{0, 0, 0, 0, 0, 0};
        bool valid = false;
        while (ld_n < rounds && !(valid = decode(ld_n, it))) ++ld_n;
        if (!valid) it = Item{0, 0, 0, 0, 0, 0};   // past the last item: harmless copies of the first slab, no advance
        ld_live = valid;
        ld_k = 0;
        ld_nk = it.nk;
        ld_slab = it.slab0;
        const half_t* bsrc = it.side ? g.B2 : g.B;
        const int nside = g.B2 ? (it.side ? g.N - g.N1 : g.N1) : g.N;
        ld_pa = unsigned(g.lda * 2);
        ld_pb = unsigned((it.side ? g.ldb2 : g.ldb) * 2);
        ld_a = reinterpret_cast<const char*>(g.A) + size_t(ld_slab) * BK * ld_pa;
        ld_b = reinterpret_cast<const char*>(bsrc) + size_t(ld_slab) * BK * ld_pb;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int sw = (2 * e + lane / 32) % 4;
            const int c = (((lane % 32) / 4) ^ sw) * 32 + (lane % 4) * 8;   // column (halfs) inside the tile
            col_a[e] = unsigned(min(it.m0 + c, g.M - 8)) * 2u;
            col_b[e] = unsigned(min(it.n0 + c, nside - 8)) * 2u;
        }
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            voff_a[e] = unsigned(cp_row) * ld_pa + col_a[e];
            voff_b[e] = unsigned(cp_row) * ld_pb + col_b[e];
        }
        ld_rows = min(BK, g.K - ld_slab * BK);
    };
    auto issue_copy = [&](int slot, int c) {
        const int i = c / 2;
        char* dst = lds + slot * kSlabBytes + (c % 2) * (BM * BK * 2) + (8 * wave + 2 * i) * 512;
        const unsigned pitch = c % 2 == 0 ? ld_pa : ld_pb;
        const char* base = c % 2 == 0 ? ld_a : ld_b;
        if (ld_rows < BK) {
            const unsigned row = unsigned(min(cp_row + 2 * i, ld_rows - 1));
            copy_1k_to_lds_unseen(base, row * pitch + (c % 2 == 0 ? col_a[i % 2] : col_b[i % 2]), dst);
        } else {
            copy_1k_to_lds_unseen(base + size_t(2 * i) * pitch, c % 2 == 0 ? voff_a[i % 2] : voff_b[i % 2], dst);
        }
    };
    auto loader_advance = [&]() {
        if (!ld_live) return;
        ld_a += size_t(BK) * ld_pa;
        ld_b += size_t(BK) * ld_pb;
        ++ld_slab;
        if (++ld_k == ld_nk) {
            ++ld_n;
            loader_open();
        } else {
            ld_rows = min(BK, g.K - ld_slab * BK);
        }
    };
    // rows >= `rows` of the slab in `st`, as far as this wave copied them, are cleared
    auto clear_tail = [&](char* st, int rows) {
        if (rows >= BK) return;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int row = 8 * wave + r;
            if (row >= rows) {
                *reinterpret_cast<unsigned long long*>(st + row * 512 + lane * 8) = 0ull;
                *reinterpret_cast<unsigned long long*>(st + BM * BK * 2 + row * 512 + lane * 8) = 0ull;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };

    // ---- consumer.  Transposing fragment read: lane (group gq = lane / 16, j = lane % 16) addresses k-row
    // 8*(gq/2) + j/4 and halfs 16*(gq%2) + 4*(j%4) of a 32-wide tile; it receives k = 8*(lane/32) .. +7 for
    // column lane % 32.  k-row % 4 = j / 4 for every read of a lane, so the chunk exchange is a per-lane
    // constant: 32-column tile t of the operand (64 bytes per k-row = one chunk) sits at chunk t ^ (j / 4).
    const int gq = lane / 16, jq = lane % 16;
    const int frag_lane = (8 * (gq / 2) + jq / 4) * 512 + 32 * (gq % 2) + 8 * (jq % 4);
    int a_frag[4], b_frag[kTN];
#pragma unroll
    for (int i = 0; i < 4; ++i) a_frag[i] = frag_lane + ((wm * 4 + i) ^ (jq / 4)) * 64;
#pragma unroll
    for (int j = 0; j < kTN; ++j) b_frag[j] = BM * BK * 2 + frag_lane + ((wn * kTN + j) ^ (jq / 4)) * 64;

    constexpr int KK = BK / 16;
    constexpr int kPerStep = 4 * kTN;
    static_assert(kPerStep == kCopiesPerWave, "one copy behind every MFMA of a slab's last k-step");
    half8 af[2][4], bf[2][kTN];
    auto read_frag = [&](const char* st, int kk, int set, int f) {
        if (f < 4) af[set][f] = read_frag_tr(st + a_frag[f] + kk * 16 * 512);
        else bf[set][f - 4] = read_frag_tr(st + b_frag[f - 4] + kk * 16 * 512);
    };
    auto read_frags = [&](const char* st, int kk, int set) {
#pragma unroll
        for (int f = 0; f < 4 + kTN; ++f) read_frag(st, kk, set, f);
    };

    loader_open();
    const int rows_first = ld_rows;
#pragma unroll
    for (int c = 0; c < kCopiesPerWave; ++c) issue_copy(0, c);
    loader_advance();
    int rows_next = ld_rows;   // valid k-rows of the slab that the next barrier completes
#pragma unroll
    for (int c = 0; c < kCopiesPerWave; ++c) issue_copy(1, c);
    loader_advance();
    wait_vm<kCopiesPerWave>();
    clear_tail(lds, rows_first);
    __builtin_amdgcn_s_barrier();
    read_frags(lds, 0, 0);

    int slot = 0;
    for (int n = 0; n < rounds; ++n) {
        Item it;
        if (!decode(n, it)) continue;
        floatx16 acc[4][kTN];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < kTN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

        for (int ks = 0; ks < it.nk; ++ks) {
            char* st = lds + slot * kSlabBytes;
            char* st_next = lds + (slot ^ 1) * kSlabBytes;
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) {
                const int cur = kk & 1;
                if (kk + 1 < KK) {
#pragma unroll
                    for (int m = 0; m < kPerStep; ++m) {
                        const int i = m / kTN, j = m % kTN;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[cur][j], af[cur][i], acc[i][j], 0, 0, 0);
                        __builtin_amdgcn_sched_barrier(0);
                        if (m < 4 + kTN) read_frag(st, kk + 1, cur ^ 1, m);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
                    // (see gemm_nt_stream: this slab's reads and this wave's copies of the next slab are
                    // complete; behind the barrier the next slab is whole and this buffer is free)
                    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                    clear_tail(st_next, rows_next);
                    __builtin_amdgcn_s_barrier();
                    const bool more = ks + 1 < it.nk;
                    __builtin_amdgcn_sched_barrier(0);
                    rows_next = ld_rows;
#pragma unroll
                    for (int m = 0; m < kPerStep; ++m) {
                        const int i = m / kTN, j = m % kTN;
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[cur][j], af[cur][i], acc[i][j], 0, 0, 0);
                        __builtin_amdgcn_sched_barrier(0);
                        if (more && m < 4 + kTN) read_frag(st_next, 0, cur ^ 1, m);
                        issue_copy(slot, m);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            loader_advance();
            slot ^= 1;
        }
        GemmNT gi = g;
        if (g.B2) {
            if (it.side) { gi.C32 += g.N1; gi.N = g.N - g.N1; }
            else gi.N = g.N1;
        }
        const bool full = (it.m0 + BM <= gi.M) && (it.n0 + BN <= gi.N) && vector_output(gi);
        if (full && gi.C32) {
            store_tile_lines_f32(gi, acc, it.m0, it.n0, wm, wn, lane, it.z, lds + 2 * kSlabBytes + wave * kEpiBytesPerWave);
        } else {
            store_tile(gi, acc, it.m0, it.n0, wm, wn, lane, it.z);
        }
        read_frags(lds + slot * kSlabBytes, 0, 0);
    }
    wait_vm<0>();   // no copy may still be heading for LDS when the workgroup retires
}

}  // namespace

static TileOrder make_order(int tiles_m, int tiles_n, int splits) {
    TileOrder o{};
    o.tiles_m = tiles_m; o.tiles_n = tiles_n; o.splits = splits;
    long best = -1;
    const int shapes[6] = {8, 4, 16, 2, 32, 1};   // sm candidates, preferred first
    for (int sm : shapes) {
        const int sn = 32 / sm;
        const long n = long((tiles_m + sm - 1) / sm) * ((tiles_n + sn - 1) / sn);
        if (best < 0 || n < best) { best = n; o.sm = sm; o.sn = sn; }
    }
    o.nsm = (tiles_m + o.sm - 1) / o.sm;
    o.nsn = (tiles_n + o.sn - 1) / o.sn;
    o.per_xcd = (o.nsm * o.nsn * splits + 7) / 8;
    return o;
}

hipError_t launch_gemm_nt(const GemmNT& g, hipStream_t stream) {
    if (g.M <= 0 || g.N <= 0 || g.K <= 0) return hipSuccess;
    if (g.K % BK != 0 || g.lda % 8 != 0 || g.ldb % 8 != 0) return hipErrorInvalidValue;
    // (a copy addresses a tile's 256 rows with 32-bit byte offsets from the tile's first row)
    if (g.lda >= (size_t(1) << 22) || g.ldb >= (size_t(1) << 22)) return hipErrorInvalidValue;
    if ((g.C16 == nullptr) == (g.C32 == nullptr)) return hipErrorInvalidValue;
    if (g.bias && (reinterpret_cast<uintptr_t>(g.bias) % 16 != 0 || g.splits > 1)) return hipErrorInvalidValue;
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
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    const TileOrder order = make_order(tiles_m, tiles_n, splits);
    // (set before every launch: the call is cheap, needs no process-wide flag and holds for whichever device is current)
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_nt_stream),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(kLdsBytesStream));
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(gemm_nt_stream, dim3(256), dim3(kThreads), kLdsBytesStream, stream, g, order,
                       slabs_per_split * BK);
    return hipGetLastError();
}

hipError_t launch_gemm_tn(const GemmNT& g, hipStream_t stream) {
    if (g.M <= 0 || g.N <= 0 || g.K <= 0) return hipSuccess;
    if (g.M % 8 != 0 || g.N % 8 != 0 || g.lda % 8 != 0 || g.ldb % 8 != 0 || g.bias) return hipErrorInvalidValue;
    if ((g.C16 == nullptr) == (g.C32 == nullptr)) return hipErrorInvalidValue;
    if (g.C32 && (reinterpret_cast<uintptr_t>(g.C32) % 16 != 0 || g.split_stride % 4 != 0)) return hipErrorInvalidValue;
    if (g.C16 && (reinterpret_cast<uintptr_t>(g.C16) % 8 != 0)) return hipErrorInvalidValue;
    const int splits = g.splits < 1 ? 1 : g.splits;
    if (splits > 1 && g.C32 == nullptr) return hipErrorInvalidValue;
    if (gemm_effective_splits(g.K, splits) != splits) return hipErrorInvalidValue;
    if (reinterpret_cast<uintptr_t>(g.A) % 16 != 0 || reinterpret_cast<uintptr_t>(g.B) % 16 != 0 ||
        (g.B2 && reinterpret_cast<uintptr_t>(g.B2) % 16 != 0))
        return hipErrorInvalidValue;
    // (a copy addresses a slab's 64 k-rows with 32-bit byte offsets from the slab's first row)
    if (g.lda >= (size_t(1) << 22) || g.ldb >= (size_t(1) << 22) || (g.B2 && g.ldb2 >= (size_t(1) << 22)))
        return hipErrorInvalidValue;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tn_stream),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(kLdsBytesStream));
    if (e != hipSuccess) return e;
    const int nslab = (g.K + BK - 1) / BK;
    const int slabs_per_split = (nslab + splits - 1) / splits;
    if (g.B2 && (g.C32 == nullptr || g.N1 <= 0 || g.N1 >= g.N || g.N1 % 8 != 0 || g.ldb2 % 8 != 0)) return hipErrorInvalidValue;
    const int tiles_m = (g.M + BM - 1) / BM;
    const int tiles_n = g.B2 ? (g.N1 + BN - 1) / BN + (g.N - g.N1 + BN - 1) / BN : (g.N + BN - 1) / BN;
    const TileOrder order = make_order(tiles_m, tiles_n, splits);
    hipLaunchKernelGGL(gemm_tn_stream, dim3(256), dim3(kThreads), kLdsBytesStream, stream, g, order,
                       slabs_per_split);
    return hipGetLastError();
}

// Split count for a TN product with fp32 partials, from the way the kernel schedules it: blocks of 32 tiles x splits
// are dealt to the 8 XCDs in rounds, a round runs K / splits, and every work item costs about 16 slabs' worth of
// prologue and partial-tile write on top.  (4096 x 2048 tiles at K = 262144: 2 splits, 4.6 ms against 8.2 at one;
// 8192 x (512 + 2048): 10 blocks, 2 rounds at one split, 5 full ones at 4, 8.2 -> 6.05 ms at K = 131072.)
int gemm_tn_auto_splits(int M, int N1, int N2, int K, int max_splits) {
    const int tiles_m = (M + BM - 1) / BM;
    const int tiles_n = (N1 + BN - 1) / BN + (N2 > 0 ? (N2 + BN - 1) / BN : 0);
    const int nslab = (K + BK - 1) / BK;
    const TileOrder o = make_order(tiles_m, tiles_n, 1);
    const long blocks = long(o.nsm) * o.nsn;
    int best_s = 1;
    double best_cost = -1.0;
    for (int sp = 1; sp <= max_splits && sp <= nslab; ++sp) {
        if (gemm_effective_splits(K, sp) != sp) continue;
        const long rounds = (blocks * sp + 7) / 8;
        const double cost = double(rounds) * (double((nslab + sp - 1) / sp) + 16.0);
        if (best_cost < 0 || cost < best_cost * (1.0 - 1e-9)) { best_cost = cost; best_s = sp; }
    }
    return best_s;
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
