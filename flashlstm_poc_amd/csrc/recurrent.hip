// Persistent W_hh-resident LSTM recurrence for gfx950: forward and backward-through-time.
//
// What the reference does per time step with a CUTLASS GEMM launch plus a pointwise launch
// (forward: src/lstm.cu:1241-1339 + src/kernels.cu:86-164; backward:
// flashlstm_v2/src/lstm_backward.cu:1057-1101 + :158-227) is done here by ONE kernel launch for
// the whole sequence:
//
//  * Work split.  The batch is cut into blocks of 32 rows and the hidden dimension into slices of
//    JB units.  A workgroup (4 wavefronts, one per SIMD, up to 512 registers each) owns one slice
//    for all row blocks of its group, i.e. all four gates of its hidden units, so the cell update
//    is local.  Its part of W_hh (forward: 4*JB gate rows x Hp; backward: 4Hp gate rows x JB
//    columns) is loaded once into registers as ready-made MFMA B-fragments and stays there.
//  * K split.  The four wavefronts split the contraction dimension (interleaved 32-wide k-steps),
//    so every element of h_{t-1} / dG_{t+1} is fetched exactly once per workgroup, straight from
//    L2 into A-fragments; partial sums meet in LDS (fp32) and the pointwise stage reads them there.
//  * Exchange.  h_t (forward) and dG_t (backward) are the only data that cross workgroups.  Groups
//    are laid out so that all workgroups of a group sit on one XCD when the slice count allows
//    (block id mod 8 is the XCD): producers use plain write-through stores, consumers fetch with
//    device-scope relaxed atomic loads (L1 bypass, served by that XCD's L2), and a per-workgroup
//    step flag in one cache line replaces the grid barrier -- no L2 write-back or invalidate is
//    ever issued.  Groups that span XCDs store the exchanged values with device-scope atomic
//    stores instead.  Every wait is bounded and reports through `status`.
//  * Fallback.  The same kernels launched once per step (no waits, kernel boundaries order
//    memory) serve shapes whose weights do not fit on chip, and are the safe path after a failed
//    persistent launch.
#include "recurrent.h"

namespace flstm_hip {
namespace {

constexpr int kThreads = 256;
constexpr int kRows = 32;  // batch rows per row block

__device__ __forceinline__ unsigned xcc_id() {
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xf;
}

struct Role {
    int g, hs;
    bool active;
};

// XCD-local mode: the hardware deals workgroups round-robin over the 8 XCDs, but where a launch
// starts in that rotation depends on what ran before, so a workgroup takes its XCD from the
// hardware register and claims the next free slot of that XCD.  A ninth... 33rd arrival on one XCD
// (uneven placement) cannot be seated: it reports status 2 and the host repeats the work step-wise.
__device__ __forceinline__ Role make_role(int nh, int ng, int gpx, int xcd_local, unsigned* seats,
                                          int* status, int* lds_role) {
    Role r;
    const int w = blockIdx.x;
    if (xcd_local) {
        if (threadIdx.x == 0) {
            const int xcd = int(xcc_id()) & 7;
            const unsigned slot = __hip_atomic_fetch_add(seats + xcd, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (slot >= 32u) __hip_atomic_store(status, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            lds_role[0] = xcd;
            lds_role[1] = int(slot);
        }
        __syncthreads();
        const int xcd = lds_role[0], slot = lds_role[1];
        const int sub = slot / nh;
        r.hs = slot % nh;
        r.g = sub * 8 + xcd;
        r.active = (slot < 32) && (sub < gpx) && (r.g < ng);
    } else {
        r.g = w / nh;
        r.hs = w % nh;
        r.active = r.g < ng;
    }
    return r;
}

// Waits until every workgroup of the group has published `target`. Returns false on abort.
__device__ __forceinline__ bool wait_group(const unsigned* gflags, int nh, unsigned target,
                                           int* status, int spin_limit, int* lds_abort) {
    if (threadIdx.x < kWave) {
        int spins = 0;
        for (;;) {
            bool ok = true;
            for (int i = threadIdx.x; i < nh; i += kWave) {
                const unsigned f = __hip_atomic_load(gflags + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = ok && (int(f - target) >= 0);
            }
            if (__all(ok)) break;
            if (++spins > spin_limit ||
                ((spins & 1023) == 0 &&
                 __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 1)) {
                if (threadIdx.x == 0) {
                    __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    *lds_abort = 1;
                }
                break;
            }
        }
    }
    __syncthreads();
    return *lds_abort == 0;
}

__device__ __forceinline__ void publish(unsigned* gflags, int hs, unsigned value) {
    __builtin_amdgcn_s_waitcnt(0);  // every store of this wave has been acknowledged by L2
    __syncthreads();
    if (threadIdx.x == 0)
        __hip_atomic_store(gflags + hs, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Exchange layout ("fragment-major").  The operand a step fetches from its peers -- h_{t-1} in the
// forward pass, dG_{t+1} in the backward pass -- is stored as ready-made MFMA A-fragments so that
// every load instruction of a wave covers one contiguous kilobyte:
//   element (row r, column k) of a [rows][K] matrix, nks = K / 32, sits at (in halfs)
//   ((r/16)*nks + k/32)*512 + (r%16 + 16*((k%32)/8))*8 + k%8
// i.e. [16-row tile][32-wide k-step][lane][8 halfs].
__device__ __forceinline__ size_t xch_offset(int r, int k, int nks) {
    return (size_t(r / 16) * nks + k / 32) * 512 + ((r % 16) + 16 * ((k % 32) / 8)) * 8 + (k % 8);
}

// One A-fragment through compiler-visible loads: two 8-byte device-scope relaxed atomic loads
// (L1 bypass, served by the XCD's L2).  Used by the step-wise / non-resident path.
__device__ __forceinline__ half8 ld_frag(const half_t* frag_lane) {
    union { u64 q[2]; half8 h; } u;
    u.q[0] = __hip_atomic_load(reinterpret_cast<const u64*>(frag_lane), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    u.q[1] = __hip_atomic_load(reinterpret_cast<const u64*>(frag_lane) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return u.h;
}

// The persistent kernels fetch fragments with ONE 16-byte load per lane carrying the device-scope bit
// (sc1: bypass the per-CU L1, hit the L2).  A CU's vector-memory path costs the same per instruction
// whether a lane moves 8 or 16 bytes: 8-byte loads top out at ~24 B/clk per CU, 16-byte loads at
// ~54 B/clk (measured), and the backward step is bound by exactly this fetch.  The compiler offers no
// 16-byte load with that scope, hence the two small asm helpers.  Loads return in issue order, so
// waiting until at most N younger loads are outstanding guarantees that everything issued before
// them has landed; the registers are listed as operands of the wait so that no consumer can be
// scheduled above it.
__device__ __forceinline__ void ld_frag_async(half8& dst, const half_t* frag_lane) {
    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(dst) : "v"(frag_lane) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_frags(half8 (&a)[4], half8 (&b)[4]) {
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3])
                 : "n"(N)
                 : "memory");
}

// acc[mt][nt] += A(32 rows x K) * Wslice, this wave's interleaved k-steps only.
// a0/a1: fragment (row tile, k-step 0) of the two 16-row tiles, already offset by lane*8 halfs.
// The last KL of a wave's KS k-steps keep their weight fragments in LDS instead of registers (wlds:
// this wave's [KL][NT][64 lanes] block); reading them back costs a few ds_read_b128 per step and frees
// 4*KL*NT registers for fragments in flight.
template <int NT, int KS, bool RESIDENT, int KL = 0>
__device__ __forceinline__ void wave_product(floatx4 (&acc)[2][NT], const half8 (&wreg)[KS - KL][NT],
                                             const half8* wlds, const half8* wfrag_wave, const half_t* a0,
                                             const half_t* a1, int wave, int lane, int nks_total,
                                             int ks_wave) {
    if constexpr (RESIDENT && (KS % 8 == 0)) {
        // Loads and MFMAs are unconditional: k-steps beyond the real contraction length fetch a
        // clamped (finite) address and meet all-zero weight fragments.  Chunks of 4 k-steps (8
        // fragments) alternate between two register sets: one is in flight while the other feeds the
        // MFMAs.
        constexpr int NCH = KS / 4;
        half8 fa[2][4], fb[2][4];
        auto issue = [&](int c, int buf) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int kg = min((c * 4 + k) * 4 + wave, nks_total - 1);
                ld_frag_async(fa[buf][k], a0 + size_t(kg) * 512);
                ld_frag_async(fb[buf][k], a1 + size_t(kg) * 512);
            }
        };
        issue(0, 0);
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int buf = c & 1;
            if (c + 1 < NCH) {
                issue(c + 1, buf ^ 1);
                wait_frags<8>(fa[buf], fb[buf]);
            } else {
                wait_frags<0>(fa[buf], fb[buf]);
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                constexpr int KR = KS - KL;
                const int ks = c * 4 + k;
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    half8 w;
                    if (ks < KR) w = wreg[ks < KR ? ks : 0][n];
                    else w = wlds[((ks - KR) * NT + n) * kWave + lane];
                    acc[0][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[buf][k], w, acc[0][n], 0, 0, 0);
                    acc[1][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[buf][k], w, acc[1][n], 0, 0, 0);
                }
            }
        }
    } else {
        for (int k = 0; k < ks_wave; ++k) {
            const int kg = k * 4 + wave;
            if (kg >= nks_total) break;
            const half8 fa = ld_frag(a0 + size_t(kg) * 512);
            const half8 fb = ld_frag(a1 + size_t(kg) * 512);
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const half8 w = wfrag_wave[(size_t(k) * NT + n) * kWave + lane];
                acc[0][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa, w, acc[0][n], 0, 0, 0);
                acc[1][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb, w, acc[1][n], 0, 0, 0);
            }
        }
    }
}

template <int NT>
__device__ __forceinline__ void spill_partials(float* part, const floatx4 (&acc)[2][NT], int wave,
                                               int lane, int pld) {
    float* base = part + size_t(wave) * kRows * pld;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                base[(m * 16 + 4 * (lane / 16) + i) * pld + n * 16 + lane % 16] = acc[m][n][i];
}

__device__ __forceinline__ void store_h2(half_t* dst, float a, float b, bool device_scope) {
    union { half_t h[2]; unsigned u; } v;
    v.h[0] = (half_t)a;
    v.h[1] = (half_t)b;
    if (device_scope)
        __hip_atomic_store(reinterpret_cast<unsigned*>(dst), v.u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        *reinterpret_cast<unsigned*>(dst) = v.u;
}

__device__ __forceinline__ void load_h2(const half_t* src, float& a, float& b) {
    union { half_t h[2]; unsigned u; } v;
    v.u = *reinterpret_cast<const unsigned*>(src);
    a = (float)v.h[0];
    b = (float)v.h[1];
}

__device__ __forceinline__ void unpack_h2(unsigned u, float& a, float& b) {
    union { half_t h[2]; unsigned u; } v;
    v.u = u;
    a = (float)v.h[0];
    b = (float)v.h[1];
}

__device__ __forceinline__ unsigned pack_h2(float a, float b) {
    union { half_t h[2]; unsigned u; } v;
    v.h[0] = (half_t)a;
    v.h[1] = (half_t)b;
    return v.u;
}

__device__ __forceinline__ void store_u32(half_t* dst, unsigned u, bool device_scope) {
    if (device_scope)
        __hip_atomic_store(reinterpret_cast<unsigned*>(dst), u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        *reinterpret_cast<unsigned*>(dst) = u;
}

// Cycle counters of workgroup 0 per phase (only when the host passes a buffer): wait, product,
// partial exchange, pointwise, publish.
struct PhaseClock {
    long long* out;
    long long last;
    __device__ __forceinline__ void start() { if (out) last = wall_clock64(); }
    __device__ __forceinline__ void lap(int slot) {
        if (out && threadIdx.x == 0) {
            const long long now = wall_clock64();
            out[slot] += now - last;
            last = now;
        }
    }
};

// ------------------------------------------------------------------------------------ forward
// Per step and row block: [wait for h_{t-1}] -> K-split MFMA product -> partial sums through LDS ->
// pointwise cell update -> store h_t, publish -> store c_t and the activated gates -> prefetch the
// next step's x-projection.  Only the h_t store and the flag sit between this step and the next one
// of the other workgroups; everything HBM-bound (x-projection fetch, cache stores) is off that path.
template <int NT, int KS, bool RESIDENT>
__global__ __launch_bounds__(kThreads) void rec_fwd_kernel(RecFwdArgs p, RecLayout L, int t_begin,
                                                           int t_end, int ks_wave) {
    constexpr int JB = 4 * NT;    // hidden units of this slice
    constexpr int NC = 16 * NT;   // gate columns of this slice (i,f,g,o blocks of JB)
    constexpr int PLD = NC + 4;
    constexpr int NPAIR = kRows * (JB / 2);                 // unit pairs per row block
    constexpr int NP = (NPAIR + kThreads - 1) / kThreads;   // pairs per thread
    extern __shared__ __attribute__((aligned(16))) float part[];  // [4][32][PLD]
    __shared__ int lds_abort;
    __shared__ int lds_role[2];

    const Role role = make_role(L.nh, L.ng, L.gpx, L.xcd_local, p.seats, p.status, lds_role);
    if (!role.active) return;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    if (tid == 0) lds_abort = 0;
    const int hs = role.hs, g = role.g;
    const int nks_total = p.Hp / 32;
    const bool device_scope = (L.persistent != 0) && (L.xcd_local == 0);
    unsigned* gflags = p.flags + size_t(g) * 256;
    PhaseClock clk{(blockIdx.x == 0) ? p.prof : nullptr, 0};

    const half8* wfrag_wave = p.wfrag + (size_t(hs) * 4 + wave) * size_t(ks_wave) * NT * kWave;
    half8 wreg[KS][NT];
    if constexpr (RESIDENT) {
#pragma unroll
        for (int k = 0; k < KS; ++k)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                wreg[k][n] = (k < ks_wave) ? wfrag_wave[(size_t(k) * NT + n) * kWave + lane] : half8{};
    }

    const size_t gld = size_t(4) * p.Hp;
    // this thread's unit pairs: row r, units jj, jj+1 of the slice
    int pr[NP], pj[NP];
    bool pv[NP];
    float2 bs[NP][4];
#pragma unroll
    for (int q = 0; q < NP; ++q) {
        const int pidx = tid + q * kThreads;
        pv[q] = pidx < NPAIR;
        pr[q] = pv[q] ? pidx / (JB / 2) : 0;
        pj[q] = pv[q] ? (pidx % (JB / 2)) * 2 : 0;
#pragma unroll
        for (int gt = 0; gt < 4; ++gt)
            bs[q][gt] = *reinterpret_cast<const float2*>(p.bias + size_t(hs) * NC + gt * JB + pj[q]);
    }
    const int rb_count = (L.nrb - g + L.ng - 1) / L.ng;
    const bool c_in_regs = (rb_count == 1) && (t_end - t_begin > 1);
    float2 creg[NP];
    unsigned xp[NP][4];
    auto prefetch = [&](int t, int rb) {
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const int b = rb * kRows + pr[q];
            if (pv[q] && b < p.B) {
                const half_t* src = p.G + (size_t(t) * p.B + b) * gld + size_t(hs) * NC + pj[q];
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) xp[q][gt] = *reinterpret_cast<const unsigned*>(src + gt * JB);
            }
        }
    };
    if (c_in_regs) {
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const int b = g * kRows + pr[q];
            creg[q] = (pv[q] && b < p.B)
                          ? *reinterpret_cast<const float2*>(p.C + (size_t(t_begin) * p.B + b) * p.Hp + hs * JB + pj[q])
                          : float2{0.f, 0.f};
        }
    }
    prefetch(t_begin, g);
    __syncthreads();
    clk.start();

    for (int t = t_begin; t < t_end; ++t) {
        if (t > t_begin) {
            if (!wait_group(gflags, L.nh, p.epoch + unsigned(t - t_begin), p.status, p.spin_limit, &lds_abort))
                return;
        }
        clk.lap(0);
        for (int rb = g; rb < L.nrb; rb += L.ng) {
            const int row0 = rb * kRows;
            const half_t* xin = p.X + size_t(t & 1) * p.x_slot;        // h_{t-1}, fragment-major
            half_t* xout = p.X + size_t((t + 1) & 1) * p.x_slot;       // h_t
            const half_t* a0 = xin + size_t(2 * rb) * nks_total * 512 + lane * 8;
            const half_t* a1 = a0 + size_t(nks_total) * 512;
            floatx4 acc[2][NT];
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int n = 0; n < NT; ++n) acc[m][n] = floatx4{0.f, 0.f, 0.f, 0.f};
            wave_product<NT, KS, RESIDENT>(acc, wreg, nullptr, wfrag_wave, a0, a1, wave, lane, nks_total, ks_wave);
            clk.lap(1);
            spill_partials<NT>(part, acc, wave, lane, PLD);
            __syncthreads();
            clk.lap(2);

            unsigned act[NP][4], hnew[NP];
            float2 cnew[NP];
#pragma unroll
            for (int q = 0; q < NP; ++q) {
                const int b = row0 + pr[q];
                if (!(pv[q] && b < p.B)) continue;
                float z[4][2];
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) {
                    const int col = gt * JB + pj[q];
                    float s0 = 0.f, s1 = 0.f;
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const float2 v = *reinterpret_cast<const float2*>(part + (size_t(w) * kRows + pr[q]) * PLD + col);
                        s0 += v.x;
                        s1 += v.y;
                    }
                    float x0, x1;
                    unpack_h2(xp[q][gt], x0, x1);
                    z[gt][0] = s0 + x0 + bs[q][gt].x;
                    z[gt][1] = s1 + x1 + bs[q][gt].y;
                }
                const int j = hs * JB + pj[q];
                const float2 cp = c_in_regs ? creg[q]
                                            : *reinterpret_cast<const float2*>(p.C + (size_t(t) * p.B + b) * p.Hp + j);
                float cn[2], hn[2], a4[4][2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const float ig = sigmoidf_dev(z[0][u]);
                    const float fg = sigmoidf_dev(z[1][u]);
                    const float gg = tanhf_dev(z[2][u]);
                    const float og = sigmoidf_dev(z[3][u]);
                    cn[u] = fg * (u == 0 ? cp.x : cp.y) + ig * gg;
                    hn[u] = og * tanhf_dev(cn[u]);
                    a4[0][u] = ig; a4[1][u] = fg; a4[2][u] = gg; a4[3][u] = og;
                }
                // the exchanged value goes out first
                hnew[q] = pack_h2(hn[0], hn[1]);
                store_u32(xout + xch_offset(b, j, nks_total), hnew[q], device_scope);
                cnew[q] = float2{cn[0], cn[1]};
                creg[q] = cnew[q];
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) act[q][gt] = pack_h2(a4[gt][0], a4[gt][1]);
            }
            clk.lap(3);
            const bool last_rb = (rb + L.ng >= L.nrb);
            if (last_rb) publish(gflags, hs, p.epoch + unsigned(t - t_begin + 1));
            else __syncthreads();
            clk.lap(4);
            // caches for the backward pass: off the critical path
#pragma unroll
            for (int q = 0; q < NP; ++q) {
                const int b = row0 + pr[q];
                if (!(pv[q] && b < p.B)) continue;
                const int j = hs * JB + pj[q];
                *reinterpret_cast<float2*>(p.C + (size_t(t + 1) * p.B + b) * p.Hp + j) = cnew[q];
                *reinterpret_cast<unsigned*>(p.Y + (size_t(t + 1) * p.B + b) * p.Hp + j) = hnew[q];
                half_t* dst = p.G + (size_t(t) * p.B + b) * gld + size_t(hs) * NC + pj[q];
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) *reinterpret_cast<unsigned*>(dst + gt * JB) = act[q][gt];
            }
            // x-projection of the next work item
            int nt_ = t, nrb_ = rb + L.ng;
            if (nrb_ >= L.nrb) { nt_ = t + 1; nrb_ = g; }
            if (nt_ < t_end) prefetch(nt_, nrb_);
        }
    }
}

// ----------------------------------------------------------------------------------- backward
// Gate order and the pointwise derivative follow flashlstm_v2/src/lstm_backward.cu:199-211, except
// that c_{t-1}, c_t come from the cell-state cache instead of being rebuilt through atanh.
template <int NT, int KS, bool RESIDENT, int KL>
__global__ __launch_bounds__(kThreads) void rec_bwd_kernel(RecBwdArgs p, RecLayout L, int t_first,
                                                           int t_last, int ks_wave) {
    constexpr int JB = 16 * NT;  // hidden units (= output columns of dG*W_hh) of this slice
    constexpr int PLD = JB + 4;
    constexpr int KR = KS - KL;  // k-steps whose weight fragments stay in registers
    constexpr int NPAIR = kRows * (JB / 2);
    constexpr int NP = (NPAIR + kThreads - 1) / kThreads;
    extern __shared__ __attribute__((aligned(16))) float part[];  // [4][32][PLD], reused for db
    __shared__ int lds_abort;
    __shared__ int lds_role[2];

    const Role role = make_role(L.nh, L.ng, L.gpx, L.xcd_local, p.seats, p.status, lds_role);
    if (!role.active) return;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    if (tid == 0) lds_abort = 0;
    const int hs = role.hs, g = role.g;
    const int nks_total = p.Hp / 8;  // contraction over 4Hp packed gate columns
    const bool device_scope = (L.persistent != 0) && (L.xcd_local == 0);
    unsigned* gflags = p.flags + size_t(g) * 256;
    const float S = p.dy_scale;
    PhaseClock clk{(blockIdx.x == 0) ? p.prof : nullptr, 0};

    const half8* wfrag_wave = p.wfrag + (size_t(hs) * 4 + wave) * size_t(ks_wave) * NT * kWave;
    half8 wreg[KR][NT];
    // LDS: [partials 4*32*PLD floats | weight fragments of the last KL k-steps, one block per wave]
    half8* wlds = reinterpret_cast<half8*>(part + 4 * kRows * PLD) + size_t(wave) * KL * NT * kWave;
    if constexpr (RESIDENT) {
#pragma unroll
        for (int k = 0; k < KR; ++k)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                wreg[k][n] = (k < ks_wave) ? wfrag_wave[(size_t(k) * NT + n) * kWave + lane] : half8{};
#pragma unroll
        for (int k = 0; k < KL; ++k)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                wlds[(k * NT + n) * kWave + lane] =
                    (KR + k < ks_wave) ? wfrag_wave[(size_t(KR + k) * NT + n) * kWave + lane] : half8{};
    }

    const size_t gld = size_t(4) * p.Hp;
    const int JF = p.jb_fwd;
    int pr[NP], pj[NP];
    bool pv[NP];
    size_t pq[NP];  // packed gate column of (unit j, gate 0)
#pragma unroll
    for (int q = 0; q < NP; ++q) {
        const int pidx = tid + q * kThreads;
        pv[q] = pidx < NPAIR;
        pr[q] = pv[q] ? pidx / (JB / 2) : 0;
        pj[q] = pv[q] ? (pidx % (JB / 2)) * 2 : 0;
        const int j = hs * JB + pj[q];
        pq[q] = size_t(j / JF) * 4 * JF + (j % JF);
    }
    const int rb_count = (L.nrb - g + L.ng - 1) / L.ng;
    const bool dc_in_regs = (rb_count == 1) && (t_first - t_last > 0);
    float2 dcreg[NP];
    if (dc_in_regs) {
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const int b = g * kRows + pr[q];
            dcreg[q] = (pv[q] && b < p.B) ? *reinterpret_cast<const float2*>(p.dC + size_t(b) * p.Hp + hs * JB + pj[q])
                                          : float2{0.f, 0.f};
        }
    }
    // prefetched per work item: activated gates, c_{t-1}, c_t, dY_t
    unsigned pg[NP][4], pdy[NP];
    float2 pcp[NP], pcc[NP];
    auto prefetch = [&](int t, int rb) {
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const int b = rb * kRows + pr[q];
            if (pv[q] && b < p.B) {
                const int j = hs * JB + pj[q];
                const half_t* gsrc = p.G + (size_t(t) * p.B + b) * gld + pq[q];
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) pg[q][gt] = *reinterpret_cast<const unsigned*>(gsrc + gt * JF);
                pcp[q] = *reinterpret_cast<const float2*>(p.C + (size_t(t) * p.B + b) * p.Hp + j);
                pcc[q] = *reinterpret_cast<const float2*>(p.C + (size_t(t + 1) * p.B + b) * p.Hp + j);
                pdy[q] = *reinterpret_cast<const unsigned*>(p.dY + (size_t(t) * p.B + b) * p.Hp + j);
            }
        }
    };
    if (t_first >= 0) prefetch(t_first, g);
    __syncthreads();
    float dbacc[4][2] = {{0.f, 0.f}, {0.f, 0.f}, {0.f, 0.f}, {0.f, 0.f}};
    clk.start();

    for (int t = t_first; t >= t_last; --t) {
        const bool from_product = (t < p.T - 1);
        if (t < t_first) {
            if (!wait_group(gflags, L.nh, p.epoch + unsigned(t_first - t), p.status, p.spin_limit, &lds_abort))
                return;
        }
        clk.lap(0);
        for (int rb = g; rb < L.nrb; rb += L.ng) {
            const int row0 = rb * kRows;
            if (from_product) {
                const half_t* xin = p.X + size_t((t + 1) & 1) * p.x_slot;   // dG_{t+1}, fragment-major
                const half_t* a0 = xin + size_t(2 * rb) * nks_total * 512 + lane * 8;
                const half_t* a1 = a0 + size_t(nks_total) * 512;
                floatx4 acc[2][NT];
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int n = 0; n < NT; ++n) acc[m][n] = floatx4{0.f, 0.f, 0.f, 0.f};
                wave_product<NT, KS, RESIDENT, KL>(acc, wreg, wlds, wfrag_wave, a0, a1, wave, lane, nks_total, ks_wave);
                clk.lap(1);
                spill_partials<NT>(part, acc, wave, lane, PLD);
                __syncthreads();
                clk.lap(2);
            }
            float2 dcnew[NP];
            unsigned dgnew[NP][4];
            half_t* xout = p.X + size_t(t & 1) * p.x_slot;   // dG_t for the peers
#pragma unroll
            for (int q = 0; q < NP; ++q) {
                const int b = row0 + pr[q];
                if (!(pv[q] && b < p.B)) continue;
                const int j = hs * JB + pj[q];
                const size_t sidx = size_t(b) * p.Hp + j;
                float dh[2];
                if (from_product) {
                    dh[0] = 0.f; dh[1] = 0.f;
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const float2 v = *reinterpret_cast<const float2*>(part + (size_t(w) * kRows + pr[q]) * PLD + pj[q]);
                        dh[0] += v.x;
                        dh[1] += v.y;
                    }
                } else {
                    const float2 v = *reinterpret_cast<const float2*>(p.dHn + sidx);
                    dh[0] = v.x; dh[1] = v.y;
                }
                if (t < 0) {  // closing pass: gradient wrt h0; dc0 is the running dc
                    *reinterpret_cast<float2*>(p.dH0 + sidx) = float2{dh[0], dh[1]};
                    if (dc_in_regs) *reinterpret_cast<float2*>(p.dC + sidx) = dcreg[q];
                    continue;
                }
                float dy0, dy1;
                unpack_h2(pdy[q], dy0, dy1);
                dh[0] += S * dy0;
                dh[1] += S * dy1;
                float2 dcin;
                if (dc_in_regs) {
                    dcin = dcreg[q];
                } else {
                    union { u64 q64; float2 f; } dcu;
                    dcu.q64 = __hip_atomic_load(reinterpret_cast<const u64*>(p.dC + sidx), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    dcin = dcu.f;
                }
                float gate[4][2];
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) unpack_h2(pg[q][gt], gate[gt][0], gate[gt][1]);
                float da[4][2], dcp[2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const float ig = gate[0][u], fg = gate[1][u], gg = gate[2][u], og = gate[3][u];
                    const float tc = tanhf_dev(u == 0 ? pcc[q].x : pcc[q].y);
                    const float cpv = (u == 0) ? pcp[q].x : pcp[q].y;
                    const float dcn = (u == 0) ? dcin.x : dcin.y;
                    const float dov = dh[u] * tc;
                    const float dc = dcn + dh[u] * og * (1.f - tc * tc);
                    da[0][u] = dc * gg * ig * (1.f - ig);
                    da[1][u] = dc * cpv * fg * (1.f - fg);
                    da[2][u] = dc * ig * (1.f - gg * gg);
                    da[3][u] = dov * og * (1.f - og);
                    dcp[u] = dc * fg;
                }
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) {
                    // db sums the values the weight-gradient GEMMs will see (fp16-rounded)
                    const unsigned u32 = pack_h2(da[gt][0], da[gt][1]);
                    float r0, r1;
                    unpack_h2(u32, r0, r1);
                    dbacc[gt][0] += r0;
                    dbacc[gt][1] += r1;
                    dgnew[q][gt] = u32;
                    store_u32(xout + xch_offset(b, int(pq[q]) + gt * JF, nks_total), u32, device_scope);
                }
                dcnew[q] = float2{dcp[0], dcp[1]};
                dcreg[q] = dcnew[q];
            }
            clk.lap(3);
            const bool last_rb = (rb + L.ng >= L.nrb);
            if (last_rb && t >= 0) publish(gflags, hs, p.epoch + unsigned(t_first - t + 1));
            else __syncthreads();
            clk.lap(4);
            if (t >= 0) {   // row-major dG for the GEMMs that follow; running dc when it lives in memory
#pragma unroll
                for (int q = 0; q < NP; ++q) {
                    const int b = row0 + pr[q];
                    if (!(pv[q] && b < p.B)) continue;
                    half_t* gdst = p.dG + (size_t(t) * p.B + b) * gld + pq[q];
#pragma unroll
                    for (int gt = 0; gt < 4; ++gt) *reinterpret_cast<unsigned*>(gdst + gt * JF) = dgnew[q][gt];
                    if (!dc_in_regs) *reinterpret_cast<float2*>(p.dC + size_t(b) * p.Hp + hs * JB + pj[q]) = dcnew[q];
                }
            }
            int nt_ = t, nrb_ = rb + L.ng;
            if (nrb_ >= L.nrb) { nt_ = t - 1; nrb_ = g; }
            if (nt_ >= t_last && nt_ >= 0) prefetch(nt_, nrb_);
        }
    }
    // single-step launches leave dc in memory for the next launch
    if (dc_in_regs && t_last >= 0) {
#pragma unroll
        for (int q = 0; q < NP; ++q) {
            const int b = g * kRows + pr[q];
            if (pv[q] && b < p.B) *reinterpret_cast<float2*>(p.dC + size_t(b) * p.Hp + hs * JB + pj[q]) = dcreg[q];
        }
    }

    // Bias gradient: fold this launch's sums over the threads that share a unit pair (fixed order).
    __syncthreads();
    float* red = part;  // [256][8]
#pragma unroll
    for (int gt = 0; gt < 4; ++gt) {
        red[tid * 8 + gt * 2 + 0] = dbacc[gt][0];
        red[tid * 8 + gt * 2 + 1] = dbacc[gt][1];
    }
    __syncthreads();
    constexpr int PAIRS = JB / 2;
    if (tid < PAIRS * 8) {
        const int prr = tid / 8, e = tid % 8;  // pair, (gate, unit)
        float sum = 0.f;
        for (int k = prr; k < kThreads; k += PAIRS) sum += red[k * 8 + e];
        const int gt = e / 2, u = e % 2;
        const int j = hs * JB + prr * 2 + u;
        const size_t q = size_t(j / JF) * 4 * JF + size_t(gt) * JF + (j % JF);
        p.db_part[size_t(g) * gld + q] += sum;
    }
}

// rows x cols row-major (ld) -> fragment-major exchange layout (one thread per pair of halfs)
__global__ void to_exchange_layout_kernel(const half_t* __restrict__ in, int rows, int cols, size_t ld,
                                          half_t* __restrict__ out, int nks) {
    const size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t pairs = size_t(rows) * (cols / 2);
    if (idx >= pairs) return;
    const int r = int(idx / (cols / 2)), k = int(idx % (cols / 2)) * 2;
    *reinterpret_cast<unsigned*>(out + xch_offset(r, k, nks)) = *reinterpret_cast<const unsigned*>(in + size_t(r) * ld + k);
}

template <typename K>
hipError_t raise_lds(K kernel, size_t bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes));
}

}  // namespace

hipError_t to_exchange_layout(const half_t* in, int rows, int cols, size_t ld, half_t* out, hipStream_t s) {
    if (rows <= 0 || cols <= 0) return hipSuccess;
    if (cols % 32 != 0) return hipErrorInvalidValue;
    const size_t pairs = size_t(rows) * (cols / 2);
    hipLaunchKernelGGL(to_exchange_layout_kernel, dim3(unsigned((pairs + 255) / 256)), dim3(256), 0, s, in, rows, cols,
                       ld, out, cols / 32);
    return hipGetLastError();
}

size_t exchange_slot_halfs(int rows, int cols) { return round_up(size_t(rows), 32) * size_t(cols); }

int rec_fwd_ks(const RecLayout&, int Hp) { return int(ceil_div(size_t(Hp) / 32, 4)); }
int rec_bwd_ks(const RecLayout&, int Hp) { return int(ceil_div(size_t(Hp) / 8, 4)); }

static void finish_layout(RecLayout& L, int B, int Hp, int num_cus, bool force_stepwise, bool fits) {
    L.nh = Hp / L.jb;
    L.nrb = int(ceil_div(size_t(B), size_t(kRows)));
    L.resident = fits ? 1 : 0;
    L.xcd_local = 0;
    L.gpx = 0;
    if (!fits || force_stepwise || L.nh > num_cus) {
        L.persistent = 0;
        L.ng = L.nrb;
        L.grid = L.ng * L.nh;
        return;
    }
    L.persistent = 1;
    if (num_cus == 256 && L.nh <= 32) {
        L.xcd_local = 1;
        L.gpx = 32 / L.nh;
        L.ng = L.nrb < 8 * L.gpx ? L.nrb : 8 * L.gpx;
        L.grid = 256;
    } else {
        const int cap = num_cus / L.nh;
        L.ng = L.nrb < cap ? L.nrb : cap;
        L.grid = L.ng * L.nh;
    }
}

RecLayout plan_rec_fwd(int B, int Hp, int num_cus, bool force_stepwise) {
    RecLayout L{};
    bool fits = true;
    if (Hp <= 1024) L.nt = 8;
    else if (Hp <= 2048) L.nt = 4;
    else { L.nt = 8; fits = false; }
    L.jb = 4 * L.nt;
    finish_layout(L, B, Hp, num_cus, force_stepwise, fits);
    return L;
}

RecLayout plan_rec_bwd(int B, int Hp, int num_cus, bool force_stepwise) {
    RecLayout L{};
    bool fits = true;
    if (Hp <= 1024) L.nt = 2;
    else if (Hp <= 2048) L.nt = 1;
    else { L.nt = 2; fits = false; }
    L.jb = 16 * L.nt;
    finish_layout(L, B, Hp, num_cus, force_stepwise, fits);
    return L;
}

template <int NT, int KS, bool RES>
static hipError_t run_fwd(const RecLayout& L, const RecFwdArgs& a, hipStream_t stream) {
    auto kernel = rec_fwd_kernel<NT, KS, RES>;
    const size_t lds = size_t(4) * kRows * (16 * NT + 4) * sizeof(float);
    hipError_t e = raise_lds(kernel, lds);
    if (e != hipSuccess) return e;
    const int ks_wave = rec_fwd_ks(L, a.Hp);
    if (L.persistent) {
        hipLaunchKernelGGL(kernel, dim3(L.grid), dim3(kThreads), lds, stream, a, L, 0, a.T, ks_wave);
        return hipGetLastError();
    }
    for (int t = 0; t < a.T; ++t) {
        hipLaunchKernelGGL(kernel, dim3(L.grid), dim3(kThreads), lds, stream, a, L, t, t + 1, ks_wave);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_rec_fwd(const RecLayout& L, const RecFwdArgs& a, hipStream_t stream) {
    if (a.T <= 0 || a.B <= 0) return hipSuccess;
    if (a.Hp % 32 != 0 || a.Hp % L.jb != 0) return hipErrorInvalidValue;
    if (!L.resident) return run_fwd<8, 1, false>(L, a, stream);
    if (L.nt == 8) return run_fwd<8, 8, true>(L, a, stream);
    if (L.nt == 4) return run_fwd<4, 16, true>(L, a, stream);
    return hipErrorInvalidValue;
}

template <int NT, int KS, bool RES, int KL>
static hipError_t run_bwd(const RecLayout& L, const RecBwdArgs& a, hipStream_t stream) {
    auto kernel = rec_bwd_kernel<NT, KS, RES, KL>;
    static_assert(size_t(4) * kRows * (16 * NT + 4) >= size_t(kThreads) * 8, "db reduction reuses the partial-sum area");
    const size_t lds = size_t(4) * kRows * (16 * NT + 4) * sizeof(float) + size_t(4) * KL * NT * kWave * sizeof(half8);
    hipError_t e = raise_lds(kernel, lds);
    if (e != hipSuccess) return e;
    const int ks_wave = rec_bwd_ks(L, a.Hp);
    if (L.persistent) {
        hipLaunchKernelGGL(kernel, dim3(L.grid), dim3(kThreads), lds, stream, a, L, a.T - 1, -1, ks_wave);
        return hipGetLastError();
    }
    for (int t = a.T - 1; t >= -1; --t) {
        hipLaunchKernelGGL(kernel, dim3(L.grid), dim3(kThreads), lds, stream, a, L, t, t, ks_wave);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_rec_bwd(const RecLayout& L, const RecBwdArgs& a, hipStream_t stream) {
    if (a.T <= 0 || a.B <= 0) return hipSuccess;
    if (a.Hp % 32 != 0 || a.Hp % L.jb != 0) return hipErrorInvalidValue;
    if (!L.resident) return run_bwd<2, 1, false, 0>(L, a, stream);
    if (L.nt == 2) return run_bwd<2, 32, true, 8>(L, a, stream);
    if (L.nt == 1) return run_bwd<1, 64, true, 16>(L, a, stream);
    return hipErrorInvalidValue;
}

}  // namespace flstm_hip
