// Persistent W_hh-resident LSTM recurrence for gfx950: forward and backward-through-time.
//
// What the reference does per time step with a CUTLASS GEMM launch plus a pointwise launch
// (forward: src/lstm.cu:1241-1339 + src/kernels.cu:86-164; backward:
// flashlstm_v2/src/lstm_backward.cu:1057-1101 + :158-227) is done here by ONE kernel launch for
// the whole sequence:
//
//  * Work split.  The batch is cut into blocks of 32 rows (two 16-row MFMA tiles; blocks of 16 rows
//    when all of those can run side by side, which halves every workgroup's work per step) and the
//    hidden dimension into slices of JB units.  A workgroup (4 wavefronts, one per SIMD, up to 512
//    registers each) owns one slice for all row blocks of its group, i.e. all four gates of its
//    hidden units, so the cell update is local; the cell state of its first two row blocks never
//    leaves registers.  Its part of W_hh (forward: 4*JB gate rows x Hp; backward: 4Hp gate rows x
//    JB columns) is loaded once into registers (and, backward, partly LDS) as ready-made MFMA
//    B-fragments and stays there.
//  * K split.  The four wavefronts split the contraction dimension (interleaved 32-wide k-steps),
//    so every element of h_{t-1} / dG_{t+1} is fetched exactly once per workgroup, straight from
//    L2 into A-fragments; partial sums meet in LDS (fp32) and the pointwise stage reads them there.
//  * Exchange.  h_t (forward) and dG_t (backward) are the only data that cross workgroups.  Groups
//    are laid out so that all workgroups of a group sit on one XCD when the slice count allows:
//    producers use plain write-through stores, consumers fetch with device-scope loads (L1 bypass,
//    served by that XCD's L2); no L2 write-back or invalidate is ever issued.  Groups that span XCDs
//    store the exchanged values with device-scope atomic stores instead.
//    There are no flags and no barrier between workgroups: the data validates itself.  The
//    exchange ring has four slots; while a workgroup writes step t into one slot it refills its own
//    region of the slot that step t+2 will use with a pattern no fp16 result can produce (0xFFFF pairs,
//    a NaN payload the arithmetic never generates).  A consumer simply loads its MFMA fragments and,
//    as long as a fragment still shows the pattern, loads it again.  The refill of step t is
//    acknowledged before the values of step t+1 are stored (every step drains its memory operations
//    once, where it picks up its prefetched operands), so whoever has seen a producer's step t+1 sees,
//    in the slot of step t+2, the pattern or the new values, never what the slot held four steps ago.
//    No wait for a store acknowledgement and no flag poll sits on the path between one step and the next.
//    Every retry loop is bounded and reports through `status`.
//  * Fallback.  The same kernels launched once per step (no waits, kernel boundaries order
//    memory) serve shapes whose weights do not fit on chip, and are the safe path after a failed
//    persistent launch.
#include <cstring>
#include <type_traits>

#include "recurrent.h"

namespace flstm_hip {
namespace {

constexpr int kThreads = 256;
constexpr int kRows = 32;  // batch rows per row block at most (two 16-row MFMA tiles; kernels with MT = 1 use one)
// Floats added to a row of partial sums in LDS.  Any pad = 4 mod 8 keeps the 16-byte accesses free of bank
// conflicts (measured: 4, 12 and 20 count the same; 8 triples the conflict cycles); what the counter still
// shows is four cycles per 16-byte store, which run at half rate whatever the layout.
constexpr int kPartPad = 4;
// Register sets of fragments in the forward kernel's tile-by-tile product: one feeds the MFMAs, the others are in
// flight.  (Three sets measured the same as two at I = H = 1024, B = 256: 3.93 against 3.86 us per step.)
constexpr int kFwdBufs = 2;

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

// Pattern that marks a not-yet-written pair of halfs in the exchange ring.
constexpr unsigned kUnwritten = 0xFFFFFFFFu;

// The abort flag of a workgroup is addressed as LDS, not through a generic pointer: a generic access is a FLAT
// instruction, which may complete out of order with the vector-memory loads, so with one anywhere in a reload loop the
// compiler ends the loop with a wait for ALL outstanding loads -- the chunk requested ahead included -- and the
// prefetch distance of the products collapses to nothing.
typedef __attribute__((address_space(3))) int lds_int_t;

// How a persistent launch validates what it fetches (off for step-wise launches, where the kernel
// boundary orders memory).
struct Poll {
    bool on;
    int limit;        // reloads of one fragment chunk before the launch gives up ...
    long long ticks;  // ... or this many ticks of the constant-rate wall clock spent reloading it, whichever comes first
    int* status;      // global: 1 = gave up
    lds_int_t* lds_abort;   // workgroup: some wave gave up
};

// How a workgroup leaves a persistent kernel once one of its waves has given up (decided after a barrier, so by all
// its waves at the same point): the wave ends here.  As an instruction rather than a `return` from inside the step
// loop, which the compiler lowers to flags that are tested on the loop's ordinary way round -- a path on which the
// checker of the build (check_inflight.py) cannot tell that the wave is on its way out.
__device__ __forceinline__ void leave_kernel() { asm volatile("s_endpgm" ::: "memory"); }

// Said before a step loop: every load issued so far (the weight fragments, the state) has landed.  As an instruction
// the compiler knows, not inline assembly: otherwise it meets the loop with loads it believes outstanding and puts
// its own wait for ALL loads in front of the first MFMA of every step, behind the fragments requested ahead.
__device__ __forceinline__ void loads_landed() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0), the other counters left alone

// Bookkeeping of one more reload of something that has not arrived; true = give up (the caller leaves its reload
// loop with garbage, and the workgroup leaves the kernel at its next barrier).  The clock and the global status word
// are looked at every 256th reload only.
__device__ __forceinline__ bool poll_give_up(const Poll& poll, int& spins, long long& spin_start, int lane) {
    ++spins;
    if (spins == 1) spin_start = wall_clock64();
    if (spins > poll.limit || *static_cast<volatile lds_int_t*>(poll.lds_abort) != 0 ||
        ((spins & 255) == 0 &&
         (wall_clock64() - spin_start > poll.ticks ||
          __hip_atomic_load(poll.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0))) {
        if (lane == 0) {
            __hip_atomic_store(poll.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *static_cast<volatile lds_int_t*>(poll.lds_abort) = 1;
        }
        return true;
    }
    return false;
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
// The same with the address as scalar base (the same for the whole wave: ring slot, row tile and k-step) + a 32-bit
// offset per lane: the k-step offsets then live in scalar registers and their arithmetic runs on the scalar unit.  For
// the kernels with two waves per SIMD, which have 256 vector registers and none to spare for addresses.
__device__ __forceinline__ void ld_frag_async_at(half8& dst, unsigned lane_off, const half_t* frag) {
    asm volatile("global_load_dwordx4 %0, %1, %2 sc1" : "=v"(dst) : "v"(lane_off), "s"(frag) : "memory");
}
// (a pointer that is the same in every lane, as a value the compiler knows to be: it then lives in scalar registers)
__device__ __forceinline__ const half_t* wave_uniform(const half_t* ptr) {
    const unsigned long long v = reinterpret_cast<unsigned long long>(ptr);
    const unsigned lo = __builtin_amdgcn_readfirstlane(unsigned(v)), hi = __builtin_amdgcn_readfirstlane(unsigned(v >> 32));
    return reinterpret_cast<const half_t*>((static_cast<unsigned long long>(hi) << 32) | lo);
}
template <int N>
__device__ __forceinline__ void wait_frags(half8 (&a)[4], half8 (&b)[4]) {
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3])
                 : "n"(N)
                 : "memory");
}
template <int N>
__device__ __forceinline__ void wait_frags(half8 (&a)[4]) {
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_frags(half8 (&a)[2]) {
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a[0]), "+v"(a[1]) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_frags(half8 (&a)[2], half8 (&b)[2]) {
    asm volatile("s_waitcnt vmcnt(%4)" : "+v"(a[0]), "+v"(a[1]), "+v"(b[0]), "+v"(b[1]) : "n"(N) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_frags(half8 (&a)[8], half8 (&b)[8]) {
    asm volatile("s_waitcnt vmcnt(%16)"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]), "+v"(b[0]),
                   "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7])
                 : "n"(N)
                 : "memory");
}
template <int N>
__device__ __forceinline__ void wait_frags(half8 (&a)[8]) {
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7])
                 : "n"(N)
                 : "memory");
}

// The same with the count as a value: for callers whose count is a constant only after unrolling.
template <int NF>
__device__ __forceinline__ void wait_frags_upto(half8 (&a)[NF], int younger) {
    switch (younger) {
#define FLSTM_WAIT_CASE(n) case n: wait_frags<n>(a); break;
        FLSTM_WAIT_CASE(1) FLSTM_WAIT_CASE(2) FLSTM_WAIT_CASE(3) FLSTM_WAIT_CASE(4) FLSTM_WAIT_CASE(5) FLSTM_WAIT_CASE(6)
        FLSTM_WAIT_CASE(7) FLSTM_WAIT_CASE(8) FLSTM_WAIT_CASE(9) FLSTM_WAIT_CASE(10) FLSTM_WAIT_CASE(11) FLSTM_WAIT_CASE(12)
        FLSTM_WAIT_CASE(13) FLSTM_WAIT_CASE(14) FLSTM_WAIT_CASE(15) FLSTM_WAIT_CASE(16) FLSTM_WAIT_CASE(17) FLSTM_WAIT_CASE(18)
        FLSTM_WAIT_CASE(19) FLSTM_WAIT_CASE(20) FLSTM_WAIT_CASE(21) FLSTM_WAIT_CASE(22) FLSTM_WAIT_CASE(23) FLSTM_WAIT_CASE(24)
#undef FLSTM_WAIT_CASE
        default: wait_frags<0>(a); break;   // (0, and anything larger than listed: waiting for more is always safe)
    }
}

// Which of a wave's KS k-steps keep their weight fragments in LDS (KL of them, spread evenly) and where the others sit
// in the register array.
__host__ __device__ constexpr int wlds_before(int ks, int KS, int KL) { return ks * KL / KS; }          // LDS k-steps below ks
__host__ __device__ constexpr bool wlds_has(int ks, int KS, int KL) { return wlds_before(ks + 1, KS, KL) > wlds_before(ks, KS, KL); }
__host__ __device__ constexpr int wreg_slot(int ks, int KS, int KL) { return ks - wlds_before(ks, KS, KL); }

// Validation by effect (LAZY).  A word of the ring that still holds the 'unwritten' pattern is a pair of fp16 NaNs, and
// a NaN anywhere in row r of the fetched operand makes EVERY column of row r of the product NaN (NaN times anything, a
// zero weight included, is NaN, and sums keep it).  With the operands swapped a lane holds row lane % 16 of each row
// tile in every one of its accumulation registers, so one register per row tile tells whether the wave multiplied
// something its producers had not written yet: two instructions per product instead of a maximum over every fetched
// word (10 vector instructions per chunk of 4 fragments).  A LAZY product checks its FIRST chunk word by word -- that
// is where a wave waits for its producers, and they finish within a fraction of a microsecond of each other -- and,
// if it did have to wait there, the chunks it had requested ahead by then; it multiplies the rest as it lands and
// repeats the wave's part of the product with every chunk checked if the result says so.  Values that are NaN in
// their own right (or sums of opposite infinities) take that second pass too and come out as what they are.
// Measured, this pays only where a wave finds its operand complete when it gets there (several row blocks per
// workgroup and step: forward at 2048 units and 128 rows 6.7 -> 6.2 us per step).  A wave that arrives ahead of its
// producers -- one row block per step, every configuration of 1024 units -- runs into words that were fetched too
// early often enough for the repeated products to cost more than the checks save (256 rows at 1024 units, backward:
// 4.9 -> 5.3 us per step; 64 rows at 2048 units: 7.3 -> 11.3), so every other kernel checks every chunk (LAZY = false).
// Checking one word per 16-byte fragment lane instead of four, with the same probe as safety net, was measured too:
// 120 vector instructions fewer per backward step and no change in time (the checks run in the shadow of the MFMAs).
template <int MT, int NT>
__device__ __forceinline__ bool product_poisoned(const floatx4 (&acc)[2][NT]) {
    float probe = acc[0][0][0];
    if constexpr (MT == 2) probe += acc[1][0][0];
    return __any(probe != probe) != 0;
}

// The same product for row blocks of two 16-row tiles whose producers publish the tiles one after the other (the
// pointwise stage of a step handles rows 0..15 first, stores them, then rows 16..31): all k-steps of tile 0 are
// fetched and multiplied before tile 1 is touched, so the first half of a step's product runs while the peers are
// still busy with the second half of their cell updates.  Chunks of CKT k-steps of ONE tile alternate between two
// register sets (as many registers as the two-tile chunks of wave_product).  Resident weights only.
template <int NT, int KS, int KL, int NPF, int NBUF, bool LAZY = false, int CKO = 0, bool REASK = false, int NW = 4, typename Prefetch>
__device__ __forceinline__ bool wave_product_tiles(floatx4 (&acc)[2][NT], const half8 (&wreg)[KS - KL][NT],
                                                   const half8* wlds, const half_t* a0, const half_t* a1, int wave,
                                                   int lane, int nks_total, int ks_wave, int rotation, const Poll& poll,
                                                   Prefetch&& prefetch) {
    static_assert(KS % 8 == 0, "whole chunks");
    constexpr int CKT = CKO ? CKO : ((KS >= 16) ? 8 : 4);
    constexpr int NCHK = KS / CKT;      // chunks per tile
    constexpr int NCH = 2 * NCHK;
    static_assert(NBUF >= 2 && NBUF <= NCH, "register sets: one feeds the MFMAs, the others are in flight");
    half8 f[NBUF][CKT];
    bool check_all = !LAZY;   // second pass: every chunk is checked word by word
    bool early = false;
    bool ahead_of_producers = false;   // the very first chunk was not there yet (returned: see FirstRequestDelay)
    for (;;) {
    // (the operand's address as a value the compiler cannot see through: the fragment addresses are then computed
    // where they are used in every pass instead of all of them ahead of this loop, in registers that are not there)
    const half_t *p0 = a0, *p1 = a1;
    if constexpr (LAZY) asm volatile("" : "+v"(p0), "+v"(p1));
    auto issue = [&](int c) {
        const half_t* base = (c / NCHK) ? p1 : p0;
#pragma unroll
        for (int k = 0; k < CKT; ++k) {
            const int kg = min(rec_kstep_of_slot((c % NCHK) * CKT + k, rotation, ks_wave) * NW + wave, nks_total - 1);
            ld_frag_async(f[c % NBUF][k], base + size_t(kg) * 512);
        }
    };
#pragma unroll
    for (int c = 0; c < NBUF - 1; ++c) issue(c);
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int buf = c % NBUF;
        const int last_issued = (c + NBUF - 1 < NCH) ? c + NBUF - 1 : NCH - 1;   // after this iteration's issue
        if (c + NBUF - 1 < NCH) {
            issue(c + NBUF - 1);
            if (c + NBUF - 1 == NCH - 1) prefetch();
        }
        // this chunk's weight fragments that live in LDS: requested now, they arrive while the wave waits for the
        // chunk's operand fragments (as in wave_product)
        half8 wl[CKT][NT];
#pragma unroll
        for (int k = 0; k < CKT; ++k)
            if (wlds_has((c % NCHK) * CKT + k, KS, KL)) {
#pragma unroll
                for (int n = 0; n < NT; ++n) wl[k][n] = wlds[(wlds_before((c % NCHK) * CKT + k, KS, KL) * NT + n) * kWave + lane];
            }
        // loads return in issue order: chunk c has landed once at most the loads issued after it are outstanding
        const int younger = (last_issued - c) * CKT + ((last_issued == NCH - 1) ? NPF : 0);
        wait_frags_upto(f[buf], younger);   // (a compile-time constant in every unrolled iteration: the switch folds)
        // A pair of halfs that still holds the pattern has not been written yet by its producer: fetch the chunk
        // again (whatever was in flight behind it lands first, loads return in order).  The decision is wave-uniform.
        // The check is peeled out of the reload loop: a chunk that is complete -- nearly all of them -- then costs the
        // comparison and ONE branch that is not taken; every taken branch stalls a wave that has its SIMD to itself.
        auto unwritten = [&]() -> bool {
            unsigned m = 0u;
#pragma unroll
            for (int k = 0; k < CKT; ++k) {
                const uint4 ua = __builtin_bit_cast(uint4, f[buf][k]);
                m = max(m, max(max(ua.x, ua.y), max(ua.z, ua.w)));
            }
            return __any(m == kUnwritten) != 0;
        };
        // LAZY: only the first chunk of a tile is checked here -- the wave waits there for its producers -- and the
        // rest by their effect on the result (product_poisoned)
        // (early: this tile's first chunk had to be fetched again, i.e. the wave got here before its producers; the
        // chunks requested ahead of that moment are then checked as well)
        const bool ahead = (c % NCHK) >= 1 && (c % NCHK) <= NBUF - 1;
        if (c % NCHK == 0) early = false;
        if (c % NCHK == 0 || (ahead && early) || __builtin_expect(check_all, 0)) {
            if (__builtin_expect(unwritten() && poll.on, 0)) {
                if (c % NCHK == 0) early = true;
                if (c == 0) ahead_of_producers = true;
                int spins = 0;
                long long spin_start = 0;
                do {
                    if (poll_give_up(poll, spins, spin_start, lane)) break;   // results are garbage from here on; the workgroup leaves at its next barrier
                    // The chunks requested ahead of this one went out at the same moment and are as stale: left alone,
                    // each of them is found unwritten in its turn and costs a round trip of its own.  REASK requests
                    // them again behind this chunk, so that the wave leaves this loop with fresh ones in flight.  That
                    // pays where a round trip is long (groups that span XCDs: 2048 units and 16 rows, forward
                    // 3.00 -> 2.85 us per step) and costs where it is short and the polls share one L2 (1024 units and
                    // 256 rows, forward 3.56 -> 3.8: twice the poll traffic in front of the producers' stores).
                    issue(c);
                    if constexpr (REASK) {
#pragma unroll
                        for (int j = c + 1; j <= last_issued; ++j) issue(j);
                        wait_frags_upto(f[buf], (last_issued - c) * CKT);   // (what was in flight before has landed as well)
                    } else {
                        wait_frags<0>(f[buf]);   // (whatever was in flight behind this chunk has landed as well)
                    }
                } while (unwritten());
            }
        }
#pragma unroll
        for (int k = 0; k < CKT; ++k) {
            const int ks = (c % NCHK) * CKT + k;
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                half8 w;
                if (!wlds_has(ks, KS, KL)) w = wreg[wreg_slot(ks, KS, KL)][n];
                else w = wl[k][n];
                acc[c / NCHK][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, f[buf][k], acc[c / NCHK][n], 0, 0, 0);
            }
        }
        // (chunks stay apart: without the checks between them the product is one long block, and a scheduler free to
        // move the address arithmetic of later chunks up runs out of registers)
        if constexpr (LAZY) __builtin_amdgcn_sched_barrier(0);
    }
    if (__builtin_expect(check_all || !poll.on || !product_poisoned<2>(acc), 1)) break;
    check_all = true;
    // Whatever this pass left in flight (the loads of `prefetch`) lands before the next one starts: that pass issues
    // them again into registers of its own, the compiler takes the old ones for dead and hands them out -- as address
    // registers, for one -- while the hardware still writes them.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[m][n] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    return ahead_of_producers;
}

// acc[mt][nt] += (A(16*MT rows x K) * Wslice)^T, this wave's interleaved k-steps only.
// a0/a1: fragment (row tile, k-step 0) of the two 16-row tiles, already offset by lane*8 halfs; with MT = 1
// (batches of at most 16 rows) the second tile is neither fetched nor multiplied.
// KL of a wave's KS k-steps keep their weight fragments in LDS instead of registers (wlds: this wave's [KL][NT][64
// lanes] block), which frees 4*KL*NT registers for fragments in flight.  They are spread evenly over the k-steps
// (wlds_has), so that every chunk holds at most its share of them and their ds_read_b128 can be issued before the
// chunk's wait for its fragments: read just in time, in front of the MFMA that needs them, each costs an LDS round
// trip (~100 clocks) of a wave that has nothing else to run.

// `prefetch` issues exactly NPF vector loads (for every wave, whatever its lanes need) behind the last
// fragment load.
template <int NT, int KS, bool RESIDENT, int KL, int NPF, int MT, int NBUF = 2, int CKO = 0, bool LAZY = false, bool REASK = false, int NW = 4, bool SADDR = (NW == 8), typename Prefetch>
__device__ __forceinline__ bool wave_product(floatx4 (&acc)[2][NT], const half8 (&wreg)[KS - KL][NT],
                                             const half8* wlds, const half8* wfrag_wave, const half_t* a0,
                                             const half_t* a1, int wave, int lane, int nks_total,
                                             int ks_wave, int rotation, const Poll& poll, Prefetch&& prefetch) {
    if constexpr (RESIDENT && (KS % 4 == 0)) {
        // Loads and MFMAs are unconditional: k-steps beyond the real contraction length fetch a
        // clamped (finite) address and meet all-zero weight fragments.  Chunks of CK k-steps (2*CK
        // fragments) alternate between two register sets: one is in flight while the other feeds the
        // MFMAs.  (Short contractions take small chunks: their kernels have no registers to spare.)
        // Chunks rotate through NBUF register sets: one feeds the MFMAs, the others are in flight (two by default; a
        // kernel that waits on a trip through memory takes more, of shorter chunks (CKO) where registers are short:
        // five sets of 2 k-steps keep as much in flight as three sets of 4 and take 5/6 of the registers).
        constexpr int CK = CKO ? CKO : ((KS >= 16) ? 4 : 2);
        constexpr int NCH = KS / CK;
        constexpr int D = NBUF - 1;   // chunks requested ahead of the one being multiplied
        half8 fa[NBUF][CK], fb[NBUF][CK];
        bool check_all = !LAZY;   // second pass: every chunk is checked word by word
        bool early = false;               // the first chunk had to be fetched again: what was requested ahead of it is checked too
        bool ahead_of_producers = false;  // ... on the first pass over the product (returned: see FirstRequestDelay)
        for (;;) {
        const half_t *p0 = a0, *p1 = a1;   // (opaque copies, as in wave_product_tiles)
        if constexpr (LAZY) asm volatile("" : "+v"(p0), "+v"(p1));
        // SADDR (kernels of two waves per SIMD): scalar base + lane offset (ld_frag_async_at)
        const unsigned lane_off = unsigned(lane) * 16u;
        const half_t *u0 = nullptr, *u1 = nullptr;
        int wv = wave;
        if constexpr (SADDR) {
            u0 = wave_uniform(a0 - lane * 8);
            u1 = wave_uniform(a1 - lane * 8);
            wv = __builtin_amdgcn_readfirstlane(wave);
        }
        auto issue = [&](int c, int buf) {
#pragma unroll
            for (int k = 0; k < CK; ++k) {
                const int kg = min(rec_kstep_of_slot(c * CK + k, rotation, ks_wave) * NW + wv, nks_total - 1);
                if constexpr (SADDR) {
                    ld_frag_async_at(fa[buf][k], lane_off, u0 + size_t(kg) * 512);
                    if constexpr (MT == 2) ld_frag_async_at(fb[buf][k], lane_off, u1 + size_t(kg) * 512);
                } else {
                    ld_frag_async(fa[buf][k], p0 + size_t(kg) * 512);
                    if constexpr (MT == 2) ld_frag_async(fb[buf][k], p1 + size_t(kg) * 512);
                }
            }
        };
        auto wait = [&](auto younger, int buf) {   // until at most `younger` loads issued later are outstanding
            constexpr int N = decltype(younger)::value;
            if constexpr (MT == 2) wait_frags<N>(fa[buf], fb[buf]);
            else wait_frags<N>(fa[buf]);
        };
#pragma unroll
        for (int j = 0; j < (D < NCH ? D : NCH); ++j) issue(j, j % NBUF);
        if (D >= NCH) prefetch();
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int buf = c % NBUF;
            if (c + D < NCH) {
                issue(c + D, (c + D) % NBUF);
                if (c + D == NCH - 1) prefetch();
            }
            // this chunk's weight fragments that live in LDS: requested now, they arrive while the wave waits for the
            // chunk's operand fragments
            half8 wl[CK][NT];
#pragma unroll
            for (int k = 0; k < CK; ++k)
                if (wlds_has(c * CK + k, KS, KL)) {
#pragma unroll
                    for (int n = 0; n < NT; ++n) wl[k][n] = wlds[(wlds_before(c * CK + k, KS, KL) * NT + n) * kWave + lane];
                }
            // requested after chunk c by now: the chunks up to c + D (or the last one), and the prefetch once the last
            // chunk is out (c, D, NCH are compile-time constants: the switch folds)
            const int last_now = (c + D < NCH - 1) ? c + D : NCH - 1;
            const bool prefetched = (c + D >= NCH - 1);
            auto wait_with = [&](int chunks_behind, bool prefetch_behind) {   // ... of chunk c; constants once unrolled
                switch (chunks_behind * 2 + (prefetch_behind ? 1 : 0)) {
                    case 0: wait(std::integral_constant<int, 0>{}, buf); break;
                    case 1: wait(std::integral_constant<int, NPF>{}, buf); break;
                    case 2: wait(std::integral_constant<int, MT * CK>{}, buf); break;
                    case 3: wait(std::integral_constant<int, MT * CK + NPF>{}, buf); break;
                    case 4: wait(std::integral_constant<int, 2 * MT * CK>{}, buf); break;
                    case 5: wait(std::integral_constant<int, 2 * MT * CK + NPF>{}, buf); break;
                    case 6: wait(std::integral_constant<int, 3 * MT * CK>{}, buf); break;
                    case 7: wait(std::integral_constant<int, 3 * MT * CK + NPF>{}, buf); break;
                    case 8: wait(std::integral_constant<int, 4 * MT * CK>{}, buf); break;
                    default: wait(std::integral_constant<int, 4 * MT * CK + NPF>{}, buf); break;
                }
            };
            wait_with(last_now - c, prefetched);
            static_assert(NBUF <= 5, "the switch above knows up to four chunks ahead");
            auto unwritten = [&]() -> bool {
                unsigned m = 0u;
#pragma unroll
                for (int k = 0; k < CK; ++k) {
                    const uint4 ua = __builtin_bit_cast(uint4, fa[buf][k]);
                    m = max(m, max(max(ua.x, ua.y), max(ua.z, ua.w)));
                    if constexpr (MT == 2) {
                        const uint4 ub = __builtin_bit_cast(uint4, fb[buf][k]);
                        m = max(m, max(max(ub.x, ub.y), max(ub.z, ub.w)));
                    }
                }
                return __any(m == kUnwritten) != 0;
            };
            if (c == 0 || (c <= D && early) || __builtin_expect(check_all, 0)) {   // (peeled; first pass: as in wave_product_tiles)
                if (__builtin_expect(unwritten() && poll.on, 0)) {
                    if (c == 0) early = true;
                    if (c == 0) ahead_of_producers = true;
                    int spins = 0;
                    long long spin_start = 0;
                    do {
                        if (poll_give_up(poll, spins, spin_start, lane)) break;
                        // (REASK: with the chunks that were requested ahead of it, which are as stale: see
                        // wave_product_tiles; not where a wave holds 64 k-steps: that kernel has no registers left
                        // for the addresses)
                        issue(c, buf);
                        if constexpr (REASK && KS < 64) {
#pragma unroll
                            for (int j = c + 1; j <= last_now; ++j) issue(j, j % NBUF);
                            wait_with(last_now - c, false);   // (also what was issued after this chunk the first time)
                        } else {
                            wait(std::integral_constant<int, 0>{}, buf);
                        }
                    } while (unwritten());
                }
            }
#pragma unroll
            for (int k = 0; k < CK; ++k) {
                const int ks = c * CK + k;
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    half8 w;
                    if (wlds_has(ks, KS, KL)) w = wl[k][n];
                    else w = wreg[wreg_slot(ks, KS, KL)][n];
                    acc[0][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, fa[buf][k], acc[0][n], 0, 0, 0);
                    if constexpr (MT == 2)
                        acc[1][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, fb[buf][k], acc[1][n], 0, 0, 0);
                }
            }
            if constexpr (LAZY) __builtin_amdgcn_sched_barrier(0);   // (chunks stay apart, as in wave_product_tiles)
        }
        if (__builtin_expect(check_all || !poll.on || !product_poisoned<MT>(acc), 1)) break;
        check_all = true;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // (as in wave_product_tiles: nothing in flight into registers the next pass reuses)
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
        return ahead_of_producers;
    } else {
        for (int k = 0; k < ks_wave; ++k) {
            const int kg = rec_kstep_of_slot(k, rotation, ks_wave) * NW + wave;
            if (kg >= nks_total) continue;
            const half8 fa = ld_frag(a0 + size_t(kg) * 512);
            half8 fb{};
            if constexpr (MT == 2) fb = ld_frag(a1 + size_t(kg) * 512);
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const half8 w = wfrag_wave[(size_t(k) * NT + n) * kWave + lane];
                acc[0][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, fa, acc[0][n], 0, 0, 0);
                if constexpr (MT == 2) acc[1][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, fb, acc[1][n], 0, 0, 0);
            }
        }
        prefetch();
        return false;
    }
}

// The products are computed transposed (weights as the first MFMA operand), so a lane ends up with four
// consecutive output columns of one batch row: tile (m, n) holds row m*16 + lane%16, columns
// n*16 + 4*(lane/16) .. +3, and goes to LDS as one 16-byte store.  The 16 rows written together are
// 4*pld banks apart; for the pitches in use that spreads them over all 64 banks.
template <int NT, int MT>
__device__ __forceinline__ void spill_partials(float* part, const floatx4 (&acc)[2][NT], int wave,
                                               int lane, int pld) {
    float* base = part + size_t(wave) * kRows * pld + size_t(lane % 16) * pld + 4 * (lane / 16);
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n)
            *reinterpret_cast<floatx4*>(base + m * 16 * pld + n * 16) = acc[m][n];
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

// The pointwise stage gives every thread one GROUP of N consecutive hidden units of one batch row
// (N = 4 for 32-unit slices, 2 for 16-unit slices: 8 groups per row, 256 groups per row block), so
// that its global accesses are as wide as the work split allows: a vector-memory instruction costs
// the same 16+ clocks of address processing whatever its width, and the steps are short enough for
// that to show.  Pack<N> is N halfs as raw bits.
template <int N> struct Pack;
template <> struct Pack<2> { unsigned v; };
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
template <> struct Pack<4> { uintx2 v; };
// N floats as one register tuple (destination of an asynchronous load)
template <int N> struct F32;
template <> struct F32<2> { floatx2 v; };
template <> struct F32<4> { floatx4 v; };

// (non-temporal: the state and gate arrays are written once per pass and read by later kernels)
__device__ __forceinline__ void st_pack(half_t* p, Pack<2> v) { __builtin_nontemporal_store(v.v, reinterpret_cast<unsigned*>(p)); }
__device__ __forceinline__ void st_pack(half_t* p, Pack<4> v) { __builtin_nontemporal_store(v.v, reinterpret_cast<uintx2*>(p)); }
__device__ __forceinline__ void unpack(Pack<2> v, float (&f)[2]) { unpack_h2(v.v, f[0], f[1]); }
__device__ __forceinline__ void unpack(Pack<4> v, float (&f)[4]) {
    unpack_h2(v.v.x, f[0], f[1]);
    unpack_h2(v.v.y, f[2], f[3]);
}
__device__ __forceinline__ Pack<2> pack(const float (&f)[2]) { return Pack<2>{pack_h2(f[0], f[1])}; }
__device__ __forceinline__ Pack<4> pack(const float (&f)[4]) {
    return Pack<4>{uintx2{pack_h2(f[0], f[1]), pack_h2(f[2], f[3])}};
}
__device__ __forceinline__ Pack<2> pack_fill(unsigned w, Pack<2>*) { return Pack<2>{w}; }
__device__ __forceinline__ Pack<4> pack_fill(unsigned w, Pack<4>*) { return Pack<4>{uintx2{w, w}}; }

// The gate values i, f, g, o of UPT consecutive hidden units as they lie in the gate arrays (x-projection / gate
// cache, dG): unit-major, 8 bytes per unit, so UPT / 2 accesses of 16 bytes.
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
template <int UPT> struct GateRow { uintx4 v[UPT / 2]; };
template <int UPT>
__device__ __forceinline__ void unpack_gates(const GateRow<UPT>& g, float (&z)[4][UPT]) {
#pragma unroll
    for (int c = 0; c < UPT / 2; ++c) {
        unpack_h2(g.v[c].x, z[0][2 * c], z[1][2 * c]);
        unpack_h2(g.v[c].y, z[2][2 * c], z[3][2 * c]);
        unpack_h2(g.v[c].z, z[0][2 * c + 1], z[1][2 * c + 1]);
        unpack_h2(g.v[c].w, z[2][2 * c + 1], z[3][2 * c + 1]);
    }
}
template <int UPT>
__device__ __forceinline__ GateRow<UPT> pack_gates(const float (&a)[4][UPT]) {
    GateRow<UPT> g;
#pragma unroll
    for (int c = 0; c < UPT / 2; ++c)
        g.v[c] = uintx4{pack_h2(a[0][2 * c], a[1][2 * c]), pack_h2(a[2][2 * c], a[3][2 * c]),
                        pack_h2(a[0][2 * c + 1], a[1][2 * c + 1]), pack_h2(a[2][2 * c + 1], a[3][2 * c + 1])};
    return g;
}
template <int UPT>
__device__ __forceinline__ GateRow<UPT> gates_fill(unsigned w) {
    GateRow<UPT> g;
#pragma unroll
    for (int c = 0; c < UPT / 2; ++c) g.v[c] = uintx4{w, w, w, w};
    return g;
}
template <int UPT>
__device__ __forceinline__ void st_gates(half_t* p, const GateRow<UPT>& g) {
#pragma unroll
    for (int c = 0; c < UPT / 2; ++c) __builtin_nontemporal_store(g.v[c], reinterpret_cast<uintx4*>(p + 8 * c));
}
// 16 bytes into the exchange ring (see below: every 32-bit word is validated on its own)
__device__ __forceinline__ void store_xch16(half_t* dst, uintx4 v, bool device_scope) {
    if (device_scope) {
        // one write-through store (device scope); issued by hand: there is no 16-byte atomic store to ask the
        // compiler for, and of two 8-byte ones it emitted the second without the scope bit
        asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
    } else {
        *reinterpret_cast<uintx4*>(dst) = v;
    }
}

// One group into the exchange ring.  Consumers validate every 32-bit word on its own, so the two words
// of an 8-byte group need not become visible together.
__device__ __forceinline__ void store_xch(half_t* dst, Pack<2> v, bool device_scope) {
    if (device_scope)
        __hip_atomic_store(reinterpret_cast<unsigned*>(dst), v.v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        *reinterpret_cast<unsigned*>(dst) = v.v;
}
__device__ __forceinline__ void store_xch(half_t* dst, Pack<4> v, bool device_scope) {
    if (device_scope) {
        const u64 w = (u64(v.v.y) << 32) | v.v.x;
        __hip_atomic_store(reinterpret_cast<u64*>(dst), w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        *reinterpret_cast<uintx2*>(dst) = v.v;
    }
}

__device__ __forceinline__ void ld_f32(const float* p, float (&f)[2]) {
    const float2 v = *reinterpret_cast<const float2*>(p);
    f[0] = v.x; f[1] = v.y;
}
__device__ __forceinline__ void ld_f32(const float* p, float (&f)[4]) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
__device__ __forceinline__ void st_f32(float* p, const float (&f)[2]) { *reinterpret_cast<float2*>(p) = float2{f[0], f[1]}; }
__device__ __forceinline__ void st_f32(float* p, const float (&f)[4]) {
    *reinterpret_cast<float4*>(p) = float4{f[0], f[1], f[2], f[3]};
}
// The same as one hand-issued load that has arrived when the call returns.  The compiler does not see
// a pending load, so it puts no wait of its own where the value is used: such a wait would sit behind
// the stores issued in between (the ring marks) and stall the step until they are acknowledged.
__device__ __forceinline__ void ld_f32_now(const float* p, float (&f)[2]) {
    floatx2 v;
    asm volatile("global_load_dwordx2 %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    f[0] = v.x; f[1] = v.y;
}
__device__ __forceinline__ void ld_f32_now(const float* p, float (&f)[4]) {
    floatx4 v;
    asm volatile("global_load_dwordx4 %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
// the same, past the L1 (the value was written by this thread through a plain store earlier on)
__device__ __forceinline__ void ld_f32_coherent(const float* p, float (&f)[2]) {
    floatx2 v;
    asm volatile("global_load_dwordx2 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    f[0] = v.x; f[1] = v.y;
}
__device__ __forceinline__ void ld_f32_coherent(const float* p, float (&f)[4]) {
    floatx4 v;
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}

// Thread -> (row, group): the 8 (or 16) groups of a row go to consecutive lanes.  The LDS serves 256 bytes per clock,
// i.e. the lanes of TOGETHER rows at once (2 rows of 128 bytes, or 4 rows of 64 bytes where 8 threads read 8 bytes
// each), so the rows are taken in the order 0, 8, 1, 9, ... (rows r and r + 8 are 32 banks apart for every row pitch
// in use: 132, 68, 36, 20 floats) or 0, 4, 8, 12, 1, 5, ... (r, r + 4, r + 8, r + 12 are 16 banks apart).
template <int TOGETHER>
__device__ __forceinline__ int group_row(int idx) {
    static_assert(TOGETHER == 2 || TOGETHER == 4, "rows whose lanes the LDS serves in one clock");
    if constexpr (TOGETHER == 4) return (idx % 4) * 4 + (idx / 4) % 4 + (idx / 16) * 16;
    return (idx % 2) * 8 + (idx / 2) % 8 + (idx / 16) * 16;
}

// Asynchronous loads of the per-step operands that come from HBM (x-projection, gate and cell caches, dY).
// They are issued by hand, right after the LAST fragment load of a step's product: loads return in issue
// order, so anything slow that sits in front of the fragment loads would hold them up, and a known number
// of them behind lets the fragment waits discount them.  The values are used only after settle().
// They carry the non-temporal hint: these arrays stream through once per pass, and their lines should not push the
// exchange ring, which is re-read every step, out of the L2.
__device__ __forceinline__ void ld_stream(uintx2& d, const void* p) {
    asm volatile("global_load_dwordx2 %0, %1, off nt" : "=v"(d) : "v"(p) : "memory");
}
__device__ __forceinline__ void ld_stream(floatx2& d, const void* p) {
    asm volatile("global_load_dwordx2 %0, %1, off nt" : "=v"(d) : "v"(p) : "memory");
}
__device__ __forceinline__ void ld_stream(unsigned& d, const void* p) {
    asm volatile("global_load_dword %0, %1, off nt" : "=v"(d) : "v"(p) : "memory");
}
__device__ __forceinline__ void ld_stream(uintx4& d, const void* p) {
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(d) : "v"(p) : "memory");
}
__device__ __forceinline__ void ld_stream(floatx4& d, const void* p) {
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(d) : "v"(p) : "memory");
}
__device__ __forceinline__ void wait_all_vm() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
template <typename T>
__device__ __forceinline__ void settle(T& x) { asm volatile("" : "+v"(x)); }   // no use of x moves above this point
__device__ __forceinline__ void to_floats(const F32<2>& r, float (&f)[2]) { f[0] = r.v.x; f[1] = r.v.y; }
__device__ __forceinline__ void to_floats(const F32<4>& r, float (&f)[4]) {
    f[0] = r.v.x; f[1] = r.v.y; f[2] = r.v.z; f[3] = r.v.w;
}

// Cycle counters of workgroup 0 per phase (only when the host passes a buffer): product (including the
// wait for the operand), partial exchange, pointwise, cache stores, wait for the prefetched operands.  Thread 0 accumulates in
// LDS and writes the totals once at the end, so the measurement adds no memory round trips to a step.
struct PhaseClock {
    long long* out;
    long long last;
    long long core_start = 0, wall_start = 0;   // slots 5 and 6: engine clocks and 100 MHz ticks of the whole launch

    __device__ __forceinline__ long long* acc() {
        __shared__ long long lds_acc[5];
        return lds_acc;
    }
    __device__ __forceinline__ void start() {
        if (out && threadIdx.x == 0) {
            for (int i = 0; i < 5; ++i) acc()[i] = 0;
            last = wall_clock64();
            wall_start = last;
            core_start = clock64();
        }
    }

    __device__ __forceinline__ void lap(int slot) {
        // (the pointer is the same for the whole workgroup: tested on its own and marked unlikely, a launch without
        // counters falls through one scalar branch instead of jumping over a masked block)
        if (__builtin_expect(out != nullptr, 0)) {
            if (threadIdx.x == 0) {
                const long long now = wall_clock64();
                acc()[slot] += now - last;
                last = now;
            }
        }
    }
    __device__ __forceinline__ void flush() {
        if (out && threadIdx.x == 0) {
            for (int i = 0; i < 5; ++i) out[i] += acc()[i];
            out[5] += clock64() - core_start;
            out[6] += wall_clock64() - wall_start;
        }
    }
};

// When to send the first request of a product.  A wave that asks before its producers have published polls, and a poll
// notices the data a full round trip after it went out; a wave that asks just after they have published has the data
// after one trip.  Where the chain from step to step is exposed (one row block per group) every wave is ahead of its
// producers at every step, by about the same time.  So a wave holds its first request back by a delay it regulates
// itself: found the first chunk unwritten -> one unit (of 64 clocks) more, found it there -> a sixteenth of a unit
// less.  It settles just behind the moment the data lands, with a miss every sixteenth step or so; where a wave is
// not ahead of its producers (several row blocks per workgroup) it decays to nothing.  Measured, forward at 2048
// units, us per step: 16 rows 2.89 -> 2.64 (the best fixed delay, 8 units: 2.56), 32 rows 3.23 -> 2.77, 64 rows
// 4.43 -> 3.73; two units up and an eighth down: 2.73 / 2.83 / 3.81.
struct FirstRequestDelay {
    static constexpr int kMost = 16 * 48;
    int sixteenths = 0;
    __device__ __forceinline__ void start_from(const int* hint) {
        if (hint) sixteenths = __builtin_amdgcn_readfirstlane(min(max(*hint, 0), kMost));
    }
    __device__ __forceinline__ void leave(int* hint) const {
        if (hint && blockIdx.x == 0 && threadIdx.x == 0) *hint = sixteenths;
    }
    __device__ __forceinline__ void hold() const {
        for (int i = 0; i < (sixteenths >> 4); ++i) __builtin_amdgcn_s_sleep(1);
    }
    __device__ __forceinline__ void learn(bool ahead_of_producers) {
        sixteenths = ahead_of_producers ? min(sixteenths + 16, kMost) : max(sixteenths - 1, 0);
    }
};

// ------------------------------------------------------------------------------------ forward
// Per step and row block: K-split MFMA product on h_{t-1} as it arrives -> partial sums through LDS
// (two buffers, one barrier per step) -> pointwise cell update -> store h_t -> store c_t and the
// activated gates -> prefetch the next step's x-projection.  Only the h_t store sits between this step
// and the next one of the other workgroups; everything HBM-bound (x-projection fetch, cache stores) is
// off that path.
// MT = 16-row tiles per row block: 2, or 1 for batches of at most 16 rows (the threads of rows 16..31 then only
// keep the barriers company).
// DEEP (2048 hidden units, 32-row blocks, several row blocks per workgroup and step): the operand comes through memory
// from the other XCDs, and a workgroup finds a block's operand complete when it gets there (it was published a block
// ago), so the product runs at the rate the fetch sustains: four sets of 2 k-steps in flight instead of two sets of 4
// (measured at 128 rows: 6.9 -> 6.4 us per step), validated by their effect on the result (product_poisoned).  With one block per step the product waits for its producers
// anyway and the longer sets are the better ones (64 rows: 4.5 against 4.65 us).
// Slices of 32 units with two row tiles run the pointwise stage in two PHASES: all 256 threads update rows 0..15
// of the block (two units each) and store that half of h_t, then rows 16..31.  The consumers fetch and multiply
// tile by tile (wave_product_tiles), so the second phase of a step overlaps the first half of the peers' next
// product instead of sitting on the path from one step to the next.
template <int NT, int KS, bool RESIDENT, int MT, bool DS, bool DEEP = false>
__global__ __launch_bounds__(kThreads) void rec_fwd_kernel(RecFwdArgs p, RecLayout L, int t_begin,
                                                           int t_end, int ks_wave) {
    constexpr int NW = 4;
    constexpr int JB = 4 * NT;    // hidden units of this slice
    constexpr int NC = 16 * NT;   // gate columns of this slice (i,f,g,o blocks of JB)
    constexpr int PLD = NC + kPartPad;
    constexpr bool SPLIT = RESIDENT && MT == 2 && JB >= 32 && (KS % 8 == 0);
    // cell updates per thread: the slice's units of one batch row are shared by GPR threads; 32 rows x 8 threads,
    // or 16 rows x 16 threads (per phase, or when a block has one row tile) where the slice is wide enough for 2 units each
    constexpr int GPR = (SPLIT || (MT == 1 && JB >= 32)) ? 16 : 8;
    constexpr int UPT = JB / GPR;
    constexpr int NPH = SPLIT ? 2 : 1;   // pointwise phases per step
    static_assert(UPT == 2 || UPT == 4, "2 or 4 hidden units per thread");
    typedef Pack<UPT> PackT;
    extern __shared__ __attribute__((aligned(16))) float part_all[];  // [2][4][32][PLD]
    __shared__ int lds_abort;
    __shared__ int lds_role[2];

    if (threadIdx.x == 0) lds_abort = 0;
    const Role role = make_role(L.nh, L.ng, L.gpx, L.xcd_local, p.seats, p.status, lds_role);
    if (!role.active) return;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int hs = role.hs, g = role.g;
    const int rotation = __builtin_amdgcn_readfirstlane(rec_kstep_rotation(hs, L.nh, ks_wave, L.rot_div));
    const int nks_total = p.Hp / 32;
    constexpr bool device_scope = DS;   // a persistent launch whose groups span XCDs (chosen by the host: no branch per store)
    const Poll poll{L.persistent != 0, p.spin_limit, p.spin_ticks, p.status, (lds_int_t*)&lds_abort};
    PhaseClock clk{(blockIdx.x == 0) ? p.prof : nullptr, 0};
    int item = 0;   // work items done: selects the partial-sum buffer
    FirstRequestDelay first_request;
    if constexpr (DS) first_request.start_from(p.delay_hint);

    const half8* wfrag_wave = p.wfrag + (size_t(hs) * NW + wave) * size_t(ks_wave) * NT * kWave;
    half8 wreg[KS][NT];
    if constexpr (RESIDENT) {
#pragma unroll
        for (int k = 0; k < KS; ++k)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                wreg[k][n] = (k < ks_wave) ? wfrag_wave[(size_t(k) * NT + n) * kWave + lane] : half8{};
    }

    const size_t gld = size_t(4) * p.Hp;
    // this thread's groups: row pr (+ 16 in the second phase) of the row block, units pj .. pj+UPT-1 of the slice
    constexpr int RB = 16 * MT;   // batch rows of a row block
    const int pr = group_row<(GPR * UPT == 16) ? 4 : 2>(tid / GPR);
    const bool row_used = pr + 16 * (NPH - 1) < RB;   // with one row tile per block the threads of rows 16..31 only keep the barriers company
    const int pj = (tid % GPR) * UPT;
    const int j = hs * JB + pj;   // first hidden unit of the group
    const int rb_count = (L.nrb - g + L.ng - 1) / L.ng;
    // the cell state of the workgroup's first and second row block stays in registers for the whole launch
    const bool c_in_regs = (rb_count <= 2) && (t_end - t_begin > 1);
    float creg[NPH][UPT] = {}, creg2[NPH][UPT] = {};
    GateRow<UPT> xp[NPH];
    auto prefetch = [&](int t, int rb) {   // NPH * UPT / 2 loads per wave; rows past B fetch row B-1 and are not used
#pragma unroll
        for (int ph = 0; ph < NPH; ++ph) {
            const int b = min(rb * RB + pr + 16 * ph, p.B - 1);
            const half_t* src = p.G + (size_t(t) * p.B + b) * gld + size_t(4) * j;
#pragma unroll
            for (int c = 0; c < UPT / 2; ++c) ld_stream(xp[ph].v[c], src + 8 * c);
        }
    };
    if (c_in_regs) {
#pragma unroll
        for (int ph = 0; ph < NPH; ++ph) {
            const int b = g * RB + pr + 16 * ph, b2 = (g + L.ng) * RB + pr + 16 * ph;
            if (row_used && b < p.B) ld_f32_now(p.C + (size_t(t_begin) * p.B + b) * p.Hp + j, creg[ph]);
            if (rb_count == 2 && row_used && b2 < p.B) ld_f32_now(p.C + (size_t(t_begin) * p.B + b2) * p.Hp + j, creg2[ph]);
        }
    }
    __syncthreads();
    loads_landed();
    clk.start();

    for (int t = t_begin; t < t_end; ++t) {
        for (int rb = g; rb < L.nrb; rb += L.ng, ++item) {
            const int row0 = rb * RB;
            float* part = part_all + size_t(item & 1) * NW * kRows * PLD;
            const half_t* xin = p.X + size_t(t & 3) * p.x_slot;          // h_{t-1}, fragment-major
            half_t* xout = p.X + size_t((t + 1) & 3) * p.x_slot;         // h_t
            half_t* xnext = p.X + size_t((t + 3) & 3) * p.x_slot;        // will take h_{t+2}: marked unwritten
            const half_t* a0 = xin + size_t(MT * rb) * nks_total * 512 + lane * 8;
            const half_t* a1 = a0 + size_t(nks_total) * 512;
            floatx4 acc[2][NT];
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int n = 0; n < NT; ++n) acc[m][n] = floatx4{0.f, 0.f, 0.f, 0.f};
            if constexpr (DS) first_request.hold();
            bool ahead;
            if constexpr (SPLIT)
                ahead = wave_product_tiles<NT, KS, 0, NPH * UPT / 2, kFwdBufs, false, 0, DS>(acc, wreg, nullptr, a0, a1, wave, lane, nks_total, ks_wave, rotation, poll,
                                                             [&]() { prefetch(t, rb); });
            else
                ahead = wave_product<NT, KS, RESIDENT, 0, UPT / 2, MT, DEEP ? 4 : 2, DEEP ? 2 : 0, DEEP, DS && !DEEP>(acc, wreg, nullptr, wfrag_wave, a0, a1, wave, lane, nks_total,
                                                               ks_wave, rotation, poll, [&]() { prefetch(t, rb); });
            if constexpr (DS) first_request.learn(ahead);
            clk.lap(0);
            spill_partials<NT, MT>(part, acc, wave, lane, PLD);
            __syncthreads();
            if (lds_abort != 0) leave_kernel();
            clk.lap(1);

            // Every peer of this group has delivered h_{t-1}, so all of them are done reading h_{t-2}:
            // its slot can be marked for reuse (it takes h_{t+2}).  The wait below also drains the mark
            // of the previous step, so that mark is in place before this step's h_t goes out.
            wait_all_vm();   // the x-projection of this step, issued during the product
#pragma unroll
            for (int ph = 0; ph < NPH; ++ph)
#pragma unroll
                for (int c = 0; c < UPT / 2; ++c) settle(xp[ph].v[c]);
            clk.lap(4);
            unsigned xoff[NPH];   // 32 bits: a slot is far below 4G halfs
#pragma unroll
            for (int ph = 0; ph < NPH; ++ph) {
                xoff[ph] = unsigned(xch_offset(row0 + pr + 16 * ph, j, nks_total));
                if (row_used) store_xch(xnext + xoff[ph], pack_fill(kUnwritten, (PackT*)nullptr), device_scope);
            }
            GateRow<UPT> act[NPH];
            float cnew[NPH][UPT] = {};
            PackT hnew[NPH];
            bool live[NPH];
            const bool second = (rb != g);
#pragma unroll
            for (int ph = 0; ph < NPH; ++ph) {
                const int prow = pr + 16 * ph, b = row0 + prow;
                hnew[ph] = pack_fill(0u, (PackT*)nullptr);   // batch rows past B travel as zeros
                live[ph] = row_used && b < p.B;
                if (live[ph]) {
                    float z[4][UPT];
                    unpack_gates(xp[ph], z);
#pragma unroll
                    for (int gt = 0; gt < 4; ++gt) {
#pragma unroll
                        for (int w = 0; w < NW; ++w) {
                            float v[UPT];
                            ld_f32(part + (size_t(w) * kRows + prow) * PLD + gt * JB + pj, v);
#pragma unroll
                            for (int u = 0; u < UPT; ++u) z[gt][u] += v[u];
                        }
                    }
                    float cp[UPT];
                    if (c_in_regs) {
#pragma unroll
                        for (int u = 0; u < UPT; ++u) cp[u] = second ? creg2[ph][u] : creg[ph][u];
                    } else {
                        ld_f32_coherent(p.C + (size_t(t) * p.B + b) * p.Hp + j, cp);
                    }
                    float hn[UPT], a4[4][UPT];
#pragma unroll
                    for (int u = 0; u < UPT; ++u) {
                        const float ig = sigmoidf_dev(z[0][u]);
                        const float fg = sigmoidf_dev(z[1][u]);
                        const float gg = tanhf_dev(z[2][u]);
                        const float og = sigmoidf_dev(z[3][u]);
                        cnew[ph][u] = fg * cp[u] + ig * gg;
                        hn[u] = og * tanhf_dev(cnew[ph][u]);
                        a4[0][u] = ig; a4[1][u] = fg; a4[2][u] = gg; a4[3][u] = og;
                        if (second) creg2[ph][u] = cnew[ph][u];
                        else creg[ph][u] = cnew[ph][u];
                    }
                    hnew[ph] = pack(hn);
                    act[ph] = pack_gates(a4);
                }
                // the exchanged value goes out first (one row tile after the other)
                if (row_used) store_xch(xout + xoff[ph], hnew[ph], device_scope);
            }
            clk.lap(2);
            // caches for the backward pass: off the critical path
#pragma unroll
            for (int ph = 0; ph < NPH; ++ph) {
                if (live[ph]) {
                    const int b = row0 + pr + 16 * ph;
                    st_f32(p.C + (size_t(t + 1) * p.B + b) * p.Hp + j, cnew[ph]);
                    st_pack(p.Y + (size_t(t + 1) * p.B + b) * p.Hp + j, hnew[ph]);
                    if (p.y_out) st_pack(p.y_out + (size_t(t) * p.B + b) * p.Hp + j, hnew[ph]);
                    st_gates(p.G + (size_t(t) * p.B + b) * gld + size_t(4) * j, act[ph]);
                }
            }
            clk.lap(3);
            // One row tile per block and 8 threads per row: the waves of rows 16..31 have no cells to update and would
            // reach the next product ahead of its operand.  A wave that finds its first chunk unwritten polls, and a
            // poll notices the data a full round trip to the L2 after it went out, whereas a wave that asks once the
            // data is there has it after one trip: measured, the early waves finished their product 0.4 us AFTER the
            // others (2048 units, 16 rows).  So all four waves start a product together.
            if constexpr (MT == 1 && GPR == 8) __syncthreads();
        }
    }
    if constexpr (DS) first_request.leave(p.delay_hint);
    clk.flush();
}


// 16 rows of partial sums per wave: [wave][16][pld] (spill_partials with one row tile and a 16-row pitch per wave)
template <int NT>
__device__ __forceinline__ void spill_partials16(float* part, const floatx4 (&acc)[2][NT], int wave, int lane, int pld) {
    float* base = part + (size_t(wave) * 16 + size_t(lane % 16)) * pld + 4 * (lane / 16);
#pragma unroll
    for (int n = 0; n < NT; ++n) *reinterpret_cast<floatx4*>(base + n * 16) = acc[0][n];
}

// ------------------------------------------------------------------- forward, interleaved chains
// The kernel above walks one dependent chain per row block: product -> partial sums -> cell update -> h_t out -> one
// trip through the L2 -> the peers' next product.  Nothing in a workgroup can run while h_t travels, so a step costs
// the sum of its parts plus the trip.  Here the two 16-row tiles of a 32-row block are two CHAINS that take turns:
// a phase multiplies one chain's tile while the other chain's h_t, published early in the phase, is on its way.
//   phase k:  request the fragments of chain k -> cell update of chain k-1 (its partial sums are in LDS), mark + h_t
//             out -> the fragments have landed: 32 MFMAs -> cache stores of chain k-1 -> x-projection of chain k+1
//             requested -> partial sums to LDS -> barrier
// Eight wavefronts, two per SIMD, at most 256 registers each; the contraction is split eight ways, so a wave holds 128
// registers of weight fragments and a product is FOUR fragment loads per wave: all are requested at once, ahead of the
// cell update, whose time hides their trip from the L2.  The 512 threads update the 16 x 32 cells of a tile, one each.
// The gate columns of the slice are packed unit-major here (column 4u + gate, pack_wfrag_fwd_kernel), so the four
// accumulation registers of a lane are the four gates of one unit, a wave's partial sums of a cell are 16 contiguous
// bytes in LDS, and a cell update reads eight 16-byte words.  Two partial-sum buffers of [8 waves][16 rows] (the one
// being read and the one being written), one barrier per phase.
// Vector-memory operations complete in issue order, and every wait below names how many YOUNGER operations may stay
// outstanding: the two ring stores of the cell update behind the fragment loads; the cache stores and the prefetch
// are issued behind the MFMAs, so no wait ever stands behind a store to memory that it does not need.
// The ring protocol is the one of rec_fwd_kernel, per chain: the cell update of (step t, chain) marks the chain's
// region of the slot of h_{t+2} (this workgroup's product of step t is complete by then, so every peer has published
// h_{t-1} and is done reading h_{t-2}) and then stores h_t; between a thread's mark and its next h store of the same
// chain lie two waits that drain everything older.  Ring words are validated as 32-bit words, so the thread of the
// even unit stores the pair (its neighbour's half comes over a DPP move).
template <int NT, int KS, bool DS>
__global__ __launch_bounds__(8 * kWave) void rec_fwd_il_kernel(RecFwdArgs p, RecLayout L, int t_begin, int t_end,
                                                               int ks_wave) {
    constexpr int NW = 8;
    constexpr int JB = 4 * NT;
    constexpr int NC = 16 * NT;
    constexpr int PLD = NC + kPartPad;
    static_assert(JB == 32 && KS == 4, "slices of 32 units; four k-steps per wave");
    extern __shared__ __attribute__((aligned(16))) float part_all[];  // [2][NW][16][PLD]
    __shared__ int lds_abort;
    __shared__ int lds_role[2];

    if (threadIdx.x == 0) lds_abort = 0;
    const Role role = make_role(L.nh, L.ng, L.gpx, L.xcd_local, p.seats, p.status, lds_role);
    if (!role.active) return;
    const int tid = threadIdx.x, lane = tid % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int hs = role.hs, g = role.g;
    const int rotation = __builtin_amdgcn_readfirstlane(rec_kstep_rotation(hs, L.nh, ks_wave, L.rot_div));
    const int nks_total = p.Hp / 32;
    const Poll poll{L.persistent != 0, p.spin_limit, p.spin_ticks, p.status, (lds_int_t*)&lds_abort};
    PhaseClock clk{(blockIdx.x == 0) ? p.prof : nullptr, 0};

    const half8* wfrag_wave = p.wfrag + (size_t(hs) * NW + wave) * size_t(ks_wave) * NT * kWave;
    half8 wreg[KS][NT];
#pragma unroll
    for (int k = 0; k < KS; ++k)
#pragma unroll
        for (int n = 0; n < NT; ++n)
            wreg[k][n] = (k < ks_wave) ? wfrag_wave[(size_t(k) * NT + n) * kWave + lane] : half8{};
    // offsets (in halfs) of this wave's k-steps inside a row tile of the ring: the same for the whole wave, so they
    // live in scalar registers and are added to the scalar base of a load
    unsigned koff[KS];
#pragma unroll
    for (int k = 0; k < KS; ++k)
        koff[k] = unsigned(min(rec_kstep_of_slot(k, rotation, ks_wave) * NW + wave, nks_total - 1)) * 512u;
    const unsigned lane_off = unsigned(lane) * 16u;

    // this thread's cell of a tile: row r, unit u of the slice.  Every address of a phase is a base that is the same
    // for the whole workgroup (scalar arithmetic) plus one of three per-thread offsets that never change.
    const int r = tid / JB, u = tid % JB;
    const int j = hs * JB + u;
    const bool even = (u % 2) == 0;
    const unsigned off_state = unsigned(r) * unsigned(p.Hp) + unsigned(j);          // [rows][Hp] arrays, in elements
    const unsigned off_gate = 4u * off_state;                                        // [rows][4Hp] arrays, in halfs
    const unsigned off_ring = unsigned(xch_offset(r, j, nks_total));                 // inside a row tile of the ring, in halfs
    const size_t tile_halfs = size_t(nks_total) * 512;
    const int rb_count = (L.nrb - g + L.ng - 1) / L.ng;
    // the cell state of a workgroup with one row block (two chains) stays in registers for the whole launch
    const bool c_in_regs = (rb_count <= 1) && (t_end - t_begin > 1);
    float creg[2] = {0.f, 0.f};   // [tile]
    uintx2 xp[2];   // x-projection of the next chain of each tile parity, requested a phase ahead of its product
    auto request_xp = [&](int t, int rb, auto tile_c) __attribute__((always_inline)) {
        constexpr int tl = decltype(tile_c)::value;
        const int b = min(rb * 32 + tl * 16 + r, p.B - 1);   // rows past B fetch row B-1 and are not used
        ld_stream(xp[tl], p.G + (size_t(t) * p.B + b) * (size_t(4) * p.Hp) + size_t(4) * j);
    };
    if (c_in_regs) {
#pragma unroll
        for (int tl = 0; tl < 2; ++tl) {
            const int b = g * 32 + tl * 16 + r;
            float v[2] = {0.f, 0.f};
            if (b < p.B) {
                floatx2 q;   // (one float is what is needed; the helper moves pairs: the even unit's pair holds both)
                asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=&v"(q.x) : "v"(p.C + (size_t(t_begin) * p.B + b) * p.Hp + j) : "memory");
                v[0] = q.x;
            }
            creg[tl] = v[0];
        }
    }
    request_xp(t_begin, g, std::integral_constant<int, 0>{});
    __syncthreads();
    loads_landed();
    clk.start();

    int pt = 0, prb = 0;      // the chain multiplied in the previous phase: step, row block (its tile is the other one)
    bool have_prev = false;
    int phase = 0;
    // one phase, product of chain (t, rb, tl) and cell update of the chain before it; (nt, nrb): the chain after it
    auto run_phase = [&](int t, int rb, auto tile_c, int nt, int nrb) __attribute__((always_inline)) {
        constexpr int tl = decltype(tile_c)::value;
        constexpr int ptl = 1 - tl;   // tile of the previous (and of the next) chain
        float* part = part_all + size_t(phase & 1) * NW * 16 * PLD;
        const float* part_prev = part_all + size_t((phase & 1) ^ 1) * NW * 16 * PLD;
        // ---- request this chain's operand: h_{t-1} of the tile, this wave's four k-steps
        const half_t* tile = wave_uniform(p.X + size_t(t & 3) * p.x_slot + size_t(2 * rb + tl) * tile_halfs);
        half8 f[KS];
        auto request = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int k = 0; k < KS; ++k) ld_frag_async_at(f[k], lane_off, tile + koff[k]);
        };
        request();
        // ---- cell update of the previous chain: everything but the cache stores
        const int row0 = prb * 32 + ptl * 16;   // first batch row of the previous chain's tile
        const bool live = have_prev && (row0 + r < p.B);
        unsigned hpair = 0u;   // h of this unit and its neighbour (batch rows past B travel as zeros)
        uintx2 act = uintx2{0u, 0u};
        float cnew = 0.f;
        if (have_prev) {
            half_t* xout = p.X + size_t((pt + 1) & 3) * p.x_slot + size_t(2 * prb + ptl) * tile_halfs;
            half_t* xnext = p.X + size_t((pt + 3) & 3) * p.x_slot + size_t(2 * prb + ptl) * tile_halfs;
            // (its x-projection was requested two phases ago, and the wait for the last product's fragments has covered it)
            settle(xp[ptl]);
            if (even) store_xch(xnext + off_ring, Pack<2>{kUnwritten}, DS);
            unsigned hbits = 0u;
            if (live) {
                float z[4];
                unpack_h2(xp[ptl].x, z[0], z[1]);
                unpack_h2(xp[ptl].y, z[2], z[3]);
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const floatx4 v = *reinterpret_cast<const floatx4*>(part_prev + (size_t(w) * 16 + r) * PLD + 4 * u);
                    z[0] += v.x; z[1] += v.y; z[2] += v.z; z[3] += v.w;
                }
                float cp;
                if (c_in_regs) {
                    cp = creg[ptl];
                } else {
                    floatx2 q;
                    asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(q.x) : "v"(p.C + size_t(pt) * p.B * p.Hp + size_t(row0) * p.Hp + off_state) : "memory");
                    cp = q.x;
                }
                const float ig = sigmoidf_dev(z[0]);
                const float fg = sigmoidf_dev(z[1]);
                const float gg = tanhf_dev(z[2]);
                const float og = sigmoidf_dev(z[3]);
                cnew = fg * cp + ig * gg;
                const float hn = og * tanhf_dev(cnew);
                creg[ptl] = cnew;
                act = uintx2{pack_h2(ig, fg), pack_h2(gg, og)};
                hbits = pack_h2(hn, 0.f);
            }
            // the neighbour's half: quad_perm(1, 0, 3, 2) swaps the lanes of a pair
            const unsigned other = unsigned(__builtin_amdgcn_mov_dpp(int(hbits), 0xB1, 0xF, 0xF, true));
            hpair = even ? (hbits | (other << 16)) : (other | (hbits << 16));
            if (even) store_xch(xout + off_ring, Pack<2>{hpair}, DS);
        }
        clk.lap(2);
        // ---- the fragments: landed once at most the two ring stores issued behind them are outstanding
        // (ONE wait statement names the fragment registers: with one in each branch the compiler joins the two
        // definitions and may copy the registers on the way there, ahead of the wait, while the loads still write them)
        if (!have_prev) wait_all_vm();
        wait_frags<2>(f);
        auto unwritten = [&]() -> bool {
            unsigned m = 0u;
#pragma unroll
            for (int k = 0; k < KS; ++k) {
                const uint4 ua = __builtin_bit_cast(uint4, f[k]);
                m = max(m, max(max(ua.x, ua.y), max(ua.z, ua.w)));
            }
            return __any(m == kUnwritten) != 0;
        };
        if (__builtin_expect(unwritten() && poll.on, 0)) {
            int spins = 0;
            long long spin_start = 0;
            do {
                if (poll_give_up(poll, spins, spin_start, lane)) break;   // results are garbage from here on; the workgroup leaves at its next barrier
                request();
                wait_frags<0>(f);
            } while (unwritten());
        }
        floatx4 acc[2][NT];
#pragma unroll
        for (int n = 0; n < NT; ++n) acc[0][n] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < KS; ++k)
#pragma unroll
            for (int n = 0; n < NT; ++n)
                acc[0][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wreg[k][n], f[k], acc[0][n], 0, 0, 0);
        clk.lap(0);
        // ---- caches of the previous chain for the backward pass, x-projection of the next chain
        if (live) {
            const size_t rows = size_t(pt) * p.B + row0;   // row of (step pt, first row of the tile) in the [T*B] arrays
            __builtin_nontemporal_store(cnew, p.C + (rows + p.B) * p.Hp + off_state);
            if (even) {
                __builtin_nontemporal_store(hpair, reinterpret_cast<unsigned*>(p.Y + (rows + p.B) * p.Hp + off_state));
                if (p.y_out) __builtin_nontemporal_store(hpair, reinterpret_cast<unsigned*>(p.y_out + rows * p.Hp + off_state));
            }
            __builtin_nontemporal_store(act, reinterpret_cast<uintx2*>(p.G + rows * (size_t(4) * p.Hp) + off_gate));
        }
        request_xp(nt, nrb, std::integral_constant<int, ptl>{});
        clk.lap(3);
        spill_partials16<NT>(part, acc, wave, lane, PLD);
        __syncthreads();
        clk.lap(1);
        pt = t; prb = rb; have_prev = true; ++phase;
        if (lds_abort != 0) leave_kernel();
    };
    for (int t = t_begin; t < t_end; ++t) {
        for (int rb = g; rb < L.nrb; rb += L.ng) {
            // the chain after (t, rb, tile 1): the next row block of this step, or the first one of the next step (past
            // the last step: a row that exists, fetched and not used)
            int nrb = rb + L.ng, nt = t;
            if (nrb >= L.nrb) { nrb = g; nt = (t + 1 < t_end) ? t + 1 : t; }
            run_phase(t, rb, std::integral_constant<int, 0>{}, t, rb);
            run_phase(t, rb, std::integral_constant<int, 1>{}, nt, nrb);
        }
    }
    // the last chain's cell update (tile 1 of the last row block and step)
    if (have_prev) {
        const float* part_prev = part_all + size_t((phase & 1) ^ 1) * NW * 16 * PLD;
        const int row0 = prb * 32 + 16;
        const bool live = row0 + r < p.B;
        half_t* xout = p.X + size_t((pt + 1) & 3) * p.x_slot + size_t(2 * prb + 1) * tile_halfs;
        half_t* xnext = p.X + size_t((pt + 3) & 3) * p.x_slot + size_t(2 * prb + 1) * tile_halfs;
        wait_all_vm();
        settle(xp[1]);
        if (even) store_xch(xnext + off_ring, Pack<2>{kUnwritten}, DS);
        unsigned hbits = 0u;
        uintx2 act = uintx2{0u, 0u};
        float cnew = 0.f;
        if (live) {
            float z[4];
            unpack_h2(xp[1].x, z[0], z[1]);
            unpack_h2(xp[1].y, z[2], z[3]);
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const floatx4 v = *reinterpret_cast<const floatx4*>(part_prev + (size_t(w) * 16 + r) * PLD + 4 * u);
                z[0] += v.x; z[1] += v.y; z[2] += v.z; z[3] += v.w;
            }
            float cp;
            if (c_in_regs) {
                cp = creg[1];
            } else {
                floatx2 q;
                asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(q.x) : "v"(p.C + size_t(pt) * p.B * p.Hp + size_t(row0) * p.Hp + off_state) : "memory");
                cp = q.x;
            }
            const float ig = sigmoidf_dev(z[0]);
            const float fg = sigmoidf_dev(z[1]);
            const float gg = tanhf_dev(z[2]);
            const float og = sigmoidf_dev(z[3]);
            cnew = fg * cp + ig * gg;
            const float hn = og * tanhf_dev(cnew);
            act = uintx2{pack_h2(ig, fg), pack_h2(gg, og)};
            hbits = pack_h2(hn, 0.f);
        }
        const unsigned other = unsigned(__builtin_amdgcn_mov_dpp(int(hbits), 0xB1, 0xF, 0xF, true));
        const unsigned hpair = even ? (hbits | (other << 16)) : (other | (hbits << 16));
        if (even) store_xch(xout + off_ring, Pack<2>{hpair}, DS);
        if (live) {
            const size_t rows = size_t(pt) * p.B + row0;
            __builtin_nontemporal_store(cnew, p.C + (rows + p.B) * p.Hp + off_state);
            if (even) {
                __builtin_nontemporal_store(hpair, reinterpret_cast<unsigned*>(p.Y + (rows + p.B) * p.Hp + off_state));
                if (p.y_out) __builtin_nontemporal_store(hpair, reinterpret_cast<unsigned*>(p.y_out + rows * p.Hp + off_state));
            }
            __builtin_nontemporal_store(act, reinterpret_cast<uintx2*>(p.G + rows * (size_t(4) * p.Hp) + off_gate));
        }
    }
    clk.lap(2);
    clk.flush();
}

// ----------------------------------------------------------------------------------- backward
// Gate order and the pointwise derivative follow flashlstm_v2/src/lstm_backward.cu:199-211, except
// that c_{t-1}, c_t come from the cell-state cache instead of being rebuilt through atanh.
template <int NT, int KS, bool RESIDENT, int KL, int MT, bool DS>
__global__ __launch_bounds__(kThreads) void rec_bwd_kernel(RecBwdArgs p, RecLayout L, int t_first,
                                                           int t_last, int ks_wave) {
    constexpr int NW = 4, THREADS = kThreads;
    constexpr int JB = 16 * NT;  // hidden units (= output columns of dG*W_hh) of this slice
    constexpr int PLD = JB + kPartPad;
    constexpr int KR = KS - KL;  // k-steps whose weight fragments stay in registers
    // As in the forward kernel: slices of 32 units with two row tiles update rows 0..15 first and publish that half of
    // dG_t, then rows 16..31, and fetch and multiply tile by tile, so the second half of a step's cell updates and its
    // cache stores run while the peers are already in the first half of their next product (measured at 1024 units
    // and 256 rows: 4.85 -> 4.5 us per step; without waiting for producers at all the step takes 4.2).
    constexpr bool SPLIT = RESIDENT && MT == 2 && JB >= 32 && (KS % 8 == 0);
    constexpr int GPR = (SPLIT || (MT == 1 && JB >= 32)) ? 16 : 8;   // threads per batch row (as in the forward kernel)
    constexpr int UPT = JB / GPR;
    constexpr int NPH = SPLIT ? 2 : 1;   // pointwise phases per step
    static_assert(UPT == 2 || UPT == 4, "2 or 4 hidden units per thread");
    typedef Pack<UPT> PackT;
    extern __shared__ __attribute__((aligned(16))) float part_all[];  // [2][NW][32][PLD], reused for db
    __shared__ int lds_abort;
    __shared__ int lds_role[2];

    if (threadIdx.x == 0) lds_abort = 0;
    const Role role = make_role(L.nh, L.ng, L.gpx, L.xcd_local, p.seats, p.status, lds_role);
    if (!role.active) return;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int hs = role.hs, g = role.g;
    const int rotation = __builtin_amdgcn_readfirstlane(rec_kstep_rotation(hs, L.nh, ks_wave, L.rot_div));
    const int nks_total = p.Hp / 8;  // contraction over 4Hp packed gate columns
    constexpr bool device_scope = DS;   // a persistent launch whose groups span XCDs (chosen by the host: no branch per store)
    const Poll poll{L.persistent != 0, p.spin_limit, p.spin_ticks, p.status, (lds_int_t*)&lds_abort};
    const float S = p.dy_scale;
    PhaseClock clk{(blockIdx.x == 0) ? p.prof : nullptr, 0};
    int item = 0;   // work items done: selects the partial-sum buffer
    FirstRequestDelay first_request;
    if constexpr (DS) first_request.start_from(p.delay_hint);

    const half8* wfrag_wave = p.wfrag + (size_t(hs) * NW + wave) * size_t(ks_wave) * NT * kWave;
    half8 wreg[KR][NT];
    // LDS: [partials 2*NW*32*PLD floats | weight fragments of KL k-steps (wlds_has), one block per wave]
    half8* wlds = reinterpret_cast<half8*>(part_all + 2 * NW * kRows * PLD) + size_t(wave) * KL * NT * kWave;
    if constexpr (RESIDENT) {
#pragma unroll
        for (int k = 0; k < KS; ++k)
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const half8 w = (k < ks_wave) ? wfrag_wave[(size_t(k) * NT + n) * kWave + lane] : half8{};
                if (wlds_has(k, KS, KL)) wlds[(wlds_before(k, KS, KL) * NT + n) * kWave + lane] = w;
                else wreg[wreg_slot(k, KS, KL)][n] = w;
            }
    }

    const size_t gld = size_t(4) * p.Hp;
    // this thread's groups: row pr (+ 16 in the second phase) of the row block, units pj .. pj+UPT-1 of the slice
    constexpr int RB = 16 * MT;   // batch rows of a row block
    const int pr = group_row<(GPR * UPT == 16) ? 4 : 2>(tid / GPR);
    const bool row_used = pr + 16 * (NPH - 1) < RB;   // with one row tile per block the threads of rows 16..31 only keep the barriers company
    const int pj = (tid % GPR) * UPT;
    const int j = hs * JB + pj;
    const size_t pq = size_t(4) * j;   // column of (unit j, gate 0) in the gate arrays
    const int rb_count = (L.nrb - g + L.ng - 1) / L.ng;
    // the running dc of the workgroup's first and second row block stays in registers for the whole launch
    const bool dc_in_regs = (rb_count <= 2) && (t_first - t_last > 0);
    float dcreg[NPH][UPT] = {}, dcreg2[NPH][UPT] = {};
    if (dc_in_regs) {
#pragma unroll
        for (int ph = 0; ph < NPH; ++ph) {
            const int b = g * RB + pr + 16 * ph, b2 = (g + L.ng) * RB + pr + 16 * ph;
            if (row_used && b < p.B) ld_f32_now(p.dC + size_t(b) * p.Hp + j, dcreg[ph]);
            if (rb_count == 2 && row_used && b2 < p.B) ld_f32_now(p.dC + size_t(b2) * p.Hp + j, dcreg2[ph]);
        }
    }
    // prefetched per work item and phase: activated gates, c_{t-1}, c_t, dY_t
    GateRow<UPT> pg[NPH];
    PackT pdy[NPH];
    F32<UPT> pcp_r[NPH], pcc_r[NPH];
    constexpr int NPF = NPH * (UPT / 2 + 3);
    auto prefetch = [&](int t, int rb) {   // NPF loads per wave; rows past B fetch row B-1, the closing pass step 0
        const int tt = max(t, 0);
#pragma unroll
        for (int ph = 0; ph < NPH; ++ph) {
            const int b = min(rb * RB + pr + 16 * ph, p.B - 1);
            const half_t* gsrc = p.G + (size_t(tt) * p.B + b) * gld + pq;
#pragma unroll
            for (int c = 0; c < UPT / 2; ++c) ld_stream(pg[ph].v[c], gsrc + 8 * c);
            ld_stream(pcp_r[ph].v, p.C + (size_t(tt) * p.B + b) * p.Hp + j);
            ld_stream(pcc_r[ph].v, p.C + (size_t(tt + 1) * p.B + b) * p.Hp + j);
            ld_stream(pdy[ph].v, p.dY + (size_t(tt) * p.B + b) * p.Hp + j);
        }
    };
    __syncthreads();
    float dbacc[4][UPT] = {};
    loads_landed();
    clk.start();

    for (int t = t_first; t >= t_last; --t) {
        const bool from_product = (t < p.T - 1);
        for (int rb = g; rb < L.nrb; rb += L.ng, ++item) {
            const int row0 = rb * RB;
            float* part = part_all + size_t(item & 1) * NW * kRows * PLD;
            // ring slot of step u is (u + 8) & 3: this step reads dG_{t+1}, writes dG_t and marks the
            // slot of dG_{t-2} unwritten
            if (from_product) {
                const half_t* xin = p.X + size_t((t + 9) & 3) * p.x_slot;   // dG_{t+1}, fragment-major
                const half_t* a0 = xin + size_t(MT * rb) * nks_total * 512 + lane * 8;
                const half_t* a1 = a0 + size_t(nks_total) * 512;
                floatx4 acc[2][NT];
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int n = 0; n < NT; ++n) acc[m][n] = floatx4{0.f, 0.f, 0.f, 0.f};
                if constexpr (DS) first_request.hold();   // (measured: 2048 units and 64 rows 7.37 -> 6.83 us per step; inside an XCD 1-6 % slower)
                bool ahead;
                if constexpr (SPLIT)
                    // (four sets of 4 k-steps: as many registers as two sets of 8, three quarters of them in flight
                    // instead of half; measured 4.59 -> 4.50 us per step, three sets of 8: 4.65)
                    ahead = wave_product_tiles<NT, KS, KL, NPF, 4, false, 4, DS>(acc, wreg, wlds, a0, a1, wave, lane, nks_total, ks_wave, rotation, poll,
                                                           [&]() { prefetch(t, rb); });
                else
                    ahead = wave_product<NT, KS, RESIDENT, KL, NPF, MT, 2, 0, false, DS>(acc, wreg, wlds, wfrag_wave, a0, a1, wave, lane, nks_total,
                                                              ks_wave, rotation, poll, [&]() { prefetch(t, rb); });
                if constexpr (DS) first_request.learn(ahead);
                clk.lap(0);
                spill_partials<NT, MT>(part, acc, wave, lane, PLD);
                __syncthreads();
                if (lds_abort != 0) leave_kernel();
                clk.lap(1);
            } else {
                prefetch(t, rb);
            }
            wait_all_vm();   // gates, cell states and dY of this step, issued during the product
#pragma unroll
            for (int ph = 0; ph < NPH; ++ph) {
#pragma unroll
                for (int c = 0; c < UPT / 2; ++c) settle(pg[ph].v[c]);
                settle(pdy[ph].v);
                settle(pcp_r[ph].v);
                settle(pcc_r[ph].v);
            }
            clk.lap(4);
            half_t* xout = p.X + size_t((t + 8) & 3) * p.x_slot;    // dG_t for the peers
            half_t* xnext = p.X + size_t((t + 6) & 3) * p.x_slot;   // will take dG_{t-2}
            unsigned xoff[NPH][UPT / 2];   // 32 bits: a slot is far below 4G halfs; 8 columns = 16 contiguous bytes
            if (t >= 0 && row_used) {
                // every peer has delivered dG_{t+1}, so all of them are done reading dG_{t+2}: mark its slot
                // (the wait above has drained the marks of the previous step)
#pragma unroll
                for (int ph = 0; ph < NPH; ++ph)
#pragma unroll
                    for (int c = 0; c < UPT / 2; ++c) {
                        xoff[ph][c] = unsigned(xch_offset(row0 + pr + 16 * ph, int(pq) + 8 * c, nks_total));
                        store_xch16(xnext + xoff[ph][c], uintx4{kUnwritten, kUnwritten, kUnwritten, kUnwritten}, device_scope);
                    }
            }
            GateRow<UPT> dgnew[NPH];
            float dcnew[NPH][UPT] = {};
            bool live[NPH];
            const bool second = (rb != g);
#pragma unroll
            for (int ph = 0; ph < NPH; ++ph) {
                const int prow = pr + 16 * ph, b = row0 + prow;
                live[ph] = row_used && b < p.B;
                const size_t sidx = size_t(b) * p.Hp + j;
                dgnew[ph] = gates_fill<UPT>(0u);   // batch rows past B travel as zeros
                if (live[ph]) {
                    float pcp[UPT], pcc[UPT];
                    to_floats(pcp_r[ph], pcp);
                    to_floats(pcc_r[ph], pcc);
                    float dh[UPT];
                    if (from_product) {
#pragma unroll
                        for (int u = 0; u < UPT; ++u) dh[u] = 0.f;
#pragma unroll
                        for (int w = 0; w < NW; ++w) {
                            float v[UPT];
                            ld_f32(part + (size_t(w) * kRows + prow) * PLD + pj, v);
#pragma unroll
                            for (int u = 0; u < UPT; ++u) dh[u] += v[u];
                        }
                    } else {
                        ld_f32_now(p.dHn + sidx, dh);
                    }
                    if (t < 0) {  // closing pass: gradient wrt h0; dc0 is the running dc
                        st_f32(p.dH0 + sidx, dh);
                        if (dc_in_regs) {
                            if (second) st_f32(p.dC + sidx, dcreg2[ph]);
                            else st_f32(p.dC + sidx, dcreg[ph]);
                        }
                    } else {
                        float dy[UPT], dcin[UPT];
                        unpack(pdy[ph], dy);
                        if (dc_in_regs) {
#pragma unroll
                            for (int u = 0; u < UPT; ++u) dcin[u] = second ? dcreg2[ph][u] : dcreg[ph][u];
                        } else {
                            ld_f32_coherent(p.dC + sidx, dcin);
                        }
                        float gate[4][UPT];
                        unpack_gates(pg[ph], gate);
                        float da[4][UPT];
#pragma unroll
                        for (int u = 0; u < UPT; ++u) {
                            const float ig = gate[0][u], fg = gate[1][u], gg = gate[2][u], og = gate[3][u];
                            const float dhu = dh[u] + S * dy[u];
                            const float tc = tanhf_dev(pcc[u]);
                            const float dov = dhu * tc;
                            const float dc = dcin[u] + dhu * og * (1.f - tc * tc);
                            da[0][u] = dc * gg * ig * (1.f - ig);
                            da[1][u] = dc * pcp[u] * fg * (1.f - fg);
                            da[2][u] = dc * ig * (1.f - gg * gg);
                            da[3][u] = dov * og * (1.f - og);
                            dcnew[ph][u] = dc * fg;
                            if (second) dcreg2[ph][u] = dcnew[ph][u];
                            else dcreg[ph][u] = dcnew[ph][u];
                        }
                        // db sums the values the weight-gradient GEMMs will see (fp16-rounded)
                        dgnew[ph] = pack_gates(da);
                        float r[4][UPT];
                        unpack_gates(dgnew[ph], r);
#pragma unroll
                        for (int gt = 0; gt < 4; ++gt)
#pragma unroll
                            for (int u = 0; u < UPT; ++u) dbacc[gt][u] += r[gt][u];
                    }
                }
                if (t >= 0 && row_used) {
                    // the exchanged values go out first (one row tile after the other)
#pragma unroll
                    for (int c = 0; c < UPT / 2; ++c) store_xch16(xout + xoff[ph][c], dgnew[ph].v[c], device_scope);
                }
            }
            clk.lap(2);
#pragma unroll
            for (int ph = 0; ph < NPH; ++ph) {
                if (t >= 0 && live[ph]) {   // row-major dG for the GEMMs that follow; running dc when it lives in memory
                    const int b = row0 + pr + 16 * ph;
                    st_gates(p.dG + (size_t(t) * p.B + b) * gld + pq, dgnew[ph]);
                    if (!dc_in_regs) st_f32(p.dC + size_t(b) * p.Hp + j, dcnew[ph]);
                }
            }
            clk.lap(3);
            if constexpr (MT == 1 && GPR == 8) __syncthreads();   // (waves without cells to update: as in the forward kernel)
        }
    }
    clk.flush();
    // single-step launches leave dc in memory for the next launch
    if (dc_in_regs && t_last >= 0) {
#pragma unroll
        for (int ph = 0; ph < NPH; ++ph) {
            const int b = g * RB + pr + 16 * ph, b2 = (g + L.ng) * RB + pr + 16 * ph;
            if (row_used && b < p.B) st_f32(p.dC + size_t(b) * p.Hp + j, dcreg[ph]);
            if (rb_count == 2 && row_used && b2 < p.B) st_f32(p.dC + size_t(b2) * p.Hp + j, dcreg2[ph]);
        }
    }

    if constexpr (DS) first_request.leave(p.delay_hint);
    // Bias gradient: fold this launch's sums over the threads that share a group column (fixed order).
    __syncthreads();
    float* red = part_all;  // [THREADS][4 * UPT]
#pragma unroll
    for (int gt = 0; gt < 4; ++gt)
#pragma unroll
        for (int u = 0; u < UPT; ++u) red[tid * (4 * UPT) + gt * UPT + u] = dbacc[gt][u];
    __syncthreads();
    if (tid < GPR * 4 * UPT) {
        const int gc = tid / (4 * UPT), e = tid % (4 * UPT);  // group column, (gate, unit)
        float sum = 0.f;
        for (int k = gc; k < THREADS; k += GPR) sum += red[k * (4 * UPT) + e];
        const int gt = e / UPT, u = e % UPT;
        const int ju = hs * JB + gc * UPT + u;
        const size_t q = size_t(4) * ju + gt;
        p.db_part[size_t(g) * gld + q] += sum;
    }
}

// --------------------------------------------------------------- backward, two-dimensional split
// For 2048 hidden units the product dG_{t+1} * W_hh^T has 32 MiB of weights.  The kernel above gives a workgroup 16
// output columns and the whole contraction (8192 packed gate columns), so every workgroup pulls all of dG_{t+1}
// of its rows through its XCD's L2 each step (512 KiB for a 32-row block); with 32 workgroups per XCD doing that,
// the step is bound by the bandwidth of the L2 (measured: 1.1 KiB per clock and XCD, 5.8 us per row block).  Here a
// workgroup owns a 64-column slice `s` (32 of them) and one of KQ slices `q` of the contraction: it fetches 1/KQ of
// dG_{t+1}, forms a partial product [rows][64], and the KQ workgroups of a column slice -- seated in one XCD -- sum
// their partials through a small ring in that XCD's L2: workgroup q sends columns (64/KQ)q' .. of its partial to
// workgroup q' of the slice and finishes the 64/KQ hidden units 64s + (64/KQ)q .. for all rows of the block.
//   KQ = 8, one group:  256 workgroups hold the weights once (128 KiB each); every workgroup takes every row block.
//                       For batches of one row block.
//   KQ = 4, two groups: a workgroup holds 256 KiB, the weights are held twice, and the groups take alternate row
//                       blocks (a workgroup makes half as many passes per step, each with a quarter of the fetch).
//
// Two rings carry a step:
//  * dG ring (p.X): 8 slots, fragment-major, written with device-scope stores and validated through the 'unwritten'
//    pattern like the rings above.  A workgroup that has its product of (step t, row block r) knows that every
//    workgroup of its group has stored dG_{t+2} of r (its producers stored dG_{t+1}, and each of those needed partials
//    from a full column slice, which together read all of dG_{t+2}), i.e. nobody reads dG_{t+3} of r any more: that
//    region is marked, five steps before it is reused.
//  * partial ring (p.P): 3 slots of fp32 partial sums, [workgroup][pass][sender][row][columns].  Plain stores,
//    XCD-local.  It needs no marks: the lowest mantissa bit of every word carries the parity of the step, and a slot
//    is reused every third step, so what a slot held before always shows the other parity (the bit costs 2^-24
//    relative precision).  A sender overwrites the partials of step t+3 after its product of step t, when all
//    workgroups of its group are past step t+2.
// A row block's partials are collected one product later (block i-1 after the product of block i), which hides the
// trip through the L2 except for the last block of a step.  The fragments are fetched as in the kernels above
// (hand-issued, counted waits, all inside wave_product); every other load is a buffer load the compiler sees, used
// in the same step it is issued in, so the compiler's own waits are exact and nothing stays in flight across the
// step loop's back edge.
constexpr int kDgSlots = 8;     // dG ring
constexpr int kTwoDWindowRows = 128;   // most rows of one launch at 2048 units (two groups, two passes of 32 rows each)
static_assert(kRecBwdPartSlots % 2 == 1, "consecutive uses of a partial-ring slot must differ in step parity");

typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, int(unsigned(bytes < 0xFFFFFFFFull ? bytes : 0xFFFFFFFFull)),
                                             0x00020000);
}
__device__ __forceinline__ void order_here() { asm volatile("" ::: "memory"); }
constexpr int kDeviceScope = 16, kNonTemporal = 2;   // cache policy of a buffer load (last argument of the builtin)

// MT: 16-row tiles per row block; KQ: contraction slices; NM: passes (row blocks) a workgroup makes per step at most;
// KS: k-steps per wave (4 waves * KS * 32 = 4 Hp / KQ packed gate columns); LOCAL: every group sits inside one XCD
// (1024 hidden units: 16 column slices x 2 contraction slices = the 32 workgroups of an XCD, group = XCD) -- else the
// groups span the XCDs (2048 hidden units: 32 column slices, 4 per XCD).
template <int MT, int KQ, int NM, int KS, bool LOCAL>
__global__ __launch_bounds__(kThreads) void rec_bwd2d_kernel(RecBwdArgs p, RecLayout L, int t_first, int t_last, int) {
    constexpr int NT = 4;            // 64 output columns
    constexpr int CPW = 64 / KQ;     // columns (hidden units) a workgroup finishes
    constexpr int UPT = CPW / 8;     // ... per thread: 8 threads share a row
    constexpr int PLD = 16 * NT + kPartPad;
    constexpr int RB = 16 * MT;
    constexpr int NPF = (UPT == 4) ? 5 : 4;   // buffer loads of load_ops
    // 256 KiB of weights per workgroup (16 k-steps per wave) would take all 256 accumulation registers of a lane and
    // leave the compiler nowhere to park what does not fit the ordinary ones: 5 of the 16 k-steps live in LDS instead
    // (80 KiB; with the partial sums 150 of the 160 KiB)
    constexpr int KL = (KS == 16) ? 5 : 0;
    constexpr int KR = KS - KL;
    static_assert(KQ == 2 || KQ == 4 || KQ == 8, "2, 4 or 8 contraction slices");
    static_assert(KS == 8 || KS == 16, "128 or 256 KiB of weights per workgroup");
    extern __shared__ __attribute__((aligned(16))) float part_all[];  // [2][4][32][PLD] partial sums | weight fragments of the last KL k-steps
    __shared__ int lds_abort;
    __shared__ int lds_role[2];
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    if (tid == 0) {
        lds_abort = 0;
        const int xcd = int(xcc_id()) & 7;
        const unsigned seat = __hip_atomic_fetch_add(p.seats + xcd, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (seat >= 32u) __hip_atomic_store(p.status, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        lds_role[0] = xcd;
        lds_role[1] = int(seat);
    }
    __syncthreads();
    if (lds_role[1] >= 32) return;
    // Seats of an XCD.  LOCAL: [column slice][KQ contraction slices], the XCD is the group.  Else [group][4 column
    // slices][KQ contraction slices].  Either way the workgroups of a column slice share the XCD.
    const int seat = __builtin_amdgcn_readfirstlane(lds_role[1]);
    const int xcd_u = __builtin_amdgcn_readfirstlane(lds_role[0]);
    const int g = LOCAL ? xcd_u : seat / (4 * KQ);
    const int s = LOCAL ? seat / KQ : xcd_u * 4 + (seat % (4 * KQ)) / KQ;
    const int q = seat % KQ;             // contraction slice; also: which CPW columns of the slice end here
    if (g >= L.ng || s * 64 >= p.Hp) return;   // (more seats than the layout uses: a group without row blocks)
    constexpr bool device_scope = !LOCAL;      // the dG ring: plain stores reach every reader inside an XCD
    const int nks = p.Hp / 8;            // k-steps of the whole contraction
    const int rotation = __builtin_amdgcn_readfirstlane(rec_bwd2d_rotation(s, KS, KQ));   // (the weight fragments are packed to match)
    const int nrb = L.nrb, ng = L.ng;
    const int nmine = (nrb - g + ng - 1) / ng;   // row blocks g, g + ng, ...
    const Poll poll{true, p.spin_limit, p.spin_ticks, p.status, (lds_int_t*)&lds_abort};
    const float S = p.dy_scale;
    PhaseClock clk{(blockIdx.x == 0) ? p.prof : nullptr, 0};

    half8 wreg[KR][NT];
    half8* wlds = reinterpret_cast<half8*>(part_all + 2 * 4 * kRows * PLD) + size_t(wave) * KL * NT * kWave;
    {
        const half8* wf = p.wfrag2 + ((size_t(s) * KQ + q) * 4 + wave) * size_t(KS) * NT * kWave;
#pragma unroll
        for (int k = 0; k < KS; ++k)
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                const half8 w = wf[(k * NT + n) * kWave + lane];
                if (wlds_has(k, KS, KL)) wlds[(wlds_before(k, KS, KL) * NT + n) * kWave + lane] = w;
                else wreg[wreg_slot(k, KS, KL)][n] = w;
            }
        // The weights belong in accumulation registers for the whole launch (an MFMA reads its operands from either
        // file).  Said outright: left to itself the register allocator keeps them in ordinary registers, runs out,
        // parks them in accumulation registers as spilled values and copies each back in front of every MFMA that
        // uses it (4 copies per 2 MFMAs, a fifth of a pass's vector instructions).
        if constexpr (KS >= 16) {
#pragma unroll
            for (int k = 0; k < KR; ++k)
#pragma unroll
                for (int n = 0; n < NT; ++n) asm volatile("" : "+a"(wreg[k][n]));
        }
    }

    // As a sender a thread sums row pr, columns 8*pj .. 8*pj+7 of the partial; as a receiver it collects the 8 columns
    // 8*(pj / KQ) .. of sender pj % KQ for row pr and ends up with UPT of them: the cells (row pr, unit j .. j+UPT-1).
    const int pr = tid / 8, pj = tid % 8;
    const bool row_used = pr < RB;
    const int j = s * 64 + q * CPW + (pj / KQ) * 8 + (pj % KQ) * UPT;
    const size_t pq = size_t(4) * j;
    const size_t gld = size_t(4) * p.Hp;
    // the running dc of every row block this workgroup takes stays in registers
    float dcreg[NM][UPT];
#pragma unroll
    for (int i = 0; i < NM; ++i) {
        const int b = p.b_lo + (g + i * ng) * RB + pr;
#pragma unroll
        for (int u = 0; u < UPT; ++u) dcreg[i][u] = (i < nmine && row_used && b < p.b_hi) ? p.dC[size_t(b) * p.Hp + j + u] : 0.f;
    }
    float dbacc[4][UPT] = {};
    int item = 0;
    const rsrc_t rp = make_rsrc(p.P, size_t(kRecBwdPartSlots) * p.p_slot * 4);
    const unsigned wg_id = unsigned((g * (p.Hp / 64) + s) * KQ);   // + receiver's q: inbox index in the partial ring

    auto spin_out = [&](int& spins, long long& spin_start) -> bool { return poll_give_up(poll, spins, spin_start, lane); };

    // Per-cell operands of a row block (activated gates, c_{t-1}, c_t, dY), NPF buffer loads.
    struct Ops {
        uintx4 g[(UPT + 1) / 2];   // four halfs (i, f, g, o) per unit
        uintx4 cp, cc;             // one fp32 per unit
        uintx2 dy;                 // one half per unit
    };
    auto load_ops = [&](int t, int rb, Ops& o) {
        const int b = min(p.b_lo + rb * RB + pr, p.b_hi - 1);
        const size_t tt = size_t(max(t, 0));
        // (a descriptor per step: the arrays of a long sequence are larger than a 32-bit offset reaches)
        const rsrc_t rg = make_rsrc(p.G + tt * p.B * gld, size_t(p.B) * gld * 2);
        const rsrc_t rc = make_rsrc(p.C + tt * p.B * p.Hp, size_t(2) * p.B * p.Hp * 4);
        const rsrc_t ry = make_rsrc(p.dY + tt * p.B * p.Hp, size_t(p.B) * p.Hp * 2);
        const unsigned cell_idx = unsigned(b) * unsigned(p.Hp) + unsigned(j);
        const unsigned goff = (unsigned(b) * unsigned(gld) + unsigned(pq)) * 2u;
        const unsigned next = unsigned(p.B) * unsigned(p.Hp);
        if constexpr (UPT == 4) {
            o.g[0] = __builtin_amdgcn_raw_buffer_load_b128(rg, goff, 0, kNonTemporal);
            o.g[1] = __builtin_amdgcn_raw_buffer_load_b128(rg, goff + 16u, 0, kNonTemporal);
            const uintx4 cp4 = __builtin_amdgcn_raw_buffer_load_b128(rc, cell_idx * 4u, 0, kNonTemporal);
            const uintx4 cc4 = __builtin_amdgcn_raw_buffer_load_b128(rc, (cell_idx + next) * 4u, 0, kNonTemporal);
            o.cp = uintx4{cp4.x, cp4.y, cp4.z, cp4.w};
            o.cc = uintx4{cc4.x, cc4.y, cc4.z, cc4.w};
            o.dy = __builtin_amdgcn_raw_buffer_load_b64(ry, cell_idx * 2u, 0, kNonTemporal);
        } else if constexpr (UPT == 2) {
            o.g[0] = __builtin_amdgcn_raw_buffer_load_b128(rg, goff, 0, kNonTemporal);
            const uintx2 cp2 = __builtin_amdgcn_raw_buffer_load_b64(rc, cell_idx * 4u, 0, kNonTemporal);
            const uintx2 cc2 = __builtin_amdgcn_raw_buffer_load_b64(rc, (cell_idx + next) * 4u, 0, kNonTemporal);
            o.cp = uintx4{cp2.x, cp2.y, 0u, 0u};
            o.cc = uintx4{cc2.x, cc2.y, 0u, 0u};
            o.dy = uintx2{__builtin_amdgcn_raw_buffer_load_b32(ry, cell_idx * 2u, 0, kNonTemporal), 0u};
        } else {
            const uintx2 g2 = __builtin_amdgcn_raw_buffer_load_b64(rg, goff, 0, kNonTemporal);
            o.g[0] = uintx4{g2.x, g2.y, 0u, 0u};
            o.cp = uintx4{__builtin_amdgcn_raw_buffer_load_b32(rc, cell_idx * 4u, 0, kNonTemporal), 0u, 0u, 0u};
            o.cc = uintx4{__builtin_amdgcn_raw_buffer_load_b32(rc, (cell_idx + next) * 4u, 0, kNonTemporal), 0u, 0u, 0u};
            o.dy = uintx2{unsigned(__builtin_amdgcn_raw_buffer_load_b16(ry, cell_idx * 2u, 0, kNonTemporal)), 0u};
        }
    };
    // the cell update of (t, pass i: row block rb) given dh from the product (or dHn), and everything it stores
    auto cell = [&](int t, int rb, float (&dcr)[UPT], const float (&dh)[UPT], const Ops& o) {
        const int b = p.b_lo + rb * RB + pr;
        const bool live = row_used && b < p.b_hi;
        const size_t sidx = size_t(b) * p.Hp + j;
        if (t < 0) {   // closing pass: gradient wrt h0; dc0 is the running dc
            if (live) {
#pragma unroll
                for (int u = 0; u < UPT; ++u) {
                    p.dH0[sidx + u] = dh[u];
                    p.dC[sidx + u] = dcr[u];
                }
            }
            return;
        }
        half_t* xout = p.X + size_t((t + 8) & (kDgSlots - 1)) * p.x_slot;     // dG_t for everybody
        half_t* xmark = p.X + size_t((t + 11) & (kDgSlots - 1)) * p.x_slot;   // dG_{t+3}: read by nobody any more
        // position of every unit's four gate columns in the fragment-major ring: eight columns (two units) are
        // contiguous, the next eight belong to another lane of the fragment
        unsigned off[UPT] = {};
        if (row_used) {
#pragma unroll
            for (int u = 0; u < UPT; ++u) off[u] = unsigned(xch_offset(b, int(pq) + 4 * u, nks));
#pragma unroll
            for (int u = 0; u < UPT; ++u) store_xch(xmark + off[u], Pack<4>{uintx2{kUnwritten, kUnwritten}}, device_scope);
        }
        Pack<4> out[UPT];
#pragma unroll
        for (int u = 0; u < UPT; ++u) out[u] = Pack<4>{uintx2{0u, 0u}};   // batch rows past B travel as zeros
        if (live) {
#pragma unroll
            for (int u = 0; u < UPT; ++u) {
                float gate[4];
                const uintx4 gw = o.g[u / 2];
                unpack(Pack<4>{(u % 2) == 0 ? uintx2{gw.x, gw.y} : uintx2{gw.z, gw.w}}, gate);
                float dyl, dyh;
                unpack_h2((u / 2) == 0 ? o.dy.x : o.dy.y, dyl, dyh);
                const float dyv = (u % 2) == 0 ? dyl : dyh;
                // (components picked by name: indexing a vector member through the reference gave wrong lanes)
                const unsigned cpw = (u == 0) ? o.cp.x : (u == 1) ? o.cp.y : (u == 2) ? o.cp.z : o.cp.w;
                const unsigned ccw = (u == 0) ? o.cc.x : (u == 1) ? o.cc.y : (u == 2) ? o.cc.z : o.cc.w;
                const float pcp = __builtin_bit_cast(float, cpw);
                const float pcc = __builtin_bit_cast(float, ccw);
                const float ig = gate[0], fg = gate[1], gg = gate[2], og_ = gate[3];
                const float dhu = dh[u] + S * dyv;
                const float tc = tanhf_dev(pcc);
                const float dov = dhu * tc;
                const float dc = dcr[u] + dhu * og_ * (1.f - tc * tc);
                float da[4];
                da[0] = dc * gg * ig * (1.f - ig);
                da[1] = dc * pcp * fg * (1.f - fg);
                da[2] = dc * ig * (1.f - gg * gg);
                da[3] = dov * og_ * (1.f - og_);
                dcr[u] = dc * fg;
                out[u] = pack(da);
                float r[4];   // db sums the values the weight-gradient GEMMs will see (fp16-rounded)
                unpack(out[u], r);
#pragma unroll
                for (int gt = 0; gt < 4; ++gt) dbacc[gt][u] += r[gt];
            }
        }
        if (row_used) {
#pragma unroll
            for (int u = 0; u < UPT; ++u) store_xch(xout + off[u], out[u], device_scope);
        }
        clk.lap(2);
        if (live) {
            half_t* dst = p.dG + (size_t(t) * p.B + b) * gld + pq;
            if constexpr (UPT == 1) {
                st_pack(dst, out[0]);
            } else {
#pragma unroll
                for (int u = 0; u < UPT; u += 2)
                    __builtin_nontemporal_store(uintx4{out[u].v.x, out[u].v.y, out[u + 1].v.x, out[u + 1].v.y},
                                                reinterpret_cast<uintx4*>(dst + 4 * u));
            }
        }
        clk.lap(3);
    };

    __syncthreads();
    loads_landed();
    clk.start();
    for (int t = t_first; t >= t_last; --t) {
        if (t >= p.T - 1) {   // the last step of the sequence: dh comes from the caller
#pragma unroll
            for (int i = 0; i < NM; ++i) {
                if (i >= nmine) break;
                const int rb = g + i * ng;
                Ops o;
                load_ops(t, rb, o);
                const int b = min(p.b_lo + rb * RB + pr, p.b_hi - 1);
                float dh[UPT];
#pragma unroll
                for (int u = 0; u < UPT; ++u) dh[u] = p.dHn[size_t(b) * p.Hp + j + u];
                cell(t, rb, dcreg[i], dh, o);
            }
            continue;
        }
        const half_t* xin = p.X + size_t((t + 9) & (kDgSlots - 1)) * p.x_slot;   // dG_{t+1}
        const unsigned pbase = unsigned((t + 3) % kRecBwdPartSlots) * unsigned(p.p_slot);   // in floats
        float* pslot = p.P + size_t(pbase);
        const unsigned par = unsigned(t) & 1u;
        Ops ops[2];
        // Pass i (unrolled): request the partials of block i-1, multiply block i (its cell operands are requested
        // behind the last fragment load), send its partials, then finish block i-1.
#pragma unroll
        for (int i = 0; i <= NM; ++i) {
            if (i > nmine) break;
            const bool product = i < nmine, finish = i >= 1;
            const int rb = g + i * ng, rb_prev = g + (i - 1) * ng;
            uintx4 in0 = {0u, 0u, 0u, 0u}, in1 = {0u, 0u, 0u, 0u};
            // partials of block i-1 in this workgroup's inbox: sender pj % KQ, row pr, 8 columns from 8 * (pj / KQ)
            const unsigned src = (pbase + ((((wg_id + unsigned(q)) * NM + unsigned(max(i - 1, 0))) * KQ + unsigned(pj % KQ)) * RB +
                                           unsigned(min(pr, RB - 1))) * CPW + unsigned(pj / KQ) * 8u) * 4u;
            if (finish) {
                in0 = __builtin_amdgcn_raw_buffer_load_b128(rp, src, 0, kDeviceScope);
                in1 = __builtin_amdgcn_raw_buffer_load_b128(rp, src + 16u, 0, kDeviceScope);
                order_here();
            }
            if (product) {
                float* part = part_all + size_t(item & 1) * 4 * kRows * PLD;
                floatx4 acc[2][NT];
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int n = 0; n < NT; ++n) acc[m][n] = floatx4{0.f, 0.f, 0.f, 0.f};
                const half_t* a0 = xin + (size_t(p.b_lo / 16 + MT * rb) * nks + size_t(q) * (KS * 4)) * 512 + lane * 8;
                const half_t* a1 = a0 + size_t(nks) * 512;
                // (where the operand comes through memory -- groups that span XCDs -- and the contraction is long, five
                // short fragment sets keep the fetch running over that trip)
                wave_product<NT, KS, true, KL, NPF, MT, ((KS >= 16 && !LOCAL) ? 5 : 2), ((KS >= 16 && !LOCAL) ? 2 : 0), false, !LOCAL>(acc, wreg, wlds, nullptr, a0, a1, wave, lane, KS * 4, KS, rotation, poll,
                                                       [&]() { load_ops(t, rb, ops[i & 1]); });
                clk.lap(0);
                spill_partials<NT, MT>(part, acc, wave, lane, PLD);
                ++item;
                __syncthreads();
                if (lds_abort != 0) leave_kernel();
                if (row_used) {   // sum the four waves' k-slices and send 8 columns to their receiver in the slice
                    floatx4 v0 = {0.f, 0.f, 0.f, 0.f}, v1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const float* src_l = part + (size_t(w) * kRows + pr) * PLD + 8 * pj;
                        v0 += *reinterpret_cast<const floatx4*>(src_l);
                        v1 += *reinterpret_cast<const floatx4*>(src_l + 4);
                    }
                    uintx4 u0 = __builtin_bit_cast(uintx4, v0), u1 = __builtin_bit_cast(uintx4, v1);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        u0[e] = (u0[e] & ~1u) | par;
                        u1[e] = (u1[e] & ~1u) | par;
                    }
                    // columns 8*pj .. belong to receiver (8*pj) / CPW, at column (8*pj) % CPW of its block
                    const unsigned recv = unsigned(8 * pj) / CPW, col = unsigned(8 * pj) % CPW;
                    float* dst = pslot + ((((size_t(wg_id) + recv) * NM + i) * KQ + q) * RB + pr) * CPW + col;
                    *reinterpret_cast<uintx4*>(dst) = u0;
                    *reinterpret_cast<uintx4*>(dst + 4) = u1;
                }
                clk.lap(1);
            }
            if (finish) {
                // (the first check stands outside the loop: the compiler then waits for exactly these two loads there)
                auto tags_bad = [&]() -> bool {
                    const unsigned all1 = in0.x & in0.y & in0.z & in0.w & in1.x & in1.y & in1.z & in1.w;
                    const unsigned any1 = in0.x | in0.y | in0.z | in0.w | in1.x | in1.y | in1.z | in1.w;
                    const bool ok = par ? ((all1 & 1u) != 0u) : ((any1 & 1u) == 0u);
                    return __any(row_used && !ok) != 0;
                };
                if (tags_bad()) {
                    int spins = 0;
                    long long spin_start = 0;
                    do {
                        if (spin_out(spins, spin_start)) break;
                        order_here();
                        in0 = __builtin_amdgcn_raw_buffer_load_b128(rp, src, 0, kDeviceScope);
                        in1 = __builtin_amdgcn_raw_buffer_load_b128(rp, src + 16u, 0, kDeviceScope);
                        order_here();
                    } while (tags_bad());
                }
                clk.lap(4);
                // Sum over the KQ senders (lanes that differ in their low bits): each halving step keeps half of the
                // columns, so lane pj ends up with columns UPT * (pj % KQ) .. of its 8.
                const floatx4 f0 = __builtin_bit_cast(floatx4, in0), f1 = __builtin_bit_cast(floatx4, in1);
                float a4[4], a2[2], dh[UPT];
                if constexpr (KQ == 8) {
                    const bool hi = (lane & 4) != 0;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const float keep = hi ? f1[k] : f0[k], send = hi ? f0[k] : f1[k];
                        a4[k] = keep + __shfl_xor(send, 4);
                    }
                    const bool hi2 = (lane & 2) != 0;
#pragma unroll
                    for (int k = 0; k < 2; ++k) {
                        const float keep = hi2 ? a4[2 + k] : a4[k], send = hi2 ? a4[k] : a4[2 + k];
                        a2[k] = keep + __shfl_xor(send, 2);
                    }
                    const bool hi1 = (lane & 1) != 0;
                    dh[0] = (hi1 ? a2[1] : a2[0]) + __shfl_xor(hi1 ? a2[0] : a2[1], 1);
                } else if constexpr (KQ == 4) {
                    const bool hi2 = (lane & 2) != 0;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const float keep = hi2 ? f1[k] : f0[k], send = hi2 ? f0[k] : f1[k];
                        a4[k] = keep + __shfl_xor(send, 2);
                    }
                    const bool hi1 = (lane & 1) != 0;
#pragma unroll
                    for (int k = 0; k < 2; ++k) {
                        const float keep = hi1 ? a4[2 + k] : a4[k], send = hi1 ? a4[k] : a4[2 + k];
                        dh[k] = keep + __shfl_xor(send, 1);
                    }
                    (void)a2;
                } else {
                    const bool hi1 = (lane & 1) != 0;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const float keep = hi1 ? f1[k] : f0[k], send = hi1 ? f0[k] : f1[k];
                        dh[k] = keep + __shfl_xor(send, 1);
                    }
                    (void)a4; (void)a2;
                }
                cell(t, rb_prev, dcreg[i >= 1 ? i - 1 : 0], dh, ops[(i + 1) & 1]);
            }
        }
        // (16-row blocks: the waves of rows 16..31 have no cells to update; all four waves start the next product
        // together, as in the forward kernel)
        if constexpr (MT == 1) __syncthreads();
    }
    clk.flush();
    if (t_last >= 0) {   // a launch that stops before the closing pass leaves dc in memory for the next one
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            const int b = p.b_lo + (g + i * ng) * RB + pr;
            if (i < nmine && row_used && b < p.b_hi) {
#pragma unroll
                for (int u = 0; u < UPT; ++u) p.dC[size_t(b) * p.Hp + j + u] = dcreg[i][u];
            }
        }
    }
    // Bias gradient: fold this launch's sums over the 32 rows (fixed order).
    __syncthreads();
    float* red = part_all;   // [256][4 * UPT]
#pragma unroll
    for (int gt = 0; gt < 4; ++gt)
#pragma unroll
        for (int u = 0; u < UPT; ++u) red[tid * (4 * UPT) + gt * UPT + u] = dbacc[gt][u];
    __syncthreads();
    if (tid < 8 * 4 * UPT) {
        const int cpos = tid / (4 * UPT), e = tid % (4 * UPT);   // thread column pj, (gate, unit)
        float sum = 0.f;
        for (int r = 0; r < kThreads / 8; ++r) sum += red[(r * 8 + cpos) * (4 * UPT) + e];
        const int gt = e / UPT, u = e % UPT;
        const int ju = s * 64 + q * CPW + (cpos / KQ) * 8 + (cpos % KQ) * UPT + u;
        p.db_part[size_t(g) * gld + size_t(4) * ju + gt] += sum;
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

// (set before every launch: the call is cheap, needs no process-wide flag and holds for whichever device is current)
template <typename K>
hipError_t raise_lds(K kernel, size_t bytes) {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes));
}

// A persistent launch needs all its workgroups running at once: they wait for each other's data.  The cooperative
// launch makes that a condition of the launch (the runtime refuses a grid that cannot be co-resident and does not
// run it beside another kernel); where the runtime has no cooperative launch the ordinary one is used, and the
// bounded waits inside the kernel cover the case that some workgroup is late.
template <typename K, typename A>
hipError_t launch_persistent(K kernel, int grid, size_t lds, hipStream_t stream, A a, RecLayout L, int t_a, int t_b,
                             int ks_wave, int threads = kThreads) {
    if (L.cooperative) {
        void* params[] = {&a, &L, &t_a, &t_b, &ks_wave};
        hipError_t e = hipLaunchCooperativeKernel(reinterpret_cast<const void*>(kernel), dim3(grid), dim3(threads), params,
                                                  unsigned(lds), stream);
        if (e == hipSuccess) return hipSuccess;
        (void)hipGetLastError();
        // A grid the runtime says cannot be co-resident is exactly what a persistent launch must not be given: nothing
        // is launched, and the caller runs the pass step-wise.  Any other refusal (no cooperative launch on this
        // runtime) falls back to the plain launch, whose bounded waits cover a late workgroup.
        if (e == hipErrorCooperativeLaunchTooLarge) return e;
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), lds, stream, a, L, t_a, t_b, ks_wave);
    return hipGetLastError();
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

int rec_fwd_ks(const RecLayout& L, int Hp) { return int(ceil_div(size_t(Hp) / 32, size_t(L.nw))); }
int rec_bwd_ks(const RecLayout& L, int Hp) { return int(ceil_div(size_t(Hp) / 8, size_t(L.nw))); }

// Wavefronts per workgroup of the forward recurrence: eight (rec_fwd_il_kernel: the two row tiles of a 32-row block
// take turns) where a slice has 32 units -- up to 1024 hidden units -- and every workgroup gets exactly one 32-row
// block: more rows than 16-row blocks can run side by side, no more than 32-row blocks can.  Measured, us per step,
// four -> eight waves: 1024 units and 256 rows 3.45 -> 3.24, 768 units and 160 rows 3.06 -> 2.84, 512 units and 512
// rows 3.19 -> 3.12; with two row blocks per workgroup (1024 units, 512 rows) 7.2 -> 8.6, so those stay with four.
int rec_waves(int B, int Hp, int num_cus, int waves) {
    if (Hp > 1024) return 4;
    if (waves == 4 || waves == 8) return waves;
    const int nh = Hp / 32;
    const bool xcd_mode = (num_cus == 256 && nh <= 32);
    const int side_by_side = nh > num_cus ? 0 : (xcd_mode ? 8 * (32 / nh) : num_cus / nh);
    const bool can_16 = int(ceil_div(size_t(B), 16)) <= side_by_side;
    const bool one_block_each = int(ceil_div(size_t(B), 32)) <= side_by_side;
    return (!can_16 && one_block_each) ? 8 : 4;
}

static void finish_layout(RecLayout& L, int B, int Hp, int num_cus, bool force_stepwise, bool fits, int force_mt) {
    L.nh = Hp / L.jb;
    L.resident = fits ? 1 : 0;
    L.rot_div = 0;   // no k-step rotation (plan_rec_bwd turns it on where it pays)
    // Row blocks of 16 rows (one MFMA row tile) when all of them can run side by side: twice the workgroups
    // of 32-row blocks, each with half the product, fetch and cell-update work per step.
    const bool xcd_mode = (num_cus == 256 && L.nh <= 32);
    const int side_by_side = L.nh > num_cus ? 0 : (xcd_mode ? 8 * (32 / L.nh) : num_cus / L.nh);
    const bool can_16 = fits && int(ceil_div(size_t(B), 16)) <= side_by_side;
    L.mt = can_16 ? 1 : 2;
    if (force_mt == 2 || (force_mt == 1 && can_16)) L.mt = force_mt;   // a tuned choice; 16-row blocks only where they fit
    if (L.nw == 8) L.mt = 2;   // the eight-wave kernels take 32-row blocks (their two row tiles take turns)
    L.nrb = int(ceil_div(size_t(B), size_t(16 * L.mt)));
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

RecLayout plan_rec_fwd(int B, int Hp, int num_cus, bool force_stepwise, int force_mt, int waves) {
    RecLayout L{};
    bool fits = true;
    if (Hp <= 1024) L.nt = 8;
    else if (Hp <= 2048) L.nt = 4;
    else { L.nt = 8; fits = false; }
    L.nw = fits ? rec_waves(B, Hp, num_cus, waves) : 4;
    L.jb = 4 * L.nt;
    finish_layout(L, B, Hp, num_cus, force_stepwise, fits, force_mt);
    return L;
}

RecLayout plan_rec_bwd(int B, int Hp, int num_cus, bool force_stepwise, int force_mt, int two_d) {
    RecLayout L{};
    bool fits = true;
    if (Hp <= 1024) L.nt = 2;
    else if (Hp <= 2048) L.nt = 1;
    else { L.nt = 2; fits = false; }
    L.nw = 4;
    L.jb = 16 * L.nt;
    finish_layout(L, B, Hp, num_cus, force_stepwise, fits, force_mt);
    // k-step rotation (recurrent.h): measured, it pays where a group spans the XCDs and a step fetches a lot -- the
    // backward pass at 2048 hidden units, 13.4 -> 12.4 us per step at 128 rows -- and costs a little where the
    // workgroups of an XCD read the same lines in step out of their own L2 (5.33 -> 5.42 us at 1024 units, where
    // reading in step is what lets the L2 serve one line to many).  A function of the sizes alone: the packed
    // weights depend on it.
    L.rot_div = (L.nh > 32) ? 8 : 0;
    if (two_d > 0 && L.persistent && rec_bwd_two_d_possible(Hp, num_cus)) {
        // 2048 units, more rows than the two-way kernel takes (two passes of 32 rows for each of two groups): batch rows
        // are independent sequences, so the batch is walked in windows of 128 rows, one persistent launch after the
        // other, instead of falling back to the one-way layout (measured, us per backward step: 160 rows 20.8 -> 17.7,
        // 256 rows 29.9 -> 18.3; the one-way layout pays per 32-row block, so a fifth block already costs more than a
        // second window).  The last window may be short; its empty row blocks travel as zeros like any rows past the
        // batch.
        const int win = (Hp == 2048 && B > kTwoDWindowRows) ? kTwoDWindowRows : 0;
        const int Bfull = B;
        if (win) B = win;
        const int mt = (B <= 16 && force_mt != 2 && Hp == 2048) ? 1 : 2;
        const int nrb = int(ceil_div(size_t(B), size_t(16 * mt)));
        const int kq = rec_bwd_two_d_kq(Bfull, Hp);
        const int ng = Hp == 1024 ? 8 : (kq == 8 ? 1 : 2);
        const int per_wg = int(ceil_div(size_t(nrb), size_t(ng)));   // passes per step and workgroup
        // 2048 units.  One row block per step: 8 contraction slices, every workgroup on that block.  More: 4 slices and
        // two groups that take alternate row blocks.  Measured, us per backward step, one-way -> two-way: 16 rows
        // 5.4 -> 4.0, 32 rows 5.8 -> 4.2, 64 rows 7.5 -> 7.6, 128 rows 12.4 -> 9.8.
        // 1024 units: 16 column slices x 2 contraction slices inside every XCD, the XCD's row blocks in turn.  Measured
        // slower than the one-way layout (256 rows: 5.3 -> 5.9 us per step; 512 rows: with two passes 10.7 -> 11.2): inside an XCD the
        // step waits on the trips through the L2, not on the amount fetched, and the second exchange adds one.
        // two_d = 1 takes the layout where it measured faster than the one-way layout, two_d = 2 wherever it can run
        // (2048 units: at most 2 passes per workgroup, a kernel unrolled for 4 does not fit the registers; 1024 units,
        // four cells per thread: one pass, i.e. 256 rows).
        const bool faster = Hp == 2048 && nrb != 2;
        if (per_wg <= (Hp == 2048 ? 2 : 1) && (two_d >= 2 || faster)) {
            L.two_d = 1;
            L.kq = kq;
            L.nm = per_wg;
            L.mt = mt;
            L.nrb = nrb;
            L.ng = ng;
            L.xcd_local = 0;
            L.gpx = 0;
            L.grid = 256;
            L.win_rows = win;
        }
    }
    return L;
}

bool rec_bwd_two_d_possible(int Hp, int num_cus) { return (Hp == 2048 || Hp == 1024) && num_cus == 256; }
// Up to two row blocks: 8 slices and one group (with two blocks every workgroup makes two passes per step, and one
// block's trip through memory hides behind the other's product: 7.0 us per step at 64 rows against 8.0 with 4 slices and
// two groups of one pass each).  More: 4 slices, two groups.
int rec_bwd_two_d_kq(int B, int Hp) { return Hp == 1024 ? 2 : (B <= 64 ? 8 : 4); }
int rec_bwd_dg_slots(const RecLayout& L) { return L.two_d ? kDgSlots : 4; }
size_t rec_bwd_part_slot_floats(const RecLayout& L) {
    // [256 workgroups][nm passes][kq senders][rows][64 / kq columns]
    return L.two_d ? size_t(256) * L.nm * 64 * (16 * L.mt) : 0;
}
size_t rec_bwd_two_d_wfrag_bytes(int Hp) { return size_t(Hp) * 4 * Hp * sizeof(half_t); }
int rec_bwd_ring_rows(const RecLayout& L, int B) {
    return (L.two_d && L.win_rows) ? int(ceil_div(size_t(B), size_t(L.win_rows))) * L.win_rows : B;
}
unsigned rec_bwd_part_fill(int slot, int T) {
    // the first product step of a pass is T-2; going down from there, the first step that lands in `slot`
    for (int t = T - 2; t >= -1 && t > T - 2 - kRecBwdPartSlots; --t)
        if ((t + 3) % kRecBwdPartSlots == slot) return (unsigned(t) & 1u) ^ 1u;
    return 0u;
}

void StepGraphCache::clear() {
    for (auto& e : entries) {
        if (e.exec) (void)hipGraphExecDestroy(e.exec);
        if (e.graph) (void)hipGraphDestroy(e.graph);
    }
    entries.clear();
}

// Runs `launch_all` (plain launches of a range of steps on `stream`) either directly or, when a cache is given and
// the stream can be captured, as a graph: built on first use for this key, replayed afterwards.
template <typename LaunchAll>
static hipError_t launch_steps(StepGraphCache* graphs, const void* kernel, const void* args, size_t args_bytes,
                               const RecLayout& L, int t_a, int t_b, int nsteps, hipStream_t stream,
                               LaunchAll&& launch_all) {
    if (!graphs || graphs->disabled || stream == nullptr || nsteps < kGraphMinSteps || nsteps > kGraphMaxSteps)
        return launch_all();
    std::vector<unsigned char> key(sizeof(kernel) + args_bytes + sizeof(RecLayout) + 2 * sizeof(int));
    unsigned char* k = key.data();
    memcpy(k, &kernel, sizeof(kernel)); k += sizeof(kernel);
    memcpy(k, args, args_bytes); k += args_bytes;
    memcpy(k, &L, sizeof(RecLayout)); k += sizeof(RecLayout);
    memcpy(k, &t_a, sizeof(int)); k += sizeof(int);
    memcpy(k, &t_b, sizeof(int));
    for (auto& e : graphs->entries)
        if (e.key == key) {
            e.stamp = ++graphs->clock;
            graphs->replays++;
            return hipGraphLaunch(e.exec, stream);
        }
    // not seen before: capture the launches (nothing runs yet), instantiate, launch
    if (hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
        (void)hipGetLastError();
        graphs->disabled = true;
        return launch_all();
    }
    hipError_t le = launch_all();
    hipGraph_t graph = nullptr;
    hipError_t ce = hipStreamEndCapture(stream, &graph);
    if (le != hipSuccess || ce != hipSuccess || !graph) {
        if (graph) (void)hipGraphDestroy(graph);
        (void)hipGetLastError();
        graphs->disabled = true;
        return le != hipSuccess ? le : launch_all();
    }
    hipGraphExec_t exec = nullptr;
    if (hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) != hipSuccess || !exec) {
        (void)hipGraphDestroy(graph);
        (void)hipGetLastError();
        graphs->disabled = true;
        return launch_all();
    }
    if (graphs->entries.size() >= kGraphCacheEntries) {   // drop the least recently used graph
        size_t victim = 0;
        for (size_t i = 1; i < graphs->entries.size(); ++i)
            if (graphs->entries[i].stamp < graphs->entries[victim].stamp) victim = i;
        (void)hipGraphExecDestroy(graphs->entries[victim].exec);
        (void)hipGraphDestroy(graphs->entries[victim].graph);
        graphs->entries.erase(graphs->entries.begin() + victim);
    }
    StepGraphCache::Entry e;
    e.key = std::move(key); e.graph = graph; e.exec = exec; e.stamp = ++graphs->clock;
    graphs->entries.push_back(std::move(e));
    graphs->captures++;
    return hipGraphLaunch(exec, stream);
}

template <int NT, int KS, bool RES, int MT, bool DS, bool DEEP = false>
static hipError_t run_fwd(const RecLayout& L, const RecFwdArgs& a, hipStream_t stream, StepGraphCache* graphs) {
    constexpr int NW = 4;
    auto kernel = rec_fwd_kernel<NT, KS, RES, MT, DS, DEEP>;
    if (L.nw != NW) return hipErrorInvalidValue;   // (the weight fragments are packed for L.nw waves)
    const size_t lds = size_t(2) * NW * kRows * (16 * NT + kPartPad) * sizeof(float);
    hipError_t e = raise_lds(kernel, lds);
    if (e != hipSuccess) return e;
    const int ks_wave = rec_fwd_ks(L, a.Hp);
    if (L.persistent) return launch_persistent(kernel, L.grid, lds, stream, a, L, a.t0, a.t1, ks_wave, NW * kWave);
    return launch_steps(graphs, reinterpret_cast<const void*>(kernel), &a, sizeof(a), L, a.t0, a.t1, a.t1 - a.t0, stream,
                        [&]() -> hipError_t {
                            for (int t = a.t0; t < a.t1; ++t) {
                                hipLaunchKernelGGL(kernel, dim3(L.grid), dim3(NW * kWave), lds, stream, a, L, t, t + 1, ks_wave);
                                hipError_t le = hipGetLastError();
                                if (le != hipSuccess) return le;
                            }
                            return hipSuccess;
                        });
}

template <bool DS>
static hipError_t run_fwd_il(const RecLayout& L, const RecFwdArgs& a, hipStream_t stream, StepGraphCache* graphs) {
    constexpr int NT = 8, NW = 8;
    auto kernel = rec_fwd_il_kernel<NT, 4, DS>;
    if (L.nw != NW || L.nt != NT || L.mt != 2 || !L.resident) return hipErrorInvalidValue;
    const size_t lds = size_t(2) * NW * 16 * (16 * NT + kPartPad) * sizeof(float);
    hipError_t e = raise_lds(kernel, lds);
    if (e != hipSuccess) return e;
    const int ks_wave = rec_fwd_ks(L, a.Hp);
    if (L.persistent) return launch_persistent(kernel, L.grid, lds, stream, a, L, a.t0, a.t1, ks_wave, NW * kWave);
    return launch_steps(graphs, reinterpret_cast<const void*>(kernel), &a, sizeof(a), L, a.t0, a.t1, a.t1 - a.t0, stream,
                        [&]() -> hipError_t {
                            for (int t = a.t0; t < a.t1; ++t) {
                                hipLaunchKernelGGL(kernel, dim3(L.grid), dim3(NW * kWave), lds, stream, a, L, t, t + 1, ks_wave);
                                hipError_t le = hipGetLastError();
                                if (le != hipSuccess) return le;
                            }
                            return hipSuccess;
                        });
}

hipError_t launch_rec_fwd(const RecLayout& L, const RecFwdArgs& a, hipStream_t stream, StepGraphCache* graphs) {
    if (a.T <= 0 || a.B <= 0 || a.t1 <= a.t0) return hipSuccess;
    if (a.Hp % 32 != 0 || a.Hp % L.jb != 0 || a.t0 < 0 || a.t1 > a.T) return hipErrorInvalidValue;
    // device-scope stores into the exchange ring: a persistent launch whose groups span XCDs
    const bool ds = L.persistent && !L.xcd_local;
    if (!L.resident) return run_fwd<8, 1, false, 2, false>(L, a, stream, graphs);
    if (L.nw == 8)   // eight waves: the interleaved kernel, 32-row blocks
        return ds ? run_fwd_il<true>(L, a, stream, graphs) : run_fwd_il<false>(L, a, stream, graphs);
    if (L.nt == 8) {
        if (L.mt == 1) return ds ? run_fwd<8, 8, true, 1, true>(L, a, stream, graphs) : run_fwd<8, 8, true, 1, false>(L, a, stream, graphs);
        return ds ? run_fwd<8, 8, true, 2, true>(L, a, stream, graphs) : run_fwd<8, 8, true, 2, false>(L, a, stream, graphs);
    }
    if (L.nt == 4) {
        if (L.mt == 1) return ds ? run_fwd<4, 16, true, 1, true>(L, a, stream, graphs) : run_fwd<4, 16, true, 1, false>(L, a, stream, graphs);
        if (!ds) return run_fwd<4, 16, true, 2, false>(L, a, stream, graphs);
        const bool several_blocks = L.nrb >= 2 * L.ng;   // every workgroup takes at least two row blocks per step
        return several_blocks ? run_fwd<4, 16, true, 2, true, true>(L, a, stream, graphs) : run_fwd<4, 16, true, 2, true>(L, a, stream, graphs);
    }
    return hipErrorInvalidValue;
}

template <int NT, int KS, bool RES, int KL, int MT, bool DS>
static hipError_t run_bwd(const RecLayout& L, const RecBwdArgs& a, hipStream_t stream, StepGraphCache* graphs) {
    constexpr int NW = 4;
    auto kernel = rec_bwd_kernel<NT, KS, RES, KL, MT, DS>;
    if (L.nw != NW) return hipErrorInvalidValue;   // (the weight fragments are packed for L.nw waves)
    static_assert(size_t(2) * NW * kRows * (16 * NT + kPartPad) >= size_t(NW * kWave) * 8 * NT, "db reduction reuses the partial-sum area");
    const size_t lds = size_t(2) * NW * kRows * (16 * NT + kPartPad) * sizeof(float) + size_t(NW) * KL * NT * kWave * sizeof(half8);
    hipError_t e = raise_lds(kernel, lds);
    if (e != hipSuccess) return e;
    const int ks_wave = rec_bwd_ks(L, a.Hp);
    if (L.persistent) return launch_persistent(kernel, L.grid, lds, stream, a, L, a.t_hi, a.t_lo, ks_wave, NW * kWave);
    return launch_steps(graphs, reinterpret_cast<const void*>(kernel), &a, sizeof(a), L, a.t_hi, a.t_lo, a.t_hi - a.t_lo + 1,
                        stream, [&]() -> hipError_t {
                            for (int t = a.t_hi; t >= a.t_lo; --t) {
                                hipLaunchKernelGGL(kernel, dim3(L.grid), dim3(NW * kWave), lds, stream, a, L, t, t, ks_wave);
                                hipError_t le = hipGetLastError();
                                if (le != hipSuccess) return le;
                            }
                            return hipSuccess;
                        });
}

template <int MT, int KQ, int NM, int KS, bool LOCAL>
static hipError_t run_bwd2d(const RecLayout& L, const RecBwdArgs& a, hipStream_t stream) {
    auto kernel = rec_bwd2d_kernel<MT, KQ, NM, KS, LOCAL>;
    constexpr int KL = (KS == 16) ? 5 : 0;   // k-steps per wave whose weights live in LDS (as in the kernel)
    const size_t lds = size_t(2) * 4 * kRows * (64 + kPartPad) * sizeof(float) + size_t(4) * KL * 4 * kWave * sizeof(half8);
    hipError_t e = raise_lds(kernel, lds);
    if (e != hipSuccess) return e;
    return launch_persistent(kernel, L.grid, lds, stream, a, L, a.t_hi, a.t_lo, 0);
}

hipError_t launch_rec_bwd(const RecLayout& L, const RecBwdArgs& a, hipStream_t stream, StepGraphCache* graphs) {
    if (a.T <= 0 || a.B <= 0 || a.t_hi < a.t_lo) return hipSuccess;
    if (a.Hp % 32 != 0 || a.Hp % L.jb != 0 || a.t_lo < -1 || a.t_hi >= a.T) return hipErrorInvalidValue;
    if (L.two_d) {
        // what the kernel's indexing assumes
        const bool local = a.Hp == 1024;
        const int ng = local ? 8 : (L.kq == 8 ? 1 : 2);
        if (!L.persistent || (a.Hp != 2048 && a.Hp != 1024) || L.grid != 256 || L.ng != ng || L.nrb < 1 ||
            (L.nrb + ng - 1) / ng > L.nm || !a.wfrag2 || !a.P || a.b_lo < 0 || a.b_lo % 32 != 0 || a.b_hi <= a.b_lo ||
            a.b_hi > a.B || L.nrb * 16 * L.mt < a.b_hi - a.b_lo ||
            a.p_slot != rec_bwd_part_slot_floats(L) || (a.Hp / 64) * L.kq * ng != 256)
            return hipErrorInvalidValue;
        if (local) {
            if (L.kq == 2 && L.mt == 2 && L.nm == 1) return run_bwd2d<2, 2, 1, 16, true>(L, a, stream);
            return hipErrorInvalidValue;
        }
        if (L.kq == 8 && L.nm == 1)
            return L.mt == 1 ? run_bwd2d<1, 8, 1, 8, false>(L, a, stream) : run_bwd2d<2, 8, 1, 8, false>(L, a, stream);
        if (L.kq == 8 && L.nm == 2 && L.mt == 2) return run_bwd2d<2, 8, 2, 8, false>(L, a, stream);
        if (L.kq == 4 && L.mt == 2) {
            if (L.nm == 1) return run_bwd2d<2, 4, 1, 16, false>(L, a, stream);
            if (L.nm == 2) return run_bwd2d<2, 4, 2, 16, false>(L, a, stream);
        }
        return hipErrorInvalidValue;
    }
    const bool ds = L.persistent && !L.xcd_local;   // (as in launch_rec_fwd)
    if (!L.resident) return run_bwd<2, 1, false, 0, 2, false>(L, a, stream, graphs);
    if (L.nt == 2) {
        if (L.mt == 1) return ds ? run_bwd<2, 32, true, 8, 1, true>(L, a, stream, graphs) : run_bwd<2, 32, true, 8, 1, false>(L, a, stream, graphs);
        return ds ? run_bwd<2, 32, true, 8, 2, true>(L, a, stream, graphs) : run_bwd<2, 32, true, 8, 2, false>(L, a, stream, graphs);
    }
    if (L.nt == 1) {
        if (L.mt == 1) return ds ? run_bwd<1, 64, true, 24, 1, true>(L, a, stream, graphs) : run_bwd<1, 64, true, 24, 1, false>(L, a, stream, graphs);
        return ds ? run_bwd<1, 64, true, 24, 2, true>(L, a, stream, graphs) : run_bwd<1, 64, true, 24, 2, false>(L, a, stream, graphs);
    }
    return hipErrorInvalidValue;
}

}  // namespace flstm_hip
