// Persistent, W_hh-resident recurrence kernels (forward and BPTT) for gfx950.
#pragma once
#include <vector>

#include "common.h"

namespace flstm_hip {

// How the hidden dimension is cut over workgroups, and how workgroups are tied into groups that
// exchange h_t (forward) or dG_t (backward) every step.
struct RecLayout {
    int nt;          // forward: 16-wide gate-column tiles per workgroup (JB = 4*nt hidden units)
    int jb;          // hidden units per workgroup slice
    int nh;          // slices = Hp / jb  (workgroups per group)
    int nrb;         // batch blocks of 16*mt rows
    int mt;          // 16-row MFMA tiles per batch block: 1 when all 16-row blocks can run side by side, else 2
    int ng;          // concurrently running groups; group g owns row blocks g, g+ng, ...
    int gpx;         // XCD-local mode: groups per XCD
    int xcd_local;   // 1: every group lives inside one XCD (plain stores + L2-served loads)
    int persistent;  // 1: one launch walks all steps, 0: one launch per step
    int resident;    // 1: weight fragments live in registers for the whole launch
    int grid;        // workgroups per launch
    int cooperative; // host side: 1 = persistent launches go through hipLaunchCooperativeKernel (set by the plan)
    int rot_div;     // k-step rotation (rec_kstep_rotation): slices rot_div apart run on the same XCD
    int two_d;       // backward, 2048 hidden units: workgroups split the product over output columns AND the contraction
                     // (32 column slices x kq contraction slices, partial sums exchanged inside an XCD); nt, jb, nh
                     // still describe the one-dimensional layout, whose weight fragments the step-wise fallback uses
    int kq;          // two_d: contraction slices, 8 (one group of 256 workgroups) or 4 (two groups of 128)
    int nm;          // two_d: passes per step the kernel is built for (row blocks per workgroup, rounded up to 1, 2, 4)
    int win_rows;    // two_d: 0, or the batch is walked in windows of this many rows, one persistent launch each (batch
                     // rows are independent sequences); nrb, mt, ng, nm then describe one window
    int nw;          // wavefronts per workgroup of the one-way kernels, which split the contraction between them: 4, or
                     // (forward, slices of 32 units) 8, two per SIMD, with 32-row blocks whose two row tiles take turns
                     // (rec_fwd_il_kernel).  The weight fragments are packed for this count, so it is a function of
                     // the sizes alone and does not follow mt
};

struct RecFwdArgs {
    const half8* wfrag;  // [nh][nw waves][ks][nt][64 lanes] MFMA B-fragments of W_hh (packed gate order)
    half_t* Y;           // [(T+1)*B][Hp]; rows [0,B) = h0, rows [(t+1)B, (t+2)B) = h_t (row-major, for later kernels)
    half_t* X;           // exchange ring, 4 slots of x_slot halfs, fragment-major; step t reads slot t%4 (h_{t-1}),
                         // writes slot (t+1)%4; before step 0 slot 0 holds h0 (padding rows zero) and the
                         // other three hold the 0xFFFF 'unwritten' pattern
    size_t x_slot;
    half_t* y_out;       // optional: the caller's output tensor [T*B][Hp] fp16 (only when its rows equal the state
                         // rows: fp16, hidden size = Hp); h_t is then stored there as well, which saves the copy
    half_t* G;           // [T*B][4Hp] packed gate order; in: x-projection + bias, out: activated i,f,g,o
    float* C;            // [(T+1)*B][Hp]; rows [0,B) = c0, rows [(t+1)B, ..) = c_t
    unsigned* seats;     // [8] zeroed before every launch: next free workgroup slot per XCD
    int* delay_hint;     // may be null: where a launch that regulates its first requests finds the delay its predecessor
                         // settled on, and leaves its own (a sequence fed in ranges of steps does not start over)
    int* status;         // 0 ok, 1 spin limit hit, 2 workgroup not on the expected XCD
    int B, Hp, T;
    int t0, t1;          // steps [t0, t1) of the sequence are run by this call (state and ring carry over)
    int spin_limit;      // reloads of a fragment chunk that still shows the 'unwritten' pattern before giving up
    long long spin_ticks;   // the same bound as time: ticks of the device's constant-rate wall clock
    long long* prof;     // optional [8] cycle counters of workgroup 0 per phase (null = off)
};

struct RecBwdArgs {
    const half8* wfrag;  // [nh][nw waves][ks][nt][64] B-fragments of W_hh^T (rows = hidden k, contraction = packed gate q)
    const half_t* G;     // activated gates cache [T*B][4Hp]
    const float* C;      // cell states [(T+1)*B][Hp]
    const half_t* dY;    // [T*B][Hp] upstream gradient
    half_t* dG;          // [T*B][4Hp] pre-activation gradients (scaled), row-major, for the GEMMs
    half_t* X;           // exchange ring, 4 slots of x_slot halfs, fragment-major; step t writes slot t%4 (dG_t);
                         // before the first step all four hold the 0xFFFF 'unwritten' pattern
                         // (two-dimensional layout: rec_bwd_dg_slots() = 8 slots, step t writes slot t%8)
    size_t x_slot;
    const half8* wfrag2; // two-dimensional layout: [32 column slices][kq contraction slices][4 waves][64/kq k-steps][4 tiles][64]
    float* P;            // two-dimensional layout: ring of 3 slots of p_slot floats for the partial sums; before the first
                         // step the lowest bit of every word of slot (t+3)%3 is the opposite of t&1 for the first step t
                         // that uses the slot (rec_bwd_part_fill)
    size_t p_slot;
    float* dHn;          // [B][Hp] scaled gradient wrt final h (zeros when absent)
    float* dC;           // [B][Hp] running scaled dc; in: gradient wrt final c, out: dc0
    float* dH0;          // [B][Hp] out: scaled gradient wrt h0
    float* db_part;      // [ng][4Hp] scaled bias-gradient partial sums (accumulated into)
    unsigned* seats;     // [8] zeroed before every launch
    int* delay_hint;     // as in RecFwdArgs
    int* status;
    int B, Hp, T;
    int b_lo, b_hi;      // two-dimensional layout: the launch works on batch rows [b_lo, b_hi) (b_lo a multiple of 32;
                         // every array keeps its full-batch strides, the rings are indexed by the row in the batch)
    float dy_scale;      // factor applied to dY on load (the loss scale, or 1 when dY is pre-scaled)
    int t_hi, t_lo;      // steps t_hi down to t_lo are run by this call; t_lo = -1 adds the closing dh0 product
    int spin_limit;
    long long spin_ticks;
    long long* prof;     // optional [8] cycle counters of workgroup 0 per phase (null = off)
};

// Which k-step a wave's register slot holds.  The workgroups of one XCD that belong to the same group fetch the same
// exchanged operand every step, and walking its k-steps in the same order they ask for the same lines at the same
// moment.  Where that operand is large and comes through memory from the other XCDs, spreading the requests pays
// (rot_div > 0; 0 = no rotation): slice `hs` starts `rotation` k-steps further on and wraps round: slot ks of a wave holds the weights of (and fetches) k-step
// 4 * ((ks + rotation) % ks_wave) + wave.  Slices that share an XCD are `rot_div` apart (1 where a group sits inside
// one XCD, 8 where the workgroups of a group are dealt round-robin over the 8 XCDs), and their rotations are spread
// evenly over the ks_wave positions.  The weight packing and the kernels use the same function.
__host__ __device__ inline int rec_kstep_rotation(int hs, int nh, int ks_wave, int rot_div) {
    if (ks_wave <= 1 || rot_div <= 0) return 0;
    const int mates = nh / rot_div > 0 ? nh / rot_div : 1;   // slices of a group on one XCD
    const int r = hs / rot_div;
    return (ks_wave >= mates ? r * (ks_wave / mates) : r) % ks_wave;
}
// The same idea in the two-way backward layout with 8 contraction slices (one group of 256 workgroups, batches of one
// row block): the 4 column slices of an XCD that share a contraction slice fetch the same fragments, and slice s starts
// a quarter of the way further round than slice s - 1.  Measured at 16 rows: 3.71 -> 3.50 us per step.  With 4
// contraction slices and two passes per step it cost 2 % (9.0 -> 9.2 us at 128 rows) and is off, as it is at 1024 units.
__host__ __device__ inline int rec_bwd2d_rotation(int s, int ks_wave, int kq) {
    if (kq != 8 || ks_wave < 4) return 0;
    return ((s % 4) * (ks_wave / 4)) % ks_wave;
}
__host__ __device__ inline int rec_kstep_of_slot(int ks, int rotation, int ks_wave) {
    if (ks >= ks_wave) return ks;   // slots past the real contraction hold zero weights
    const int k = ks + rotation;
    return k >= ks_wave ? k - ks_wave : k;
}

// Step-wise launches as hipGraphs.  Where the persistent kernels cannot be used (weights that do not fit on chip,
// a plan demoted after a give-up, "stepwise" forced) a pass is one launch per time step; the launches of a range of
// steps are captured once into a graph and replayed on later passes with the same arguments (what the reference
// does with its CUDA graph, src/lstm.cu:1373-1895).  A cache belongs to one plan and holds a few instantiated
// graphs keyed by the complete kernel arguments; streams that cannot be captured (the legacy default stream) and
// ranges shorter than kGraphMinSteps take plain launches.
struct StepGraphCache {
    struct Entry {
        std::vector<unsigned char> key;
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        unsigned long stamp = 0;
    };
    std::vector<Entry> entries;
    unsigned long clock = 0;
    long captures = 0, replays = 0;   // graphs built / graph launches (for tests and tuning)
    bool disabled = false;            // capture failed once on this plan's stream: plain launches from then on
    ~StepGraphCache() { clear(); }
    void clear();
};
constexpr int kGraphMinSteps = 8;
constexpr int kGraphMaxSteps = 1 << 16;
constexpr size_t kGraphCacheEntries = 4;

// Picks tile shapes and the group structure for a problem size on the current device.  force_mt: 0 = the rule of
// thumb (16-row blocks whenever all of them can run side by side), 1 / 2 = that many 16-row tiles per row block
// (1 only where it fits).  The choice does not change the weight-fragment layout.
// waves: 0 = the rule of thumb (rec_waves), 4 or 8 = that many wavefronts per workgroup (8 only up to 1024 units).
RecLayout plan_rec_fwd(int B, int Hp, int num_cus, bool force_stepwise, int force_mt = 0, int waves = 0);
// two_d: 0 = never the two-way split, 1 = where it is the faster layout, 2 = wherever it can run
RecLayout plan_rec_bwd(int B, int Hp, int num_cus, bool force_stepwise, int force_mt = 0, int two_d = 1);
// Wavefronts per workgroup the forward kernel runs with for these sizes (a function of the sizes alone).
int rec_waves(int B, int Hp, int num_cus, int waves);

// The two-dimensional backward layout: whether a device/size can use it at all (decides whether its weight fragments
// are packed) and with how many contraction slices (a function of the sizes alone, so that the packed weights fit
// whatever the options say later), slots of its dG ring, floats per slot of its partial ring and bytes of its weight
// fragments.
bool rec_bwd_two_d_possible(int Hp, int num_cus);
int rec_bwd_two_d_kq(int B, int Hp);
int rec_bwd_dg_slots(const RecLayout& L);
size_t rec_bwd_part_slot_floats(const RecLayout& L);
constexpr int kRecBwdPartSlots = 3;
size_t rec_bwd_two_d_wfrag_bytes(int Hp);
// Word to fill slot `slot` of the partial ring with before a pass over T steps (see RecBwdArgs::P).
unsigned rec_bwd_part_fill(int slot, int T);
// Batch rows the rings of a backward layout are sized for (whole windows where the batch is walked in windows).
int rec_bwd_ring_rows(const RecLayout& L, int B);

// Halfs in one slot of an exchange ring for a [rows][cols] operand (rows padded to 32).
size_t exchange_slot_halfs(int rows, int cols);
// Row-major [rows][cols] (cols % 32 == 0) -> fragment-major exchange layout.
hipError_t to_exchange_layout(const half_t* in, int rows, int cols, size_t ld, half_t* out, hipStream_t s);

// Number of k-steps (32 wide) every wave holds for a layout (sizes the fragment arrays).
int rec_fwd_ks(const RecLayout& L, int Hp);
int rec_bwd_ks(const RecLayout& L, int Hp);

// Runs steps [t0, t1). Persistent layouts use one launch; otherwise one launch per step.
hipError_t launch_rec_fwd(const RecLayout& L, const RecFwdArgs& a, hipStream_t stream, StepGraphCache* graphs = nullptr);
// Runs steps t_hi .. t_lo (the whole pass is T-1 .. -1: all steps and the final dh0 product).
hipError_t launch_rec_bwd(const RecLayout& L, const RecBwdArgs& a, hipStream_t stream, StepGraphCache* graphs = nullptr);

}  // namespace flstm_hip
