// Plan object and orchestration of the device-resident LSTM forward / BPTT core.
//
// Forward  = [convert x] -> MFMA GEMM  G = X * W_ih^T  (hoisted input projection, the chunked
//            "projchunksz" GEMM of src/lstm.cu:1204-1239) -> persistent recurrence kernel that turns G
//            in place into the fp16 gate cache and fills the h / c state arrays -> [unpad outputs].
// Backward = persistent BPTT kernel (reads gate cache + c states, writes dG) -> dX = dG * W_ih
//            -> dW = dG^T * [X ; H_prev] as one split-K GEMM -> reductions into caller layout.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <cmath>
#include <mutex>
#include <new>
#include <vector>

#include "../../include/flashlstm/lstm_core.h"
#include "gemm.h"
#include "pack.h"
#include "recurrent.h"

using namespace flstm_hip;

// Scratch memory of flstm_core_forward_static: everything that entry point's kernels need beyond the caller's
// tensors and the plan's packed weights (status word and seat counters, converted x rows, x-projection / gate rows,
// state rows, exchange ring).  One array per device, owned by the code object; host code reaches it only through
// the address hipGetSymbolAddress returns for the device that is current (static_scratch()).
static constexpr size_t kStaticScratchBytes = size_t(64) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

// address of `scratch` on the current device (looked up once per device)
static int static_scratch(int dev, void** out) {
    if (dev < 0 || dev >= kMaxDevices) return FLSTM_E_INVALID;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return int(e);
        if (!ptr) return int(hipErrorInvalidSymbol);
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

namespace {

struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
    bool borrowed = false;   // a view of memory owned elsewhere: never grown, never freed
    // grows (never shrinks); contents are lost on growth
    hipError_t reserve(size_t need) {
        if (need <= bytes) return hipSuccess;
        if (borrowed) return hipErrorOutOfMemory;
        if (p) { hipError_t e = hipFree(p); p = nullptr; bytes = 0; if (e != hipSuccess) return e; }
        hipError_t e = hipMalloc(&p, need);
        if (e == hipSuccess) bytes = need;
        return e;
    }
    void release() { if (p && !borrowed) (void)hipFree(p); p = nullptr; bytes = 0; borrowed = false; }
    template <typename T> T* as() const { return static_cast<T*>(p); }
    static DevBuf view(void* ptr, size_t n) { DevBuf b; b.p = ptr; b.bytes = n; b.borrowed = true; return b; }
};

struct PhaseTimer {
    hipEvent_t ev[8] = {};
    bool ok = false;
    hipError_t init() {
        for (auto& e : ev) { hipError_t r = hipEventCreate(&e); if (r != hipSuccess) return r; }
        ok = true;
        return hipSuccess;
    }
    void destroy() { if (ok) for (auto& e : ev) (void)hipEventDestroy(e); ok = false; }
};

}  // namespace

constexpr int kFirstHold = 8, kMaxHold = 1024;

struct flstm_core_plan {
    int device = 0;
    int num_cus = 0;
    int clock_khz = 0;   // maximum engine clock the runtime reports
    Dims d{};
    RecLayout Lf{}, Lb{};
    int ks_f = 0, ks_b = 0;
    // options
    int opt_stepwise = 0, opt_proj_chunk = 0, opt_spin_limit = 1 << 30, opt_spin_ms = 250, opt_dw_splits = 0, opt_accumulate = 0;
    // A persistent launch that gave up (its workgroups were not all running at once, or not spread over the XCDs
    // as expected) demotes that direction to step-wise launches for `hold` passes; then the persistent kernel is
    // tried again.  Every further give-up doubles the hold (at most kMaxHold passes).
    int hold_fwd = 0, hold_bwd = 0, backoff_fwd = kFirstHold, backoff_bwd = kFirstHold;
    long fallbacks = 0, demotions_fwd = 0, demotions_bwd = 0;
    // A cooperative launch refused because the grid cannot be co-resident: that direction runs step-wise from then on.
    bool refused_fwd = false, refused_bwd = false;
    long coop_refusals = 0;
    bool static_call = false;   // flstm_core_forward_static in force: nothing may allocate (no graph capture either)
    // Tuned launch choices per sequence length (flstm_core_tune): 16- or 32-row blocks and persistent or step-wise
    // launches per direction, split-K count of the weight-gradient GEMM.  eff_* hold the entry in force for the
    // sequence length of the current pass (0 = no tuned value: the rules of thumb decide); explicit options win.
    struct Tuned { size_t T; int mt_f, mt_b, step_f, step_b, dw_splits, two_d; float ms_f, ms_b, ms_dw; };   // two_d: -1 = not tuned, else the bwd_two_d option
    std::vector<Tuned> tuned;
    int opt_mt_f = 0, opt_mt_b = 0;
    int eff_mt_f = 0, eff_mt_b = 0, eff_step_f = 0, eff_step_b = 0, eff_dw = 0, eff_two_d = -1;
    bool two_d_explicit = false;   // option "bwd_two_d" (or its environment variable) was given: a tuned value does not replace it
    size_t eff_T = 0;
    int opt_cooperative = 1;
    StepGraphCache graphs_f, graphs_b;   // captured step-wise launches (only used where the persistent kernels are not)
    int opt_graphs = 1;
    int opt_two_d = 1;   // backward recurrence for 2048 hidden units, two-way split: 0 never, 1 where it is faster, 2 wherever it can run
    int opt_waves_f = 0;   // wavefronts per workgroup of the forward recurrence: 0 = by size, 4, 8 (the weights are packed for it)
    int* status_host = nullptr;   // pinned: the device status word lands here with the end-of-pass copy
    int inject_stall = 0;         // test hook: treat the next N passes as if their launches had given up
    // weights
    DevBuf wih_p, wih_t, wfrag_f, wfrag_b, wfrag_b2, bias_p;
    bool weights_packed = false, bias_packed = false;
    // forward state / caches
    DevBuf X16, G, Y, C, status, xch_f, xch_b;
    size_t T_cache = 0;
    bool have_cache = false;
    // pass in progress (begin / steps / end)
    struct { size_t T = 0; const void* x = nullptr; flstm_dtype x_dtype = FLSTM_F16; bool open = false;
             half_t* y_direct = nullptr; bool seats_clean = false; } fw;   // y_direct: the recurrence writes the caller's y itself
    // (seats_clean: the pass's setup has zeroed the seat counters for the first recurrence launch that follows it)
    struct { size_t T = 0; const half_t* dYk = nullptr; const void* dY = nullptr; flstm_dtype dy_dtype = FLSTM_F16;
             float S = 1.f, dy_scale = 1.f; void* dx = nullptr; flstm_dtype dx_dtype = FLSTM_F16; bool open = false;
             bool seats_clean = false; } bw;
    // backward scratch
    DevBuf dYp, dG, dHn, dC, dH0, db_part, dw_part, prof, part_b;
    int opt_profile = 0, wall_khz = 100000;
    long long prof_f[8] = {}, prof_b[8] = {};
    PhaseTimer tm;
    float ms_fwd[3] = {-1, -1, -1}, ms_bwd[4] = {-1, -1, -1, -1};
};

namespace {

#define FL_TRY(expr)                                  \
    do {                                              \
        hipError_t _e = (expr);                       \
        if (_e != hipSuccess) return int(_e);         \
    } while (0)

void replan(flstm_core_plan* p) {
    p->Lf = plan_rec_fwd(p->d.B, p->d.Hp, p->num_cus, p->opt_stepwise || p->hold_fwd > 0 || p->eff_step_f || p->refused_fwd,
                         p->opt_mt_f ? p->opt_mt_f : p->eff_mt_f, p->opt_waves_f);
    p->Lb = plan_rec_bwd(p->d.B, p->d.Hp, p->num_cus, p->opt_stepwise || p->hold_bwd > 0 || p->eff_step_b || p->refused_bwd,
                         p->opt_mt_b ? p->opt_mt_b : p->eff_mt_b,
                         (!p->two_d_explicit && p->eff_two_d >= 0) ? p->eff_two_d : p->opt_two_d);
    p->Lf.cooperative = p->Lb.cooperative = p->opt_cooperative;
    p->ks_f = rec_fwd_ks(p->Lf, p->d.Hp);
    p->ks_b = rec_bwd_ks(p->Lb, p->d.Hp);
}

// Puts the tuned entry for sequence length T in force: the entry tuned at exactly T, else the nearest one within a
// factor of two, else none.
void use_tuned(flstm_core_plan* p, size_t T) {
    const flstm_core_plan::Tuned* best = nullptr;
    double best_d = 1.0;   // |log2(T / T')| <= 1
    for (const auto& t : p->tuned) {
        const double dist = std::fabs(std::log2(double(T) / double(t.T)));
        if (dist <= best_d && (!best || dist < best_d)) { best = &t; best_d = dist; }
    }
    const int mt_f = best ? best->mt_f : 0, mt_b = best ? best->mt_b : 0, sf = best ? best->step_f : 0,
              sb = best ? best->step_b : 0, td = best ? best->two_d : -1;
    p->eff_dw = best ? best->dw_splits : 0;
    p->eff_T = best ? best->T : 0;
    if (mt_f != p->eff_mt_f || mt_b != p->eff_mt_b || sf != p->eff_step_f || sb != p->eff_step_b || td != p->eff_two_d) {
        p->eff_mt_f = mt_f; p->eff_mt_b = mt_b; p->eff_step_f = sf; p->eff_step_b = sb; p->eff_two_d = td;
        replan(p);
    }
}

// The status word of the recurrence kernels travels to pinned host memory behind the pass's last kernel, so the
// wait that ends the pass anyway is also the one that makes it readable: no second round trip to the device.
int enqueue_status_copy(flstm_core_plan* p, hipStream_t s) {
    FL_TRY(hipMemcpyAsync(p->status_host, p->status.p, sizeof(int), hipMemcpyDeviceToHost, s));
    return 0;
}
// after the stream has been waited for: the status of the pass; a non-zero one is cleared on the device
int take_status(flstm_core_plan* p, bool fwd, hipStream_t s, int* out) {
    *out = *static_cast<volatile int*>(p->status_host);
    if (*out != 0) FL_TRY(fill_zero(p->status.p, sizeof(int), s));
    (void)fwd;
    if (*out == 0 && p->inject_stall > 0) {   // (2 in a row: the step-wise repeat of a pass fails too, i.e. the call does)
        p->inject_stall--;
        *out = 1;
    }
    return 0;
}
int wait_status(flstm_core_plan* p, bool fwd, hipStream_t s, int* out) {
    int rc = enqueue_status_copy(p, s);
    if (rc) return rc;
    FL_TRY(hipStreamSynchronize(s));
    return take_status(p, fwd, s, out);
}

// A persistent launch gave up: step-wise launches for the next `hold` passes of that direction.
void demote(flstm_core_plan* p, bool fwd) {
    int& hold = fwd ? p->hold_fwd : p->hold_bwd;
    int& backoff = fwd ? p->backoff_fwd : p->backoff_bwd;
    hold = backoff;
    backoff = backoff * 2 > kMaxHold ? kMaxHold : backoff * 2;
    (fwd ? p->demotions_fwd : p->demotions_bwd)++;
    p->fallbacks++;
    replan(p);
}
// A pass of a demoted direction went through: one pass less to hold; at zero the persistent kernel is back.
void pass_done(flstm_core_plan* p, bool fwd) {
    int& hold = fwd ? p->hold_fwd : p->hold_bwd;
    if (hold > 0 && --hold == 0) replan(p);
}

float elapsed(hipEvent_t a, hipEvent_t b) {
    float ms = -1.f;
    if (hipEventElapsedTime(&ms, a, b) != hipSuccess) return -1.f;
    return ms;
}

}  // namespace

extern "C" int flstm_core_create(size_t batch, size_t input_size, size_t hidden_size, flstm_core_plan** out) {
    if (!out) return FLSTM_E_INVALID;
    *out = nullptr;
    if (batch == 0 || input_size == 0 || hidden_size == 0) return FLSTM_E_INVALID;
    if (batch > (1u << 20) || input_size > (1u << 20) || hidden_size > (1u << 18)) return FLSTM_E_INVALID;
    auto* p = new (std::nothrow) flstm_core_plan();
    if (!p) return int(hipErrorOutOfMemory);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&p->num_cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess && hipDeviceGetAttribute(&p->clock_khz, hipDeviceAttributeClockRate, dev) != hipSuccess)
        p->clock_khz = 0;
    if (e == hipSuccess && (hipDeviceGetAttribute(&p->wall_khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess ||
                            p->wall_khz <= 0))
        p->wall_khz = 100000;
    if (e != hipSuccess) { delete p; return int(e); }
    p->device = dev;
    {   // this device's copy of the static scratch array: looked up now, while its device is current
        void* sp = nullptr;
        const int rc = static_scratch(dev, &sp);
        if (rc) { delete p; return rc; }
    }
    p->d.B = int(batch);
    p->d.I = int(input_size);
    p->d.H = int(hidden_size);
    p->d.Ip = int(round_up(input_size, 64));
    p->d.Hp = int(round_up(hidden_size, 32));
    // Persistent launches are cooperative launches (co-residency of the whole grid is then a condition of the launch
    // instead of an assumption) -- except under a rocprofiler-sdk tool: with rocprofv3 attached, a process that has
    // made a cooperative launch takes a segmentation fault inside the tool when it exits (results and traces are
    // complete by then; seen with ROCm 7.2), so plain launches are used there.  FLASHLSTM_COOPERATIVE_LAUNCH=0/1
    // or the option "cooperative" decides explicitly.
    {
        const char* preload = getenv("LD_PRELOAD");
        const bool profiled = (preload && strstr(preload, "rocprofiler")) || getenv("ROCPROFILER_REGISTER_LIBRARY") ||
                              getenv("ROCP_TOOL_LIBRARIES") || getenv("ROCPROF_OUTPUT_PATH");
        p->opt_cooperative = profiled ? 0 : 1;
        if (const char* v = getenv("FLASHLSTM_COOPERATIVE_LAUNCH")) p->opt_cooperative = atoi(v) != 0;
        if (const char* v = getenv("FLASHLSTM_STEP_GRAPHS")) p->opt_graphs = atoi(v) != 0;
        if (const char* v = getenv("FLASHLSTM_BWD_TWO_D")) { p->opt_two_d = atoi(v) < 0 ? 0 : (atoi(v) > 2 ? 2 : atoi(v)); p->two_d_explicit = true; }
        if (const char* v = getenv("FLASHLSTM_WAVES_FWD")) p->opt_waves_f = (atoi(v) == 4 || atoi(v) == 8) ? atoi(v) : 0;
    }
    replan(p);
    e = p->status.reserve(64);
    if (e == hipSuccess) e = hipMemset(p->status.p, 0, 64);
    if (e == hipSuccess) e = hipHostMalloc(reinterpret_cast<void**>(&p->status_host), 64, hipHostMallocDefault);
    if (e == hipSuccess) p->status_host[0] = 0;
    if (e == hipSuccess) e = p->tm.init();
    if (e != hipSuccess) { flstm_core_destroy(p); return int(e); }
    *out = p;
    return 0;
}

extern "C" int flstm_core_destroy(flstm_core_plan* p) {
    if (!p) return FLSTM_E_INVALID;
    for (DevBuf* b : {&p->wih_p, &p->wih_t, &p->wfrag_f, &p->wfrag_b, &p->wfrag_b2, &p->part_b, &p->bias_p, &p->X16, &p->G, &p->Y, &p->C,
                      &p->status, &p->xch_f, &p->xch_b, &p->dYp, &p->dG, &p->dHn, &p->dC,
                      &p->dH0, &p->db_part, &p->dw_part, &p->prof})
        b->release();
    p->tm.destroy();
    if (p->status_host) (void)hipHostFree(p->status_host);
    delete p;
    return 0;
}

extern "C" int flstm_core_set_option(flstm_core_plan* p, const char* name, long value) {
    if (!p || !name) return FLSTM_E_INVALID;
    if (!strcmp(name, "stepwise")) { p->opt_stepwise = value != 0; replan(p); return 0; }
    if (!strcmp(name, "proj_chunk")) { p->opt_proj_chunk = int(value); return 0; }
    if (!strcmp(name, "spin_limit")) { if (value < 0) return FLSTM_E_INVALID; p->opt_spin_limit = int(value); return 0; }
    if (!strcmp(name, "spin_ms")) { if (value < 1 || value > 60000) return FLSTM_E_INVALID; p->opt_spin_ms = int(value); return 0; }
    if (!strcmp(name, "profile")) {
        p->opt_profile = value != 0;
        if (p->opt_profile) {
            FL_TRY(p->prof.reserve(16 * sizeof(long long)));
        }
        return 0;
    }
    if (!strcmp(name, "row_tiles_fwd") || !strcmp(name, "row_tiles_bwd")) {
        if (value < 0 || value > 2) return FLSTM_E_INVALID;
        (name[10] == 'f' ? p->opt_mt_f : p->opt_mt_b) = int(value);
        replan(p);
        return 0;
    }
    if (!strcmp(name, "clear_tuned")) { p->tuned.clear(); use_tuned(p, 1); return 0; }
    if (!strcmp(name, "cooperative")) { p->opt_cooperative = value != 0; replan(p); return 0; }
    if (!strcmp(name, "step_graphs")) { p->opt_graphs = value != 0; return 0; }
    if (!strcmp(name, "bwd_two_d")) { if (value < 0 || value > 2) return FLSTM_E_INVALID; p->opt_two_d = int(value); p->two_d_explicit = true; replan(p); return 0; }
    if (!strcmp(name, "waves_fwd")) {
        // wavefronts per workgroup of the forward recurrence: the weight fragments are packed for it, so a change
        // un-packs them
        if (value != 0 && value != 4 && value != 8) return FLSTM_E_INVALID;
        const int before = p->Lf.nw;
        p->opt_waves_f = int(value);
        replan(p);
        if (p->Lf.nw != before) p->weights_packed = false;
        return 0;
    }
    if (!strcmp(name, "inject_stall")) { if (value < 0) return FLSTM_E_INVALID; p->inject_stall = int(value); return 0; }
    if (!strcmp(name, "dw_splits")) { if (value < 0) return FLSTM_E_INVALID; p->opt_dw_splits = int(value); return 0; }
    if (!strcmp(name, "accumulate_grads")) { p->opt_accumulate = value != 0; return 0; }
    return FLSTM_E_INVALID;
}

extern "C" long flstm_core_get_info(const flstm_core_plan* p, const char* name) {
    if (!p || !name) return -1;
    if (!strcmp(name, "persistent_fwd")) return p->Lf.persistent;
    if (!strcmp(name, "persistent_bwd")) return p->Lb.persistent;
    if (!strcmp(name, "xcd_local_fwd")) return p->Lf.xcd_local;
    if (!strcmp(name, "xcd_local_bwd")) return p->Lb.xcd_local;
    if (!strcmp(name, "resident_fwd")) return p->Lf.resident;
    if (!strcmp(name, "resident_bwd")) return p->Lb.resident;
    if (!strcmp(name, "row_tiles")) return p->Lf.mt;
    if (!strcmp(name, "row_tiles_fwd")) return p->Lf.mt;
    if (!strcmp(name, "row_tiles_bwd")) return p->Lb.mt;
    if (!strcmp(name, "cooperative")) return p->opt_cooperative;
    if (!strcmp(name, "bwd_two_d")) return p->Lb.two_d;
    if (!strcmp(name, "waves_fwd")) return p->Lf.nw;
    if (!strcmp(name, "graph_captures")) return p->graphs_f.captures + p->graphs_b.captures;
    if (!strcmp(name, "graph_replays")) return p->graphs_f.replays + p->graphs_b.replays;
    if (!strcmp(name, "graphs_disabled")) return (p->graphs_f.disabled ? 1 : 0) + (p->graphs_b.disabled ? 2 : 0);
    if (!strcmp(name, "tuned_entries")) return long(p->tuned.size());
    if (!strcmp(name, "tuned_T")) return long(p->eff_T);
    if (!strcmp(name, "tuned_row_tiles_fwd")) return p->eff_mt_f;
    if (!strcmp(name, "tuned_row_tiles_bwd")) return p->eff_mt_b;
    if (!strcmp(name, "tuned_stepwise_fwd")) return p->eff_step_f;
    if (!strcmp(name, "tuned_stepwise_bwd")) return p->eff_step_b;
    if (!strcmp(name, "tuned_dw_splits")) return p->eff_dw;
    if (!strcmp(name, "tuned_bwd_two_d")) return p->eff_two_d;
    if (!strcmp(name, "device_bytes")) {
        size_t sum = 0;
        for (const DevBuf* b : {&p->wih_p, &p->wih_t, &p->wfrag_f, &p->wfrag_b, &p->wfrag_b2, &p->part_b, &p->bias_p, &p->X16, &p->G, &p->Y, &p->C,
                                &p->status, &p->xch_f, &p->xch_b, &p->dYp, &p->dG, &p->dHn, &p->dC, &p->dH0, &p->db_part,
                                &p->dw_part, &p->prof})
            sum += b->bytes;
        return long(sum);
    }
    if (!strcmp(name, "slice_fwd")) return p->Lf.jb;
    if (!strcmp(name, "slice_bwd")) return p->Lb.jb;
    if (!strcmp(name, "groups_fwd")) return p->Lf.ng;
    if (!strcmp(name, "groups_bwd")) return p->Lb.ng;
    if (!strcmp(name, "fallbacks")) return p->fallbacks;
    if (!strcmp(name, "demotions_fwd")) return p->demotions_fwd;
    if (!strcmp(name, "demotions_bwd")) return p->demotions_bwd;
    if (!strcmp(name, "cooperative_refusals")) return p->coop_refusals;
    if (!strcmp(name, "hold_fwd")) return p->hold_fwd;
    if (!strcmp(name, "hold_bwd")) return p->hold_bwd;
    if (!strcmp(name, "static_scratch_bytes")) return long(kStaticScratchBytes);
    if (!strcmp(name, "num_cus")) return p->num_cus;
    if (!strcmp(name, "clock_khz")) return p->clock_khz;
    if (!strcmp(name, "hidden_padded")) return p->d.Hp;
    if (!strcmp(name, "input_padded")) return p->d.Ip;
    return -1;
}

extern "C" int flstm_core_pack_weights(flstm_core_plan* p, const float* w_ih, const float* w_hh, void* stream) {
    if (!p || !w_ih || !w_hh) return FLSTM_E_INVALID;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Dims& d = p->d;
    FL_TRY(p->wih_p.reserve(size_t(4) * d.Hp * d.Ip * sizeof(half_t)));
    FL_TRY(p->wih_t.reserve(size_t(4) * d.Hp * d.Ip * sizeof(half_t)));
    FL_TRY(p->wfrag_f.reserve(size_t(p->Lf.nh) * p->Lf.nw * p->ks_f * p->Lf.nt * kWave * sizeof(half8)));
    FL_TRY(p->wfrag_b.reserve(size_t(p->Lb.nh) * p->Lb.nw * p->ks_b * p->Lb.nt * kWave * sizeof(half8)));
    FL_TRY(pack_weights(d, w_ih, w_hh, p->wih_p.as<half_t>(), p->wih_t.as<half_t>(), p->wfrag_f.as<half8>(),
                        p->ks_f, p->Lf.nt, p->Lf.rot_div, p->Lf.nw, p->wfrag_b.as<half8>(), p->ks_b, p->Lb.nt,
                        p->Lb.rot_div, p->Lb.nw, s));
    if (rec_bwd_two_d_possible(d.Hp, p->num_cus)) {   // whether or not the current layout uses them
        FL_TRY(p->wfrag_b2.reserve(rec_bwd_two_d_wfrag_bytes(d.Hp)));
        FL_TRY(pack_wfrag_bwd2d(d, w_hh, p->wfrag_b2.as<half8>(), rec_bwd_two_d_kq(d.B, d.Hp), s));
    }
    FL_TRY(hipStreamSynchronize(s));
    p->weights_packed = true;
    return 0;
}

extern "C" int flstm_core_pack_bias(flstm_core_plan* p, const float* b_ih, const float* b_hh, void* stream) {
    if (!p) return FLSTM_E_INVALID;
    hipStream_t s = static_cast<hipStream_t>(stream);
    FL_TRY(p->bias_p.reserve(size_t(4) * p->d.Hp * sizeof(float)));
    if (!b_ih || !b_hh) {
        // zeros for a missing vector: pack against a zeroed scratch vector
        FL_TRY(p->db_part.reserve(size_t(4) * p->d.Hp * sizeof(float)));
        FL_TRY(fill_zero(p->db_part.p, size_t(4) * p->d.Hp * sizeof(float), s));
        const float* z = p->db_part.as<float>();
        FL_TRY(pack_bias(p->d, b_ih ? b_ih : z, b_hh ? b_hh : z, p->bias_p.as<float>(), s));
    } else {
        FL_TRY(pack_bias(p->d, b_ih, b_hh, p->bias_p.as<float>(), s));
    }
    p->bias_packed = true;
    return 0;
}

namespace {

// Forward pass in three parts so that a caller can feed it in ranges of steps: setup (state rows, exchange
// ring), any number of step ranges in order (x rows -> projection -> recurrence), and the status check.
int forward_setup(flstm_core_plan* p, size_t T, const void* x, flstm_dtype x_dtype, const void* h0,
                  const void* c0, flstm_dtype state_dtype, hipStream_t s) {
    const Dims& d = p->d;
    const size_t TB = T * size_t(d.B);
    p->fw.T = T; p->fw.x = x; p->fw.x_dtype = x_dtype; p->fw.open = true;
    if (!(x_dtype == FLSTM_F16 && d.I == d.Ip)) FL_TRY(p->X16.reserve(TB * d.Ip * sizeof(half_t)));
    FL_TRY(p->G.reserve(TB * 4 * d.Hp * sizeof(half_t)));
    FL_TRY(p->Y.reserve((TB + d.B) * d.Hp * sizeof(half_t)));
    FL_TRY(p->C.reserve((TB + d.B) * d.Hp * sizeof(float)));
    const size_t xslot = exchange_slot_halfs(d.B, d.Hp);
    FL_TRY(p->xch_f.reserve(4 * xslot * sizeof(half_t)));
    // One launch: the initial state rows (a null h0 / c0 reads as zeros), the exchange ring -- slot 0 zero (h0 goes in
    // below; rows past B stay zero), slots 1 to 3 the 'unwritten' pattern --, the seat counters and the phase counters.
    PrepList prep;
    prep.to_half(h0, state_dtype == FLSTM_F32, size_t(d.B), d.H, size_t(d.H), 1.f, p->Y.as<half_t>(), size_t(d.B), size_t(d.Hp));
    prep.to_float(c0, state_dtype == FLSTM_F32, size_t(d.B), d.H, 1.f, p->C.as<float>(), size_t(d.Hp));
    prep.fill(p->xch_f.p, xslot * sizeof(half_t), 0u);
    prep.fill(p->xch_f.as<half_t>() + xslot, 3 * xslot * sizeof(half_t), 0xFFFFFFFFu);
    prep.fill(p->status.as<unsigned>() + 8, 8 * sizeof(unsigned), 0u);
    if (p->opt_profile) prep.fill(p->prof.p, 8 * sizeof(long long), 0u);
    FL_TRY(run_prep(prep, s));
    p->fw.seats_clean = true;
    FL_TRY(to_exchange_layout(p->Y.as<half_t>(), d.B, d.Hp, size_t(d.Hp), p->xch_f.as<half_t>(), s));
    return 0;
}

// x rows of steps [t0, t0+n) -> fp16 operand -> x-projection (+ bias) in G
int forward_project(flstm_core_plan* p, size_t t0, size_t n, hipStream_t s) {
    const Dims& d = p->d;
    const half_t* A = nullptr;   // first row of step t0
    size_t lda = 0;
    if (p->fw.x_dtype == FLSTM_F16 && d.I == d.Ip) {
        A = static_cast<const half_t*>(p->fw.x) + t0 * d.B * d.I;
        lda = size_t(d.I);
    } else {
        const size_t esz = p->fw.x_dtype == FLSTM_F32 ? 4 : 2;
        const char* src = static_cast<const char*>(p->fw.x) + t0 * d.B * d.I * esz;
        half_t* dst = p->X16.as<half_t>() + t0 * d.B * d.Ip;
        FL_TRY(convert_pad(src, p->fw.x_dtype == FLSTM_F32, n * d.B, d.I, size_t(d.I), 1.f, dst, n * d.B, size_t(d.Ip), s));
        A = dst;
        lda = size_t(d.Ip);
    }
    // hoisted input projection, optionally in chunks of time steps
    size_t chunk_steps = (p->opt_proj_chunk <= 0 || size_t(p->opt_proj_chunk) > n) ? n : size_t(p->opt_proj_chunk);
    for (size_t c0 = 0; c0 < n; c0 += chunk_steps) {
        const size_t steps = (c0 + chunk_steps <= n) ? chunk_steps : n - c0;
        GemmNT g{};
        g.A = A + c0 * d.B * lda; g.lda = lda;
        g.B = p->wih_p.as<half_t>(); g.ldb = size_t(d.Ip);
        g.M = int(steps * d.B); g.N = 4 * d.Hp; g.K = d.Ip;
        g.C16 = p->G.as<half_t>() + (t0 + c0) * d.B * 4 * d.Hp; g.C32 = nullptr; g.ldc = size_t(4) * d.Hp;
        g.alpha = 1.f; g.splits = 1; g.split_stride = 0;
        g.bias = p->bias_p.as<float>();   // b_ih + b_hh, packed gate order: the recurrence reads x-projection + bias
        FL_TRY(launch_gemm_nt(g, s));
    }
    return 0;
}

int forward_recur(flstm_core_plan* p, size_t t0, size_t n, hipStream_t s) {
    const Dims& d = p->d;
    RecFwdArgs a{};
    a.wfrag = p->wfrag_f.as<half8>();
    a.Y = p->Y.as<half_t>(); a.G = p->G.as<half_t>(); a.C = p->C.as<float>();
    a.y_out = p->fw.y_direct;
    a.X = p->xch_f.as<half_t>(); a.x_slot = exchange_slot_halfs(d.B, d.Hp);
    a.status = p->status.as<int>();
    a.seats = p->status.as<unsigned>() + 8;
    a.delay_hint = p->status.as<int>() + 1;   // (the status block: word 0 status, 1 / 2 delay hints, 8..15 seats)
    if (!p->fw.seats_clean) FL_TRY(fill_zero(a.seats, 8 * sizeof(unsigned), s));
    p->fw.seats_clean = false;
    a.B = d.B; a.Hp = d.Hp; a.T = int(p->fw.T); a.t0 = int(t0); a.t1 = int(t0 + n);
    a.spin_limit = p->opt_spin_limit;
    a.spin_ticks = (long long)p->opt_spin_ms * p->wall_khz;
    a.prof = p->opt_profile ? p->prof.as<long long>() : nullptr;
    // Step-wise launches are replayed from a captured graph only for whole passes: a sequence fed in ranges has a new
    // range (a new graph) every call, each used once.  Never inside flstm_core_forward_static (a capture allocates).
    const bool whole = (t0 == 0 && n == p->fw.T);
    hipError_t e = launch_rec_fwd(p->Lf, a, s, (p->opt_graphs && whole && !p->static_call) ? &p->graphs_f : nullptr);
    if (e == hipErrorCooperativeLaunchTooLarge && p->Lf.persistent) {
        // the grid cannot be co-resident: this direction runs step-wise from now on, starting with these steps
        p->refused_fwd = true;
        p->coop_refusals++;
        replan(p);
        e = launch_rec_fwd(p->Lf, a, s, nullptr);
    }
    FL_TRY(e);
    return 0;
}

int forward_once(flstm_core_plan* p, size_t T, const void* x, flstm_dtype x_dtype, const void* h0,
                 const void* c0, flstm_dtype state_dtype, hipStream_t s) {
    int rc = forward_setup(p, T, x, x_dtype, h0, c0, state_dtype, s);
    if (rc) return rc;
    FL_TRY(hipEventRecord(p->tm.ev[0], s));
    rc = forward_project(p, 0, T, s);
    if (rc) return rc;
    FL_TRY(hipEventRecord(p->tm.ev[1], s));
    rc = forward_recur(p, 0, T, s);
    if (rc) return rc;
    FL_TRY(hipEventRecord(p->tm.ev[2], s));
    return 0;
}

// One whole forward pass: projection, recurrence, outputs, one wait, status.  The outputs are written behind the
// recurrence without waiting for its status: if the persistent launch gave up, the whole pass is repeated
// step-wise and overwrites them.
int forward_pass(flstm_core_plan* p, size_t T, const void* x, flstm_dtype x_dtype, const void* h0, const void* c0,
                 flstm_dtype state_dtype, void* y, flstm_dtype y_dtype, void* hy, void* cy,
                 flstm_dtype out_state_dtype, hipStream_t s) {
    const Dims& d = p->d;
    const size_t TB = T * size_t(d.B);
    use_tuned(p, T);
    for (int attempt = 0;; ++attempt) {
        // An fp16 output whose rows are the state rows is written by the persistent recurrence itself (no copy
        // afterwards).  Step-wise launches leave it to the copy: every argument of theirs is then plan-owned, and
        // the graph they were captured into can be replayed on the next pass.
        half_t* const y_direct =
            (y && y_dtype == FLSTM_F16 && d.H == d.Hp && p->Lf.persistent) ? static_cast<half_t*>(y) : nullptr;
        p->fw.y_direct = y_direct;
        int rc = forward_once(p, T, x, x_dtype, h0, c0, state_dtype, s);
        p->fw.y_direct = nullptr;
        if (rc) return rc;
        if (!y_direct)
            FL_TRY(unpad_from_half(p->Y.as<half_t>() + size_t(d.B) * d.Hp, size_t(d.Hp), TB, d.H, y, y_dtype == FLSTM_F32, s));
        PrepList out;   // final states, one launch
        out.unpad(p->Y.as<half_t>() + TB * d.Hp, 0, size_t(d.Hp), size_t(d.B), d.H, 1.f, hy, out_state_dtype == FLSTM_F32);
        out.unpad(p->C.as<float>() + TB * d.Hp, 1, size_t(d.Hp), size_t(d.B), d.H, 1.f, cy, out_state_dtype == FLSTM_F32);
        FL_TRY(run_prep(out, s));
        int st = 0;
        rc = wait_status(p, true, s, &st);
        if (rc) return rc;
        if (st == 0) break;
        if (!p->Lf.persistent || attempt > 0) return FLSTM_E_STALLED;
        demote(p, true);   // workgroups not co-resident or not where expected: redo with one launch per step
    }
    pass_done(p, true);
    if (p->opt_profile) FL_TRY(hipMemcpy(p->prof_f, p->prof.p, sizeof(p->prof_f), hipMemcpyDeviceToHost));
    p->ms_fwd[0] = elapsed(p->tm.ev[0], p->tm.ev[1]);
    p->ms_fwd[1] = elapsed(p->tm.ev[1], p->tm.ev[2]);
    p->ms_fwd[2] = elapsed(p->tm.ev[0], p->tm.ev[2]);
    p->fw.open = false;
    return 0;
}

}  // namespace

extern "C" int flstm_core_forward(flstm_core_plan* p, size_t T, const void* x, flstm_dtype x_dtype,
                                  const void* h0, const void* c0, flstm_dtype state_dtype, void* y,
                                  flstm_dtype y_dtype, void* hy, void* cy, flstm_dtype out_state_dtype,
                                  int save_for_backward, void* stream) {
    if (!p) return FLSTM_E_INVALID;
    if (!p->weights_packed || !p->bias_packed) return FLSTM_E_NOT_PACKED;
    if (T == 0) return 0;
    if (!x || T > (size_t(1) << 24)) return FLSTM_E_INVALID;
    p->have_cache = false;
    int rc = forward_pass(p, T, x, x_dtype, h0, c0, state_dtype, y, y_dtype, hy, cy, out_state_dtype,
                          static_cast<hipStream_t>(stream));
    p->fw.open = false;   // (also when the pass failed: no range of steps may follow it)
    if (rc) return rc;
    if (save_for_backward) { p->have_cache = true; p->T_cache = T; }
    return 0;
}

namespace {

size_t align256(size_t v) { return (v + 255) / 256 * 256; }

}  // namespace

extern "C" int flstm_core_forward_static(flstm_core_plan* p, size_t T, const void* x, flstm_dtype x_dtype,
                                         const void* h0, const void* c0, flstm_dtype state_dtype, void* y,
                                         flstm_dtype y_dtype, void* hy, void* cy, flstm_dtype out_state_dtype,
                                         void* stream) {
    if (!p) return FLSTM_E_INVALID;
    if (!p->weights_packed || !p->bias_packed) return FLSTM_E_NOT_PACKED;
    if (T == 0) return 0;
    if (!x || T > (size_t(1) << 24) || p->fw.open || p->bw.open) return FLSTM_E_INVALID;
    int dev = -1;
    FL_TRY(hipGetDevice(&dev));
    if (dev != p->device) return FLSTM_E_INVALID;
    void* base = nullptr;
    int rc = static_scratch(dev, &base);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Dims& d = p->d;
    const size_t TB = T * size_t(d.B);
    // the same buffers forward_setup() sizes, carved out of the static array instead of allocated
    const bool x_in_place = (x_dtype == FLSTM_F16 && d.I == d.Ip);
    const size_t need[6] = {256,
                            x_in_place ? 0 : TB * d.Ip * sizeof(half_t),
                            TB * 4 * d.Hp * sizeof(half_t),
                            (TB + d.B) * d.Hp * sizeof(half_t),
                            (TB + d.B) * d.Hp * sizeof(float),
                            4 * exchange_slot_halfs(d.B, d.Hp) * sizeof(half_t)};
    size_t off[6], total = 0;
    for (int i = 0; i < 6; ++i) { off[i] = total; total += align256(need[i]); }
    if (total > kStaticScratchBytes) return FLSTM_E_TOO_LARGE;
    char* b = static_cast<char*>(base);
    DevBuf* slot[6] = {&p->status, &p->X16, &p->G, &p->Y, &p->C, &p->xch_f};
    DevBuf saved[6];
    for (int i = 0; i < 6; ++i) { saved[i] = *slot[i]; *slot[i] = DevBuf::view(b + off[i], need[i]); }
    const bool had_cache = p->have_cache;
    p->have_cache = false;   // (the plan's own caches are untouched, but no pass may use the borrowed ones later)
    // status word and seat counters start at zero; the array keeps whatever the last call left
    rc = int(fill_zero(p->status.p, 64, s));
    p->static_call = true;   // (step-wise launches, if the pass comes to them, are plain launches: a graph capture allocates)
    if (rc == 0)
        rc = forward_pass(p, T, x, x_dtype, h0, c0, state_dtype, y, y_dtype, hy, cy, out_state_dtype, s);
    p->static_call = false;
    p->fw.open = false;   // (also when the pass failed: the next call must not find a pass in progress)
    for (int i = 0; i < 6; ++i) *slot[i] = saved[i];
    p->have_cache = had_cache;
    return rc;
}

namespace {

// Backward recurrence in parts, like the forward pass: setup, step ranges from the end of the sequence towards
// its start (dY rows -> BPTT steps -> dX rows), and the weight-gradient GEMMs over the whole sequence.
int backward_setup(flstm_core_plan* p, size_t T, const void* dY, flstm_dtype dy_dtype, const void* d_hn,
                   const void* d_cn, flstm_dtype dstate_dtype, float S, void* dx, flstm_dtype dx_dtype,
                   hipStream_t s) {
    const Dims& d = p->d;
    const size_t TB = T * size_t(d.B);
    p->bw.T = T; p->bw.dY = dY; p->bw.dy_dtype = dy_dtype; p->bw.S = S; p->bw.dx = dx; p->bw.dx_dtype = dx_dtype;
    p->bw.open = true;
    // (step-wise launches always read a plan-owned copy, so that their captured graph can be replayed)
    if (dy_dtype == FLSTM_F16 && d.H == d.Hp && p->Lb.persistent) {
        p->bw.dYk = static_cast<const half_t*>(dY);
        p->bw.dy_scale = S;
    } else {
        FL_TRY(p->dYp.reserve(TB * d.Hp * sizeof(half_t)));
        p->bw.dYk = p->dYp.as<half_t>();
        p->bw.dy_scale = 1.f;   // the scale is applied while the rows are converted
    }
    const size_t st_bytes = size_t(d.B) * d.Hp * sizeof(float);
    FL_TRY(p->dHn.reserve(st_bytes));
    FL_TRY(p->dC.reserve(st_bytes));
    FL_TRY(p->dH0.reserve(st_bytes));
    FL_TRY(p->dG.reserve(TB * 4 * d.Hp * sizeof(half_t)));
    FL_TRY(p->db_part.reserve(size_t(p->Lb.ng) * 4 * d.Hp * sizeof(float)));
    const size_t xslot = exchange_slot_halfs(rec_bwd_ring_rows(p->Lb, d.B), 4 * d.Hp);
    const size_t dg_slots = size_t(rec_bwd_dg_slots(p->Lb));
    FL_TRY(p->xch_b.reserve(dg_slots * xslot * sizeof(half_t)));
    // One launch (see forward_setup): the dG ring 'unwritten', the ring of partial sums in its starting parities, the
    // scaled state gradients, the bias-gradient partials, the seat counters, the phase counters.
    static_assert(kRecBwdPartSlots + 6 <= 10, "PrepList holds ten operations");
    PrepList prep;
    prep.fill(p->xch_b.p, dg_slots * xslot * sizeof(half_t), 0xFFFFFFFFu);
    if (p->Lb.two_d) {
        const size_t pslot = rec_bwd_part_slot_floats(p->Lb) * sizeof(float);
        FL_TRY(p->part_b.reserve(kRecBwdPartSlots * pslot));
        for (int k = 0; k < kRecBwdPartSlots; ++k)
            prep.fill(static_cast<char*>(p->part_b.p) + size_t(k) * pslot, pslot, rec_bwd_part_fill(k, int(T)));
    }
    prep.to_float(d_hn, dstate_dtype == FLSTM_F32, size_t(d.B), d.H, S, p->dHn.as<float>(), size_t(d.Hp));
    prep.to_float(d_cn, dstate_dtype == FLSTM_F32, size_t(d.B), d.H, S, p->dC.as<float>(), size_t(d.Hp));
    prep.fill(p->db_part.p, size_t(p->Lb.ng) * 4 * d.Hp * sizeof(float), 0u);
    prep.fill(p->status.as<unsigned>() + 8, 8 * sizeof(unsigned), 0u);
    if (p->opt_profile) prep.fill(p->prof.as<long long>() + 8, 8 * sizeof(long long), 0u);
    FL_TRY(run_prep(prep, s));
    p->bw.seats_clean = true;
    return 0;
}

// steps t_hi .. t_lo (t_lo = -1 includes the closing dh0 product); dY rows of these steps are converted first
// when the caller's dY cannot be used in place
int backward_recur(flstm_core_plan* p, long t_hi, long t_lo, hipStream_t s) {
    const Dims& d = p->d;
    const long lo = t_lo < 0 ? 0 : t_lo;
    if (p->bw.dYk != p->bw.dY && t_hi >= lo) {
        const size_t esz = p->bw.dy_dtype == FLSTM_F32 ? 4 : 2;
        const size_t rows = size_t(t_hi - lo + 1) * d.B;
        const char* src = static_cast<const char*>(p->bw.dY) + size_t(lo) * d.B * d.H * esz;
        half_t* dst = p->dYp.as<half_t>() + size_t(lo) * d.B * d.Hp;
        FL_TRY(convert_pad(src, p->bw.dy_dtype == FLSTM_F32, rows, d.H, size_t(d.H), p->bw.S, dst, rows, size_t(d.Hp), s));
    }
    RecBwdArgs a{};
    a.wfrag = p->wfrag_b.as<half8>();
    a.G = p->G.as<half_t>(); a.C = p->C.as<float>(); a.dY = p->bw.dYk; a.dG = p->dG.as<half_t>();
    a.dHn = p->dHn.as<float>(); a.dC = p->dC.as<float>(); a.dH0 = p->dH0.as<float>();
    a.X = p->xch_b.as<half_t>(); a.x_slot = exchange_slot_halfs(rec_bwd_ring_rows(p->Lb, d.B), 4 * d.Hp);
    if (p->Lb.two_d) {
        a.wfrag2 = p->wfrag_b2.as<half8>();
        a.P = p->part_b.as<float>();
        a.p_slot = rec_bwd_part_slot_floats(p->Lb);
    }
    a.db_part = p->db_part.as<float>();
    a.status = p->status.as<int>();
    a.seats = p->status.as<unsigned>() + 8;
    a.delay_hint = p->status.as<int>() + 2;
    a.B = d.B; a.Hp = d.Hp; a.T = int(p->bw.T); a.dy_scale = p->bw.dy_scale;
    a.t_hi = int(t_hi); a.t_lo = int(t_lo);
    a.spin_limit = p->opt_spin_limit;
    a.spin_ticks = (long long)p->opt_spin_ms * p->wall_khz;
    a.prof = p->opt_profile ? p->prof.as<long long>() + 8 : nullptr;
    // One launch, or one per window of batch rows (RecLayout::win_rows).  The windows share the ring of partial sums,
    // so every launch of a windowed pass starts from a ring prepared for ITS first product step (a single window's
    // launches continue each other's parities instead).
    const int win = (p->Lb.two_d && p->Lb.win_rows) ? p->Lb.win_rows : d.B;
    for (int b_lo = 0; b_lo < d.B; b_lo += win) {
        a.b_lo = b_lo;
        a.b_hi = b_lo + win < d.B ? b_lo + win : d.B;
        if (!p->bw.seats_clean) FL_TRY(fill_zero(a.seats, 8 * sizeof(unsigned), s));
        p->bw.seats_clean = false;
        if (win < d.B) {
            const size_t pslot = a.p_slot * sizeof(float);
            const int first_T = t_hi >= long(p->bw.T) - 1 ? int(p->bw.T) : int(t_hi) + 2;   // (its first product step is first_T - 2)
            for (int k = 0; k < kRecBwdPartSlots; ++k)
                FL_TRY(fill_words(static_cast<char*>(p->part_b.p) + size_t(k) * pslot, pslot, rec_bwd_part_fill(k, first_T), s));
        }
        const bool whole = (t_hi == long(p->bw.T) - 1 && t_lo == -1);   // (graphs for whole passes only: see forward_recur)
        hipError_t e = launch_rec_bwd(p->Lb, a, s, (p->opt_graphs && whole) ? &p->graphs_b : nullptr);
        if (e == hipErrorCooperativeLaunchTooLarge && p->Lb.persistent) return int(e);   // (handled by the caller: the layout changes)
        FL_TRY(e);
    }
    return 0;
}

// dX rows of steps [t_lo, t_hi] = dG * W_ih  (contraction over the packed gate columns)
int backward_dx(flstm_core_plan* p, long t_hi, long t_lo, hipStream_t s) {
    const Dims& d = p->d;
    if (!p->bw.dx || t_hi < t_lo) return 0;
    const size_t row0 = size_t(t_lo) * d.B, rows = size_t(t_hi - t_lo + 1) * d.B;
    GemmNT g{};
    g.A = p->dG.as<half_t>() + row0 * 4 * d.Hp; g.lda = size_t(4) * d.Hp;
    g.B = p->wih_t.as<half_t>(); g.ldb = size_t(4) * d.Hp;
    g.M = int(rows); g.N = d.I; g.K = 4 * d.Hp;
    if (p->bw.dx_dtype == FLSTM_F32) g.C32 = static_cast<float*>(p->bw.dx) + row0 * d.I;
    else g.C16 = static_cast<half_t*>(p->bw.dx) + row0 * d.I;
    g.ldc = size_t(d.I); g.alpha = 1.f / p->bw.S; g.splits = 1; g.split_stride = 0;
    FL_TRY(launch_gemm_nt(g, s));
    return 0;
}

int backward_rec_once(flstm_core_plan* p, size_t T, const void* dY, flstm_dtype dy_dtype, const void* d_hn,
                      const void* d_cn, flstm_dtype dstate_dtype, float S, void* dx, flstm_dtype dx_dtype,
                      hipStream_t s) {
    int rc = backward_setup(p, T, dY, dy_dtype, d_hn, d_cn, dstate_dtype, S, dx, dx_dtype, s);
    if (rc) return rc;
    FL_TRY(hipEventRecord(p->tm.ev[3], s));
    rc = backward_recur(p, long(T) - 1, -1, s);
    if (rc) return rc;
    FL_TRY(hipEventRecord(p->tm.ev[4], s));
    return 0;
}

// dW_ih = dG^T * X and dW_hh = dG^T * H_prev over the whole sequence, bias gradient and state gradients
int backward_finish(flstm_core_plan* p, const void* x, flstm_dtype x_dtype, float* dW_ih, float* dW_hh,
                    float* db_ih, float* db_hh, float* dh0, float* dc0, hipStream_t s) {
    const Dims& d = p->d;
    const size_t TB = p->bw.T * size_t(d.B);
    const float invS = 1.f / p->bw.S;
    // k-major operands exactly as the recurrence left them (H_prev of step t is row block t of the state array,
    // row block 0 = h0), split over K, fp32 partials.  Both gradients come out of ONE launch, dG^T * [X | H_prev]:
    // dG (the large operand) is read once, and the tiles of both products fill the machine together.
    const bool direct = (x_dtype == FLSTM_F16 && d.I == d.Ip);
    const half_t* Xop = direct ? static_cast<const half_t*>(x) : p->X16.as<half_t>();
    const half_t* Hop = p->Y.as<half_t>();
    const int n_ih = dW_ih ? d.Ip : 0, n_hh = dW_hh ? d.Hp : 0, ncols = n_ih + n_hh;
    if (ncols > 0) {
        // automatic: what the kernel's own schedule makes fastest (gemm_tn_auto_splits), at least four 64-row slabs
        // per split
        int want = p->opt_dw_splits > 0 ? p->opt_dw_splits : p->eff_dw;
        if (want <= 0) {
            const size_t cap = TB / 256 < 64 ? TB / 256 : 64;
            want = gemm_tn_auto_splits(4 * d.Hp, n_ih ? n_ih : n_hh, n_ih ? n_hh : 0, int(TB), cap < 1 ? 1 : int(cap));
        }
        if (want > 64) want = 64;
        const int splits = gemm_effective_splits(int(TB), want);
        const size_t per = size_t(4) * d.Hp * ncols;
        FL_TRY(p->dw_part.reserve(per * splits * sizeof(float)));
        GemmNT g{};
        g.A = p->dG.as<half_t>(); g.lda = size_t(4) * d.Hp;
        g.M = 4 * d.Hp; g.N = ncols; g.K = int(TB);
        if (n_ih && n_hh) {
            g.B = Xop; g.ldb = size_t(d.Ip); g.N1 = n_ih;
            g.B2 = Hop; g.ldb2 = size_t(d.Hp);
        } else {
            g.B = n_ih ? Xop : Hop; g.ldb = size_t(n_ih ? d.Ip : d.Hp);
        }
        g.C16 = nullptr; g.C32 = p->dw_part.as<float>(); g.ldc = size_t(ncols);
        g.alpha = 1.f; g.splits = splits; g.split_stride = per;
        FL_TRY(launch_gemm_tn(g, s));
        FL_TRY(reduce_dw(d, p->dw_part.as<float>(), splits, size_t(ncols), 0, n_ih, d.I, invS, p->opt_accumulate != 0, dW_ih, s));
        FL_TRY(reduce_dw(d, p->dw_part.as<float>(), splits, size_t(ncols), n_ih, n_hh, d.H, invS, p->opt_accumulate != 0, dW_hh, s));
    }
    FL_TRY(hipEventRecord(p->tm.ev[6], s));
    if (db_ih || db_hh)
        FL_TRY(reduce_db(d, p->db_part.as<float>(), p->Lb.ng, invS, p->opt_accumulate != 0, db_ih, db_hh, s));
    PrepList out;   // state gradients, one launch
    out.unpad(p->dH0.as<float>(), 1, size_t(d.Hp), size_t(d.B), d.H, invS, dh0, 1);
    out.unpad(p->dC.as<float>(), 1, size_t(d.Hp), size_t(d.B), d.H, invS, dc0, 1);
    FL_TRY(run_prep(out, s));
    FL_TRY(hipEventRecord(p->tm.ev[7], s));
    int rc = enqueue_status_copy(p, s);
    if (rc) return rc;
    FL_TRY(hipStreamSynchronize(s));
    p->bw.open = false;
    return 0;
}

}  // namespace

extern "C" int flstm_core_backward(flstm_core_plan* p, size_t T, const void* x, flstm_dtype x_dtype,
                                   const void* dY, flstm_dtype dy_dtype, const void* d_hn, const void* d_cn,
                                   flstm_dtype dstate_dtype, float grad_scale, void* dx, flstm_dtype dx_dtype,
                                   float* dW_ih, float* dW_hh, float* db_ih, float* db_hh, float* dh0,
                                   float* dc0, void* stream) {
    if (!p) return FLSTM_E_INVALID;
    if (T == 0) return 0;
    if (!p->have_cache || p->T_cache != T) return FLSTM_E_NO_CACHE;
    if (!dY) return FLSTM_E_INVALID;
    if (dW_ih && !x) return FLSTM_E_INVALID;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const float S = grad_scale > 0.f ? grad_scale : 1.f;
    use_tuned(p, T);

    // dX and the weight gradients follow the recurrence without waiting for its status (one wait per pass); a
    // persistent launch that gave up is found at the end and the pass repeated step-wise over the same outputs.
    // Only when the caller's gradients are added to (accumulate_grads) the status is checked first.
    for (int attempt = 0;; ++attempt) {
        int rc = backward_rec_once(p, T, dY, dy_dtype, d_hn, d_cn, dstate_dtype, S, dx, dx_dtype, s);
        if (rc == int(hipErrorCooperativeLaunchTooLarge) && p->Lb.persistent && !p->refused_bwd) {
            // the grid cannot be co-resident: nothing was launched; this direction runs step-wise from now on
            p->refused_bwd = true;
            p->coop_refusals++;
            replan(p);
            continue;
        }
        if (rc) return rc;
        int st = 0;
        if (p->opt_accumulate) {
            rc = wait_status(p, false, s, &st);
            if (rc) return rc;
        }
        if (st == 0) {
            rc = backward_dx(p, long(T) - 1, 0, s);
            if (rc) return rc;
            FL_TRY(hipEventRecord(p->tm.ev[5], s));
            rc = backward_finish(p, x, x_dtype, dW_ih, dW_hh, db_ih, db_hh, dh0, dc0, s);
            if (rc) return rc;
            rc = take_status(p, false, s, &st);
            if (rc) return rc;
            if (st == 0) break;
        }
        if (!p->Lb.persistent || attempt > 0) return FLSTM_E_STALLED;
        demote(p, false);
    }
    pass_done(p, false);
    if (p->opt_profile)
        FL_TRY(hipMemcpy(p->prof_b, p->prof.as<long long>() + 8, sizeof(p->prof_b), hipMemcpyDeviceToHost));
    p->ms_bwd[0] = elapsed(p->tm.ev[3], p->tm.ev[4]);
    p->ms_bwd[1] = elapsed(p->tm.ev[4], p->tm.ev[5]);
    p->ms_bwd[2] = elapsed(p->tm.ev[5], p->tm.ev[6]);
    p->ms_bwd[3] = elapsed(p->tm.ev[3], p->tm.ev[7]);
    return 0;
}

// ---- the same passes fed in ranges of steps (for callers that stream the sequence through the device)

extern "C" int flstm_core_forward_begin(flstm_core_plan* p, size_t T, const void* x, flstm_dtype x_dtype,
                                        const void* h0, const void* c0, flstm_dtype state_dtype, void* stream) {
    if (!p) return FLSTM_E_INVALID;
    if (!p->weights_packed || !p->bias_packed) return FLSTM_E_NOT_PACKED;
    if (T == 0 || !x || T > (size_t(1) << 24)) return FLSTM_E_INVALID;
    p->have_cache = false;
    for (float& m : p->ms_fwd) m = -1.f;
    use_tuned(p, T);
    return forward_setup(p, T, x, x_dtype, h0, c0, state_dtype, static_cast<hipStream_t>(stream));
}

extern "C" int flstm_core_forward_steps(flstm_core_plan* p, size_t t0, size_t nsteps, void* stream) {
    if (!p || !p->fw.open || t0 + nsteps > p->fw.T) return FLSTM_E_INVALID;
    if (nsteps == 0) return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc = forward_project(p, t0, nsteps, s);
    if (rc) return rc;
    return forward_recur(p, t0, nsteps, s);
}

extern "C" int flstm_core_forward_end(flstm_core_plan* p, void* hy, void* cy, flstm_dtype out_state_dtype,
                                      int save_for_backward, void* stream) {
    if (!p || !p->fw.open) return FLSTM_E_INVALID;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Dims& d = p->d;
    const size_t TB = p->fw.T * size_t(d.B);
    p->fw.open = false;
    FL_TRY(unpad_from_half(p->Y.as<half_t>() + TB * d.Hp, size_t(d.Hp), size_t(d.B), d.H, hy,
                           out_state_dtype == FLSTM_F32, s));
    FL_TRY(unpad_from_float(p->C.as<float>() + TB * d.Hp, size_t(d.Hp), size_t(d.B), d.H, 1.f, cy,
                            out_state_dtype == FLSTM_F32, s));
    int st = 0;
    int rc = wait_status(p, true, s, &st);
    if (rc) return rc;
    if (st != 0) {   // a persistent launch gave up: the caller repeats the pass through flstm_core_forward
        if (p->Lf.persistent) demote(p, true);
        return FLSTM_E_STALLED;
    }
    pass_done(p, true);
    if (save_for_backward) { p->have_cache = true; p->T_cache = p->fw.T; }
    return 0;
}

extern "C" int flstm_core_backward_begin(flstm_core_plan* p, size_t T, const void* dY, flstm_dtype dy_dtype,
                                         const void* d_hn, const void* d_cn, flstm_dtype dstate_dtype,
                                         float grad_scale, void* dx, flstm_dtype dx_dtype, void* stream) {
    if (!p || !dY || T == 0) return FLSTM_E_INVALID;
    if (!p->have_cache || p->T_cache != T) return FLSTM_E_NO_CACHE;
    for (float& m : p->ms_bwd) m = -1.f;
    const float S = grad_scale > 0.f ? grad_scale : 1.f;
    use_tuned(p, T);
    return backward_setup(p, T, dY, dy_dtype, d_hn, d_cn, dstate_dtype, S, dx, dx_dtype, static_cast<hipStream_t>(stream));
}

extern "C" int flstm_core_backward_steps(flstm_core_plan* p, size_t t_hi, size_t nsteps, void* stream) {
    if (!p || !p->bw.open || t_hi >= p->bw.T || nsteps == 0 || nsteps > t_hi + 1) return FLSTM_E_INVALID;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const long lo = long(t_hi) - long(nsteps) + 1;
    // the range that reaches step 0 also runs the closing product for dh0
    int rc = backward_recur(p, long(t_hi), lo == 0 ? -1 : lo, s);
    if (rc == int(hipErrorCooperativeLaunchTooLarge) && p->Lb.persistent && !p->refused_bwd) {
        // the grid cannot be co-resident: step-wise from now on; the rings of this pass were laid out for the persistent
        // kernel, so the caller repeats the pass (as after a launch that gave up)
        p->refused_bwd = true;
        p->coop_refusals++;
        p->bw.open = false;
        replan(p);
        return FLSTM_E_STALLED;
    }
    if (rc) return rc;
    return backward_dx(p, long(t_hi), lo, s);
}

extern "C" int flstm_core_backward_end(flstm_core_plan* p, const void* x, flstm_dtype x_dtype, float* dW_ih,
                                       float* dW_hh, float* db_ih, float* db_hh, float* dh0, float* dc0,
                                       void* stream) {
    if (!p || !p->bw.open) return FLSTM_E_INVALID;
    if (dW_ih && !x) return FLSTM_E_INVALID;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the caller's gradients may be accumulated into: the status of the recurrence is checked before they are touched
    int st = 0;
    int rc = wait_status(p, false, s, &st);
    if (rc) return rc;
    if (st != 0) {   // the caller repeats the pass through flstm_core_backward
        p->bw.open = false;
        if (p->Lb.persistent) demote(p, false);
        return FLSTM_E_STALLED;
    }
    rc = backward_finish(p, x, x_dtype, dW_ih, dW_hh, db_ih, db_hh, dh0, dc0, s);
    if (rc) return rc;
    pass_done(p, false);
    return 0;
}

extern "C" int flstm_core_cache_ptr(const flstm_core_plan* p, int which, const void** ptr, size_t* ld) {
    if (!p || !ptr || !ld || !(p->have_cache || p->fw.open)) return FLSTM_E_INVALID;
    switch (which) {
        case 0: *ptr = p->Y.p; *ld = size_t(p->d.Hp); return 0;
        case 1: *ptr = p->C.p; *ld = size_t(p->d.Hp); return 0;
        case 2: *ptr = p->G.p; *ld = size_t(4) * p->d.Hp; return 0;
    }
    return FLSTM_E_INVALID;
}

extern "C" double flstm_core_last_ms(const flstm_core_plan* p, const char* phase) {
    if (!p || !phase) return -1.0;
    if (!strcmp(phase, "fwd_proj")) return p->ms_fwd[0];
    if (!strcmp(phase, "fwd_rec")) return p->ms_fwd[1];
    if (!strcmp(phase, "fwd_total")) return p->ms_fwd[2];
    if (!strcmp(phase, "bwd_rec")) return p->ms_bwd[0];
    if (!strcmp(phase, "bwd_dx")) return p->ms_bwd[1];
    if (!strcmp(phase, "bwd_dw")) return p->ms_bwd[2];
    if (!strcmp(phase, "bwd_total")) return p->ms_bwd[3];
    // counters of workgroup 0 (option "profile"), in milliseconds of the constant-rate clock: 0..4 wait, product, partials,
    // pointwise, publish; 6 the whole launch; 5 the launch in shader-engine clocks / the constant clock's rate, so that
    // clk5 / clk6 x that rate is the engine clock the kernel ran at
    if (!strncmp(phase, "fwd_clk", 7) && phase[7] >= '0' && phase[7] <= '7')
        return double(p->prof_f[phase[7] - '0']) / p->wall_khz;
    if (!strncmp(phase, "bwd_clk", 7) && phase[7] >= '0' && phase[7] <= '7')
        return double(p->prof_b[phase[7] - '0']) / p->wall_khz;
    return -1.0;
}

// ---- the GEMMs the passes are built from, callable on their own

extern "C" int flstm_gemm_nt(const void* A, size_t lda, const void* B, size_t ldb, size_t M, size_t N, size_t K,
                             void* C, flstm_dtype c_dtype, size_t ldc, float alpha, const float* bias, void* stream) {
    if (!A || !B || !C || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return FLSTM_E_INVALID;
    GemmNT g{};
    g.A = static_cast<const half_t*>(A); g.lda = lda;
    g.B = static_cast<const half_t*>(B); g.ldb = ldb;
    g.M = int(M); g.N = int(N); g.K = int(K);
    if (c_dtype == FLSTM_F32) g.C32 = static_cast<float*>(C);
    else g.C16 = static_cast<half_t*>(C);
    g.ldc = ldc; g.alpha = alpha; g.splits = 1; g.split_stride = 0; g.bias = bias;
    if (lda < K || ldb < K || ldc < N) return FLSTM_E_INVALID;
    FL_TRY(launch_gemm_nt(g, static_cast<hipStream_t>(stream)));
    return 0;
}

extern "C" size_t flstm_gemm_tn_workspace_bytes(size_t M, size_t N, size_t K, int splits) {
    if (splits <= 1 || K == 0 || K > (1u << 30)) return 0;
    const int eff = gemm_effective_splits(int(K), splits);
    return eff <= 1 ? 0 : size_t(eff) * M * N * sizeof(float);
}

extern "C" int flstm_gemm_tn_auto_splits(size_t M, size_t N, size_t K, int max_splits) {
    if (M == 0 || N == 0 || K == 0 || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return 1;
    return gemm_tn_auto_splits(int(M), int(N), 0, int(K), max_splits < 1 ? 1 : (max_splits > 64 ? 64 : max_splits));
}

extern "C" int flstm_gemm_tn(const void* A, size_t lda, const void* B, size_t ldb, size_t M, size_t N, size_t K,
                             float* C, size_t ldc, float alpha, int splits, void* workspace, void* stream) {
    if (!A || !B || !C || M > (1u << 30) || N > (1u << 30) || K > (1u << 30)) return FLSTM_E_INVALID;
    if (lda < M || ldb < N || ldc < N) return FLSTM_E_INVALID;
    if (M == 0 || N == 0 || K == 0) return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int eff = gemm_effective_splits(int(K), splits < 1 ? 1 : splits);
    GemmNT g{};
    g.A = static_cast<const half_t*>(A); g.lda = lda;
    g.B = static_cast<const half_t*>(B); g.ldb = ldb;
    g.M = int(M); g.N = int(N); g.K = int(K);
    g.alpha = alpha; g.bias = nullptr;
    if (eff <= 1) {
        g.C32 = C; g.ldc = ldc; g.splits = 1; g.split_stride = 0;
        FL_TRY(launch_gemm_tn(g, s));
        return 0;
    }
    if (!workspace) return FLSTM_E_INVALID;
    g.C32 = static_cast<float*>(workspace); g.ldc = N; g.splits = eff; g.split_stride = M * N;
    FL_TRY(launch_gemm_tn(g, s));
    FL_TRY(reduce_partials(static_cast<const float*>(workspace), eff, M * N, int(M), int(N), ldc, C, s));
    return 0;
}

// ---- tuner

extern "C" int flstm_core_tune(flstm_core_plan* p, size_t T, int repeats, int try_stepwise, void* stream) {
    if (!p || T == 0 || T > (size_t(1) << 24) || p->fw.open || p->bw.open) return FLSTM_E_INVALID;
    if (!p->weights_packed || !p->bias_packed) return FLSTM_E_NOT_PACKED;
    if (repeats < 1) repeats = 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Dims& d = p->d;
    const size_t TB = T * size_t(d.B);
    // synthetic inputs: varied values (the matrix cores draw more power on them than on constants, and the GEMMs run
    // about a fifth slower: candidates are compared under the clock they will run at)
    DevBuf x, dy, dwi, dwh;
    int rc = 0;
    auto fail = [&](int code) { x.release(); dy.release(); dwi.release(); dwh.release(); return code; };
    if (x.reserve(TB * d.I * sizeof(half_t)) != hipSuccess || dy.reserve(TB * d.H * sizeof(half_t)) != hipSuccess ||
        dwi.reserve(size_t(4) * d.H * d.I * sizeof(float)) != hipSuccess ||
        dwh.reserve(size_t(4) * d.H * d.H * sizeof(float)) != hipSuccess)
        return fail(int(hipErrorOutOfMemory));
    if (fill_noise(x.as<half_t>(), TB * d.I, 0x1234567u, 1.7f, s) != hipSuccess ||
        fill_noise(dy.as<half_t>(), TB * d.H, 0x89ABCDEu, 1.7f, s) != hipSuccess)
        return fail(int(hipErrorUnknown));
    // the plan's explicit options and tuned state are set aside while candidates run
    const int keep_step = p->opt_stepwise, keep_mtf = p->opt_mt_f, keep_mtb = p->opt_mt_b, keep_dw = p->opt_dw_splits,
              keep_acc = p->opt_accumulate, keep_two_d = p->opt_two_d;
    const bool keep_two_d_explicit = p->two_d_explicit;
    const bool keep_cache = p->have_cache;
    const std::vector<flstm_core_plan::Tuned> keep_tuned = p->tuned;
    p->tuned.clear();
    p->opt_accumulate = 0;
    auto restore = [&]() {
        p->opt_stepwise = keep_step; p->opt_mt_f = keep_mtf; p->opt_mt_b = keep_mtb; p->opt_dw_splits = keep_dw;
        p->opt_accumulate = keep_acc; p->opt_two_d = keep_two_d; p->two_d_explicit = keep_two_d_explicit;
        p->tuned = keep_tuned;
        p->have_cache = false;   // the caches now hold the synthetic sequence
        (void)keep_cache;
        use_tuned(p, T);
        replan(p);
    };
    flstm_core_plan::Tuned best{};
    best.T = T; best.ms_f = best.ms_b = best.ms_dw = -1.f; best.two_d = -1;
    auto run = [&](float& f_ms, float& b_ms, float& dw_ms) -> int {
        f_ms = b_ms = dw_ms = 1e30f;
        for (int r = 0; r <= repeats; ++r) {   // first pass is a warm-up
            int e = flstm_core_forward(p, T, x.p, FLSTM_F16, nullptr, nullptr, FLSTM_F16, nullptr, FLSTM_F16, nullptr, nullptr,
                                       FLSTM_F16, 1, s);
            if (e) return e;
            e = flstm_core_backward(p, T, x.p, FLSTM_F16, dy.p, FLSTM_F16, nullptr, nullptr, FLSTM_F16, 1.f, nullptr, FLSTM_F16,
                                    dwi.as<float>(), dwh.as<float>(), nullptr, nullptr, nullptr, nullptr, s);
            if (e) return e;
            if (r == 0) continue;
            if (p->ms_fwd[1] > 0 && p->ms_fwd[1] < f_ms) f_ms = p->ms_fwd[1];
            if (p->ms_bwd[0] > 0 && p->ms_bwd[0] < b_ms) b_ms = p->ms_bwd[0];
            if (p->ms_bwd[2] > 0 && p->ms_bwd[2] < dw_ms) dw_ms = p->ms_bwd[2];
        }
        return 0;
    };
    // 1) row-block height and launch mode of the two recurrences (independent of each other and of the GEMMs)
    p->opt_dw_splits = 0;
    for (int step = 0; step <= (try_stepwise ? 1 : 0); ++step) {
        for (int mt = 1; mt <= 2; ++mt) {
            p->opt_stepwise = step; p->opt_mt_f = mt; p->opt_mt_b = mt;
            replan(p);
            const bool f_is = (p->Lf.mt == mt), b_is = (p->Lb.mt == mt);   // 16-row blocks may not fit
            if (!f_is && !b_is) continue;
            float f_ms, b_ms, dw_ms;
            rc = run(f_ms, b_ms, dw_ms);
            if (rc) { restore(); return fail(rc); }
            if (f_is && (best.ms_f < 0 || f_ms < best.ms_f)) { best.ms_f = f_ms; best.mt_f = mt; best.step_f = step; }
            if (b_is && (best.ms_b < 0 || b_ms < best.ms_b)) { best.ms_b = b_ms; best.mt_b = mt; best.step_b = step; }
        }
    }
    // 1b) the layout of the backward recurrence where the two-way split can run (2048 and 1024 hidden units): off /
    // where the rule of thumb has it / wherever it fits, with the row-block height the rule picks for each
    if (rec_bwd_two_d_possible(d.Hp, p->num_cus) && !keep_two_d_explicit) {
        p->opt_stepwise = 0; p->opt_mt_f = best.mt_f; p->opt_mt_b = 0;
        p->two_d_explicit = true;
        float best_td_ms = -1.f;
        for (int td = 0; td <= 2; ++td) {
            p->opt_two_d = td;
            replan(p);
            if (!p->Lb.persistent) continue;
            if (td == 2 && !p->Lb.two_d) continue;   // (nothing new: the split does not fit this batch)
            float f_ms, b_ms, dw_ms;
            rc = run(f_ms, b_ms, dw_ms);
            if (rc) { restore(); return fail(rc); }
            if (best_td_ms < 0 || b_ms < best_td_ms) { best_td_ms = b_ms; best.two_d = td; }
        }
        // (the entry keeps the better of: the best row-block height under the plan's own setting, the best setting)
        if (best_td_ms >= 0 && best_td_ms < best.ms_b) { best.ms_b = best_td_ms; best.mt_b = 0; best.step_b = 0; }
        else best.two_d = -1;
        p->opt_two_d = keep_two_d; p->two_d_explicit = keep_two_d_explicit;
    }
    // 2) split-K count of the weight-gradient GEMM around what the schedule model picks
    p->opt_stepwise = best.step_f && best.step_b; p->opt_mt_f = best.mt_f; p->opt_mt_b = best.mt_b;
    replan(p);
    const size_t cap = TB / 256 < 64 ? TB / 256 : 64;
    const int rule = gemm_tn_auto_splits(4 * d.Hp, d.Ip, d.Hp, int(TB), cap < 1 ? 1 : int(cap));
    int last_eff = -1;
    for (int cand : {rule / 2, rule, rule + 1, rule * 2, rule * 4}) {
        if (cand < 1 || cand > 64) continue;
        const int eff = gemm_effective_splits(int(TB), cand);
        if (eff == last_eff) continue;
        last_eff = eff;
        p->opt_dw_splits = cand;
        float f_ms, b_ms, dw_ms;
        rc = run(f_ms, b_ms, dw_ms);
        if (rc) { restore(); return fail(rc); }
        if (best.ms_dw < 0 || dw_ms < best.ms_dw) { best.ms_dw = dw_ms; best.dw_splits = cand; }
    }
    restore();
    for (auto it = p->tuned.begin(); it != p->tuned.end();)
        it = (it->T == T) ? p->tuned.erase(it) : it + 1;
    p->tuned.push_back(best);
    use_tuned(p, T);
    return fail(0);
}

// A tuned entry written into / read out of a plan: what a tuning run found, kept by the caller between processes.
extern "C" int flstm_core_set_tuned(flstm_core_plan* p, size_t T, int row_tiles_fwd, int row_tiles_bwd, int stepwise_fwd,
                                    int stepwise_bwd, int dw_splits, int bwd_two_d) {
    if (!p || T == 0 || T > (size_t(1) << 24) || row_tiles_fwd < 0 || row_tiles_fwd > 2 || row_tiles_bwd < 0 ||
        row_tiles_bwd > 2 || dw_splits < 0 || dw_splits > 64 || bwd_two_d < -1 || bwd_two_d > 2)
        return FLSTM_E_INVALID;
    flstm_core_plan::Tuned t{};
    t.T = T; t.mt_f = row_tiles_fwd; t.mt_b = row_tiles_bwd; t.step_f = stepwise_fwd != 0; t.step_b = stepwise_bwd != 0;
    t.dw_splits = dw_splits; t.two_d = bwd_two_d; t.ms_f = t.ms_b = t.ms_dw = -1.f;
    for (auto it = p->tuned.begin(); it != p->tuned.end();)
        it = (it->T == T) ? p->tuned.erase(it) : it + 1;
    p->tuned.push_back(t);
    use_tuned(p, T);
    return 0;
}

extern "C" int flstm_core_get_tuned(const flstm_core_plan* p, size_t index, size_t* T, int* row_tiles_fwd, int* row_tiles_bwd,
                                    int* stepwise_fwd, int* stepwise_bwd, int* dw_splits, int* bwd_two_d) {
    if (!p || index >= p->tuned.size()) return FLSTM_E_INVALID;
    const auto& t = p->tuned[index];
    if (T) *T = t.T;
    if (row_tiles_fwd) *row_tiles_fwd = t.mt_f;
    if (row_tiles_bwd) *row_tiles_bwd = t.mt_b;
    if (stepwise_fwd) *stepwise_fwd = t.step_f;
    if (stepwise_bwd) *stepwise_bwd = t.step_b;
    if (dw_splits) *dw_splits = t.dw_splits;
    if (bwd_two_d) *bwd_two_d = t.two_d;
    return 0;
}

extern "C" double flstm_core_tuned_ms(const flstm_core_plan* p, size_t T, const char* phase) {
    if (!p || !phase) return -1.0;
    for (const auto& t : p->tuned)
        if (t.T == T) {
            if (!strcmp(phase, "fwd_rec")) return t.ms_f;
            if (!strcmp(phase, "bwd_rec")) return t.ms_b;
            if (!strcmp(phase, "bwd_dw")) return t.ms_dw;
        }
    return -1.0;
}
