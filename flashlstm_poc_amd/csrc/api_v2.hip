// Host-streaming forward / backward (include/flashlstm_v2/lstm.hpp) on top of the device-resident
// core.  Replaces flstm::StreamingLstmForward (reference flashlstm_v2/src/lstm_forward.cu:464-966)
// and flstm::StreamingLstmBackward (flashlstm_v2/src/lstm_backward.cu:643-1250).
//
// Two levels.  A WINDOW is what the device holds at once: x, the gate / state caches, dG, dY and dx of up to W
// time steps.  288 GB of HBM hold whole sequences of ordinary length, so there is normally ONE window; longer
// sequences (or a smaller FLASHLSTM_V2_DEVICE_BUDGET_MB / a forced FLASHLSTM_V2_WINDOW_STEPS) run as several
// windows with the state carried between them in fp32, which is exact.  Inside a window the work is streamed
// in CHUNKS: x (dY) goes up in chunks of time steps on the h2d stream, each chunk's projection + recurrence
// (BPTT steps + dX) is enqueued on the compute stream behind an event, and its y (dx) rows leave on the d2h
// stream behind another, so the three streams overlap as in the reference's 32-step pipeline
// (flashlstm_v2/src/lstm_forward.cu:646-940).  FLASHLSTM_V2_CHUNK_STEPS sets the chunk length (default 64;
// 0 = whole window).
//
// Backward needs the gate cache of the steps it walks.  With one window, forward keeps it on the device in a
// small registry, and a backward call reuses it when it names the same buffers AND their contents are what
// the forward pass saw: the device tensors (both weight matrices, both biases, h0, c0) are checksummed in full
// on the device by either call, the host buffers x and y at 16 sampled places; any other backward call first
// recomputes the forward pass from x, h0 and c0 (FLASHLSTM_V2_RECOMPUTE=1 forces that).  What the sampled
// check cannot see is a rewrite of x or y between the two calls that misses all 16 samples.  With several
// windows, backward takes them last to first and recomputes each window's forward pass from the state at the
// window's start: the one the forward call left on the device when the registry matches, otherwise the host
// checkpoint at or before it (flashlstm_v2/src/lstm_backward.cu:897-1056 recomputes from the checkpoints in
// the same way), running forward over the steps in between.  dh / dc travel from window to window in fp32
// and dW / db are added up, so the results equal the single-window ones (dW, db: up to summation order).
// The host checkpoints are written with the reference's meaning: entry k = (h, c) before step
// k * recompute_interval.  Host buffers may be pageable (copies are then staged by the runtime and overlap
// less).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iterator>
#include <list>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/flashlstm/lstm_core.h"
#include "../../include/flashlstm_v2/lstm.hpp"
#include "instrument.h"
#include "pack.h"

namespace {

using flstm_hip::half_t;

void check(hipError_t e, const char* what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
void check_core(int rc, const char* what) {
    if (rc != 0) throw std::runtime_error(std::string(what) + " failed with status " + std::to_string(rc));
}

struct Buf {
    void* p = nullptr;
    size_t bytes = 0;
    void reserve(size_t need) {
        if (need <= bytes) return;
        if (p) check(hipFree(p), "hipFree");
        p = nullptr; bytes = 0;
        check(hipMalloc(&p, need), "hipMalloc");
        bytes = need;
    }
    void release() { if (p) (void)hipFree(p); p = nullptr; bytes = 0; }
};

struct ForwardKey {
    const void *x = nullptr, *y = nullptr, *ch = nullptr, *cc = nullptr, *h0 = nullptr, *c0 = nullptr;
    const void *w_ih = nullptr, *w_hh = nullptr;
    size_t T = 0, R = 0, W = 0;
    unsigned long long x_print = 0, y_print = 0, dev_print = 0;
    bool valid = false;
};

struct Entry {
    size_t B = 0, I = 0, H = 0;
    int device = 0;
    flstm_core_plan* plan = nullptr;
    Buf x_dev, y_dev, dy_dev, dx_dev, ck_h, ck_c;
    Buf carry_h, carry_c, carry_dh, carry_dc;   // fp32 (B, H): state / state gradient between windows
    Buf sum_dev;                                // one 64-bit checksum accumulator
    Buf starts;                                 // fp32 [window][h, c][B * H]: state at the start of each window
    std::vector<char> start_known;              // which entries of `starts` hold the current sequence's states
    ForwardKey last;
    hipEvent_t ev_in = nullptr, ev_out = nullptr;
    std::vector<hipEvent_t> chunk_in, chunk_out;   // one pair per chunk of a streamed pass
    void need_chunk_events(size_t n) {
        while (chunk_in.size() < n) {
            hipEvent_t a = nullptr, b = nullptr;
            check(hipEventCreateWithFlags(&a, hipEventDisableTiming), "hipEventCreate");
            check(hipEventCreateWithFlags(&b, hipEventDisableTiming), "hipEventCreate");
            chunk_in.push_back(a);
            chunk_out.push_back(b);
        }
    }
    size_t device_bytes() const {
        size_t sum = 0;
        for (const Buf* b : {&x_dev, &y_dev, &dy_dev, &dx_dev, &ck_h, &ck_c, &carry_h, &carry_c, &carry_dh, &carry_dc,
                             &starts, &sum_dev})
            sum += b->bytes;
        const long held = plan ? flstm_core_get_info(plan, "device_bytes") : 0;
        return sum + size_t(held > 0 ? held : 0);
    }
    ~Entry() {
        if (plan) flstm_core_destroy(plan);
        for (Buf* b : {&x_dev, &y_dev, &dy_dev, &dx_dev, &ck_h, &ck_c, &carry_h, &carry_c, &carry_dh, &carry_dc, &starts,
                       &sum_dev})
            b->release();
        if (ev_in) (void)hipEventDestroy(ev_in);
        if (ev_out) (void)hipEventDestroy(ev_out);
        for (hipEvent_t ev : chunk_in) (void)hipEventDestroy(ev);
        for (hipEvent_t ev : chunk_out) (void)hipEventDestroy(ev);
    }
};

std::mutex g_mutex;
std::list<Entry> g_entries;  // most recently used first
constexpr size_t kMaxEntries = 4;

// Every entry keeps whole-sequence caches alive (8 MiB per step at B = 256, H = 1024), so the registry is bounded
// in bytes as well as in count: shapes other than the one in use are dropped, least recently used first, while
// they hold more than FLASHLSTM_V2_REGISTRY_MB together (default: a quarter of the device's memory).
void trim_registry() {
    size_t cap = 0;
    if (const char* v = getenv("FLASHLSTM_V2_REGISTRY_MB")) cap = size_t(atol(v) > 0 ? atol(v) : 0) << 20;
    if (cap == 0) {
        size_t free_b = 0, total_b = 0;
        if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) return;
        cap = total_b / 4;
    }
    while (g_entries.size() > 1) {
        size_t others = 0;
        for (auto it = std::next(g_entries.begin()); it != g_entries.end(); ++it) others += it->device_bytes();
        if (others <= cap) break;
        g_entries.pop_back();
    }
}

Entry& entry_for(size_t B, size_t I, size_t H) {
    int dev = 0;
    check(hipGetDevice(&dev), "hipGetDevice");
    for (auto it = g_entries.begin(); it != g_entries.end(); ++it) {
        if (it->B == B && it->I == I && it->H == H && it->device == dev) {
            g_entries.splice(g_entries.begin(), g_entries, it);
            trim_registry();
            return g_entries.front();
        }
    }
    while (g_entries.size() >= kMaxEntries) g_entries.pop_back();
    g_entries.emplace_front();
    Entry& e = g_entries.front();
    e.B = B; e.I = I; e.H = H; e.device = dev;
    check_core(flstm_core_create(B, I, H, &e.plan), "flstm_core_create");
    check(hipEventCreateWithFlags(&e.ev_in, hipEventDisableTiming), "hipEventCreate");
    check(hipEventCreateWithFlags(&e.ev_out, hipEventDisableTiming), "hipEventCreate");
    trim_registry();
    return e;
}

// FNV-1a over 16 evenly spread 256-byte samples of a host buffer (all of it when it is no longer than that):
// cheap evidence that it still holds what the cached forward pass saw.
unsigned long long fingerprint(const void* p, size_t bytes) {
    const unsigned char* b = static_cast<const unsigned char*>(p);
    unsigned long long h = 1469598103934665603ull;
    constexpr size_t kSamples = 16, kWin = 256;
    if (bytes <= kSamples * kWin) {
        for (size_t i = 0; i < bytes; ++i) { h ^= b[i]; h *= 1099511628211ull; }
        return h;
    }
    for (size_t k = 0; k < kSamples; ++k) {
        const size_t s = (bytes - kWin) / (kSamples - 1) * k;
        for (size_t i = 0; i < kWin; ++i) { h ^= b[s + i]; h *= 1099511628211ull; }
    }
    return h;
}

// Checksum over the full contents of the device tensors a pass depends on (computed on the device, 8 bytes come
// back): weights or initial states updated in place between forward and backward change it.
unsigned long long device_print(Entry& e, hipStream_t s, const float* w_ih, const float* w_hh, const float* b_ih,
                                const float* b_hh, const __half* h0, const __half* c0) {
    using flstm_hip::checksum_add;
    const size_t G = 4 * e.H;
    e.sum_dev.reserve(sizeof(unsigned long long));   // (throws if the allocation fails)
    auto* acc = static_cast<flstm_hip::u64*>(e.sum_dev.p);
    check(flstm_hip::fill_zero(acc, sizeof(unsigned long long), s), "checksum");
    check(checksum_add(w_ih, G * e.I * sizeof(float), 0x1000000000ull, acc, s), "checksum");
    check(checksum_add(w_hh, G * e.H * sizeof(float), 0x2000000000ull, acc, s), "checksum");
    check(checksum_add(b_ih, G * sizeof(float), 0x3000000000ull, acc, s), "checksum");
    check(checksum_add(b_hh, G * sizeof(float), 0x4000000000ull, acc, s), "checksum");
    check(checksum_add(h0, e.B * e.H * sizeof(half_t), 0x5000000000ull, acc, s), "checksum");
    check(checksum_add(c0, e.B * e.H * sizeof(half_t), 0x6000000000ull, acc, s), "checksum");
    unsigned long long host = 0;
    check(hipMemcpyAsync(&host, acc, sizeof(host), hipMemcpyDeviceToHost, s), "checksum");
    check(hipStreamSynchronize(s), "checksum");
    // which of the optional tensors are present is part of the identity
    return host ^ (b_ih ? 1ull : 0) ^ (b_hh ? 2ull : 0) ^ (h0 ? 4ull : 0) ^ (c0 ? 8ull : 0);
}

void validate_common(size_t R, hipStream_t c, hipStream_t h2d, hipStream_t d2h) {
    if (R == 0) throw std::runtime_error("recompute_interval must be >= 1");
    if (c == h2d || c == d2h || h2d == d2h)
        throw std::runtime_error("compute, h2d and d2h streams must be pairwise distinct");
}

size_t chunk_steps_for(size_t T) {
    const char* v = getenv("FLASHLSTM_V2_CHUNK_STEPS");   // read per call: cheap, and tests switch it
    const long env = v ? atol(v) : 64L;
    return (env <= 0 || size_t(env) > T) ? T : size_t(env);
}

// rows [row0, row0+rows) of a device matrix with pitch ld (elements of esz bytes, `cols` used) -> packed host rows
void download_rows(void* host, const void* dev, size_t ld, size_t cols, size_t esz, size_t row0, size_t rows,
                   hipStream_t s) {
    char* dst = static_cast<char*>(host) + row0 * cols * esz;
    const char* src = static_cast<const char*>(dev) + row0 * ld * esz;
    if (ld == cols) check(hipMemcpyAsync(dst, src, rows * cols * esz, hipMemcpyDeviceToHost, s), "download");
    else check(hipMemcpy2DAsync(dst, cols * esz, src, ld * esz, cols * esz, rows, hipMemcpyDeviceToHost, s), "download");
}

struct Streams { hipStream_t cs, h2d, d2h; };

void sync_all(const Streams& st) {
    check(hipStreamSynchronize(st.cs), "sync compute");
    check(hipStreamSynchronize(st.h2d), "sync h2d");
    check(hipStreamSynchronize(st.d2h), "sync d2h");
}

// Steps per window: everything a pass keeps per time step on the device (staging + the core's caches),
// against a budget of FLASHLSTM_V2_DEVICE_BUDGET_MB (default: 70 % of the device's memory, and no more than
// 85 % of what is free now plus what this shape's buffers already hold).  FLASHLSTM_V2_WINDOW_STEPS forces a
// value.  Read per call: cheap, and tests switch them.
size_t window_steps_for(const Entry& e, size_t T) {
    const size_t B = e.B, I = e.I, H = e.H;
    if (const char* v = getenv("FLASHLSTM_V2_WINDOW_STEPS")) {
        const long w = atol(v);
        if (w > 0) return size_t(w) < T ? size_t(w) : T;
    }
    const size_t Hp = (H + 31) / 32 * 32, Ip = (I + 63) / 64 * 64;
    const size_t per_step = B * (4 * I + 2 * Ip + 24 * Hp + 2 * H);
    size_t budget = 0;
    if (const char* v = getenv("FLASHLSTM_V2_DEVICE_BUDGET_MB")) budget = size_t(atol(v) > 0 ? atol(v) : 0) << 20;
    if (budget == 0) {
        size_t free_b = 0, total_b = 0;
        check(hipMemGetInfo(&free_b, &total_b), "hipMemGetInfo");
        size_t held = size_t(flstm_core_get_info(e.plan, "device_bytes") > 0 ? flstm_core_get_info(e.plan, "device_bytes") : 0);
        for (const Buf* b : {&e.x_dev, &e.y_dev, &e.dy_dev, &e.dx_dev}) held += b->bytes;
        budget = total_b / 10 * 7;
        if (budget > (free_b + held) / 20 * 17) budget = (free_b + held) / 20 * 17;
    }
    size_t w = budget / per_step;
    if (w >= T) return T;
    const size_t c = chunk_steps_for(T);
    if (w > c) w -= w % c;   // whole chunks
    return w ? w : 1;
}

struct CachePtrs { const half_t* h = nullptr; const float* c = nullptr; size_t ldh = 0, ldc = 0; };

CachePtrs cache_ptrs(Entry& e) {
    CachePtrs cp;
    const void* hp = nullptr; const void* cptr = nullptr;
    check_core(flstm_core_cache_ptr(e.plan, 0, &hp, &cp.ldh), "flstm_core_cache_ptr");
    check_core(flstm_core_cache_ptr(e.plan, 1, &cptr, &cp.ldc), "flstm_core_cache_ptr");
    cp.h = static_cast<const half_t*>(hp);
    cp.c = static_cast<const float*>(cptr);
    return cp;
}

// Forward pass over the n steps of one window, from the state (h_in, c_in) of `state_dtype`: x rows up, chunk
// by chunk, projection + recurrence behind them, y rows down.  Leaves the window's caches in the plan (row
// block 0 of the state arrays = the state the window started from) and x in e.x_dev; writes the final state
// to (hy, cy) in `out_dtype` when they are given.  The compute stream is idle when it returns.
CachePtrs forward_window(Entry& e, const Streams& st, size_t n, const __half* x_host, const void* h_in,
                         const void* c_in, flstm_dtype state_dtype, __half* y_host, void* hy, void* cy,
                         flstm_dtype out_dtype) {
    const size_t B = e.B, I = e.I, H = e.H;
    e.x_dev.reserve(n * B * I * sizeof(half_t));
    check_core(flstm_core_forward_begin(e.plan, n, e.x_dev.p, FLSTM_F16, h_in, c_in, state_dtype, st.cs),
               "flstm_core_forward_begin");
    CachePtrs cp = cache_ptrs(e);
    const size_t C = chunk_steps_for(n), nchunks = (n + C - 1) / C;
    e.need_chunk_events(nchunks);
    auto upload = [&](size_t k) {
        const size_t t0 = k * C, m = (t0 + C <= n) ? C : n - t0;
        check(hipMemcpyAsync(static_cast<char*>(e.x_dev.p) + t0 * B * I * sizeof(half_t),
                             reinterpret_cast<const char*>(x_host) + t0 * B * I * sizeof(half_t), m * B * I * sizeof(half_t),
                             hipMemcpyHostToDevice, st.h2d), "x upload");
        check(hipEventRecord(e.chunk_in[k], st.h2d), "hipEventRecord");
    };
    upload(0);
    for (size_t k = 0; k < nchunks; ++k) {
        const size_t t0 = k * C, m = (t0 + C <= n) ? C : n - t0;
        if (k + 1 < nchunks) upload(k + 1);
        check(hipStreamWaitEvent(st.cs, e.chunk_in[k], 0), "hipStreamWaitEvent");
        check_core(flstm_core_forward_steps(e.plan, t0, m, st.cs), "flstm_core_forward_steps");
        check(hipEventRecord(e.chunk_out[k], st.cs), "hipEventRecord");
        if (y_host) {   // h_t of step t is row block t+1 of the state cache
            check(hipStreamWaitEvent(st.d2h, e.chunk_out[k], 0), "hipStreamWaitEvent");
            download_rows(y_host, cp.h + B * cp.ldh, cp.ldh, H, sizeof(half_t), t0 * B, m * B, st.d2h);
        }
    }
    int rc = flstm_core_forward_end(e.plan, hy, cy, out_dtype, 1, st.cs);
    if (rc == FLSTM_E_STALLED) {
        // a persistent launch gave up: repeat the pass through the entry point that falls back to step-wise launches
        check(hipStreamSynchronize(st.d2h), "sync d2h");
        const size_t y_bytes = n * B * H * sizeof(half_t);
        e.y_dev.reserve(y_bytes);
        check_core(flstm_core_forward(e.plan, n, e.x_dev.p, FLSTM_F16, h_in, c_in, state_dtype, y_host ? e.y_dev.p : nullptr,
                                      FLSTM_F16, hy, cy, out_dtype, 1, st.cs), "flstm_core_forward");
        if (y_host) check(hipMemcpyAsync(y_host, e.y_dev.p, y_bytes, hipMemcpyDeviceToHost, st.d2h), "y download");
        cp = cache_ptrs(e);
    } else {
        check_core(rc, "flstm_core_forward_end");
    }
    return cp;
}

// Checkpoints that fall into the window of steps [t0, t0 + n): entry k = state before step k * R, which is row
// block k * R - t0 of the window's state arrays.
void write_checkpoints(Entry& e, const Streams& st, const CachePtrs& cp, size_t t0, size_t n, size_t R,
                       flstm::GateCacheHost cache, flstm::StreamingLstmOptions opt) {
    const size_t B = e.B, H = e.H;
    const size_t k0 = (t0 + R - 1) / R, k1 = (t0 + n + R - 1) / R;   // k * R in [t0, t0 + n)
    if (k1 <= k0 || (!cache.h_ptr && !cache.c_ptr)) return;
    const size_t nk = k1 - k0, row0 = (k0 * R - t0) * B;
    const bool h32 = opt.h_dtype == flstm::GateCacheDType::kFloat32;
    const bool c32 = opt.c_dtype == flstm::GateCacheDType::kFloat32;
    const size_t hsz = h32 ? 4 : 2, csz = c32 ? 4 : 2;
    if (cache.h_ptr) {
        e.ck_h.reserve(nk * B * H * hsz);
        check(flstm_hip::gather_from_half(cp.h + row0 * cp.ldh, cp.ldh, nk * B, int(H), e.ck_h.p, h32, B, R * B, st.cs),
              "checkpoint gather");
    }
    if (cache.c_ptr) {
        e.ck_c.reserve(nk * B * H * csz);
        check(flstm_hip::gather_from_float(cp.c + row0 * cp.ldc, cp.ldc, nk * B, int(H), 1.f, e.ck_c.p, c32, B, R * B,
                                           st.cs), "checkpoint gather");
    }
    check(hipEventRecord(e.ev_out, st.cs), "hipEventRecord");
    check(hipStreamWaitEvent(st.d2h, e.ev_out, 0), "hipStreamWaitEvent");
    if (cache.h_ptr)
        check(hipMemcpyAsync(static_cast<char*>(cache.h_ptr) + k0 * B * H * hsz, e.ck_h.p, nk * B * H * hsz,
                             hipMemcpyDeviceToHost, st.d2h), "h checkpoints");
    if (cache.c_ptr)
        check(hipMemcpyAsync(static_cast<char*>(cache.c_ptr) + k0 * B * H * csz, e.ck_c.p, nk * B * H * csz,
                             hipMemcpyDeviceToHost, st.d2h), "c checkpoints");
}

float* start_state(Entry& e, size_t window, int which) {   // which: 0 = h, 1 = c
    return static_cast<float*>(e.starts.p) + (window * 2 + which) * e.B * e.H;
}

void copy_state(float* dst, const void* src, size_t count, hipStream_t s) {
    check(hipMemcpyAsync(dst, src, count * sizeof(float), hipMemcpyDeviceToDevice, s), "state copy");
}

void run_forward(Entry& e, size_t T, size_t R, const __half* x_host, const __half* h0, const __half* c0,
                 const float* w_ih, const float* w_hh, const float* b_ih, const float* b_hh, __half* y_host,
                 flstm::GateCacheHost cache, flstm::StreamingLstmOptions opt, __half* hy, __half* cy,
                 const Streams& st) {
    const size_t B = e.B, I = e.I, H = e.H, BH = B * H;
    e.last.valid = false;
    check_core(flstm_core_pack_weights(e.plan, w_ih, w_hh, st.cs), "flstm_core_pack_weights");
    check_core(flstm_core_pack_bias(e.plan, b_ih, b_hh, st.cs), "flstm_core_pack_bias");
    const size_t W = window_steps_for(e, T), nwin = (T + W - 1) / W;
    e.start_known.assign(nwin, 0);
    if (nwin == 1) {
        const CachePtrs cp = forward_window(e, st, T, x_host, h0, c0, FLSTM_F16, y_host, hy, cy, FLSTM_F16);
        write_checkpoints(e, st, cp, 0, T, R, cache, opt);
    } else {
        e.carry_h.reserve(BH * sizeof(float));
        e.carry_c.reserve(BH * sizeof(float));
        e.starts.reserve(nwin * 2 * BH * sizeof(float));
        for (size_t j = 0; j < nwin; ++j) {
            const size_t t0 = j * W, n = (t0 + W <= T) ? W : T - t0;
            const bool first = (j == 0), last = (j + 1 == nwin);
            if (!first) {   // keep the state this window starts from for a backward call on the same buffers
                copy_state(start_state(e, j, 0), e.carry_h.p, BH, st.cs);
                copy_state(start_state(e, j, 1), e.carry_c.p, BH, st.cs);
                e.start_known[j] = 1;
            }
            const CachePtrs cp = forward_window(
                e, st, n, x_host + t0 * B * I, first ? static_cast<const void*>(h0) : e.carry_h.p,
                first ? static_cast<const void*>(c0) : e.carry_c.p, first ? FLSTM_F16 : FLSTM_F32,
                y_host ? y_host + t0 * B * H : nullptr, last ? static_cast<void*>(hy) : e.carry_h.p,
                last ? static_cast<void*>(cy) : e.carry_c.p, last ? FLSTM_F16 : FLSTM_F32);
            write_checkpoints(e, st, cp, t0, n, R, cache, opt);
            sync_all(st);   // the next window reuses every buffer
        }
    }
    sync_all(st);
    ForwardKey k;
    k.x = x_host; k.y = y_host; k.ch = cache.h_ptr; k.cc = cache.c_ptr; k.h0 = h0; k.c0 = c0;
    k.w_ih = w_ih; k.w_hh = w_hh; k.T = T; k.R = R; k.W = W;
    k.x_print = fingerprint(x_host, T * B * I * sizeof(half_t));
    k.y_print = y_host ? fingerprint(y_host, T * B * H * sizeof(half_t)) : 0;
    k.dev_print = device_print(e, st.cs, w_ih, w_hh, b_ih, b_hh, h0, c0);
    k.valid = true;
    e.last = k;
}

// BPTT over the n steps of the window whose forward caches the plan holds (and whose x rows are in e.x_dev):
// dY rows up chunk by chunk from the end, BPTT steps + dX behind them, dx rows down; then the weight-gradient
// GEMMs over the window.  (d_hn, d_cn) of `dstate_dtype` is the gradient flowing in at the window's end,
// (dh0, dc0) the one flowing out at its start (fp32).
void backward_window(Entry& e, const Streams& st, size_t n, const __half* dY_host, const void* d_hn, const void* d_cn,
                     flstm_dtype dstate_dtype, __half* dx_host, bool accumulate, float* dW_ih, float* dW_hh,
                     float* db_ih, float* db_hh, float* dh0, float* dc0) {
    const size_t B = e.B, I = e.I, H = e.H;
    const size_t x_bytes = n * B * I * sizeof(half_t), y_bytes = n * B * H * sizeof(half_t);
    e.dy_dev.reserve(y_bytes);
    if (dx_host) e.dx_dev.reserve(x_bytes);
    check_core(flstm_core_set_option(e.plan, "accumulate_grads", accumulate ? 1 : 0), "flstm_core_set_option");
    check_core(flstm_core_backward_begin(e.plan, n, e.dy_dev.p, FLSTM_F16, d_hn, d_cn, dstate_dtype, 1.f,
                                         dx_host ? e.dx_dev.p : nullptr, FLSTM_F16, st.cs), "flstm_core_backward_begin");
    const size_t C = chunk_steps_for(n), nchunks = (n + C - 1) / C;
    e.need_chunk_events(nchunks);
    auto chunk_range = [&](size_t k, size_t& lo, size_t& m) {   // chunk k counts from the end; the first one takes the remainder
        const size_t rem = n % C, first = rem ? rem : C;
        m = (k == 0) ? first : C;
        const size_t hi = n - 1 - (k == 0 ? 0 : first + (k - 1) * C);
        lo = hi + 1 - m;
    };
    auto upload = [&](size_t k) {
        size_t lo, m;
        chunk_range(k, lo, m);
        check(hipMemcpyAsync(static_cast<char*>(e.dy_dev.p) + lo * B * H * sizeof(half_t),
                             reinterpret_cast<const char*>(dY_host) + lo * B * H * sizeof(half_t), m * B * H * sizeof(half_t),
                             hipMemcpyHostToDevice, st.h2d), "dY upload");
        check(hipEventRecord(e.chunk_in[k], st.h2d), "hipEventRecord");
    };
    upload(0);
    for (size_t k = 0; k < nchunks; ++k) {
        size_t lo, m;
        chunk_range(k, lo, m);
        if (k + 1 < nchunks) upload(k + 1);
        check(hipStreamWaitEvent(st.cs, e.chunk_in[k], 0), "hipStreamWaitEvent");
        check_core(flstm_core_backward_steps(e.plan, lo + m - 1, m, st.cs), "flstm_core_backward_steps");
        check(hipEventRecord(e.chunk_out[k], st.cs), "hipEventRecord");
        if (dx_host) {
            check(hipStreamWaitEvent(st.d2h, e.chunk_out[k], 0), "hipStreamWaitEvent");
            download_rows(dx_host, e.dx_dev.p, I, I, sizeof(half_t), lo * B, m * B, st.d2h);
        }
    }
    int rc = flstm_core_backward_end(e.plan, e.x_dev.p, FLSTM_F16, dW_ih, dW_hh, db_ih, db_hh, dh0, dc0, st.cs);
    if (rc == FLSTM_E_STALLED) {
        // a persistent launch gave up: repeat the pass through the entry point that falls back to step-wise launches
        check(hipStreamSynchronize(st.d2h), "sync d2h");
        check_core(flstm_core_backward(e.plan, n, e.x_dev.p, FLSTM_F16, e.dy_dev.p, FLSTM_F16, d_hn, d_cn, dstate_dtype,
                                       1.f, dx_host ? e.dx_dev.p : nullptr, FLSTM_F16, dW_ih, dW_hh, db_ih, db_hh, dh0,
                                       dc0, st.cs), "flstm_core_backward");
        if (dx_host) check(hipMemcpyAsync(dx_host, e.dx_dev.p, x_bytes, hipMemcpyDeviceToHost, st.d2h), "dx download");
    } else {
        check_core(rc, "flstm_core_backward_end");
    }
    check_core(flstm_core_set_option(e.plan, "accumulate_grads", 0), "flstm_core_set_option");
}

// The state at the start of window j (step j * W) from the host checkpoints: entry floor(j * W / R) is the
// state before step t_ck <= j * W; forward over [t_ck, j * W) brings it there.  Every window start passed on
// the way is kept, so the windows of one checkpoint interval share this work.  Returns the steps recomputed.
size_t rebuild_start_state(Entry& e, const Streams& st, size_t j, size_t W, size_t R, const __half* x_host,
                           flstm::GateCacheHost cache, flstm::StreamingLstmOptions opt) {
    const size_t B = e.B, I = e.I, H = e.H, BH = B * H;
    const size_t target = j * W, k = target / R, t_ck = k * R;
    const bool h32 = opt.h_dtype == flstm::GateCacheDType::kFloat32;
    const bool c32 = opt.c_dtype == flstm::GateCacheDType::kFloat32;
    e.carry_h.reserve(BH * sizeof(float));
    e.carry_c.reserve(BH * sizeof(float));
    e.ck_h.reserve(BH * 4);
    e.ck_c.reserve(BH * 4);
    check(hipMemcpyAsync(e.ck_h.p, static_cast<const char*>(cache.h_ptr) + k * BH * (h32 ? 4 : 2), BH * (h32 ? 4 : 2),
                         hipMemcpyHostToDevice, st.cs), "h checkpoint upload");
    check(hipMemcpyAsync(e.ck_c.p, static_cast<const char*>(cache.c_ptr) + k * BH * (c32 ? 4 : 2), BH * (c32 ? 4 : 2),
                         hipMemcpyHostToDevice, st.cs), "c checkpoint upload");
    if (h32) copy_state(static_cast<float*>(e.carry_h.p), e.ck_h.p, BH, st.cs);
    else check(flstm_hip::unpad_from_half(static_cast<const half_t*>(e.ck_h.p), H, B, int(H), e.carry_h.p, 1, st.cs), "h checkpoint");
    if (c32) copy_state(static_cast<float*>(e.carry_c.p), e.ck_c.p, BH, st.cs);
    else check(flstm_hip::unpad_from_half(static_cast<const half_t*>(e.ck_c.p), H, B, int(H), e.carry_c.p, 1, st.cs), "c checkpoint");
    size_t cur = t_ck;
    while (cur < target) {
        const size_t end = (cur / W + 1) * W < target ? (cur / W + 1) * W : target;   // stop at every window start
        forward_window(e, st, end - cur, x_host + cur * B * I, e.carry_h.p, e.carry_c.p, FLSTM_F32, nullptr, e.carry_h.p,
                       e.carry_c.p, FLSTM_F32);
        sync_all(st);
        cur = end;
        if (cur % W == 0) {
            copy_state(start_state(e, cur / W, 0), e.carry_h.p, BH, st.cs);
            copy_state(start_state(e, cur / W, 1), e.carry_c.p, BH, st.cs);
            e.start_known[cur / W] = 1;
        }
    }
    if (t_ck == target) {   // the checkpoint is the window start itself
        copy_state(start_state(e, j, 0), e.carry_h.p, BH, st.cs);
        copy_state(start_state(e, j, 1), e.carry_c.p, BH, st.cs);
        e.start_known[j] = 1;
    }
    return target - t_ck;
}

}  // namespace

namespace flstm {

void StreamingLstmForward(size_t T, size_t B, size_t I, size_t H, size_t R, const __half* x_host,
                          const __half* h0, const __half* c0, const float* w_ih, const float* w_hh,
                          const float* b_ih, const float* b_hh, __half* y_host, GateCacheHost cache,
                          StreamingLstmOptions opt, __half* hy, __half* cy, hipStream_t cs, hipStream_t h2d,
                          hipStream_t d2h) {
    if (T == 0 || B == 0 || I == 0 || H == 0) return;
    validate_common(R, cs, h2d, d2h);
    if (!x_host || !w_ih || !w_hh) throw std::runtime_error("StreamingLstmForward: null input tensor");
    std::lock_guard<std::mutex> lock(g_mutex);
    flstm_hip::RangeGuard range("FlashLSTM::StreamingLstmForward");
    flstm_hip::MfuProfiler prof("forward");   // (same label and line as flashlstm_v2/src/lstm_forward.cu:492)
    Entry& e = entry_for(B, I, H);
    run_forward(e, T, R, x_host, h0, c0, w_ih, w_hh, b_ih, b_hh, y_host, cache, opt, hy, cy, Streams{cs, h2d, d2h});
    prof.add_useful(double(T) * flstm_hip::gemm_flops(4 * H, B, I + H));
    prof.finish();
}

void StreamingLstmBackward(size_t T, size_t B, size_t I, size_t H, size_t R, const __half* x_host,
                           const __half* y_host, GateCacheHost cache, StreamingLstmOptions opt,
                           const __half* dY_host, const __half* d_hn, const __half* d_cn, const __half* h0,
                           const __half* c0, const float* w_ih, const float* w_hh, const float* b_ih,
                           const float* b_hh, __half* dx_host, float* dW_ih, float* dW_hh, float* db_ih,
                           float* db_hh, float* dh0, float* dc0, hipStream_t cs, hipStream_t h2d,
                           hipStream_t d2h) {
    if (T == 0 || B == 0 || I == 0 || H == 0) return;
    validate_common(R, cs, h2d, d2h);
    if (!x_host || !dY_host || !w_ih || !w_hh) throw std::runtime_error("StreamingLstmBackward: null input tensor");
    if (!cache.h_ptr || !cache.c_ptr) throw std::runtime_error("StreamingLstmBackward: gate cache pointers are null");
    std::lock_guard<std::mutex> lock(g_mutex);
    flstm_hip::RangeGuard range("FlashLSTM::StreamingLstmBackward");
    flstm_hip::MfuProfiler prof("backward");   // (flashlstm_v2/src/lstm_backward.cu:679)
    Entry& e = entry_for(B, I, H);
    const Streams st{cs, h2d, d2h};
    const size_t x_bytes = T * B * I * sizeof(half_t), y_bytes = T * B * H * sizeof(half_t), BH = B * H;
    const size_t W = window_steps_for(e, T), nwin = (T + W - 1) / W;
    static const bool always_recompute = (getenv("FLASHLSTM_V2_RECOMPUTE") != nullptr);
    const ForwardKey& k = e.last;
    bool hit = !always_recompute && k.valid && k.x == x_host && k.y == y_host && k.ch == cache.h_ptr &&
               k.cc == cache.c_ptr && k.h0 == h0 && k.c0 == c0 && k.w_ih == w_ih && k.w_hh == w_hh && k.T == T &&
               k.W == W;
    if (hit) hit = (k.x_print == fingerprint(x_host, x_bytes)) && (!y_host || k.y_print == fingerprint(y_host, y_bytes));
    if (hit) hit = (k.dev_print == device_print(e, cs, w_ih, w_hh, b_ih, b_hh, h0, c0));
    const double fwd_flops_per_step = flstm_hip::gemm_flops(4 * H, B, I + H);
    if (nwin == 1) {
        if (!hit) {
            // rebuild the device-side caches from the inputs (no host outputs are touched)
            run_forward(e, T, R, x_host, h0, c0, w_ih, w_hh, b_ih, b_hh, nullptr, GateCacheHost{nullptr, nullptr},
                        StreamingLstmOptions{}, nullptr, nullptr, st);
            prof.add_total(double(T) * fwd_flops_per_step);   // recomputation
        }
        backward_window(e, st, T, dY_host, d_hn, d_cn, FLSTM_F16, dx_host, false, dW_ih, dW_hh, db_ih, db_hh, dh0, dc0);
    } else {
        if (!hit) {   // nothing on the device describes this sequence: weights again, window starts from the checkpoints
            e.last.valid = false;
            check_core(flstm_core_pack_weights(e.plan, w_ih, w_hh, cs), "flstm_core_pack_weights");
            check_core(flstm_core_pack_bias(e.plan, b_ih, b_hh, cs), "flstm_core_pack_bias");
            e.starts.reserve(nwin * 2 * BH * sizeof(float));
            e.start_known.assign(nwin, 0);
        }
        e.carry_dh.reserve(BH * sizeof(float));
        e.carry_dc.reserve(BH * sizeof(float));
        for (size_t j = nwin; j-- > 0;) {
            const size_t t0 = j * W, n = (t0 + W <= T) ? W : T - t0;
            const bool first = (j == 0), last = (j + 1 == nwin);
            if (!first && !e.start_known[j])
                prof.add_total(double(rebuild_start_state(e, st, j, W, R, x_host, cache, opt)) * fwd_flops_per_step);
            // this window's gate cache
            forward_window(e, st, n, x_host + t0 * B * I, first ? static_cast<const void*>(h0) : start_state(e, j, 0),
                           first ? static_cast<const void*>(c0) : start_state(e, j, 1), first ? FLSTM_F16 : FLSTM_F32,
                           nullptr, nullptr, nullptr, FLSTM_F16);
            prof.add_total(double(n) * fwd_flops_per_step);
            backward_window(e, st, n, dY_host + t0 * B * H, last ? static_cast<const void*>(d_hn) : e.carry_dh.p,
                            last ? static_cast<const void*>(d_cn) : e.carry_dc.p, last ? FLSTM_F16 : FLSTM_F32,
                            dx_host ? dx_host + t0 * B * I : nullptr, !last, dW_ih, dW_hh, db_ih, db_hh,
                            first ? dh0 : static_cast<float*>(e.carry_dh.p), first ? dc0 : static_cast<float*>(e.carry_dc.p));
            sync_all(st);   // the next window reuses every buffer
        }
    }
    sync_all(st);
    // dh = dG W_hh per step, dX = dG W_ih, dW_ih = dG^T X, dW_hh = dG^T H over the whole sequence
    prof.add_useful(double(T) * flstm_hip::gemm_flops(H, B, 4 * H) + flstm_hip::gemm_flops(I, T * B, 4 * H) +
                    flstm_hip::gemm_flops(I, 4 * H, T * B) + flstm_hip::gemm_flops(H, 4 * H, T * B));
    prof.finish();
}

}  // namespace flstm

extern "C" void flstm_StreamingLstmForward(
    size_t T, size_t B, size_t I, size_t H, size_t R, const __half* x_host, const __half* h0, const __half* c0,
    const float* w_ih, const float* w_hh, const float* b_ih, const float* b_hh, __half* y_host,
    flstm_GateCacheHost cache, const flstm_StreamingLstmOptions* options, __half* hy, __half* cy,
    hipStream_t cs, hipStream_t h2d, hipStream_t d2h) {
    try {
        flstm::StreamingLstmOptions opt;
        if (options) {
            opt.h_dtype = static_cast<flstm::GateCacheDType>(options->h_dtype);
            opt.c_dtype = static_cast<flstm::GateCacheDType>(options->c_dtype);
        }
        flstm::StreamingLstmForward(T, B, I, H, R, x_host, h0, c0, w_ih, w_hh, b_ih, b_hh, y_host,
                                    flstm::GateCacheHost{cache.h_ptr, cache.c_ptr}, opt, hy, cy, cs, h2d, d2h);
    } catch (const std::exception& ex) {
        std::fprintf(stderr, "flstm_StreamingLstmForward failed: %s\n", ex.what());
        std::abort();
    }
}

extern "C" void flstm_StreamingLstmBackward(
    size_t T, size_t B, size_t I, size_t H, size_t R, const __half* x_host, const __half* y_host,
    flstm_GateCacheHost cache, const __half* dY_host, const __half* d_hn, const __half* d_cn, const __half* h0,
    const __half* c0, const float* w_ih, const float* w_hh, const float* b_ih, const float* b_hh, __half* dx_host,
    float* dW_ih, float* dW_hh, float* db_ih, float* db_hh, float* dh0, float* dc0, hipStream_t cs,
    hipStream_t h2d, hipStream_t d2h, const flstm_StreamingLstmOptions* options) {
    try {
        flstm::StreamingLstmOptions opt;
        if (options) {
            opt.h_dtype = static_cast<flstm::GateCacheDType>(options->h_dtype);
            opt.c_dtype = static_cast<flstm::GateCacheDType>(options->c_dtype);
        }
        flstm::StreamingLstmBackward(T, B, I, H, R, x_host, y_host, flstm::GateCacheHost{cache.h_ptr, cache.c_ptr},
                                     opt, dY_host, d_hn, d_cn, h0, c0, w_ih, w_hh, b_ih, b_hh, dx_host, dW_ih,
                                     dW_hh, db_ih, db_hh, dh0, dc0, cs, h2d, d2h);
    } catch (const std::exception& ex) {
        std::fprintf(stderr, "flstm_StreamingLstmBackward failed: %s\n", ex.what());
        std::abort();
    }
}

// Drops every cached plan and staging buffer of the streaming entry points.
extern "C" void flstm_ReleaseStreamingCaches(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_entries.clear();
}
