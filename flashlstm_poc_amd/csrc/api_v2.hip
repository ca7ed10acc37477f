// Host-streaming forward / backward (include/flashlstm_v2/lstm.hpp) on top of the device-resident
// core.  Replaces flstm::StreamingLstmForward (reference flashlstm_v2/src/lstm_forward.cu:464-966)
// and flstm::StreamingLstmBackward (flashlstm_v2/src/lstm_backward.cu:643-1250).
//
// 288 GB of HBM hold whole sequences, so instead of walking 32-step chunks through small device
// buffers the sequence is copied in once on the h2d stream, processed by the core on the compute
// stream, and results leave on the d2h stream.  Forward keeps its device-side gate cache in a small
// registry; a backward call that names the same host buffers (and whose sampled contents still
// match) reuses it, any other backward call first recomputes the forward pass from x, h0 and c0 --
// which yields exactly the states the host checkpoints describe.  The host checkpoints are written
// with the reference's meaning: entry k = (h, c) before step k * recompute_interval.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <list>
#include <mutex>
#include <stdexcept>
#include <string>

#include "../../include/flashlstm/lstm_core.h"
#include "../../include/flashlstm_v2/lstm.hpp"
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
    size_t T = 0, R = 0;
    unsigned long long x_print = 0, y_print = 0;
    bool valid = false;
};

struct Entry {
    size_t B = 0, I = 0, H = 0;
    int device = 0;
    flstm_core_plan* plan = nullptr;
    Buf x_dev, y_dev, dy_dev, dx_dev, ck_h, ck_c;
    ForwardKey last;
    hipEvent_t ev_in = nullptr, ev_out = nullptr;
    ~Entry() {
        if (plan) flstm_core_destroy(plan);
        for (Buf* b : {&x_dev, &y_dev, &dy_dev, &dx_dev, &ck_h, &ck_c}) b->release();
        if (ev_in) (void)hipEventDestroy(ev_in);
        if (ev_out) (void)hipEventDestroy(ev_out);
    }
};

std::mutex g_mutex;
std::list<Entry> g_entries;  // most recently used first
constexpr size_t kMaxEntries = 4;

Entry& entry_for(size_t B, size_t I, size_t H) {
    int dev = 0;
    check(hipGetDevice(&dev), "hipGetDevice");
    for (auto it = g_entries.begin(); it != g_entries.end(); ++it) {
        if (it->B == B && it->I == I && it->H == H && it->device == dev) {
            g_entries.splice(g_entries.begin(), g_entries, it);
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
    return e;
}

// FNV-1a over three 256-byte samples of a host buffer: cheap evidence that it still holds what the
// cached forward pass saw.
unsigned long long fingerprint(const void* p, size_t bytes) {
    const unsigned char* b = static_cast<const unsigned char*>(p);
    unsigned long long h = 1469598103934665603ull;
    const size_t win = bytes < 256 ? bytes : 256;
    const size_t starts[3] = {0, bytes > win ? (bytes - win) / 2 : 0, bytes - win};
    for (size_t s : starts)
        for (size_t i = 0; i < win; ++i) { h ^= b[s + i]; h *= 1099511628211ull; }
    return h;
}

void validate_common(size_t R, hipStream_t c, hipStream_t h2d, hipStream_t d2h) {
    if (R == 0) throw std::runtime_error("recompute_interval must be >= 1");
    if (c == h2d || c == d2h || h2d == d2h)
        throw std::runtime_error("compute, h2d and d2h streams must be pairwise distinct");
}

void run_forward(Entry& e, size_t T, size_t R, const __half* x_host, const __half* h0, const __half* c0,
                 const float* w_ih, const float* w_hh, const float* b_ih, const float* b_hh, __half* y_host,
                 flstm::GateCacheHost cache, flstm::StreamingLstmOptions opt, __half* hy, __half* cy,
                 hipStream_t cs, hipStream_t h2d, hipStream_t d2h) {
    const size_t B = e.B, I = e.I, H = e.H;
    const size_t x_bytes = T * B * I * sizeof(half_t), y_bytes = T * B * H * sizeof(half_t);
    e.last.valid = false;
    e.x_dev.reserve(x_bytes);
    e.y_dev.reserve(y_bytes);
    check(hipMemcpyAsync(e.x_dev.p, x_host, x_bytes, hipMemcpyHostToDevice, h2d), "x upload");
    check(hipEventRecord(e.ev_in, h2d), "hipEventRecord");
    check_core(flstm_core_pack_weights(e.plan, w_ih, w_hh, cs), "flstm_core_pack_weights");
    check_core(flstm_core_pack_bias(e.plan, b_ih, b_hh, cs), "flstm_core_pack_bias");
    check(hipStreamWaitEvent(cs, e.ev_in, 0), "hipStreamWaitEvent");
    check_core(flstm_core_forward(e.plan, T, e.x_dev.p, FLSTM_F16, h0, c0, FLSTM_F16, y_host ? e.y_dev.p : nullptr,
                                  FLSTM_F16, hy, cy, FLSTM_F16, 1, cs),
               "flstm_core_forward");
    // checkpoints: state before step k*R, k = 0 .. ceil(T/R)-1
    const size_t nck = (T + R - 1) / R;
    const void* hptr = nullptr; const void* cptr = nullptr; size_t ldh = 0, ldc = 0;
    check_core(flstm_core_cache_ptr(e.plan, 0, &hptr, &ldh), "flstm_core_cache_ptr");
    check_core(flstm_core_cache_ptr(e.plan, 1, &cptr, &ldc), "flstm_core_cache_ptr");
    const bool h32 = opt.h_dtype == flstm::GateCacheDType::kFloat32;
    const bool c32 = opt.c_dtype == flstm::GateCacheDType::kFloat32;
    const size_t ckh_bytes = nck * B * H * (h32 ? 4 : 2), ckc_bytes = nck * B * H * (c32 ? 4 : 2);
    if (cache.h_ptr) {
        e.ck_h.reserve(ckh_bytes);
        check(flstm_hip::gather_from_half(static_cast<const half_t*>(hptr), ldh, nck * B, int(H), e.ck_h.p, h32, B,
                                          R * B, cs), "checkpoint gather");
    }
    if (cache.c_ptr) {
        e.ck_c.reserve(ckc_bytes);
        check(flstm_hip::gather_from_float(static_cast<const float*>(cptr), ldc, nck * B, int(H), 1.f, e.ck_c.p, c32,
                                           B, R * B, cs), "checkpoint gather");
    }
    check(hipEventRecord(e.ev_out, cs), "hipEventRecord");
    check(hipStreamWaitEvent(d2h, e.ev_out, 0), "hipStreamWaitEvent");
    if (y_host) check(hipMemcpyAsync(y_host, e.y_dev.p, y_bytes, hipMemcpyDeviceToHost, d2h), "y download");
    if (cache.h_ptr) check(hipMemcpyAsync(cache.h_ptr, e.ck_h.p, ckh_bytes, hipMemcpyDeviceToHost, d2h), "h checkpoints");
    if (cache.c_ptr) check(hipMemcpyAsync(cache.c_ptr, e.ck_c.p, ckc_bytes, hipMemcpyDeviceToHost, d2h), "c checkpoints");
    check(hipStreamSynchronize(cs), "sync compute");
    check(hipStreamSynchronize(h2d), "sync h2d");
    check(hipStreamSynchronize(d2h), "sync d2h");
    ForwardKey k;
    k.x = x_host; k.y = y_host; k.ch = cache.h_ptr; k.cc = cache.c_ptr; k.h0 = h0; k.c0 = c0;
    k.w_ih = w_ih; k.w_hh = w_hh; k.T = T; k.R = R;
    k.x_print = fingerprint(x_host, x_bytes);
    k.y_print = y_host ? fingerprint(y_host, y_bytes) : 0;
    k.valid = true;
    e.last = k;
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
    Entry& e = entry_for(B, I, H);
    run_forward(e, T, R, x_host, h0, c0, w_ih, w_hh, b_ih, b_hh, y_host, cache, opt, hy, cy, cs, h2d, d2h);
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
    (void)opt;
    std::lock_guard<std::mutex> lock(g_mutex);
    Entry& e = entry_for(B, I, H);
    const size_t x_bytes = T * B * I * sizeof(half_t), y_bytes = T * B * H * sizeof(half_t);
    static const bool always_recompute = (getenv("FLASHLSTM_V2_RECOMPUTE") != nullptr);
    const ForwardKey& k = e.last;
    bool hit = !always_recompute && k.valid && k.x == x_host && k.y == y_host && k.ch == cache.h_ptr &&
               k.cc == cache.c_ptr && k.h0 == h0 && k.c0 == c0 && k.w_ih == w_ih && k.w_hh == w_hh && k.T == T;
    if (hit) hit = (k.x_print == fingerprint(x_host, x_bytes)) && (!y_host || k.y_print == fingerprint(y_host, y_bytes));
    if (!hit) {
        // rebuild the device-side caches from the inputs (no host outputs are touched)
        run_forward(e, T, R, x_host, h0, c0, w_ih, w_hh, b_ih, b_hh, nullptr, GateCacheHost{nullptr, nullptr},
                    StreamingLstmOptions{}, nullptr, nullptr, cs, h2d, d2h);
    }
    e.dy_dev.reserve(y_bytes);
    if (dx_host) e.dx_dev.reserve(x_bytes);
    check(hipMemcpyAsync(e.dy_dev.p, dY_host, y_bytes, hipMemcpyHostToDevice, h2d), "dY upload");
    check(hipEventRecord(e.ev_in, h2d), "hipEventRecord");
    check(hipStreamWaitEvent(cs, e.ev_in, 0), "hipStreamWaitEvent");
    check_core(flstm_core_backward(e.plan, T, e.x_dev.p, FLSTM_F16, e.dy_dev.p, FLSTM_F16, d_hn, d_cn, FLSTM_F16,
                                   1.f, dx_host ? e.dx_dev.p : nullptr, FLSTM_F16, dW_ih, dW_hh, db_ih, db_hh, dh0,
                                   dc0, cs),
               "flstm_core_backward");
    check(hipEventRecord(e.ev_out, cs), "hipEventRecord");
    check(hipStreamWaitEvent(d2h, e.ev_out, 0), "hipStreamWaitEvent");
    if (dx_host) check(hipMemcpyAsync(dx_host, e.dx_dev.p, x_bytes, hipMemcpyDeviceToHost, d2h), "dx download");
    check(hipStreamSynchronize(cs), "sync compute");
    check(hipStreamSynchronize(h2d), "sync h2d");
    check(hipStreamSynchronize(d2h), "sync d2h");
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
