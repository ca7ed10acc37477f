// Host-streaming forward / backward (include/flashlstm_v2/lstm.hpp) on top of the device-resident
// core.  Replaces flstm::StreamingLstmForward (reference flashlstm_v2/src/lstm_forward.cu:464-966)
// and flstm::StreamingLstmBackward (flashlstm_v2/src/lstm_backward.cu:643-1250).
//
// 288 GB of HBM hold whole sequences, so the device buffers are sequence-sized; what is streamed is the
// work: x (dY) goes up in chunks of time steps on the h2d stream, each chunk's projection + recurrence
// (BPTT steps + dX) is enqueued on the compute stream behind an event, and its y (dx) rows leave on the d2h
// stream behind another, so the three streams overlap as in the reference's 32-step pipeline
// (flashlstm_v2/src/lstm_forward.cu:646-940).  FLASHLSTM_V2_CHUNK_STEPS sets the chunk length (default 64;
// 0 = whole sequence).  Forward keeps its device-side gate cache in a small registry; a backward call that
// names the same host buffers (and whose sampled contents still match) reuses it, any other backward call
// first recomputes the forward pass from x, h0 and c0 -- which yields exactly the states the host
// checkpoints describe.  The host checkpoints are written with the reference's meaning: entry k = (h, c)
// before step k * recompute_interval.  Host buffers may be pageable (copies are then staged by the runtime
// and overlap less).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
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
    ~Entry() {
        if (plan) flstm_core_destroy(plan);
        for (Buf* b : {&x_dev, &y_dev, &dy_dev, &dx_dev, &ck_h, &ck_c}) b->release();
        if (ev_in) (void)hipEventDestroy(ev_in);
        if (ev_out) (void)hipEventDestroy(ev_out);
        for (hipEvent_t ev : chunk_in) (void)hipEventDestroy(ev);
        for (hipEvent_t ev : chunk_out) (void)hipEventDestroy(ev);
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

void run_forward(Entry& e, size_t T, size_t R, const __half* x_host, const __half* h0, const __half* c0,
                 const float* w_ih, const float* w_hh, const float* b_ih, const float* b_hh, __half* y_host,
                 flstm::GateCacheHost cache, flstm::StreamingLstmOptions opt, __half* hy, __half* cy,
                 hipStream_t cs, hipStream_t h2d, hipStream_t d2h) {
    const size_t B = e.B, I = e.I, H = e.H;
    const size_t x_bytes = T * B * I * sizeof(half_t), y_bytes = T * B * H * sizeof(half_t);
    e.last.valid = false;
    e.x_dev.reserve(x_bytes);
    check_core(flstm_core_pack_weights(e.plan, w_ih, w_hh, cs), "flstm_core_pack_weights");
    check_core(flstm_core_pack_bias(e.plan, b_ih, b_hh, cs), "flstm_core_pack_bias");
    check_core(flstm_core_forward_begin(e.plan, T, e.x_dev.p, FLSTM_F16, h0, c0, FLSTM_F16, cs), "flstm_core_forward_begin");
    const void* hptr = nullptr; const void* cptr = nullptr; size_t ldh = 0, ldc = 0;
    check_core(flstm_core_cache_ptr(e.plan, 0, &hptr, &ldh), "flstm_core_cache_ptr");
    check_core(flstm_core_cache_ptr(e.plan, 1, &cptr, &ldc), "flstm_core_cache_ptr");
    const size_t C = chunk_steps_for(T), nchunks = (T + C - 1) / C;
    e.need_chunk_events(nchunks);
    auto upload = [&](size_t k) {
        const size_t t0 = k * C, n = (t0 + C <= T) ? C : T - t0;
        check(hipMemcpyAsync(static_cast<char*>(e.x_dev.p) + t0 * B * I * sizeof(half_t),
                             reinterpret_cast<const char*>(x_host) + t0 * B * I * sizeof(half_t), n * B * I * sizeof(half_t),
                             hipMemcpyHostToDevice, h2d), "x upload");
        check(hipEventRecord(e.chunk_in[k], h2d), "hipEventRecord");
    };
    upload(0);
    for (size_t k = 0; k < nchunks; ++k) {
        const size_t t0 = k * C, n = (t0 + C <= T) ? C : T - t0;
        if (k + 1 < nchunks) upload(k + 1);
        check(hipStreamWaitEvent(cs, e.chunk_in[k], 0), "hipStreamWaitEvent");
        check_core(flstm_core_forward_steps(e.plan, t0, n, cs), "flstm_core_forward_steps");
        check(hipEventRecord(e.chunk_out[k], cs), "hipEventRecord");
        if (y_host) {   // h_t of step t is row block t+1 of the state cache
            check(hipStreamWaitEvent(d2h, e.chunk_out[k], 0), "hipStreamWaitEvent");
            download_rows(y_host, static_cast<const half_t*>(hptr) + B * ldh, ldh, H, sizeof(half_t), t0 * B, n * B, d2h);
        }
    }
    int rc = flstm_core_forward_end(e.plan, hy, cy, FLSTM_F16, 1, cs);
    if (rc == FLSTM_E_STALLED) {
        // a persistent launch gave up: repeat the pass through the entry point that falls back to step-wise launches
        check(hipStreamSynchronize(d2h), "sync d2h");
        e.y_dev.reserve(y_bytes);
        check_core(flstm_core_forward(e.plan, T, e.x_dev.p, FLSTM_F16, h0, c0, FLSTM_F16, y_host ? e.y_dev.p : nullptr,
                                      FLSTM_F16, hy, cy, FLSTM_F16, 1, cs), "flstm_core_forward");
        if (y_host) check(hipMemcpyAsync(y_host, e.y_dev.p, y_bytes, hipMemcpyDeviceToHost, d2h), "y download");
        check_core(flstm_core_cache_ptr(e.plan, 0, &hptr, &ldh), "flstm_core_cache_ptr");
        check_core(flstm_core_cache_ptr(e.plan, 1, &cptr, &ldc), "flstm_core_cache_ptr");
    } else {
        check_core(rc, "flstm_core_forward_end");
    }
    // checkpoints: state before step k*R, k = 0 .. ceil(T/R)-1
    const size_t nck = (T + R - 1) / R;
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
    flstm_hip::RangeGuard range("FlashLSTM::StreamingLstmForward");
    flstm_hip::MfuProfiler prof("forward");   // (same label and line as flashlstm_v2/src/lstm_forward.cu:492)
    Entry& e = entry_for(B, I, H);
    run_forward(e, T, R, x_host, h0, c0, w_ih, w_hh, b_ih, b_hh, y_host, cache, opt, hy, cy, cs, h2d, d2h);
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
    (void)opt;
    std::lock_guard<std::mutex> lock(g_mutex);
    flstm_hip::RangeGuard range("FlashLSTM::StreamingLstmBackward");
    flstm_hip::MfuProfiler prof("backward");   // (flashlstm_v2/src/lstm_backward.cu:679)
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
        prof.add_total(double(T) * flstm_hip::gemm_flops(4 * H, B, I + H));   // recomputation
    }
    e.dy_dev.reserve(y_bytes);
    if (dx_host) e.dx_dev.reserve(x_bytes);
    check_core(flstm_core_backward_begin(e.plan, T, e.dy_dev.p, FLSTM_F16, d_hn, d_cn, FLSTM_F16, 1.f,
                                         dx_host ? e.dx_dev.p : nullptr, FLSTM_F16, cs), "flstm_core_backward_begin");
    // chunks from the end of the sequence: dY rows up, BPTT steps + dX, dx rows down
    const size_t C = chunk_steps_for(T), nchunks = (T + C - 1) / C;
    e.need_chunk_events(nchunks);
    auto chunk_range = [&](size_t k, size_t& lo, size_t& n) {   // chunk k counts from the end; the first one takes the remainder
        const size_t rem = T % C, first = rem ? rem : C;
        n = (k == 0) ? first : C;
        const size_t hi = T - 1 - (k == 0 ? 0 : first + (k - 1) * C);
        lo = hi + 1 - n;
    };
    auto upload = [&](size_t k) {
        size_t lo, n;
        chunk_range(k, lo, n);
        check(hipMemcpyAsync(static_cast<char*>(e.dy_dev.p) + lo * B * H * sizeof(half_t),
                             reinterpret_cast<const char*>(dY_host) + lo * B * H * sizeof(half_t), n * B * H * sizeof(half_t),
                             hipMemcpyHostToDevice, h2d), "dY upload");
        check(hipEventRecord(e.chunk_in[k], h2d), "hipEventRecord");
    };
    upload(0);
    for (size_t k = 0; k < nchunks; ++k) {
        size_t lo, n;
        chunk_range(k, lo, n);
        if (k + 1 < nchunks) upload(k + 1);
        check(hipStreamWaitEvent(cs, e.chunk_in[k], 0), "hipStreamWaitEvent");
        check_core(flstm_core_backward_steps(e.plan, lo + n - 1, n, cs), "flstm_core_backward_steps");
        check(hipEventRecord(e.chunk_out[k], cs), "hipEventRecord");
        if (dx_host) {
            check(hipStreamWaitEvent(d2h, e.chunk_out[k], 0), "hipStreamWaitEvent");
            download_rows(dx_host, e.dx_dev.p, I, I, sizeof(half_t), lo * B, n * B, d2h);
        }
    }
    int rc = flstm_core_backward_end(e.plan, e.x_dev.p, FLSTM_F16, dW_ih, dW_hh, db_ih, db_hh, dh0, dc0, cs);
    if (rc == FLSTM_E_STALLED) {
        // a persistent launch gave up: repeat the pass through the entry point that falls back to step-wise launches
        check(hipStreamSynchronize(d2h), "sync d2h");
        check_core(flstm_core_backward(e.plan, T, e.x_dev.p, FLSTM_F16, e.dy_dev.p, FLSTM_F16, d_hn, d_cn, FLSTM_F16,
                                       1.f, dx_host ? e.dx_dev.p : nullptr, FLSTM_F16, dW_ih, dW_hh, db_ih, db_hh, dh0,
                                       dc0, cs), "flstm_core_backward");
        if (dx_host) check(hipMemcpyAsync(dx_host, e.dx_dev.p, x_bytes, hipMemcpyDeviceToHost, d2h), "dx download");
    } else {
        check_core(rc, "flstm_core_backward_end");
    }
    check(hipStreamSynchronize(cs), "sync compute");
    check(hipStreamSynchronize(h2d), "sync h2d");
    check(hipStreamSynchronize(d2h), "sync d2h");
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
