// Optional instrumentation of the host entry points: roctx ranges with the names of the reference's NVTX
// ranges (src/nvtx_profinst.h:19-54, src/lstm.cu:1341,1911) and the environment-gated MFU report of
// flashlstm_v2/include/mfu_profiler.hpp:21-100 (FLASHLSTM_PROFILE_MFU, FLASHLSTM_MFU_PEAK_TFLOPS), with the
// same output line.  Both cost nothing when unused: the roctx library is looked up at run time and the
// ranges are no-ops without it.
#pragma once
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <string>

namespace flstm_hip {

class RangeGuard {
public:
    explicit RangeGuard(const char* name) {
        if (api().push) api().push(name);
    }
    ~RangeGuard() {
        if (api().pop) api().pop();
    }
    RangeGuard(const RangeGuard&) = delete;
    RangeGuard& operator=(const RangeGuard&) = delete;

private:
    struct Api {
        int (*push)(const char*) = nullptr;
        int (*pop)() = nullptr;
    };
    static const Api& api() {
        static const Api a = [] {
            Api r;
            void* lib = dlopen("librocprofiler-sdk-roctx.so", RTLD_LAZY | RTLD_GLOBAL);
            if (!lib) lib = dlopen("libroctx64.so", RTLD_LAZY | RTLD_GLOBAL);
            if (lib) {
                r.push = reinterpret_cast<int (*)(const char*)>(dlsym(lib, "roctxRangePushA"));
                r.pop = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
                if (!r.push || !r.pop) r.push = nullptr, r.pop = nullptr;
            }
            return r;
        }();
        return a;
    }
};

inline double gemm_flops(size_t m, size_t n, size_t k) { return 2.0 * double(m) * double(n) * double(k); }

// Wall-clock MFU / HFU of one call.  "Useful" FLOPs are those of the algorithm, "total" adds recomputation.
class MfuProfiler {
public:
    explicit MfuProfiler(const char* label) : enabled_(std::getenv("FLASHLSTM_PROFILE_MFU") != nullptr), label_(label) {
        if (!enabled_) return;
        peak_ = peak_flops();
        start_ = Clock::now();
    }
    void add_useful(double f) { if (enabled_) { useful_ += f; total_ += f; } }
    void add_total(double f) { if (enabled_) total_ += f; }
    void finish() {
        if (!enabled_ || finished_) return;
        finished_ = true;
        const double s = std::chrono::duration<double>(Clock::now() - start_).count();
        if (s <= 0.0) return;
        const double peak_t = peak_ / 1e12, useful_t = useful_ / s / 1e12, total_t = total_ / s / 1e12;
        std::printf("[flashlstm][%s] MFU=%.2f%% HFU=%.2f%% (useful=%.3f TFLOP/s, matmul=%.3f TFLOP/s, peak=%.3f TFLOP/s)\n",
                    label_.c_str(), peak_t > 0 ? useful_t / peak_t * 100.0 : 0.0, peak_t > 0 ? total_t / peak_t * 100.0 : 0.0,
                    useful_t, total_t, peak_t);
        std::fflush(stdout);
    }

private:
    using Clock = std::chrono::steady_clock;
    // FLASHLSTM_MFU_PEAK_TFLOPS, or clock x CUs x 4096 FLOP/clk/CU (dense fp16 MFMA rate of a CDNA4 CU)
    static double peak_flops() {
        static const double cached = [] {   // initialised once, also when several threads arrive together
            const char* ov = std::getenv("FLASHLSTM_MFU_PEAK_TFLOPS");
            if (ov && ov[0]) return std::strtod(ov, nullptr) * 1e12;
            int dev = 0;
            hipDeviceProp_t prop{};
            if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0.0;
            return double(prop.clockRate) * 1000.0 * double(prop.multiProcessorCount) * 4096.0;
        }();
        return cached;
    }
    bool enabled_ = false, finished_ = false;
    std::string label_;
    double useful_ = 0.0, total_ = 0.0, peak_ = 0.0;
    Clock::time_point start_{};
};

}  // namespace flstm_hip
