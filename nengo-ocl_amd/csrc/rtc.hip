// Function nodes compiled at run time.  The host translates a Python function into
// the body of a small element-wise kernel (one thread per node instance); this file
// compiles that source with hiprtc for gfx950, loads it, and launches it like any
// other plan (the launch is an ordinary kernel node when a timestep is recorded into
// a graph).  The reference builds such kernels from OpenCL text with
// `cl.Program(ctx, text).build()` (clra_nonlinearities.py:954-1025).
#include <hip/hiprtc.h>

#include <cstring>
#include <string>
#include <vector>

#include "nhip_common.h"

namespace {

struct RtcProgram {
    std::vector<char> code;
    hipModule_t module = nullptr;
};

void copy_log(const std::string& text, char* log, int log_len) {
    if (!log || log_len <= 0) return;
    const size_t n = text.size() < (size_t)log_len - 1 ? text.size() : (size_t)log_len - 1;
    memcpy(log, text.data(), n);
    log[n] = 0;
}

}  // namespace

extern "C" int nhip_rtc_compile(const char* source, const char* arch, void** program_out,
                                char* log, int log_len) {
    if (!source || !program_out) return NHIP_E_BADARG;
    *program_out = nullptr;
    copy_log("", log, log_len);
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, source, "function_node.hip", 0, nullptr, nullptr) !=
        HIPRTC_SUCCESS)
        return NHIP_E_RTC;
    const std::string arch_opt = std::string("--offload-arch=") + (arch && *arch ? arch : "gfx950");
    // same code generation rules as the library's own kernels: no contraction of
    // separately written products and sums, no packed-FP32 instruction selection
    const char* opts[] = {arch_opt.c_str(), "-O3", "-ffp-contract=off", "-Xclang",
                          "-target-feature", "-Xclang", "-packed-fp32-ops"};
    const hiprtcResult res = hiprtcCompileProgram(prog, 7, opts);
    size_t log_size = 0;
    if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
        std::string text(log_size, 0);
        if (hiprtcGetProgramLog(prog, &text[0]) == HIPRTC_SUCCESS) copy_log(text, log, log_len);
    }
    if (res != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&prog);
        return NHIP_E_RTC;
    }
    size_t code_size = 0;
    RtcProgram* p = new RtcProgram;
    if (hiprtcGetCodeSize(prog, &code_size) != HIPRTC_SUCCESS || code_size == 0) {
        hiprtcDestroyProgram(&prog);
        delete p;
        return NHIP_E_RTC;
    }
    p->code.resize(code_size);
    const hiprtcResult got = hiprtcGetCode(prog, p->code.data());
    hiprtcDestroyProgram(&prog);
    if (got != HIPRTC_SUCCESS) {
        delete p;
        return NHIP_E_RTC;
    }
    *program_out = p;
    return 0;
}

extern "C" int nhip_rtc_load(void* program, const char* kernel_name, void** function_out) {
    if (!program || !kernel_name || !function_out) return NHIP_E_BADARG;
    RtcProgram* p = static_cast<RtcProgram*>(program);
    if (!p->module) {
        const hipError_t e = hipModuleLoadData(&p->module, p->code.data());
        if (e != hipSuccess) return (int)e;
    }
    hipFunction_t fn;
    const hipError_t e = hipModuleGetFunction(&fn, p->module, kernel_name);
    if (e != hipSuccess) return (int)e;
    *function_out = fn;
    return 0;
}

extern "C" int nhip_rtc_destroy(void* program) {
    if (!program) return 0;
    RtcProgram* p = static_cast<RtcProgram*>(program);
    hipError_t e = hipSuccess;
    if (p->module) e = hipModuleUnload(p->module);
    delete p;
    return (int)e;
}

extern "C" int nhip_rtc_launch_direct(void* stream, void* function, int n, const int* t_starts,
                                      const float* T, const int* x_starts, const float* X,
                                      const int* y_starts, float* Y) {
    if (n == 0) return 0;
    if (n < 0 || !function || !y_starts || !Y) return NHIP_E_BADARG;
    void* args[] = {&n, &t_starts, &T, &x_starts, &X, &y_starts, &Y};
    const unsigned block = 64, grid = ((unsigned)n + block - 1) / block;
    return (int)hipModuleLaunchKernel(static_cast<hipFunction_t>(function), grid, 1, 1, block, 1,
                                      1, 0, static_cast<hipStream_t>(stream), args, nullptr);
}
