// Error state and identification of libdistdl_hip.
#include "ddl_common.h"

namespace ddl {

char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return 0;
    return fail(static_cast<int>(e), "%s: %s", what, hipGetErrorString(e));
}

namespace {
__global__ void probe_kernel() {}
}  // namespace

}  // namespace ddl

extern "C" {

int ddl_probe_launch(int64_t workgroups, int threads, void* stream) {
    if (workgroups < 1 || workgroups > 0x7FFFFFFFll || threads < 1 || threads > 1024)
        return ddl::fail(DDL_E_ARG, "probe: %lld workgroups of %d threads", (long long)workgroups, threads);
    hipLaunchKernelGGL(ddl::probe_kernel, dim3(static_cast<uint32_t>(workgroups)), dim3(threads), 0, static_cast<hipStream_t>(stream));
    return ddl::check_launch("probe_kernel");
}

const char* ddl_version(void) { return "distdl_hip 0.1.0 gfx950"; }

const char* ddl_last_error(void) { return ddl::error_buffer(); }

}  // extern "C"
