// Library-level entry points of libmuon_amd: version, error string, struct sizes.
#include "common.h"

namespace muon_amd {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(err));
        return MUON_AMD_ELAUNCH;
    }
    return MUON_AMD_OK;
}

}  // namespace muon_amd

extern "C" {

int muon_amd_abi_version(void) { return MUON_AMD_ABI_VERSION; }
const char* muon_amd_last_error(void) { return muon_amd::g_error; }

size_t muon_amd_sizeof_mat_desc(void) { return sizeof(MuonMatDesc); }
size_t muon_amd_sizeof_gemm_desc(void) { return sizeof(MuonGemmDesc); }
size_t muon_amd_sizeof_tile_job(void) { return sizeof(MuonTileJob); }
size_t muon_amd_sizeof_adam_desc(void) { return sizeof(MuonAdamDesc); }

}  // extern "C"
