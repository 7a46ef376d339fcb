// Status reporting shared by every entry point of the library.
#include "ri_common.h"

static thread_local int g_last_hip_error = 0;

void ri_set_last_hip_error(int e) { g_last_hip_error = e; }

extern "C" int ri_last_hip_error(void) { return g_last_hip_error; }

extern "C" int ri_abi_version(void) { return 5; }

// An empty launch: what a dependent kernel dispatch costs on this stream, for callers that want to
// separate dispatch overhead from kernel time in event measurements.
__global__ void null_kernel() {}

extern "C" int ri_null_launch(ri_stream_t stream) {
  null_kernel<<<1, 64, 0, (hipStream_t)stream>>>();
  RI_HIP_CHECK_LAUNCH();
  return RI_OK;
}

extern "C" const char* ri_status_string(int status) {
  switch (status) {
    case RI_OK: return "ok";
    case RI_ERR_ARG: return "invalid argument (shape, null pointer or unsupported size)";
    case RI_ERR_LAUNCH: return "HIP launch error";
    case RI_ERR_WORKSPACE: return "workspace too small";
    case RI_ERR_STATE: return "host object used before it was set up";
    default: return "unknown status";
  }
}
