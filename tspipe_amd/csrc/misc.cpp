// Library identification, status text and the per-thread record of the last
// HIP error a launch reported.
#include "common.h"

namespace ts {
static thread_local int g_last_hip_error = 0;
void set_last_hip_error(int code) { g_last_hip_error = code; }
}  // namespace ts

extern "C" {

const char* ts_version(void) { return "tspipe_amd 0.1 (gfx950)"; }

const char* ts_error_string(int status) {
  switch (status) {
    case TS_OK: return "ok";
    case TS_ERR_ARG: return "invalid argument";
    case TS_ERR_CAPACITY: return "chunk table too small for the plan";
    case TS_ERR_LAUNCH: return "HIP launch failed";
    case TS_ERR_ALIGN: return "pointer not aligned to its element size";
    case TS_ERR_RANGE: return "size outside the supported range";
    default: return "unknown status";
  }
}

int ts_last_hip_error(void) { return ts::g_last_hip_error; }

}  // extern "C"
