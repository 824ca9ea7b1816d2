// Library identification, status text, the per-thread record of the last HIP
// error a launch reported, and the per-thread pair of timing events for the
// next launch.
#include "common.h"

namespace ts {
static thread_local int g_last_hip_error = 0;
void set_last_hip_error(int code) { g_last_hip_error = code; }

static thread_local hipEvent_t g_time_start = nullptr, g_time_stop = nullptr;
bool take_launch_events(hipEvent_t* start, hipEvent_t* stop) {
  *start = g_time_start;
  *stop = g_time_stop;
  g_time_start = g_time_stop = nullptr;
  return *start != nullptr && *stop != nullptr;
}
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

int ts_time_next_launch(void* start_event, void* stop_event) {
  if ((start_event == nullptr) != (stop_event == nullptr)) return TS_ERR_ARG;
  ts::g_time_start = (hipEvent_t)start_event;
  ts::g_time_stop = (hipEvent_t)stop_event;
  return TS_OK;
}

}  // extern "C"
