// Ordering one stream after another: the second stream of a prompt portion's shared
// expert starts after the main stream's work so far and is waited for before its result
// is read. One host call records the event and queues the wait.
#include "common.h"

// An event without timing, for ordering one stream after another. Never destroyed: a
// process makes a handful.
extern "C" void* ninfer_event_create() {
  hipEvent_t ev = nullptr;
  if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
    ninfer::set_error(-2, "hipEventCreateWithFlags failed");
    return nullptr;
  }
  return ev;
}

// Work given to `later` after this call starts once everything given to `earlier` so far
// is done. One host call for the record and the wait.
extern "C" int ninfer_stream_after(hipStream_t later, hipStream_t earlier, void* event) {
  hipEvent_t ev = (hipEvent_t)event;
  if (ev == nullptr) return ninfer::set_error(-1, "stream_after: no event");
  hipError_t e = hipEventRecord(ev, earlier);
  if (e == hipSuccess) e = hipStreamWaitEvent(later, ev, 0);
  if (e != hipSuccess) return ninfer::set_error(-2, "stream_after: %s", hipGetErrorString(e));
  return 0;
}
